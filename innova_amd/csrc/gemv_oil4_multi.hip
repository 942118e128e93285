// gemv_oil4_multi.hip -- decode GEMV over uniform OIL4 tensors for a handful of activation rows
// (up to 8, 16 or 32 tokens per pass): Qwen35Engine::gemm with small B (src/adapters/tools/qwen35_engine.cpp:47-85)
// and the per-expert batches of moe_dispatch_batched (src/moe_variants.cpp:767-827).
//
// The products run on the matrix cores in FP16 with both operands split in two: a level L of the table is
// Lh + Ll (Lh = fp16(L), Ll = fp16(L - Lh)), an activation x is xh + xl the same way, and
// L x = Lh xh + Lh xl + Ll xh up to 2^-22 relative (the Ll xl term is dropped); every product of two FP16 values is
// exact in the FP32 accumulator of v_mfma_f32_16x16x32_f16, so three matrix instructions stand for one FP32 one at
// a quarter of its cost per flop.  The FP16 block scale multiplies the block's 16 x 16 partial sums afterwards.
// Lane l = 16*kq + i supplies row i of a group of 16 rows; of a 128-byte block it owns the 16-byte chunks kq and
// kq+4 (64 nibbles), one dword (8 nibbles) per matrix instruction.  Lane 16*kq + j supplies token j at the same
// nibble positions, and accumulator register v of that lane collects row 4*kq + v x token j.
//
// A wavefront owns two blocks of the row per K-pass (blocks w and w + 8 of the pass; 8 wavefronts = 16 blocks = 4096 columns) and keeps the split
// activations of those blocks in registers (2 x 64 FP16 pairs per lane), so the main loop is: two 16-byte loads per
// lane and unit (16 rows x 1 block), 32 byte-pair table lookups (each returns the two high and the two low halves
// of a byte's levels, already packed as matrix operands), 24 matrix instructions, 4 scale multiplies.  The
// activations are split and laid out in this operand order once per launch by pack_x_kernel (every workgroup needs
// all of them), so the main kernel fetches its 128 operand dwords with plain 16-byte loads.  Partial sums of the
// wavefronts are added through LDS once per tile of 64 rows.
// Single tensors with more than 16 tokens run passes of 32: a wavefront then owns one block per K-pass and multiplies each
// decoded weight operand with the activations of two token tiles (the table look-ups, which bound the main loop, are
// shared), a row tile is 32 rows.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <mutex>
#include <numeric>

#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using namespace oil4;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const u32x2 lds_cu32x2;

// L -> fp16(L) in the low half, fp16(L - fp16(L)) in the high half
__device__ __forceinline__ uint32_t split_level(float L) {
    const __half h = __float2half_rn(L);
    const __half l = __float2half_rn(L - __half2float(h));
    return (uint32_t)__half_as_ushort(h) | ((uint32_t)__half_as_ushort(l) << 16);
}

constexpr size_t kBatchCounterBytes = kGemvBatchCounterBytes;   // a page of slab counters for each of up to 32 jobs of a grouped launch
constexpr int kGroups = 4;                // 16 x 16 partial-sum tiles per wavefront and row tile (groups of 16 rows x token tiles)
constexpr int kRedBase = kTabBytes;       // partial sums follow the level table
// partial sums of a 16 x 16 tile, accumulator lane 16 q + j, element v at float q*68 + 4 j + v of 272: for one token j the
// 64 (group, row) pairs of a tile fall into 64 different banks
constexpr int kRedTile = 272;
constexpr int kRedBytes = 8 * kGroups * kRedTile * 4;

// Packed activations of one pass of 16 tokens (x, or silu(x) * x2 when x2 is given): for block blk of the row, half h and lane l = 16*kq + t (token t) 32
// dwords: the high FP16 parts of the lane's 32 nibble positions (positions 2c, 2c+1 in dword c, c = 0..15), then the
// low parts.  Piece j (dwords 4j .. 4j+3 of the 32) of all 64 lanes is one contiguous KB at
// ((blk*2 + h)*8 + j)*1024 + l*16 bytes, so that a wavefront fetches it with one coalesced 16-byte load per lane.  Nibble p = 32*(kq + 4h) + s of a block holds weight
// i = q + q/63 with q = p - 4 (p < 4: the block's scale, activation 0).
// A workgroup packs one block of the row for all token columns of a tile (or a quarter of them), a wavefront one token
// column (256 activations) at a time: it finds their largest magnitude, scales them by
// the power of two that brings it to [2^14, 2^15) (so the FP16 split keeps 22 bits whatever the magnitude of the
// activations; blocks that are zero or hold a non-finite value stay unscaled) and leaves the exponent at
// xp_exp[(tile * bpr + blk) * 16 + column] for the main kernel, which undoes it on the block's partial sums.

// silu(a) * b, the SwiGLU product in front of an expert's down projection (ExpertFFN::forward,
// src/moe_variants.cpp:77-91), formed while the activations are split instead of in a kernel of its own
__device__ __forceinline__ float swiglu_value(float a, float b) { return (a / (1.0f + expf(-a))) * b; }

__global__ void __launch_bounds__(256) zero_words_kernel(uint32_t* __restrict__ p, uint32_t n) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// Several batches in one launch (the experts of a mixture-of-experts step): batch j packs M[j] rows of x into
// xp + xp_off[j] (exponents at xp_exp + exp_off[j]); its rows are list[row0[j] + m] when use_list is set, else
// row0[j] + m.  The list travels by value with the launch, so the host needs no copy and no synchronisation.
constexpr int kMaxJobs = 32, kMaxListed = 448;
static_assert(kBatchCounterBytes == (size_t)kMaxJobs * 4096u, "one page of counters per job");
struct PackJobs {
    uint32_t n, wgs_per_job;
    int M[kMaxJobs], row0[kMaxJobs];
    uint32_t xp_off[kMaxJobs], exp_off[kMaxJobs];
    uint8_t kind[kMaxJobs];     // pass size of the batch: 0 = 8 tokens, 1 = 16, 2 = 32 (wgs_per_job is that of the largest one present)
    float* clear0[kMaxJobs];    // outputs of the batch (M rows of clear_rows floats) that two row parts add into: they start at zero
    float* clear1[kMaxJobs];
    uint32_t clear_rows, clear_ld;
    int use_list;
    int list[kMaxListed];
};

// Rows [m_lo, m_hi) of y (n floats each, ld apart) set to zero by `threads` threads of which this one is number `id`:
// the threads are dealt over (row, 16-byte piece) so that all of them store, with one division per thread.
__device__ __forceinline__ void clear_rows_2d(float* __restrict__ y, uint32_t n, uint32_t ld, int m_lo, int m_hi, uint32_t id, uint32_t threads) {
    if (!y) return;
    const bool vec = ((reinterpret_cast<uintptr_t>(y) & 15u) | (n & 3u) | (ld & 3u)) == 0u;
    const uint32_t per_row = vec ? n >> 2 : n;                             // stores per row
    const uint32_t lanes = per_row < threads ? per_row : threads;          // threads that share a row
    const uint32_t rows_at_once = threads / lanes, slot = id / lanes, col = id - slot * lanes;
    if (slot >= rows_at_once) return;
    for (int mm = m_lo + (int)slot; mm < m_hi; mm += (int)rows_at_once)
        for (uint32_t c = col; c < per_row; c += lanes) {
            if (vec) *reinterpret_cast<float4*>(y + (size_t)mm * ld + 4u * c) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            else y[(size_t)mm * ld + c] = 0.0f;
        }
}

// What both pre-pass kernels do first: a workgroup of a grouped launch finds its batch (activation rows, pass size,
// place of the packed data), and the outputs that the main kernel's two row parts add into are cleared.  PARKED selects
// the workgroup count of a batch.  Returns false for workgroups beyond the batch's own count.
template <bool PARKED>
__device__ __forceinline__ bool pack_prologue(uint32_t& bid, int& M, int& row0, int& half, uint32_t*& xp, int*& xp_exp, uint32_t cols, int m0,
                                              float* yc0, uint32_t yc0_rows, uint32_t yc0_ld, float* yc1, uint32_t yc1_rows, uint32_t yc1_ld,
                                              const PackJobs& jobs) {
    const uint32_t bpr = cols >> 8, tid = threadIdx.x;
    if (jobs.n) {                                                          // workgroup -> (batch, index within the batch)
        const uint32_t job = bid / jobs.wgs_per_job;
        bid -= job * jobs.wgs_per_job;
        M = jobs.M[job]; row0 = jobs.row0[job];
        xp += jobs.xp_off[job]; xp_exp += jobs.exp_off[job];
        const uint32_t kind = jobs.kind[job];
        half = kind == 0u ? 1 : 0;
        for (int o = 0; o < 2; ++o) clear_rows_2d(o ? jobs.clear1[job] : jobs.clear0[job], jobs.clear_rows, jobs.clear_ld, 0, M, bid * 256u + tid, jobs.wgs_per_job * 256u);
        // a smaller pass than the launch's largest: fewer workgroups
        const uint32_t own = PARKED ? (kind == 2u ? 2u : 1u) * bpr : (kind == 0u ? 8u : kind == 1u ? 16u : 32u) * ((bpr + 3u) / 4u);
        if (bid >= own) return false;
    }
    clear_rows_2d(yc0, yc0_rows, yc0_ld, m0, M, blockIdx.x * 256u + tid, gridDim.x * 256u);
    clear_rows_2d(yc1, yc1_rows, yc1_ld, m0, M, blockIdx.x * 256u + tid, gridDim.x * 256u);
    return true;
}

// Small launches (a single tensor, few blocks per row): a wavefront packs one block of one token column straight from
// memory to memory -- the shortest chain of round trips, at the price of 4-byte stores that share their lines with
// other workgroups.  Workgroup = 4 blocks of token column t of a tile.
__global__ void __launch_bounds__(256)
pack_x_cols_kernel(const float* __restrict__ x, const float* __restrict__ x2, const int* __restrict__ tok, uint32_t* __restrict__ xp,
                   int* __restrict__ xp_exp, uint32_t cols, int m0, int M, uint32_t ldx, uint32_t xrows, int half,
                   float* __restrict__ yc0, uint32_t yc0_rows, uint32_t yc0_ld, float* __restrict__ yc1, uint32_t yc1_rows, uint32_t yc1_ld,
                   const PackJobs jobs) {
    const uint32_t bpr = cols >> 8, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t bid = blockIdx.x;
    int row0 = 0;
    uint32_t* xq = xp;
    int* xe = xp_exp;
    if (!pack_prologue<false>(bid, M, row0, half, xq, xe, cols, m0, yc0, yc0_rows, yc0_ld, yc1, yc1_rows, yc1_ld, jobs)) return;
    const uint32_t ncol = half ? 8u : 16u, nbg = (bpr + 3u) / 4u;
    const uint32_t blk = (bid % nbg) * 4u + wave, t = (bid / nbg) % ncol, tile = bid / (nbg * ncol);
    if (blk >= bpr) return;
    const int m = m0 + 16 * (int)tile + (int)t;
    xq += (size_t)tile * bpr * 4096u;
    uint32_t src = 0xFFFFFFFFu;
    if (m < M) src = jobs.n ? (jobs.use_list ? (uint32_t)jobs.list[row0 + m] : (uint32_t)(row0 + m)) : (tok ? (uint32_t)tok[m] : (uint32_t)m);
    const bool live = src < xrows;
    const size_t at = live ? (size_t)src * ldx + (size_t)blk * 256u : 0;
    // this lane's two pairs: pair id = lane + 64 k holds positions 2c, 2c+1 of chunk kq + 4h
    float v[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
    uint32_t mx = 0u;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const uint32_t id = lane + 64u * k, c = id & 15u, kq = (id >> 4) & 3u, h = id >> 6;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t pn = 32u * (kq + 4u * h) + 2u * c + e;
            if (live && pn >= 4u) {
                const uint32_t q = pn - 4u, col = q + q / 63u;
                v[k][e] = x2 ? swiglu_value(x[at + col], x2[at + col]) : x[at + col];
            }
            mx = max(mx, __float_as_uint(v[k][e]) & 0x7FFFFFFFu);
        }
    }
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
    const int ex = (int)(mx >> 23);
    const int e2 = (mx == 0u || ex == 255) ? 0 : 14 - (ex - 127);
    if (lane == 0) {
        xe[(tile * bpr + blk) * 16u + t] = e2;
        if (half) xe[(tile * bpr + blk) * 16u + t + 8u] = e2;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const uint32_t id = lane + 64u * k, c = id & 15u, kq = (id >> 4) & 3u, h = id >> 6;
        const float s0 = ldexpf(v[k][0], e2), s1 = ldexpf(v[k][1], e2);
        const auto ph = __builtin_amdgcn_cvt_pkrtz(s0, s1);           // x = xh + xl, both FP16 (round toward zero)
        const auto pl = __builtin_amdgcn_cvt_pkrtz(s0 - (float)ph[0], s1 - (float)ph[1]);
        uint32_t* o = xq + ((size_t)(blk * 2u + h) * 8u * 64u + 16u * kq + t) * 4u + (c & 3u);     // piece 0 of lane 16 kq + t, element c & 3
        o[(size_t)(c >> 2) * 256u] = __builtin_bit_cast(uint32_t, ph);
        o[(size_t)(c >> 2) * 256u + (half ? 32u : 1024u)] = __builtin_bit_cast(uint32_t, pl);      // lane 16 kq + t + 8, or piece 4 + (c >> 2)
    }
}

// Bulk launches (the batches of a mixture-of-experts step, wide rows): a workgroup parks a block's scaled activations for
// all token columns of a tile in LDS and writes whole 1 KB operand pieces.
__global__ void __launch_bounds__(256)
pack_x_kernel(const float* __restrict__ x, const float* __restrict__ x2, const int* __restrict__ tok, uint32_t* __restrict__ xp,
              int* __restrict__ xp_exp, uint32_t cols, int m0, int M, uint32_t ldx, uint32_t xrows, int half, int aligned,
              float* __restrict__ yc0, uint32_t yc0_rows, uint32_t yc0_ld, float* __restrict__ yc1, uint32_t yc1_rows, uint32_t yc1_ld,
              const PackJobs jobs) {
    // scaled activations of the workgroup's block, by nibble position: row (chunk of 32 positions, token column), 36
    // floats apart
    __shared__ __align__(16) float park[8 * 16 * 36];
    const uint32_t bpr = cols >> 8, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    uint32_t bid = blockIdx.x;
    int row0 = 0;
    uint32_t* xq = xp;
    int* xe = xp_exp;
    if (!pack_prologue<true>(bid, M, row0, half, xq, xe, cols, m0, yc0, yc0_rows, yc0_ld, yc1, yc1_rows, yc1_ld, jobs)) return;
    // workgroup = one block of the row for the 16 token columns of a tile (a pass of 32 tokens is two tiles of 16, the
    // second one's data behind the first's); passes of 8 tokens have 8 token columns: columns 0..7 of the operand
    // carry their high parts and columns 8..15 their low parts, in the pieces that otherwise hold the high parts of 16
    // tokens
    const uint32_t ncol = half ? 8u : 16u;
    const uint32_t blk = bid % bpr, tile = bid / bpr;
    xq += (size_t)tile * bpr * 4096u;
    // ---- a wavefront takes one token column at a time: 256 columns of x as one 16-byte load per lane, the largest
    // magnitude of the 252 that carry a weight, the power of two that brings it to [2^14, 2^15), the scaled values
    // parked by nibble position (column i of the block sits at nibble 4 + i - i/64; columns 63, 127, 191, 255 meet the
    // block's empty slots and are dropped; nibbles 0..3 hold the block's scale and see activation 0) ---------------
    float v[4][4];                                                         // [token column of this wavefront][column of the lane]
#pragma unroll
    for (int k = 0; k < 4; ++k) {                                          // all loads first: one round trip for the wavefront's columns
        const uint32_t t = wave + 4u * (uint32_t)k;
        const int m = m0 + 16 * (int)tile + (int)t;
        uint32_t src = 0xFFFFFFFFu;
        if (t < ncol && m < M)
            src = jobs.n ? (jobs.use_list ? (uint32_t)jobs.list[row0 + m] : (uint32_t)(row0 + m)) : (tok ? (uint32_t)tok[m] : (uint32_t)m);
        const bool live = src < xrows;
        const size_t at = live ? (size_t)src * ldx + (size_t)blk * 256u + 4u * lane : 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[k][e] = 0.0f;
        if (live && aligned) {                                             // rows that start on 16-byte boundaries
            const float4 a = *reinterpret_cast<const float4*>(x + at);
            v[k][0] = a.x; v[k][1] = a.y; v[k][2] = a.z; v[k][3] = a.w;
            if (x2) {
                const float4 b = *reinterpret_cast<const float4*>(x2 + at);
                v[k][0] = swiglu_value(v[k][0], b.x); v[k][1] = swiglu_value(v[k][1], b.y);
                v[k][2] = swiglu_value(v[k][2], b.z); v[k][3] = swiglu_value(v[k][3], b.w);
            }
        } else if (live) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[k][e] = x2 ? swiglu_value(x[at + e], x2[at + e]) : x[at + e];
        }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t t = wave + 4u * (uint32_t)k;
        if (t >= ncol) break;
        if ((lane & 15u) == 15u) v[k][3] = 0.0f;                           // column 64 n + 63: no weight there
        uint32_t mx = 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = max(mx, __float_as_uint(v[k][e]) & 0x7FFFFFFFu);
        for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
        const int ex = (int)(mx >> 23);
        const int e2 = (mx == 0u || ex == 255) ? 0 : 14 - (ex - 127);
        if (lane == 0) {
            xe[(tile * bpr + blk) * 16u + t] = e2;
            if (half) xe[(tile * bpr + blk) * 16u + t + 8u] = e2;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t i = 4u * lane + (uint32_t)e, pn = 4u + i - (i >> 6);
            if ((i & 63u) != 63u) park[((pn >> 5) * 16u + t) * 36u + (pn & 31u)] = ldexpf(v[k][e], e2);
        }
        if (lane < 4u) park[t * 36u + lane] = 0.0f;                        // nibbles 0..3 (chunk 0)
    }
    __syncthreads();
    // ---- a thread takes 8 consecutive nibble positions of one token column: four FP16 pairs of high parts
    // (x = xh + xl, both FP16, round toward zero) and four of low parts, 16 bytes each.  Piece j (dwords 4j .. 4j+3 of a
    // lane's 32) of lanes 16 kq + t is one contiguous KB, written here by 64 neighbouring threads -------------------
    for (uint32_t task = tid; task < 32u * ncol; task += 256u) {
        const uint32_t t = task % ncol, kq = (task / ncol) & 3u, jj = (task / (ncol * 4u)) & 3u, h = task / (ncol * 16u);
        const float* p = park + ((kq + 4u * h) * 16u + t) * 36u + 8u * jj;
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        const float sv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float s0 = sv[2 * c], s1 = sv[2 * c + 1];
            const auto ph = __builtin_amdgcn_cvt_pkrtz(s0, s1);
            const auto pl = __builtin_amdgcn_cvt_pkrtz(s0 - (float)ph[0], s1 - (float)ph[1]);
            hi[c] = __builtin_bit_cast(uint32_t, ph); lo[c] = __builtin_bit_cast(uint32_t, pl);
        }
        uint32_t* o = xq + ((size_t)(blk * 2u + h) * 8u * 64u + 16u * kq + t) * 4u + (size_t)jj * 256u;   // piece jj of lane 16 kq + t
        *reinterpret_cast<uint4*>(o) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *reinterpret_cast<uint4*>(o + (half ? 32u : 1024u)) = make_uint4(lo[0], lo[1], lo[2], lo[3]);   // lane + 8 of the piece, or piece 4 + jj
    }
}

// HALF: passes of 8 tokens.  The activation operand then holds high parts (columns 0..7) and low parts (columns 8..15)
// at once, so L x = (Lh + Ll)(xh + xl) takes two matrix instructions per 32 columns instead of three, the activations
// are half as many bytes, and an output is the sum of accumulator columns j and j + 8.
// NT = 2: passes of 32 tokens.  A wavefront then owns one block of the row per K-pass (8 blocks per pass) and keeps
// the split activations of two token tiles of it, so a decoded weight operand serves two matrix instructions per
// product term; a row tile is two groups of 16 rows.
// Several tensors of one shape in one launch (the experts of a mixture-of-experts step): each tensor (job) owns a range
// of the launch's workgroups and brings its packed activations, batch size and output.
struct MultiJobs {
    uint32_t n;
    uint32_t wg_begin[kMaxJobs + 1];   // job j runs workgroups [wg_begin[j], wg_begin[j + 1]): as many as its share of the launch's work
    uint32_t g_base[kMaxJobs], g_rem[kMaxJobs];   // row groups per slab of the job: g_base, and one more for the first g_rem slabs
    uint32_t pstride;                  // floats between two K parts of one output row when the parts are left for a later launch to sum
    const uint8_t* W[kMaxJobs];
    float* y[kMaxJobs];
    int M[kMaxJobs];
    uint32_t xp_off[kMaxJobs], exp_off[kMaxJobs], partial_off[kMaxJobs], counter_off[kMaxJobs];
};

template <bool HALF, int NT>
__device__ __forceinline__ void
multi_body(const uint8_t* __restrict__ W, const uint32_t* __restrict__ xp, const int* __restrict__ xp_exp, float* __restrict__ y,
           uint32_t rows, uint32_t cols, int m0, int M, uint32_t ldy, uint32_t g_base, uint32_t g_rem,
           uint32_t ksplit, float* __restrict__ partial, uint32_t* __restrict__ counter, int ordered, uint32_t pstride, uint32_t bid) {
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                            // 64 KB pair table, built once
    float* red = reinterpret_cast<float*>(lds + kRedBase);                 // [8 waves][kGroups][kRedTile]
    float* undo = reinterpret_cast<float*>(lds + kRedBase + kRedBytes);    // [NT][blocks of this part][16 columns]: 2^-e of the packed activations

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t li = lane & 15u, kq = lane >> 4;
    const uint32_t bpr = cols >> 8, row_bytes = bpr * 128u;
    // ksplit > 1: workgroup blockIdx.x takes part blockIdx.x % ksplit of every row (at most 16 blocks, so its
    // activations are loaded once and stay in registers) for row slab blockIdx.x / ksplit.  Two parts add into a zeroed
    // y with float atomics (two addends: the sum does not depend on their order); three or more parts write their sums
    // to `partial` and the workgroup that arrives last at the slab's counter adds them in ascending order
    uint32_t slab = bid, part = 0u;
    if (ksplit > 1u) { slab = bid / ksplit; part = bid - slab * ksplit; }   // (a uniform branch: no division otherwise)
    static_assert(NT == 1 || !HALF, "passes of 8 tokens have one token tile");
    constexpr int BPW = NT == 2 ? 1 : 2;                                   // blocks of the row per wavefront and pass
    constexpr uint32_t PB = 8u * BPW;                                      // blocks per pass
    constexpr int KG = kGroups / NT;                                       // groups of 16 rows per tile
    // Parts of near-equal length, unless full passes leave a last part of at most half a pass: block b2 of a wavefront
    // is block 8 b2 + wave of the pass, so such a part keeps every wavefront busy with one block and takes half the
    // time (56 blocks: 16 + 16 + 16 + 8 is three and a half units of work, four parts of 14 are four).
    const bool full_parts = ksplit > 1u && bpr - (ksplit - 1u) * PB <= PB / 2u;
    uint32_t blk_lo = 0u, blk_hi = bpr;
    if (full_parts) { blk_lo = part * PB; blk_hi = blk_lo + PB < bpr ? blk_lo + PB : bpr; }
    else if (ksplit > 1u) { blk_lo = bpr * part / ksplit; blk_hi = bpr * (part + 1u) / ksplit; }
    const uint32_t npass = (blk_hi - blk_lo + PB - 1u) / PB;

    // groups of 16 rows [g0, g1) of this workgroup
    auto group_begin = [&](uint32_t j) { return j * g_base + (j < g_rem ? j : g_rem); };
    const uint32_t g0 = group_begin(slab), g1 = group_begin(slab + 1);
    const uint32_t ntiles = (g1 - g0 + KG - 1) / KG;
    const uint64_t remain = (uint64_t)(rows - g0 * 16u) * row_bytes;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)g0 * 16u * row_bytes), 0, (int)(remain < 0x80000000ull ? remain : 0x80000000ull), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)xp, 0, (int)(bpr * 128u * 128u * NT), 0x00020000);

    // activations of this wavefront's two blocks (NT = 2: of its block for two token tiles), token li, chunks kq and
    // kq+4: FP16 pairs (positions 2c, 2c+1), high parts and low parts
    uint32_t bh[2][2][16], bl[HALF ? 1 : 2][HALF ? 1 : 2][HALF ? 1 : 16];
    v4f acc[kGroups];                      // [group][token tile]
    const uint32_t lanebase = (lane & 31u) * 8u;

    u32x4 wv[2][BPW][2];                   // [buffer][block of the wavefront][half]
    auto issue_group = [&](int buf, uint32_t g, uint32_t pass) {
        const uint32_t r = g * 16u + li;
#pragma unroll
        for (int b2 = 0; b2 < BPW; ++b2) {
            const uint32_t blk = blk_lo + pass * PB + (uint32_t)b2 * 8u + wave;
            const bool ok = g < g1 && r < rows && blk < blk_hi;
            const uint32_t off = (r - g0 * 16u) * row_bytes + blk * 128u + kq * 16u;
            wv[buf][b2][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? off : kOobOffset, 0, 2);
            wv[buf][b2][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? off + 64u : kOobOffset, 0, 2);
        }
    };

    // split activations of this wavefront's two blocks of K-pass `pass` -> registers: 8 (4 for passes of 8 tokens)
    // loads of 16 bytes per block half
    auto load_b = [&](uint32_t pass) {
#pragma unroll
        for (int b2 = 0; b2 < 2; ++b2) {   // NT = 2: b2 is the token tile, whose activations follow those of tile 0
            const uint32_t blk = blk_lo + pass * PB + (NT == 2 ? 0u : (uint32_t)b2 * 8u) + wave;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t off = blk < blk_hi ? (blk * 2u + h) * 8192u + lane * 16u + (NT == 2 ? b2 * bpr * 16384u : 0u) : kOobOffset;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const u32x4 vh = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off == kOobOffset ? kOobOffset : off + 1024u * j, 0, 0);
                    bh[b2][h][4 * j] = vh.x; bh[b2][h][4 * j + 1] = vh.y; bh[b2][h][4 * j + 2] = vh.z; bh[b2][h][4 * j + 3] = vh.w;
                    if constexpr (!HALF) {
                        const u32x4 vl = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off == kOobOffset ? kOobOffset : off + 4096u + 1024u * j, 0, 0);
                        bl[b2][h][4 * j] = vl.x; bl[b2][h][4 * j + 1] = vl.y; bl[b2][h][4 * j + 2] = vl.z; bl[b2][h][4 * j + 3] = vl.w;
                    }
                }
            }
        }
    };
    issue_group(0, g0, 0);                 // weights of the first group fly during the set-up
    {   // pair table from literals: entry of byte v = (b << 4 | a), lane copy c at byte v*256 + c*8 =
        // { Lh[a] | Lh[b] << 16, Ll[a] | Ll[b] << 16 }; thread tid writes float4 number tid + 512*k (two copies of
        // one entry): a = (tid >> 4) & 15 is fixed, b = (tid >> 8) + 2k is uniform across the wavefront
        const uint32_t lv_lane = split_level(level_literal(lane & 15u));
        const uint32_t pa = split_level(level_literal((tid >> 4) & 15u));
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t pb = (uint32_t)__builtin_amdgcn_readlane((int)lv_lane, (int)((tid >> 8) + 2u * k));
            const uint32_t e_hi = (pa & 0xFFFFu) | (pb << 16), e_lo = (pa >> 16) | (pb & 0xFFFF0000u);
            reinterpret_cast<uint4*>(tab)[tid + 512u * k] = make_uint4(e_hi, e_lo, e_hi, e_lo);
        }
    }
    {
        const uint32_t per_tile = (blk_hi - blk_lo) * 16u;
        for (uint32_t i = tid; i < (uint32_t)NT * per_tile; i += 512u) {
            const uint32_t t = NT == 2 && i >= per_tile ? 1u : 0u, rem = i - t * per_tile;
            // 2^-e: a bit pattern where it is a normal number, else (activations below 2^-113) the library call
            const int e = xp_exp[(t * bpr + blk_lo) * 16u + rem], be = 127 - e;
            undo[i] = be > 0 && be < 255 ? __uint_as_float((uint32_t)be << 23) : ldexpf(1.0f, -e);
        }
    }
    bool table_synced = false;

    for (uint32_t tile = 0; tile < ntiles; ++tile) {
        const uint32_t tg0 = g0 + tile * KG;
#pragma unroll
        for (int a = 0; a < kGroups; ++a) acc[a] = v4f{0.f, 0.f, 0.f, 0.f};
        for (uint32_t pass = 0; pass < npass; ++pass) {
            if (npass > 1 || tile == 0) load_b(pass);
            if (!table_synced) { __syncthreads(); table_synced = true; }   // the level table is complete
            // the (tile, pass) that follows this one: groups past the slab's last one load nothing
            const bool last_pass = pass + 1u == npass;
            const uint32_t next_tg0 = last_pass ? tg0 + KG : tg0, next_pass = last_pass ? 0u : pass + 1u;
            // ---- main loop: groups of the tile, two blocks each -------------------------------------------
#pragma unroll
            for (int g = 0; g < KG; ++g) {
                static_assert(KG % 2 == 0, "the first group of a tile lands in buffer 0");
                if (g + 1 < KG) issue_group((g + 1) & 1, tg0 + g + 1, pass);
                else issue_group(0, next_tg0, next_pass);                  // flies during the tile's sums
                const bool g_on = tg0 + g < g1;                            // wave-uniform
#pragma unroll
                for (int b2 = 0; b2 < BPW; ++b2) {
                    const bool on = g_on && blk_lo + pass * PB + (uint32_t)b2 * 8u + wave < blk_hi;     // wave-uniform
                    if (!on) continue;
                    const u32x4 w0 = wv[g & 1][b2][0], w1 = wv[g & 1][b2][1];
                    v4f t0[NT], t1[NT];                                    // this block: Lh xh, and Lh xl + Ll xh, per token tile
#pragma unroll
                    for (int t = 0; t < NT; ++t) { t0[t] = v4f{0.f, 0.f, 0.f, 0.f}; t1[t] = v4f{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const u32x4 wh = h == 0 ? w0 : w1;
                        const uint32_t wd[4] = {wh.x, wh.y, wh.z, wh.w};
                        constexpr int DS = HALF ? 4 : 2;                   // dwords decoded per batch of table reads (register budget)
#pragma unroll
                        for (int d0 = 0; d0 < 4; d0 += DS) {
                            uint32_t ah[4 * DS], al[4 * DS];
#pragma unroll
                            for (int d = 0; d < DS; ++d) {
#pragma unroll
                                for (int J = 0; J < 4; ++J) {
                                    const uint32_t addr = __builtin_amdgcn_perm(wd[d0 + d], lanebase, 0x0C0C0000u | ((4u + J) << 8));
                                    const u32x2 e = *(lds_cu32x2*)(uintptr_t)addr;
                                    ah[4 * d + J] = e.x; al[4 * d + J] = e.y;
                                }
                            }
                            __builtin_amdgcn_sched_barrier(0);             // the batch's table reads in flight before its first product
#pragma unroll
                            for (int d = 0; d < DS; ++d) {
                                const int dd = d0 + d;
                                const h8 Ah = __builtin_bit_cast(h8, u32x4{ah[4 * d], ah[4 * d + 1], ah[4 * d + 2], ah[4 * d + 3]});
                                const h8 Al = __builtin_bit_cast(h8, u32x4{al[4 * d], al[4 * d + 1], al[4 * d + 2], al[4 * d + 3]});
#pragma unroll
                                for (int t = 0; t < NT; ++t) {
                                    const int s2 = NT == 2 ? t : b2;       // register set of the activations
                                    const h8 Bh = __builtin_bit_cast(h8, u32x4{bh[s2][h][4 * dd], bh[s2][h][4 * dd + 1], bh[s2][h][4 * dd + 2], bh[s2][h][4 * dd + 3]});
                                    t0[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah, Bh, t0[t], 0, 0, 0);
                                    if constexpr (!HALF) {
                                        const h8 Bl = __builtin_bit_cast(h8, u32x4{bl[s2][h][4 * dd], bl[s2][h][4 * dd + 1], bl[s2][h][4 * dd + 2], bl[s2][h][4 * dd + 3]});
                                        t1[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah, Bl, t1[t], 0, 0, 0);
                                    }
                                    t1[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al, Bh, t1[t], 0, 0, 0);
                                }
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    // 2^-e of this lane's token column for this block (per token tile), left in LDS by the prologue
                    float unscale[NT];
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                        unscale[t] = undo[((uint32_t)t * (blk_hi - blk_lo) + pass * PB + (uint32_t)b2 * 8u + wave) * 16u + li];
                    // the block's FP16 scale of row r sits in the low half of the first dword of lane r (kq = 0)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const uint32_t sbits = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((4u * kq + v) * 4u), (int)w0.x) & 0xFFFFu;
                        const float scale = __half2float(__ushort_as_half((unsigned short)sbits));
#pragma unroll
                        for (int t = 0; t < NT; ++t)
                            acc[g * NT + t][v] = __fmaf_rn((t0[t][v] + t1[t][v]) * unscale[t], scale, acc[g * NT + t][v]);
                    }
                }
            }
        }
        // ---- tile finished: add the wavefronts' partial sums (the staging areas are idle now) ------------------
        __syncthreads();
#pragma unroll
        for (int a = 0; a < kGroups; ++a) {
            const v4f d = acc[a];
            *reinterpret_cast<float4*>(red + ((size_t)wave * kGroups + a) * kRedTile + kq * 68u + li * 4u) = make_float4(d[0], d[1], d[2], d[3]);
        }
        __syncthreads();
        constexpr uint32_t RT = KG * 16u;                                  // rows of a tile
        for (uint32_t o = tid; o < RT * 16u * NT; o += 512u) {
            const uint32_t rl = o % RT, jj = o / RT;                       // row of the tile, token of the pass
            const uint32_t g = rl >> 4, i = rl & 15u, t = jj >> 4, j = jj & 15u;
            const uint32_t r = (tg0 + g) * 16u + i;
            if (tg0 + g < g1 && r < rows && m0 + (int)jj < M && (!HALF || j < 8u)) {
                float s = 0.f;
#pragma unroll
                for (uint32_t w8 = 0; w8 < 8; ++w8) {
                    const float* cell = red + ((size_t)w8 * kGroups + g * NT + t) * kRedTile + (i >> 2) * 68u + (i & 3u);
                    s += cell[j * 4u];
                    if (HALF) s += cell[(j + 8u) * 4u];
                }
                if (ksplit == 2u || (ksplit > 2u && !ordered)) unsafeAtomicAdd(y + (size_t)(m0 + jj) * ldy + r, s);
                else if (ksplit > 2u)
                    if (ordered == 2) partial[(size_t)part * pstride + (size_t)jj * rows + r] = s;   // summed by a later launch
                    else __hip_atomic_store(&partial[((size_t)part * (uint32_t)(M - m0) + jj) * rows + r], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else y[(size_t)(m0 + jj) * ldy + r] = s;
            }
        }
        if (tile + 1 < ntiles) __syncthreads();                            // red is rewritten by the next tile
    }
    if (ksplit <= 2u || ordered != 1) return;                              // (ordered == 2: the parts are summed by the caller's next launch)
    // ---- rows cut into three or more parts: the last workgroup of the slab adds the parts in ascending order, so the result does
    // not depend on the order in which workgroups run.  The parts' sums are written and read with device-scope
    // accesses that go through to memory (no cache of another XCD can hold a stale copy), so no cache-wide write-back
    // or invalidate is needed: every thread waits until its own stores are acknowledged, the barrier collects the
    // workgroup, then one thread counts the workgroup in.  The last one leaves the counter at zero for the next launch.
    // This hand-off deliberately stays below the language's memory model: an agent-scope release (a fence, or an
    // acq_rel counter) makes the compiler write back the whole L2 of the XCD, which holds the y lines of every other
    // workgroup (measured: 40 us per part).  What it rests on instead: (1) sc1 stores are complete at device scope
    // when vmcnt reaches zero, (2) the counter's atomic is issued after the barrier that follows that wait, (3) sc1
    // loads of the reader are served from device scope, never from an XCD's L2 or a vector L1 line fetched earlier
    // (the reader has not touched these addresses before).  tests: the rows-cut-along-K cases compare three runs bit
    // for bit and against the oracle.
    volatile uint32_t* last = reinterpret_cast<volatile uint32_t*>(lds + kRedBase + kRedBytes + 8192);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        const uint32_t seen = __hip_atomic_fetch_add(&counter[slab], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *last = seen == ksplit - 1u ? 1u : 0u;
        if (seen == ksplit - 1u) __hip_atomic_store(&counter[slab], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!*last) return;
    const uint32_t r_lo = g0 * 16u, r_hi = g1 * 16u < rows ? g1 * 16u : rows, nr = r_hi - r_lo, Mp = (uint32_t)(M - m0);
    // 8 outputs x 8 parts of loads in flight per thread (device scope: sc1), so the slab's sums cost one round trip
    const uint64_t pbytes = (uint64_t)ksplit * Mp * rows * 4u;
    const __amdgpu_buffer_rsrc_t prsrc = __builtin_amdgcn_make_buffer_rsrc((void*)partial, 0, (int)(uint32_t)(pbytes < 0xFFFFFFFFull ? pbytes : 0xFFFFFFFFull), 0x00020000);
    for (uint32_t o0 = tid; o0 < nr * Mp; o0 += 512u * 8u) {
        float sum[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) sum[q] = 0.0f;
        for (uint32_t p0 = 0; p0 < ksplit; p0 += 8u) {
            float v[8][8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const uint32_t o = o0 + 512u * q, jj = o / nr, r = r_lo + o % nr;
#pragma unroll
                for (int p2 = 0; p2 < 8; ++p2) {
                    const bool ok = o < nr * Mp && p0 + p2 < ksplit;
                    const uint32_t off = ok ? (uint32_t)((((size_t)(p0 + p2) * Mp + jj) * rows + r) * 4u) : kOobOffset;
                    v[q][p2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(prsrc, off, 0, 16));
                }
            }
#pragma unroll
            for (int q = 0; q < 8; ++q)
#pragma unroll
                for (int p2 = 0; p2 < 8; ++p2) sum[q] += v[q][p2];   // parts in ascending order (absent ones read as zero)
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t o = o0 + 512u * q, jj = o / nr, r = r_lo + o % nr;
            if (o < nr * Mp) y[(size_t)(m0 + jj) * ldy + r] = sum[q];
        }
    }
}

template <bool HALF, int NT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_oil4_multi_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ xp, const int* __restrict__ xp_exp, float* __restrict__ y,
                       uint32_t rows, uint32_t cols, int m0, int M, uint32_t ldy, uint32_t g_base, uint32_t g_rem,
                       uint32_t ksplit, float* __restrict__ partial, uint32_t* __restrict__ counter, int ordered, const MultiJobs jobs) {
    uint32_t bid = blockIdx.x;
    if (jobs.n) {
        uint32_t job = 0;
        while (job + 1u < jobs.n && bid >= jobs.wg_begin[job + 1u]) ++job;   // uniform: a few scalar steps
        bid -= jobs.wg_begin[job];
        W = jobs.W[job]; y = jobs.y[job]; M = jobs.M[job];
        xp += jobs.xp_off[job]; xp_exp += jobs.exp_off[job];
        partial += jobs.partial_off[job]; counter += jobs.counter_off[job];
        g_base = jobs.g_base[job]; g_rem = jobs.g_rem[job];
    }
    multi_body<HALF, NT>(W, xp, xp_exp, y, rows, cols, m0, M, ldy, g_base, g_rem, ksplit, partial, counter, ordered, jobs.pstride, bid);
}

// `ordered` in these kernels: 0 = three or more K parts add into y with atomics, 1 = the parts meet in `partial` and the
// workgroup that arrives last sums them in ascending order, 2 (grouped launches only) = the parts are stored at
// partial[part * pstride + token * rows + row] and left for the caller's next launch to sum in ascending order.
// Batches of different pass sizes in one launch: the job's pass size selects the body, and with it the number of K
// parts (a job's workgroup count is a multiple of it).
struct MixedPlan {
    uint8_t kind[kMaxJobs];
    uint32_t ksplit[3];
};

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_oil4_multi_mixed_kernel(const uint32_t* __restrict__ xp, const int* __restrict__ xp_exp, uint32_t rows, uint32_t cols, uint32_t ldy,
                             float* __restrict__ partial, uint32_t* __restrict__ counter, int ordered, const MultiJobs jobs,
                             const MixedPlan plan) {
    uint32_t job = 0;
    while (job + 1u < jobs.n && blockIdx.x >= jobs.wg_begin[job + 1u]) ++job;
    const uint32_t bid = blockIdx.x - jobs.wg_begin[job], g_base = jobs.g_base[job], g_rem = jobs.g_rem[job];
    const uint8_t* W = jobs.W[job];
    float* y = jobs.y[job];
    const int M = jobs.M[job];
    xp += jobs.xp_off[job]; xp_exp += jobs.exp_off[job];
    partial += jobs.partial_off[job]; counter += jobs.counter_off[job];
    const uint32_t kind = plan.kind[job];                                   // workgroup-uniform
    if (kind == 0u)
        multi_body<true, 1>(W, xp, xp_exp, y, rows, cols, 0, M, ldy, g_base, g_rem, plan.ksplit[0], partial, counter, ordered, jobs.pstride, bid);
    else if (kind == 1u)
        multi_body<false, 1>(W, xp, xp_exp, y, rows, cols, 0, M, ldy, g_base, g_rem, plan.ksplit[1], partial, counter, ordered, jobs.pstride, bid);
    else
        multi_body<false, 2>(W, xp, xp_exp, y, rows, cols, 0, M, ldy, g_base, g_rem, plan.ksplit[2], partial, counter, ordered, jobs.pstride, bid);
}


// the packed activations of one pass (two token tiles) live in a scratch buffer of the stream the call runs on, or in
// the buffer the caller hands in
constexpr uint32_t kMaxPackCols = kGemvPackMaxCols;
constexpr size_t kPackBytes = kGemvPackBytes;

// The same scratch for the entry point that allocates nothing: a fixed array in the code object (8 MB, held by every
// GPU the library runs on until the process ends).  In host code the array's name is only a stand-in: the device
// address comes from hipGetSymbolAddress, once per device with that device current, and only that pointer is ever
// handed to a kernel.
// rows cut into three or more parts: sums added in a fixed order through the workspace (default), or with float atomics
std::atomic<int> g_ordered_sums{1};

constexpr size_t kStaticScratchBytes = 8u << 20;
static_assert(kStaticScratchBytes > kPackBytes + 4096u, "the static scratch holds the packed activations and the counters");
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];
std::mutex g_static_mu;
uint32_t* g_static_ptr[64] = {};

int static_pack_buffer(uint32_t** out) {
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(OILHIP_E_ARG, "device index out of range");
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (!g_static_ptr[dev]) {
        void* p = nullptr;
        OILHIP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(OILHIP_E_DEVICE, "hipGetSymbolAddress returned a null address for the static scratch");
        g_static_ptr[dev] = static_cast<uint32_t*>(p);
    }
    *out = g_static_ptr[dev];
    return OILHIP_OK;
}

}  // namespace

void g_ordered_sums_set(int v) { g_ordered_sums.store(v ? 1 : 0, std::memory_order_relaxed); }

// Y[m][r] for m < M: x row tok[m] (or m when tok is null) of an [xrows][ldx] activation matrix; with w2 the same
// activations also go through a second tensor of the same width into d_y2 (the gate and up projections of an expert):
// they are split and ordered once per pass for both.  With d_x2 (same layout as d_x) the activations are silu(x) * x2.
// Returns 1 when the shape is outside what this kernel covers.
int launch_gemv_oil4_multi(const oilhip_weights& w, const float* d_x, const int* d_tok, float* d_y, int M,
                           uint32_t ldx, uint32_t ldy, uint32_t xrows, hipStream_t s, const oilhip_weights* w2, float* d_y2,
                           uint32_t ldy2, const float* d_x2, uint32_t* d_pack, size_t pack_cap) {
    if (w.rows == 0 || w.rows > 0x7FFFFFFFull || w.cols > kMaxPackCols || (w.cols & 255u) || (uint64_t)xrows * ldx > 0x1FFFFFFFull) return 1;
    if (w2 && (w2->cols != w.cols || w2->rows == 0 || w2->rows > 0x7FFFFFFFull || !plain_oil4(*w2) || !d_y2)) return 1;
    static std::atomic<uint64_t> attr_done[3];
    if (int rc = ensure_max_lds(attr_done[0], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<false, 1>), kMaxLds)) return rc;
    if (int rc = ensure_max_lds(attr_done[1], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<false, 2>), kMaxLds)) return rc;
    if (int rc = ensure_max_lds(attr_done[2], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<true, 1>), kMaxLds)) return rc;
    const uint32_t bpr = (uint32_t)(w.cols >> 8);
    // rows wider than one K-pass (16 blocks, 8 for passes of 32 tokens): the row is cut into parts of at most one pass
    // that go to different workgroups, so that a workgroup fetches the split activations of its part once instead of
    // once per pass and tile; the parts' sums meet in a workspace behind the packed activations (4096 bytes of
    // counters, then [parts][tokens of the pass][rows] floats)
    auto split_of = [&](uint32_t pass_blocks) -> uint32_t {
        const uint32_t np = (bpr + pass_blocks - 1u) / pass_blocks;
        return np >= 2u && np <= (uint32_t)device_cu_count() ? np : 1u;
    };
    const bool ordered = g_ordered_sums.load(std::memory_order_relaxed) != 0;
    const uint64_t max_rows = w2 && w2->rows > w.rows ? w2->rows : w.rows;
    size_t need = kPackBytes;
    {
        const uint32_t ks16 = split_of(16u), ks8 = split_of(8u);
        const uint64_t parts_tokens = M > 16 ? std::max<uint64_t>((uint64_t)ks8 * 32u, (uint64_t)ks16 * 16u) : (uint64_t)ks16 * (uint64_t)(M < 16 ? M : 16);
        if (ordered && (M > 16 ? ks8 : ks16) > 2u) {
            // the kernel addresses the partial sums with 32-bit byte offsets
            if (parts_tokens * max_rows * 4u >= 0x100000000ull) return 1;
            need += 4096u + (size_t)(parts_tokens * max_rows * 4u);
        }
    }
    uint32_t* xp = d_pack;
    if (xp && pack_cap < need) return 1;                                   // the caller's buffer cannot take this shape
    if (!xp)
        if (int rc = stream_scratch(s, kScratchGemvPack, need, reinterpret_cast<void**>(&xp))) return rc;
    uint32_t* counter = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(xp) + kPackBytes);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(xp) + kPackBytes + 4096u);
    int* xp_exp = reinterpret_cast<int*>(reinterpret_cast<uint8_t*>(xp) + kGemvPackBytes - kGemvPackExpBytes);   // exponents behind the packed data
    const size_t lds_bytes = (size_t)kRedBase + kRedBytes + kGemvPackExpBytes + 64;   // table, partial sums, the activations' scale factors
    auto main_launch = [&](const oilhip_weights& t, float* y, uint32_t ld, int kind, int m0, int m1) {
        const uint32_t groups = ((uint32_t)t.rows + 15u) / 16u;
        const uint32_t ks = split_of(kind == 2 ? 8u : 16u);
        uint32_t slabs = (uint32_t)device_cu_count() / ks;
        if (slabs > groups) slabs = groups;
        auto kern = kind == 0 ? gemv_oil4_multi_kernel<true, 1> : kind == 1 ? gemv_oil4_multi_kernel<false, 1> : gemv_oil4_multi_kernel<false, 2>;
        hipLaunchKernelGGL(kern, dim3(slabs * ks), dim3(512), lds_bytes, s, t.d_payload, xp, xp_exp, y, (uint32_t)t.rows,
                           (uint32_t)t.cols, m0, m1, ld, groups / slabs, groups % slabs, ks, partial, counter, ordered ? 1 : 0, MultiJobs{});
    };
    const int x_aligned = ((reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_x2)) & 15u) == 0 && (ldx & 3u) == 0;
    for (int m0 = 0; m0 < M;) {       // passes of 32 tokens while more than 16 are left, then one of 16 or of 8
        const int left = M - m0;
        const int kind = left <= 8 ? 0 : left <= 16 ? 1 : 2;
        const int m1 = left <= 32 ? M : m0 + 32;
        const uint32_t ksp = split_of(kind == 2 ? 8u : 16u);
        const bool two = ksp == 2u || (ksp > 2u && !ordered);              // row parts that add into y, which then starts at zero
        if ((kind == 2 ? 2u : 1u) * bpr < 512u)
            hipLaunchKernelGGL(pack_x_cols_kernel, dim3((kind == 0 ? 8u : kind == 1 ? 16u : 32u) * ((bpr + 3u) / 4u)), dim3(256), 0, s, d_x, d_x2, d_tok, xp, xp_exp,
                               (uint32_t)w.cols, m0, m1, ldx, xrows, kind == 0 ? 1 : 0, two ? d_y : nullptr, (uint32_t)w.rows, ldy,
                           w2 && two ? d_y2 : nullptr, w2 ? (uint32_t)w2->rows : 0u, ldy2, PackJobs{});
        else
            hipLaunchKernelGGL(pack_x_kernel, dim3((kind == 2 ? 2u : 1u) * bpr), dim3(256), 0, s, d_x, d_x2, d_tok, xp, xp_exp,
                               (uint32_t)w.cols, m0, m1, ldx, xrows, kind == 0 ? 1 : 0, x_aligned, two ? d_y : nullptr, (uint32_t)w.rows, ldy,
                           w2 && two ? d_y2 : nullptr, w2 ? (uint32_t)w2->rows : 0u, ldy2, PackJobs{});
        OILHIP_HIP(hipGetLastError());
        main_launch(w, d_y, ldy, kind, m0, m1);
        OILHIP_HIP(hipGetLastError());
        if (w2) {
            main_launch(*w2, d_y2, ldy2, kind, m0, m1);
            OILHIP_HIP(hipGetLastError());
        }
        m0 = m1;
    }
    return OILHIP_OK;
}


// ---- several batches in one launch (the experts of a mixture-of-experts step) ---------------------------------------
// Batch b multiplies M[b] <= (8, 16, 32 for kinds[b] = 0, 1, 2) activation rows with tensor wa[b] (and, with wb, with a
// second tensor of the same shape: an expert's gate and up projections share their activations).  All tensors have
// one shape; the batches may differ in pass size (one launch then runs the three kernel bodies side by side).  The
// activation rows of batch b are rows list[row0[b] + m] of x when `list` is given (the list is passed by value with
// the launch), else rows row0[b] + m; with x2 they are silu(x) * x2.  Outputs: ya[b][m * ldy + r].
// Workspace layout: one counter page per job, then packed activations and exponents per batch (sized for two token
// tiles), then one partial-sum area per job (sized for the pass size that needs most).
namespace {
uint32_t parts_of(int kind, uint32_t bpr) {
    const uint32_t pb = kind == 2 ? 8u : 16u;
    uint32_t ks = (bpr + pb - 1u) / pb;
    if (ks < 2u || ks > (uint32_t)device_cu_count()) ks = 1u;
    return ks;
}
uint32_t tokens_of(int kind) { return kind == 0 ? 8u : kind == 1 ? 16u : 32u; }
size_t job_partial_floats(uint32_t bpr, uint64_t rows) {
    size_t m = 0;
    for (int kind = 0; kind < 3; ++kind) {
        const uint32_t ks = parts_of(kind, bpr);
        if (ks > 2u) m = std::max(m, (size_t)ks * tokens_of(kind) * rows);
    }
    return m;
}
}  // namespace

// K parts of a row of `cols` weights for a pass size (1: the row is not cut)
uint32_t gemv_oil4_multi_parts(int kind, uint64_t cols) { return parts_of(kind, (uint32_t)(cols >> 8)); }
bool gemv_oil4_multi_ordered() { return g_ordered_sums.load(std::memory_order_relaxed) != 0; }

size_t gemv_oil4_multi_batches_bytes(int nb, uint64_t rows, uint64_t cols, bool two_tensors) {
    const uint32_t bpr = (uint32_t)(cols >> 8);
    const size_t per_batch = (size_t)2 * bpr * 16384u + (size_t)2 * bpr * 64u;
    return kBatchCounterBytes + (size_t)nb * per_batch + (size_t)(two_tensors ? 2 : 1) * nb * job_partial_floats(bpr, rows) * 4u + 256u;
}

// Whether a grouped launch with passes of this size over tensors with rows of `cols` weights adds partial sums into its
// outputs with atomics (two K parts, or more with the ordered sums switched off): the outputs must then start at zero.
bool gemv_oil4_multi_batches_accumulate(int kind, uint64_t cols) {
    const uint32_t ks = parts_of(kind, (uint32_t)(cols >> 8));
    return ks == 2u || (ks > 2u && g_ordered_sums.load(std::memory_order_relaxed) == 0);
}

// The slab counters of the ordered K-split sums sit at the start of a batch workspace, one 4 KB page per job.  Every
// launch leaves them at zero, so a caller that runs several launches over one workspace clears them once.
int zero_gemv_oil4_multi_batch_counters(void* d_ws, hipStream_t s) {
    hipLaunchKernelGGL(zero_words_kernel, dim3((uint32_t)(kBatchCounterBytes / 1024u)), dim3(256), 0, s, static_cast<uint32_t*>(d_ws),
                       (uint32_t)(kBatchCounterBytes / 4u));
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int launch_gemv_oil4_multi_batches(int nb, const int* kinds, const oilhip_weights* const* wa, float* const* ya,
                                   const oilhip_weights* const* wb, float* const* yb, const int* M, const int* row0,
                                   const int* list, int nlist, const float* d_x, const float* d_x2, uint32_t ldx, uint32_t xrows,
                                   uint32_t ldy, void* d_ws, size_t ws_bytes, hipStream_t s, bool counters_clean, float* d_parts,
                                   uint32_t parts_rows) {
    if (nb < 1 || nb > kMaxJobs / (wb ? 2 : 1) || nlist > kMaxListed) return 1;
    const oilhip_weights& w0 = *wa[0];
    if (w0.rows == 0 || w0.rows > 0x7FFFFFFFull || w0.cols > kMaxPackCols || (w0.cols & 255u) || (uint64_t)xrows * ldx > 0x1FFFFFFFull) return 1;
    if (ws_bytes < gemv_oil4_multi_batches_bytes(nb, w0.rows, w0.cols, wb != nullptr)) return 1;
    static std::atomic<uint64_t> attr_done[4];
    if (int rc = ensure_max_lds(attr_done[0], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<false, 1>), kMaxLds)) return rc;
    if (int rc = ensure_max_lds(attr_done[1], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<false, 2>), kMaxLds)) return rc;
    if (int rc = ensure_max_lds(attr_done[2], reinterpret_cast<const void*>(gemv_oil4_multi_kernel<true, 1>), kMaxLds)) return rc;
    if (int rc = ensure_max_lds(attr_done[3], reinterpret_cast<const void*>(gemv_oil4_multi_mixed_kernel), kMaxLds)) return rc;
    const bool ordered = g_ordered_sums.load(std::memory_order_relaxed) != 0;
    const uint32_t bpr = (uint32_t)(w0.cols >> 8);
    bool present[3] = {false, false, false};
    for (int b = 0; b < nb; ++b) {
        if (kinds[b] < 0 || kinds[b] > 2) return 1;
        present[kinds[b]] = true;
    }
    const int nkinds = (int)present[0] + (int)present[1] + (int)present[2];
    const int only = present[0] ? 0 : present[1] ? 1 : 2;                   // the kind of a launch with one pass size
    const size_t xp_dwords = (size_t)2 * bpr * 4096u, exp_ints = (size_t)2 * bpr * 16u;
    uint32_t* counter = static_cast<uint32_t*>(d_ws);
    uint8_t* base = static_cast<uint8_t*>(d_ws) + kBatchCounterBytes;
    uint32_t* xp = reinterpret_cast<uint32_t*>(base);
    int* xp_exp = reinterpret_cast<int*>(base + (size_t)nb * xp_dwords * 4u);
    const int njobs = wb ? 2 * nb : nb;
    uint8_t* jobs_base = base + (size_t)nb * (xp_dwords * 4u + exp_ints * 4u);
    const size_t part_floats = job_partial_floats(bpr, w0.rows);
    float* partial = reinterpret_cast<float*>(jobs_base);
    // 32-bit offsets: a job's place in the areas (in dwords and floats), and bytes within one job's partial sums
    if (xp_dwords * (size_t)nb > 0xFFFFFFFFull || part_floats * (size_t)njobs > 0xFFFFFFFFull || part_floats * 4u >= 0x100000000ull) return 1;

    // The launch as a whole fills the device about twice over, so that a workgroup keeps its table and its activations
    // for many row groups.  A job's share of the workgroups follows its cost, so that all workgroups run about equally
    // long: a pass of 32 tokens counts 1.5 times a pass of 16 (1.36 on single tensors, where the fixed costs weigh
    // more), a pass of 8 the same as one of 16 (0.87 on single tensors; shares below 1 only left workgroups that end
    // late) -- the step time is flat within 1 % around these values.  A job's count is a multiple of its K parts.
    const uint32_t groups = ((uint32_t)w0.rows + 15u) / 16u;
    static const double kCost[3] = {1.0, 1.0, 1.5};
    uint32_t ks[3];
    bool any_ordered_parts = false;
    double cost_sum = 0.0;
    for (int k = 0; k < 3; ++k) {
        ks[k] = parts_of(k, bpr);
        any_ordered_parts = any_ordered_parts || (present[k] && ks[k] > 2u);
    }
    for (int b = 0; b < nb; ++b) cost_sum += kCost[kinds[b]] * (wb ? 2.0 : 1.0);
    const double total = 2.0 * (double)device_cu_count();
    MixedPlan plan{};
    for (int k = 0; k < 3; ++k) plan.ksplit[k] = ks[k];
    // d_parts: batch b's three or more K parts go to d_parts[part * parts_rows * rows + (row0[b] + m) * rows + r] and
    // are summed by the caller (one tensor per batch only: two would share the rows)
    const bool leave_parts = d_parts && ordered && any_ordered_parts && !wb;
    if (leave_parts && (uint64_t)parts_rows * w0.rows * std::max(ks[0], std::max(ks[1], ks[2])) > 0xFFFFFFFFull) return 1;
    const int x_aligned = ((reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_x2)) & 15u) == 0 && (ldx & 3u) == 0;
    // the LDS-parked pre-pass from 512 (tile, block) pairs on (the SwiGLU pre-pass of a MoE step: 1008), below that the
    // memory-to-memory one (the step's first pre-pass, 288 pairs: 3 us faster that way)
    const bool parked = (present[2] ? 2u : 1u) * bpr * (uint32_t)nb >= 512u;
    PackJobs pj{};
    pj.n = (uint32_t)nb;
    pj.wgs_per_job = parked ? (present[2] ? 2u : 1u) * bpr : tokens_of(present[2] ? 2 : present[1] ? 1 : 0) * ((bpr + 3u) / 4u);
    pj.use_list = list ? 1 : 0;
    for (int i = 0; i < nlist; ++i) pj.list[i] = list[i];
    MultiJobs mj{};
    mj.n = (uint32_t)njobs;
    pj.clear_rows = (uint32_t)w0.rows; pj.clear_ld = ldy;
    uint32_t job_slabs[kMaxJobs];
    for (int b = 0; b < nb; ++b) {
        if (M[b] < 1 || M[b] > (int)tokens_of(kinds[b])) return fail(OILHIP_E_ARG, "multi-row batches: a batch exceeds the pass size");
        pj.M[b] = M[b]; pj.row0[b] = row0[b]; pj.kind[b] = (uint8_t)kinds[b];
        pj.xp_off[b] = (uint32_t)(b * xp_dwords); pj.exp_off[b] = (uint32_t)(b * exp_ints);
        for (int t = 0; t < (wb ? 2 : 1); ++t) {
            const int j = t * nb + b;
            const oilhip_weights* w = t ? wb[b] : wa[b];
            if (!plain_oil4(*w) || w->rows != w0.rows || w->cols != w0.cols) return 1;
            mj.W[j] = w->d_payload; mj.y[j] = t ? yb[b] : ya[b]; mj.M[j] = M[b];
            mj.xp_off[j] = pj.xp_off[b]; mj.exp_off[j] = pj.exp_off[b];
            mj.partial_off[j] = leave_parts ? (uint32_t)((uint64_t)row0[b] * w0.rows) : (uint32_t)(j * part_floats);
            mj.counter_off[j] = (uint32_t)(j * 1024);
            plan.kind[j] = (uint8_t)kinds[b];
            const uint32_t k = ks[kinds[b]];
            uint32_t slabs = (uint32_t)(total * kCost[kinds[b]] / cost_sum / (double)k);   // rounded down: one workgroup past two rounds costs a third
            slabs = std::min(std::max(slabs, 1u), std::min(groups, 1024u));      // a slab holds at least one group; 1024 counters per job
            job_slabs[j] = slabs;
            mj.g_base[j] = groups / slabs; mj.g_rem[j] = groups % slabs;
        }
        // two row parts add into the outputs with atomics: the pack launch clears them
        if (gemv_oil4_multi_batches_accumulate(kinds[b], w0.cols)) { pj.clear0[b] = ya[b]; pj.clear1[b] = wb ? yb[b] : nullptr; }
    }
    for (int j = 0; j < njobs; ++j) mj.wg_begin[j + 1] = mj.wg_begin[j] + job_slabs[j] * ks[plan.kind[j]];
    const uint32_t wgs_total = mj.wg_begin[njobs];
    mj.pstride = leave_parts ? (uint32_t)((uint64_t)parts_rows * w0.rows) : 0u;
    if (leave_parts) partial = d_parts;
    const int mode = !ordered ? 0 : leave_parts ? 2 : 1;
    if (any_ordered_parts && ordered && !counters_clean && !leave_parts)  // the caller's workspace is not known to be zero
        hipLaunchKernelGGL(zero_words_kernel, dim3((uint32_t)njobs * 4u), dim3(256), 0, s, counter, (uint32_t)njobs * 1024u);
    if (parked)
        hipLaunchKernelGGL(pack_x_kernel, dim3(pj.wgs_per_job * (uint32_t)nb), dim3(256), 0, s, d_x, d_x2, (const int*)nullptr, xp, xp_exp,
                           (uint32_t)w0.cols, 0, 0, ldx, xrows, 0, x_aligned, (float*)nullptr, 0u, 0u, (float*)nullptr, 0u, 0u, pj);
    else
        hipLaunchKernelGGL(pack_x_cols_kernel, dim3(pj.wgs_per_job * (uint32_t)nb), dim3(256), 0, s, d_x, d_x2, (const int*)nullptr, xp, xp_exp,
                           (uint32_t)w0.cols, 0, 0, ldx, xrows, 0, (float*)nullptr, 0u, 0u, (float*)nullptr, 0u, 0u, pj);
    OILHIP_HIP(hipGetLastError());
    const size_t lds_bytes = (size_t)kRedBase + kRedBytes + kGemvPackExpBytes + 64;
    if (nkinds == 1) {
        auto kern = only == 0 ? gemv_oil4_multi_kernel<true, 1> : only == 1 ? gemv_oil4_multi_kernel<false, 1> : gemv_oil4_multi_kernel<false, 2>;
        hipLaunchKernelGGL(kern, dim3(wgs_total), dim3(512), lds_bytes, s, (const uint8_t*)nullptr, xp, xp_exp, (float*)nullptr,
                           (uint32_t)w0.rows, (uint32_t)w0.cols, 0, 0, ldy, 0u, 0u, ks[only], partial, counter, mode, mj);
    } else {
        hipLaunchKernelGGL(gemv_oil4_multi_mixed_kernel, dim3(wgs_total), dim3(512), lds_bytes, s, xp, xp_exp, (uint32_t)w0.rows,
                           (uint32_t)w0.cols, ldy, partial, counter, mode, mj, plan);
    }
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace oilhip

extern "C" int oilhip_gemv_oil4_f32_noalloc(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream) {
    using namespace oilhip;
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    if (!plain_oil4(*w)) return fail(OILHIP_E_ARG, "gemv_oil4_f32_noalloc: the tensor must be uniform OIL4 in the plain 128-byte block layout");
    if (w->cols > kGemvPackMaxCols)
        return fail(OILHIP_E_ARG, "gemv_oil4_f32_noalloc: rows of " + std::to_string(w->cols) + " weights exceed the static scratch (at most " +
                                      std::to_string(kGemvPackMaxCols) + " columns)");
    hipStream_t s = (hipStream_t)stream;
    int rc = 1;                                                             // 1: shape not covered by that kernel
    if (M <= 2) rc = launch_gemv_oil4(*w, d_x, d_y, M, s);                  // the register-resident kernel uses no scratch
    if (rc == 1 && M >= 2) {
        uint32_t* pack = nullptr;
        if (int e = static_pack_buffer(&pack)) return e;
        rc = launch_gemv_oil4_multi(*w, d_x, nullptr, d_y, M, (uint32_t)w->cols, (uint32_t)w->rows, (uint32_t)M, s, nullptr, nullptr, 0,
                                    nullptr, pack, kStaticScratchBytes);
    }
    if (rc == 1 && M > 2 && M <= 4) rc = launch_gemv_oil4(*w, d_x, d_y, M, s);
    if (rc == 1) return fail(OILHIP_E_ARG, "gemv_oil4_f32_noalloc: this shape needs a kernel that allocates; use oilhip_gemv_f32");
    return rc;
}

extern "C" int oilhip_set_ordered_sums(int ordered) {
    oilhip::g_ordered_sums_set(ordered);
    return OILHIP_OK;
}
