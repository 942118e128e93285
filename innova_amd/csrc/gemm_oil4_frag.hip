// gemm_oil4_frag.hip -- prefill GEMM over uniform OIL4 tensors (any batch size; 16-byte aligned activations):
// Y[M][N] = X[M][K] . W^T, X in bf16 (or FP32, rounded once to bf16), W dequantized to bf16 on the fly,
// v_mfma_f32_32x32x16_bf16 with FP32 accumulation, FP32 output.  Same contraction as the reference's FP32
// prefill (Qwen35Engine::gemm with B up to 512, src/adapters/tools/qwen35_engine.cpp:47-85,630-753) over
// dequant_lattice blocks (src/block_codec.cpp:173-182).
//
// Shape of the kernel.  A workgroup is four wavefronts, one per SIMD, as 2 x 2; a wavefront owns FM x FN
// blocks of 32 x 32 outputs (4 x 4: a 256 x 256 workgroup tile, 256 accumulator registers per lane), so one
// 16-byte operand fragment feeds four matrix instructions.
//  * Activations never pass through LDS.  A pre-pass writes X' in the order the matrix instruction wants its
//    A operand: [32-token block][16-column group][lane][8 bf16], columns in nibble order (the 4-bit index of
//    weight i of a 256-weight block sits at nibble 4 + i - i/64; nibbles 0..3 are the FP16 scale and meet
//    zeros in X').  A fragment is then one coalesced 1 KB load straight into registers, issued two 64-column
//    steps ahead through a buffer resource (the scalar offset of a step is clamped on the host side of the loop:
//    the hardware does not range-check it).
//  * Weights: a lane loads 16 bytes (32 nibbles) of one weight row per step, four steps ahead.  Every packed byte
//    becomes an LDS address (v_perm_b32) into a 64 KB table whose row v holds 64 lane-private copies of the FP16 pair
//    (level[v & 15], level[v >> 4]); a 4-byte read returns both levels, v_fma_mix_f32 multiplies each by the block's
//    FP16 scale in FP32, one v_cvt_pk_bf16_f32 rounds the pair, and 16-byte stores put the result in B-operand
//    fragment order.  Each weight is decoded once per workgroup; the four wavefronts read the fragments back with
//    conflict-free 16-byte LDS reads.  Two tile buffers, one workgroup barrier per step: the fragments of step s
//    are read and the tile of step s + 1 is written between the same two barriers.
//  * Issue order is fixed by hand.  A 32x32x16 matrix instruction keeps the wavefront's issue port for half of its
//    32 cycles, which leaves four slots for other instructions; the decode of a step is cut into quarters of three
//    stages (addresses, table reads, multiply/round/store) that ride in those slots behind the four groups of sixteen
//    matrix instructions of a step, every side instruction at a fixed place (a scheduling barrier after each
//    matrix instruction), fragment re-reads after the last use of a register, A loads after the group's last
//    matrix instruction.
//  * A shape whose tiles do not fill whole rounds of compute units runs its last round as half tiles: 256 tokens x
//    128 rows with all of K (no partial sums) for the 256 x 256 tiling; two K halves added into a zeroed Y with
//    float atomics (two addends: the sum does not depend on their order) for the 128 x 128 tiling.  Tile order
//    keeps the workgroups of one XCD on few token blocks and neighbouring weight rows so that its L2 serves most of
//    their reads.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using oil4::kTabBytes;
using oil4::level_literal;
using oil4::LevelPair;
using oil4::lookup;
using oil4::u32x4;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Tile order: token blocks in groups of four; inside a group weight-row blocks ascending, the group's token blocks
// innermost.  A run of consecutive tiles therefore covers few token blocks and neighbouring weight rows.
__host__ __device__ inline void frag_tile_of(uint32_t T, uint32_t MT, uint32_t NT, uint32_t& mt, uint32_t& nt) {
    const uint32_t per = 4u * NT, lastg = (MT - 1u) / 4u;
    uint32_t mg = T / per;
    if (mg > lastg) mg = lastg;
    const uint32_t rem = T - mg * per, left = MT - 4u * mg, gm = left < 4u ? left : 4u;
    nt = rem / gm;
    mt = 4u * mg + rem % gm;
}

// Workgroups are dealt to the eight XCDs in turn; XCD x takes the x-th run of n / 8 consecutive items.
__device__ inline uint32_t xcd_chunk(uint32_t b, uint32_t n) {
    const uint32_t x = b & 7u, q = b >> 3, c = n >> 3, r = n & 7u;
    return (x < r ? x * (c + 1u) : r * (c + 1u) + (x - r) * c) + q;
}

struct FragGrid {
    uint32_t MT, NT;        // tiles along tokens and weight rows
    uint32_t nfull;         // the first nfull tiles (in tile order) run all of K in one workgroup
    uint32_t ksplit;        // the others are cut into this many parts along K (1 or 2) ...
    uint32_t halves;        // ... or into two halves along the weight rows (2; 256-row tiles only), each with all of K
};

// X ([M][K], bf16 bit patterns or FP32) -> X' in A-fragment order, rows >= M zero: fragment (32-token block, 16-column
// group g) is 1 KB, lane = 32 * (column half) + token % 32 holds columns 16 g + 8 half .. + 7 of X' (nibble order).
// Workgroups past the packing ones clear the Y tiles whose K parts are added: tile nfull + (index).
template <bool F32, int TM, int TN>
__global__ void __launch_bounds__(256)
pack_x_frag_kernel(const void* __restrict__ xin, uint16_t* __restrict__ xf, uint32_t M, uint32_t K, uint32_t npack,
                   float* __restrict__ y, uint32_t N, uint32_t ldy, FragGrid gr) {
    const uint32_t tid = threadIdx.x;
    if (blockIdx.x >= npack) {
        uint32_t mt, nt;
        frag_tile_of(gr.nfull + (blockIdx.x - npack), gr.MT, gr.NT, mt, nt);
        const uint32_t m0 = mt * TM, n0 = nt * TN;
        const uint32_t nc = N - n0 < (uint32_t)TN ? N - n0 : (uint32_t)TN;
        for (uint32_t r = tid >> 6; r < (uint32_t)TM && m0 + r < M; r += 4u) {
            float* yr = y + (size_t)(m0 + r) * ldy + n0;
            for (uint32_t c = tid & 63u; c < nc; c += 64u) yr[c] = 0.0f;
        }
        return;
    }
    // One workgroup = 32 tokens x one 256-column block: rows are read whole (a wavefront reads eight rows of 512
    // bytes, FP32: 1 KB), rounded to bf16 and parked in LDS; then every wavefront writes four of the block's sixteen
    // 1 KB fragments.  X' column p of a block (p >= 4) is X column p - 4 + (slots before it): the eight columns of a
    // lane come from the 16 aligned X columns [c - 8, c + 8) of the block, window index k + 4 + slots.
    constexpr uint32_t PITCH = 256u + 8u;                                    // bf16 per parked row: 16-byte reads of 16 rows hit every bank once
    __shared__ __align__(16) uint16_t park[32u * PITCH];
    const uint32_t bpr = K >> 8, G = K >> 4;
    const uint32_t mb = blockIdx.x / bpr, blk = blockIdx.x % bpr;
    {
        const uint32_t r = tid >> 3, q = tid & 7u, m = mb * 32u + r;         // row of the tile; 8-column pieces q, q + 8, q + 16, q + 24 of it
        uint4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = make_uint4(0u, 0u, 0u, 0u);
        if (m < M) {
            if constexpr (F32) {
                const float4* xr = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xin) + (size_t)m * K + blk * 256u);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float4 f0 = xr[2u * (q + 8u * j)], f1 = xr[2u * (q + 8u * j) + 1u];
                    const bf16x2 p0 = bf16x2{(__bf16)f0.x, (__bf16)f0.y}, p1 = bf16x2{(__bf16)f0.z, (__bf16)f0.w};
                    const bf16x2 p2 = bf16x2{(__bf16)f1.x, (__bf16)f1.y}, p3 = bf16x2{(__bf16)f1.z, (__bf16)f1.w};
                    v[j] = make_uint4(*reinterpret_cast<const uint32_t*>(&p0), *reinterpret_cast<const uint32_t*>(&p1),
                                      *reinterpret_cast<const uint32_t*>(&p2), *reinterpret_cast<const uint32_t*>(&p3));
                }
            } else {
                const uint4* xr = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(xin) + (size_t)m * K + blk * 256u);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = xr[q + 8u * j];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint4*>(park + r * PITCH + (q + 8u * j) * 8u) = v[j];
    }
    __syncthreads();
    const uint32_t lane = tid & 63u, r = lane & 31u, half = lane >> 5;
#pragma unroll
    for (int f = 0; f < 4; ++f) {
        const uint32_t gl = (tid >> 6) + 4u * f, p0 = gl * 16u + half * 8u;   // fragment of the block, first X' column of the lane
        uint4 w0 = make_uint4(0u, 0u, 0u, 0u);
        if (p0 != 0u) w0 = *reinterpret_cast<const uint4*>(park + r * PITCH + p0 - 8u);
        const uint4 w1 = *reinterpret_cast<const uint4*>(park + r * PITCH + p0);
        const uint32_t wd[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        uint16_t e[16];
#pragma unroll
        for (int k = 0; k < 8; ++k) { e[2 * k] = (uint16_t)wd[k]; e[2 * k + 1] = (uint16_t)(wd[k] >> 16); }
        uint16_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t p = p0 + k, sl = (p >= 67u) + (p >= 130u) + (p >= 193u);
            const uint16_t t = sl == 0u ? e[k + 4] : sl == 1u ? e[k + 5] : sl == 2u ? e[k + 6] : e[k + 7];
            v[k] = p >= 4u ? t : (uint16_t)0;
        }
        uint4 o;
        o.x = v[0] | ((uint32_t)v[1] << 16); o.y = v[2] | ((uint32_t)v[3] << 16);
        o.z = v[4] | ((uint32_t)v[5] << 16); o.w = v[6] | ((uint32_t)v[7] << 16);
        *reinterpret_cast<uint4*>(xf + (((size_t)mb * G + blk * 16u + gl) * 64u + lane) * 8u) = o;
    }
}

template <int V> using IC = std::integral_constant<int, V>;

constexpr int kFragAhead = 2;

// One workgroup's tile: tokens [m0, m0 + 64 FM), weight rows [n0, n0 + 64 FN), part kpart of `parts` along K.
template <int FM, int FN>
__device__ __forceinline__ void frag_tile(const uint8_t* __restrict__ W, const uint16_t* __restrict__ Xf, float* __restrict__ Y,
                                          uint32_t M, uint32_t N, uint32_t K, uint32_t ldy, uint32_t m0, uint32_t n0,
                                          uint32_t kpart, uint32_t parts) {
    static_assert((FN == 2 || FN == 4) && (FM == 2 || FM == 4), "wavefront tiles of 64 or 128 tokens and weight rows");
    constexpr int TN = 64 * FN;                     // weight rows of the workgroup tile
    constexpr int NB = TN / 32;                     // 32-row blocks of weight rows in the tile
    constexpr int NBW = NB / 4;                     // ... that one wavefront decodes
    constexpr int BUF = NB * 4096;                  // bytes of one tile buffer: [NB][4 column groups][64 lanes][16 B]
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t* tab = reinterpret_cast<uint32_t*>(lds);   // pair table at LDS offset 0 (the look-up builds absolute addresses)

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));    // scalar: buffer resources and LDS bases depend on it
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t bpr = K >> 8, G = K >> 4;
    // steps of 64 columns [kbeg, kend): whole blocks, so that both are multiples of 4
    const uint32_t bsplit = (bpr + parts - 1u) / parts;
    const uint32_t kbeg = kpart * bsplit * 4u, kend = (kpart + 1u == parts ? bpr : (kpart + 1u) * bsplit) * 4u;

    {   // pair table from literals: row v (256 bytes) = 64 copies of fp16(level[v & 15]) | fp16(level[v >> 4]) << 16;
        // uint4 e = tid + 256 * k belongs to row e >> 4: low level (tid >> 4) & 15, high level k
        const uint32_t lv_lane = (uint32_t)__half_as_ushort(__float2half_rn(level_literal(lane & 15u)));
        const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(((tid >> 4) & 15u) * 4u), (int)lv_lane);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const uint32_t e = lo | ((uint32_t)__half_as_ushort(__float2half_rn(level_literal(k))) << 16);
            reinterpret_cast<uint4*>(tab)[tid + 256u * k] = make_uint4(e, e, e, e);
        }
    }

    const uint32_t nrows = N - n0 < (uint32_t)TN ? N - n0 : (uint32_t)TN;
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)n0 * bpr * 128u), 0, (int)((uint64_t)nrows * bpr * 128u), 0x00020000);
    const uint32_t r32 = lane & 31u, hh = lane >> 5;
    const uint32_t lanebase = lane * 4u;                   // this lane's copy of a table row
    // weight bytes of this lane: row (wave * NBW + j) * 32 + r32 of the tile, 16 bytes at step * 32 + hh * 16
    uint32_t woff[NBW];
#pragma unroll
    for (int j = 0; j < NBW; ++j) woff[j] = ((wave * NBW + j) * 32u + r32) * bpr * 128u;
    // A fragments through a buffer resource over this wavefront's FM token blocks: lane part in the vector offset,
    // the 16-column group in the scalar offset, no address arithmetic per load
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(Xf + ((size_t)(m0 / 32u + wm * FM) * G) * 512u), 0, (int)((uint32_t)FM * G * 1024u), 0x00020000);
    uint32_t xoff[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) xoff[i] = (uint32_t)i * G * 1024u + lane * 16u;

    const uint32_t klast = bpr * 4u - 1u;                 // last 64-column step of a row
    constexpr int AD = kFragAhead;  // steps of A fragments in flight
    u32x4 fa[AD][4][FM];        // A fragments of AD steps: set = step % AD, slot = column group of the step
    u32x4 fb[FN];               // B fragments of the column group in work; each is re-read for the next group after its last use
    u32x4 wr[4][NBW];           // packed weights of four steps in flight, slot = step & 3
    float scA[NBW], scB[NBW];   // block scales of the current and the next 256-column block
    uint32_t scraw[NBW];
    // decode pipeline, one quarter of a step per group of matrix instructions and three quarters in flight: table
    // addresses of quarter g + 2, table reads of quarter g + 1, scale + round + store of quarter g
    uint32_t tadr[NBW][4];
    uint32_t tv[2][NBW][4];

    // set = step & 1, slot = column group of the step; sbase = byte offset of the step's first column group.  Loads
    // run two steps ahead: with the matrix pipe and the LDS returns busy, a fragment that misses L2 needs more than
    // one step to arrive.
    auto load_a1 = [&](int set, int slot, int i, uint32_t sbase) {
        fa[set][slot][i] = __builtin_amdgcn_raw_buffer_load_b128(xrs, xoff[i] + (uint32_t)slot * 1024u, sbase, 0);
    };
    auto load_w = [&](int slot, uint32_t step) {
#pragma unroll
        for (int j = 0; j < NBW; ++j) wr[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(wrs, woff[j] + hh * 16u, step * 32u, 0);
    };
    auto load_scale = [&](uint32_t blk) {
#pragma unroll
        for (int j = 0; j < NBW; ++j) scraw[j] = __builtin_amdgcn_raw_buffer_load_b16(wrs, woff[j], blk * 128u, 0);
    };
    auto cvt_scale = [&](float (&dst)[NBW]) {
#pragma unroll
        for (int j = 0; j < NBW; ++j) dst[j] = __half2float(__ushort_as_half((unsigned short)scraw[j]));
    };
    // A quarter of a step's decode is NBW dwords (8 nibbles each) per lane -> NBW 16-byte pieces in fragment order.
    // Quarter q, piece t is dword (q * NBW + t) % 4 of the lane's 16 bytes of weight-row block (q * NBW + t) / 4.
    auto q_addr = [&](int q, int slot, int t, int b) {
        const int e = q * NBW + t, j = e >> 2, d = e & 3;
        const uint32_t word = d == 0 ? wr[slot][j].x : d == 1 ? wr[slot][j].y : d == 2 ? wr[slot][j].z : wr[slot][j].w;
        tadr[t][b] = __builtin_amdgcn_perm(word, lanebase, 0x0C0C0000u | ((4u + (uint32_t)b) << 8));
    };
    auto q_read = [&](int set, int t, int b) { tv[set][t][b] = *(oil4::lds_cuint*)(uintptr_t)tadr[t][b]; };
    uint32_t tout[NBW][4];
    // FP16 level x FP32 scale in one instruction each (v_fma_mix_f32; the product is exact in FP32), rounded once to
    // bf16.  The rounding reads its operands one place after the products write them: placed right behind them it
    // costs a wait state each time.
    float tlo[NBW][4], thi[NBW][4];
    auto q_mul = [&](int set, int t, int b, float s) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const f16x2 h = *reinterpret_cast<const f16x2*>(&tv[set][t][b]);
        tlo[t][b] = __builtin_fmaf((float)h.x, s, 0.0f);
        thi[t][b] = __builtin_fmaf((float)h.y, s, 0.0f);
    };
    auto q_round = [&](int t, int b) {
        const bf16x2 o = bf16x2{(__bf16)tlo[t][b], (__bf16)thi[t][b]};
        tout[t][b] = *reinterpret_cast<const uint32_t*>(&o);
    };
    auto q_math = [&](int set, int t, int b, float s) { q_mul(set, t, b, s); q_round(t, b); };
    const uint32_t wbase = kTabBytes + wave * (NBW * 4096u) + hh * 2048u + r32 * 16u;
    auto q_store = [&](int q, int t, int buf) {
        const int e = q * NBW + t, j = e >> 2, d = e & 3;
        *reinterpret_cast<u32x4*>(lds + wbase + buf * BUF + j * 4096 + (d >> 1) * 1024 + (d & 1) * 512) =
            u32x4{tout[t][0], tout[t][1], tout[t][2], tout[t][3]};
    };
    const uint32_t rbase = kTabBytes + wn * (FN * 4096u) + lane * 16u;
    auto read_frag1 = [&](int kk, int buf, int j) {
        fb[j] = *reinterpret_cast<const u32x4*>(lds + rbase + buf * BUF + j * 4096 + kk * 1024);
    };
    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    auto mfma1 = [&](int as, int kk, int i, int j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&fa[as][kk][i]),
                                                            *reinterpret_cast<const bf16x8*>(&fb[j]), acc[i][j], 0, 0, 0);
    };

    // One group: the FM * FN matrix instructions of column group kk of a step (B fragment outermost, so that a
    // fragment's registers are free for the next group's after FM instructions) and, in fixed places between them
    // (nothing moves across a matrix instruction): scale, round and store of quarter q0 (table entries of set
    // kk & 1) into buffer wbuf; the table reads of the quarter after it; the table addresses of quarter q2 of the
    // weights in slot s2 (each written after the read that used its register); the fragment reads of column group rk
    // of buffer rbuf; after the last instruction the A fragments of the step after next.
    // A wavefront alone on its SIMD issues one instruction per four clocks, and a 32x32x16 matrix instruction
    // holds the issue port for 16 of its 32: four other instructions ride for free behind each, a fifth delays
    // the next one.  The places below keep the gaps at four or fewer (five behind the last).  Table entries and A
    // fragments are consumed youngest first, so that one wait covers all of them.
    auto group = [&](auto kkc, int as, int q0, int wbuf, const float (&sc)[NBW], int q2, int s2, int rk, int rbuf, uint32_t abase) {
        constexpr int kk = decltype(kkc)::value, cs = kk & 1, ns = cs ^ 1;
        constexpr int NM = FM * FN, NU = NBW * 4;            // matrix instructions, decode units (bytes per lane) of the group
        // place of math unit k (k-th in processing order) together with the table read of unit k
        auto mslot = [](int k) { return NM == 16 ? k + k / 4 : NM == 8 ? k : k / 2; };
        // place of the two (NM == 4: four) table addresses from u on: behind the read that used the register
        auto pslot = [](int u) { return NM == 16 ? (u < 2 ? 4 : 8 + u / 2) : NM == 8 ? 4 + u / 2 : 3; };
#pragma unroll
        for (int n = 0; n < NM; ++n) {
            const int j = n / FM, i = FM - 1 - n % FM;           // A fragment FM - 1 (the youngest load) first
            mfma1(as, kk, i, j);
#pragma unroll
            for (int k = 0; k < NU; ++k) {
                if (mslot(k) != n) continue;
                const int un = NU - 1 - k;                       // youngest table entry first
                q_mul(cs, un >> 2, un & 3, sc[(q0 * NBW + (un >> 2)) >> 2]);
                q_read(ns, k >> 2, k & 3);
            }
#pragma unroll
            for (int k = 0; k < NU; ++k)                         // rounding of the unit whose products sit one place back
                if (mslot(k) + 1 == n) { const int un = NU - 1 - k; q_round(un >> 2, un & 3); }
#pragma unroll
            for (int t = 0; t < NBW; ++t)                        // piece t is complete behind the rounding of its unit 4 t
                if (mslot(NU - 1 - 4 * t) + 1 == n) q_store(q0, t, wbuf);
            if (n % FM == FM - 1 && (NM != 16 || (n != 3 && n != 7))) read_frag1(rk, rbuf, j);
            if (NM == 16 && (n == 4 || n == 9)) read_frag1(rk, rbuf, n == 4 ? 0 : 1);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (pslot(u) == n) q_addr(q2, s2, u >> 2, u & 3);
            if (n == NM - 1) {
#pragma unroll
                for (int ii = 0; ii < FM; ++ii) load_a1(as, kk, ii, abase);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- prologue: loads of the first steps; tile kbeg whole and the first quarter of tile kbeg + 1 decoded, the
    // second quarter's table entries read and the third's addresses formed
    load_w(1, kbeg + 1u);                                 // (a part is at least one block: four steps)
    load_w(2, kbeg + 2u);
    load_w(3, kbeg + 3u);
    load_w(0, kbeg);
    // both scales ahead of the A loads: every wait on them then leaves a whole step of loads in flight
    uint32_t scraw0[NBW], scraw1[NBW];
#pragma unroll
    for (int j = 0; j < NBW; ++j) {
        scraw0[j] = __builtin_amdgcn_raw_buffer_load_b16(wrs, woff[j], (kbeg >> 2) * 128u, 0);
        scraw1[j] = __builtin_amdgcn_raw_buffer_load_b16(wrs, woff[j], ((kbeg >> 2) + 1u < bpr ? (kbeg >> 2) + 1u : bpr - 1u) * 128u, 0);
    }
#pragma unroll
    for (int d = 0; d < AD; ++d)
#pragma unroll
        for (int kk = 0; kk < (d == AD - 1 ? 3 : 4); ++kk)
#pragma unroll
            for (int i = 0; i < FM; ++i) load_a1(d, kk, i, (kbeg + d < klast ? kbeg + d : klast) * 4096u);
#pragma unroll
    for (int j = 0; j < NBW; ++j) {
        scA[j] = __half2float(__ushort_as_half((unsigned short)scraw0[j]));
        scB[j] = __half2float(__ushort_as_half((unsigned short)scraw1[j]));
    }
    __syncthreads();                                   // table complete
    auto whole = [&](int q, int slot, int buf) {
#pragma unroll
        for (int t = 0; t < NBW; ++t) {
#pragma unroll
            for (int b = 0; b < 4; ++b) { q_addr(q, slot, t, b); q_read(0, t, b); }
#pragma unroll
            for (int b = 0; b < 4; ++b) q_math(0, t, b, scA[(q * NBW + t) >> 2]);
            q_store(q, t, buf);
        }
    };
    whole(0, 0, 0); whole(1, 0, 0); whole(2, 0, 0); whole(3, 0, 0);
    whole(0, 1, 1);                                    // nobody reads buffer 1 yet
#pragma unroll
    for (int t = 0; t < NBW; ++t)
#pragma unroll
        for (int b = 0; b < 4; ++b) { q_addr(1, 1, t, b); q_read(0, t, b); q_addr(2, 1, t, b); }
    load_w(0, kbeg + 4u < klast ? kbeg + 4u : klast);
#pragma unroll
    for (int i = 0; i < FM; ++i) load_a1(AD - 1, 3, i, (kbeg + AD - 1u < klast ? kbeg + AD - 1u : klast) * 4096u);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < FN; ++j) read_frag1(0, 0, j);

    // ---- main loop: one 256-column block (four steps) per trip.  In step s (u = s & 3, tile s in buffer u & 1) the
    // groups 0..2 read the fragments of column groups 1..3 and finish the quarters 1..3 of tile s + 1 into the other
    // buffer; after the barrier group 3 reads the first fragments of tile s + 1 and finishes the first quarter of
    // tile s + 2 into the buffer that tile s has just left.  Tile s + 1 belongs to the next block from u = 3 on,
    // tile s + 2 from u = 2 on.  The weights of tile s + 5 replace those of tile s + 1 once its last table addresses
    // are formed (group 0).
    auto step = [&](auto uc, uint32_t s) {
        constexpr int u = decltype(uc)::value, cur = u & 1, nxt = cur ^ 1, s1 = (u + 1) & 3, s2 = (u + 2) & 3;
        const float (&sc1)[NBW] = u == 3 ? scB : scA;
        const float (&sc2)[NBW] = u >= 2 ? scB : scA;
        // steps past the end of the row are loaded and never used; the scalar offsets are outside the buffer range
        // check, so they are clamped to the row's last step / block
        const uint32_t an = (s + AD < klast ? s + AD : klast) * 4096u;
        constexpr int as = u % AD;
        group(IC<0>{}, as, 1, nxt, sc1, 3, s1, 1, cur, an);
        group(IC<1>{}, as, 2, nxt, sc1, 0, s2, 2, cur, an);
        group(IC<2>{}, as, 3, nxt, sc1, 1, s2, 3, cur, an);
        load_w(s1, s + 5u < klast ? s + 5u : klast);
        if constexpr (u == 0) load_scale((s >> 2) + 2u < bpr - 1u ? (s >> 2) + 2u : bpr - 1u);
        __syncthreads();
        group(IC<3>{}, as, 0, cur, sc2, 2, s2, 0, nxt, an);
    };
    for (uint32_t s = kbeg; s < kend; s += 4u) {
        step(IC<0>{}, s);
        step(IC<1>{}, s + 1u);
        step(IC<2>{}, s + 2u);
        step(IC<3>{}, s + 3u);
#pragma unroll
        for (int j = 0; j < NBW; ++j) scA[j] = scB[j];
        cvt_scale(scB);
    }

    // C layout of the 32x32 matrix instruction: lane l holds column l % 32; register v holds row 8 * (v / 4) + 4 * (l / 32) + v % 4
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const uint32_t col = n0 + (wn * FN + j) * 32u + r32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + (wm * FM + i) * 32u + 8u * (v >> 2) + 4u * hh + (v & 3u);
                if (row < M && col < N) {
                    if (parts > 1u) unsafeAtomicAdd(Y + (size_t)row * ldy + col, acc[i][j][v]);
                    else Y[(size_t)row * ldy + col] = acc[i][j][v];
                }
            }
        }
}

template <int FM, int FN>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_oil4_frag_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ Xf, float* __restrict__ Y,
                      uint32_t M, uint32_t N, uint32_t K, uint32_t ldy, FragGrid gr) {
    constexpr int TM = 64 * FM, TN = 64 * FN;
    const uint32_t b = blockIdx.x;
    uint32_t mt, nt;
    if (b < gr.nfull) {
        frag_tile_of(xcd_chunk(b, gr.nfull), gr.MT, gr.NT, mt, nt);
        frag_tile<FM, FN>(W, Xf, Y, M, N, K, ldy, mt * TM, nt * TN, 0u, 1u);
        return;
    }
    // the tiles of the last round, in two pieces each: 256-row tiles as halves of 128 weight rows, others as halves of K
    const uint32_t u = xcd_chunk(b - gr.nfull, (gr.MT * gr.NT - gr.nfull) * 2u);
    frag_tile_of(gr.nfull + u / 2u, gr.MT, gr.NT, mt, nt);
    if constexpr (FN == 4) {
        const uint32_t n0 = nt * TN + (u & 1u) * (TN / 2);
        if (n0 < N) frag_tile<FM, 2>(W, Xf, Y, M, N, K, ldy, mt * TM, n0, 0u, 1u);
    } else {
        frag_tile<FM, FN>(W, Xf, Y, M, N, K, ldy, mt * TM, nt * TN, u & 1u, 2u);
    }
}

template <int FM, int FN, bool F32>
int launch_frag(const oilhip_weights& w, const void* d_x, float* d_y, uint32_t M, hipStream_t s) {
    constexpr int TM = 64 * FM, TN = 64 * FN;
    const uint32_t N = (uint32_t)w.rows, K = (uint32_t)w.cols, cus = (uint32_t)device_cu_count();
    FragGrid gr;
    gr.MT = (M + TM - 1) / TM;
    gr.NT = (N + TN - 1) / TN;
    const uint32_t tiles = gr.MT * gr.NT, tail = tiles % cus;
    // A last round that fills at most half of the compute units is cut in two: 256-row tiles into halves of 128 weight
    // rows (each with all of K: no partial sums), smaller tiles along K (two addends into a cleared Y; a row of one
    // block cannot be cut).
    const bool split = tail != 0u && tail * 2u <= cus && (FN == 4 || K >= 512u);
    gr.nfull = split ? tiles - tail : tiles;
    gr.halves = split && FN == 4 ? 2u : 1u;
    gr.ksplit = split && FN != 4 ? 2u : 1u;
    const uint32_t Mpad = gr.MT * TM;
    uint16_t* xf = nullptr;
    if (int rc = stream_scratch(s, kScratchGemmX, (size_t)Mpad * K * 2, reinterpret_cast<void**>(&xf))) return rc;
    const uint32_t npack = (Mpad / 32u) * (K >> 8), nzero = gr.ksplit > 1u ? tiles - gr.nfull : 0u;
    hipLaunchKernelGGL((pack_x_frag_kernel<F32, TM, TN>), dim3(npack + nzero), dim3(256), 0, s, d_x, xf, M, K, npack, d_y, N, N, gr);
    OILHIP_HIP(hipGetLastError());
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemm_oil4_frag_kernel<FM, FN>;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
    const size_t lds_bytes = (size_t)kTabBytes + 2ull * (TN / 32) * 4096;
    hipLaunchKernelGGL(kern, dim3(gr.nfull + (tiles - gr.nfull) * (split ? 2u : 1u)), dim3(256), lds_bytes, s, w.d_payload, xf, d_y, M, N, K, N, gr);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace

// Prefill over a plain uniform OIL4 tensor with the fragment-order kernel; x is bf16 bit patterns, or FP32 when x_is_f32.
int launch_gemm_oil4_frag(const oilhip_weights& w, const void* d_x, bool x_is_f32, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull) return fail(OILHIP_E_ARG, "matrix too large for the prefill kernel");
    const uint32_t N = (uint32_t)w.rows, K = (uint32_t)w.cols, cus = (uint32_t)device_cu_count();
    // 32-bit byte offsets inside a workgroup's 256 weight rows and inside a wavefront's four token blocks of X'
    if ((uint64_t)256 * (K >> 8) * 128u >= 0x80000000ull || (uint64_t)K * 256u >= 0x80000000ull)
        return fail(OILHIP_E_ARG, "rows too wide for the prefill kernel");
    // 256 x 256 tiles unless they would leave three quarters of the compute units without work even when cut along K
    const uint32_t big_tiles = (((uint32_t)M + 255u) / 256u) * ((N + 255u) / 256u);
    const bool small = big_tiles * 4u <= cus;
    if (small) return x_is_f32 ? launch_frag<2, 2, true>(w, d_x, d_y, (uint32_t)M, s) : launch_frag<2, 2, false>(w, d_x, d_y, (uint32_t)M, s);
    return x_is_f32 ? launch_frag<4, 4, true>(w, d_x, d_y, (uint32_t)M, s) : launch_frag<4, 4, false>(w, d_x, d_y, (uint32_t)M, s);
}

}  // namespace oilhip
