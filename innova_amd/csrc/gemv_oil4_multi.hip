// gemv_oil4_multi.hip -- decode GEMV over uniform OIL4 tensors for a handful of activation rows
// (2..16 tokens per pass): Qwen35Engine::gemm with small B (src/adapters/tools/qwen35_engine.cpp:47-85)
// and the per-expert batches of moe_dispatch_batched (src/moe_variants.cpp:767-827).
//
// Every weight is decoded once (dequant_lattice: level * FP16 scale in FP32, bit-identical to the
// reference decode) and multiplied into all tokens on the matrix cores with the FP32 instruction
// v_mfma_f32_16x16x4_f32 (A = 16 weight rows x 4 positions, B = 4 positions x 16 tokens).
// Lane l = 16*kq + i supplies row i of a group of 16 rows; of a 128-byte block it owns the
// 16-byte chunks kq and kq+4 (64 nibbles), one nibble per instruction.  Lane 16*kq + j supplies
// token j at the same nibble positions, and accumulator register v of that lane collects
// row 4*kq + v x token j.
//
// A wavefront owns two blocks of the row per K-pass (8 wavefronts = 16 blocks = 4096 columns) and
// keeps the activations of those blocks in registers (2 x 64 per lane), so the main loop is:
// two 16-byte loads per lane and unit (16 rows x 1 block), 32 byte-pair table lookups, 64
// multiplies by the block scale, 64 MFMAs.  The activations reach nibble order through a
// wave-private LDS staging area that is reused for the 64 KB level table afterwards.  Partial
// sums of the wavefronts are added through LDS once per tile of 64 rows.
#include <hip/hip_fp16.h>

#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using namespace oil4;

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kGroups = 4;                // groups of 16 rows per tile
constexpr int kTokStride = 292;           // floats per token in the staging area: 36 mod 64 spreads 16 tokens over all banks
constexpr int kStageBytes = 16 * kTokStride * 4;   // per wavefront: 16 tokens x one block

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_oil4_multi_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, const int* __restrict__ tok,
                       float* __restrict__ y, uint32_t rows, uint32_t cols, int m0, int M, uint32_t ldx, uint32_t ldy,
                       uint32_t xrows, uint32_t g_base, uint32_t g_rem) {
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                            // 64 KB pair table (main loop)
    float* red = reinterpret_cast<float*>(lds + kTabBytes);                // [8 waves][kGroups][64 lanes][4]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t li = lane & 15u, kq = lane >> 4;
    const uint32_t bpr = cols >> 8, row_bytes = bpr * 128u;
    const uint32_t npass = (bpr + 15u) / 16u;

    // groups of 16 rows [g0, g1) of this workgroup
    auto group_begin = [&](uint32_t j) { return j * g_base + (j < g_rem ? j : g_rem); };
    const uint32_t g0 = group_begin(blockIdx.x), g1 = group_begin(blockIdx.x + 1);
    const uint32_t ntiles = (g1 - g0 + kGroups - 1) / kGroups;
    const uint64_t remain = (uint64_t)(rows - g0 * 16u) * row_bytes;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)g0 * 16u * row_bytes), 0, (int)(remain < 0x80000000ull ? remain : 0x80000000ull), 0x00020000);
    const uint64_t xbytes = (uint64_t)xrows * ldx * 4u;
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)x, 0, (int)(xbytes < 0x80000000ull ? xbytes : 0x80000000ull), 0x00020000);

    // nibble-order offsets of the four floats of float4 number `lane` of a block:
    // weight i sits at nibble p = i - i/64 + 4; position p is float (p/4 % 8)*32 + (p/32)*4 + p%4
    uint32_t xoff[4];
    bool xlast_ok;
    {
        const uint32_t w = lane * 4u;
        xlast_ok = (w & 63u) != 60u;                                       // i % 64 == 63 is a slot
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t pnib = w + k - (w >> 6) + 4u;
            xoff[k] = ((pnib >> 2) & 7u) * 32u + (pnib >> 5) * 4u + (pnib & 3u);
        }
    }
    float* stage = reinterpret_cast<float*>(lds + wave * kStageBytes);

    float breg[2][64];                     // activations of this wavefront's two blocks, token li, chunks kq and kq+4
    v4f acc[kGroups];
    const uint32_t lanebase = (lane & 31u) * 8u;

    u32x4 wv[2][2][2];                     // [buffer][block of the pair][half]
    auto issue_group = [&](int buf, uint32_t g, uint32_t pass) {
        const uint32_t r = g * 16u + li;
#pragma unroll
        for (int b2 = 0; b2 < 2; ++b2) {
            const uint32_t blk = pass * 16u + wave * 2u + b2;
            const bool ok = g < g1 && r < rows && blk < bpr;
            const uint32_t off = (r - g0 * 16u) * row_bytes + blk * 128u + kq * 16u;
            wv[buf][b2][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? off : kOobOffset, 0, 0);
            wv[buf][b2][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? off + 64u : kOobOffset, 0, 0);
        }
    };

    for (uint32_t tile = 0; tile < ntiles; ++tile) {
        const uint32_t tg0 = g0 + tile * kGroups;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) acc[g] = v4f{0.f, 0.f, 0.f, 0.f};
        for (uint32_t pass = 0; pass < npass; ++pass) {
            issue_group(0, tg0, pass);                                     // weights of the first group fly during the set-up
            if (npass > 1 || tile == 0) {
                if (tile > 0 || pass > 0) __syncthreads();                 // the table is about to be overwritten
                // ---- activations of this wavefront's two blocks -> registers, via wave-private LDS --------
                // every activation load of the pass is requested at once: one memory round trip
                u32x4 xv[2][16];
#pragma unroll
                for (int b2 = 0; b2 < 2; ++b2) {
                    const uint32_t blk = pass * 16u + wave * 2u + b2;
#pragma unroll
                    for (int t = 0; t < 16; ++t) {
                        const int m = m0 + t;
                        const uint32_t src = m < M ? (tok ? (uint32_t)tok[m] : (uint32_t)m) : 0xFFFFFFFFu;
                        xv[b2][t] = __builtin_amdgcn_raw_buffer_load_b128(
                            xrsrc, (blk < bpr && src < xrows) ? src * ldx * 4u + (blk * 256u + lane * 4u) * 4u : kOobOffset, 0, 0);
                    }
                }
#pragma unroll
                for (int b2 = 0; b2 < 2; ++b2) {
#pragma unroll
                    for (int t = 0; t < 16; ++t) {
                        float* dst = stage + t * kTokStride;
                        dst[xoff[0]] = __uint_as_float(xv[b2][t].x);
                        dst[xoff[1]] = __uint_as_float(xv[b2][t].y);
                        dst[xoff[2]] = __uint_as_float(xv[b2][t].z);
                        if (xlast_ok) dst[xoff[3]] = __uint_as_float(xv[b2][t].w);
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int c8 = 0; c8 < 8; ++c8) {
                            const float4 v = *reinterpret_cast<const float4*>(stage + li * kTokStride + c8 * 32 + (kq + 4 * h) * 4);
                            breg[b2][32 * h + 4 * c8 + 0] = v.x; breg[b2][32 * h + 4 * c8 + 1] = v.y;
                            breg[b2][32 * h + 4 * c8 + 2] = v.z; breg[b2][32 * h + 4 * c8 + 3] = v.w;
                        }
                    if (kq == 0) {                                         // nibbles 0..3 of a block hold its scale
                        breg[b2][0] = 0.f; breg[b2][1] = 0.f; breg[b2][2] = 0.f; breg[b2][3] = 0.f;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
                __syncthreads();                                           // every wavefront has left its staging area
                {   // pair table from literals (see gemv_oil4.hip)
                    const float lv_lane = level_literal(lane & 15u);
                    const float lo_fix = __int_as_float(__builtin_amdgcn_ds_bpermute((int)(((tid >> 4) & 15u) * 4u), __float_as_int(lv_lane)));
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lv_lane), (int)((tid >> 8) + 2u * k)));
                        reinterpret_cast<float4*>(tab)[tid + 512u * k] = make_float4(lo_fix, hi, lo_fix, hi);
                    }
                }
                __syncthreads();
            }
            // ---- main loop: groups of the tile, two blocks each -------------------------------------------
            LevelPair lv[16];
#pragma unroll
            for (int g = 0; g < kGroups; ++g) {
                if (g + 1 < kGroups) issue_group((g + 1) & 1, tg0 + g + 1, pass);
                const bool g_on = tg0 + g < g1;                            // wave-uniform
#pragma unroll
                for (int b2 = 0; b2 < 2; ++b2) {
                    const bool on = g_on && pass * 16u + wave * 2u + b2 < bpr;     // wave-uniform
                    if (!on) continue;
                    const u32x4 w0 = wv[g & 1][b2][0], w1 = wv[g & 1][b2][1];
                    const uint32_t sbits = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(li * 4u), (int)w0.x) & 0xFFFFu;
                    const float scale = __half2float(__ushort_as_half((unsigned short)sbits));
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        lookup_load(h == 0 ? w0 : w1, lanebase, lv);
                        __builtin_amdgcn_sched_barrier(0);                 // all 16 table reads in flight before the first multiply
#pragma unroll
                        for (int k = 0; k < 16; ++k) {
                            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv[k].lo * scale, breg[b2][32 * h + 2 * k], acc[g], 0, 0, 0);
                            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv[k].hi * scale, breg[b2][32 * h + 2 * k + 1], acc[g], 0, 0, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        // ---- tile finished: add the wavefronts' partial sums --------------------------------------------------
#pragma unroll
        for (int g = 0; g < kGroups; ++g)
            *reinterpret_cast<float4*>(red + (((size_t)wave * kGroups + g) * 64 + lane) * 4) =
                make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
        __syncthreads();
        for (uint32_t o = tid; o < kGroups * 16u * 16u; o += 512u) {
            const uint32_t rl = o & 63u, j = o >> 6;                       // row of the tile, token of the pass
            const uint32_t g = rl >> 4, i = rl & 15u;
            const uint32_t r = (tg0 + g) * 16u + i;
            if (tg0 + g < g1 && r < rows && m0 + (int)j < M) {
                float s = 0.f;
#pragma unroll
                for (uint32_t w8 = 0; w8 < 8; ++w8)
                    s += red[(((size_t)w8 * kGroups + g) * 64 + (i >> 2) * 16u + j) * 4 + (i & 3u)];
                y[(size_t)(m0 + j) * ldy + r] = s;
            }
        }
        if (tile + 1 < ntiles && npass == 1) __syncthreads();              // red is rewritten by the next tile
    }
}

}  // namespace

// Y[m][r] for m < M: x row tok[m] (or m when tok is null) of an [xrows][ldx] activation matrix.
// Returns 1 when the shape is outside what this kernel covers.
int launch_gemv_oil4_multi(const oilhip_weights& w, const float* d_x, const int* d_tok, float* d_y, int M,
                           uint32_t ldx, uint32_t ldy, uint32_t xrows, hipStream_t s) {
    if (w.rows == 0 || w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull || (uint64_t)xrows * ldx > 0x1FFFFFFFull) return 1;
    static bool attr_done = false;
    if (!attr_done) {
        OILHIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_oil4_multi_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
        attr_done = true;
    }
    const size_t lds_bytes = 8 * (size_t)kStageBytes + 64;                // covers table (64 KB) + partial sums (32 KB)
    static_assert(8 * kStageBytes >= kTabBytes + 8 * kGroups * 64 * 16, "staging area must cover table and partial sums");
    const uint32_t groups = ((uint32_t)w.rows + 15u) / 16u;
    uint32_t grid = (uint32_t)device_cu_count();
    if (grid > groups) grid = groups;
    for (int m0 = 0; m0 < M; m0 += 16) {          // passes of at most 16 tokens
        const int m1 = M - m0 < 16 ? M : m0 + 16;
        hipLaunchKernelGGL(gemv_oil4_multi_kernel, dim3(grid), dim3(512), lds_bytes, s, w.d_payload, d_x, d_tok, d_y,
                           (uint32_t)w.rows, (uint32_t)w.cols, m0, m1, ldx, ldy, xrows, groups / grid, groups % grid);
        OILHIP_HIP(hipGetLastError());
    }
    return OILHIP_OK;
}

}  // namespace oilhip
