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
// multiplies by the block scale, 64 MFMAs.  The activations pass through a wave-private LDS
// staging area in natural order; each lane gathers the values of its nibble positions from it.
// Partial sums of the wavefronts are added through LDS once per tile of 64 rows.
#include <hip/hip_fp16.h>

#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using namespace oil4;

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kGroups = 4;                // groups of 16 rows per tile
constexpr int kTokStride = 132;           // floats per token in the staging area: half a block plus the overlap
constexpr int kStageBytes = 16 * kTokStride * 4;   // per wavefront: 16 tokens x 132 weights, natural order
constexpr int kStageBase = kTabBytes;     // staging areas follow the level table

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_oil4_multi_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, const int* __restrict__ tok,
                       float* __restrict__ y, uint32_t rows, uint32_t cols, int m0, int M, uint32_t ldx, uint32_t ldy,
                       uint32_t xrows, uint32_t g_base, uint32_t g_rem) {
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                            // 64 KB pair table, built once
    float* red = reinterpret_cast<float*>(lds + kStageBase);               // [8 waves][kGroups][64 lanes][4], over the staging areas

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

    float* stage = reinterpret_cast<float*>(lds + kStageBase + wave * kStageBytes);

    float breg[2][64];                     // activations of this wavefront's two blocks, token li, chunks kq and kq+4
    v4f acc[kGroups][2];                   // two accumulation chains per group: consecutive MFMAs do not wait for each other
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

    // Nibble p = 32*(kq + 4h) + s of a block holds weight i = q + q/63 with q = p - 4 (p < 4: the scale).
    // Inside a chunk q/63 steps at most once, at s = thr[h]; below it the weight index is base[h] + s.
    int32_t gbase[2], gthr[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int32_t q0 = 32 * (int32_t)(kq + 4u * h) - 4;
        const int32_t c0 = q0 >= 0 ? q0 / 63 : 0;
        const int32_t t = 63 * (c0 + 1) - q0;                              // first s with q/63 == c0 + 1
        gbase[h] = q0 + c0;
        gthr[h] = t < 32 ? t : 32;
    }

    issue_group(0, g0, 0);                 // weights of the first group fly during the set-up
    {   // pair table from literals (see gemv_oil4.hip)
        const float lv_lane = level_literal(lane & 15u);
        const float lo_fix = __int_as_float(__builtin_amdgcn_ds_bpermute((int)(((tid >> 4) & 15u) * 4u), __float_as_int(lv_lane)));
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lv_lane), (int)((tid >> 8) + 2u * k)));
            reinterpret_cast<float4*>(tab)[tid + 512u * k] = make_float4(lo_fix, hi, lo_fix, hi);
        }
    }
    bool table_synced = false;

    for (uint32_t tile = 0; tile < ntiles; ++tile) {
        const uint32_t tg0 = g0 + tile * kGroups;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) { acc[g][0] = v4f{0.f, 0.f, 0.f, 0.f}; acc[g][1] = v4f{0.f, 0.f, 0.f, 0.f}; }
        for (uint32_t pass = 0; pass < npass; ++pass) {
            if (tile > 0 || pass > 0) issue_group(0, tg0, pass);
            if (npass > 1 || tile == 0) {
                // ---- activations of this wavefront's two blocks -> registers.  The wavefront copies them in natural
                // order (one 16-byte store per lane and token) into its own staging area, half a block at a time,
                // and every lane then picks the 32 values of its token and chunk, skipping slot weights.
                if (tile > 0) __syncthreads();                             // partial sums of the previous tile have been read
#pragma unroll
                for (int b2 = 0; b2 < 2; ++b2) {
                    const uint32_t blk = pass * 16u + wave * 2u + b2;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {                          // weights 0..131 and 124..255 of the block
                        u32x4 xv[16];
#pragma unroll
                        for (int t = 0; t < 16; ++t) {
                            const int m = m0 + t;
                            const uint32_t src = m < M ? (tok ? (uint32_t)tok[m] : (uint32_t)m) : 0xFFFFFFFFu;
                            xv[t] = __builtin_amdgcn_raw_buffer_load_b128(
                                xrsrc, (lane < 33u && blk < bpr && src < xrows) ? src * ldx * 4u + (blk * 256u + h * 124u + lane * 4u) * 4u : kOobOffset, 0, 0);
                        }
                        if (lane < 33u) {
#pragma unroll
                            for (int t = 0; t < 16; ++t)
                                *reinterpret_cast<u32x4*>(stage + t * kTokStride + lane * 4u) = xv[t];
                        }
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                        {
                            // LDS byte address of the value below the step of q/63; from the step on it is one float
                            // further.  The address is made opaque so that the 64 element addresses are formed here,
                            // next to their reads, instead of being precomputed for the whole kernel.
                            uint32_t lo = (uint32_t)(kStageBase + wave * kStageBytes) + (li * kTokStride + (uint32_t)(gbase[h] - h * 124)) * 4u;
                            asm volatile("" : "+v"(lo));
                            const uint32_t thr = (uint32_t)gthr[h];
#pragma unroll
                            for (int sI = 0; sI < 32; ++sI) {
                                const uint32_t a = ((uint32_t)sI >= thr ? lo + 4u : lo) + 4u * sI;
                                const float v = *(lds_cfloat*)(uintptr_t)a;
                                if (h == 0 && sI < 4) breg[b2][sI] = kq == 0u ? 0.f : v;        // nibbles 0..3 of a block: its scale
                                else breg[b2][32 * h + sI] = v;
                            }
                        }
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    }
                }
            }
            if (!table_synced) { __syncthreads(); table_synced = true; }   // the level table is complete
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
                            acc[g][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv[k].lo * scale, breg[b2][32 * h + 2 * k], acc[g][0], 0, 0, 0);
                            acc[g][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv[k].hi * scale, breg[b2][32 * h + 2 * k + 1], acc[g][1], 0, 0, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        // ---- tile finished: add the wavefronts' partial sums (the staging areas are idle now) ------------------
        __syncthreads();
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
            const v4f d = acc[g][0] + acc[g][1];
            *reinterpret_cast<float4*>(red + (((size_t)wave * kGroups + g) * 64 + lane) * 4) = make_float4(d[0], d[1], d[2], d[3]);
        }
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
    const size_t lds_bytes = (size_t)kStageBase + 8 * (size_t)kStageBytes + 64;   // table, then staging areas / partial sums
    static_assert(8 * kStageBytes >= 8 * kGroups * 64 * 16, "the staging areas must cover the partial sums");
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
