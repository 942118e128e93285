// gemv_oil4.hip -- decode GEMV over uniform OIL4 tensors (128-byte blocks), the
// HBM-bound kernel of the decode path (Qwen35Engine::gemm with B small,
// src/adapters/tools/qwen35_engine.cpp:47-85, fused with dequant_lattice,
// src/block_codec.cpp:173-182).
//
// Block layout (little endian, LSB-first): 16-bit FP16 scale, then one 4-bit
// level index per non-slot weight; weights 63,127,191,255 are slots (decode to
// zero, own no bits).  In nibble units: nibbles 0..3 hold the scale, nibble
// p >= 4 holds weight i(p) = (p-4) + (p-4)/63.
//
// Mapping.  Work is cut into "slabs" of SB consecutive blocks of a row.  A
// wavefront owns one slab position and walks down rows: 8 lanes cover one
// 128-byte block with one 16-byte load each (32 nibbles per lane), so a wave
// load covers RW = 8/SB rows x SB blocks.  Because a lane sees the same 32
// nibble positions in every row, its 32 activations live in registers for the
// whole kernel, pre-permuted into nibble order (scale nibbles and out-of-range
// blocks get activation 0).  Per packed byte the two level values come from one
// LDS read of a 256-entry pair table (address built with a single v_perm_b32),
// followed by two FP32 FMAs.  The per-block FP16 scale is applied once per
// block after an 8-lane DPP reduction; slab partials meet in LDS.
#include <hip/hip_fp16.h>

#include <cstdlib>

#include "common.h"

namespace oilhip {
namespace {

constexpr int kTabBytes = 256 * 64 * 4;   // [byte value][low|high nibble][32 lane copies] floats
constexpr int kMaxLds = 160 * 1024;

__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
}
__device__ __forceinline__ float dpp_half_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
}
__device__ __forceinline__ float dpp_row_ror8(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));  // row_ror:8
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const float lds_cfloat;

constexpr uint32_t kOobOffset = 0xFFFFFF00u;   // beyond any buffer range: the load returns zeros, no fetch

// The two level values of one packed byte: (low nibble, high nibble).
struct LevelPair { float lo, hi; };

template <int J>
__device__ __forceinline__ LevelPair lookup(uint32_t word, uint32_t lanebase) {
    // byte J of the dword -> address bits 8..15, this lane's table copy -> bits 0..7
    const uint32_t addr = __builtin_amdgcn_perm(word, lanebase, 0x0C0C0000u | ((4u + J) << 8));
    lds_cfloat* tp = (lds_cfloat*)(uintptr_t)addr;
    return LevelPair{tp[0], tp[32]};
}

__device__ __forceinline__ void lookup_row(const u32x4& w, uint32_t lanebase, LevelPair (&t)[16]) {
    const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        t[d * 4 + 0] = lookup<0>(wd[d], lanebase);
        t[d * 4 + 1] = lookup<1>(wd[d], lanebase);
        t[d * 4 + 2] = lookup<2>(wd[d], lanebase);
        t[d * 4 + 3] = lookup<3>(wd[d], lanebase);
    }
}

// SB: blocks per slab (8, 4, 2 or 1); RPW: wave-loads per chunk (all in flight
// at once); MB: activation rows handled together; MAXT: workgroup size bound.
template <int SB, int RPW, int MB, int MAXT>
__global__ void __launch_bounds__(MAXT)
gemv_oil4_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* __restrict__ y,
                 uint32_t rows, uint32_t cols, uint32_t S, uint32_t G, uint32_t nchunks, int m0, int M) {
    constexpr int LS = 8 * SB;        // lanes across one slab row
    constexpr int RW = 64 / LS;       // rows per wave-load
    constexpr int CH = RPW * RW;      // rows per chunk and row group
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                        // LDS byte offset 0
    float* xs = reinterpret_cast<float*>(lds + kTabBytes);             // [MB][S*SB*256] nibble-ordered
    const uint32_t kpad = S * SB * 256;
    float* red = xs + (size_t)MB * kpad;                               // [G][CH][MB][S]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t slab = wave % S, grp = wave / S;
    const uint32_t bpr = cols >> 8;
    const uint32_t sub = lane / LS, l = lane % LS, lp = l & 7u;
    const uint32_t kb = slab * SB + (l >> 3);
    const bool col_ok = kb < bpr;

    const uint32_t J = gridDim.x * G, jg = blockIdx.x * G + grp;
    const uint32_t r0 = (uint32_t)(((uint64_t)rows * jg) / J);
    const uint32_t r1 = (uint32_t)(((uint64_t)rows * (jg + 1)) / J);
    const uint32_t row_bytes = bpr * 128u;
    // buffer resource over this workgroup's rows (offsets stay below 2^31)
    const uint32_t wg_r0 = (uint32_t)(((uint64_t)rows * (blockIdx.x * G)) / J);
    const uint64_t remain = (uint64_t)(rows - wg_r0) * row_bytes;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)wg_r0 * row_bytes), 0, (int)(remain < 0x80000000ull ? remain : 0x80000000ull), 0x00020000);
    const uint32_t lane_off = kb * 128u + lp * 16u;

    // ---- activations first (they are needed soonest), then the first chunk of weights ----
    // xs[m][b*256 + c*32 + q8*4 + e] = x'(p = 32*q8 + 4c + e): nibble order, 0 under the scale
    // nibbles and beyond the last block.  XPT elements per thread are fetched up front so the
    // table build and these loads overlap the weight loads that follow them in the queue.
    constexpr int XPT = 8;
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(x + (size_t)m0 * cols), 0, (int)((uint64_t)(M - m0 < MB ? M - m0 : MB) * cols * 4u), 0x00020000);
    auto x_offset = [&](uint32_t d) -> uint32_t {          // byte offset of x' element d, or out of range
        const uint32_t b = d >> 8, rem = d & 255u;
        const uint32_t c = rem >> 5, q8 = (rem >> 2) & 7u, e = rem & 3u;
        const uint32_t p = 32 * q8 + 4 * c + e;
        const uint32_t q = p - 4;
        const uint32_t i = q + (q >= 63) + (q >= 126) + (q >= 189);
        return (p >= 4 && b < bpr && d < kpad) ? (b * 256u + i) * 4u : kOobOffset;
    };
    float xpre[MB][XPT];
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t off = x_offset(tid + u * blockDim.x);
#pragma unroll
        for (int m = 0; m < MB; ++m)
            xpre[m][u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
                xrsrc, off == kOobOffset ? off : off + m * cols * 4u, 0, 0));
    }
    u32x4 wv[RPW];
#pragma unroll
    for (int it = 0; it < RPW; ++it) {
        const uint32_t r = r0 + it * RW + sub;
        const uint32_t off = (col_ok && r < r1) ? (r - wg_r0) * row_bytes + lane_off : kOobOffset;
        wv[it] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
    }

    // ---- pair table: tab[v*64 + h*32 + c] = level[h ? v>>4 : v&15] ----------------
    for (uint32_t e = tid; e < 256 * 64 / 4; e += blockDim.x) {
        const uint32_t rowi = e >> 3;                 // (v, h) pair: 8 float4 hold its 32 copies
        const uint32_t v = rowi >> 1, h = rowi & 1u;
        const float lv = kLv4[h ? (v >> 4) : (v & 15u)];
        reinterpret_cast<float4*>(tab)[e] = make_float4(lv, lv, lv, lv);
    }
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t d = tid + u * blockDim.x;
        if (d < kpad) {
#pragma unroll
            for (int m = 0; m < MB; ++m) xs[(size_t)m * kpad + d] = xpre[m][u];
        }
    }
    for (uint32_t d = tid + XPT * blockDim.x; d < kpad; d += blockDim.x) {     // rows wider than XPT * workgroup
        const uint32_t off = x_offset(d);
#pragma unroll
        for (int m = 0; m < MB; ++m)
            xs[(size_t)m * kpad + d] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
                xrsrc, off == kOobOffset ? off : off + m * cols * 4u, 0, 0));
    }
    __syncthreads();

    float xr[MB][32];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float4 t = *reinterpret_cast<const float4*>(xs + (size_t)m * kpad + (size_t)(slab * SB + (l >> 3)) * 256 + c * 32 + lp * 4);
            xr[m][4 * c + 0] = t.x; xr[m][4 * c + 1] = t.y; xr[m][4 * c + 2] = t.z; xr[m][4 * c + 3] = t.w;
        }

    const uint32_t lanebase = (lane & 31u) * 4u;      // byte offset of this lane's table copy

    for (uint32_t ch = 0; ch < nchunks; ++ch) {
        const uint32_t cbase = r0 + ch * CH;
        if (ch > 0) {
#pragma unroll
            for (int it = 0; it < RPW; ++it) {
                const uint32_t r = cbase + it * RW + sub;
                const uint32_t off = (col_ok && r < r1) ? (r - wg_r0) * row_bytes + lane_off : kOobOffset;
                wv[it] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
            }
        }
        LevelPair cur[16];
        lookup_row(wv[0], lanebase, cur);
#pragma unroll
        for (int it = 0; it < RPW; ++it) {
            LevelPair nxt[16];
            if (it + 1 < RPW) lookup_row(wv[it + 1], lanebase, nxt);      // next row's table reads fly during this row's FMAs
            float acc[MB][4];
#pragma unroll
            for (int m = 0; m < MB; ++m) acc[m][0] = acc[m][1] = acc[m][2] = acc[m][3] = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; ++k)
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    acc[m][k & 3] = __fmaf_rn(cur[k].lo, xr[m][2 * k], acc[m][k & 3]);
                    acc[m][k & 3] = __fmaf_rn(cur[k].hi, xr[m][2 * k + 1], acc[m][k & 3]);
                }
            const float scale = __half2float(__ushort_as_half((unsigned short)(wv[it].x & 0xFFFFu)));
            float tot[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                float s = (acc[m][0] + acc[m][1]) + (acc[m][2] + acc[m][3]);
                s += dpp_quad_xor1(s);
                s += dpp_quad_xor2(s);
                s += dpp_half_mirror(s);                       // all 8 lanes of the block: block sum
                float v = (lp == 0) ? s * scale : 0.0f;        // one scaled value per block
                if (SB >= 2) v += dpp_row_ror8(v);             // lanes 0 and 8 of each row of 16
                if (SB == 8) tot[m] = (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
                else if (SB == 4) tot[m] = sub == 0 ? lane_value(v, 0) + lane_value(v, 16) : lane_value(v, 32) + lane_value(v, 48);
                else tot[m] = v;                               // SB <= 2: lane l == 0 of each slab row holds it
            }
            if (l == 0) {
#pragma unroll
                for (int m = 0; m < MB; ++m)
                    red[(((size_t)grp * CH + it * RW + sub) * MB + m) * S + slab] = tot[m];
            }
            if (it + 1 < RPW) {
#pragma unroll
                for (int k = 0; k < 16; ++k) cur[k] = nxt[k];
            }
        }
        __syncthreads();
        // ---- slab partials -> y -------------------------------------------------
        for (uint32_t o = tid; o < G * CH * MB; o += blockDim.x) {
            const uint32_t g2 = o / (CH * MB), rem = o % (CH * MB), slot = rem / MB, m = rem % MB;
            const uint32_t jg2 = blockIdx.x * G + g2;
            const uint32_t q0 = (uint32_t)(((uint64_t)rows * jg2) / J);
            const uint32_t q1 = (uint32_t)(((uint64_t)rows * (jg2 + 1)) / J);
            const uint32_t r = q0 + ch * CH + slot;
            if (r < q1 && m0 + (int)m < M) {
                const float* pr = red + (size_t)o * S;
                float s = 0.0f;
                for (uint32_t k = 0; k < S; ++k) s += pr[k];
                y[(size_t)(m0 + m) * rows + r] = s;
            }
        }
        __syncthreads();
    }
}

// One launch configuration of the kernel above.
struct Oil4Plan {
    int sb, rpw, maxt;     // template choice
    uint32_t S, G, grid, nchunks;
    size_t lds_bytes;
};

template <int SB, int RPW, int MB, int MAXT>
int launch(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s, const Oil4Plan& p) {
    static bool attr_done = false;
    auto kern = gemv_oil4_kernel<SB, RPW, MB, MAXT>;
    if (!attr_done) {
        OILHIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
        attr_done = true;
    }
    for (int m0 = 0; m0 < M; m0 += MB) {
        hipLaunchKernelGGL(kern, dim3(p.grid), dim3(p.S * p.G * 64), p.lds_bytes, s, w.d_payload, d_x, d_y,
                           (uint32_t)w.rows, (uint32_t)w.cols, p.S, p.G, p.nchunks, m0, M);
        OILHIP_HIP(hipGetLastError());
    }
    return OILHIP_OK;
}

// Chooses slab width, waves per workgroup and chunking for a shape.
// waves_target: 8 (two waves per SIMD, deep per-wave pipelining) or 16.
bool make_plan(uint32_t rows, uint32_t cols, int MB, int waves_target, Oil4Plan* p) {
    const uint32_t bpr = cols >> 8;
    int sb = 1;
    for (int cand : {8, 4, 2}) {       // widest slab that wastes <= ~3 % of lanes on the ragged last slab
        const uint32_t slabs = (bpr + cand - 1) / cand;
        if ((double)(slabs * cand - bpr) / (double)(slabs * cand) <= 0.03) { sb = cand; break; }
    }
    uint32_t S = (bpr + sb - 1) / sb;
    while (S > 16 && sb < 8) { sb *= 2; S = (bpr + sb - 1) / sb; }
    if (S > 16) return false;
    uint32_t G = (uint32_t)waves_target / S;
    if (G == 0) G = 1;
    const int RW = 64 / (8 * sb);
    uint32_t grid = (uint32_t)device_cu_count();
    const uint32_t max_groups = (rows + RW - 1) / RW;
    if (grid * G > max_groups) grid = (max_groups + G - 1) / G;
    if (grid == 0) grid = 1;
    const uint32_t Jn = grid * G;
    const uint32_t max_rows = (rows + Jn - 1) / Jn;                 // rows of the largest row group
    const uint32_t loads = (max_rows + RW - 1) / RW;                // wave-loads it needs
    const int rpw = loads <= 4 ? 4 : (loads <= 6 ? 6 : (loads <= 8 ? 8 : 12));
    const uint32_t CH = (uint32_t)rpw * RW;
    p->sb = sb; p->rpw = rpw; p->maxt = (S * G > 12) ? 1024 : ((S * G > 8) ? 768 : 512);
    p->S = S; p->G = G; p->grid = grid;
    p->nchunks = (max_rows + CH - 1) / CH;
    if (p->nchunks == 0) p->nchunks = 1;
    p->lds_bytes = (size_t)kTabBytes + 4ull * MB * S * sb * 256 + 4ull * G * CH * MB * S;
    return p->lds_bytes <= (size_t)kMaxLds;
}

template <int MB>
int dispatch(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s, const Oil4Plan& p) {
#define OIL4_CASE(SB_, RPW_, MAXT_) \
    if (p.sb == SB_ && p.rpw == RPW_ && p.maxt == MAXT_) return launch<SB_, RPW_, MB, MAXT_>(w, d_x, d_y, M, s, p);
    OIL4_CASE(8, 4, 512) OIL4_CASE(8, 6, 512) OIL4_CASE(8, 8, 512) OIL4_CASE(8, 12, 512)
    OIL4_CASE(4, 4, 512) OIL4_CASE(4, 6, 512) OIL4_CASE(4, 8, 512) OIL4_CASE(4, 12, 512)
    OIL4_CASE(2, 4, 512) OIL4_CASE(2, 6, 512) OIL4_CASE(2, 8, 512) OIL4_CASE(2, 12, 512)
    OIL4_CASE(1, 4, 512) OIL4_CASE(1, 6, 512) OIL4_CASE(1, 8, 512) OIL4_CASE(1, 12, 512)
    OIL4_CASE(8, 4, 768) OIL4_CASE(8, 8, 768) OIL4_CASE(4, 4, 768) OIL4_CASE(4, 8, 768)
    OIL4_CASE(2, 4, 768) OIL4_CASE(2, 8, 768) OIL4_CASE(1, 4, 768) OIL4_CASE(1, 8, 768)
    if constexpr (MB == 1) {
        OIL4_CASE(8, 4, 1024) OIL4_CASE(4, 4, 1024) OIL4_CASE(2, 4, 1024) OIL4_CASE(1, 4, 1024)
    }
#undef OIL4_CASE
    return 1;
}

}  // namespace

// OILHIP_OIL4_WAVES=8|16 overrides the waves-per-workgroup target (tuning aid).
static int waves_target_default() {
    static int v = [] {
        const char* e = getenv("OILHIP_OIL4_WAVES");
        const int n = e ? atoi(e) : 0;
        return (n == 8 || n == 16) ? n : 8;
    }();
    return v;
}

int launch_gemv_oil4(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull || M > 16) return 1;
    Oil4Plan p;
    const int MB = M == 1 ? 1 : 2;
    int wt = waves_target_default();
    if (!make_plan((uint32_t)w.rows, (uint32_t)w.cols, MB, wt, &p)) return 1;
    // register budget: 12 waves leave 170 VGPRs (chunks of <= 8 loads), 16 waves 128 (chunks of 4, M = 1 only)
    const int cap = p.maxt == 1024 ? 4 : (p.maxt == 768 ? (MB == 1 ? 8 : 4) : 12);
    if (p.maxt == 1024 && MB != 1) return 1;
    if (p.maxt == 768 && p.rpw == 6) p.rpw = 8;
    if (p.rpw > cap) p.rpw = cap;
    {
        const uint32_t RW = 64u / (8u * p.sb), Jn = p.grid * p.G;
        const uint32_t max_rows = ((uint32_t)w.rows + Jn - 1) / Jn, CH = (uint32_t)p.rpw * RW;
        p.nchunks = (max_rows + CH - 1) / CH;
        if (p.nchunks == 0) p.nchunks = 1;
        p.lds_bytes = (size_t)kTabBytes + 4ull * MB * p.S * p.sb * 256 + 4ull * p.G * CH * MB * p.S;
        if (p.lds_bytes > (size_t)kMaxLds) return 1;
    }
    return MB == 1 ? dispatch<1>(w, d_x, d_y, M, s, p) : dispatch<2>(w, d_x, d_y, M, s, p);
}

}  // namespace oilhip
