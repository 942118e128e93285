// gemv_oil8.hip -- decode GEMV for tensors whose blocks are all full OIL8 blocks: Qwen35Engine::gemm
// (src/adapters/tools/qwen35_engine.cpp:47-85) fused with the OIL8 branch of dequantize_block_all
// (src/block_codec.cpp:173-182, level table :131).
//
// A full OIL8 block is 256 bytes: the FP16 scale, then one byte per weight; weights 127 and 255 are
// slots and own no byte, so weight i sits at byte p = i + 2 - (i >= 128).  The 256 levels are the
// affine ramp -8 + 16 q / 255 = (16/255) (q - 127.5), so no table is needed:
//     y = (16/255) * sum over blocks of scale * (sum_p q_p x_p  -  127.5 * sum_p x_p)
// with x_p the activation that belongs to byte p (0 for the two scale bytes).  Per byte that is one
// v_cvt_f32_ubyte and one v_fma_f32; the second sum is formed once per lane when x is staged.
//
// 16 lanes x one 16-byte load cover a block, a wave-load (1 KB) covers 4 blocks (a "column set"); a
// wavefront owns CS column sets and walks down RPW rows per chunk with all loads of the chunk in
// flight, exactly like the OIL4 kernel.  The lane's 16*CS activations stay in registers in byte order.
//
// FLAT = true is the same frame for kernel::oil8_gemm (include/oil/kernel.h, src/kernel_oil8.cpp): rows of K index
// bytes without block structure and an arbitrary 256-entry FP32 codebook.  x stays in natural order, and each byte
// is looked up in a copy of the codebook that the lane owns (64 KB of LDS: entry v of lane l at byte v*256 + l*4,
// every lane on its own bank).
#include <hip/hip_fp16.h>

#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using namespace oil4;      // DPP helpers, u32x4

constexpr int kXs8Block = 288;       // floats per block in the LDS copy of x: 256 + 32 so that neighbouring blocks start 32 banks apart
constexpr int kPFA = 3, kPFB = 6;    // wave-loads queued before / by the end of the prologue
constexpr int kFlatTabBytes = 256 * 64 * 4;

// value of the first lane of each group of 16 lanes (a DPP row), in all 16 lanes
__device__ __forceinline__ uint32_t dpp_bcast16(uint32_t v) {
    const int q = __builtin_amdgcn_update_dpp(0, (int)v, 0x00, 0xF, 0xF, true);       // quad_perm [0,0,0,0]
    const int h = __builtin_amdgcn_update_dpp(q, q, 0x114, 0xF, 0xA, false);          // row_shr:4 into quads 1 and 3
    return (uint32_t)__builtin_amdgcn_update_dpp(h, h, 0x118, 0xF, 0xC, false);       // row_shr:8 into quads 2 and 3
}

// CS: column sets (wave-loads) per row and wave; RPW: rows per chunk; MB: activation rows handled together;
// ROLL: several chunks per wavefront, loads rolling from one chunk into the next.
template <int CS, int RPW, int MB, bool ROLL, bool FLAT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_oil8_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* __restrict__ y,
                 uint32_t rows, uint32_t cols, uint32_t S, uint32_t G, uint32_t nchunks, int m0, int M,
                 uint32_t rg_base, uint32_t rg_rem, uint32_t wave_groups, const float* __restrict__ cb, float out_scale) {
    constexpr int NL = CS * RPW;      // wave-loads per chunk
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t nblk = S * CS * 4;                                         // blocks covered by all slabs (>= cols/256)
    const uint32_t xstride = nblk * kXs8Block;                                // floats per activation row in LDS
    float* tab = reinterpret_cast<float*>(lds);                               // FLAT: [256 v][64 lanes], LDS byte offset 0
    float* xs = reinterpret_cast<float*>(lds + (FLAT ? kFlatTabBytes : 0));   // [MB][nblk][4 c][16 lp][4 e] (+32 pad), byte order
    float* red = xs + (size_t)MB * xstride;                                   // [G][RPW][MB][S]

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t grp = (wave_groups >> (4u * wave)) & 15u, slab = wave - grp * S;         // wave / S, wave % S
    const uint32_t bpr = cols >> 8;
    const uint32_t lp = lane & 15u;

    auto group_begin = [&](uint32_t j) { return j * rg_base + (j < rg_rem ? j : rg_rem); };
    const uint32_t jg = blockIdx.x * G + grp;
    const bool working = wave < S * G;
    const uint32_t r0 = working ? group_begin(jg) : 0u, r1 = working ? group_begin(jg + 1) : 0u;
    const uint32_t row_bytes = FLAT ? cols : bpr * 256u;
    // buffer resource over this wavefront's rows only: a load of a row past r1 is out of range (zeros, no fetch)
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)r0 * row_bytes), 0, (int)((r1 - r0) * row_bytes), 0x00020000);

    // ---- x first, then the first weight loads -------------------------------------------------------
    constexpr int XPT = 4;            // float4 pieces of x fetched up front per thread
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(x + (size_t)m0 * cols), 0, (int)((uint32_t)(M - m0 < MB ? M - m0 : MB) * cols * 4u), 0x00020000);
    u32x4 xpre[MB][XPT];
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t d4 = tid + u * 512u;
#pragma unroll
        for (int m = 0; m < MB; ++m)
            xpre[m][u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (d4 * 4u < cols && m0 + m < M) ? d4 * 16u + m * cols * 4u : kOobOffset, 0, 0);
    }
    uint32_t vcol[CS];
#pragma unroll
    for (int cs = 0; cs < CS; ++cs) {
        if (FLAT) {
            const uint32_t off = ((slab * CS + cs) * 64u + lane) * 16u;       // rows are a whole number of 16-byte pieces
            vcol[cs] = off < cols ? off : 0x80000000u;
        } else {
            const uint32_t blk = (slab * CS + cs) * 4u + (lane >> 4);
            vcol[cs] = blk < bpr ? blk * 256u + lp * 16u : 0x80000000u;
        }
    }
    constexpr int PFA = NL < kPFA ? NL : kPFA, PFB = NL < kPFB ? NL : kPFB;
    u32x4 wv[NL];
    auto issue_load = [&](int n, uint32_t rel) {           // rel: first row of the chunk, counted from r0
        const int it = n / CS, cs = n % CS;
        wv[n] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, vcol[cs] + (rel + it) * row_bytes, 0, 2);
    };
#pragma unroll
    for (int n = 0; n < PFA; ++n) issue_load(n, 0u);
    __builtin_amdgcn_sched_barrier(0);
    if (FLAT) {       // float4 number e of the table holds entry v = e >> 4 for four lanes; thread tid writes e = tid + 512*k
        float cv[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) cv[k] = cb[(tid >> 4) + 32u * k];
#pragma unroll
        for (int k = 0; k < 8; ++k) reinterpret_cast<float4*>(tab)[tid + 512u * k] = make_float4(cv[k], cv[k], cv[k], cv[k]);
    }

    // ---- x into LDS in byte order ----------------------------------------------------------------------
    // x[i] of a block belongs to byte p = i + 2 - (i >= 128); lane lp of the block holds bytes 16*lp .. 16*lp+15
    // and reads them as 4 float4 (c = 0..3), so x[i] goes to xs[blk*288 + c*64 + lp*4 + e] with p = 16*lp + 4*c + e.
    // FLAT: natural order; float4 number d4 (columns 4*d4 ..) of a 1024-column set belongs to lane (d4 >> 2) & 63 as
    // its float4 number c = d4 & 3 and goes to xs[set*1152 + c*256 + lane*4].
    uint32_t xoff[4];
    bool xlast_ok;
    {
        const uint32_t w = (tid * 4u) & 255u;
        xlast_ok = (w & 127u) != 124u;                                        // i % 128 == 127 is a slot
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t p = w + k + 2u - (w >> 7);
            xoff[k] = ((p >> 2) & 3u) * 64u + (p >> 4) * 4u + (p & 3u);
        }
    }
    auto scatter4 = [&](uint32_t d4, const u32x4& v, int m) {
        if (FLAT) {
            float* dst = xs + (size_t)m * xstride + (d4 >> 8) * (4u * kXs8Block) + (d4 & 3u) * 256u + ((d4 >> 2) & 63u) * 4u;
            *reinterpret_cast<u32x4*>(dst) = v;
            return;
        }
        float* dst = xs + (size_t)m * xstride + (d4 >> 6) * kXs8Block;
        dst[xoff[0]] = __uint_as_float(v.x);
        dst[xoff[1]] = __uint_as_float(v.y);
        dst[xoff[2]] = __uint_as_float(v.z);
        if (xlast_ok) dst[xoff[3]] = __uint_as_float(v.w);
    };
    if (FLAT) {
        for (uint32_t d4 = (cols >> 2) + tid; d4 < nblk * 64u; d4 += 512u) {  // columns past the end of the row
#pragma unroll
            for (int m = 0; m < MB; ++m) scatter4(d4, u32x4{0u, 0u, 0u, 0u}, m);
        }
    } else {
        for (uint32_t bz = tid; bz < nblk * MB; bz += 512u) {                 // the two scale bytes of every block
            const uint32_t m = bz / nblk, b = bz % nblk;
            *reinterpret_cast<float2*>(xs + (size_t)m * xstride + b * kXs8Block) = make_float2(0.f, 0.f);
        }
        for (uint32_t z = bpr * 64u + tid; z < nblk * 64u; z += 512u) {       // blocks past the end of the row
#pragma unroll
            for (int m = 0; m < MB; ++m)
                reinterpret_cast<float4*>(xs + (size_t)m * xstride + (z >> 6) * kXs8Block)[z & 63u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t d4 = tid + u * 512u;
        if (d4 * 4u < cols) {
#pragma unroll
            for (int m = 0; m < MB; ++m) scatter4(d4, xpre[m][u], m);
        }
    }
    for (uint32_t d4 = tid + XPT * 512u; d4 * 4u < cols; d4 += 512u) {        // rows wider than 8192 columns
#pragma unroll
        for (int m = 0; m < MB; ++m)
            scatter4(d4, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (m0 + m < M) ? d4 * 16u + m * cols * 4u : kOobOffset, 0, 0), m);
    }
#pragma unroll
    for (int n = PFA; n < PFB; ++n) issue_load(n, 0u);
    __syncthreads();

    // ---- this lane's activations: 4 float4 per column set, and their sum ------------------------
    float xr[MB][CS][16], xsum[MB][CS];
#pragma unroll
    for (int cs = 0; cs < CS; ++cs) {
        const uint32_t blk = (slab * CS + cs) * 4u + (lane >> 4);
        const uint32_t base = FLAT ? (slab * CS + cs) * (4u * kXs8Block) + lane * 4u : blk * kXs8Block + lp * 4u;
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float4 t = *reinterpret_cast<const float4*>(xs + (size_t)m * xstride + base + c * (FLAT ? 256 : 64));
                xr[m][cs][4 * c + 0] = t.x; xr[m][cs][4 * c + 1] = t.y; xr[m][cs][4 * c + 2] = t.z; xr[m][cs][4 * c + 3] = t.w;
                s += (t.x + t.y) + (t.z + t.w);
            }
            xsum[m][cs] = FLAT ? 0.0f : s * -127.5f;
        }
    }

#pragma unroll
    for (int n = PFB; n < NL; ++n) issue_load(n, 0u);     // rest of the first chunk
    for (uint32_t ch = 0; ch < nchunks; ++ch) {
        const uint32_t cbase = r0 + ch * RPW;
        if (!ROLL && ch > 0) {
#pragma unroll
            for (int n = 0; n < NL; ++n) issue_load(n, ch * RPW);
        }
        float part[MB][RPW];                              // per-lane partial of each row, block scales applied
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int it = n / CS, cs = n % CS;
            const uint32_t wd[4] = {wv[n].x, wv[n].y, wv[n].z, wv[n].w};
            float q[16];                                  // the 16 weights of this lane, still without the block scale
            float scale = 1.0f;
            if (FLAT) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    q[4 * d + 0] = *(lds_cfloat*)(uintptr_t)__builtin_amdgcn_perm(wd[d], lane * 4u, 0x0C0C0400u);
                    q[4 * d + 1] = *(lds_cfloat*)(uintptr_t)__builtin_amdgcn_perm(wd[d], lane * 4u, 0x0C0C0500u);
                    q[4 * d + 2] = *(lds_cfloat*)(uintptr_t)__builtin_amdgcn_perm(wd[d], lane * 4u, 0x0C0C0600u);
                    q[4 * d + 3] = *(lds_cfloat*)(uintptr_t)__builtin_amdgcn_perm(wd[d], lane * 4u, 0x0C0C0700u);
                }
            } else {
                // the block's FP16 scale sits in the low half of its first lane's first dword
                scale = __half2float(__ushort_as_half((unsigned short)(dpp_bcast16(wv[n].x) & 0xFFFFu)));
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    q[4 * d + 0] = (float)(wd[d] & 0xFFu);
                    q[4 * d + 1] = (float)((wd[d] >> 8) & 0xFFu);
                    q[4 * d + 2] = (float)((wd[d] >> 16) & 0xFFu);
                    q[4 * d + 3] = (float)(wd[d] >> 24);
                }
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                float a0 = xsum[m][cs], a1 = 0.0f;
#pragma unroll
                for (int k = 0; k < 16; k += 2) {
                    a0 = __fmaf_rn(q[k], xr[m][cs][k], a0);
                    a1 = __fmaf_rn(q[k + 1], xr[m][cs][k + 1], a1);
                }
                if (FLAT) part[m][it] = cs == 0 ? a0 + a1 : part[m][it] + (a0 + a1);
                else part[m][it] = cs == 0 ? (a0 + a1) * scale : __fmaf_rn(a0 + a1, scale, part[m][it]);
            }
            if (ROLL) issue_load(n, (ch + 1u) * RPW);     // unconditional: past the last row the offset is out of range
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- all rows of the chunk reduced over the 64 lanes together ----
#pragma unroll
        for (int it = 0; it < RPW; ++it)
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                float v = part[m][it];
                v += dpp_quad_xor1(v);
                v += dpp_quad_xor2(v);
                v += dpp_half_mirror(v);
                v += dpp_row_mirror(v);
                v += dpp_row_bcast15(v);
                v += dpp_row_bcast31(v);
                part[m][it] = v * out_scale;              // lane 63 holds the slab's dot product
            }
        if (S == 1) {                                     // a wave covers whole rows: lane 63 stores y
            if (lane == 63) {
#pragma unroll
                for (int it = 0; it < RPW; ++it)
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        if (cbase + it < r1 && m0 + m < M) y[(size_t)(m0 + m) * rows + cbase + it] = part[m][it];
            }
            continue;
        }
        if (lane == 63 && working) {
#pragma unroll
            for (int it = 0; it < RPW; ++it)
#pragma unroll
                for (int m = 0; m < MB; ++m)
                    red[(((size_t)grp * RPW + it) * MB + m) * S + slab] = part[m][it];
        }
        __syncthreads();
        for (uint32_t o = tid; o < G * RPW * MB; o += 512u) {
            const uint32_t g2 = o / (RPW * MB), rem = o % (RPW * MB), slot = rem / MB, m = rem % MB;
            const uint32_t jg2 = blockIdx.x * G + g2;
            const uint32_t q0 = group_begin(jg2), q1 = group_begin(jg2 + 1);
            const uint32_t r = q0 + ch * RPW + slot;
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

struct Oil8Plan {
    int cs, rpw;
    uint32_t S, G, grid, nchunks;
    size_t lds_bytes;
};

template <int CS, int RPW, int MB, bool ROLL, bool FLAT>
int launch(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s, const Oil8Plan& p, const float* d_cb, float out_scale) {
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemv_oil8_kernel<CS, RPW, MB, ROLL, FLAT>;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), kMaxLds)) return rc;
    const uint32_t J = p.grid * p.G;
    uint32_t wave_groups = 0;                                   // wave / S for each of the 8 wavefronts, 4 bits each
    for (uint32_t wv = 0; wv < 8; ++wv) wave_groups |= (wv / p.S) << (4u * wv);
    for (int m0 = 0; m0 < M; m0 += MB) {
        hipLaunchKernelGGL(kern, dim3(p.grid), dim3(512), p.lds_bytes, s, w.d_payload + w.uniform_base, d_x, d_y,
                           (uint32_t)w.rows, (uint32_t)w.cols, p.S, p.G, p.nchunks, m0, M,
                           (uint32_t)w.rows / J, (uint32_t)w.rows % J, wave_groups, d_cb, out_scale);
        OILHIP_HIP(hipGetLastError());
    }
    return OILHIP_OK;
}

bool make_plan(uint32_t rows, uint32_t cols, int MB, bool flat, Oil8Plan* p) {
    const uint32_t sets = (cols + 1023u) / 1024u;                 // column sets (1 KB wave-loads) per row
    const int cs_max = MB == 1 ? 4 : (MB == 2 ? 2 : 1);           // register budget: 16*CS*MB activations per lane
    int best_cs = 1; uint32_t best_S = sets; double best_cost = 1e30;
    for (int cs = 1; cs <= cs_max; ++cs) {
        const uint32_t S = (sets + cs - 1) / cs;
        if (S > 8u) continue;
        const double waste = (double)(S * cs) / (double)sets;
        const double cost = waste + 0.04 * (S > 1 ? S : 0);
        if (cost < best_cost) { best_cost = cost; best_cs = cs; best_S = S; }
    }
    if (best_cost > 1e29) return false;
    const uint32_t S = best_S;
    uint32_t G = 8u / S;
    if (G == 0) G = 1;
    uint32_t grid = (uint32_t)device_cu_count();
    if (grid * G > rows) grid = (rows + G - 1) / G;
    if (grid == 0) grid = 1;
    const uint32_t Jn = grid * G;
    const uint32_t max_rows = (rows + Jn - 1) / Jn;
    const int budget = 12 / best_cs;                               // wave-loads in flight per wave (register budget)
    int rpw = 1;
    if (max_rows <= (uint32_t)budget) {
        for (int cand : {1, 2, 3, 4, 6, 12}) if ((uint32_t)cand >= max_rows) { rpw = cand; break; }
    } else {
        int lo = (6 + best_cs - 1) / best_cs;
        if (lo > budget) lo = budget;
        uint32_t best_slots = ~0u;
        for (int cand : {1, 2, 3, 4, 6, 12}) {
            if (cand < lo || cand > budget) continue;
            const uint32_t slots = (max_rows + cand - 1) / cand * cand;
            if (slots < best_slots) { best_slots = slots; rpw = cand; }
        }
    }
    p->cs = best_cs; p->rpw = rpw;
    p->S = S; p->G = G; p->grid = grid;
    p->nchunks = (max_rows + rpw - 1) / rpw;
    if (p->nchunks == 0) p->nchunks = 1;
    p->lds_bytes = (flat ? (size_t)kFlatTabBytes : 0) + 4ull * MB * (S * best_cs * 4 * kXs8Block) + 4ull * G * rpw * MB * S + 64;
    if ((uint64_t)(max_rows + 2u * (uint32_t)rpw) * (uint64_t)cols >= 0x80000000ull) return false;   // per-wave buffer range
    return p->lds_bytes <= (size_t)kMaxLds && S * G <= 8;
}

template <int MB, bool FLAT>
int dispatch(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s, const Oil8Plan& p, const float* d_cb, float out_scale) {
#define OIL8_CASE(CS_, RPW_) \
    if (p.cs == CS_ && p.rpw == RPW_) \
        return p.nchunks > 1 ? launch<CS_, RPW_, MB, true, FLAT>(w, d_x, d_y, M, s, p, d_cb, out_scale) \
                             : launch<CS_, RPW_, MB, false, FLAT>(w, d_x, d_y, M, s, p, d_cb, out_scale);
    OIL8_CASE(1, 1) OIL8_CASE(1, 2) OIL8_CASE(1, 3) OIL8_CASE(1, 4) OIL8_CASE(1, 6) OIL8_CASE(1, 12)
    if constexpr (MB <= 2) { OIL8_CASE(2, 1) OIL8_CASE(2, 2) OIL8_CASE(2, 3) OIL8_CASE(2, 4) OIL8_CASE(2, 6) }
    if constexpr (MB == 1) {
        OIL8_CASE(3, 1) OIL8_CASE(3, 2) OIL8_CASE(3, 3) OIL8_CASE(3, 4)
        OIL8_CASE(4, 1) OIL8_CASE(4, 2) OIL8_CASE(4, 3)
    }
#undef OIL8_CASE
    return 1;
}

}  // namespace

// y = W x for a tensor of full OIL8 blocks laid out back to back.  Returns 1 when the shape is not covered.
int launch_gemv_oil8(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull || M > 16 || (w.uniform_base & 15u)) return 1;
    Oil8Plan p;
    const int MB = M == 1 ? 1 : (M == 2 ? 2 : 4);
    if (!make_plan((uint32_t)w.rows, (uint32_t)w.cols, MB, false, &p)) return 1;
    const float k = 16.0f / 255.0f;
    return MB == 1 ? dispatch<1, false>(w, d_x, d_y, M, s, p, nullptr, k)
         : MB == 2 ? dispatch<2, false>(w, d_x, d_y, M, s, p, nullptr, k) : dispatch<4, false>(w, d_x, d_y, M, s, p, nullptr, k);
}

// kernel::oil8_gemm: out[m*N + n] = scale * sum_k cb[idx[n*K + k]] * act[m*K + k].  Returns 1 when the shape is not covered.
int launch_gemv_flat8(const uint8_t* d_idx, const float* d_cb, const float* d_act, float* d_out, int M, int N, int K, float scale,
                      hipStream_t s) {
    if (M < 1 || M > 16 || N < 1 || K < 16 || (K & 15) || (reinterpret_cast<uintptr_t>(d_idx) & 15u)) return 1;
    oilhip_weights w;                                             // a view: rows of K bytes
    w.d_payload = const_cast<uint8_t*>(d_idx);
    w.rows = (uint64_t)N; w.cols = (uint64_t)K;
    Oil8Plan p;
    const int MB = M == 1 ? 1 : (M == 2 ? 2 : 4);
    if (!make_plan((uint32_t)N, (uint32_t)K, MB, true, &p)) return 1;
    return MB == 1 ? dispatch<1, true>(w, d_act, d_out, M, s, p, d_cb, scale)
         : MB == 2 ? dispatch<2, true>(w, d_act, d_out, M, s, p, d_cb, scale) : dispatch<4, true>(w, d_act, d_out, M, s, p, d_cb, scale);
}

}  // namespace oilhip
