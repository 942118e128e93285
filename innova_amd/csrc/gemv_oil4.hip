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
// Mapping.  8 lanes cover one 128-byte block with one 16-byte load each (32
// nibbles per lane), so one wave-load covers 8 consecutive blocks of a row (a
// "column set", 1 KB).  A wavefront owns CS consecutive column sets (a slab of
// the row) and walks down rows.  A lane sees the same 32*CS nibble positions in
// every row, so its activations live in registers for the whole kernel,
// gathered once from an LDS copy of x (scale nibbles and blocks past the end of
// the row get activation 0).  Per packed byte the two level values come from
// one LDS read of a 256-entry pair table whose address is built by a single
// v_perm_b32, followed by two FP32 FMAs.  The block's FP16 scale is applied to
// the lane's 32-nibble partial sum; one 6-step DPP reduction per row and slab
// finishes the dot product.  The kernel is issue-bound on the vector ALU, so
// everything outside the per-byte perm + 2 FMAs is kept to a handful of
// instructions per row.
#include <hip/hip_fp16.h>


#include "common.h"
#include "oil4_lds.h"

namespace oilhip {
namespace {

using namespace oil4;

constexpr int kXsBlock = 288;  // floats per block in the LDS copy of x: 256 + 32 so that neighbouring blocks start 32 banks apart

// CS: column sets (wave-loads) per row and wave; RPW: rows per chunk, all loads of
// a chunk in flight at once; MB: activation rows handled together; MAXT: workgroup size bound.
// XF = 1: the activation row is not x itself but silu(h[k]) * h[cols + k] of a row h of 2*cols floats (the gate and
// up projections of an MLP step, Qwen35Engine::mlp_step, src/adapters/tools/qwen35_engine.cpp:611-621), formed
// while x is staged, so the SwiGLU product never makes a round trip through memory.
// XF = 2: the activation row is rmsnorm(x) = x * r * (1 + xw), r = 1 / sqrt(mean(x^2) + 1e-6) (rmsnorm, same file :39-44):
// x * (1 + xw) is staged, every workgroup forms r from the whole row it loads anyway, and r scales the dot products.
// XF = 3: not a block tensor but rows of cols/2 bytes of packed codes (low nibble first) with a 16-entry FP16 codebook
// passed through xw and one scale for the whole matrix (gemv_oil4 of src/kernel_production.cpp): x stays in natural
// order, the pair table is built from the codebook, there is no block scale and y is multiplied by out_scale.
template <int CS, int RPW, int MB, int WGT, int XF = 0, bool ROLL = false>
__global__ void __launch_bounds__(WGT) __attribute__((amdgpu_waves_per_eu(WGT / 256, WGT / 256)))
gemv_oil4_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, const float* __restrict__ xw, float* __restrict__ y,
                 uint32_t rows, uint32_t cols, uint32_t S, uint32_t G, uint32_t nchunks, int m0, int M,
                 uint32_t rg_base, uint32_t rg_rem, uint32_t wave_groups_lo, uint32_t wave_groups_hi, float out_scale) {
    constexpr uint32_t NW = WGT / 64;   // wavefronts per workgroup
    constexpr int NL = CS * RPW;      // wave-loads per chunk
    constexpr int LA = 4;             // dwords of a wave-load decoded per pipeline step: two wavefronts per SIMD stage a whole wave-load
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                               // LDS byte offset 0
    const uint32_t nblk = S * CS * 8;                                         // blocks covered by all slabs (>= cols/256)
    const uint32_t xstride = nblk * kXsBlock;                                 // floats per activation row in LDS
    float* xs = reinterpret_cast<float*>(lds + kTabBytes);                    // [MB][nblk][8 c][8 lp][4 e] (+32 pad), nibble order
    float* red = xs + (size_t)MB * xstride;                                   // [G][RPW][MB][S]

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));      // uniform: scalar registers
    const uint32_t grp = ((wave < 8u ? wave_groups_lo : wave_groups_hi) >> (4u * (wave & 7u))) & 15u, slab = wave - grp * S;   // wave / S, wave % S
    const uint32_t bpr = cols >> 8;
    const uint32_t lp = lane & 7u;

    // row group j owns rows [j*rg_base + min(j, rg_rem), ...): rows split evenly over gridDim.x * G groups
    auto group_begin = [&](uint32_t j) { return j * rg_base + (j < rg_rem ? j : rg_rem); };
    const uint32_t jg = blockIdx.x * G + grp;
    const bool working = wave < S * G;                                        // spare wavefronts only help with the prologue
    const uint32_t r0 = working ? group_begin(jg) : 0u, r1 = working ? group_begin(jg + 1) : 0u;
    const uint32_t row_bytes = bpr * 128u;
    // Buffer resource over this wavefront's rows only: a load of a row past r1 is out of range (zeros, no fetch)
    // without any compare.  The host checks that a row group plus two chunks of rows stays below 2^31 bytes.
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)r0 * row_bytes), 0, (int)((r1 - r0) * row_bytes), 0x00020000);

    // ---- x first (needed soonest), then every weight load of the first chunk ----------
    // Nothing that waits on vector memory may follow the weight loads before their use:
    // loads return in order, so it would wait for every weight byte.
    constexpr int XPT = 2048 / WGT;   // float4 pieces of x fetched up front per thread
    constexpr uint32_t XW = XF == 1 ? 2u : 1u;                                // input floats per activation
    const __amdgpu_buffer_rsrc_t nrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(XF == 2 ? xw : x), 0, (int)(cols * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(x + (size_t)m0 * cols * XW), 0, (int)((uint32_t)(M - m0 < MB ? M - m0 : MB) * cols * XW * 4u), 0x00020000);
    u32x4 xpre[MB][XPT], xup[XF ? MB : 1][XF ? XPT : 1];
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t d4 = tid + u * (uint32_t)WGT;                    // float4 index into the padded row
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const uint32_t off = (d4 * 4u < cols && m0 + m < M) ? d4 * 16u + m * cols * XW * 4u : kOobOffset;
            xpre[m][u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 0, 0);
            if (XF == 1) xup[m][u] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off == kOobOffset ? kOobOffset : off + cols * 4u, 0, 0);
            if (XF == 2) xup[m][u] = __builtin_amdgcn_raw_buffer_load_b128(nrsrc, d4 * 4u < cols ? d4 * 16u : kOobOffset, 0, 0);
        }
    }
    auto swiglu4 = [&](const u32x4& g, const u32x4& up) {                     // (g * sigmoid(g)) * up, sigmoid = 1 / (1 + exp(-g))
        u32x4 r;
        const uint32_t gg[4] = {g.x, g.y, g.z, g.w}, uu[4] = {up.x, up.y, up.z, up.w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float v = __uint_as_float(gg[k]);
            o[k] = __float_as_uint((v * __builtin_amdgcn_rcpf(1.0f + __expf(-v))) * __uint_as_float(uu[k]));
        }
        r.x = o[0]; r.y = o[1]; r.z = o[2]; r.w = o[3];
        return r;
    };
    float ssq = 0.0f;                                                         // XF = 2: this thread's share of sum(x^2)
    auto norm4 = [&](const u32x4& g, const u32x4& nw) {                       // x * (1 + xw), and x^2 into ssq
        u32x4 r;
        const uint32_t gg[4] = {g.x, g.y, g.z, g.w}, ww[4] = {nw.x, nw.y, nw.z, nw.w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float v = __uint_as_float(gg[k]);
            ssq = __fmaf_rn(v, v, ssq);
            o[k] = __float_as_uint(v * (1.0f + __uint_as_float(ww[k])));
        }
        r.x = o[0]; r.y = o[1]; r.z = o[2]; r.w = o[3];
        return r;
    };
    auto transform4 = [&](const u32x4& g, const u32x4& b) {
        if constexpr (XF == 1) return swiglu4(g, b);
        else if constexpr (XF == 2) return norm4(g, b);
        else return g;
    };
    // Byte offset of this lane inside a row for each column set; lanes past the end of the row get an offset that
    // stays out of range whatever row offset is added.
    uint32_t vcol[CS];
#pragma unroll
    for (int cs = 0; cs < CS; ++cs) {
        const uint32_t blk = (slab * CS + cs) * 8u + (lane >> 3);
        vcol[cs] = blk < bpr ? blk * 128u + lp * 16u : 0x80000000u;
    }
    // Wave-load n of a chunk: row n / CS of the chunk, column set n % CS.  About six loads per wavefront are
    // queued before the prologue is over (the memory pipeline of a CU holds a limited number of outstanding
    // lines; queueing more only stalls the wavefront in front of its prologue), the first three while the table
    // is written so that the younger wavefronts get their first rows early too; the rest follow once the
    // prologue is done, while the first ones are being consumed.
    constexpr int PFA = NL < 3 ? NL : 3;          // queued while the table is written
    constexpr int PFB = NL < 6 ? NL : 6;          // ... by the time x is staged
    constexpr int PFC = NL < 6 ? NL : 6;          // ... by the barrier
    u32x4 wv[NL];
    auto issue_load = [&](int n, uint32_t rel) {           // rel: first row of the chunk, counted from r0
        const int it = n / CS, cs = n % CS;
        wv[n] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, vcol[cs] + (rel + it) * row_bytes, 0, 2);   // aux 2 = nt: streamed once, not kept in L2 / the Infinity Cache
    };
    // The 64 KB pair table is written while the weight loads queue up: float4 number e of the
    // table is (lo, hi, lo, hi) of byte value v = e >> 4, and thread tid writes e = tid + WGT*k,
    // k = 0 .. 4096/WGT - 1, so its low nibble (tid >> 4) & 15 is fixed and its high nibble is
    // (tid >> 8) + (WGT/256) k, uniform across the wavefront.  Levels come from literals: no memory access, no barrier.
    // A wave-load takes the address unit of the CU a good dozen cycles and eight wavefronts queue there, so the
    // table writes are slotted in between the loads instead of after them.
    issue_load(0, 0u);
    __builtin_amdgcn_sched_barrier(0);
    float lv_lane, lo_fix;                                                    // lane i holds level[i & 15]
    if (XF == 3) {
        const uint16_t* cb16 = reinterpret_cast<const uint16_t*>(xw);
        auto widen = [](uint32_t h) {                                         // fp16_to_float of the flat kernels: NaNs become the default NaN
            return ((h >> 10) & 31u) == 31u && (h & 0x3FFu) != 0u ? __uint_as_float(0x7FC00000u) : half_bits_to_float(h);
        };
        lv_lane = widen(cb16[lane & 15u]);
        lo_fix = widen(cb16[(tid >> 4) & 15u]);
    } else {
        lv_lane = level_literal(lane & 15u);
        lo_fix = level_literal((tid >> 4) & 15u);
    }
    constexpr int TK = 4096 / WGT;                                            // table writes per thread
#pragma unroll
    for (int k = 0; k < TK; ++k) {
        if (k + 1 < PFA) issue_load(k + 1, 0u);
        const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lv_lane), (int)((wave >> 2) + (uint32_t)(WGT / 256) * k)));
        reinterpret_cast<float4*>(tab)[tid + (uint32_t)WGT * k] = make_float4(lo_fix, hi, lo_fix, hi);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int n = (PFA < TK + 1 ? PFA : TK + 1); n < PFB; ++n) issue_load(n, 0u);
    __builtin_amdgcn_sched_barrier(0);

    // ---- x into LDS in nibble order -------------------------------------------------------------
    // Weight i of a block sits at nibble p = i - i/64 + 4 (slots i % 64 == 63 own no nibble); lane
    // lp of the block holds nibbles 32*lp .. 32*lp+31 and reads them as 8 float4 (c = 0..7), so
    // x[i] goes to xs[blk*288 + c*32 + lp*4 + e] with p = 32*lp + 4*c + e.  The four scale
    // nibbles (p < 4) and blocks past the end of the row hold zeros.
    // A thread's float4 number d4 = tid + u*blockDim keeps the same position inside its block for
    // every u when blockDim is a multiple of 64, so the four target offsets are computed once.
    uint32_t xoff[4];
    bool xlast_ok;
    {
        const uint32_t w = (tid * 4u) & 255u;
        xlast_ok = XF == 3 || (w & 63u) != 60u;                               // i % 64 == 63 is a slot
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t pnib = XF == 3 ? w + k : w + k - (w >> 6) + 4u;
            xoff[k] = ((pnib >> 2) & 7u) * 32u + (pnib >> 5) * 4u + (pnib & 3u);
        }
    }
    auto scatter4 = [&](uint32_t d4, const u32x4& v, int m) {
        float* dst = xs + (size_t)m * xstride + (d4 >> 6) * kXsBlock;
        dst[xoff[0]] = __uint_as_float(v.x);
        dst[xoff[1]] = __uint_as_float(v.y);
        dst[xoff[2]] = __uint_as_float(v.z);
        if (xlast_ok) dst[xoff[3]] = __uint_as_float(v.w);
    };
    for (uint32_t bz = tid; XF != 3 && bz < nblk * MB; bz += (uint32_t)WGT) { // scale nibbles of every block
        const uint32_t m = bz / nblk, b = bz % nblk;
        *reinterpret_cast<float4*>(xs + (size_t)m * xstride + b * kXsBlock) = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (uint32_t z = bpr * 64u + tid; z < nblk * 64u; z += (uint32_t)WGT) {  // blocks past the end of the row
#pragma unroll
        for (int m = 0; m < MB; ++m)
            reinterpret_cast<float4*>(xs + (size_t)m * xstride + (z >> 6) * kXsBlock)[z & 63u] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
        const uint32_t d4 = tid + u * (uint32_t)WGT;
        if (d4 * 4u < cols) {
#pragma unroll
            for (int m = 0; m < MB; ++m) scatter4(d4, transform4(xpre[m][u], xup[XF ? m : 0][XF ? u : 0]), m);
        }
    }
    for (uint32_t d4 = tid + XPT * (uint32_t)WGT; d4 * 4u < cols; d4 += (uint32_t)WGT) {    // rows wider than XPT*4*workgroup
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const uint32_t off = (m0 + m < M) ? d4 * 16u + m * cols * XW * 4u : kOobOffset;
            const u32x4 g = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 0, 0);
            if (XF == 1) scatter4(d4, swiglu4(g, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, off == kOobOffset ? kOobOffset : off + cols * 4u, 0, 0)), m);
            else if (XF == 2) scatter4(d4, norm4(g, __builtin_amdgcn_raw_buffer_load_b128(nrsrc, d4 * 16u, 0, 0)), m);
            else scatter4(d4, g, m);
        }
    }
#pragma unroll
    for (int n = PFB; n < PFC; ++n) issue_load(n, 0u);
    float* ssq_part = red + (size_t)G * RPW * MB * S;                         // one float per wavefront past the slab partials
    if (XF == 2) {
        float v = ssq;
        v += dpp_quad_xor1(v);
        v += dpp_quad_xor2(v);
        v += dpp_half_mirror(v);
        v += dpp_row_mirror(v);
        v += dpp_row_bcast15(v);
        v += dpp_row_bcast31(v);
        if (lane == 63) ssq_part[wave] = v;
    }
    __syncthreads();
    float yscale = XF == 3 ? out_scale : 1.0f;
    if (XF == 2) {
        float tot = 0.0f;
#pragma unroll
        for (uint32_t q = 0; q < NW; q += 4) tot += (ssq_part[q] + ssq_part[q + 1]) + (ssq_part[q + 2] + ssq_part[q + 3]);
        yscale = 1.0f / sqrtf(tot / (float)cols + 1e-6f);
    }

    // ---- this lane's activations: 8 float4 per column set ------------------------------------
    float xr[MB][CS][32];
#pragma unroll
    for (int cs = 0; cs < CS; ++cs) {
        const uint32_t blk = (slab * CS + cs) * 8u + (lane >> 3);
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float4 t = *reinterpret_cast<const float4*>(xs + (size_t)m * xstride + blk * kXsBlock + c * 32 + lp * 4);
                xr[m][cs][4 * c + 0] = t.x; xr[m][cs][4 * c + 1] = t.y; xr[m][cs][4 * c + 2] = t.z; xr[m][cs][4 * c + 3] = t.w;
            }
    }

    const uint32_t lanebase = (lane & 31u) * 8u;          // byte offset of this lane's table copy

#pragma unroll
    for (int n = PFC; n < NL; ++n) issue_load(n, 0u);     // rest of the first chunk
    for (uint32_t ch = 0; ch < nchunks; ++ch) {
        const uint32_t cbase = r0 + ch * RPW;
        if (!ROLL && ch > 0) {
#pragma unroll
            for (int n = 0; n < NL; ++n) issue_load(n, ch * RPW);
        }
        float part[MB][RPW];                              // per-lane partial of each row, block scales applied
        // A wave-load is consumed in units of LA dwords (4 LA packed bytes): the table reads of the next unit are in
        // flight while the products of the current one are formed; with two wavefronts per SIMD a unit is a whole
        // wave-load.
        constexpr int UPL = 4 / LA, UB = 4 * LA;          // units per wave-load, packed bytes per unit
        LevelPair cur[UB];
        auto lookup_unit = [&](int u, LevelPair (&t)[UB]) {
            const u32x4 w4 = wv[u / UPL];
            const uint32_t wd[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int d = 0; d < LA; ++d) {
                const uint32_t word = wd[(u % UPL) * LA + d];
                t[4 * d + 0] = lookup<0>(word, lanebase);
                t[4 * d + 1] = lookup<1>(word, lanebase);
                t[4 * d + 2] = lookup<2>(word, lanebase);
                t[4 * d + 3] = lookup<3>(word, lanebase);
            }
        };
        lookup_unit(0, cur);
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int it = n / CS, cs = n % CS;
            // The wavefronts of a SIMD are served oldest first; left alone the older one runs ahead and the
            // younger finishes its rows on its own.  Priority falls with progress, so whichever is behind goes first.
            if (!ROLL && (n == 0 || (n * 4) / NL != ((n - 1) * 4) / NL)) {
                const int pr = 3 - (n * 4) / NL;
                if (pr == 3) __builtin_amdgcn_s_setprio(3);
                else if (pr == 2) __builtin_amdgcn_s_setprio(2);
                else if (pr == 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
            }
            float a0[MB], a1[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) { a0[m] = 0.0f; a1[m] = 0.0f; }
#pragma unroll
            for (int q = 0; q < UPL; ++q) {
                const int u = n * UPL + q;
                LevelPair nxt[UB];
                const bool more = u + 1 < NL * UPL;
                if (more) lookup_unit(u + 1, nxt);                    // next unit's table reads fly during these FMAs
                __builtin_amdgcn_sched_barrier(0);                    // keep them above the FMAs
#pragma unroll
                for (int m = 0; m < MB; ++m) {
#pragma unroll
                    for (int k = 0; k < UB; k += 2) {
                        const int kb = q * UB + k;                    // packed byte of the wave-load
                        a0[m] = __fmaf_rn(cur[k].lo, xr[m][cs][2 * kb], a0[m]);
                        a0[m] = __fmaf_rn(cur[k].hi, xr[m][cs][2 * kb + 1], a0[m]);
                        a1[m] = __fmaf_rn(cur[k + 1].lo, xr[m][cs][2 * kb + 2], a1[m]);
                        a1[m] = __fmaf_rn(cur[k + 1].hi, xr[m][cs][2 * kb + 3], a1[m]);
                    }
                }
                if (q == UPL - 1) {
                    // the block's FP16 scale sits in the low half of its first lane's first dword
                    const float scale = XF == 3 ? 1.0f : __half2float(__ushort_as_half((unsigned short)(dpp_bcast8(wv[n].x) & 0xFFFFu)));
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        part[m][it] = cs == 0 ? (a0[m] + a1[m]) * scale : __fmaf_rn(a0[m] + a1[m], scale, part[m][it]);
                    // ROLL (shapes with more than one chunk): wv[n] is free, the same wave-load of the next chunk takes its
                    // place, so NL loads stay in flight across chunks.  Issued unconditionally (past the last row the offset is
                    // out of range: zeros, no fetch), which keeps the count of outstanding loads at every wait a constant.
                    if (ROLL) issue_load(n, (ch + 1u) * RPW);
                }
                if (more) {
#pragma unroll
                    for (int k = 0; k < UB; ++k) cur[k] = nxt[k];
                }
                __builtin_amdgcn_sched_barrier(0);                    // one scheduling region per unit
            }
        }
        // ---- all rows of the chunk reduced over the 64 lanes together (independent chains) ----
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
                part[m][it] = v;                          // lane 63 holds the slab's dot product
            }
        if (S == 1) {                                     // a wave covers whole rows: lane 63 stores y
            if (lane == 63) {
#pragma unroll
                for (int it = 0; it < RPW; ++it)
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        if (cbase + it < r1 && m0 + m < M) y[(size_t)(m0 + m) * rows + cbase + it] = XF >= 2 ? part[m][it] * yscale : part[m][it];
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
        // ---- slab partials -> y -------------------------------------------------
        for (uint32_t o = tid; o < G * RPW * MB; o += (uint32_t)WGT) {
            const uint32_t g2 = o / (RPW * MB), rem = o % (RPW * MB), slot = rem / MB, m = rem % MB;
            const uint32_t jg2 = blockIdx.x * G + g2;
            const uint32_t q0 = group_begin(jg2), q1 = group_begin(jg2 + 1);
            const uint32_t r = q0 + ch * RPW + slot;
            if (r < q1 && m0 + (int)m < M) {
                const float* pr = red + (size_t)o * S;
                float s = 0.0f;
                for (uint32_t k = 0; k < S; ++k) s += pr[k];
                y[(size_t)(m0 + m) * rows + r] = XF >= 2 ? s * yscale : s;
            }
        }
        __syncthreads();
    }
}

constexpr int kWgt = 512;          // threads per workgroup of the decode kernel

// One launch configuration of the kernel above.
struct Oil4Plan {
    int cs, rpw, maxt;     // template choice
    uint32_t S, G, grid, nchunks;
    size_t lds_bytes;
};

template <int CS, int RPW, int MB, int WGT, int XF, bool ROLL>
int launch(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, int M, hipStream_t s, const Oil4Plan& p,
           float out_scale = 1.0f) {
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemv_oil4_kernel<CS, RPW, MB, WGT, XF, ROLL>;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), kMaxLds)) return rc;
    const uint32_t J = p.grid * p.G;
    uint64_t wave_groups = 0;                                   // wave / S for each of the wavefronts, 4 bits each
    for (uint32_t wv = 0; wv < (uint32_t)WGT / 64u; ++wv) wave_groups |= (uint64_t)(wv / p.S) << (4u * wv);
    for (int m0 = 0; m0 < M; m0 += MB) {
        hipLaunchKernelGGL(kern, dim3(p.grid), dim3(WGT), p.lds_bytes, s, w.d_payload, d_x, d_xw, d_y,
                           (uint32_t)w.rows, (uint32_t)w.cols, p.S, p.G, p.nchunks, m0, M,
                           (uint32_t)w.rows / J, (uint32_t)w.rows % J, (uint32_t)wave_groups, (uint32_t)(wave_groups >> 32), out_scale);
        OILHIP_HIP(hipGetLastError());
    }
    return OILHIP_OK;
}

// Chooses column sets per wave, slabs, waves per workgroup and chunking for a shape.
bool make_plan(uint32_t rows, uint32_t cols, int MB, int waves_target, Oil4Plan* p) {
    const uint32_t sets = ((cols >> 8) + 7) / 8;                  // column sets (1 KB wave-loads) per row
    // register budget: 32*CS*MB activations per lane, out of 256 registers (two wavefronts per SIMD)
    const int cs_max = MB == 1 ? 3 : 1;
    // fewest slabs first (less cross-wave reduction), then least padding
    int best_cs = 1; uint32_t best_S = sets; double best_cost = 1e30;
    for (int cs = 1; cs <= cs_max; ++cs) {
        const uint32_t S = (sets + cs - 1) / cs;
        if (S > (uint32_t)waves_target) continue;
        const double waste = (double)(S * cs) / (double)sets;      // >= 1: padded column sets cost ALU time
        const double cost = waste + 0.04 * (S > 1 ? S : 0);
        if (cost < best_cost) { best_cost = cost; best_cs = cs; best_S = S; }
    }
    if (best_cost > 1e29) return false;
    const uint32_t S = best_S;
    uint32_t G = (uint32_t)waves_target / S;
    if (G == 0) G = 1;
    uint32_t grid = (uint32_t)device_cu_count();
    if (grid * G > rows) grid = (rows + G - 1) / G;
    if (grid == 0) grid = 1;
    const uint32_t Jn = grid * G;
    const uint32_t max_rows = (rows + Jn - 1) / Jn;                // rows of the largest row group
    const int budget = 12 / best_cs;                               // wave-loads in flight per wave (register budget)
    int rpw = 1;
    if (max_rows <= (uint32_t)budget) {                            // one chunk: the smallest that holds every row
        for (int cand : {1, 2, 3, 4, 6, 12}) if ((uint32_t)cand >= max_rows) { rpw = cand; break; }
    } else {                                                       // several chunks, loads rolling from one into the next:
        int lo = (6 + best_cs - 1) / best_cs;                      // about six wave-loads in flight are enough, more only
        if (lo > budget) lo = budget;                              // crowd the memory pipeline; least padded row slots
        uint32_t best_slots = ~0u;
        for (int cand : {1, 2, 3, 4, 6, 12}) {
            if (cand < lo || cand > budget) continue;
            const uint32_t slots = (max_rows + cand - 1) / cand * cand;
            if (slots < best_slots) { best_slots = slots; rpw = cand; }
        }
    }
    p->cs = best_cs; p->rpw = rpw; p->maxt = kWgt;
    p->S = S; p->G = G; p->grid = grid;
    p->nchunks = (max_rows + rpw - 1) / rpw;
    if (p->nchunks == 0) p->nchunks = 1;
    p->lds_bytes = (size_t)kTabBytes + 4ull * MB * (S * best_cs * 8 * kXsBlock) + 4ull * G * rpw * MB * S + 64;
    if ((uint64_t)(max_rows + 2u * (uint32_t)rpw) * ((uint64_t)(cols >> 8) * 128u) >= 0x80000000ull) return false;   // per-wave buffer range
    return p->lds_bytes <= (size_t)kMaxLds && S * G <= (uint32_t)kWgt / 64u;
}

template <int MB, int XF = 0>
int dispatch(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, int M, hipStream_t s, const Oil4Plan& p,
             float out_scale = 1.0f) {
#define OIL4_CASE(CS_, RPW_) \
    if (p.cs == CS_ && p.rpw == RPW_) \
        return p.nchunks > 1 ? launch<CS_, RPW_, MB, kWgt, XF, true>(w, d_x, d_xw, d_y, M, s, p, out_scale) \
                             : launch<CS_, RPW_, MB, kWgt, XF, false>(w, d_x, d_xw, d_y, M, s, p, out_scale);
    OIL4_CASE(1, 1) OIL4_CASE(1, 2) OIL4_CASE(1, 3) OIL4_CASE(1, 4) OIL4_CASE(1, 6) OIL4_CASE(1, 12)
    if constexpr (MB == 1) {
        OIL4_CASE(2, 1) OIL4_CASE(2, 2) OIL4_CASE(2, 3) OIL4_CASE(2, 4) OIL4_CASE(2, 6)
        OIL4_CASE(3, 1) OIL4_CASE(3, 2) OIL4_CASE(3, 3) OIL4_CASE(3, 4)
    }
#undef OIL4_CASE
    return 1;
}

}  // namespace

int launch_gemv_oil4(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull || M > 16) return 1;
    Oil4Plan p;                                   // rows beyond two go in passes of two (the matrix-core kernel is the
    const int MB = M == 1 ? 1 : 2;                // better choice there and the caller tries it first)
    if (!make_plan((uint32_t)w.rows, (uint32_t)w.cols, MB, kWgt / 64, &p)) return 1;
    return MB == 1 ? dispatch<1>(w, d_x, nullptr, d_y, M, s, p) : dispatch<2>(w, d_x, nullptr, d_y, M, s, p);
}

// y = W . (silu(h[0..K)) * h[K..2K)) for one activation row h of 2K floats.  Returns 1 when the shape is not covered.
int launch_gemv_oil4_swiglu(const oilhip_weights& w, const float* d_h, float* d_y, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x3FFFFFFFull) return 1;
    Oil4Plan p;
    if (!make_plan((uint32_t)w.rows, (uint32_t)w.cols, 1, kWgt / 64, &p)) return 1;
    return dispatch<1, 1>(w, d_h, nullptr, d_y, 1, s, p);
}

// y = W . rmsnorm(x; xw) for one activation row.  Returns 1 when the shape is not covered.
int launch_gemv_oil4_rmsnorm(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x3FFFFFFFull) return 1;
    Oil4Plan p;
    if (!make_plan((uint32_t)w.rows, (uint32_t)w.cols, 1, kWgt / 64, &p)) return 1;
    return dispatch<1, 2>(w, d_x, d_xw, d_y, 1, s, p);
}

// gemv_oil4 of src/kernel_production.cpp for one activation row: y[r] = scale * sum_k f16(cb16[code(r, k)]) * x[k], rows
// of K/2 bytes, low nibble first.  Returns 1 when the shape is not covered (K must be a multiple of 256).
int launch_gemv_flat4(const uint8_t* d_w, const uint16_t* d_cb16, float scale, const float* d_x, float* d_y, int rows, int K,
                      hipStream_t s) {
    if (rows < 1 || K < 256 || (K & 255) || (reinterpret_cast<uintptr_t>(d_w) & 15u)) return 1;
    oilhip_weights w;                                             // a view: rows of K/2 bytes
    w.d_payload = const_cast<uint8_t*>(d_w);
    w.rows = (uint64_t)rows; w.cols = (uint64_t)K;
    Oil4Plan p;
    if (!make_plan((uint32_t)rows, (uint32_t)K, 1, kWgt / 64, &p)) return 1;
    return dispatch<1, 3>(w, d_x, reinterpret_cast<const float*>(d_cb16), d_y, 1, s, p, scale);
}

}  // namespace oilhip
