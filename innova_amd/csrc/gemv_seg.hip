// gemv_seg.hip -- decode GEMV for tensors whose rows mix wire formats (the 1.50-bpw stacks
// FormatPlanner::allocate produces, src/format_planner.cpp:133-315, and the SPARK mixes of
// FormatRegistry::allocate_mix_blocks, src/format_registry.cpp:477-599): Qwen35Engine::gemm
// (src/adapters/tools/qwen35_engine.cpp:47-85) fused with dequantize_block_all (src/block_codec.cpp:576-720).
//
// Such a tensor is a few MB of small blocks (16 bytes for OIL1, 48 for SPARK_Q0), so the launch is bound by
// dependent memory round trips, not by bandwidth.  The upload therefore stores it as one stream of windows (at most
// 4 KB each) per wavefront, the first at an address that follows from the wavefront's number alone: it is fetched
// blind together with the activations, and a window describes itself and says where the next one is (entries: format, block count, where the blocks and their tags
// sit in the window, which rows they belong to).  A stream covers rows chosen so that all streams weigh about the same, in tiles of up to four;
// inside a tile the blocks are ordered by format, inside a format by row and column, so a step of 8 blocks has one
// format for all 64 lanes.  The wavefront copies a window to LDS with plain 16-byte loads, fetches the next one while it works,
// and decodes from LDS: a lane owns one run of 32 weights and adds its dot product to its accumulator of the run's
// row; when an entry closes its tile each row is summed across the wavefront in a fixed order.
//
// SPARK_Q0 runs (FP16 scale + 32 sign bits) are multiplied as FP16 pairs (+-scale is exact in FP16) through the
// mixed-precision FMA; OIL1 runs are mean * (sum of the run's activations), the sums formed once per launch while x
// is staged.
#include "common.h"
#include "oil4_lds.h"
#include "run_decode.h"

namespace oilhip {
namespace {

constexpr int kRunPad = 36;                // floats per run of 32 activations in LDS: 16-byte reads of neighbouring lanes
                                           // fall into different banks
constexpr int kWaves = 8;                  // wavefronts (streams) per workgroup
constexpr int TR = kSegTileRows;           // accumulators per lane and activation row: a tile has at most this many rows
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct SegArgs {
    uint32_t nstreams, blind16, tag_bytes;
    uint64_t stream_bytes;
    uint32_t cb_bytes[kSegMaxFormats], idx_bytes[kSegMaxFormats], stride[kSegMaxFormats];
};

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// One entry of a window: nblk blocks of format FMT, `stride` bytes apart from `data`, their tags from `tags` (both in LDS).
// adds a run's dot products to the accumulators of its row of the tile
template <int MB>
__device__ __forceinline__ void add_to_row(float (&acc)[MB][TR], uint32_t rowl, const float (&part)[MB]) {
#pragma unroll
    for (int j = 0; j < TR; ++j) {
        const bool mine = rowl == (uint32_t)j;
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m][j] += mine ? part[m] : 0.f;
    }
}

template <int FMT, int MB>
__device__ __forceinline__ void run_entry(const uint8_t* data, const uint8_t* tags, uint32_t tagw, uint32_t nblk, uint32_t stride,
                                          uint32_t cb_bytes, uint32_t idx_bytes, const DecodeTables* __restrict__ T,
                                          const LdsTables& L, const float* xs, const float* rs, float (&acc)[MB][TR],
                                          uint32_t xpad, uint32_t nruns, uint32_t lane) {
    constexpr int N = run_raw_dwords(FMT);
    const uint32_t steps = (nblk + 7u) >> 3, r = lane & 7u, g = lane >> 3;
    // a block's tag: row of the tile and column block, one byte (row << 6 | column) or two (row << 12 | column)
    const uint32_t tshift = tagw == 1u ? 6u : 12u, tmask = tagw == 1u ? 0x3Fu : 0xFFFu;
    auto tag_of = [&](uint32_t b) -> uint32_t {
        return tagw == 1u ? (uint32_t)tags[b] : (uint32_t)reinterpret_cast<const uint16_t*>(tags)[b];
    };
    if constexpr (FMT == 0) {
        // a block is 8 FP16 run means: a lane takes a whole block, 16 bytes of means against 8 run sums
        for (uint32_t b0 = 0; b0 < nblk; b0 += 64u) {
            const uint32_t blk = b0 + lane;
            const bool live = blk < nblk;
            const uint32_t bc = live ? blk : nblk - 1u;
            const uint32_t tag = tag_of(bc);
            const u32x4 mv = *reinterpret_cast<const u32x4*>(data + bc * stride);
            const float mean[8] = {f16_bits(mv.x), f16_bits(mv.x >> 16), f16_bits(mv.y), f16_bits(mv.y >> 16),
                                   f16_bits(mv.z), f16_bits(mv.z >> 16), f16_bits(mv.w), f16_bits(mv.w >> 16)};
            float part[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const float4* sp = reinterpret_cast<const float4*>(rs + (size_t)m * nruns + (tag & tmask) * 8u);
                const float4 s0 = sp[0], s1 = sp[1];
                float a0 = mean[0] * s0.x, a1 = mean[1] * s0.y;
                a0 = __fmaf_rn(mean[2], s0.z, a0);
                a1 = __fmaf_rn(mean[3], s0.w, a1);
                a0 = __fmaf_rn(mean[4], s1.x, a0);
                a1 = __fmaf_rn(mean[5], s1.y, a1);
                a0 = __fmaf_rn(mean[6], s1.z, a0);
                a1 = __fmaf_rn(mean[7], s1.w, a1);
                part[m] = live ? a0 + a1 : 0.f;
            }
            add_to_row<MB>(acc, tag >> tshift, part);
        }
    } else {
    for (uint32_t st = 0; st < steps; ++st) {
        const uint32_t blk = st * 8u + g;
        const bool live = blk < nblk;
        const uint32_t bc = live ? blk : nblk - 1u;                     // past the end: the last block again, result unused
        const uint32_t tag = tag_of(bc);
        const uint8_t* cb = data + bc * stride;
        uint32_t raw[N];
        fetch_run<FMT>(cb, cb_bytes, r, raw);
        const uint32_t rowl = tag >> tshift, run = (tag & tmask) * 8u + r;
        float part[MB];
        if constexpr (FMT == 1) {
            // weight k = bit k ? +scale : -scale; as FP16: |scale| with the sign bit from the (inverted) sign word.
            // Pair k holds weights k (low half) and k + 16 (high half).
            const uint32_t s16 = raw[0] & 0xFFFFu;
            const uint32_t mag = s16 & 0x7FFFu;
            uint32_t mag2 = mag | (mag << 16);
            asm volatile("" : "+v"(mag2));                             // one v_and_or_b32 per pair below, not a multiply-add
            const uint32_t negm = ~raw[1] ^ (0u - (s16 >> 15));
            uint32_t w2[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) w2[k] = ((negm << (15 - k)) & 0x80008000u) | mag2;
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const float* xr = xs + (size_t)m * xpad + run * kRunPad;
                float4 xv[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) xv[c] = *reinterpret_cast<const float4*>(xr + 4 * c);
                float a0 = 0.f, a1 = 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const h2v p0 = __builtin_bit_cast(h2v, w2[4 * c]), p1 = __builtin_bit_cast(h2v, w2[4 * c + 1]);
                    const h2v p2 = __builtin_bit_cast(h2v, w2[4 * c + 2]), p3 = __builtin_bit_cast(h2v, w2[4 * c + 3]);
                    a0 = __fmaf_rn((float)p0[0], xv[c].x, a0);
                    a1 = __fmaf_rn((float)p0[1], xv[c + 4].x, a1);
                    a0 = __fmaf_rn((float)p1[0], xv[c].y, a0);
                    a1 = __fmaf_rn((float)p1[1], xv[c + 4].y, a1);
                    a0 = __fmaf_rn((float)p2[0], xv[c].z, a0);
                    a1 = __fmaf_rn((float)p2[1], xv[c + 4].z, a1);
                    a0 = __fmaf_rn((float)p3[0], xv[c].w, a0);
                    a1 = __fmaf_rn((float)p3[1], xv[c + 4].w, a1);
                }
                part[m] = a0 + a1;
            }
        } else if constexpr (has_dot_run(FMT)) {
            constexpr int MH = MB > 2 ? 2 : MB;          // activation rows per pass: 32 registers of x each
#pragma unroll
            for (int h = 0; h < MB; h += MH) {
                f32x4_t xv[MH][8];
                float xsum[MH], sub[MH];
#pragma unroll
                for (int m = 0; m < MH; ++m) {
                    const float* xr = xs + (size_t)(h + m) * xpad + run * kRunPad;
#pragma unroll
                    for (int c = 0; c < 8; ++c) xv[m][c] = *reinterpret_cast<const f32x4_t*>(xr + 4 * c);
                    xsum[m] = rs[(size_t)(h + m) * nruns + run];
                }
                dot_run<FMT, MH>(raw, r, xv, xsum, sub);
#pragma unroll
                for (int m = 0; m < MH; ++m) part[h + m] = sub[m];
            }
        } else {
            float w[32];
            expand_run<FMT>(raw, cb, cb_bytes, idx_bytes, r, T, L, w);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const float* xr = xs + (size_t)m * xpad + run * kRunPad;
                float a0 = 0.f, a1 = 0.f;
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const float4 xv = *reinterpret_cast<const float4*>(xr + 4 * c);
                    a0 = __fmaf_rn(w[4 * c], xv.x, a0);
                    a1 = __fmaf_rn(w[4 * c + 1], xv.y, a1);
                    a0 = __fmaf_rn(w[4 * c + 2], xv.z, a0);
                    a1 = __fmaf_rn(w[4 * c + 3], xv.w, a1);
                }
                part[m] = a0 + a1;
            }
        }
        if (!live) {
#pragma unroll
            for (int m = 0; m < MB; ++m) part[m] = 0.f;
        }
        add_to_row<MB>(acc, rowl, part);
    }
    }
}

#define OILHIP_SEG_FORMATS(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14)

// MB activation rows per launch.  Dynamic LDS: level tables, MB * (padded x + run sums), two windows per wavefront.
// XF (one activation row only) transforms x while it is staged: 1 = the row holds 2 * cols floats h and the kernel
// multiplies with siluf(h[k]) * h[cols + k] (the SwiGLU product of Qwen35Engine::mlp_step,
// src/adapters/tools/qwen35_engine.cpp:611-621); 2 = x * (1 + xw[k]) is staged and every output is scaled by
// 1 / sqrt(mean(x^2) + 1e-6), which each workgroup forms from the row it loads anyway (Qwen35Engine::rmsnorm, :39-44).
template <int MB, int XF>
__global__ void __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemv_seg_kernel(const uint8_t* __restrict__ streams, const DecodeTables* __restrict__ T, const float* __restrict__ x,
                const float* __restrict__ xw, float* __restrict__ y, uint32_t rows, uint32_t cols, int m0, int M,
                const SegArgs A) {
    static_assert(XF == 0 || MB == 1, "the fused input transforms serve one activation row");
    extern __shared__ __align__(16) float smem[];
    const uint32_t nruns = cols >> 5, xpad = nruns * kRunPad;
    float* ssq_part = smem + kLevelTabBytes / 4;       // XF = 2: sum(x^2) per wavefront
    float* xs = ssq_part + 16;                         // [MB][nruns][36], behind the level tables of dot_run
    float* rs = xs + (size_t)MB * xpad;                // [MB][nruns] run sums
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = uniform(tid >> 6);
    uint8_t* win = reinterpret_cast<uint8_t*>(rs + (size_t)MB * nruns) + (size_t)wave * 2u * kSegWindow;
    const LdsTables L{nullptr, nullptr, nullptr, nullptr};      // the formats that expand weight by weight here use no level table

    const uint32_t sid = blockIdx.x * kWaves + wave;
    const bool active = sid < A.nstreams;
    const uint8_t* sp = streams + (active ? (size_t)sid * A.stream_bytes : 0);
    u32x4 wreg[4];                                     // a window in flight: 4 x 16 bytes per lane
    // the first window is fetched before anything is known about it: as many 16-byte pieces as the fullest first
    // window of the tensor has
    // (pieces past that size repeat the last one: every lane loads, unconditionally, so that nothing waits here)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t piece = j * 64u + lane < A.blind16 ? j * 64u + lane : A.blind16 - 1u;
        wreg[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sp + (size_t)piece * 16u));
    }

    build_level_tables(smem, tid);
    // x -> LDS, 36 floats per run; 8 consecutive threads hold one run and add it up on the way
    const uint32_t nq = cols >> 2;
    float ssq = 0.f;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const bool on = m0 + m < M;
        const float4* xrow = reinterpret_cast<const float4*>(x + (size_t)(on ? m0 + m : 0) * cols * (XF == 1 ? 2u : 1u));
        for (uint32_t c0 = tid; c0 < nq; c0 += 256u * kWaves) {
            float4 v[4], b[XF ? 4 : 1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t c4 = c0 + 64u * kWaves * j;
                v[j] = xrow[c4 < nq ? c4 : c0];
                if constexpr (XF == 1) b[j] = xrow[nq + (c4 < nq ? c4 : c0)];
                if constexpr (XF == 2) b[j] = reinterpret_cast<const float4*>(xw)[c4 < nq ? c4 : c0];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t c4 = c0 + 64u * kWaves * j;
                if (c4 < nq) {
                    float4 t = on ? v[j] : make_float4(0.f, 0.f, 0.f, 0.f);
                    if constexpr (XF == 1) {
                        t.x = (t.x * __builtin_amdgcn_rcpf(1.0f + __expf(-t.x))) * b[j].x;
                        t.y = (t.y * __builtin_amdgcn_rcpf(1.0f + __expf(-t.y))) * b[j].y;
                        t.z = (t.z * __builtin_amdgcn_rcpf(1.0f + __expf(-t.z))) * b[j].z;
                        t.w = (t.w * __builtin_amdgcn_rcpf(1.0f + __expf(-t.w))) * b[j].w;
                    }
                    if constexpr (XF == 2) {
                        ssq = __fmaf_rn(t.x, t.x, __fmaf_rn(t.y, t.y, __fmaf_rn(t.z, t.z, __fmaf_rn(t.w, t.w, ssq))));
                        t.x *= 1.0f + b[j].x; t.y *= 1.0f + b[j].y; t.z *= 1.0f + b[j].z; t.w *= 1.0f + b[j].w;
                    }
                    *reinterpret_cast<float4*>(xs + (size_t)m * xpad + (c4 >> 3) * kRunPad + (c4 & 7u) * 4) = t;
                    float s = (t.x + t.y) + (t.z + t.w);
                    s += oil4::dpp_quad_xor1(s);
                    s += oil4::dpp_quad_xor2(s);
                    s += oil4::dpp_half_mirror(s);
                    if ((c4 & 7u) == 0u) rs[(size_t)m * nruns + (c4 >> 3)] = s;
                }
            }
        }
    }
    if constexpr (XF == 2) {
        float v = ssq;
        v += oil4::dpp_quad_xor1(v);
        v += oil4::dpp_quad_xor2(v);
        v += oil4::dpp_half_mirror(v);
        v += oil4::dpp_row_mirror(v);
        v += oil4::dpp_row_bcast15(v);
        v += oil4::dpp_row_bcast31(v);
        if (lane == 63) ssq_part[wave] = v;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(win + ((size_t)j * 64u + lane) * 16u) = wreg[j];
    __syncthreads();
    if (!active) return;
    float yscale = 1.0f;
    if constexpr (XF == 2) {
        const float tot = ((ssq_part[0] + ssq_part[1]) + (ssq_part[2] + ssq_part[3])) + ((ssq_part[4] + ssq_part[5]) + (ssq_part[6] + ssq_part[7]));
        yscale = 1.0f / sqrtf(tot / (float)cols + 1e-6f);
    }

    float acc[MB][TR];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int j = 0; j < TR; ++j) acc[m][j] = 0.f;
    for (uint32_t wi = 0;; ++wi) {
        const uint8_t* cur = win + (wi & 1u) * kSegWindow;
        const uint32_t* hdr = reinterpret_cast<const uint32_t*>(cur);
        const uint32_t h0 = uniform(hdr[0]);           // 8-byte units of records | another window follows << 12 | its 16-byte pieces << 16
        const bool more = (h0 >> 12) & 1u;
        if (more) {                                    // the next window: its size and place are in this one's header
            const uint32_t used16 = h0 >> 16;
            const uint8_t* np = streams + (size_t)uniform(hdr[1]) * 16u;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t piece = j * 64u + lane < used16 ? j * 64u + lane : used16 - 1u;
                wreg[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(np + (size_t)piece * 16u));
            }
        }
        const uint32_t ne = h0 & 0xFFFu;               // an entry is one unit, the row numbers behind a closing entry two
        for (uint32_t i = 0; i < ne; ++i) {
            const uint32_t* rec = reinterpret_cast<const uint32_t*>(cur) + 2u + 2u * i;
            const uint32_t r0 = uniform(rec[0]), r1 = uniform(rec[1]);
            const uint32_t sl = r0 & 15u, nblk = r0 >> 16, nrows = (r0 >> 9) & 7u;
            const uint8_t* data = cur + (r1 & 0xFFFFu);
            const uint8_t* tags = cur + (r1 >> 16);
#define OILHIP_SEG_CASE(F)                                                                                              \
    case F:                                                                                                             \
        run_entry<F, MB>(data, tags, A.tag_bytes, nblk, A.stride[sl], A.cb_bytes[sl], A.idx_bytes[sl], T, L, xs, rs, acc, xpad,  \
                         nruns, lane);                                                                                  \
        break;
            switch ((r0 >> 4) & 15u) { OILHIP_SEG_FORMATS(OILHIP_SEG_CASE) default: break; }
#undef OILHIP_SEG_CASE
            if ((r0 >> 8) & 1u) {                      // the tile is complete: sum each row across the wavefront
                i += 2;                                // the two units behind a closing entry: the tile's row numbers
                const uint32_t trow[TR] = {uniform(rec[2]), uniform(rec[3]), uniform(rec[4]), uniform(rec[5])};
#pragma unroll
                for (int m = 0; m < MB; ++m)
#pragma unroll
                    for (int j = 0; j < TR; ++j) {
                        float v = acc[m][j];
                        acc[m][j] = 0.f;
                        v += oil4::dpp_quad_xor1(v);
                        v += oil4::dpp_quad_xor2(v);
                        v += oil4::dpp_half_mirror(v);
                        v += oil4::dpp_row_mirror(v);
                        v += oil4::dpp_row_bcast15(v);
                        v += oil4::dpp_row_bcast31(v);
                        if (lane == 63 && (uint32_t)j < nrows && m0 + m < M) y[(size_t)(m0 + m) * rows + trow[j]] = v * yscale;
                    }
            }
        }
        if (more) {
            uint8_t* nxt = win + ((wi + 1u) & 1u) * kSegWindow;
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(nxt + ((size_t)j * 64u + lane) * 16u) = wreg[j];
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");       // other lanes read what this lane wrote
        } else {
            break;
        }
    }
}

template <int MB>
size_t seg_lds_bytes(const oilhip_weights& w) {
    return kLevelTabBytes + 64 + (size_t)MB * ((w.cols >> 5) * (kRunPad + 1)) * 4 + (size_t)kWaves * 2 * kSegWindow;
}

template <int MB, int XF = 0>
int launch_seg(const oilhip_weights& w, const DecodeTables* T, const float* d_x, float* d_y, int m0, int M, hipStream_t s,
               const float* d_xw = nullptr) {
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemv_seg_kernel<MB, XF>;
    const SegLayout& g = w.seg;
    const size_t lds = seg_lds_bytes<MB>(w);
    if (lds > 160 * 1024) return 1;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
    SegArgs A{};
    A.nstreams = g.nstreams; A.blind16 = g.blind16; A.tag_bytes = g.tag_bytes; A.stream_bytes = g.stream_bytes;
    for (uint32_t i = 0; i < g.nf; ++i) { A.cb_bytes[i] = g.cb_bytes[i]; A.idx_bytes[i] = g.idx_bytes[i]; A.stride[i] = g.stride[i]; }
    hipLaunchKernelGGL(kern, dim3((g.nstreams + kWaves - 1) / kWaves), dim3(64 * kWaves), lds, s, w.d_payload, T, d_x, d_xw,
                       d_y, (uint32_t)w.rows, (uint32_t)w.cols, m0, M, A);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace

// Returns 1 when the tensor has no window streams or the shape is outside what this kernel covers.
int launch_gemv_seg(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    if (!w.seg.nstreams || !w.all_full || (w.cols & 255u) || w.rows == 0) return 1;
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    if (seg_lds_bytes<1>(w) > 160 * 1024) return 1;
    int m0 = 0;
    while (m0 < M) {
        const int left = M - m0;
        int rc;
        if (left >= 3 && seg_lds_bytes<4>(w) <= 160 * 1024) { rc = launch_seg<4>(w, T, d_x, d_y, m0, M, s); m0 += 4; }
        else if (left >= 2 && seg_lds_bytes<2>(w) <= 160 * 1024) { rc = launch_seg<2>(w, T, d_x, d_y, m0, M, s); m0 += 2; }
        else { rc = launch_seg<1>(w, T, d_x, d_y, m0, M, s); m0 += 1; }
        if (rc) return rc;
    }
    return OILHIP_OK;
}

// y = W . (siluf(h[0..K)) * h[K..2K)) for one activation row h of 2K floats.  Returns 1 when the tensor is not covered.
int launch_gemv_seg_swiglu(const oilhip_weights& w, const float* d_h, float* d_y, hipStream_t s) {
    if (!w.seg.nstreams || !w.all_full || (w.cols & 255u) || w.rows == 0 || seg_lds_bytes<1>(w) > 160 * 1024) return 1;
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    return launch_seg<1, 1>(w, T, d_h, d_y, 0, 1, s);
}

// y = W . rmsnorm(x; xw) for one activation row.  Returns 1 when the tensor is not covered.
int launch_gemv_seg_rmsnorm(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, hipStream_t s) {
    if (!w.seg.nstreams || !w.all_full || (w.cols & 255u) || w.rows == 0 || seg_lds_bytes<1>(w) > 160 * 1024) return 1;
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    return launch_seg<1, 2>(w, T, d_x, d_y, 0, 1, s, d_xw);
}

}  // namespace oilhip
