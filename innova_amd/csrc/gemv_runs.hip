// gemv_runs.hip -- decode GEMV for uniform tensors of every wire format that has no kernel of its own (all but OIL4
// and OIL8), and the fallback for mixed tensors the window-stream kernel does not take: Qwen35Engine::gemm
// (src/adapters/tools/qwen35_engine.cpp:47-85) fused with dequantize_block_all (src/block_codec.cpp:576-720).
//
// A lane owns one run of 32 consecutive weights: 8 lanes cover a 256-weight block and a
// wavefront-step covers 8 consecutive blocks of a row.  Each lane fetches only the bytes of its
// run (2 bytes for OIL1, 6 for SPARK_Q0, 16 for OIL4, ...), decodes them with the format's own
// short routine into 32 registers and multiplies them with its 32 activations, which sit in LDS
// with 4 floats of padding per run so that the 16-byte reads of neighbouring lanes fall into
// different banks.  OIL1 needs no per-weight work at all: its run contributes mean * sum(x over
// the run), and the run sums are computed once per launch.  Block addresses follow from the constant
// stride of a uniform tensor, or from the 16-byte descriptors otherwise (lanes of a step whose blocks
// differ in format then diverge by 8-lane group).  Formats without a short routine go through the
// general per-weight decoder.
#include "common.h"
#include "run_decode.h"

namespace oilhip {
namespace {

constexpr int kRunPad = 36;                // floats per run of 32 activations in LDS

struct Run {                                // what a lane needs to know about its run
    const uint8_t* cb;                      // block payload: codebook channel, then index channel
    uint32_t cb_bytes, idx_bytes;
    uint32_t fmt, r;                        // format id, run 0..7 inside the block
};

template <int FMT>
__device__ __forceinline__ void decode_one(const Run& R, const DecodeTables* __restrict__ T, const LdsTables& L, float (&w)[32]) {
    uint32_t raw[run_raw_dwords(FMT)];
    fetch_run<FMT>(R.cb, R.cb_bytes, R.r, raw);
    expand_run<FMT>(raw, R.cb, R.cb_bytes, R.idx_bytes, R.r, T, L, w);
}

// Decodes the lane's 32 weights.  Returns false when the run was handled as OIL1 (w untouched, *mean set).
__device__ __forceinline__ bool decode_run(const Run& R, const DecodeTables* __restrict__ T, const LdsTables& L, float (&w)[32], float* mean) {
    switch (R.fmt) {
        case 0: {
            uint32_t raw[1];
            fetch_run<0>(R.cb, R.cb_bytes, R.r, raw);
            *mean = oil1_mean(raw);
            return false;
        }
        case 1: decode_one<1>(R, T, L, w); return true;
        case 2: decode_one<2>(R, T, L, w); return true;
        case 3: decode_one<3>(R, T, L, w); return true;
        case 4: decode_one<4>(R, T, L, w); return true;
        case 5: decode_one<5>(R, T, L, w); return true;
        case 6: decode_one<6>(R, T, L, w); return true;
        case 7: decode_one<7>(R, T, L, w); return true;
        case 9: decode_one<9>(R, T, L, w); return true;
        case 10: decode_one<10>(R, T, L, w); return true;
        case 11: decode_one<11>(R, T, L, w); return true;
        case 12: decode_one<12>(R, T, L, w); return true;
        default: {  // SPARK_Q0_GRP, sparse formats: the general decoder, weight by weight
            for (int k = 0; k < 32; ++k)
                w[k] = decode_weight(R.fmt, R.cb, R.cb_bytes, R.cb + R.cb_bytes, R.idx_bytes, 256u, 32u * R.r + (uint32_t)k, T);
            return true;
        }
    }
}

// MB activation rows per launch.  Dynamic LDS: MB * (padded x + run sums).
template <int MB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
gemv_runs_kernel(const uint8_t* __restrict__ payload, const DevBlock* __restrict__ blocks, const DecodeTables* __restrict__ T,
                 const float* __restrict__ x, float* __restrict__ y, uint32_t rows, uint32_t cols, int m0, int M,
                 int uniform_fmt, uint32_t uniform_stride, uint32_t uniform_cb, uint32_t uniform_idx, uint32_t uniform_base) {
    extern __shared__ __align__(16) float smem[];
    const uint32_t bpr = cols >> 8, nruns = cols >> 5;
    const uint32_t xpad = nruns * kRunPad;
    float* xs = smem;                                  // [MB][nruns][36]
    float* rs = smem + (size_t)MB * xpad;              // [MB][nruns] run sums
    float* tb = rs + (size_t)MB * nruns;               // level tables: lv8[256] t255[256] lv4[16] lv2[4]
    for (uint32_t i = threadIdx.x; i < 532u; i += 256u)
        tb[i] = i < 256u ? T->lv8[i] : i < 512u ? T->t255[i - 256u] : i < 528u ? kLv4[i - 512u] : kLv2[i - 528u];
    const LdsTables L{tb + 528, tb + 512, tb, tb + 256};
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    for (uint32_t k4 = tid; k4 < (cols >> 2) * MB; k4 += 256u) {
        const uint32_t m = k4 / (cols >> 2), c4 = k4 % (cols >> 2);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m0 + (int)m < M) v = *reinterpret_cast<const float4*>(x + (size_t)(m0 + m) * cols + c4 * 4);
        *reinterpret_cast<float4*>(xs + (size_t)m * xpad + (c4 >> 3) * kRunPad + (c4 & 7u) * 4) = v;
    }
    __syncthreads();
    for (uint32_t q = tid; q < nruns * MB; q += 256u) {
        const float* p = xs + (size_t)(q / nruns) * xpad + (q % nruns) * kRunPad;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 32; ++k) s += p[k];
        rs[q] = s;
    }
    __syncthreads();

    const uint32_t steps_per_row = (bpr + 7u) / 8u;
    const uint32_t nwaves = gridDim.x * 4u, gw = blockIdx.x * 4u + wave;
    const uint32_t r = lane & 7u;
    for (uint32_t row = gw; row < rows; row += nwaves) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.f;
        for (uint32_t st = 0; st < steps_per_row; ++st) {
            const uint32_t blk = st * 8u + (lane >> 3);
            if (blk < bpr) {
                const size_t b = (size_t)row * bpr + blk;
                Run R;
                if (uniform_fmt >= 0) {
                    R.cb = payload + uniform_base + b * uniform_stride;
                    R.cb_bytes = uniform_cb; R.idx_bytes = uniform_idx; R.fmt = (uint32_t)uniform_fmt;
                } else {
                    const DevBlock d = blocks[b];
                    R.cb = payload + (size_t)d.off16 * 16;
                    R.cb_bytes = d.cb_bytes; R.idx_bytes = d.idx_bytes; R.fmt = d.fmt;
                }
                R.r = r;
                const uint32_t run = blk * 8u + r;
                float w[32], mean = 0.f;
                if (decode_run(R, T, L, w, &mean)) {
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
                        acc[m] += a0 + a1;
                    }
                } else {
#pragma unroll
                    for (int m = 0; m < MB; ++m) acc[m] = __fmaf_rn(mean, rs[(size_t)m * nruns + run], acc[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float v = acc[m];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0 && m0 + m < M) y[(size_t)(m0 + m) * rows + row] = v;
        }
    }
}

template <int MB>
int launch_runs(const oilhip_weights& w, const DecodeTables* T, const float* d_x, float* d_y, int m0, int M, hipStream_t s) {
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemv_runs_kernel<MB>;
    const size_t lds = (size_t)MB * ((w.cols >> 5) * kRunPad + (w.cols >> 5)) * 4 + 532 * 4;
    if (lds > 160 * 1024) return 1;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
    uint32_t per_cu = (uint32_t)((160 * 1024) / lds);                 // workgroups a CU can hold: small loads need many waves in flight
    if (per_cu > 3) per_cu = 3;                                       // register budget: 3 wavefronts per SIMD
    uint32_t grid = (uint32_t)device_cu_count() * per_cu;
    const uint32_t need = ((uint32_t)w.rows + 3u) / 4u;
    if (grid > need) grid = need;
    const bool uni = w.uniform_fmt >= 0 && w.uniform_stride > 0;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, w.d_payload, w.d_blocks, T, d_x, d_y, (uint32_t)w.rows,
                       (uint32_t)w.cols, m0, M, uni ? w.uniform_fmt : -1, w.uniform_stride, w.uniform_cb, w.uniform_idx, w.uniform_base);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace

// Returns 1 when the shape is outside what this kernel covers (the caller falls back).
int launch_gemv_runs(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    if (!w.nominal || (w.cols & 255u) || w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull || w.rows == 0) return 1;
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    if ((size_t)((w.cols >> 5) * (kRunPad + 1)) * 4 + 532 * 4 > 160 * 1024) return 1;
    int m0 = 0;
    while (m0 < M) {
        const int left = M - m0;
        const size_t per = (size_t)((w.cols >> 5) * (kRunPad + 1)) * 4;
        int rc;
        if (left >= 4 && 4 * per + 532 * 4 <= 160 * 1024) { rc = launch_runs<4>(w, T, d_x, d_y, m0, M, s); m0 += 4; }
        else if (left >= 2 && 2 * per + 532 * 4 <= 160 * 1024) { rc = launch_runs<2>(w, T, d_x, d_y, m0, M, s); m0 += 2; }
        else { rc = launch_runs<1>(w, T, d_x, d_y, m0, M, s); m0 += 1; }
        if (rc) return rc;
    }
    return OILHIP_OK;
}

}  // namespace oilhip
