// layer_ops.hip -- the pieces of a decode step around the quantized matmuls, as Qwen35Engine runs them
// (src/adapters/tools/qwen35_engine.cpp): rmsnorm (:39-44), mlp_step (:611-621) and the embedding row
// lookup of append_token (:756-760).
#include <vector>

#include "common.h"

namespace oilhip {
int launch_gemv_oil4_swiglu(const oilhip_weights& w, const float* d_h, float* d_y, hipStream_t s);
int launch_gemv_oil4_rmsnorm(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, hipStream_t s);
int launch_gemv_seg_swiglu(const oilhip_weights& w, const float* d_h, float* d_y, hipStream_t s);
int launch_gemv_seg_rmsnorm(const oilhip_weights& w, const float* d_x, const float* d_xw, float* d_y, hipStream_t s);

namespace {

// out = x * r * (1 + w), r = 1 / sqrt(sum(x^2) / n + 1e-6); one workgroup per row.  Rows of up to 16384 floats
// (n % 4 == 0) are held in registers between the two passes: one round of loads, all in flight together.
__global__ void __launch_bounds__(1024)
rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, int n, float* __restrict__ out) {
    __shared__ float part[16];
    const float* xr = x + (size_t)blockIdx.x * n;
    float* orow = out + (size_t)blockIdx.x * n;
    const uint32_t tid = threadIdx.x;
    const bool in_regs = (n & 3) == 0 && n <= 16384;
    float4 v[4], g[4];
    float s = 0.f;
    if (in_regs) {
        const uint32_t n4 = (uint32_t)n >> 2;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = tid + u * 1024u;
            v[u] = i < n4 ? reinterpret_cast<const float4*>(xr)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            g[u] = i < n4 ? reinterpret_cast<const float4*>(w)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            s = __fmaf_rn(v[u].w, v[u].w, __fmaf_rn(v[u].z, v[u].z, __fmaf_rn(v[u].y, v[u].y, __fmaf_rn(v[u].x, v[u].x, s))));
    } else {
        for (int i = tid; i < n; i += 1024) s = __fmaf_rn(xr[i], xr[i], s);
    }
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if ((tid & 63) == 0) part[tid >> 6] = s;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) tot += part[k];
    const float r = 1.0f / sqrtf(tot / (float)n + 1e-6f);
    if (in_regs) {
        const uint32_t n4 = (uint32_t)n >> 2;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = tid + u * 1024u;
            if (i < n4)
                reinterpret_cast<float4*>(orow)[i] = make_float4(v[u].x * r * (1.0f + g[u].x), v[u].y * r * (1.0f + g[u].y),
                                                                 v[u].z * r * (1.0f + g[u].z), v[u].w * r * (1.0f + g[u].w));
        }
    } else {
        for (int i = tid; i < n; i += 1024) orow[i] = xr[i] * r * (1.0f + w[i]);
    }
}

// h[m][k] = siluf(g[m][k]) * g[m][F + k] with siluf(v) = v * (1 / (1 + exp(-v)))  (:31,37,617)
__global__ void __launch_bounds__(256)
swiglu_rows_kernel(const float* __restrict__ g, float* __restrict__ h, uint32_t F, uint32_t M) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)F * M; i += (size_t)gridDim.x * 256) {
        const size_t m = i / F, k = i % F;
        const float v = g[m * 2 * F + k];
        h[i] = (v * (1.0f / (1.0f + expf(-v)))) * g[m * 2 * F + F + k];
    }
}

// decode_block over the 256-weight blocks of the rows ids[i] (:17-28,756-760)
__global__ void __launch_bounds__(256)
embed_rows_kernel(const uint8_t* __restrict__ payload, const DevBlock* __restrict__ blocks, const DecodeTables* __restrict__ T,
                  const int32_t* __restrict__ ids, uint32_t bpr, uint32_t vocab, float* __restrict__ out) {
    const int32_t id = ids[blockIdx.y];
    float* o = out + ((size_t)blockIdx.y * bpr + blockIdx.x) * 256;
    if (id < 0 || (uint32_t)id >= vocab) { o[threadIdx.x] = 0.0f; return; }
    const DevBlock d = blocks[(size_t)id * bpr + blockIdx.x];
    const uint8_t* cb = payload + (size_t)d.off16 * 16;
    o[threadIdx.x] = decode_weight(d.fmt, cb, d.cb_bytes, cb + d.cb_bytes, d.idx_bytes, d.nw, threadIdx.x, T);
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" {

int oilhip_rmsnorm_f32(const float* d_x, const float* d_w, int n, int rows, float* d_out, void* stream) {
    if (n <= 0 || rows < 0) return fail(OILHIP_E_ARG, "rmsnorm: bad sizes");
    if (rows == 0) return OILHIP_OK;
    if (!d_x || !d_w || !d_out) return fail(OILHIP_E_ARG, "rmsnorm: null argument");
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((uint32_t)rows), dim3(1024), 0, (hipStream_t)stream, d_x, d_w, n, d_out);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_gemv_rmsnorm_f32(const oilhip_weights* w, const float* d_x, const float* d_normw, float* d_y, int M, float* d_xn,
                            void* stream) {
    if (!w || !d_x || !d_normw || !d_y || M <= 0) return fail(OILHIP_E_ARG, "gemv_rmsnorm: bad arguments");
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    if (M == 1 && plain_oil4(*w)) {
        const int rc = launch_gemv_oil4_rmsnorm(*w, d_x, d_normw, d_y, (hipStream_t)stream);   // the norm rides on the staging of x
        if (rc <= 0) return rc;
    }
    if (M == 1 && w->seg.nstreams) {
        const int rc = launch_gemv_seg_rmsnorm(*w, d_x, d_normw, d_y, (hipStream_t)stream);    // likewise for window-stream tensors
        if (rc <= 0) return rc;
    }
    if (!d_xn) return fail(OILHIP_E_ARG, "gemv_rmsnorm: this shape needs the d_xn workspace");
    if (int rc = oilhip_rmsnorm_f32(d_x, d_normw, (int)w->cols, M, d_xn, stream)) return rc;
    return oilhip_gemv_f32(w, d_xn, d_y, M, stream);
}

int oilhip_mlp_step_f32(const oilhip_weights* gate_up, const oilhip_weights* down, const float* d_x, const float* d_normw,
                        float* d_y, int M, float* d_scratch, void* stream) {
    if (!gate_up || !down || !d_x || !d_y || !d_scratch || M <= 0) return fail(OILHIP_E_ARG, "mlp_step: bad arguments");
    const uint64_t F = down->cols;
    if (gate_up->rows != 2 * F || gate_up->cols != down->rows)
        return fail(OILHIP_E_ARG, "mlp_step: gate_up must be 2F x D (gate rows first) and down D x F");
    if (int rc = check_matmul_shape(gate_up, d_x, d_y, M)) return rc;
    if (int rc = check_matmul_shape(down, d_x, d_y, M)) return rc;
    hipStream_t s = (hipStream_t)stream;
    float* h2 = d_scratch;                                   // [M][2F]
    float* h = d_scratch + (size_t)M * 2 * F;                // [M][F]
    float* xn = h + (size_t)M * F;                           // [M][D], only with d_normw
    if (int rc = d_normw ? oilhip_gemv_rmsnorm_f32(gate_up, d_x, d_normw, h2, M, xn, stream)
                         : oilhip_gemv_f32(gate_up, d_x, h2, M, stream)) return rc;
    if (M == 1 && plain_oil4(*down)) {
        const int rc = launch_gemv_oil4_swiglu(*down, h2, d_y, s);      // SwiGLU formed while the activations are staged
        if (rc <= 0) return rc;
    }
    if (M == 1 && down->seg.nstreams) {
        const int rc = launch_gemv_seg_swiglu(*down, h2, d_y, s);
        if (rc <= 0) return rc;
    }
    const size_t n = (size_t)F * (size_t)M;
    hipLaunchKernelGGL(swiglu_rows_kernel, dim3((uint32_t)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096)), dim3(256), 0, s,
                       h2, h, (uint32_t)F, (uint32_t)M);
    OILHIP_HIP(hipGetLastError());
    return oilhip_gemv_f32(down, h, d_y, M, stream);
}

int oilhip_embed_rows_f32(const oilhip_weights* w, const int32_t* d_ids, int n, float* d_out, void* stream) {
    if (!w || n < 0) return fail(OILHIP_E_ARG, "embed_rows: bad arguments");
    if (n == 0) return OILHIP_OK;
    if (!d_ids || !d_out) return fail(OILHIP_E_ARG, "embed_rows: null argument");
    if (!w->all_full || (w->cols & 255) || w->cols == 0) return fail(OILHIP_E_ARG, "embed_rows: rows must be whole 256-weight blocks");
    if (n > 65535) return fail(OILHIP_E_ARG, "embed_rows: at most 65535 rows per call");
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    hipLaunchKernelGGL(embed_rows_kernel, dim3((uint32_t)(w->cols >> 8), (uint32_t)n), dim3(256), 0, (hipStream_t)stream,
                       w->d_payload, w->d_blocks, T, d_ids, (uint32_t)(w->cols >> 8), (uint32_t)w->rows, d_out);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // extern "C"
