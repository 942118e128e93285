// dense_ops.hip -- the dense FP32 operations of backend::ComputeBackend (include/oil/backend.h:49-80) on device
// pointers, so that a gfx950 backend object can sit behind the reference's factory.  Semantics follow the CPU
// bodies in src/math.cpp: gemv :50-70, gemm :72-95, relu/gelu/silu :97-126, layer_norm :146-178, rms_norm :180-203,
// softmax :205-247, add/mul/scale :249-283.  These are plain bandwidth- or FMA-bound kernels beside the quantized
// path, not part of it.
#include "common.h"

namespace oilhip {
namespace {

constexpr int kTile = 64;     // C tile edge of the GEMM
constexpr int kStep = 16;     // K step staged through LDS

// C = alpha * A[M][K] . B[K][N] + beta * C; a 64x64 tile per workgroup of 256 threads, 4x4 outputs per thread.
__global__ void __launch_bounds__(256)
dense_gemm_kernel(float alpha, const float* __restrict__ A, const float* __restrict__ B, float beta,
                  float* __restrict__ C, int64_t M, int64_t N, int64_t K) {
    __shared__ float sa[kStep][kTile + 4];   // A tile, transposed: [k][row]
    __shared__ float sb[kStep][kTile + 4];   // B tile: [k][col]
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.y * kTile, col0 = (int64_t)blockIdx.x * kTile;
    const int tr = (tid >> 4) * 4, tc = (tid & 15) * 4;
    float acc[4][4] = {};
    for (int64_t k0 = 0; k0 < K; k0 += kStep) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = tid + u * 256;                 // 1024 elements per tile
            const int ar = e >> 4, ak = e & 15;          // A: 64 rows x 16 k
            const int64_t gr = row0 + ar, gk = k0 + ak;
            sa[ak][ar] = gr < M && gk < K ? A[gr * K + gk] : 0.f;
            const int bk = e >> 6, bc = e & 63;          // B: 16 k x 64 cols
            const int64_t gk2 = k0 + bk, gc = col0 + bc;
            sb[bk][bc] = gk2 < K && gc < N ? B[gk2 * N + gc] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kStep; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = sa[k][tr + i]; b[i] = sb[k][tc + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __fmaf_rn(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + tr + i, c = col0 + tc + j;
            if (r < M && c < N) {
                // beta == 0 leaves C's old contents unread, like BLAS; the CPU body multiplies them in, which only
                // differs when C holds NaN or infinity
                const float old = beta != 0.f ? C[r * N + c] : 0.f;
                C[r * N + c] = alpha * acc[i][j] + beta * old;
            }
        }
}

// y = alpha * A[M][N] . x + beta * y; a wavefront per row.
__global__ void __launch_bounds__(256)
dense_gemv_kernel(float alpha, const float* __restrict__ A, const float* __restrict__ x, float beta,
                  float* __restrict__ y, int64_t M, int64_t N) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int lane = threadIdx.x & 63;
    const float* a = A + row * N;
    float s = 0.f;
    for (int64_t j = lane; j < N; j += 64) s = __fmaf_rn(a[j], x[j], s);
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (lane == 0) y[row] = alpha * s + (beta != 0.f ? beta * y[row] : 0.f);
}

__device__ inline double wave_sum(double v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ inline double block_sum(double v, double* part) {   // 256 threads
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    return part[0] + part[1] + part[2] + part[3];
}

// One workgroup per row; sums in double like the CPU bodies.  MODE 0: layer_norm, 1: rms_norm.
template <int MODE>
__global__ void __launch_bounds__(256)
dense_norm_kernel(const float* __restrict__ x, const float* __restrict__ gamma, const float* __restrict__ beta,
                  float eps, float* __restrict__ y, int64_t n) {
    __shared__ double part[4];
    const float* row = x + (int64_t)blockIdx.x * n;
    float* out = y + (int64_t)blockIdx.x * n;
    if (MODE == 0) {
        double s = 0.0;
        for (int64_t j = threadIdx.x; j < n; j += 256) s += (double)row[j];
        const double mu = block_sum(s, part) / (double)n;
        double v = 0.0;
        for (int64_t j = threadIdx.x; j < n; j += 256) { const double d = (double)row[j] - mu; v += d * d; }
        const double inv = 1.0 / sqrt(block_sum(v, part) / (double)n + (double)eps);
        for (int64_t j = threadIdx.x; j < n; j += 256)
            out[j] = (float)(((double)row[j] - mu) * inv) * gamma[j] + beta[j];
    } else {
        double s = 0.0;
        for (int64_t j = threadIdx.x; j < n; j += 256) s += (double)row[j] * (double)row[j];
        const double inv = 1.0 / sqrt(block_sum(s, part) / (double)n + (double)eps);
        for (int64_t j = threadIdx.x; j < n; j += 256) out[j] = (float)((double)row[j] * inv) * gamma[j];
    }
}

// softmax over `dim` entries `inner` apart; a wavefront per (outer, inner) line.
__global__ void __launch_bounds__(256)
dense_softmax_kernel(const float* __restrict__ x, float* __restrict__ y, int64_t lines, int64_t dim, int64_t inner) {
    const int64_t line = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (line >= lines) return;
    const int lane = threadIdx.x & 63;
    const int64_t base = (line / inner) * dim * inner + line % inner;
    float mx = -INFINITY;
    for (int64_t d = lane; d < dim; d += 64) mx = fmaxf(mx, x[base + d * inner]);
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    double s = 0.0;
    for (int64_t d = lane; d < dim; d += 64) s += (double)expf(x[base + d * inner] - mx);
    const double inv = 1.0 / wave_sum(s);
    for (int64_t d = lane; d < dim; d += 64)
        y[base + d * inner] = (float)((double)expf(x[base + d * inner] - mx) * inv);
}

// elementwise: op 0 relu, 1 gelu (erf form), 2 silu, 3 a + b, 4 a * b, 5 s * a, 6 fill with s
__global__ void __launch_bounds__(256)
dense_map_kernel(int op, const float* __restrict__ a, const float* __restrict__ b, float s, float* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        float v;
        switch (op) {
            case 0: v = a[i] > 0.f ? a[i] : 0.f; break;
            case 1: v = 0.5f * a[i] * (1.0f + erff(a[i] * 0.7071067811865475f)); break;
            case 2: v = a[i] / (1.0f + expf(-a[i])); break;
            case 3: v = a[i] + b[i]; break;
            case 4: v = a[i] * b[i]; break;
            case 5: v = s * a[i]; break;
            default: v = s; break;
        }
        y[i] = v;
    }
}

int done(hipStream_t) {
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" int oilhip_dense_gemm_f32(float alpha, const float* d_a, const float* d_b, float beta, float* d_c,
                                     int64_t M, int64_t N, int64_t K, void* stream) {
    if (M < 0 || N < 0 || K < 0) return fail(OILHIP_E_ARG, "dense_gemm: negative size");
    if (M == 0 || N == 0) return OILHIP_OK;
    if (!d_c || (K > 0 && (!d_a || !d_b))) return fail(OILHIP_E_ARG, "dense_gemm: null pointer");
    const int64_t gx = (N + kTile - 1) / kTile, gy = (M + kTile - 1) / kTile;
    if (gx > 0x7fffffffLL || gy > 65535) return fail(OILHIP_E_ARG, "dense_gemm: shape beyond the launch grid");
    auto s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(dense_gemm_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, alpha, d_a, d_b, beta, d_c, M, N, K);
    return done(s);
}

extern "C" int oilhip_dense_gemv_f32(float alpha, const float* d_a, const float* d_x, float beta, float* d_y,
                                     int64_t M, int64_t N, void* stream) {
    if (M < 0 || N < 0) return fail(OILHIP_E_ARG, "dense_gemv: negative size");
    if (M == 0) return OILHIP_OK;
    if (!d_y || (N > 0 && (!d_a || !d_x))) return fail(OILHIP_E_ARG, "dense_gemv: null pointer");
    if ((M + 3) / 4 > 0x7fffffffLL) return fail(OILHIP_E_ARG, "dense_gemv: too many rows");
    auto s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(dense_gemv_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, s, alpha, d_a, d_x, beta, d_y, M, N);
    return done(s);
}

extern "C" int oilhip_dense_norm_f32(int kind, const float* d_x, const float* d_gamma, const float* d_beta, float eps,
                                     float* d_y, int64_t rows, int64_t n, void* stream) {
    if (kind != 0 && kind != 1) return fail(OILHIP_E_ARG, "dense_norm: kind must be 0 (layer_norm) or 1 (rms_norm)");
    if (rows < 0 || n < 0) return fail(OILHIP_E_ARG, "dense_norm: negative size");
    if (rows == 0 || n == 0) return OILHIP_OK;
    if (!d_x || !d_gamma || !d_y || (kind == 0 && !d_beta)) return fail(OILHIP_E_ARG, "dense_norm: null pointer");
    if (rows > 0x7fffffffLL) return fail(OILHIP_E_ARG, "dense_norm: too many rows");
    auto s = static_cast<hipStream_t>(stream);
    if (kind == 0)
        hipLaunchKernelGGL(dense_norm_kernel<0>, dim3((unsigned)rows), dim3(256), 0, s, d_x, d_gamma, d_beta, eps, d_y, n);
    else
        hipLaunchKernelGGL(dense_norm_kernel<1>, dim3((unsigned)rows), dim3(256), 0, s, d_x, d_gamma, d_beta, eps, d_y, n);
    return done(s);
}

extern "C" int oilhip_dense_softmax_f32(const float* d_x, float* d_y, int64_t outer, int64_t dim, int64_t inner, void* stream) {
    if (outer < 0 || dim < 0 || inner < 0) return fail(OILHIP_E_ARG, "dense_softmax: negative size");
    const int64_t lines = outer * inner;
    if (lines == 0 || dim == 0) return OILHIP_OK;
    if (!d_x || !d_y) return fail(OILHIP_E_ARG, "dense_softmax: null pointer");
    if ((lines + 3) / 4 > 0x7fffffffLL) return fail(OILHIP_E_ARG, "dense_softmax: too many lines");
    auto s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(dense_softmax_kernel, dim3((unsigned)((lines + 3) / 4)), dim3(256), 0, s, d_x, d_y, lines, dim, inner);
    return done(s);
}

extern "C" int oilhip_dense_map_f32(int op, const float* d_a, const float* d_b, float s_, float* d_y, int64_t n, void* stream) {
    if (op < 0 || op > 6) return fail(OILHIP_E_ARG, "dense_map: unknown operation");
    if (n < 0) return fail(OILHIP_E_ARG, "dense_map: negative size");
    if (n == 0) return OILHIP_OK;
    if (!d_y || (op != 6 && !d_a) || ((op == 3 || op == 4) && !d_b)) return fail(OILHIP_E_ARG, "dense_map: null pointer");
    auto s = static_cast<hipStream_t>(stream);
    const int64_t wgs = std::min<int64_t>((n + 255) / 256, 8192);
    hipLaunchKernelGGL(dense_map_kernel, dim3((unsigned)wgs), dim3(256), 0, s, op, d_a, d_b, s_, d_y, n);
    return done(s);
}
