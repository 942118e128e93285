// tl_kernels.hip -- oil::kernel::tl1_gemm / tl2_gemm (include/oil/kernel.h:11-18, src/kernel_tl.cpp:32-90,124-184):
// activations [N][K] quantized per row to int8 with scale 127 / max|a|, one packed row of K two-bit ternary codes
// (0 -> -1, 1 -> 0, else +1; four per byte, low bits first) per (m, n) pair,
// out[m*N+n] = (sum of int8 x ternary products) / scale[n].  TL1 adds the products in pairs and stores every pair
// sum as int8 (clamped) first, its lookup table's element type; TL2 adds them as they are.  Integer work: results
// are the reference's bit for bit.
#include "common.h"

namespace oilhip {
namespace {

// one workgroup per activation row: scale and int8 codes (src/kernel_tl.cpp:39-50)
__global__ void __launch_bounds__(256)
tl_quantize_kernel(const float* __restrict__ a, int K, int8_t* __restrict__ q, float* __restrict__ scales) {
    __shared__ float part[4];
    const float* row = a + (size_t)blockIdx.x * K;
    float mx = 0.f;
    for (int k = threadIdx.x; k < K; k += 256) mx = fmaxf(mx, fabsf(row[k]));
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    if (mx < 1e-10f) mx = 1e-10f;
    const float sc = 127.0f / mx;
    if (threadIdx.x == 0) scales[blockIdx.x] = sc;
    for (int k = threadIdx.x; k < K; k += 256) q[(size_t)blockIdx.x * K + k] = (int8_t)roundf(row[k] * sc);
}

__device__ inline int ternary(uint32_t byte, int j) {
    const uint32_t c = (byte >> (2 * j)) & 3u;
    return c == 0 ? -1 : (c == 1 ? 0 : 1);
}

// a wavefront per output element; a lane takes whole bytes (four weights, two pairs), so no pair straddles lanes
template <int KIND>
__global__ void __launch_bounds__(256)
tl_gemm_kernel(const uint8_t* __restrict__ w, const int8_t* __restrict__ q, const float* __restrict__ scales,
               float* __restrict__ out, int64_t outputs, int N, int K, int row_bytes) {
    const int64_t o = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (o >= outputs) return;
    const int lane = threadIdx.x & 63;
    const int n = (int)(o % N);
    const uint8_t* wr = w + (size_t)o * row_bytes;
    const int8_t* ar = q + (size_t)n * K;
    long long total = 0;
    for (int b = lane; b * 4 < K; b += 64) {
        const uint32_t byte = wr[b];
        const int k0 = b * 4;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = k0 + 2 * h;
            if (k >= K) break;
            int sum = (int)ar[k] * ternary(byte, 2 * h);
            if (k + 1 < K) {
                sum += (int)ar[k + 1] * ternary(byte, 2 * h + 1);
                if (KIND == 1) sum = min(127, max(-128, sum));
            }
            total += sum;
        }
    }
    for (int s = 32; s > 0; s >>= 1) total += __shfl_xor(total, s, 64);
    if (lane == 0) out[o] = (KIND == 1 ? (float)(int)total : (float)total) / scales[n];
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" int oilhip_tl_gemm(int kind, const uint8_t* d_w, const float* d_act, float* d_out, int M, int N, int K, void* stream) {
    if (kind != 1 && kind != 2) return fail(OILHIP_E_ARG, "tl_gemm: kind must be 1 (TL1) or 2 (TL2)");
    if (M < 0 || N < 0 || K < 0) return fail(OILHIP_E_ARG, "tl_gemm: negative size");
    if (M == 0 || N == 0) return OILHIP_OK;
    // a TL2 triple that straddles the end of a row makes the reference read activations past that row
    if (kind == 2 && K % 3 != 0) return fail(OILHIP_E_ARG, "tl_gemm: TL2 needs K to be a multiple of 3");
    if (!d_out || (K > 0 && (!d_w || !d_act))) return fail(OILHIP_E_ARG, "tl_gemm: null pointer");
    auto s = static_cast<hipStream_t>(stream);
    const size_t qbytes = ((size_t)N * (size_t)K + 255) & ~(size_t)255;
    void* ws = nullptr;
    if (int rc = stream_scratch(s, kScratchTl, qbytes + sizeof(float) * (size_t)N, &ws)) return rc;
    int8_t* q = static_cast<int8_t*>(ws);
    float* scales = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + qbytes);
    hipLaunchKernelGGL(tl_quantize_kernel, dim3((unsigned)N), dim3(256), 0, s, d_act, K, q, scales);
    const int64_t outputs = (int64_t)M * N;
    if ((outputs + 3) / 4 > 0x7fffffffLL) return fail(OILHIP_E_ARG, "tl_gemm: too many outputs");
    const int row_bytes = kind == 1 ? (K + 3) / 4 : ((K + 11) / 12) * 3;
    const unsigned wgs = (unsigned)((outputs + 3) / 4);
    if (kind == 1)
        hipLaunchKernelGGL(tl_gemm_kernel<1>, dim3(wgs), dim3(256), 0, s, d_w, q, scales, d_out, outputs, N, K, row_bytes);
    else
        hipLaunchKernelGGL(tl_gemm_kernel<2>, dim3(wgs), dim3(256), 0, s, d_w, q, scales, d_out, outputs, N, K, row_bytes);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}
