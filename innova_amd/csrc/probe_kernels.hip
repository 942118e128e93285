// probe_kernels.hip -- a read-only streaming kernel with the decode GEMVs' load pattern (16 bytes per lane, a KB per
// wavefront and load, nothing but an XOR done with the data), so that the rate a pure reader reaches on the device at
// hand is a measured number beside the HBM peak the roofline fractions are quoted against.  No reference counterpart.
//
// Built into liboilhip_probe.so, a measurement tool beside the product library (bench.py loads it; nothing in
// liboilhip.so or its header refers to it).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace oilhip {
namespace {

thread_local std::string g_probe_error;
int fail(int code, const char* msg) { g_probe_error = msg; return code; }
constexpr int OILHIP_OK = 0, OILHIP_E_ARG = -1, OILHIP_E_DEVICE = -3;
#define OILHIP_HIP(call)                                                                              \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) { g_probe_error = std::string(#call) + ": " + hipGetErrorString(e_); return OILHIP_E_DEVICE; } \
    } while (0)

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// U loads in flight per wavefront.  PAT 0: each wavefront streams its own contiguous share (as the GEMVs' row groups
// do); PAT 1: wavefronts interleaved KB by KB; PAT 2: the multi-token GEMV's pattern over rows of 2 KB: a workgroup of
// 8 wavefronts walks groups of 16 rows, wavefront w reads blocks 2w and 2w+1 of each row with four loads whose lane
// 16*kq + i fetches 16 bytes of row i (64 contiguous bytes per row and load).  NT: loads marked non-temporal
// (streaming, no reuse expected).
template <int U, bool NT, int PAT>
__global__ void __launch_bounds__(1024)
read_probe_kernel(const uint8_t* __restrict__ base, uint64_t bytes, uint32_t* __restrict__ sink) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, wpb = blockDim.x >> 6;
    const uint64_t nw = (uint64_t)gridDim.x * wpb, gw = (uint64_t)blockIdx.x * wpb + wave;
    const uint64_t kbs = bytes >> 10;
    uint64_t k0, k1, step;
    if (PAT == 0) { k0 = kbs * gw / nw; k1 = kbs * (gw + 1) / nw; step = 1; }
    else { k0 = gw; k1 = kbs; step = nw; }
    uint32_t acc = 0;
    if (PAT == 2) {
        constexpr int UG = U >= 4 ? U / 4 : 1;                     // groups of 16 rows in flight
        const uint64_t ng = bytes >> 15, g0 = ng * blockIdx.x / gridDim.x, g1 = ng * (blockIdx.x + 1) / gridDim.x;
        for (uint64_t g = g0; g < g1; g += UG) {
            u32x4 v[UG * 4];
#pragma unroll
            for (int u = 0; u < UG * 4; ++u) {
                const uint64_t gg = g + u / 4 < g1 ? g + u / 4 : g0;
                const u32x4* p = reinterpret_cast<const u32x4*>(base + gg * 32768ull + (lane & 15u) * 2048u +
                                                                (2u * (wave & 7u) + ((u >> 1) & 1)) * 128u + (u & 1) * 64u + (lane >> 4) * 16u);
                v[u] = NT ? __builtin_nontemporal_load(p) : *p;
            }
#pragma unroll
            for (int u = 0; u < UG * 4; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
        }
        if (acc == 0x9e3779b9u) sink[gw] = acc;
        return;
    }
    for (uint64_t k = k0; k < k1; k += step * U) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t kk = k + (uint64_t)u * step;
            const u32x4* p = reinterpret_cast<const u32x4*>(base + (kk < k1 ? kk : k0) * 1024ull + lane * 16u);
            v[u] = NT ? __builtin_nontemporal_load(p) : *p;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) sink[gw] = acc;       // keeps the loads alive; practically never taken
}

template <int U, bool NT>
void launch_pat(int pattern, dim3 g, dim3 b, hipStream_t s, const uint8_t* p, uint64_t bytes, uint32_t* sink) {
    if (pattern == 0) hipLaunchKernelGGL((read_probe_kernel<U, NT, 0>), g, b, 0, s, p, bytes, sink);
    else if (pattern == 2) hipLaunchKernelGGL((read_probe_kernel<U, NT, 2>), g, b, 0, s, p, bytes, sink);
    else hipLaunchKernelGGL((read_probe_kernel<U, NT, 1>), g, b, 0, s, p, bytes, sink);
}
template <int U>
void launch_nt(int streaming, int pattern, dim3 g, dim3 b, hipStream_t s, const uint8_t* p, uint64_t bytes, uint32_t* sink) {
    if (streaming) launch_pat<U, true>(pattern, g, b, s, p, bytes, sink);
    else launch_pat<U, false>(pattern, g, b, s, p, bytes, sink);
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" const char* oilprobe_last_error() { return g_probe_error.c_str(); }

// bytes are read once by workgroups x threads / 64 wavefronts, each with in_flight (1, 2, 4, 8) loads outstanding;
// streaming != 0 marks the loads non-temporal; pattern 0 gives each wavefront a contiguous share, 1 interleaves them
// KB by KB, 2 is the multi-token GEMV's pattern (512 threads, 4 or 8 loads in flight: a load fetches 64 bytes of each
// of 16 rows of 2 KB).  d_sink needs workgroups x threads / 64 words (practically never written).  0 = ok.
extern "C" int oilprobe_read(const void* d_buf, uint64_t bytes, int in_flight, int streaming, int pattern,
                                 int workgroups, int threads, uint32_t* d_sink, void* stream) {
    if (!d_buf || !d_sink) return fail(OILHIP_E_ARG, "read_probe: null pointer");
    if (bytes < 1024 || ((uintptr_t)d_buf & 15u)) return fail(OILHIP_E_ARG, "read_probe: needs at least 1 KB, 16-byte aligned");
    if (in_flight != 1 && in_flight != 2 && in_flight != 4 && in_flight != 8)
        return fail(OILHIP_E_ARG, "read_probe: loads in flight must be 1, 2, 4 or 8");
    if (threads < 64 || threads > 1024 || threads % 64 != 0 || workgroups < 1 || workgroups > 65536)
        return fail(OILHIP_E_ARG, "read_probe: threads must be a multiple of 64 up to 1024, workgroups 1..65536");
    if (pattern < 0 || pattern > 2) return fail(OILHIP_E_ARG, "read_probe: pattern must be 0 (contiguous shares), 1 (interleaved) or 2 (16 rows of 2 KB per load)");
    if (pattern == 2 && (threads != 512 || in_flight < 4 || bytes < 32768 * (uint64_t)workgroups))
        return fail(OILHIP_E_ARG, "read_probe: pattern 2 needs 512 threads, 4 or 8 loads in flight and at least 32 KB per workgroup");
    auto s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)workgroups), b((unsigned)threads);
    const uint8_t* p = static_cast<const uint8_t*>(d_buf);
    switch (in_flight) {
        case 1: launch_nt<1>(streaming, pattern, g, b, s, p, bytes, d_sink); break;
        case 2: launch_nt<2>(streaming, pattern, g, b, s, p, bytes, d_sink); break;
        case 4: launch_nt<4>(streaming, pattern, g, b, s, p, bytes, d_sink); break;
        default: launch_nt<8>(streaming, pattern, g, b, s, p, bytes, d_sink); break;
    }
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}
