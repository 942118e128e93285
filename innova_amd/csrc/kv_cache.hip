// kv_cache.hip -- the OIL4 KV cache of the reference (oil::OIL4KVCache, include/oil/kv_cache_oil4.h:26-83,
// src/kv_cache_oil4.cpp) held in HBM: 4-bit codes, two per byte (low nibble first), and 16 FP16 centroids per block of
// 32 / 64 / 128 consecutive values of a layer's [token][heads * dim] stream.
//
//   append    : every chunk (a token's values cut at block boundaries, :207-291) is quantized by one wavefront with
//               the reference's 16-level Lloyd-Max (:75-153) step for step -- same initial centroids, same 20
//               iterations over the sorted values, same sequential sums -- so codes and centroids are identical.
//   get_range : codes -> centroids -> FP32 [len][heads * dim] through the cache's own half decode
//               (CodebookOIL4::half_to_float, src/codebook.cpp:36-64, which is not IEEE for subnormals).
//
// A chunk's codes are packed from its own first byte, block * (block / 2) + offset / 2 (:246).  With an even number
// of values per token that makes element e of a layer nibble e & 1 of byte e / 2.  With an odd number a chunk that
// starts at an even offset and holds an odd count shares its last byte with the chunk behind it, and the later write
// wins (the earlier chunk's last code is lost, as in the reference); the kernels reproduce that by leaving the shared
// byte to the later chunk.
#include <algorithm>
#include <new>
#include <vector>

#include "common.h"

struct oilhip_kv {
    int device = 0;
    int layers = 0;
    int64_t max_seq = 0, heads = 0, dim = 0, block = 64, per_token = 0;
    int64_t idx_bytes = 0;          // per layer and side, (max_seq * per_token + 1) / 2
    int64_t nblocks = 0;            // per layer and side
    int64_t idx_stride = 0;         // idx_bytes rounded up to 256
    uint8_t* d_idx = nullptr;       // [layers][2 (K, V)][idx_stride]
    uint16_t* d_cb = nullptr;       // [layers][2][nblocks * 16]
    std::vector<int64_t> pos;       // tokens appended per layer (the reference's current_pos: counts dropped tokens too)
};

namespace oilhip {
namespace {

// CodebookOIL4::float_to_half (src/codebook.cpp:16-34): the mantissa is truncated, magnitudes below 2^-25 become zero.
__device__ __forceinline__ uint32_t kv_float_to_half(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e = (int)((u >> 23) & 0xFFu) - 112;
    uint32_t mant = u & 0x007FFFFFu;
    if (e <= 0) {
        if (e < -10) return sign;
        mant = (mant | 0x00800000u) >> (1 - e);
        return sign | (mant >> 13);
    }
    if (e >= 31) return sign | 0x7C00u | (mant ? 0x0200u : 0u);
    return sign | ((uint32_t)e << 10) | (mant >> 13);
}

// CodebookOIL4::half_to_float (src/codebook.cpp:36-64).  A subnormal half whose highest set mantissa bit is p gets the
// exponent field 113 - p, and of its normalised mantissa << 13 only the low 16 bits (the reference holds it in a
// uint16_t, :52).
__device__ __forceinline__ float kv_half_to_float(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t mant = h & 0x03FFu;
    uint32_t f;
    if (e == 0) {
        if (mant == 0) {
            f = sign;
        } else {
            const uint32_t p = 31u - (uint32_t)__clz((int)mant);
            f = sign | ((113u - p) << 23) | ((((mant << (10u - p)) & 0x03FFu) << 13) & 0xFFFFu);
        }
    } else if (e == 31) {
        f = sign | 0x7F800000u | (mant << 13);
    } else {
        f = sign | ((e + 112u) << 23) | (mant << 13);
    }
    return __uint_as_float(f);
}

__device__ __forceinline__ uint32_t kv_nearest(const float (&cen)[16], float x) {
    float best = fabsf(__fsub_rn(x, cen[0]));
    uint32_t bi = 0;
#pragma unroll
    for (int c = 1; c < 16; ++c) {
        const float d = fabsf(__fsub_rn(x, cen[c]));
        if (d < best) { best = d; bi = (uint32_t)c; }
    }
    return bi;
}

struct KvLds {
    float srt[128];
    float cen[16];
    uint8_t code[128];
};

// Minimum (the first of equal values: the sign of a zero minimum reaches a constant chunk's centroids) and maximum of
// the chunk, in every lane.
__device__ __forceinline__ void kv_min_max(float x0, float x1, uint32_t n, uint32_t lane, float& lo, float& hi) {
    lo = lane < n ? x0 : __builtin_inff();
    uint32_t lo_i = lane;
    if (lane + 64 < n && x1 < lo) { lo = x1; lo_i = lane + 64; }
    hi = lane < n ? x0 : -__builtin_inff();
    if (lane + 64 < n && x1 > hi) hi = x1;
    for (int o = 32; o > 0; o >>= 1) {
        const float ol = __shfl_xor(lo, o, 64);
        const uint32_t oi = (uint32_t)__shfl_xor((int)lo_i, o, 64);
        if (ol < lo || (ol == lo && oi < lo_i)) { lo = ol; lo_i = oi; }
        const float oh = __shfl_xor(hi, o, 64);
        if (oh > hi) hi = oh;
    }
}

// lloyd_max_16 (src/kv_cache_oil4.cpp:75-153) for n <= 128 values by one wavefront.  Leaves the n codes in L.code and
// the 16 centroids (FP32) in L.cen.
__device__ void kv_quantize_chunk(const float* __restrict__ src, uint32_t n, uint32_t lane, KvLds& L) {
    const float x0 = lane < n ? src[lane] : 0.f;
    const float x1 = lane + 64 < n ? src[lane + 64] : 0.f;
    // Ascending sort of the n values, padded with +inf: a bitonic network, in registers with one value per lane for
    // chunks of up to 64 values (both lanes of a pair evaluate the same comparison, so equal values are never
    // duplicated), over 128 LDS slots otherwise.  The sorted ends are the minimum and the maximum.
    float s0, s1, lo, hi;
    if (n <= 64) {
        s0 = lane < n ? x0 : __builtin_inff();
        s1 = __builtin_inff();
#pragma unroll
        for (uint32_t k = 2; k <= 64; k <<= 1) {
#pragma unroll
            for (uint32_t j = k >> 1; j > 0; j >>= 1) {
                const float other = __shfl_xor(s0, (int)j, 64);
                const bool keep_small = ((lane & j) == 0) == ((lane & k) == 0);
                const bool take = keep_small ? other < s0 : other > s0;
                s0 = take ? other : s0;
            }
        }
        lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s0), 0));
        hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s0), (int)n - 1));
    } else {
        kv_min_max(x0, x1, n, lane, lo, hi);
    }
    const float range = __fsub_rn(hi, lo);
    if (range < 1e-10f) {
        if (n <= 64) kv_min_max(x0, x1, n, lane, lo, hi);       // which of several equal zeros comes first
        if (lane < n) L.code[lane] = 8;
        if (lane + 64 < n) L.code[lane + 64] = 8;
        if (lane < 16) L.cen[lane] = lo;
        __syncthreads();
        return;
    }
    if (lane < 16) L.cen[lane] = __fadd_rn(lo, __fdiv_rn(__fmul_rn(range, (float)lane + 0.5f), 16.0f));
    if (n <= 64) {
        L.srt[lane] = s0;
        __syncthreads();
    } else {
        L.srt[lane] = x0;
        L.srt[lane + 64] = lane + 64 < n ? x1 : __builtin_inff();
        __syncthreads();
        for (uint32_t k = 2; k <= 128; k <<= 1) {
            for (uint32_t j = k >> 1; j > 0; j >>= 1) {
                const uint32_t i = ((lane & ~(j - 1)) << 1) | (lane & (j - 1));
                const uint32_t p = i | j;
                const bool up = (i & k) == 0;
                const float a = L.srt[i], b = L.srt[p];
                if ((a > b) == up) { L.srt[i] = b; L.srt[p] = a; }
                __syncthreads();
            }
        }
        s0 = L.srt[lane];
        s1 = L.srt[lane + 64];
    }
    float cen[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) cen[c] = L.cen[c];
    for (int it = 0; it < 20; ++it) {
        const uint32_t b0 = lane < n ? kv_nearest(cen, s0) : 16u;
        bool moved = false;
        // the cluster of the value to the left (wave_shr:1; lane 0 reads 0)
        const uint32_t prev = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)b0, 0x138, 0xF, 0xF, true);
        if (n <= 64 && __ballot(lane > 0 && b0 < prev) == 0) {
            // Cluster numbers do not fall along the sorted values (the usual case), so every cluster is one run of
            // lanes.  Each lane folds its run from the left, one neighbour step at a time: after step t the lanes at
            // depth <= t of their run hold 0 + x_first + ... + x_self in exactly the reference's order.  The last lane
            // of a run owns the cluster's sum and count.
            const uint64_t heads = __ballot(lane == 0 || b0 != prev);
            const uint32_t first = 63u - (uint32_t)__builtin_clzll(heads & (~0ull >> (63u - lane)));
            const uint32_t depth = lane - first;
            float fold = __fadd_rn(0.f, s0);
            for (uint32_t t = 1; __ballot(depth >= t) != 0; ++t) {
                const float left = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(fold), 0x138, 0xF, 0xF, true));
                const float next = __fadd_rn(left, s0);
                fold = depth >= t ? next : fold;
            }
            const bool tail = lane == 63 || ((heads >> ((lane + 1) & 63u)) & 1ull) != 0;
            if (tail && b0 < 16) {
                const float nv = __fdiv_rn(fold, (float)(depth + 1));
                moved = __float_as_uint(nv) != __float_as_uint(L.cen[b0]);
                L.cen[b0] = nv;
            }
        } else {
            // lane c < 16 collects the members of cluster c as bit masks over the sorted order and adds them up in that
            // order, as the reference's loop over the sorted values does (four LDS reads in flight per round)
            const uint32_t b1 = lane + 64 < n ? kv_nearest(cen, s1) : 16u;
            uint64_t m0 = 0, m1 = 0;
#pragma unroll
            for (uint32_t c = 0; c < 16; ++c) {
                const uint64_t w0 = __ballot(b0 == c);
                const uint64_t w1 = n > 64 ? __ballot(b1 == c) : 0ull;
                if (lane == c) { m0 = w0; m1 = w1; }
            }
            float sum = 0.f;
            const int cnt = __popcll(m0) + __popcll(m1);
            for (int half = 0; half < 2; ++half) {
                uint64_t m = half ? m1 : m0;
                const float* base = L.srt + 64 * half;
                while (m) {
                    uint32_t i[4];
                    bool h[4];
                    float val[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        h[u] = m != 0;
                        i[u] = h[u] ? (uint32_t)__builtin_ctzll(m) : 0u;
                        m &= m - 1;
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) val[u] = base[i[u]];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (h[u]) sum = __fadd_rn(sum, val[u]);
                }
            }
            if (lane < 16 && cnt > 0) {                                              // an empty cluster keeps its centroid
                const float nv = __fdiv_rn(sum, (float)cnt);
                moved = __float_as_uint(nv) != __float_as_uint(L.cen[lane]);
                L.cen[lane] = nv;
            }
        }
        const bool any_moved = __ballot(moved) != 0;
        __syncthreads();
        if (!any_moved) break;           // a fixed point: the remaining iterations would reproduce these centroids bit for bit
#pragma unroll
        for (int c = 0; c < 16; ++c) cen[c] = L.cen[c];
        __syncthreads();
    }
    if (lane < n) L.code[lane] = (uint8_t)kv_nearest(cen, x0);
    if (lane + 64 < n) L.code[lane + 64] = (uint8_t)kv_nearest(cen, x1);
    __syncthreads();
}

// One wavefront per (token, chunk of the token, K or V).  pos = tokens the layer held before this call, ntok = tokens
// of this call that fit.  K centroids are stored by the chunk that opens a block, or -- while the layer is empty, and
// for V always -- by the last chunk of the call that touches the block (:256-261, :277-279: later writes win).
__global__ void __launch_bounds__(64)
kv_append_kernel(uint8_t* __restrict__ k_idx, uint8_t* __restrict__ v_idx, uint16_t* __restrict__ k_cb,
                 uint16_t* __restrict__ v_cb, const float* __restrict__ k, const float* __restrict__ v, int64_t pos,
                 int64_t ntok, int64_t per_token, uint32_t block, uint32_t chunks_per_token, int64_t idx_bytes) {
    __shared__ KvLds L;
    const uint32_t lane = threadIdx.x;
    const int64_t s = blockIdx.x / chunks_per_token;
    const uint32_t c = blockIdx.x % chunks_per_token;
    const bool is_v = blockIdx.y != 0;
    const int64_t tok_lo = (pos + s) * per_token, tok_hi = tok_lo + per_token;
    const int64_t blk = tok_lo / block + c;
    const int64_t a = c == 0 ? tok_lo : blk * block;
    if (a >= tok_hi) return;
    const int64_t b = (blk + 1) * block < tok_hi ? (blk + 1) * block : tok_hi;
    const uint32_t n = (uint32_t)(b - a);
    const float* src = (is_v ? v : k) + (a - pos * per_token);
    kv_quantize_chunk(src, n, lane, L);
    const bool last_on_block = (b % block) == 0 || b == (pos + ntok) * per_token;
    const uint32_t off = (uint32_t)(a % block);
    const int64_t at = blk * (int64_t)(block >> 1) + (off >> 1);
    uint32_t nbytes = (n + 1) >> 1;
    if (!(off & 1u) && (n & 1u) && !last_on_block) --nbytes;        // that byte belongs to the next chunk of this call
    if (at + nbytes > idx_bytes) nbytes = at < idx_bytes ? (uint32_t)(idx_bytes - at) : 0u;   // :248-249
    uint8_t* idx = (is_v ? v_idx : k_idx) + at;
    if (lane < nbytes) idx[lane] = (uint8_t)(L.code[2 * lane] | (2 * lane + 1 < n ? L.code[2 * lane + 1] << 4 : 0));
    const bool store_cb = (is_v || pos == 0) ? last_on_block : (a % block) == 0;
    if (store_cb && lane < 16) (is_v ? v_cb : k_cb)[blk * 16 + lane] = (uint16_t)kv_float_to_half(L.cen[lane]);
}

// OIL4KVCache::quantize_block_oil4 over nblocks independent runs of n <= 128 values: one code per byte, 16 centroids.
__global__ void __launch_bounds__(64)
kv_quantize_blocks_kernel(const float* __restrict__ src, uint32_t n, uint8_t* __restrict__ codes, uint16_t* __restrict__ cb) {
    __shared__ KvLds L;
    const uint32_t lane = threadIdx.x;
    const size_t at = (size_t)blockIdx.x * n;
    kv_quantize_chunk(src + at, n, lane, L);
    if (lane < n) codes[at + lane] = L.code[lane];
    if (lane + 64 < n) codes[at + lane + 64] = L.code[lane + 64];
    if (lane < 16) cb[(size_t)blockIdx.x * 16 + lane] = (uint16_t)kv_float_to_half(L.cen[lane]);
}

// dequantize_block_oil4 (:155-161): dst[b][i] = half_to_float(cb[b][codes[b][i] & 15])
__global__ void __launch_bounds__(256)
kv_dequantize_blocks_kernel(const uint8_t* __restrict__ codes, const uint16_t* __restrict__ cb, float* __restrict__ dst,
                            uint32_t n, uint64_t total) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    dst[i] = kv_half_to_float(cb[(i / n) * 16 + (codes[i] & 15u)]);
}

// get_range for tokens whose value count is a multiple of 4 (value e is then nibble e & 1 of byte e / 2).  A workgroup decodes kTile consecutive elements of K
// (blockIdx.y = 0) or V (1): the centroids of the blocks under the tile go to LDS as FP32 once, then each thread
// turns 2 bytes of codes into one 16-byte store, four times.
constexpr uint32_t kTile = 4096;
__global__ void __launch_bounds__(256)
kv_get_range_kernel(const uint8_t* __restrict__ k_idx, const uint8_t* __restrict__ v_idx, const uint16_t* __restrict__ k_cb,
                    const uint16_t* __restrict__ v_cb, float* __restrict__ k_out, float* __restrict__ v_out, uint64_t first,
                    uint64_t count, uint32_t block_shift, uint64_t ncb) {
    __shared__ float cen[(kTile / 32 + 1) * 16];
    const uint8_t* idx = blockIdx.y ? v_idx : k_idx;
    const uint16_t* cb = blockIdx.y ? v_cb : k_cb;
    float* out = blockIdx.y ? v_out : k_out;
    const uint64_t j0 = (uint64_t)blockIdx.x * kTile;
    const uint64_t jn = count - j0 < kTile ? count - j0 : kTile;
    const uint64_t blk0 = (first + j0) >> block_shift;
    const uint32_t nent = (uint32_t)((((first + j0 + jn - 1) >> block_shift) - blk0 + 1) * 16);
    for (uint32_t i = threadIdx.x; i < nent; i += 256) {
        const uint64_t at = blk0 * 16 + i;
        cen[i] = at < ncb ? kv_half_to_float(cb[at]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t it = 0; it < kTile / 1024; ++it) {
        const uint64_t j = (uint64_t)it * 1024 + threadIdx.x * 4;
        if (j < jn) {
            const uint64_t e = first + j0 + j;
            const uint32_t codes = *reinterpret_cast<const uint16_t*>(idx + (e >> 1));
            const float* t = cen + (uint32_t)((e >> block_shift) - blk0) * 16;
            *reinterpret_cast<float4*>(out + j0 + j) =
                make_float4(t[codes & 15u], t[(codes >> 4) & 15u], t[(codes >> 8) & 15u], t[(codes >> 12) & 15u]);
        }
    }
}

// get_range, one value per thread, with the reference's chunk arithmetic (:318-334): the chunk of a value starts at
// the later of its token's first value and its block's first value, and its codes count from the chunk's own byte.
__global__ void __launch_bounds__(256)
kv_get_range_scalar_kernel(const uint8_t* __restrict__ k_idx, const uint8_t* __restrict__ v_idx,
                           const uint16_t* __restrict__ k_cb, const uint16_t* __restrict__ v_cb, float* __restrict__ k_out,
                           float* __restrict__ v_out, uint64_t first, uint64_t count, uint32_t block_shift, uint64_t per_token,
                           uint64_t idx_bytes) {
    const uint64_t j = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (j >= count) return;
    const uint64_t e = first + j;
    const uint64_t blk = e >> block_shift;
    const uint64_t tok_lo = e / per_token * per_token, blk_lo = blk << block_shift;
    const uint64_t a = tok_lo > blk_lo ? tok_lo : blk_lo;
    const uint64_t at = (blk << (block_shift - 1)) + ((a - blk_lo) >> 1) + ((e - a) >> 1);
    const uint8_t* idx = blockIdx.y ? v_idx : k_idx;
    const uint16_t* cb = blockIdx.y ? v_cb : k_cb;
    const uint32_t byte = at < idx_bytes ? idx[at] : 0u;                              // :322-325
    const uint32_t code = (byte >> (4 * (uint32_t)((e - a) & 1))) & 15u;
    (blockIdx.y ? v_out : k_out)[j] = kv_half_to_float(cb[blk * 16 + code]);
}

__global__ void __launch_bounds__(256) kv_zero_kernel(uint4* p, uint64_t n16) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256)
        p[i] = make_uint4(0, 0, 0, 0);
}

int kv_alloc(oilhip_kv* c) {
    const int64_t total = c->max_seq * c->per_token;
    c->idx_bytes = (total + 1) / 2;
    c->nblocks = (total + c->block - 1) / c->block;
    c->idx_stride = (c->idx_bytes + 255) / 256 * 256;
    const size_t ib = (size_t)c->layers * 2 * (size_t)c->idx_stride;
    const size_t cbb = (size_t)c->layers * 2 * (size_t)c->nblocks * 32;
    c->d_idx = nullptr;
    c->d_cb = nullptr;
    if (ib == 0) return OILHIP_OK;
    if (hipMalloc((void**)&c->d_idx, ib) != hipSuccess) return fail(OILHIP_E_NOMEM, "kv cache: hipMalloc of the code arrays failed");
    if (hipMalloc((void**)&c->d_cb, cbb) != hipSuccess) {
        (void)hipFree(c->d_idx);
        c->d_idx = nullptr;
        return fail(OILHIP_E_NOMEM, "kv cache: hipMalloc of the centroid arrays failed");
    }
    OILHIP_HIP(hipMemset(c->d_idx, 0, ib));
    OILHIP_HIP(hipMemset(c->d_cb, 0, cbb));
    return OILHIP_OK;
}

inline uint8_t* kv_idx(const oilhip_kv* c, int layer, int side) { return c->d_idx + ((size_t)layer * 2 + side) * (size_t)c->idx_stride; }
inline uint16_t* kv_cb(const oilhip_kv* c, int layer, int side) { return c->d_cb + ((size_t)layer * 2 + side) * (size_t)c->nblocks * 16; }

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" {

int oilhip_kv_create(int num_layers, int64_t max_seq_len, int64_t num_heads, int64_t head_dim, int64_t block_size,
                     oilhip_kv** out) {
    if (!out) return fail(OILHIP_E_ARG, "kv_create: out is null");
    *out = nullptr;
    if (num_layers < 0 || max_seq_len < 0 || num_heads < 0 || head_dim < 0) return fail(OILHIP_E_ARG, "kv_create: negative size");
    const int64_t per_token = num_heads * head_dim;
    if (per_token > 0 && max_seq_len > ((int64_t)1 << 40) / per_token) return fail(OILHIP_E_ARG, "kv_create: cache too large");
    oilhip_kv* c = new (std::nothrow) oilhip_kv;
    if (!c) return fail(OILHIP_E_NOMEM, "kv_create: out of host memory");
    if (hipGetDevice(&c->device) != hipSuccess) { delete c; return fail(OILHIP_E_NOGPU, "kv_create: no HIP device"); }
    c->layers = num_layers;
    c->max_seq = max_seq_len;
    c->heads = num_heads;
    c->dim = head_dim;
    c->per_token = per_token;
    c->block = (block_size == 32 || block_size == 64 || block_size == 128) ? block_size : 64;   // kv_cache_oil4.cpp:25-26
    c->pos.assign((size_t)num_layers, 0);
    const int rc = kv_alloc(c);
    if (rc != OILHIP_OK) { delete c; return rc; }
    *out = c;
    return OILHIP_OK;
}

int oilhip_kv_destroy(oilhip_kv* c) {
    if (!c) return OILHIP_OK;
    if (c->d_idx) (void)hipFree(c->d_idx);
    if (c->d_cb) (void)hipFree(c->d_cb);
    delete c;
    return OILHIP_OK;
}

int oilhip_kv_append(oilhip_kv* c, int layer, const float* d_k, const float* d_v, int64_t seq_len, void* stream) {
    if (!c) return fail(OILHIP_E_ARG, "kv_append: cache is null");
    if (layer < 0 || seq_len < 0) return fail(OILHIP_E_ARG, "kv_append: negative layer or length");
    if (layer >= c->layers) return OILHIP_OK;                                       // :209
    const int64_t pos = c->pos[(size_t)layer];
    int64_t ntok = c->max_seq - pos;                                               // tokens past max_seq_len are dropped (:224)
    if (ntok > seq_len) ntok = seq_len;
    if (ntok > 0 && c->per_token > 0) {
        if (!d_k || !d_v) return fail(OILHIP_E_ARG, "kv_append: null input");
        const uint32_t cpt = (uint32_t)((c->per_token + c->block - 1) / c->block + 1);
        if (ntok * (int64_t)cpt > 0x7FFFFFFF) return fail(OILHIP_E_ARG, "kv_append: too many tokens for one call");
        hipLaunchKernelGGL(kv_append_kernel, dim3((uint32_t)(ntok * cpt), 2), dim3(64), 0, (hipStream_t)stream,
                           kv_idx(c, layer, 0), kv_idx(c, layer, 1), kv_cb(c, layer, 0), kv_cb(c, layer, 1), d_k, d_v, pos, ntok,
                           c->per_token, (uint32_t)c->block, cpt, c->idx_bytes);
        OILHIP_HIP(hipGetLastError());
    }
    c->pos[(size_t)layer] = pos + seq_len;                                          // :290, dropped tokens counted as well
    return OILHIP_OK;
}

int oilhip_kv_get_range(const oilhip_kv* c, int layer, int64_t start, int64_t end, float* d_k, float* d_v, int64_t* len_out,
                        void* stream) {
    if (len_out) *len_out = 0;
    if (!c) return fail(OILHIP_E_ARG, "kv_get_range: cache is null");
    if (layer < 0 || start < 0) return fail(OILHIP_E_ARG, "kv_get_range: negative layer or start");
    if (layer >= c->layers) return OILHIP_OK;                                       // :295
    int64_t held = c->pos[(size_t)layer];
    if (held > c->max_seq) held = c->max_seq;          // the reference would read past its arrays here; tokens that were dropped are not returned
    int64_t len = end - start;
    if (len <= 0) return OILHIP_OK;
    if (start + len > held) len = held - start;
    if (len <= 0 || c->per_token == 0) return OILHIP_OK;
    if (!d_k || !d_v) return fail(OILHIP_E_ARG, "kv_get_range: null output");
    const uint64_t first = (uint64_t)start * (uint64_t)c->per_token, count = (uint64_t)len * (uint64_t)c->per_token;
    const uint32_t shift = c->block == 32 ? 5u : c->block == 64 ? 6u : 7u;
    if ((c->per_token & 3) == 0 && (((uintptr_t)d_k | (uintptr_t)d_v) & 15) == 0) {
        const uint64_t tiles = (count + kTile - 1) / kTile;
        if (tiles > 0x7FFFFFFFull) return fail(OILHIP_E_ARG, "kv_get_range: range too long for one call");
        hipLaunchKernelGGL(kv_get_range_kernel, dim3((uint32_t)tiles, 2), dim3(256), 0, (hipStream_t)stream, kv_idx(c, layer, 0),
                           kv_idx(c, layer, 1), kv_cb(c, layer, 0), kv_cb(c, layer, 1), d_k, d_v, first, count, shift,
                           (uint64_t)c->nblocks * 16);
    } else {
        const uint64_t groups = (count + 255) / 256;
        if (groups > 0x7FFFFFFFull) return fail(OILHIP_E_ARG, "kv_get_range: range too long for one call");
        hipLaunchKernelGGL(kv_get_range_scalar_kernel, dim3((uint32_t)groups, 2), dim3(256), 0, (hipStream_t)stream,
                           kv_idx(c, layer, 0), kv_idx(c, layer, 1), kv_cb(c, layer, 0), kv_cb(c, layer, 1), d_k, d_v, first, count,
                           shift, (uint64_t)c->per_token, (uint64_t)c->idx_bytes);
    }
    OILHIP_HIP(hipGetLastError());
    if (len_out) *len_out = len;
    return OILHIP_OK;
}

int oilhip_kv_info(const oilhip_kv* c, int* context_len, int64_t* block_size, uint64_t* size_bytes, uint64_t* fp32_bytes) {
    if (!c) return fail(OILHIP_E_ARG, "kv_info: cache is null");
    const int64_t tokens = c->pos.empty() ? 0 : c->pos[0];                          // context_len(): layer 0 (:368-370)
    if (context_len) *context_len = (int)tokens;
    if (block_size) *block_size = c->block;
    if (size_bytes) *size_bytes = (uint64_t)c->layers * (2ull * (uint64_t)c->idx_bytes + 2ull * (uint64_t)c->nblocks * 32ull);   // :372-380
    if (fp32_bytes) *fp32_bytes = (uint64_t)(tokens * c->per_token * 2 * 4);        // :382-386
    return OILHIP_OK;
}

int oilhip_kv_clear(oilhip_kv* c, void* stream) {
    if (!c) return fail(OILHIP_E_ARG, "kv_clear: cache is null");
    const uint64_t n_idx = (uint64_t)c->layers * 2 * (uint64_t)c->idx_stride / 16, n_cb = (uint64_t)c->layers * 2 * (uint64_t)c->nblocks * 32 / 16;
    if (n_idx) hipLaunchKernelGGL(kv_zero_kernel, dim3((uint32_t)std::min<uint64_t>((n_idx + 255) / 256, 4096)), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<uint4*>(c->d_idx), n_idx);
    if (n_cb) hipLaunchKernelGGL(kv_zero_kernel, dim3((uint32_t)std::min<uint64_t>((n_cb + 255) / 256, 4096)), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<uint4*>(c->d_cb), n_cb);
    OILHIP_HIP(hipGetLastError());
    for (auto& p : c->pos) p = 0;
    return OILHIP_OK;
}

int oilhip_kv_resize(oilhip_kv* c, int64_t new_max_seq_len) {
    if (!c) return fail(OILHIP_E_ARG, "kv_resize: cache is null");
    if (new_max_seq_len < 0) return fail(OILHIP_E_ARG, "kv_resize: negative length");
    OILHIP_HIP(hipDeviceSynchronize());
    if (c->d_idx) (void)hipFree(c->d_idx);
    if (c->d_cb) (void)hipFree(c->d_cb);
    c->max_seq = new_max_seq_len;
    for (auto& p : c->pos) p = 0;                                                   // :408 -- every layer starts empty again
    return kv_alloc(c);
}

int oilhip_kv_state(const oilhip_kv* c, int layer, uint8_t* k_idx, uint8_t* v_idx, uint16_t* k_cb, uint16_t* v_cb) {
    if (!c || layer < 0 || layer >= c->layers) return fail(OILHIP_E_ARG, "kv_state: bad cache or layer");
    OILHIP_HIP(hipDeviceSynchronize());
    if (c->idx_bytes) {
        if (k_idx) OILHIP_HIP(hipMemcpy(k_idx, kv_idx(c, layer, 0), (size_t)c->idx_bytes, hipMemcpyDeviceToHost));
        if (v_idx) OILHIP_HIP(hipMemcpy(v_idx, kv_idx(c, layer, 1), (size_t)c->idx_bytes, hipMemcpyDeviceToHost));
        if (k_cb) OILHIP_HIP(hipMemcpy(k_cb, kv_cb(c, layer, 0), (size_t)c->nblocks * 32, hipMemcpyDeviceToHost));
        if (v_cb) OILHIP_HIP(hipMemcpy(v_cb, kv_cb(c, layer, 1), (size_t)c->nblocks * 32, hipMemcpyDeviceToHost));
    }
    return OILHIP_OK;
}

int oilhip_kv_quantize_blocks(const float* d_src, int64_t n, int64_t nblocks, uint8_t* d_codes, uint16_t* d_cb16, void* stream) {
    if (n < 0 || nblocks < 0) return fail(OILHIP_E_ARG, "kv_quantize_blocks: negative size");
    if (n > 128) return fail(OILHIP_E_ARG, "kv_quantize_blocks: at most 128 values per block on the device (the cache's largest block)");
    if (n == 0 || nblocks == 0) return OILHIP_OK;                                   // :78
    if (!d_src || !d_codes || !d_cb16) return fail(OILHIP_E_ARG, "kv_quantize_blocks: null pointer");
    if (nblocks > 0x7FFFFFFF) return fail(OILHIP_E_ARG, "kv_quantize_blocks: too many blocks for one call");
    hipLaunchKernelGGL(kv_quantize_blocks_kernel, dim3((uint32_t)nblocks), dim3(64), 0, (hipStream_t)stream, d_src, (uint32_t)n, d_codes, d_cb16);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_kv_dequantize_blocks(const uint8_t* d_codes, const uint16_t* d_cb16, float* d_dst, int64_t n, int64_t nblocks, void* stream) {
    if (n < 0 || nblocks < 0) return fail(OILHIP_E_ARG, "kv_dequantize_blocks: negative size");
    if (n == 0 || nblocks == 0) return OILHIP_OK;
    if (!d_codes || !d_cb16 || !d_dst) return fail(OILHIP_E_ARG, "kv_dequantize_blocks: null pointer");
    const uint64_t total = (uint64_t)n * (uint64_t)nblocks;
    if ((total + 255) / 256 > 0x7FFFFFFFull || n > 0x7FFFFFFF) return fail(OILHIP_E_ARG, "kv_dequantize_blocks: too large for one call");
    hipLaunchKernelGGL(kv_dequantize_blocks_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d_codes, d_cb16, d_dst, (uint32_t)n, total);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // extern "C"
