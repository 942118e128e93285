// gemm_oil4_mfma.hip -- prefill GEMM over uniform OIL4 tensors on the matrix cores:
// Y[M][N] = X[M][K] . W^T with X in bf16, W dequantized tile by tile to bf16 in LDS,
// v_mfma_f32_32x32x16_bf16, FP32 accumulation, FP32 output.  Same contraction as the
// reference's FP32 prefill (Qwen35Engine::gemm with B up to 512,
// src/adapters/tools/qwen35_engine.cpp:47-85,630-753) over dequant_lattice blocks
// (src/block_codec.cpp:173-182).
//
// The contraction runs in nibble order: inside a 256-weight block the 4-bit index of
// weight i sits at nibble p = 4 + i - i/64 (nibbles 0..3 are the FP16 scale, weights
// 63,127,191,255 are slots that decode to zero and own no nibble).  A small pre-pass
// writes X' with X'[m][blk*256 + p] = X[m][blk*256 + i(p)] and zeros at p < 4, so the
// main kernel multiplies consecutive nibbles with consecutive X' columns and never
// needs a shift across bytes; the scale nibbles meet zeros.
//
// Main kernel: workgroup = 2 x 2 wavefronts, each wavefront owns WBM x WBN blocks of
// 32 x 32 outputs.  Per 64-column step the workgroup stages an X' tile and a weight tile
// in LDS; the weight tile goes through the same byte -> (level, level) pair table as the
// decode GEMV (one v_perm_b32 + one LDS read per packed byte), is multiplied by the
// block's FP16 scale in FP32 and rounded once to bf16.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "common.h"

namespace oilhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const f32x2 lds_cfloat2;

constexpr int kTabBytes = 256 * 64 * 4;     // pair table: byte v, lane copy c at v*256 + c*8
constexpr int BK = 64;                      // columns per step (a quarter of a block)
constexpr int LDK = BK + 8;                 // LDS row pitch in bf16: 144 bytes keeps 16-byte reads of 16 rows on distinct banks

__device__ __forceinline__ float level_literal(uint32_t i) {      // kOIL4Levels, src/block_codec.cpp:18-23; selects only
    const uint32_t m = i < 8u ? 7u - i : i - 8u;
    uint32_t bits = __float_as_uint(0.1260f);
    bits = m == 1u ? __float_as_uint(0.3976f) : bits;
    bits = m == 2u ? __float_as_uint(0.6508f) : bits;
    bits = m == 3u ? __float_as_uint(0.9275f) : bits;
    bits = m == 4u ? __float_as_uint(1.2392f) : bits;
    bits = m == 5u ? __float_as_uint(1.5995f) : bits;
    bits = m == 6u ? __float_as_uint(2.0522f) : bits;
    bits = m == 7u ? __float_as_uint(2.7178f) : bits;
    return __uint_as_float(bits | (i < 8u ? 0x80000000u : 0u));
}

// X (bf16 bit patterns, [M][K]) -> X' ([Mpad][K], rows >= M zero), columns in nibble order: a thread forms eight
// consecutive columns of X' (one 16-byte store).  The same launch clears Y (zn floats per row, ldy apart) for the
// launches whose two K halves add into it.
__global__ void __launch_bounds__(256)
permute_x_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ xp, uint32_t M, uint32_t K, uint32_t Mpad,
                 float* __restrict__ y, uint32_t zn, uint32_t ldy) {
    const uint32_t row = blockIdx.y;
    for (uint32_t c8 = blockIdx.x * 256 + threadIdx.x; c8 * 8u < K; c8 += gridDim.x * 256) {
        const uint32_t c = c8 * 8u, p0 = c & 255u;
        uint16_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t p = p0 + k;
            v[k] = 0;
            if (p >= 4 && row < M) {
                const uint32_t q = p - 4;
                v[k] = x[(size_t)row * K + (c - p0) + q + (q >= 63) + (q >= 126) + (q >= 189)];
            }
        }
        uint4 o;
        o.x = v[0] | ((uint32_t)v[1] << 16); o.y = v[2] | ((uint32_t)v[3] << 16);
        o.z = v[4] | ((uint32_t)v[5] << 16); o.w = v[6] | ((uint32_t)v[7] << 16);
        *reinterpret_cast<uint4*>(xp + (size_t)row * K + c) = o;
    }
    if (y && row < M) {
        float* yr = y + (size_t)row * ldy;
        if (((ldy | zn) & 3u) == 0u && (reinterpret_cast<uintptr_t>(y) & 15u) == 0u) {
            for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i * 4u < zn; i += gridDim.x * 256)
                reinterpret_cast<float4*>(yr)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < zn; i += gridDim.x * 256) yr[i] = 0.0f;
        }
    }
}

template <int WBM, int WBN>
__global__ void __launch_bounds__(256)
gemm_oil4_bf16_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ Xp, float* __restrict__ Y,
                      uint32_t M, uint32_t N, uint32_t K, uint32_t Mpad) {
    constexpr int BM = 64 * WBM, BN = 64 * WBN;
    constexpr int A_CHUNKS = BM * 8 / 256;          // 16-byte pieces of the X' tile per thread
    constexpr int B_CHUNKS = BN * 2 / 256;          // 16-byte pieces (32 nibbles) of the weight tile per thread
    static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);                                   // LDS byte offset 0
    __bf16* As = reinterpret_cast<__bf16*>(lds + kTabBytes);                      // [BM][LDK]
    __bf16* Bs = As + BM * LDK;                                                   // [BN][LDK]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t bpr = K >> 8, KT = K / BK;

    {   // pair table from literals: float4 e = (lo, hi, lo, hi) of byte value v = e >> 4; e = tid + 256*k
        const float lv_lane = level_literal(lane & 15u);
        const float lo = __int_as_float(__builtin_amdgcn_ds_bpermute((int)(((tid >> 4) & 15u) * 4u), __float_as_int(lv_lane)));
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const float hi = level_literal(k);
            reinterpret_cast<float4*>(tab)[tid + 256u * k] = make_float4(lo, hi, lo, hi);
        }
    }

    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)n0 * bpr * 128u), 0,
        (int)((uint64_t)(N - n0 < (uint32_t)BN ? N - n0 : (uint32_t)BN) * bpr * 128u), 0x00020000);
    const uint16_t* xa = Xp + (size_t)m0 * K;

    u32x4 ar[A_CHUNKS], br[B_CHUNKS];
    uint32_t sr[B_CHUNKS];
    auto load_tiles = [&](uint32_t kt) {
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            const uint32_t id = tid + c * 256u, row = id >> 3, kc = id & 7u;
            ar[c] = *reinterpret_cast<const u32x4*>(xa + (size_t)row * K + kt * BK + kc * 8u);
        }
#pragma unroll
        for (int c = 0; c < B_CHUNKS; ++c) {
            const uint32_t id = tid + c * 256u, row = id >> 1, half = id & 1u;
            const uint32_t blk_off = (row * bpr + (kt >> 2)) * 128u;
            br[c] = __builtin_amdgcn_raw_buffer_load_b128(wrs, blk_off + (kt & 3u) * 32u + half * 16u, 0, 0);
            sr[c] = __builtin_amdgcn_raw_buffer_load_b16(wrs, blk_off, 0, 0);     // the block's FP16 scale
        }
    };
    const uint32_t lanebase = (lane & 31u) * 8u;
    auto store_tiles = [&]() {
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            const uint32_t id = tid + c * 256u, row = id >> 3, kc = id & 7u;
            *reinterpret_cast<u32x4*>(As + row * LDK + kc * 8u) = ar[c];
        }
#pragma unroll
        for (int c = 0; c < B_CHUNKS; ++c) {
            const uint32_t id = tid + c * 256u, row = id >> 1, half = id & 1u;
            const float scale = __half2float(__ushort_as_half((unsigned short)sr[c]));
            const uint32_t wd[4] = {br[c].x, br[c].y, br[c].z, br[c].w};
            uint32_t packed[16];
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t addr = __builtin_amdgcn_perm(wd[d], lanebase, 0x0C0C0000u | ((4u + j) << 8));
                    const f32x2 t = *(lds_cfloat2*)(uintptr_t)addr;
                    const bf16x2 pr = bf16x2{(__bf16)(t.x * scale), (__bf16)(t.y * scale)};
                    packed[d * 4 + j] = *reinterpret_cast<const uint32_t*>(&pr);
                }
            u32x4* dst = reinterpret_cast<u32x4*>(Bs + row * LDK + half * 32u);
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[q] = u32x4{packed[4 * q], packed[4 * q + 1], packed[4 * q + 2], packed[4 * q + 3]};
        }
    };

    f32x16 acc[WBM][WBN];
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    load_tiles(0);
    __syncthreads();                                   // table complete
    for (uint32_t kt = 0; kt < KT; ++kt) {
        store_tiles();
        __syncthreads();
        if (kt + 1 < KT) load_tiles(kt + 1);           // next tile's global loads fly during the MFMAs
        const __bf16* ap = As + (wm * WBM * 32u + (lane & 31u)) * LDK + (lane >> 5) * 8u;
        const __bf16* bp = Bs + (wn * WBN * 32u + (lane & 31u)) * LDK + (lane >> 5) * 8u;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            bf16x8 a[WBM], b[WBN];
#pragma unroll
            for (int i = 0; i < WBM; ++i) a[i] = *reinterpret_cast<const bf16x8*>(ap + i * 32 * LDK + kk * 16);
#pragma unroll
            for (int j = 0; j < WBN; ++j) b[j] = *reinterpret_cast<const bf16x8*>(bp + j * 32 * LDK + kk * 16);
#pragma unroll
            for (int i = 0; i < WBM; ++i)
#pragma unroll
                for (int j = 0; j < WBN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout of the 32x32 MFMA: lane l holds column l % 32; register v holds row 8*(v/4) + 4*(l/32) + v%4
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j) {
            const uint32_t col = n0 + (wn * WBN + j) * 32u + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + (wm * WBM + i) * 32u + 8u * (v >> 2) + 4u * (lane >> 5) + (v & 3u);
                if (row < M && col < N) Y[(size_t)row * N + col] = acc[i][j][v];
            }
        }
}

// Y <- 0 in front of a launch whose workgroups add partial sums (a fill kernel, so that a caller may capture it in a graph)
__global__ void __launch_bounds__(256) zero_y_kernel(float* __restrict__ y, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (size_t)gridDim.x * 256u) y[i] = 0.f;
}

// Y[m][0..n) <- 0 for rows of ldy floats
__global__ void __launch_bounds__(256) zero_y2d_kernel(float* __restrict__ y, uint32_t n, uint32_t ldy) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c < n) y[(size_t)blockIdx.y * ldy + c] = 0.f;
}

// Pipelined kernel for larger M: TBM (256 or 128) tokens x 128 weight rows per workgroup, 8 wavefronts (TBM = 256:
// 4 x 2 wavefronts of 64 x 64 outputs; TBM = 128: 2 x 4 of 64 x 32), 64 columns per step, two LDS tile buffers.
// Per step a thread stages TBM / 4 bytes of X' and decodes 8 bytes (16 nibbles) of weights; the global loads of two
// further steps are in flight.
//
// The eight wavefronts work as two groups of four (one per SIMD each), half a step apart: while one group reads
// its fragments of a step from LDS, the other multiplies, finishes the decode of a later tile and stores it, so
// the LDS pipe and the matrix cores are busy at the same time instead of one after the other.  Slots are
// separated by workgroup barriers; group g reads step r in slot 2r + g and multiplies in slot 2r + 1 + g, and
// during that product stores its share of tile r + 1 + g (buffer (r + 1 + g) & 1): group 0's target was last read
// in slot 2r - 1 and is needed from slot 2r + 2, group 1's was last read in slot 2r + 1 and is needed from
// slot 2r + 4.  Both groups pass 2 * steps + 1 barriers after the prologue.
constexpr int PK = 64;                      // columns per step
constexpr int PLD = PK;                     // LDS row pitch in bf16: 128 bytes = 8 chunks of 16 bytes; the chunk index of a
                                            // row is XOR-swizzled with (row / 2) % 8 so that the tile stores (2 rows x 8
                                            // chunks per 16 lanes) and the fragment reads (16 rows x 1 chunk) touch every bank once
constexpr int PBN = 128;
constexpr int PD = 2;                       // steps of global loads in flight: even, divides K / 64 / 2 (4 measured the same)
__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row >> 1) & 7u; }

//
// DENSE: the weight operand is a bf16 matrix [N][K] in natural column order (a tensor of any format, decoded to
// bf16 beforehand) and Xp is X itself, [M][K]; rows past M and N read as zero through the buffer bounds.  Y has ldy
// floats per row.
template <int TBM, bool DENSE>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_oil4_bf16_pipe_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ Xp, float* __restrict__ Y,
                           uint32_t M, uint32_t N, uint32_t K, uint32_t ksplit, uint32_t ldy) {
    static_assert(TBM == 256 || TBM == 128, "workgroup tiles of 256 or 128 tokens");
    constexpr int WN = TBM == 256 ? 2 : 4;              // wavefronts along the weight rows
    constexpr int NJ = PBN / WN / 32;                   // 32-row fragments per wavefront along the weight rows
    constexpr int AC = TBM / 64;                        // 16-byte pieces of the X' tile per thread
    constexpr int D = PD;
    extern __shared__ __align__(16) uint8_t lds[];
    float* tab = reinterpret_cast<float*>(lds);
    __bf16* As = reinterpret_cast<__bf16*>(lds + kTabBytes);                      // [2][TBM][PLD]
    __bf16* Bs = As + 2 * TBM * PLD;                                              // [2][PBN][PLD]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t m0 = blockIdx.y * TBM, n0 = blockIdx.x * PBN;
    const uint32_t bpr = K >> 8, KT = K / PK;

    if constexpr (!DENSE) {   // pair table from literals: float4 e = (lo, hi, lo, hi) of byte value v = e >> 4; e = tid + 512*k
        const float lv_lane = level_literal(lane & 15u);
        const float lo = __int_as_float(__builtin_amdgcn_ds_bpermute((int)(((tid >> 4) & 15u) * 4u), __float_as_int(lv_lane)));
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lv_lane), (int)((tid >> 8) + 2u * k)));
            reinterpret_cast<float4*>(tab)[tid + 512u * k] = make_float4(lo, hi, lo, hi);
        }
    }

    const uint32_t nrows = N - n0 < (uint32_t)PBN ? N - n0 : (uint32_t)PBN;
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(W + (size_t)n0 * (DENSE ? (size_t)K * 2u : (size_t)bpr * 128u)), 0,
        (int)((uint64_t)nrows * (DENSE ? (uint64_t)K * 2u : (uint64_t)bpr * 128u)), 0x00020000);
    const uint16_t* xa = Xp + (size_t)m0 * K;
    const uint32_t mrows = DENSE ? (M - m0 < (uint32_t)TBM ? M - m0 : (uint32_t)TBM) : (uint32_t)TBM;
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc((void*)xa, 0, (int)((uint64_t)mrows * K * 2u), 0x00020000);
    const uint32_t brow = tid >> 2, bq = tid & 3u;                               // weight row of the tile, 8-byte piece of the 32 bytes of a step
    const uint32_t lanebase = (lane & 31u) * 8u;

    u32x4 ar[D][AC], bd[D][DENSE ? 2 : 1];
    uint32_t br[D][2], sr[D];
    auto load_regs = [&](int set, uint32_t kt) {
#pragma unroll
        for (int c = 0; c < AC; ++c) {
            const uint32_t id = tid + c * 512u, row = id >> 3, kc = id & 7u;
            if constexpr (DENSE) ar[set][c] = __builtin_amdgcn_raw_buffer_load_b128(xrs, (row * K + kt * PK + kc * 8u) * 2u, 0, 0);
            else ar[set][c] = *reinterpret_cast<const u32x4*>(xa + (size_t)row * K + kt * PK + kc * 8u);
        }
        if constexpr (DENSE) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const uint32_t id = tid + c * 512u, row = id >> 3, kc = id & 7u;
                bd[set][c] = __builtin_amdgcn_raw_buffer_load_b128(wrs, (row * K + kt * PK + kc * 8u) * 2u, 0, 0);
            }
            return;
        }
        const uint32_t blk_off = (brow * bpr + (kt >> 2)) * 128u;
        const uint32_t off = blk_off + (kt & 3u) * 32u + bq * 8u;
        br[set][0] = __builtin_amdgcn_raw_buffer_load_b32(wrs, off, 0, 0);
        br[set][1] = __builtin_amdgcn_raw_buffer_load_b32(wrs, off + 4u, 0, 0);
        sr[set] = __builtin_amdgcn_raw_buffer_load_b16(wrs, blk_off, 0, 0);
    };
    // decode of a later step, split so that its table reads are issued with the fragment reads and its arithmetic
    // runs in the shadow of the MFMAs
    auto lookup_tiles = [&](int set, f32x2 (&t)[8]) {
        if constexpr (DENSE) return;
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t addr = __builtin_amdgcn_perm(br[set][d], lanebase, 0x0C0C0000u | ((4u + j) << 8));
                t[d * 4 + j] = *(lds_cfloat2*)(uintptr_t)addr;
            }
    };
    auto finish_tiles = [&](int set, int buf, const f32x2 (&t)[8]) {
#pragma unroll
        for (int c = 0; c < AC; ++c) {
            const uint32_t id = tid + c * 512u, row = id >> 3, kc = id & 7u;
            *reinterpret_cast<u32x4*>(As + (buf * TBM + row) * PLD + ((kc ^ swz(row)) * 8u)) = ar[set][c];
        }
        if constexpr (DENSE) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const uint32_t id = tid + c * 512u, row = id >> 3, kc = id & 7u;
                *reinterpret_cast<u32x4*>(Bs + (buf * PBN + row) * PLD + ((kc ^ swz(row)) * 8u)) = bd[set][c];
            }
            return;
        }
        const float scale = __half2float(__ushort_as_half((unsigned short)sr[set]));
        uint32_t packed[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bf16x2 pr = bf16x2{(__bf16)(t[j].x * scale), (__bf16)(t[j].y * scale)};
            packed[j] = *reinterpret_cast<const uint32_t*>(&pr);
        }
        const uint32_t sb = swz(brow);
        __bf16* dst = Bs + (buf * PBN + brow) * PLD;
        // odd rows store their second 16 bytes first: the two rows that share a swizzle value then fall into different
        // banks within one store instruction
        const bool odd = brow & 1u;
        const u32x4 c0 = u32x4{packed[0], packed[1], packed[2], packed[3]}, c1 = u32x4{packed[4], packed[5], packed[6], packed[7]};
        *reinterpret_cast<u32x4*>(dst + (((2u * bq + (odd ? 1u : 0u)) ^ sb) * 8u)) = odd ? c1 : c0;
        *reinterpret_cast<u32x4*>(dst + (((2u * bq + (odd ? 0u : 1u)) ^ sb) * 8u)) = odd ? c0 : c1;
    };
    auto store_tiles = [&](int set, int buf) {
        f32x2 t[8];
        lookup_tiles(set, t);
        finish_tiles(set, buf, t);
    };

    f32x16 acc[2][NJ];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const uint32_t sw = swz(lane & 31u);
    bf16x8 fa[4][2], fb[4][NJ];
    auto read_frags = [&](int buf) {
        const __bf16* ap = As + (buf * TBM + wm * 64u + (lane & 31u)) * PLD;
        const __bf16* bp = Bs + (buf * PBN + wn * (NJ * 32u) + (lane & 31u)) * PLD;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const uint32_t ch = (((uint32_t)kk * 2u + (lane >> 5)) ^ sw) * 8u;
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[kk][i] = *reinterpret_cast<const bf16x8*>(ap + i * 32 * PLD + ch);
#pragma unroll
            for (int j = 0; j < NJ; ++j) fb[kk][j] = *reinterpret_cast<const bf16x8*>(bp + j * 32 * PLD + ch);
        }
    };
    auto do_mfmas = [&]() {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk][i], fb[kk][j], acc[i][j], 0, 0, 0);
    };

    // K is a multiple of 256, so KT is a multiple of 4; a workgroup's share of the steps (all, a half or a quarter of
    // them) is a multiple of D.  Every load and every decode below is issued unconditionally (steps past the end are
    // clamped to the last one and decoded into a buffer nobody reads any more): the number of loads in flight is then
    // a compile-time fact and each wait covers exactly the step it needs.
    // ksplit > 1: workgroup blockIdx.z takes the steps [kbeg, kend) of the row and adds its partial sums to a zeroed Y
    // (two parts at most, so the sum does not depend on which arrives first)
    const uint32_t kbeg = KT / ksplit * blockIdx.z, kend = blockIdx.z + 1u == ksplit ? KT : kbeg + KT / ksplit;
    const uint32_t last = kend - 1u, nk = kend - kbeg;
    auto clampk = [&](uint32_t k) { return k < last ? k : last; };
#pragma unroll
    for (int u = 0; u < D; ++u) load_regs(u, clampk(kbeg + (uint32_t)u));
    __syncthreads();                                   // table complete
    store_tiles(0, 0);
    load_regs(0, clampk(kbeg + (uint32_t)D));
    // The two wavefront groups run different instantiations of `run` and meet at workgroup barriers written at
    // different places of the code: the hardware barrier only counts arrivals, so the two instantiations must execute
    // the same number of barriers in total (group 0: 1 + 2 per step + 1, group 1: 2 + 2 per step).  Any change to one
    // instantiation's barriers needs the matching change in the other.
    static_assert(D >= 2 && D % 2 == 0, "the tile buffer of a step is (u + 1 + G) & 1: the unrolled steps must come in pairs");
    auto run = [&](auto gc) {
        constexpr int G = decltype(gc)::value;
        if constexpr (G == 1) {                        // the late group also brings its share of tile 1
            store_tiles(1 % D, 1);
            load_regs(1 % D, clampk(kbeg + 1u + (uint32_t)D));
        }
        __syncthreads();                               // tile 0 (and the late group's share of tile 1) in place
        if constexpr (G == 1) __syncthreads();         // slot 0 belongs to the early group
        for (uint32_t r0 = 0; r0 < nk; r0 += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const int set = (u + 1 + G) % D, buf = (u + 1 + G) & 1;
                f32x2 t[8];
                lookup_tiles(set, t);
                read_frags(u & 1);
                __syncthreads();
                do_mfmas();
                finish_tiles(set, buf, t);
                load_regs(set, clampk(kbeg + r0 + (uint32_t)(u + 1 + G + D)));
                __syncthreads();
            }
        }
        if constexpr (G == 0) __syncthreads();
    };
    if (wave < 4u) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const uint32_t col = n0 + (wn * NJ + j) * 32u + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + (wm * 2 + i) * 32u + 8u * (v >> 2) + 4u * (lane >> 5) + (v & 3u);
                if (row < M && col < N) {
                    if (ksplit > 1u) unsafeAtomicAdd(Y + (size_t)row * ldy + col, acc[i][j][v]);
                    else Y[(size_t)row * ldy + col] = acc[i][j][v];
                }
            }
        }
}


template <int WBM, int WBN>
int launch(const oilhip_weights& w, const uint16_t* xp, float* d_y, uint32_t M, uint32_t Mpad, hipStream_t s) {
    constexpr int BM = 64 * WBM, BN = 64 * WBN;
    const size_t lds_bytes = (size_t)kTabBytes + (size_t)(BM + BN) * LDK * 2;
    static std::atomic<uint64_t> attr_done{0};
    auto kern = gemm_oil4_bf16_kernel<WBM, WBN>;
    if (int rc = ensure_max_lds(attr_done, reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
    const uint32_t N = (uint32_t)w.rows, K = (uint32_t)w.cols;
    hipLaunchKernelGGL(kern, dim3((N + BN - 1) / BN, Mpad / BM), dim3(256), lds_bytes, s, w.d_payload, xp, d_y, M, N, K, Mpad);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

// Tiling of the pipelined kernel for M tokens and Nc weight rows
struct PipePlan { bool wide; uint32_t ntn, tbm, mt, ksplit; };
PipePlan pipe_plan(uint32_t M, uint32_t Nc, uint32_t K) {
    PipePlan p;
    const uint32_t cus = (uint32_t)device_cu_count();
    p.ntn = (Nc + PBN - 1) / PBN;
    p.wide = M > 256u && p.ntn * ((M + 255u) / 256u) * 2u > cus;
    p.tbm = p.wide ? 256u : 128u;
    p.mt = (M + p.tbm - 1) / p.tbm;
    p.ksplit = p.ntn * p.mt * 2u <= cus && (K / PK) % 8u == 0u ? 2u : 1u;
    return p;
}

// The pipelined kernel over Nc weight rows (OIL4 blocks, or DENSE: bf16 [Nc][K]); Y + column offset already applied,
// ldy floats per output row.  A grid that leaves half of the compute units idle is cut in two along K (two partial
// sums into a zeroed Y: the order of two addends does not matter).
template <bool DENSE>
int launch_pipe(const uint8_t* wmat, const uint16_t* x, float* d_y, uint32_t M, uint32_t Nc, uint32_t K, uint32_t ldy, hipStream_t s,
                bool y_is_zero = false) {
    static std::atomic<uint64_t> attr_done[2];
    const PipePlan pl = pipe_plan(M, Nc, K);
    const bool wide = pl.wide;
    const uint32_t ntn = pl.ntn, tbm = pl.tbm, mt = pl.mt, ksplit = pl.ksplit;
    if (ksplit > 1u && !y_is_zero) {
        if (ldy == Nc) {
            hipLaunchKernelGGL(zero_y_kernel, dim3((uint32_t)std::min<size_t>(((size_t)M * Nc + 255) / 256, 4096)), dim3(256), 0, s, d_y, (size_t)M * Nc);
        } else {
            hipLaunchKernelGGL(zero_y2d_kernel, dim3((Nc + 255u) / 256u, M), dim3(256), 0, s, d_y, Nc, ldy);
        }
        OILHIP_HIP(hipGetLastError());
    }
    const size_t lds_bytes = (size_t)kTabBytes + 2ull * (tbm + PBN) * PLD * 2;
    if (wide) {
        auto kern = gemm_oil4_bf16_pipe_kernel<256, DENSE>;
        if (int rc = ensure_max_lds(attr_done[0], reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
        hipLaunchKernelGGL(kern, dim3(ntn, mt, ksplit), dim3(512), lds_bytes, s, wmat, x, d_y, M, Nc, K, ksplit, ldy);
    } else {
        auto kern = gemm_oil4_bf16_pipe_kernel<128, DENSE>;
        if (int rc = ensure_max_lds(attr_done[1], reinterpret_cast<const void*>(kern), 160 * 1024)) return rc;
        hipLaunchKernelGGL(kern, dim3(ntn, mt, ksplit), dim3(512), lds_bytes, s, wmat, x, d_y, M, Nc, K, ksplit, ldy);
    }
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // namespace

// FP32 -> bf16 (round to nearest even), four values per thread
__global__ void __launch_bounds__(256) x_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ o, uint64_t n) {
    for (uint64_t i = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 4u; i < n; i += (uint64_t)gridDim.x * 1024u) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (i + k < n) { const __bf16 b = (__bf16)x[i + k]; o[i + k] = *reinterpret_cast<const uint16_t*>(&b); }
    }
}

int launch_x_to_bf16(const float* d_x, uint64_t n, uint16_t** out, hipStream_t s) {
    uint16_t* xb = nullptr;
    if (int rc = stream_scratch(s, kScratchGemmXb, (size_t)n * 2, reinterpret_cast<void**>(&xb))) return rc;
    hipLaunchKernelGGL(x_to_bf16_kernel, dim3((uint32_t)std::min<uint64_t>((n + 1023) / 1024, 8192)), dim3(256), 0, s, d_x, xb, n);
    OILHIP_HIP(hipGetLastError());
    *out = xb;
    return OILHIP_OK;
}

// Prefill over a tensor of any format (full 256-weight blocks): slabs of weight rows are decoded to bf16 in a scratch
// buffer of the stream (dequantize_block_all's values, each rounded once to bf16) and multiplied by the same pipelined
// kernel reading a dense operand.  Returns 1 when the tensor's layout is not covered.
int launch_gemm_any_bf16(const oilhip_weights& w, const uint16_t* d_x, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull) return fail(OILHIP_E_ARG, "matrix too large for the prefill kernel");
    const uint32_t N = (uint32_t)w.rows, K = (uint32_t)w.cols, bpr = K >> 8;
    if ((uint64_t)M * K * 2u >= 0x80000000ull) return fail(OILHIP_E_ARG, "activation matrix too large for the prefill kernel");
    if (!dequant_bf16_blocks_covers(w)) return 1;      // before any scratch is allocated for it
    // slab: at most 64 MB of bf16, a multiple of 128 rows
    uint32_t slab = (uint32_t)std::min<uint64_t>(N, std::max<uint64_t>(128, ((64ull << 20) / ((uint64_t)K * 2u)) & ~127ull));
    uint16_t* wd = nullptr;
    if (int rc = stream_scratch(s, kScratchGemmW, (size_t)slab * K * 2, reinterpret_cast<void**>(&wd))) return rc;
    for (uint32_t n0 = 0; n0 < N; n0 += slab) {
        const uint32_t nc = std::min(slab, N - n0);
        if (int rc = launch_dequant_bf16_blocks(w, n0 * bpr, nc * bpr, wd, s)) return rc;
        if (int rc = launch_pipe<true>(reinterpret_cast<const uint8_t*>(wd), d_x, d_y + n0, (uint32_t)M, nc, K, N, s)) return rc;
    }
    return OILHIP_OK;
}

int launch_gemm_oil4_bf16(const oilhip_weights& w, const uint16_t* d_x, float* d_y, int M, hipStream_t s) {
    if (w.rows > 0x7FFFFFFFull || w.cols > 0x7FFFFFFFull) return fail(OILHIP_E_ARG, "matrix too large for the prefill kernel");
    const uint32_t K = (uint32_t)w.cols;
    // the fragment-order kernel (it loads X in 16-byte pieces) for every batch size: at 64 to 256 tokens it is two to
    // three and a half times faster than the tiles below (11008 x 4096: 25.6 - 39.4 us against 68.5 - 70.6 us), which
    // remain for activations that are not 16-byte aligned
    if ((reinterpret_cast<uintptr_t>(d_x) & 15u) == 0u) return launch_gemm_oil4_frag(w, d_x, false, d_y, M, s);
    const bool big = M > 256;
    const uint32_t N = (uint32_t)w.rows, ntn = (N + PBN - 1) / PBN, cus = (uint32_t)device_cu_count();
    // M > 256 runs the pipelined kernel.  Its 256-token tiles decode each weight tile once per 256 tokens; when they
    // leave more than half of the compute units without a workgroup, 128-token tiles put twice as many to work.
    const bool wide = big && ntn * (((uint32_t)M + 255u) / 256u) * 2u > cus;
    const uint32_t BM = wide ? 256 : 128;
    const uint32_t Mpad = ((uint32_t)M + BM - 1) / BM * BM;
    uint16_t* xp = nullptr;
    if (int rc = stream_scratch(s, kScratchGemmX, (size_t)Mpad * K * 2, reinterpret_cast<void**>(&xp))) return rc;
    // the launch that follows adds two K halves into Y: cleared here, in the same launch
    const bool clear_y = big && pipe_plan((uint32_t)M, N, K).ksplit > 1u;
    uint32_t gx = std::max<uint32_t>((K / 8u + 255u) / 256u, clear_y ? (N / 4u + 255u) / 256u : 1u);
    if (gx > 64) gx = 64;
    hipLaunchKernelGGL(permute_x_kernel, dim3(gx, Mpad), dim3(256), 0, s, d_x, xp, (uint32_t)M, K, Mpad, clear_y ? d_y : (float*)nullptr, N, N);
    OILHIP_HIP(hipGetLastError());
    if (big) return launch_pipe<false>(w.d_payload, xp, d_y, (uint32_t)M, N, K, N, s, clear_y);
    return launch<2, 2>(w, xp, d_y, (uint32_t)M, Mpad, s);
}

}  // namespace oilhip
