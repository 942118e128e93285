// oil4_lds.h -- device helpers shared by the OIL4 decode kernels: DPP moves, the level table
// of dequant_lattice (src/block_codec.cpp:18-23,173-182) and the LDS byte-pair lookup.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace oilhip {
namespace oil4 {

constexpr int kTabBytes = 256 * 64 * 4;   // [byte value][low|high nibble][32 lane copies] floats
constexpr int kMaxLds = 160 * 1024;

__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
}
__device__ __forceinline__ float dpp_half_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
}
__device__ __forceinline__ float dpp_row_ror8(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));  // row_ror:8
}
__device__ __forceinline__ float dpp_row_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
}
// lane 15 of rows 0 and 2 into every lane of rows 1 and 3 (other rows receive 0)
__device__ __forceinline__ float dpp_row_bcast15(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));
}
// lane 31 into every lane of rows 2 and 3 (other rows receive 0)
__device__ __forceinline__ float dpp_row_bcast31(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));
}
// value of the first lane of each group of 8 lanes, in all 8 lanes
__device__ __forceinline__ uint32_t dpp_bcast8(uint32_t v) {
    const int q = __builtin_amdgcn_update_dpp(0, (int)v, 0x00, 0xF, 0xF, true);      // quad_perm [0,0,0,0]
    return (uint32_t)__builtin_amdgcn_update_dpp(q, q, 0x114, 0xF, 0xA, false);     // row_shr:4 into quads 1 and 3
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kOobOffset = 0xFFFFFF00u;   // beyond any buffer range: the load returns zeros, no fetch

// The two level values of one packed byte: (low nibble, high nibble).
struct LevelPair { float lo, hi; };

// kOIL4Levels (src/block_codec.cpp:18-23) selected by compares on literals: no memory access.
__device__ __forceinline__ float level_literal(uint32_t i) {
    // selects only: a branch tree here costs the prologue a string of instruction-cache misses
    const uint32_t m = i < 8u ? 7u - i : i - 8u;                   // magnitude index, 0 = innermost level
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

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const f32x2 lds_cfloat2;
typedef __attribute__((address_space(3))) const float lds_cfloat;
typedef __attribute__((address_space(3))) const uint32_t lds_cuint;

// Pair table, 64 KB at LDS offset 0: entry of byte value v and lane copy c at
// byte v*256 + c*8 = (level[v & 15], level[v >> 4]).  32 lane-private copies:
// lanes of a half-wave never meet in a bank at different addresses.
template <int J>
__device__ __forceinline__ LevelPair lookup(uint32_t word, uint32_t lanebase) {
    // byte J of the dword -> address bits 8..15, this lane's copy -> bits 0..7
    const uint32_t addr = __builtin_amdgcn_perm(word, lanebase, 0x0C0C0000u | ((4u + J) << 8));
    const f32x2 t = *(lds_cfloat2*)(uintptr_t)addr;
    return LevelPair{t.x, t.y};
}

__device__ __forceinline__ void lookup_load(const u32x4& w, uint32_t lanebase, LevelPair (&t)[16]) {
    const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        t[d * 4 + 0] = lookup<0>(wd[d], lanebase);
        t[d * 4 + 1] = lookup<1>(wd[d], lanebase);
        t[d * 4 + 2] = lookup<2>(wd[d], lanebase);
        t[d * 4 + 3] = lookup<3>(wd[d], lanebase);
    }
}

}  // namespace oil4
}  // namespace oilhip
