// check_reference_signatures.cpp -- compile-time check that every function the shims define has exactly the type the
// reference declares.  Compiled (syntax only) with the reference's include directory on the path, so that
// oilhip_shims.hpp takes its reference-tree branch; a shim whose arguments drift from the reference's declaration
// would otherwise be a silent overload that nothing calls.  The expected types are spelled out here by hand, from the
// declarations the stand-alone branch of oilhip_shims.hpp uses.
#include <cstddef>
#include <cstdint>
#include <type_traits>
#include <vector>

#include "oil/backend.h"
#include "oil/block_codec.h"
#include "oil/kernel.h"
#include "oil/kernel_production.h"
#include "oil/kv_cache_oil4.h"
#include "oil/oil_engines.h"

#include "oilhip_shims.hpp"

#ifndef OILHIP_REFERENCE_TREE
#error "compile with the reference's include directory on the include path"
#endif

namespace {
using u8 = uint8_t;
using u16 = uint16_t;
template <class Got, class Want> constexpr bool same = std::is_same_v<Got, Want>;

// include/oil/block_codec.h:55-63
static_assert(same<decltype(&oil::quantize_block_all), bool (*)(oil::Format, const float*, int, std::vector<u8>&, std::vector<u8>&)>);
static_assert(same<decltype(&oil::dequantize_block_all), void (*)(oil::Format, const u8*, size_t, const u8*, size_t, uint32_t, float*)>);
// include/oil/kernel.h:11-32
static_assert(same<decltype(&oil::kernel::oil8_gemm), void (*)(const u8*, const float*, const float*, float*, int, int, int)>);
static_assert(same<decltype(&oil::kernel::oil4_gemm), void (*)(const u8*, const u16*, const float*, float*, int, int, int)>);
static_assert(same<decltype(&oil::kernel::tl1_gemm), void (*)(const oil::Tensor&, const oil::Tensor&, oil::Tensor&, int, int, int)>);
static_assert(same<decltype(&oil::kernel::tl2_gemm), void (*)(const oil::Tensor&, const oil::Tensor&, oil::Tensor&, int, int, int)>);
// include/oil/kernel_production.h:19-82
namespace prod = oil::adapters::prod;
static_assert(same<decltype(&prod::detect_cpu_isa), int (*)()>);
static_assert(same<decltype(&prod::gemv_spark_tiled), void (*)(const u8*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::gemv_oil4_tiled), void (*)(const u8*, const u16*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::gemv_oil8_tiled), void (*)(const u8*, const float*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::gemv_spark_batch), void (*)(const u8*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::gemv_oil4_batch), void (*)(const u8*, const u16*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::gemv_oil8_batch), void (*)(const u8*, const float*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::profile_gemv_spark), prod::KernelPerf (*)(const u8*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::profile_gemv_oil4), prod::KernelPerf (*)(const u8*, const u16*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(&prod::profile_gemv_oil8), prod::KernelPerf (*)(const u8*, const float*, float, const float*, float*, int, int, int)>);
static_assert(same<decltype(prod::KernelPerf::cycles), uint64_t> && same<decltype(prod::KernelPerf::bytes_read), uint64_t> &&
              same<decltype(prod::KernelPerf::bytes_written), uint64_t> && same<decltype(prod::KernelPerf::gflops), double>);
// include/oil/oil_engines.h:43-49,72-78,150-151,103,123,167,183
namespace eng = oil::engines;
using oil::Tensor;
static_assert(same<decltype(&eng::OIL8Engine::quant_gemm), Tensor (eng::OIL8Engine::*)(const Tensor&, const u8*, int64_t, int64_t, int64_t) const>);
static_assert(same<decltype(&eng::OIL4Engine::quant_gemm), Tensor (eng::OIL4Engine::*)(const Tensor&, const u8*, int64_t, int64_t, int64_t) const>);
static_assert(same<decltype(&eng::OIL2Engine::quant_gemm), Tensor (eng::OIL2Engine::*)(const Tensor&, const u8*, int64_t, int64_t, int64_t) const>);
static_assert(same<decltype(&eng::OIL8Engine::dequant_tensor), Tensor (eng::OIL8Engine::*)(const u8*, int64_t) const>);
static_assert(same<decltype(&eng::OIL4Engine::dequant_tensor), Tensor (eng::OIL4Engine::*)(const u8*, int64_t) const>);
static_assert(same<decltype(&eng::OIL2Engine::dequant_tensor), Tensor (eng::OIL2Engine::*)(const u8*, int64_t) const>);
static_assert(same<decltype(&eng::OIL8Engine::dequantize_per_block), void (eng::OIL8Engine::*)(const u8*, const float*, int64_t, int64_t, float*) const>);
static_assert(same<decltype(&eng::OIL4Engine::dequantize_per_block), void (eng::OIL4Engine::*)(const u8*, const float*, int64_t, int64_t, float*) const>);
static_assert(same<decltype(&eng::Oil1Engine::quant_gemm), Tensor (eng::Oil1Engine::*)(const Tensor&, const Tensor&, float, int64_t, int64_t, int64_t)>);
static_assert(same<decltype(&eng::SparkEngine::quant_gemm), Tensor (eng::SparkEngine::*)(const Tensor&, const Tensor&, const Tensor&, int64_t, int64_t, int64_t)>);
static_assert(same<decltype(&eng::OIL16Engine::quant_gemm), Tensor (eng::OIL16Engine::*)(const Tensor&, const Tensor&, int64_t, int64_t, int64_t) const>);
static_assert(same<decltype(&eng::OIL32Engine::quant_gemm), Tensor (eng::OIL32Engine::*)(const Tensor&, const Tensor&, int64_t, int64_t, int64_t) const>);
// include/oil/kv_cache_oil4.h:26-83: the methods gfx950::OIL4KVCache mirrors, where their types do not involve Tensor
static_assert(same<decltype(&oil::OIL4KVCache::quantize_block_oil4), void (*)(const float*, u8*, u16*, int64_t)>);
static_assert(same<decltype(&oil::OIL4KVCache::dequantize_block_oil4), void (*)(const u8*, const u16*, float*, int64_t)>);
static_assert(same<decltype(&oil::OIL4KVCache::context_len), int (oil::OIL4KVCache::*)() const>);
static_assert(same<decltype(&oil::OIL4KVCache::size_bytes), size_t (oil::OIL4KVCache::*)() const>);
static_assert(same<decltype(&oil::OIL4KVCache::clear), void (oil::OIL4KVCache::*)()>);
static_assert(same<decltype(&oil::OIL4KVCache::resize), void (oil::OIL4KVCache::*)(int64_t)>);
static_assert(same<decltype(&oil::gfx950::OIL4KVCache::context_len), int (oil::gfx950::OIL4KVCache::*)() const>);
static_assert(same<decltype(&oil::gfx950::OIL4KVCache::size_bytes), size_t (oil::gfx950::OIL4KVCache::*)() const>);
static_assert(same<decltype(&oil::gfx950::OIL4KVCache::quantize_block_oil4), decltype(&oil::OIL4KVCache::quantize_block_oil4)>);
static_assert(same<decltype(&oil::gfx950::OIL4KVCache::dequantize_block_oil4), decltype(&oil::OIL4KVCache::dequantize_block_oil4)>);
// include/oil/backend.h:49-80
namespace be = oil::backend;
static_assert(same<decltype(&be::ComputeBackend::gemm), void (be::ComputeBackend::*)(float, const Tensor&, const Tensor&, float, Tensor&)>);
static_assert(same<decltype(&be::ComputeBackend::gemv), void (be::ComputeBackend::*)(float, const Tensor&, const Tensor&, float, Tensor&)>);
static_assert(same<decltype(&be::ComputeBackend::create), be::ComputeBackend* (*)(const be::BackendConfig&)>);
static_assert(same<decltype(&be::probe_hardware), be::HardwareProfile (*)()>);
static_assert(same<decltype(&be::select_optimal_backend), be::BackendConfig (*)(const be::HardwareProfile&, int64_t)>);
// oil::Format values the C ABI's format ids rely on (include/oil/types.h:19-35)
static_assert((int)oil::Format::OIL1 == 0 && (int)oil::Format::SPARK_Q0 == 1 && (int)oil::Format::OIL2 == 2 &&
              (int)oil::Format::OIL4 == 3 && (int)oil::Format::OIL8 == 4 && (int)oil::Format::OIL16 == 5 &&
              (int)oil::Format::OIL32 == 6 && (int)oil::Format::OIL1_GRP == 7 && (int)oil::Format::SPARK_SPARSE_GRP == 14);
}  // namespace

int main() { return 0; }
