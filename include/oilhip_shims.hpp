// oilhip_shims.hpp -- C++20 drop-in layer over the C ABI (oilhip.h): the reference's own
// entry points for this path, same namespaces, names, argument meaning and error
// behaviour, taking host pointers like the reference does.  Each shim uploads its
// operands, runs the HIP kernel and copies the result back; there is no CPU fallback
// (a missing GPU or a failed launch throws oil::Error).
//
// Built inside the reference tree the shim sources include the reference's own headers
// (oil/types.h ...) so the signatures are the reference's by construction; built
// stand-alone they use the minimal declarations below.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#if __has_include("oil/types.h")
// Inside the reference tree: the reference's own declarations are the interface, and the shim sources define them.
#define OILHIP_REFERENCE_TREE 1
#include "oil/types.h"
#include "oil/block_codec.h"
#include "oil/kernel.h"
#include "oil/kernel_production.h"
#else
namespace oil {
// include/oil/types.h:19-35 (values pinned by tests/test_format.cpp:183-186)
enum class Format : uint8_t {
    OIL1 = 0, SPARK_Q0 = 1, OIL2 = 2, OIL4 = 3, OIL8 = 4, OIL16 = 5, OIL32 = 6, OIL1_GRP = 7,
    SPARK_Q0_GRP = 8, OIL2_GRP = 9, OIL4_GRP = 10, OIL8_GRP = 11, OIL16_GRP = 12,
    SPARK_SPARSE = 13, SPARK_SPARSE_GRP = 14,
};
// include/oil/types.h:184-187
class Error : public std::runtime_error {
public:
    explicit Error(const std::string& msg) : std::runtime_error(msg) {}
};

// include/oil/block_codec.h:55-63
bool quantize_block_all(Format fmt, const float* w, int n, std::vector<uint8_t>& indices, std::vector<uint8_t>& codebook);
void dequantize_block_all(Format fmt, const uint8_t* indices, size_t idx_bytes, const uint8_t* codebook,
                          size_t cb_bytes, uint32_t nw, float* out);

namespace kernel {
// include/oil/kernel.h:24-32
void oil8_gemm(const uint8_t* indices, const float* codebook, const float* activations, float* output, int M, int N, int K);
void oil4_gemm(const uint8_t* packed_indices, const uint16_t* codebook, const float* activations, float* output, int M, int N, int K);
}  // namespace kernel

namespace adapters::prod {
// include/oil/kernel_production.h:19-52; detect_cpu_isa() keeps its name, 950 = the gfx950 device path
int detect_cpu_isa();
void gemv_spark_tiled(const uint8_t* packed_w, float scale, const float* x, float* y, int M, int K, int tile_m = 32);
void gemv_oil4_tiled(const uint8_t* packed_indices, const uint16_t* codebook, float scale, const float* x, float* y, int M, int K, int tile_m = 32);
void gemv_oil8_tiled(const uint8_t* indices, const float* codebook, float scale, const float* x, float* y, int M, int K, int tile_m = 32);
void gemv_spark_batch(const uint8_t* packed_w, float scale, const float* X, float* Y, int M, int N, int K);
void gemv_oil4_batch(const uint8_t* packed_indices, const uint16_t* codebook, float scale, const float* X, float* Y, int M, int N, int K);
void gemv_oil8_batch(const uint8_t* indices, const float* codebook, float scale, const float* X, float* Y, int M, int N, int K);
// include/oil/kernel_production.h:68-82.  `cycles` is the time per launch in shader clocks at the device's peak
// frequency (the reference reads the CPU's timestamp counter); the byte counts and gflops follow the reference's
// formulas (src/kernel_production.cpp:433-485).
struct KernelPerf {
    uint64_t cycles = 0;
    uint64_t bytes_read = 0;
    uint64_t bytes_written = 0;
    double   gflops = 0.0;
};
KernelPerf profile_gemv_spark(const uint8_t* packed_w, float scale, const float* x, float* y, int M, int K, int repeats = 100);
KernelPerf profile_gemv_oil4(const uint8_t* packed_indices, const uint16_t* codebook, float scale, const float* x, float* y, int M, int K, int repeats = 100);
KernelPerf profile_gemv_oil8(const uint8_t* indices, const float* codebook, float scale, const float* x, float* y, int M, int K, int repeats = 100);
}  // namespace adapters::prod
}  // namespace oil
#endif

namespace oil {

namespace gfx950 {

// Body of OIL{8,4,2}Engine::quant_gemm (include/oil/oil_engines.h:49,78,151) on host pointers:
// C[m*N+n] = sum_k A[m*K+k] * codebook[code(k*N+n)].
void engine_quant_gemm(int bits, const float* a, const uint8_t* b_idx, const float* codebook, float* c,
                       int64_t M, int64_t N, int64_t K);
// Bodies of OIL{8,4,2}Engine::dequant_tensor (oil_engines.h:48,77,150; scales == nullptr: n packed codes ->
// codebook values) and of OIL8Engine / OIL4Engine::dequantize_per_block (:43-44, :72-73; one index byte per weight,
// OIL8: one scale per block, OIL4: {center, half_range} per block).
void engine_dequant(int bits, const uint8_t* indices, const float* codebook, int64_t n, const float* scales,
                    int64_t block_size, float* out);
// Bodies of the engines whose B operand is not a codebook index, [K][N] flat layout: kind 1 Oil1Engine::quant_gemm
// (oil_engines.h:123; b = one float per 32 flat positions), 3 SparkEngine::quant_gemm (:103; b = 2-bit codes, scales[flat /
// block_size]), 16 OIL16Engine::quant_gemm (:167; b = FP16 bits), 32 OIL32Engine::quant_gemm (:183; b = FP32).
void engine_dense_gemm(int kind, const float* a, const void* b, const float* scales, int64_t block_size, float* c,
                       int64_t M, int64_t N, int64_t K);
// Bodies of tl1_gemm (kind 1) / tl2_gemm (kind 2) (include/oil/kernel.h:11-18) on host pointers: weights = one packed
// row of K ternary codes per (m, n), activations [N][K], output [M][N].
void tl_gemm(int kind, const uint8_t* weights, const float* activations, float* output, int M, int N, int K);

// One block as the .oil file stores it (OILWriter::write_block, src/oil_format.cpp:219-233).
struct BlockRef {
    Format format;
    const uint8_t* codebook; uint32_t cb_bytes;
    const uint8_t* indices;  uint32_t idx_bytes;
    uint32_t num_weights;
};

// A tensor of .oil blocks resident in HBM: what Qwen35Engine::Th + OILReader give the
// reference's gemm (include/oil/qwen35_engine.h:29,38).  gemm() is that function:
// Y[b*rows + r] = sum_c W[r][c] * X[b*cols + c], host pointers, FP32, any B >= 1.
// Batches of at least `min_batch` activation rows go through the bf16 matrix-core prefill kernel (oilhip_gemm_f32:
// X rounded once to bf16: relative L2 error <= 2e-3 against the FP32 contraction over the rounded activations, about
// 2.4e-3 against the one over the FP32 activations for Gaussian data) instead of the FP32 decode kernels (<= 1e-5).  0 (the default) keeps every batch on the FP32 path, as the reference computes it; 32 or more is where
// the prefill kernel is faster.  Process-wide; Qwen35Engine::prefill calls gemm with up to 512 rows
// (src/adapters/tools/qwen35_engine.cpp:12,630-753).
void set_prefill_min_batch(int min_batch);
int prefill_min_batch();
// DeviceTensor::gemm keeps the device buffers its host-pointer arguments pass through between calls (a pair per
// thread that is inside gemm at once, grown on demand); this returns them to the driver.
void release_staging();

class DeviceTensor {
public:
    DeviceTensor(const std::vector<BlockRef>& blocks, uint64_t rows, uint64_t cols);
    // raw block records [nw][cb_bytes][cb][idx_bytes][idx] back to back + one format id per block
    DeviceTensor(const uint8_t* records, uint64_t record_bytes, const uint8_t* formats, uint32_t nblocks,
                 uint64_t rows, uint64_t cols);
    ~DeviceTensor();
    DeviceTensor(const DeviceTensor&) = delete;
    DeviceTensor& operator=(const DeviceTensor&) = delete;
    void gemm(const float* X, float* Y, int B) const;       // Y[B][rows] = X[B][cols] . W^T (Qwen35Engine::gemm); see set_prefill_min_batch
    void dequantize(float* out) const;                    // rows*cols floats, bit-exact with dequantize_block_all
    uint64_t rows() const { return rows_; }
    uint64_t cols() const { return cols_; }
    uint64_t payload_bytes() const;
private:
    void* handle_ = nullptr;
    uint64_t rows_ = 0, cols_ = 0;
};

// oil::OIL4KVCache (include/oil/kv_cache_oil4.h:26-83) with its state in HBM.  Same methods and meaning; where the
// reference passes oil::Tensor, host pointers over the same memory: k / v of append are [seq_len][heads * dim] floats
// (what the reference reads from its [1, heads, seq, dim] tensors, src/kv_cache_oil4.cpp:213-229), get_range returns
// the two [len][heads * dim] arrays.  Errors throw oil::Error.
class OIL4KVCache {
public:
    OIL4KVCache(int num_layers, int64_t max_seq_len, int64_t num_heads, int64_t head_dim, int64_t block_size = 64);
    ~OIL4KVCache();
    OIL4KVCache(const OIL4KVCache&) = delete;
    OIL4KVCache& operator=(const OIL4KVCache&) = delete;
    void append(int layer, const float* k, const float* v, int64_t seq_len);
    std::pair<std::vector<float>, std::vector<float>> get_range(int layer, int64_t start, int64_t end) const;
    std::pair<std::vector<float>, std::vector<float>> get_all(int layer) const;
    int context_len() const;
    int64_t max_seq_len() const { return max_seq_len_; }
    int64_t block_size() const;
    int num_layers() const { return num_layers_; }
    int64_t num_heads() const { return num_heads_; }
    int64_t head_dim() const { return head_dim_; }
    size_t size_bytes() const;
    size_t size_bytes_fp32_equivalent() const;
    double compression_ratio() const;
    void clear();
    void resize(int64_t new_max_seq_len);
    // n <= 128 values; indices one code per byte
    static void quantize_block_oil4(const float* src, uint8_t* indices, uint16_t* codebook_fp16, int64_t n);
    static void dequantize_block_oil4(const uint8_t* indices, const uint16_t* codebook_fp16, float* dst, int64_t n);
    static constexpr int OIL4_CODEBOOK_SIZE = 16;
private:
    void* handle_ = nullptr;
    int num_layers_ = 0;
    int64_t max_seq_len_ = 0, num_heads_ = 0, head_dim_ = 0;
};

// backend::probe_hardware / select_optimal_backend hook (include/oil/backend.h:98-139):
// true when a gfx950 device is usable; fills name and HBM size when given.
bool probe(std::string* name = nullptr, uint64_t* hbm_bytes = nullptr, int* compute_units = nullptr);

}  // namespace gfx950
}  // namespace oil
