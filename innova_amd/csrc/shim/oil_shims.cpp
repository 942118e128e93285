// oil_shims.cpp -- host-pointer C++ shims over the C ABI (see include/oilhip_shims.hpp).
#include "../../../include/oilhip_shims.hpp"

#include <atomic>
#include <mutex>
#include <vector>
#include <hip/hip_runtime.h>

#include <cstring>

#include <algorithm>

#include "../../../include/oilhip.h"

namespace {

[[noreturn]] void raise(const char* what) {
    throw oil::Error(std::string(what) + ": " + oilhip_last_error());
}
void ok(int rc, const char* what) {
    if (rc != OILHIP_OK) raise(what);
}
void hip_ok(hipError_t e, const char* what) {
    if (e != hipSuccess) throw oil::Error(std::string(what) + ": " + hipGetErrorString(e));
}

// Device buffer holding a copy of a host range (or an output range).
template <class T>
class Dev {
public:
    Dev(const T* host, size_t n) : n_(n) {
        if (n_ == 0) return;
        hip_ok(hipMalloc(&p_, n_ * sizeof(T)), "hipMalloc");
        if (host) hip_ok(hipMemcpy(p_, host, n_ * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy H2D");
    }
    ~Dev() { if (p_) (void)hipFree(p_); }
    Dev(const Dev&) = delete;
    Dev& operator=(const Dev&) = delete;
    T* get() const { return p_; }
    void to_host(T* host) const {
        if (n_) hip_ok(hipMemcpy(host, p_, n_ * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy D2H");
    }
private:
    T* p_ = nullptr;
    size_t n_;
};

size_t sz(long long v) { return v < 0 ? 0 : (size_t)v; }

// Device staging for DeviceTensor::gemm: the reference hands over host pointers on every call (seven projections per
// layer and token), so its activations and outputs pass through a pair of device buffers that are kept between
// calls instead of a hipMalloc / hipFree pair per call (hipFree waits for the device).  A call leases a pair from a
// small pool (one pair per thread that is inside gemm at the same moment); buffers grow, never shrink, and are
// returned to the driver by release_staging().
constexpr size_t kPinnedFloats = 64 * 1024;   // small transfers (a decode step's activations and outputs) go through pinned memory
struct Stage { float* x = nullptr; size_t nx = 0; float* y = nullptr; size_t ny = 0; float* hx = nullptr; float* hy = nullptr; };
std::mutex g_stage_mu;
std::vector<Stage> g_stage_free;

class StageLease {
public:
    StageLease(size_t nx, size_t ny) {
        {
            std::lock_guard<std::mutex> lk(g_stage_mu);
            if (!g_stage_free.empty()) { s_ = g_stage_free.back(); g_stage_free.pop_back(); }
        }
        grow(s_.x, s_.nx, nx);
        grow(s_.y, s_.ny, ny);
        if (!s_.hx) {                                                  // pinned host memory is allocated, never registered
            hip_ok(hipHostMalloc(reinterpret_cast<void**>(&s_.hx), kPinnedFloats * sizeof(float), hipHostMallocDefault), "hipHostMalloc");
            hip_ok(hipHostMalloc(reinterpret_cast<void**>(&s_.hy), kPinnedFloats * sizeof(float), hipHostMallocDefault), "hipHostMalloc");
        }
    }
    ~StageLease() {
        std::lock_guard<std::mutex> lk(g_stage_mu);
        g_stage_free.push_back(s_);
    }
    StageLease(const StageLease&) = delete;
    StageLease& operator=(const StageLease&) = delete;
    float* x() const { return s_.x; }
    float* y() const { return s_.y; }
    float* hx() const { return s_.hx; }
    float* hy() const { return s_.hy; }
private:
    static void grow(float*& p, size_t& have, size_t want) {
        if (want <= have) return;
        if (p) { (void)hipFree(p); p = nullptr; have = 0; }
        hip_ok(hipMalloc(&p, want * sizeof(float)), "hipMalloc");
        have = want;
    }
    Stage s_;
};

}  // namespace

namespace oil {

bool quantize_block_all(Format fmt, const float* w, int n, std::vector<uint8_t>& indices, std::vector<uint8_t>& codebook) {
    indices.clear();
    codebook.clear();
    if (!w || n <= 0 || (int)fmt > 14) return false;                  // block_codec.cpp:370,571-572
    const size_t bound = oilhip_payload_bound((int)fmt, n);
    indices.resize(bound ? bound : 1);
    codebook.resize(2 * (((size_t)n + 31) / 32) + 2);
    size_t il = 0, cl = 0;
    if (oilhip_quantize_block((int)fmt, w, n, indices.data(), indices.size(), &il, codebook.data(), codebook.size(), &cl) != OILHIP_OK)
        return false;
    indices.resize(il);
    codebook.resize(cl);
    return true;
}

void dequantize_block_all(Format fmt, const uint8_t* indices, size_t idx_bytes, const uint8_t* codebook,
                          size_t cb_bytes, uint32_t nw, float* out) {
    if (!out || nw == 0) return;                                       // block_codec.cpp:580
    if ((int)fmt > 14 || nw > (1u << 24) || cb_bytes > 0xFFFF) {       // unhandled input decodes to zeros (:717-718)
        std::memset(out, 0, sizeof(float) * nw);
        return;
    }
    const gfx950::BlockRef b{fmt, codebook, (uint32_t)cb_bytes, indices, (uint32_t)idx_bytes, nw};
    gfx950::DeviceTensor t(std::vector<gfx950::BlockRef>{b}, 1, nw);
    t.dequantize(out);
}

namespace kernel {

void oil8_gemm(const uint8_t* indices, const float* codebook, const float* activations, float* output, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    Dev<uint8_t> i(indices, sz(N) * sz(K));
    Dev<float> c(codebook, 256), a(activations, sz(M) * sz(K)), o(nullptr, sz(M) * sz(N));
    ok(oilhip_flat_oil8_gemm(i.get(), c.get(), a.get(), o.get(), M, N, K, nullptr), "oil8_gemm");
    o.to_host(output);
}

void oil4_gemm(const uint8_t* packed, const uint16_t* codebook, const float* activations, float* output, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    Dev<uint8_t> i(packed, (sz(M) * sz(N) * sz(K) + 1) / 2);
    Dev<uint16_t> c(codebook, 16);
    Dev<float> a(activations, sz(N) * sz(K)), o(nullptr, sz(M) * sz(N));
    ok(oilhip_flat_oil4_gemm(i.get(), c.get(), a.get(), o.get(), M, N, K, nullptr), "oil4_gemm");
    o.to_host(output);
}

}  // namespace kernel

namespace adapters::prod {

int detect_cpu_isa() {
    int gfx = 0;
    return oilhip_probe(&gfx, nullptr, nullptr, nullptr, 0) == OILHIP_OK ? gfx : 0;
}

void gemv_spark_batch(const uint8_t* w, float scale, const float* X, float* Y, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    Dev<uint8_t> dw(w, sz(M) * ((sz(K) + 3) / 4));
    Dev<float> x(X, sz(N) * sz(K)), y(nullptr, sz(N) * sz(M));
    ok(oilhip_prod_gemv_spark(dw.get(), scale, x.get(), y.get(), M, K, N, nullptr), "gemv_spark");
    y.to_host(Y);
}
void gemv_oil4_batch(const uint8_t* w, const uint16_t* cb, float scale, const float* X, float* Y, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    Dev<uint8_t> dw(w, sz(M) * ((sz(K) + 1) / 2));
    Dev<uint16_t> c(cb, 16);
    Dev<float> x(X, sz(N) * sz(K)), y(nullptr, sz(N) * sz(M));
    ok(oilhip_prod_gemv_oil4(dw.get(), c.get(), scale, x.get(), y.get(), M, K, N, nullptr), "gemv_oil4");
    y.to_host(Y);
}
void gemv_oil8_batch(const uint8_t* w, const float* cb, float scale, const float* X, float* Y, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    Dev<uint8_t> dw(w, sz(M) * sz(K));
    Dev<float> c(cb, 256), x(X, sz(N) * sz(K)), y(nullptr, sz(N) * sz(M));
    ok(oilhip_prod_gemv_oil8(dw.get(), c.get(), scale, x.get(), y.get(), M, K, N, nullptr), "gemv_oil8");
    y.to_host(Y);
}
void gemv_spark_tiled(const uint8_t* w, float scale, const float* x, float* y, int M, int K, int) {
    gemv_spark_batch(w, scale, x, y, M, 1, K);
}
void gemv_oil4_tiled(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y, int M, int K, int) {
    gemv_oil4_batch(w, cb, scale, x, y, M, 1, K);
}
void gemv_oil8_tiled(const uint8_t* w, const float* cb, float scale, const float* x, float* y, int M, int K, int) {
    gemv_oil8_batch(w, cb, scale, x, y, M, 1, K);
}


namespace {
KernelPerf profile(int kind, const uint8_t* w, size_t w_bytes, const void* cb, size_t cb_bytes, float scale,
                   const float* x, float* y, int M, int K, int repeats) {
    KernelPerf p;
    if (M <= 0) return p;
    Dev<uint8_t> dw(w, w_bytes), dc(static_cast<const uint8_t*>(cb), cb_bytes);
    Dev<float> dx(x, sz(K)), dy(nullptr, sz(M));
    oilhip_kernel_perf_t r{};
    ok(oilhip_profile_gemv(kind, dw.get(), dc.get(), scale, dx.get(), dy.get(), M, K, repeats, &r, nullptr), "profile_gemv");
    dy.to_host(y);
    p.cycles = r.cycles;
    p.bytes_read = r.bytes_read;
    p.bytes_written = r.bytes_written;
    p.gflops = r.gflops;
    return p;
}
}  // namespace

KernelPerf profile_gemv_spark(const uint8_t* w, float scale, const float* x, float* y, int M, int K, int repeats) {
    return profile(0, w, sz(M) * ((sz(K) + 3) / 4), nullptr, 0, scale, x, y, M, K, repeats);
}
KernelPerf profile_gemv_oil4(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y, int M, int K, int repeats) {
    return profile(4, w, sz(M) * ((sz(K) + 1) / 2), cb, 32, scale, x, y, M, K, repeats);
}
KernelPerf profile_gemv_oil8(const uint8_t* w, const float* cb, float scale, const float* x, float* y, int M, int K, int repeats) {
    return profile(8, w, sz(M) * sz(K), cb, 1024, scale, x, y, M, K, repeats);
}

}  // namespace adapters::prod

namespace gfx950 {

void engine_dequant(int bits, const uint8_t* indices, const float* codebook, int64_t n, const float* scales,
                    int64_t block_size, float* out) {
    if (n <= 0) return;
    if (bits != 2 && bits != 4 && bits != 8) throw Error("engine_dequant: bits must be 2, 4 or 8");
    const size_t idx_bytes = scales ? sz(n) : (sz(n) * (size_t)bits + 7) / 8;
    const size_t nblocks = scales && block_size > 0 ? (sz(n) + sz(block_size) - 1) / sz(block_size) : 0;
    Dev<uint8_t> di(indices, idx_bytes);
    Dev<float> dc(codebook, (size_t)1 << bits), ds(scales, nblocks * (bits == 4 ? 2 : 1)), dout(nullptr, sz(n));
    ok(oilhip_engine_dequant(bits, di.get(), dc.get(), n, scales ? ds.get() : nullptr, block_size, dout.get(), nullptr),
       "engine_dequant");
    dout.to_host(out);
}

void engine_dense_gemm(int kind, const float* a, const void* b, const float* scales, int64_t block_size, float* c,
                       int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0) return;
    const size_t flat = sz(K) * sz(N);
    size_t b_bytes = 0, nscales = 0;
    switch (kind) {
        case 1: b_bytes = ((flat + 31) / 32) * 4; break;
        case 3:
            if (block_size <= 0) throw Error("engine_dense_gemm: the SPARK engine needs a block size");
            b_bytes = (flat + 3) / 4;
            nscales = (flat + sz(block_size) - 1) / sz(block_size);
            break;
        case 16: b_bytes = flat * 2; break;
        case 32: b_bytes = flat * 4; break;
        default: throw Error("engine_dense_gemm: kind must be 1, 3, 16 or 32");
    }
    Dev<float> da(a, sz(M) * sz(K)), ds(scales, nscales), out(nullptr, sz(M) * sz(N));
    Dev<uint8_t> db(static_cast<const uint8_t*>(b), b_bytes);
    ok(oilhip_engine_dense_gemm(kind, da.get(), db.get(), nscales ? ds.get() : nullptr, block_size, out.get(), M, N, K, nullptr),
       "engine_dense_gemm");
    out.to_host(c);
}

void tl_gemm(int kind, const uint8_t* weights, const float* activations, float* output, int M, int N, int K) {
    if (M <= 0 || N <= 0) return;
    const size_t row = kind == 1 ? (sz(K) + 3) / 4 : ((sz(K) + 11) / 12) * 3;
    Dev<uint8_t> dw(weights, sz(M) * sz(N) * row);
    Dev<float> da(activations, sz(N) * sz(K)), dout(nullptr, sz(M) * sz(N));
    ok(oilhip_tl_gemm(kind, dw.get(), da.get(), dout.get(), M, N, K, nullptr), "tl_gemm");
    dout.to_host(output);
}

void engine_quant_gemm(int bits, const float* a, const uint8_t* b_idx, const float* codebook, float* c,
                       int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0) return;
    if (bits != 2 && bits != 4 && bits != 8) throw Error("engine_quant_gemm: bits must be 2, 4 or 8");
    Dev<float> da(a, sz(M) * sz(K)), dc(codebook, (size_t)1 << bits), out(nullptr, sz(M) * sz(N));
    Dev<uint8_t> db(b_idx, (sz(K) * sz(N) * (size_t)bits + 7) / 8);
    ok(oilhip_engine_quant_gemm(bits, da.get(), db.get(), dc.get(), out.get(), M, N, K, nullptr), "quant_gemm");
    out.to_host(c);
}

DeviceTensor::DeviceTensor(const std::vector<BlockRef>& blocks, uint64_t rows, uint64_t cols) : rows_(rows), cols_(cols) {
    std::vector<uint8_t> pay;
    std::vector<oilhip_block_t> desc(blocks.size());
    for (size_t b = 0; b < blocks.size(); ++b) {
        const BlockRef& s = blocks[b];
        desc[b] = oilhip_block_t{pay.size(), pay.size() + s.cb_bytes, s.cb_bytes, s.idx_bytes, s.num_weights, (uint8_t)s.format, {0, 0, 0}};
        if (s.cb_bytes) pay.insert(pay.end(), s.codebook, s.codebook + s.cb_bytes);
        if (s.idx_bytes) pay.insert(pay.end(), s.indices, s.indices + s.idx_bytes);
    }
    oilhip_weights* h = nullptr;
    ok(oilhip_weights_create(pay.data(), pay.size(), desc.data(), (uint32_t)desc.size(), rows, cols, &h), "DeviceTensor");
    handle_ = h;
}

DeviceTensor::DeviceTensor(const uint8_t* records, uint64_t record_bytes, const uint8_t* formats, uint32_t nblocks,
                           uint64_t rows, uint64_t cols) : rows_(rows), cols_(cols) {
    oilhip_weights* h = nullptr;
    ok(oilhip_weights_create_from_records(records, record_bytes, formats, nblocks, rows, cols, &h), "DeviceTensor");
    handle_ = h;
}

DeviceTensor::~DeviceTensor() { oilhip_weights_destroy(static_cast<oilhip_weights*>(handle_)); }

static std::atomic<int> g_prefill_min_batch{0};
void set_prefill_min_batch(int min_batch) { g_prefill_min_batch.store(min_batch < 0 ? 0 : min_batch, std::memory_order_relaxed); }
int prefill_min_batch() { return g_prefill_min_batch.load(std::memory_order_relaxed); }

void release_staging() {
    std::lock_guard<std::mutex> lk(g_stage_mu);
    for (Stage& s : g_stage_free) {
        if (s.x) (void)hipFree(s.x);
        if (s.y) (void)hipFree(s.y);
        if (s.hx) (void)hipHostFree(s.hx);
        if (s.hy) (void)hipHostFree(s.hy);
    }
    g_stage_free.clear();
}

void DeviceTensor::gemm(const float* X, float* Y, int B) const {
    if (B <= 0) return;
    const size_t nx = (size_t)B * cols_, ny = (size_t)B * rows_;
    StageLease st(nx, ny);
    // a decode step's few KB travel through pinned memory with asynchronous copies and one wait at the end; large
    // batches are copied straight from and to the caller's memory
    const bool small = nx <= kPinnedFloats && ny <= kPinnedFloats;
    if (small) {
        std::memcpy(st.hx(), X, nx * sizeof(float));
        hip_ok(hipMemcpyAsync(st.x(), st.hx(), nx * sizeof(float), hipMemcpyHostToDevice, nullptr), "hipMemcpyAsync H2D");
    } else {
        hip_ok(hipMemcpy(st.x(), X, nx * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy H2D");
    }
    const int pmin = prefill_min_batch();
    if (pmin > 0 && B >= pmin) ok(oilhip_gemm_f32(static_cast<oilhip_weights*>(handle_), st.x(), st.y(), B, nullptr), "gemm (prefill)");
    else ok(oilhip_gemv_f32(static_cast<oilhip_weights*>(handle_), st.x(), st.y(), B, nullptr), "gemm");
    if (small) {
        hip_ok(hipMemcpyAsync(st.hy(), st.y(), ny * sizeof(float), hipMemcpyDeviceToHost, nullptr), "hipMemcpyAsync D2H");
        hip_ok(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
        std::memcpy(Y, st.hy(), ny * sizeof(float));
    } else {
        hip_ok(hipMemcpy(Y, st.y(), ny * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy D2H");
    }
}

void DeviceTensor::dequantize(float* out) const {
    Dev<float> o(nullptr, (size_t)rows_ * cols_);
    ok(oilhip_dequant_f32(static_cast<oilhip_weights*>(handle_), o.get(), nullptr), "dequantize");
    o.to_host(out);
}

uint64_t DeviceTensor::payload_bytes() const {
    uint64_t v = 0;
    ok(oilhip_weights_info(static_cast<oilhip_weights*>(handle_), nullptr, nullptr, nullptr, &v, nullptr), "info");
    return v;
}

// ---- OIL4KVCache (include/oil/kv_cache_oil4.h:26-83)
OIL4KVCache::OIL4KVCache(int num_layers, int64_t max_seq_len, int64_t num_heads, int64_t head_dim, int64_t block_size)
    : num_layers_(num_layers), max_seq_len_(max_seq_len), num_heads_(num_heads), head_dim_(head_dim) {
    oilhip_kv* h = nullptr;
    ok(oilhip_kv_create(num_layers, max_seq_len, num_heads, head_dim, block_size, &h), "OIL4KVCache");
    handle_ = h;
}
OIL4KVCache::~OIL4KVCache() { oilhip_kv_destroy(static_cast<oilhip_kv*>(handle_)); }

void OIL4KVCache::append(int layer, const float* k, const float* v, int64_t seq_len) {
    const size_t n = sz(seq_len) * sz(num_heads_ * head_dim_);
    Dev<float> dk(k, n), dv(v, n);
    ok(oilhip_kv_append(static_cast<oilhip_kv*>(handle_), layer, dk.get(), dv.get(), seq_len, nullptr), "OIL4KVCache::append");
    hip_ok(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
}

std::pair<std::vector<float>, std::vector<float>> OIL4KVCache::get_range(int layer, int64_t start, int64_t end) const {
    const int64_t want = std::max<int64_t>(0, std::min(end, max_seq_len_) - start);
    const size_t per_token = sz(num_heads_ * head_dim_);
    Dev<float> dk(nullptr, sz(want) * per_token), dv(nullptr, sz(want) * per_token);
    int64_t len = 0;
    ok(oilhip_kv_get_range(static_cast<const oilhip_kv*>(handle_), layer, start, end, dk.get(), dv.get(), &len, nullptr),
       "OIL4KVCache::get_range");
    std::pair<std::vector<float>, std::vector<float>> out;
    out.first.resize(sz(len) * per_token);
    out.second.resize(sz(len) * per_token);
    if (len > 0) {
        hip_ok(hipMemcpy(out.first.data(), dk.get(), out.first.size() * 4, hipMemcpyDeviceToHost), "hipMemcpy D2H");
        hip_ok(hipMemcpy(out.second.data(), dv.get(), out.second.size() * 4, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    }
    return out;
}
std::pair<std::vector<float>, std::vector<float>> OIL4KVCache::get_all(int layer) const { return get_range(layer, 0, max_seq_len_); }

int OIL4KVCache::context_len() const {
    int v = 0;
    ok(oilhip_kv_info(static_cast<const oilhip_kv*>(handle_), &v, nullptr, nullptr, nullptr), "kv_info");
    return v;
}
int64_t OIL4KVCache::block_size() const {
    int64_t v = 0;
    ok(oilhip_kv_info(static_cast<const oilhip_kv*>(handle_), nullptr, &v, nullptr, nullptr), "kv_info");
    return v;
}
size_t OIL4KVCache::size_bytes() const {
    uint64_t v = 0;
    ok(oilhip_kv_info(static_cast<const oilhip_kv*>(handle_), nullptr, nullptr, &v, nullptr), "kv_info");
    return (size_t)v;
}
size_t OIL4KVCache::size_bytes_fp32_equivalent() const {
    uint64_t v = 0;
    ok(oilhip_kv_info(static_cast<const oilhip_kv*>(handle_), nullptr, nullptr, nullptr, &v), "kv_info");
    return (size_t)v;
}
double OIL4KVCache::compression_ratio() const {
    const size_t q = size_bytes();
    return q == 0 ? 0.0 : (double)size_bytes_fp32_equivalent() / (double)q;
}
void OIL4KVCache::clear() {
    ok(oilhip_kv_clear(static_cast<oilhip_kv*>(handle_), nullptr), "OIL4KVCache::clear");
    hip_ok(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
}
void OIL4KVCache::resize(int64_t new_max_seq_len) {
    ok(oilhip_kv_resize(static_cast<oilhip_kv*>(handle_), new_max_seq_len), "OIL4KVCache::resize");
    max_seq_len_ = new_max_seq_len;
}
void OIL4KVCache::quantize_block_oil4(const float* src, uint8_t* indices, uint16_t* codebook_fp16, int64_t n) {
    if (n <= 0) return;
    Dev<float> ds(src, sz(n));
    Dev<uint8_t> dc(nullptr, sz(n));
    Dev<uint16_t> db(nullptr, 16);
    ok(oilhip_kv_quantize_blocks(ds.get(), n, 1, dc.get(), db.get(), nullptr), "OIL4KVCache::quantize_block_oil4");
    dc.to_host(indices);
    db.to_host(codebook_fp16);
}
void OIL4KVCache::dequantize_block_oil4(const uint8_t* indices, const uint16_t* codebook_fp16, float* dst, int64_t n) {
    if (n <= 0) return;
    Dev<uint8_t> dc(indices, sz(n));
    Dev<uint16_t> db(codebook_fp16, 16);
    Dev<float> dd(nullptr, sz(n));
    ok(oilhip_kv_dequantize_blocks(dc.get(), db.get(), dd.get(), n, 1, nullptr), "OIL4KVCache::dequantize_block_oil4");
    dd.to_host(dst);
}

bool probe(std::string* name, uint64_t* hbm_bytes, int* compute_units) {
    char buf[256] = {0};
    int gfx = 0;
    if (oilhip_probe(&gfx, hbm_bytes, compute_units, buf, sizeof buf) != OILHIP_OK) return false;
    if (name) *name = buf;
    return gfx == 950;
}

}  // namespace gfx950
}  // namespace oil
