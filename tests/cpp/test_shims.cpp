// test_shims.cpp -- the C++ drop-in layer called the way the reference's own tests call
// its kernels (tests/test_kernel.cpp:82-103, tests/test_quant_engines.cpp:229-263,
// tests/test_block_codec.cpp), with results checked against brute-force double loops.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/oilhip_shims.hpp"

static int g_fail = 0, g_checks = 0;
#define CHECK(cond, ...) do { ++g_checks; if (!(cond)) { ++g_fail; std::printf("FAIL %s:%d: ", __FILE__, __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } } while (0)

static uint32_t g_state = 12345u;
static float frand() {   // the LCG of tests/test_quant_engines.cpp:298-308
    g_state = g_state * 1103515245u + 12345u;
    return ((float)((g_state >> 8) & 0xFFFF) / 65535.0f - 0.5f) * 2.0f;
}
static double rel_l2(const std::vector<float>& a, const std::vector<double>& b) {
    double num = 0, den = 0;
    for (size_t i = 0; i < a.size(); ++i) { num += (a[i] - b[i]) * (a[i] - b[i]); den += b[i] * b[i]; }
    return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}

int main() {
    using namespace oil;
    std::string name; uint64_t hbm = 0; int cus = 0;
    CHECK(gfx950::probe(&name, &hbm, &cus), "no gfx950 device");
    CHECK(adapters::prod::detect_cpu_isa() == 950, "detect_cpu_isa() should report the device path");
    std::printf("device: %s, %d CUs\n", name.c_str(), cus);

    {   // oil8_gemm: shape + finite (tests/test_kernel.cpp:82-103) and values
        const int M = 3, N = 50, K = 300;
        std::vector<uint8_t> idx((size_t)N * K); for (auto& v : idx) v = (uint8_t)(std::fabs(frand()) * 255);
        std::vector<float> cb(256), act((size_t)M * K), out((size_t)M * N, 0.f);
        for (auto& v : cb) v = frand() * 0.02f;
        for (auto& v : act) v = frand();
        kernel::oil8_gemm(idx.data(), cb.data(), act.data(), out.data(), M, N, K);
        std::vector<double> want((size_t)M * N, 0.0);
        for (int m = 0; m < M; ++m) for (int n = 0; n < N; ++n) for (int k = 0; k < K; ++k)
            want[m * N + n] += (double)cb[idx[(size_t)n * K + k]] * act[(size_t)m * K + k];
        bool finite = true; for (float v : out) finite &= std::isfinite(v);
        CHECK(finite, "oil8_gemm produced non-finite output");
        CHECK(rel_l2(out, want) <= 1e-5, "oil8_gemm rel-L2 %.3g", rel_l2(out, want));
    }
    {   // oil4_gemm: weights per (m,n) pair, activations per n (src/kernel_oil4.cpp:38-56)
        const int M = 2, N = 7, K = 64;
        std::vector<uint8_t> pk((size_t)M * N * K / 2); for (auto& v : pk) v = (uint8_t)(std::fabs(frand()) * 255);
        std::vector<uint16_t> cb16(16); for (int i = 0; i < 16; ++i) cb16[i] = (uint16_t)(0x3800 + 64 * i);   // 0.5 .. ~1
        std::vector<float> act((size_t)N * K), out((size_t)M * N);
        for (auto& v : act) v = frand();
        kernel::oil4_gemm(pk.data(), cb16.data(), act.data(), out.data(), M, N, K);
        std::vector<double> want((size_t)M * N, 0.0);
        for (int m = 0; m < M; ++m) for (int n = 0; n < N; ++n) for (int k = 0; k < K; ++k) {
            const uint8_t b = pk[(((size_t)m * N + n) * K) / 2 + k / 2];
            const int code = (k & 1) ? (b >> 4) : (b & 15);
            const double c = std::ldexp(1.0 + (double)((0x3800 + 64 * code) & 0x3FF) / 1024.0, ((0x3800 + 64 * code) >> 10) - 15);
            want[m * N + n] += c * act[(size_t)n * K + k];
        }
        CHECK(rel_l2(out, want) <= 1e-5, "oil4_gemm rel-L2 %.3g", rel_l2(out, want));
    }
    {   // production GEMV batch: Y + n*M holds activation row n
        const int M = 40, N = 3, K = 130;
        std::vector<uint8_t> w((size_t)M * K); for (auto& v : w) v = (uint8_t)(std::fabs(frand()) * 255);
        std::vector<float> cb(256), X((size_t)N * K), Y((size_t)N * M);
        for (auto& v : cb) v = frand();
        for (auto& v : X) v = frand();
        adapters::prod::gemv_oil8_batch(w.data(), cb.data(), 0.25f, X.data(), Y.data(), M, N, K);
        std::vector<double> want((size_t)N * M, 0.0);
        for (int n = 0; n < N; ++n) for (int m = 0; m < M; ++m) {
            double s = 0; for (int k = 0; k < K; ++k) s += (double)cb[w[(size_t)m * K + k]] * X[(size_t)n * K + k];
            want[(size_t)n * M + m] = 0.25 * s;
        }
        CHECK(rel_l2(Y, want) <= 1e-5, "gemv_oil8_batch rel-L2 %.3g", rel_l2(Y, want));
        std::vector<uint8_t> ws((size_t)M * ((K + 3) / 4)); for (auto& v : ws) v = (uint8_t)(std::fabs(frand()) * 255);
        std::vector<float> y1(M);
        adapters::prod::gemv_spark_tiled(ws.data(), 2.0f, X.data(), y1.data(), M, K);
        std::vector<double> w1(M, 0.0);
        for (int m = 0; m < M; ++m) for (int k = 0; k < K; ++k) {
            const int code = (ws[(size_t)m * ((K + 3) / 4) + k / 4] >> ((k % 4) * 2)) & 3;
            w1[m] += 2.0 * (code == 0 ? -1.0 : code == 1 ? 0.0 : 1.0) * X[k];
        }
        CHECK(rel_l2(y1, w1) <= 1e-5, "gemv_spark_tiled rel-L2 %.3g", rel_l2(y1, w1));
    }
    {   // engine quant_gemm: shape + finite (tests/test_quant_engines.cpp:229-263) and values
        const int64_t M = 4, N = 33, K = 20;
        std::vector<float> A((size_t)(M * K)), cb(16), C((size_t)(M * N));
        for (auto& v : A) v = frand();
        A[3] = 0.0f;
        for (auto& v : cb) v = frand();
        std::vector<uint8_t> b((size_t)(K * N + 1) / 2); for (auto& v : b) v = (uint8_t)(std::fabs(frand()) * 255);
        gfx950::engine_quant_gemm(4, A.data(), b.data(), cb.data(), C.data(), M, N, K);
        std::vector<double> want((size_t)(M * N), 0.0);
        for (int64_t m = 0; m < M; ++m) for (int64_t k = 0; k < K; ++k) for (int64_t n = 0; n < N; ++n) {
            const int64_t flat = k * N + n;
            const int code = (flat % 2 == 0) ? (b[flat / 2] & 15) : (b[flat / 2] >> 4);
            want[m * N + n] += (double)A[m * K + k] * cb[code];
        }
        CHECK(rel_l2(C, want) <= 1e-5, "engine_quant_gemm rel-L2 %.3g", rel_l2(C, want));
    }
    {   // block codec: every format round-trips cleanly (tests/test_block_codec.cpp:64-88), OIL32 bitwise,
        // zero block decodes to zero, and the tensor GEMM equals the double dot of its own decode
        std::vector<float> w(256); for (auto& v : w) v = frand() * 0.85f + 0.6f;
        for (int f = 0; f <= 14; ++f) {
            std::vector<uint8_t> idx, cb;
            CHECK(quantize_block_all((Format)f, w.data(), 256, idx, cb), "quantize failed fmt=%d", f);
            std::vector<float> out(256, 1.0f);
            dequantize_block_all((Format)f, idx.data(), idx.size(), cb.data(), cb.size(), 256, out.data());
            bool finite = true; for (float v : out) finite &= std::isfinite(v);
            CHECK(finite, "fmt=%d produced non-finite output", f);
            if ((Format)f == Format::OIL32) CHECK(std::memcmp(out.data(), w.data(), 1024) == 0, "OIL32 not bitwise");
            std::vector<float> z(256, 0.0f), zo(256, 1.0f);
            quantize_block_all((Format)f, z.data(), 256, idx, cb);
            dequantize_block_all((Format)f, idx.data(), idx.size(), cb.data(), cb.size(), 256, zo.data());
            bool allzero = true; for (float v : zo) allzero &= (v == 0.0f);
            CHECK(allzero, "zero block not zero fmt=%d", f);
        }
        const int rows = 24, cols = 512, B = 3;
        std::vector<float> W((size_t)rows * cols); for (auto& v : W) v = frand() * 0.02f;
        std::vector<std::vector<uint8_t>> idxs(rows * 2), cbs(rows * 2);
        std::vector<gfx950::BlockRef> refs;
        for (int b = 0; b < rows * 2; ++b) {
            const Format fmt = (b % 3 == 0) ? Format::OIL4 : (b % 3 == 1 ? Format::OIL8_GRP : Format::SPARK_Q0);
            quantize_block_all(fmt, W.data() + (size_t)b * 256, 256, idxs[b], cbs[b]);
            refs.push_back({fmt, cbs[b].data(), (uint32_t)cbs[b].size(), idxs[b].data(), (uint32_t)idxs[b].size(), 256});
        }
        gfx950::DeviceTensor t(refs, rows, cols);
        std::vector<float> deq((size_t)rows * cols), X((size_t)B * cols), Y((size_t)B * rows);
        for (auto& v : X) v = frand();
        t.dequantize(deq.data());
        t.gemm(X.data(), Y.data(), B);
        std::vector<double> want((size_t)B * rows, 0.0);
        for (int b = 0; b < B; ++b) for (int r = 0; r < rows; ++r) for (int c = 0; c < cols; ++c)
            want[(size_t)b * rows + r] += (double)deq[(size_t)r * cols + c] * X[(size_t)b * cols + c];
        CHECK(rel_l2(Y, want) <= 1e-5, "DeviceTensor::gemm rel-L2 %.3g", rel_l2(Y, want));
        bool threw = false;
        try { gfx950::DeviceTensor bad(refs, rows + 1, cols); } catch (const oil::Error&) { threw = true; }
        CHECK(threw, "shape mismatch must throw oil::Error");
    }
    {   // DeviceTensor::gemm at the reference's prefill batch (MAX_BATCH = 512, src/adapters/tools/qwen35_engine.cpp:12,
        // 630-753) on the Llama-7B up projection: with the prefill threshold set, B = 512 runs on the bf16 matrix-core
        // kernel (<= 2e-3), B = 8 stays on the FP32 decode kernels (<= 1e-5).  Yardstick: double dot of the tensor's
        // own decode over a sample of weight rows.
        const int rows = 11008, cols = 4096, bpr = cols / 256;
        std::vector<float> W((size_t)rows * cols);
        for (auto& v : W) v = frand() * 0.04f;
        std::vector<std::vector<uint8_t>> idxs((size_t)rows * bpr), cbs((size_t)rows * bpr);
        std::vector<gfx950::BlockRef> refs;
        refs.reserve(idxs.size());
        for (size_t b = 0; b < idxs.size(); ++b) {
            quantize_block_all(Format::OIL4, W.data() + b * 256, 256, idxs[b], cbs[b]);
            refs.push_back({Format::OIL4, cbs[b].data(), (uint32_t)cbs[b].size(), idxs[b].data(), (uint32_t)idxs[b].size(), 256});
        }
        gfx950::DeviceTensor t(refs, rows, cols);
        t.dequantize(W.data());                                  // W is now the decoded tensor
        std::vector<int> sel;
        for (int r = 0; r < rows; r += 257) sel.push_back(r);
        sel.push_back(rows - 1);
        auto check = [&](int B, double tol, const char* what) {
            std::vector<float> X((size_t)B * cols), Y((size_t)B * rows), got;
            for (auto& v : X) v = frand() * 1.7f;
            t.gemm(X.data(), Y.data(), B);
            std::vector<double> want;
            for (int b = 0; b < B; ++b)
                for (int r : sel) {
                    double a = 0;
                    for (int c = 0; c < cols; ++c) a += (double)W[(size_t)r * cols + c] * X[(size_t)b * cols + c];
                    want.push_back(a);
                    got.push_back(Y[(size_t)b * rows + r]);
                }
            bool finite = true; for (float v : Y) finite &= std::isfinite(v);
            CHECK(finite, "%s: non-finite output", what);
            CHECK(rel_l2(got, want) <= tol, "%s: rel-L2 %.3g > %.1g", what, rel_l2(got, want), tol);
            return rel_l2(got, want);
        };
        CHECK(gfx950::prefill_min_batch() == 0, "prefill threshold must default to off");
        const double e0 = check(512, 1e-5, "gemm B=512, FP32 path");
        gfx950::set_prefill_min_batch(32);
        const double e1 = check(512, 2e-3, "gemm B=512, prefill path");
        const double e2 = check(8, 1e-5, "gemm B=8 below the prefill threshold");
        CHECK(e1 > 1e-5, "B=512 with the threshold set should have run on the bf16 kernel (rel-L2 %.3g)", e1);
        std::printf("DeviceTensor::gemm 11008x4096: B=512 fp32 %.2g, B=512 prefill %.2g, B=8 %.2g\n", e0, e1, e2);
        {   // host-pointer calls in a row, as the engine's decode loop makes them (the staging buffers are kept between calls)
            std::vector<float> X(cols, 0.25f), Y(rows);
            for (int i = 0; i < 5; ++i) t.gemm(X.data(), Y.data(), 1);
            const auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < 200; ++i) t.gemm(X.data(), Y.data(), 1);
            const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / 200.0;
            std::printf("DeviceTensor::gemm 11008x4096, B=1, host pointers: %.1f us per call\n", us);
            gfx950::release_staging();
            t.gemm(X.data(), Y.data(), 1);                        // allocates afresh after a release
            CHECK(std::isfinite(Y[0]), "gemm after release_staging");
        }
        gfx950::set_prefill_min_batch(0);
    }
    {   // OIL4KVCache: prefill + two decode appends; ranges are slices of the whole, the static pair round-trips
        // through the cache's own centroids, appends past max_seq_len are dropped but counted
        const int heads = 4, dim = 64, pt = heads * dim, n = 9;
        gfx950::OIL4KVCache cache(2, 10, heads, dim, 64);
        std::vector<float> k((size_t)n * pt), v((size_t)n * pt);
        for (auto& x : k) x = frand();
        for (auto& x : v) x = frand() * 3.0f;
        cache.append(0, k.data(), v.data(), 7);
        cache.append(0, k.data() + 7 * pt, v.data() + 7 * pt, 1);
        cache.append(0, k.data() + 8 * pt, v.data() + 8 * pt, 1);
        CHECK(cache.context_len() == 9 && cache.block_size() == 64 && cache.num_layers() == 2, "kv accessors");
        auto all = cache.get_all(0);
        CHECK(all.first.size() == (size_t)n * pt && all.second.size() == (size_t)n * pt, "get_all size %zu", all.first.size());
        auto part = cache.get_range(0, 2, 5);
        CHECK(part.first.size() == (size_t)3 * pt && std::memcmp(part.first.data(), all.first.data() + 2 * pt, (size_t)3 * pt * 4) == 0, "get_range slice");
        float worst = 0.f;
        for (size_t i = 0; i < all.first.size(); ++i) worst = std::max(worst, std::fabs(all.first[i] - k[i]));
        CHECK(worst < 0.25f, "kv quantization error %.3g", worst);
        CHECK(cache.get_all(1).first.empty() && cache.get_range(5, 0, 3).first.empty(), "empty layer / no such layer");
        std::vector<uint8_t> codes(64);
        std::vector<uint16_t> cb(16);
        std::vector<float> back(64);
        gfx950::OIL4KVCache::quantize_block_oil4(k.data(), codes.data(), cb.data(), 64);
        gfx950::OIL4KVCache::dequantize_block_oil4(codes.data(), cb.data(), back.data(), 64);
        CHECK(std::memcmp(back.data(), all.first.data(), 64 * 4) == 0, "static pair equals the cache's first block");
        cache.append(0, k.data(), v.data(), 3);
        CHECK(cache.context_len() == 12 && cache.get_all(0).first.size() == (size_t)10 * pt, "overflow: dropped, counted");
        cache.clear();
        CHECK(cache.context_len() == 0 && cache.get_all(0).first.empty(), "clear");
        gfx950::OIL4KVCache odd(1, 4, 3, 5);            // an odd value count per token: chunks share bytes, as in the reference
        odd.append(0, k.data(), v.data(), 3);
        CHECK(odd.get_all(0).first.size() == 45, "odd token size");
        bool threw = false;
        try { gfx950::OIL4KVCache bad(1, -4, 3, 5); } catch (const oil::Error&) { threw = true; }
        CHECK(threw, "negative size must throw oil::Error");
    }
    std::printf("test_shims: %d checks, %d failures\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
