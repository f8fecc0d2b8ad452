// A C++ caller of the C ABI with nothing in between: no Python, no torch. Device buffers come from hipMalloc, the launches go
// to a stream of its own, results are copied back and compared bit for bit with the CPU oracle (test infrastructure: this file
// lives under tests/ and links oracle/liborc.so). This is the shape of the reference's second caller, its C++ runtime
// (runtime/rt.cpp:61-78 loads a module and launches by name); here the functions are linked by name through include/camx.h.
//
// cpp_caller_run(msg, len) -> 0 on success; on failure a short description is written to msg.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "camx.h"

extern "C" {
void orc_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h, uint16_t * h16, uint8_t * q8, int N, int n);
void orc_kv_q8_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, int rows, int T, int * err);
void orc_mmq_q8_1(const float * x, const int32_t * ids, uint8_t * y, int64_t K, int64_t s01, int ncols, int layout);
}

namespace {

struct DeviceBuffer {                      // hipMalloc / hipFree with the bytes uploaded at construction
    void * p = nullptr; size_t bytes = 0;
    DeviceBuffer(const void * host, size_t n) : bytes(n) { if (hipMalloc(&p, n ? n : 1) != hipSuccess) p = nullptr; else if (host) (void)hipMemcpy(p, host, n, hipMemcpyHostToDevice); else (void)hipMemset(p, 0, n); }
    ~DeviceBuffer() { if (p) (void)hipFree(p); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    template <typename T> T * as() const { return (T *)p; }
    template <typename T> std::vector<T> download() const { std::vector<T> v(bytes / sizeof(T)); (void)hipMemcpy(v.data(), p, bytes, hipMemcpyDeviceToHost); return v; }
};

template <typename T> bool same(const std::vector<T> & a, const std::vector<T> & b) { return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0; }

int fail(char * msg, int len, const char * what, int code = -1) { std::snprintf(msg, (size_t)len, "%s (%d: %s)", what, code, code >= 0 ? camx_error_string(code) : "mismatch"); return 1; }

}   // namespace

extern "C" __attribute__((visibility("default"))) int cpp_caller_run(char * msg, int len) {
    if (len > 0) msg[0] = 0;
    hipStream_t st;
    if (hipStreamCreate(&st) != hipSuccess) return fail(msg, len, "hipStreamCreate");
    std::mt19937 rng(20260);
    std::normal_distribution<float> normal(0.0f, 1.0f);
    int rc = 0;
    {   // residual add + RMSNorm with fp32, fp16 and q8_1 copies
        const int n = 37, N = 2048;
        std::vector<float> x((size_t)n * N), d((size_t)n * N), nw(N);
        for (auto & v : x) v = normal(rng);
        for (auto & v : d) v = normal(rng);
        for (auto & v : nw) v = 1.0f + 0.1f * normal(rng);
        DeviceBuffer dx(x.data(), x.size() * 4), dd(d.data(), d.size() * 4), dnw(nw.data(), nw.size() * 4), dh(nullptr, x.size() * 4), dh16(nullptr, x.size() * 2),
            dq8(nullptr, (size_t)n * (N / 32) * 36);
        const int e = camx_add_rms_q8_1(dx.as<float>(), dd.as<float>(), nullptr, 1, dnw.as<float>(), 1e-6f, dh.as<float>(), dh16.as<uint16_t>(), dq8.p, N, n, st);
        if (e) rc = fail(msg, len, "camx_add_rms_q8_1", e);
        (void)hipStreamSynchronize(st);
        std::vector<float> h(x.size()); std::vector<uint16_t> h16(x.size()); std::vector<uint8_t> q8((size_t)n * (N / 32) * 36);
        orc_add_rms16(x.data(), d.data(), nullptr, 1, nw.data(), 1e-6f, h.data(), h16.data(), q8.data(), N, n);
        if (!rc && !(same(dx.download<float>(), x) && same(dh.download<float>(), h) && same(dh16.download<uint16_t>(), h16) && same(dq8.download<uint8_t>(), q8)))
            rc = fail(msg, len, "add + RMSNorm + q8_1 differs from the oracle");
    }
    if (!rc) {   // fp32 rows -> q8_1 blocks in the MMQ layout, through the persistent kernel (>= 256 columns)
        const int ncols = 300; const long K = 900, Kp = 1024;
        std::vector<float> x((size_t)ncols * K);
        for (auto & v : x) v = normal(rng);
        DeviceBuffer dx(x.data(), x.size() * 4), dy(nullptr, (size_t)(Kp / 128) * ncols * 144);
        const int e = camx_quantize_mmq_q8_1(dx.as<float>(), nullptr, dy.p, K, K, 0, 0, Kp, ncols, 1, 0, 1, st);
        if (e) rc = fail(msg, len, "camx_quantize_mmq_q8_1", e);
        (void)hipStreamSynchronize(st);
        std::vector<uint8_t> y((size_t)(Kp / 128) * ncols * 144);
        orc_mmq_q8_1(x.data(), nullptr, y.data(), K, K, ncols, 1);
        if (!rc && !same(dy.download<uint8_t>(), y)) rc = fail(msg, len, "MMQ q8_1 blocks differ from the oracle");
    }
    if (!rc) {   // Q8 KV rows, with one refused block and the sticky error word
        const int T = 9, M = 512, rows = 16;
        std::vector<float> k((size_t)T * M), v((size_t)T * M);
        for (auto & e : k) e = normal(rng);
        for (auto & e : v) e = normal(rng);
        k[3 * M + 40] = INFINITY;                                            // block 1 of token 3 is refused
        std::vector<uint8_t> cache((size_t)rows * 2 * (M / 32) * 34, 0xa5);
        DeviceBuffer dk(k.data(), k.size() * 4), dv(v.data(), v.size() * 4), dc(cache.data(), cache.size()), derr(nullptr, 4);
        const int e = camx_own_kv_q8_append(dk.as<float>(), M, dv.as<float>(), M, M, dc.as<uint8_t>(), 2, rows, derr.as<int>(), T, st);
        if (e) rc = fail(msg, len, "camx_own_kv_q8_append", e);
        (void)hipStreamSynchronize(st);
        int werr = 0;
        orc_kv_q8_append(k.data(), M, v.data(), M, M, cache.data(), 2, rows, T, &werr);
        if (!rc && !(same(dc.download<uint8_t>(), cache) && derr.download<int>()[0] == werr && werr == 2)) rc = fail(msg, len, "Q8 KV rows or error word differ from the oracle");
    }
    if (!rc) {   // the tape's form of the same append: tables filled up front, the position in a device word, advanced between two calls
        const int T = 2, M = 256, rows = 8;
        if (const int e = camx_init(st)) rc = fail(msg, len, "camx_init", e);
        std::vector<float> k((size_t)T * M), v((size_t)T * M);
        for (auto & e : k) e = normal(rng);
        for (auto & e : v) e = normal(rng);
        std::vector<uint8_t> cache((size_t)rows * 2 * (M / 32) * 34, 0x5a);
        int pos = 1, werr = 0;
        DeviceBuffer dk(k.data(), k.size() * 4), dv(v.data(), v.size() * 4), dc(cache.data(), cache.size()), derr(nullptr, 4), dpos(&pos, 4);
        for (int call = 0; call < 2 && !rc; call++, pos += 5) {              // rows 1, 2, then 6, 7
            if (hipMemcpyAsync(dpos.p, &pos, 4, hipMemcpyHostToDevice, st) != hipSuccess) rc = fail(msg, len, "hipMemcpyAsync");
            const int e = camx_op_kv_append(dk.as<float>(), dv.as<float>(), dc.p, dpos.as<int32_t>(), M, 2, derr.as<int>(), rows, T, st);
            if (e) rc = fail(msg, len, "camx_op_kv_append", e);
            (void)hipStreamSynchronize(st);
            orc_kv_q8_append(k.data(), M, v.data(), M, M, cache.data(), pos, rows, T, &werr);
        }
        if (!rc && !(same(dc.download<uint8_t>(), cache) && derr.download<int>()[0] == 0 && werr == 0)) rc = fail(msg, len, "tape-form Q8 KV rows differ from the oracle");
    }
    if (!rc) {   // a decode token's attention inputs: the tape's three launches (k norm + rotary, append, q norm + rotary) and the one that replaces them
        const int T = 1, nh = 32, nkv = 4, D = 128, M = nkv * D, rows = 64;
        std::vector<float> q((size_t)T * nh * D), k((size_t)T * M), v((size_t)T * M), wq(D), wk(D);
        for (auto & e : q) e = normal(rng);
        for (auto & e : k) e = normal(rng);
        for (auto & e : v) e = normal(rng);
        for (auto & e : wq) e = 1.0f + 0.1f * normal(rng);
        for (auto & e : wk) e = 1.0f + 0.1f * normal(rng);
        const float eps = 1e-6f, ts = 0.80584f; int eb; std::memcpy(&eb, &eps, 4);
        int pos = 41;
        DeviceBuffer dq(q.data(), q.size() * 4), dk(k.data(), k.size() * 4), dv(v.data(), v.size() * 4), dwq(wq.data(), D * 4), dwk(wk.data(), D * 4), dpos(&pos, 4), derr(nullptr, 4);
        DeviceBuffer qo1(nullptr, q.size() * 4), ko1(nullptr, k.size() * 4), c1(nullptr, (size_t)rows * 2 * M * 2), qo2(nullptr, q.size() * 4), c2(nullptr, (size_t)rows * 2 * M * 2);
        int e = camx_op_qk_nr(dk.as<float>(), D, nkv, D, dwk.as<float>(), dpos.as<int32_t>(), ko1.as<float>(), D, ts, eb, T, st);
        if (!e) e = camx_op_kv_append(ko1.as<float>(), dv.as<float>(), c1.p, dpos.as<int32_t>(), M, 0, derr.as<int>(), rows, T, st);
        if (!e) e = camx_op_qk_nr(dq.as<float>(), D, nh, D, dwq.as<float>(), dpos.as<int32_t>(), qo1.as<float>(), D, ts, eb, T, st);
        if (!e) e = camx_qk_nr_kv(dq.as<float>(), D, nh, dwq.as<float>(), dk.as<float>(), D, dv.as<float>(), M, nkv, dwk.as<float>(), D, D, ts, eps, 0, dpos.as<int32_t>(), nullptr,
                                  qo2.as<float>(), nullptr, c2.p, 0, rows, derr.as<int>(), T, st);
        if (e) rc = fail(msg, len, "camx_qk_nr_kv or the launches it replaces", e);
        (void)hipStreamSynchronize(st);
        const std::vector<uint16_t> row = c2.download<uint16_t>();
        bool written = false;
        for (int i = 0; i < 2 * M; i++) written |= row[(size_t)pos * 2 * M + i] != 0;
        if (!rc && !(same(qo1.download<float>(), qo2.download<float>()) && same(c1.download<uint16_t>(), row) && written && derr.download<int>()[0] == 0))
            rc = fail(msg, len, "camx_qk_nr_kv differs from the three launches");
    }
    if (!rc && camx_add_rms_q8_1(nullptr, nullptr, nullptr, 0, nullptr, 1e-6f, nullptr, nullptr, nullptr, 2048, 1, st) != 1) rc = fail(msg, len, "a null row pointer was not refused");
    (void)hipStreamDestroy(st);
    return rc;
}
