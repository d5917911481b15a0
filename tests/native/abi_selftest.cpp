// A host program that uses libprime_hip.so the way a C or C++ caller of the reference's
// compression ops would: plain HIP allocations, the C ABI of include/prime_hip.h, no Python and
// no torch.  It runs uniform_8bit_quantize (compression.cpp:106-125), one ring hop
// (collectives.cpp:124-138), the all-gather requantization (collectives.cpp:204-215) and a
// dequantize (collectives.cpp:16-22) on seeded data and checks every result against the CPU
// oracle it is linked with (test infrastructure: oracle/prime_oracle.cpp).
//
// Built by tests/native/build.py; run by tests/test_gpu_native.py.  Exit code 0 = all checks passed.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include <cstring>
#include "prime_hip.h"

extern "C" {
void oracle_quantize_per_tensor(const float* x, int64_t n, float scale, int32_t zero_point, int num_threads, uint8_t* out);
void oracle_average_buckets_f64(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins, double* mean_out,
                                int64_t* counts_out);
float oracle_scale_exact(const float* x, int64_t n);
void oracle_index_add(float* out, const float* lut, const uint8_t* idx, int64_t n);
void oracle_index_set(float* out, const float* lut, const uint8_t* idx, int64_t n);
}

namespace {

int g_failures = 0;

#define HIP_OK(call)                                                                       \
    do {                                                                                   \
        hipError_t e_ = (call);                                                            \
        if (e_ != hipSuccess) {                                                            \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)

#define PRIME_OK(call)                                                                     \
    do {                                                                                   \
        int rc_ = (call);                                                                  \
        if (rc_ != 0) {                                                                    \
            std::fprintf(stderr, "%s:%d %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, prime_hip_last_error()); \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)

void expect(bool ok, const char* what) {
    std::printf("  %-66s %s\n", what, ok ? "ok" : "FAILED");
    if (!ok) ++g_failures;
}

// seeded, roughly normal values (sum of uniforms), scaled
std::vector<float> make_input(int64_t n, uint64_t seed, float scale) {
    std::vector<float> v(static_cast<size_t>(n));
    uint64_t s = seed * 6364136223846793005ull + 1442695040888963407ull;
    for (auto& f : v) {
        float acc = 0.0f;
        for (int k = 0; k < 4; ++k) {
            s = s * 6364136223846793005ull + 1442695040888963407ull;
            acc += static_cast<float>((s >> 40) & 0xffffff) / 16777216.0f - 0.5f;
        }
        f = acc * scale;
    }
    return v;
}

template <typename T>
T* to_device(const std::vector<T>& h) {
    T* d = nullptr;
    HIP_OK(hipMalloc(&d, h.size() * sizeof(T) + 16));
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

template <typename T>
std::vector<T> to_host(const T* d, size_t count) {
    std::vector<T> h(count);
    HIP_OK(hipMemcpy(h.data(), d, count * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

bool lut_close(const std::vector<float>& lut, const std::vector<double>& mean, float scale) {
    for (int b = 0; b < 256; ++b) {
        const double floor = std::fabs(mean[b]) > scale ? std::fabs(mean[b]) : scale;
        if (std::fabs(lut[b] - mean[b]) > 1e-6 * floor) return false;
    }
    return true;
}

// codes and lookup of `x` (host copy) under the device's scale, against the oracle
void check_quantization(const char* label, const std::vector<float>& x, const prime_qparams& qp, const std::vector<uint8_t>& codes,
                        const std::vector<float>& lut) {
    const int64_t n = static_cast<int64_t>(x.size());
    char what[128];
    std::snprintf(what, sizeof what, "%s: scale is the formula on the exact sum of squares", label);
    expect(qp.scale == oracle_scale_exact(x.data(), n) && qp.n == n, what);
    std::vector<uint8_t> want(x.size());
    oracle_quantize_per_tensor(x.data(), n, qp.scale, 128, 1, want.data());
    std::snprintf(what, sizeof what, "%s: codes bit-exact", label);
    expect(want == codes, what);
    std::vector<double> mean(256);
    std::vector<int64_t> counts(256);
    oracle_average_buckets_f64(x.data(), want.data(), n, 256, mean.data(), counts.data());
    std::snprintf(what, sizeof what, "%s: lookup within 1e-6 of the fp64 bin means", label);
    expect(lut_close(lut, mean, qp.scale), what);
}

}  // namespace

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices < 1) {
        std::fprintf(stderr, "no GPU visible\n");
        return 3;
    }
    HIP_OK(hipSetDevice(0));
    std::printf("libprime_hip ABI version %d\n", prime_hip_abi_version());
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    void* ws = nullptr;
    const int64_t ws_bytes = prime_workspace_bytes();
    HIP_OK(hipMalloc(&ws, static_cast<size_t>(ws_bytes)));
    PRIME_OK(prime_workspace_init(ws, ws_bytes, stream));

    for (int64_t n : {int64_t(1), int64_t(4099), int64_t(1) << 20, (int64_t(1) << 22) + 3}) {
        std::printf("n = %lld\n", static_cast<long long>(n));
        const std::vector<float> x = make_input(n, 1, 1e-3f), acc0 = make_input(n, 2, 1e-3f);
        float* d_x = to_device(x);
        float* d_acc = to_device(acc0);
        uint8_t *d_c1, *d_c2, *d_c3;
        float *d_l1, *d_l2, *d_l3, *d_out;
        prime_qparams* d_qp;
        HIP_OK(hipMalloc(&d_c1, n + 16));
        HIP_OK(hipMalloc(&d_c2, n + 16));
        HIP_OK(hipMalloc(&d_c3, n + 16));
        HIP_OK(hipMalloc(&d_l1, 1024));
        HIP_OK(hipMalloc(&d_l2, 1024));
        HIP_OK(hipMalloc(&d_l3, 1024));
        HIP_OK(hipMalloc(&d_out, n * sizeof(float) + 16));
        HIP_OK(hipMalloc(&d_qp, 3 * sizeof(prime_qparams)));

        // uniform_8bit_quantize(x); acc += lut[codes], requantize; requantize what was just sent; dequantize
        PRIME_OK(prime_uniform_8bit_quantize(d_x, n, d_c1, d_l1, d_qp, ws, stream));
        PRIME_OK(prime_ring_reduce_step(d_acc, d_c1, d_l1, n, d_c2, d_l2, d_qp + 1, ws, stream));
        PRIME_OK(prime_requantize_codes(d_c2, d_l2, n, d_c3, d_l3, d_qp + 2, ws, stream));
        PRIME_OK(prime_dequant_set(d_out, d_l2, d_c2, n, stream));
        HIP_OK(hipStreamSynchronize(stream));

        const auto c1 = to_host(d_c1, n), c2 = to_host(d_c2, n), c3 = to_host(d_c3, n);
        const auto l1 = to_host(d_l1, 256), l2 = to_host(d_l2, 256), l3 = to_host(d_l3, 256);
        const auto qp = to_host(d_qp, 3);
        const auto acc = to_host(d_acc, n), out = to_host(d_out, n);
        if (n > 1) check_quantization("uniform_8bit_quantize", x, qp[0], c1, l1);
        std::vector<float> want_acc = acc0;
        oracle_index_add(want_acc.data(), l1.data(), c1.data(), n);
        expect(want_acc == acc, "ring hop: accumulator bit-exact");
        if (n > 1) check_quantization("ring hop requantize", want_acc, qp[1], c2, l2);
        std::vector<float> want_out(static_cast<size_t>(n));
        oracle_index_set(want_out.data(), l2.data(), c2.data(), n);
        expect(want_out == out, "dequantize: lut[codes] bit-exact");
        if (n > 1) check_quantization("requantize from codes", want_out, qp[2], c3, l3);
        expect(to_host(d_x, n) == x, "input untouched");

        for (void* p : {(void*)d_x, (void*)d_acc, (void*)d_c1, (void*)d_c2, (void*)d_c3, (void*)d_l1, (void*)d_l2, (void*)d_l3,
                        (void*)d_out, (void*)d_qp})
            HIP_OK(hipFree(p));
    }

    // several tensors in one segmented call: every tensor's results are those of the one-tensor entry point
    {
        const std::vector<int64_t> ns = {int64_t(3) << 18, 0, 70001, (int64_t(1) << 20) + 1, 5, 300000};
        const int64_t count = static_cast<int64_t>(ns.size());
        std::vector<float*> xs(ns.size()), accs(ns.size());
        std::vector<uint8_t*> cs(ns.size()), cs1(ns.size()), cs2(ns.size());
        std::vector<const float*> xs_c(ns.size()), luts_in(ns.size());
        std::vector<const uint8_t*> codes_in(ns.size());
        float *d_luts, *d_luts2, *d_lut1;
        prime_qparams *d_qps, *d_qp1;
        HIP_OK(hipMalloc(&d_luts, ns.size() * 1024));
        HIP_OK(hipMalloc(&d_luts2, ns.size() * 1024));
        HIP_OK(hipMalloc(&d_lut1, 1024));
        HIP_OK(hipMalloc(&d_qps, ns.size() * sizeof(prime_qparams)));
        HIP_OK(hipMalloc(&d_qp1, sizeof(prime_qparams)));
        for (size_t t = 0; t < ns.size(); ++t) {
            xs[t] = to_device(make_input(ns[t] ? ns[t] : 1, 10 + static_cast<int>(t), 1e-3f));
            accs[t] = to_device(make_input(ns[t] ? ns[t] : 1, 30 + static_cast<int>(t), 1e-3f));
            xs_c[t] = xs[t];
            HIP_OK(hipMalloc(&cs[t], ns[t] + 16));
            HIP_OK(hipMalloc(&cs1[t], ns[t] + 16));
            HIP_OK(hipMalloc(&cs2[t], ns[t] + 16));
        }
        PRIME_OK(prime_uniform_8bit_quantize_segmented(xs_c.data(), ns.data(), count, cs.data(), d_luts, d_qps, ws, stream));
        HIP_OK(hipStreamSynchronize(stream));
        const auto seg_luts = to_host(d_luts, 256 * count);
        const auto seg_qps = to_host(d_qps, count);
        for (size_t t = 0; t < ns.size(); ++t) {
            if (ns[t] == 0) continue;
            PRIME_OK(prime_uniform_8bit_quantize(xs[t], ns[t], cs1[t], d_lut1, d_qp1, ws, stream));
            HIP_OK(hipStreamSynchronize(stream));
            expect(to_host(cs[t], ns[t]) == to_host(cs1[t], ns[t]), "segmented call: codes of the one-tensor call");
            const auto l1 = to_host(d_lut1, 256);
            expect(std::memcmp(l1.data(), seg_luts.data() + 256 * t, 1024) == 0, "segmented call: lookup table of the one-tensor call, bit for bit");
            const auto q1 = to_host(d_qp1, 1);
            expect(std::memcmp(&q1[0], &seg_qps[t], sizeof(prime_qparams)) == 0, "segmented call: statistics record of the one-tensor call");
            codes_in[t] = cs[t];
            luts_in[t] = d_luts + 256 * t;
        }
        codes_in[1] = cs[1];
        luts_in[1] = d_luts + 256;
        // a ring step on every accumulator with its tensor's message, in one call; then one by one on copies
        std::vector<std::vector<float>> acc_before(ns.size());
        for (size_t t = 0; t < ns.size(); ++t) acc_before[t] = to_host(accs[t], ns[t]);
        PRIME_OK(prime_ring_reduce_step_segmented(accs.data(), codes_in.data(), luts_in.data(), ns.data(), count, cs2.data(), d_luts2, nullptr, ws,
                                                  stream));
        HIP_OK(hipStreamSynchronize(stream));
        const auto seg_luts2 = to_host(d_luts2, 256 * count);
        for (size_t t = 0; t < ns.size(); ++t) {
            if (ns[t] == 0) continue;
            float* d_acc = to_device(acc_before[t]);
            PRIME_OK(prime_ring_reduce_step(d_acc, cs[t], d_luts + 256 * t, ns[t], cs1[t], d_lut1, nullptr, ws, stream));
            HIP_OK(hipStreamSynchronize(stream));
            expect(to_host(d_acc, ns[t]) == to_host(accs[t], ns[t]), "segmented ring step: accumulator of the one-tensor call");
            expect(to_host(cs2[t], ns[t]) == to_host(cs1[t], ns[t]), "segmented ring step: codes of the one-tensor call");
            const auto l1 = to_host(d_lut1, 256);
            expect(std::memcmp(l1.data(), seg_luts2.data() + 256 * t, 1024) == 0, "segmented ring step: lookup table of the one-tensor call");
            HIP_OK(hipFree(d_acc));
        }
        for (size_t t = 0; t < ns.size(); ++t)
            for (void* p : {(void*)xs[t], (void*)accs[t], (void*)cs[t], (void*)cs1[t], (void*)cs2[t]}) HIP_OK(hipFree(p));
        for (void* p : {(void*)d_luts, (void*)d_luts2, (void*)d_lut1, (void*)d_qps, (void*)d_qp1}) HIP_OK(hipFree(p));
    }

    // error behaviour: rejected arguments return non-zero with a message, and launch nothing
    expect(prime_uniform_8bit_quantize(nullptr, 8, nullptr, nullptr, nullptr, ws, stream) != 0 && prime_hip_last_error()[0] != 0,
           "null pointers are rejected with a message");
    expect(prime_uniform_8bit_quantize(reinterpret_cast<const float*>(ws), -1, reinterpret_cast<uint8_t*>(ws),
                                       reinterpret_cast<float*>(ws), nullptr, ws, stream) != 0,
           "negative sizes are rejected");
    expect(prime_workspace_init(ws, 16, stream) != 0, "a workspace that is too small is rejected");
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipFree(ws));
    HIP_OK(hipStreamDestroy(stream));
    std::printf(g_failures ? "%d check(s) FAILED\n" : "all checks passed\n", g_failures);
    return g_failures ? 1 : 0;
}
