// TEST INFRASTRUCTURE - CPU oracle for the int8 pseudo-gradient compression path.
//
// A torch-free restatement of the reference's CPU algorithm, used only as the
// checker in tests/, in __graft_entry__.smoke() and as bench.py's cpu_baseline
// leg.  Nothing in the product package may link, load or call this file.
//
// Each function names the reference lines it restates (paths relative to the
// reference checkout):
//   src/zeroband/C/csrc/compression.cpp  - quantize / average_buckets / uniform_8bit_quantize
//   src/zeroband/C/csrc/collectives.cpp  - fast_index_add / fast_index_set
//
// How each function is pinned (checks live in tests/test_oracle_*.py):
//   oracle_quantize_per_tensor  closed forms (power-of-two scales, ties away from zero, the
//                               reference test's ones*10 / 0.01 vector -> 255), brute force
//                               around every bin boundary, and the compiled reference (oracle/_ref)
//   oracle_average_buckets      exact bincount; integer-valued inputs (order independent sums);
//                               fp64 closed form; compiled reference
//   oracle_uniform_8bit_quantize closed forms (constant tensor -> code 171, zero tensor, n = 1),
//                               golden fixtures written by the compiled reference
//   oracle_norm_literal         bit-for-bit against libtorch's at::norm over sizes 1..70 and larger
//                               (observed order: 8 fp32 FMA lanes, lanes summed 0..7, tail, sqrtf);
//                               the order used by the reference's pinned torch 2.5.1 cannot be
//                               checked offline: "parity unpinned" for that version only
//   oracle_index_add / _set     numpy lut[codes] bitwise
//   oracle_pseudo_gradient      torch (a - b).div_(W) bitwise
//   oracle_outer_sgd_nesterov   torch.optim.SGD(momentum, nesterov=True) on CPU, bitwise over several
//                               steps and sizes (vector body and scalar tail of libtorch's kernels)
//
// Build: see oracle/build.py (g++ -O3, the reference's only flag, src/zeroband/C/compression.py:8).

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

namespace {

constexpr int kBins = 256;               // compression.cpp:5
constexpr double kRangeInSigmas = 6.0;   // compression.cpp:6

// float -> int32 conversion as x86 performs it (cvttss2si / cvttps2dq): values that do
// not fit, and NaN, give the "integer indefinite" 0x80000000.  compression.cpp:23 relies
// on this conversion; in C++ the out-of-range case is undefined, so it is spelled out.
inline int32_t x86_cvtt_f32_i32(float r) {
    if (!(r >= -2147483648.0f && r < 2147483648.0f)) return std::numeric_limits<int32_t>::min();
    return static_cast<int32_t>(r);
}

// One element of compression.cpp:23-24.  The "+ zero_point" wraps like the two's
// complement add the compiled reference executes.
inline uint8_t quantize_one(float x, float inv_scale, int32_t zero_point) {
    int32_t q = x86_cvtt_f32_i32(std::round(x * inv_scale));
    q = static_cast<int32_t>(static_cast<uint32_t>(q) + static_cast<uint32_t>(zero_point));
    return static_cast<uint8_t>(std::clamp(q, 0, 255));
}

int resolve_threads(int num_threads) {
    if (num_threads > 0) return num_threads;
    int hw = static_cast<int>(std::thread::hardware_concurrency());   // compression.cpp:7
    return hw > 0 ? hw : 1;
}

}  // namespace

extern "C" {

int oracle_hardware_threads() { return resolve_threads(0); }

// compression.cpp:9-43  quantize_per_tensor_multithreaded.
// Slicing as the reference: chunk = numel / T, the last thread takes the remainder.
void oracle_quantize_per_tensor(const float* x, int64_t n, float scale, int32_t zero_point,
                                int num_threads, uint8_t* out) {
    const int T = resolve_threads(num_threads);
    const float inv_scale = 1.0f / scale;                       // :16
    const int64_t chunk = n / T;                                // :19
    auto work = [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) out[i] = quantize_one(x[i], inv_scale, zero_point);
    };
    std::vector<std::thread> pool;
    for (int t = 0; t < T - 1; ++t) pool.emplace_back(work, t * chunk, (t + 1) * chunk);   // :28-32
    pool.emplace_back(work, (T - 1) * chunk, n);                                           // :35
    for (auto& th : pool) th.join();
}

// compression.cpp:45-104  average_buckets_multithread.
// Per-thread fp32 sums and int64 counts over contiguous slices (:64-74), merged into the
// shared fp32 sums (:79-82), then sum / count with the count converted to float (:100).
// The reference merges in thread *finish* order under a mutex, which is not
// reproducible; this restatement merges in thread index order.
void oracle_average_buckets(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins,
                            int num_threads, float* lut, int64_t* counts_out) {
    const int T = resolve_threads(num_threads);
    std::vector<std::vector<float>> sums(T, std::vector<float>(n_bins, 0.0f));
    std::vector<std::vector<int64_t>> counts(T, std::vector<int64_t>(n_bins, 0));
    const int64_t chunk = n / T;                                // :86
    auto work = [&](int t, int64_t lo, int64_t hi) {
        float* s = sums[t].data();
        int64_t* c = counts[t].data();
        for (int64_t i = lo; i < hi; ++i) {
            const uint8_t b = codes[i];
            if (b < n_bins) {                                   // :70
                s[b] += x[i];
                c[b] += 1;
            }
        }
    };
    std::vector<std::thread> pool;
    for (int t = 0; t < T; ++t)
        pool.emplace_back(work, t, t * chunk, t == T - 1 ? n : (t + 1) * chunk);   // :87-91
    for (auto& th : pool) th.join();
    for (int64_t b = 0; b < n_bins; ++b) {
        float s = 0.0f;
        int64_t c = 0;
        for (int t = 0; t < T; ++t) {
            s += sums[t][b];
            c += counts[t][b];
        }
        lut[b] = c > 0 ? s / static_cast<float>(c) : 0.0f;      // :100
        if (counts_out) counts_out[b] = c;
    }
}

// fp64 statement of the same quantity: exact counts, sums accumulated in double,
// mean rounded to float once.  This is what tolerance checks compare against.
void oracle_average_buckets_f64(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins,
                                double* mean_out, int64_t* counts_out) {
    std::vector<double> s(n_bins, 0.0);
    std::vector<int64_t> c(n_bins, 0);
    for (int64_t i = 0; i < n; ++i) {
        const uint8_t b = codes[i];
        if (b < n_bins) {
            s[b] += static_cast<double>(x[i]);
            c[b] += 1;
        }
    }
    for (int64_t b = 0; b < n_bins; ++b) {
        mean_out[b] = c[b] > 0 ? s[b] / static_cast<double>(c[b]) : 0.0;
        if (counts_out) counts_out[b] = c[b];
    }
}

// The value `tensor.norm()` (compression.cpp:113) returns for a contiguous fp32 CPU tensor
// in libtorch 2.10 on x86-64, found by matching it bit for bit: eight fp32 lanes, lane j
// accumulating elements j, j+8, ... with a fused multiply-add; lanes added 0..7; then the
// n % 8 tail in order, a group of four as rounded products added one by one (the compiler's
// in-order vectorisation of the scalar tail loop) and the last n % 4 elements by fused
// multiply-add; and a float square root.
float oracle_norm_literal(const float* x, int64_t n) {
    float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const int64_t m = n - (n % 8);
    for (int64_t i = 0; i < m; i += 8)
        for (int j = 0; j < 8; ++j) lane[j] = std::fma(x[i + j], x[i + j], lane[j]);
    float s = lane[0];
    for (int j = 1; j < 8; ++j) s += lane[j];
    int64_t i = m;
    if (n - i >= 4) {
        for (int k = 0; k < 4; ++k) {
            volatile float sq = x[i + k] * x[i + k];   // product rounded on its own: no contraction
            s += sq;
        }
        i += 4;
    }
    for (; i < n; ++i) s = std::fma(x[i], x[i], s);
    return std::sqrt(s);
}

// Sum and sum of squares in fp64 (x*x is exact in double for float x).
void oracle_stats_f64(const float* x, int64_t n, double* sum, double* sumsq) {
    // pairwise over blocks keeps the error far below 1e-12 relative at 2^30 elements
    const int64_t B = 4096;
    std::vector<double> ps, pq;
    for (int64_t i = 0; i < n; i += B) {
        double s = 0.0, q = 0.0;
        const int64_t hi = std::min(n, i + B);
        for (int64_t k = i; k < hi; ++k) {
            const double v = x[k];
            s += v;
            q += v * v;
        }
        ps.push_back(s);
        pq.push_back(q);
    }
    auto tree = [](std::vector<double>& v) {
        if (v.empty()) return 0.0;
        size_t m = v.size();
        while (m > 1) {
            size_t h = (m + 1) / 2;
            for (size_t k = 0; k + h < m; ++k) v[k] += v[k + h];
            m = h;
        }
        return v[0];
    };
    *sum = tree(ps);
    *sumsq = tree(pq);
}

// compression.cpp:113-116 given the float norm: std = double(norm) / sqrt(numel - 1),
// scale = 6 * std / 256, narrowed to float where it is passed to the quantizer (:119).
float oracle_scale_from_norm(float norm, int64_t n) {
    const double std_unbiased = static_cast<double>(norm) / std::sqrt(static_cast<double>(n - 1));
    const double scale = kRangeInSigmas * std_unbiased / kBins;
    return static_cast<float>(scale);
}

// The scale the formula specifies when the sum of squares carries no accumulation error:
// norm = float(sqrt(sum of squares in fp64)).
float oracle_scale_exact(const float* x, int64_t n) {
    double s, q;
    oracle_stats_f64(x, n, &s, &q);
    return oracle_scale_from_norm(static_cast<float>(std::sqrt(q)), n);
}

float oracle_scale_literal(const float* x, int64_t n) {
    return oracle_scale_from_norm(oracle_norm_literal(x, n), n);
}

// compression.cpp:106-125  uniform_8bit_quantize.  norm_mode 0 = literal libtorch
// accumulation order, 1 = exact sum of squares, 2 = use *scale_io as given.
// zero_point is n_bins / 2 (:107); no mean is subtracted (:109-110).
void oracle_uniform_8bit_quantize(const float* x, int64_t n, int num_threads, int norm_mode,
                                  uint8_t* codes, float* lut, float* scale_io) {
    float scale;
    if (norm_mode == 0) scale = oracle_scale_literal(x, n);
    else if (norm_mode == 1) scale = oracle_scale_exact(x, n);
    else scale = *scale_io;
    oracle_quantize_per_tensor(x, n, scale, kBins / 2, num_threads, codes);     // :119
    oracle_average_buckets(x, codes, n, kBins, num_threads, lut, nullptr);      // :122
    if (scale_io) *scale_io = scale;
}

// collectives.cpp:8-14  fast_index_add_omp<float>.  As shipped the loop is serial: the
// build passes no -fopenmp (src/zeroband/C/collectives.py:17), so the pragma is inert.
void oracle_index_add(float* out, const float* lut, const uint8_t* idx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] += lut[idx[i]];
}

// collectives.cpp:16-22  fast_index_set_omp<float>.
void oracle_index_set(float* out, const float* lut, const uint8_t* idx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = lut[idx[i]];
}

// collectives.cpp:36-50 / :60-74  the std::thread variants the reference defines but never calls.
void oracle_index_add_threads(float* out, const float* lut, const uint8_t* idx, int64_t n, int num_threads) {
    const int T = resolve_threads(num_threads);
    const int64_t chunk = n / T;
    std::vector<std::thread> pool;
    for (int t = 0; t < T; ++t) {
        const int64_t lo = t * chunk, hi = t == T - 1 ? n : (t + 1) * chunk;
        pool.emplace_back([=] { for (int64_t i = lo; i < hi; ++i) out[i] += lut[idx[i]]; });
    }
    for (auto& th : pool) th.join();
}

void oracle_index_set_threads(float* out, const float* lut, const uint8_t* idx, int64_t n, int num_threads) {
    const int T = resolve_threads(num_threads);
    const int64_t chunk = n / T;
    std::vector<std::thread> pool;
    for (int t = 0; t < T; ++t) {
        const int64_t lo = t * chunk, hi = t == T - 1 ? n : (t + 1) * chunk;
        pool.emplace_back([=] { for (int64_t i = lo; i < hi; ++i) out[i] = lut[idx[i]]; });
    }
    for (auto& th : pool) th.join();
}

// collectives.cpp:157  chunk.div_(world_size): libtorch divides fp32 by the scalar in fp32.
void oracle_div_scalar(float* x, int64_t n, float d) {
    for (int64_t i = 0; i < n; ++i) x[i] = x[i] / d;
}

// Diloco.sync_pseudo_gradient, src/zeroband/diloco.py:93-101: grad = outer - inner (fp32), then
// the flat gradient buffer divided by the world size (fp32 division).
void oracle_pseudo_gradient(const float* outer, const float* inner, int64_t n, float world_size, float* out) {
    for (int64_t i = 0; i < n; ++i) {
        volatile float d = outer[i] - inner[i];
        out[i] = d / world_size;
    }
}

// torch.optim.SGD(lr, momentum, nesterov=True).step() on fp32 CPU tensors (the outer optimizer,
// src/zeroband/diloco.py:72-74,212-213), as libtorch rounds it, found by matching torch bit for
// bit: buf.mul_(mu).add_(g) is a rounded product plus a rounded sum (buf = g on the first
// step); g.add(buf, alpha=mu) and p.add_(d, alpha=-lr) are fused multiply-adds.
void oracle_outer_sgd_nesterov(float* param, float* buf, const float* grad, int64_t n, float lr, float mu, int first_step) {
    const float neg_lr = -lr;
    for (int64_t i = 0; i < n; ++i) {
        const float g = grad[i];
        if (first_step) {
            buf[i] = g;
        } else {
            volatile float prod = buf[i] * mu;   // rounded on its own
            buf[i] = prod + g;
        }
        const float d = std::fma(buf[i], mu, g);
        param[i] = std::fma(d, neg_lr, param[i]);
    }
}

}  // extern "C"
