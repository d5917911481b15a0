// Either side of the all-reduce: division, pseudo-gradient, a chunk's first touch in the ring,
// the SGD-Nesterov outer step (from fp32 or from codes), and the plain copy and fill kernels.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

__global__ void fill_zero_kernel(uint32_t* p, int64_t nwords) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < nwords;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = 0u;
}

// chunk /= world_size for ReduceOp::AVG (collectives.cpp:155-159): an fp32 division in place.
template <bool ALIGNED, int POLICY, bool ONESHOT = false, int ST = kStreamShotThreads, int SU = kStreamShotRows>
__global__ __launch_bounds__(ONESHOT ? ST : kThreads, ONESHOT ? 8 : kWavesPerSimd) void div_kernel(float* __restrict__ x, int64_t n, float d) {
    using M = Mem<ALIGNED, false>;
    const int64_t nvec = n >> 2;
    constexpr int T = ONESHOT ? ST : kThreads;
    constexpr int U = ONESHOT ? SU : kDivUnroll;
    walk_tiles<T, U, ONESHOT>(nvec, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window win(x + base * 4, (nvec - base) * 16);
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
                if (ALIGNED) win.template st128<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 16u, v[j] / d);
                else M::stf4(x, i, v[j] / d, false);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        x[i] = x[i] / d;
    }
}

// The pseudo-gradient of one bucket as Diloco.sync_pseudo_gradient forms it
// (src/zeroband/diloco.py:93-101): grad = outer_param - inner_param, then the whole flat buffer
// divided by the world size; an fp32 subtraction and an fp32 division per element.
// 12 bytes per element.
// pseudo_gradient_block is the pass for the calling workgroup as workgroup `slot` of a grid of G.
template <bool ALIGNED, bool NT, int POLICY, bool ONESHOT, int ST = kStreamShotThreads, int SU = kStreamShotRows>
__device__ __forceinline__ void pseudo_gradient_block(const float* __restrict__ outer, const float* __restrict__ inner, int64_t n,
                                                      float world_size, float* __restrict__ out, int64_t slot, int64_t G) {
    using M = Mem<ALIGNED, NT>;
    const int64_t nvec = n >> 2;
    constexpr int T = ONESHOT ? ST : kThreads;
    constexpr int U = ONESHOT ? SU : kDivUnroll;
    walk_tiles_of<T, U, ONESHOT>(nvec, slot, G, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window win(out + base * 4, (nvec - base) * 16);
        f4a a[U], b[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            a[j] = ok ? M::ldf4(outer, i) : f4a{0.f, 0.f, 0.f, 0.f};
            b[j] = ok ? M::ldf4(inner, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
                const f4a g = (a[j] - b[j]) / world_size;
                if (ALIGNED) win.template st128<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 16u, g);
                else M::stf4(out, i, g, false);
            }
        }
    });
    if (slot == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        out[i] = (outer[i] - inner[i]) / world_size;
    }
}

template <bool ALIGNED, bool NT, int POLICY, bool ONESHOT = false>
__global__ __launch_bounds__(ONESHOT ? kStreamShotThreads : kThreads, ONESHOT ? 8 : kWavesPerSimd) void pseudo_gradient_kernel(const float* __restrict__ outer, const float* __restrict__ inner, int64_t n,
                                            float world_size, float* __restrict__ out) {
    pseudo_gradient_block<ALIGNED, NT, POLICY, ONESHOT>(outer, inner, n, world_size, out, blockIdx.x, gridDim.x);
}

// A chunk's first touch in the ring when the pseudo-gradient has not been written yet: every
// chunk of a rank is visited exactly once in the reduce-scatter (collectives.cpp:115-116), so
// grad = (outer - inner) / world_size (diloco.py:93-101) can be formed in the pass that would
// otherwise read it back.  With CODES the received message is accumulated,
// acc = grad + lut[codes] (collectives.cpp:128-133), and with a divisor other than 1 the sum is
// divided (ReduceOp::AVG, :155-159).  The fp64 sum and sum of squares of what is stored are the
// statistics of the quantization that follows.  12 bytes per element, 13 with codes.  (Only the
// variant with CODES is launched: without a message the pseudo-gradient as one workgroup per tile
// followed by the statistics kernel is faster than this loop.)
// RECIP: world_size and divisor are powers of two and arrive as their reciprocals; x * 2^-k is x / 2^k bit for
// bit, and the pass then takes tiles of four rows instead of two (no division sequences to hold registers for).
template <bool CODES, bool ALIGNED, bool NT, int POLICY, bool RECIP = false>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void first_touch_kernel(const float* __restrict__ outer,
                                                                               const float* __restrict__ inner, int64_t n,
                                                                               float world_size, const uint8_t* __restrict__ codes,
                                                                               const float* __restrict__ lut, float divisor,
                                                                               float* __restrict__ out, Workspace* ws) {
    using M = Mem<ALIGNED, NT>;
    __shared__ float s_lut[kBins];
    if (blockIdx.x == 0 && threadIdx.x == 0) ws->tile_counter = 0u;      // for the quantize pass that follows (sweep_tiles_dynamic)
    if (CODES) {
        for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut[b];
        __syncthreads();
    }
    const bool div = divisor != 1.0f;
    const int64_t nvec = n >> 2;
    constexpr int U = RECIP ? kUnroll : kDivUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    sweep_tiles<U>(nvec, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window win(out + base * 4, (nvec - base) * 16);
        f4a a[U], b[U];
        uint32_t c[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            a[j] = ok ? M::ldf4(outer, i) : f4a{0.f, 0.f, 0.f, 0.f};
            b[j] = ok ? M::ldf4(inner, i) : f4a{0.f, 0.f, 0.f, 0.f};
            if (CODES) c[j] = ok ? M::ldu32(codes, i) : 0u;
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            f4a v = RECIP ? (a[j] - b[j]) * world_size : (a[j] - b[j]) / world_size;
            if (CODES) {
                f4a l;
                l.x = s_lut[c[j] & 255];
                l.y = s_lut[(c[j] >> 8) & 255];
                l.z = s_lut[(c[j] >> 16) & 255];
                l.w = s_lut[c[j] >> 24];
                v += l;
                if (div) v = RECIP ? v * divisor : v / divisor;
            }
            if (full || i < nvec) {
                if (ALIGNED) win.template st128<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 16u, v);
                else M::stf4(out, i, v, false);
                if (j & 1) stats_add4(v, s1, q1); else stats_add4(v, s0, q0);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float v = RECIP ? (outer[i] - inner[i]) * world_size : (outer[i] - inner[i]) / world_size;
        if (CODES) {
            v += s_lut[codes[i]];
            if (div) v = RECIP ? v * divisor : v / divisor;
        }
        out[i] = v;
        const double d = v;
        s0 += d;
        q0 = fma(d, d, q0);
    }
    block_stats_store(s0 + s1, q0 + q1, ws, blockIdx.x);
}

// One element of the outer optimizer, torch.optim.SGD(lr, momentum, nesterov=True) as the
// reference builds it (src/zeroband/diloco.py:72-74) and libtorch's CPU kernels round it:
//   buf = buf * mu + g     (a product and a sum, each rounded; buf = g on the first step)
//   d   = fma(buf, mu, g)  (add with alpha: one rounding)
//   p   = fma(d, -lr, p)
__device__ __forceinline__ void outer_sgd_one(float& p, float& buf, float g, float neg_lr, float mu, bool first) {
    buf = first ? g : buf * mu + g;
    const float d = fmaf(buf, mu, g);
    p = fmaf(d, neg_lr, p);
}

// Outer step of DiLoCo on one bucket (diloco.py:212-215): SGD with Nesterov momentum on the
// outer parameters with the reduced pseudo-gradient, and the copy of the new parameters to
// the inner model (sync_inner_model, :137-144) in the same pass.  The gradient is fp32
// (24 bytes per element) or, with CODES, uint8 codes and their lookup table (21 bytes per
// element, and the dequantize pass is saved).
// outer_step_block is the pass for the calling workgroup as workgroup `slot` of a grid of G (s_lut: 256
// floats of LDS, used with CODES).
template <bool CODES, bool ALIGNED, bool NT, int POLICY, bool ONESHOT, int ST = CODES ? kCodesStepShotThreads : kStreamShotThreads,
          int SU = CODES ? kCodesStepShotRows : kStreamShotRows>
__device__ __forceinline__ void outer_step_block(float* __restrict__ param, float* __restrict__ mom, const float* __restrict__ grad,
                                                 const uint8_t* __restrict__ codes, const float* __restrict__ lut, float* __restrict__ inner,
                                                 int64_t n, float neg_lr, float mu, int first, int64_t slot, int64_t G, float* s_lut) {
    using M = Mem<ALIGNED, NT>;
    constexpr int T = ONESHOT ? ST : kThreads;
    constexpr int U = ONESHOT ? SU : kUnroll;
    if (CODES) {
        for (int b = threadIdx.x; b < kBins; b += T) s_lut[b] = lut[b];
        __syncthreads();
    }
    const int64_t nvec = n >> 2;
    walk_tiles_of<T, U, ONESHOT>(nvec, slot, G, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window wp(param + base * 4, (nvec - base) * 16), wm(mom + base * 4, (nvec - base) * 16),
            wi(inner ? inner + base * 4 : nullptr, inner ? (nvec - base) * 16 : 0);
        f4a p[U], m[U], g[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            p[j] = ok ? M::ldf4(param, i) : f4a{0.f, 0.f, 0.f, 0.f};
            m[j] = (ok && !first) ? M::ldf4(mom, i) : f4a{0.f, 0.f, 0.f, 0.f};
            if (CODES) {
                const uint32_t c = ok ? M::ldu32(codes, i) : 0u;
                g[j] = f4a{s_lut[c & 255], s_lut[(c >> 8) & 255], s_lut[(c >> 16) & 255], s_lut[c >> 24]};
            } else {
                g[j] = ok ? M::ldf4(grad, i) : f4a{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float pc = p[j][c], mc = m[j][c];
                    outer_sgd_one(pc, mc, g[j][c], neg_lr, mu, first);
                    p[j][c] = pc;
                    m[j][c] = mc;
                }
                if (ALIGNED) {
                    const uint32_t off = static_cast<uint32_t>(threadIdx.x + j * stride) * 16u;
                    wp.template st128<POLICY>(off, p[j]);
                    wm.template st128<POLICY>(off, m[j]);
                    wi.template st128<POLICY>(off, p[j]);      // an empty window without an inner model: dropped
                } else {
                    M::stf4(param, i, p[j], false);
                    M::stf4(mom, i, m[j], false);
                    if (inner) M::stf4(inner, i, p[j], true);
                }
            }
        }
    });
    if (slot == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float p = param[i];
        float m = first ? 0.f : mom[i];
        const float g = CODES ? s_lut[codes[i]] : grad[i];
        outer_sgd_one(p, m, g, neg_lr, mu, first);
        param[i] = p;
        mom[i] = m;
        if (inner) inner[i] = p;
    }
}

template <bool CODES, bool ALIGNED, bool NT, int POLICY, bool ONESHOT = false>
__global__ __launch_bounds__(ONESHOT ? (CODES ? kCodesStepShotThreads : kStreamShotThreads) : kThreads, ONESHOT ? 8 : kWavesPerSimd) void outer_step_kernel(float* __restrict__ param, float* __restrict__ mom, const float* __restrict__ grad,
                                       const uint8_t* __restrict__ codes, const float* __restrict__ lut, float* __restrict__ inner,
                                       int64_t n, float neg_lr, float mu, int first) {
    __shared__ float s_lut[CODES ? kBins : 1];
    outer_step_block<CODES, ALIGNED, NT, POLICY, ONESHOT>(param, mom, grad, codes, lut, inner, n, neg_lr, mu, first, blockIdx.x, gridDim.x, s_lut);
}

template <int POLICY, bool ONESHOT = false>
__global__ __launch_bounds__(ONESHOT ? kStreamShotThreads : kThreads, ONESHOT ? 8 : kWavesPerSimd) void copy_kernel(f4a* __restrict__ dst, const f4a* __restrict__ src, int64_t nvec) {
    using M = Mem<true, true>;
    constexpr int T = ONESHOT ? kStreamShotThreads : kThreads;
    constexpr int U = ONESHOT ? kStreamShotRows : kUnroll;
    walk_tiles<T, U, ONESHOT>(nvec, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window win(dst + base, (nvec - base) * 16);
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) v[j] = M::ldf4(reinterpret_cast<const float*>(src), i);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) win.template st128<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 16u, v[j]);
        }
    });
}
