// Work on received codes: requantization in the code domain (count, total, plan, remap) and the
// lookup dequantization (set / add, with statistics and division for the ring steps).
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

// ---- requantization in the code domain ----------------------------------------------------
// The all-gather forwards uniform_8bit_quantize(chunk) of a chunk that was just set to
// lut_in[codes_in] (collectives.cpp:204-215).  Such a chunk holds at most 256 distinct values, so
// its quantization is a function of the received codes alone: the statistics follow from the
// population of each code, the new code of an element from a 256-entry map, and a new lookup
// entry is the population-weighted mean of the old entries that map to it.  3 bytes per element
// (codes read twice, written once) instead of a pass over the fp32 chunk.

// 16 codes at vector index i; ALIGNED means both code buffers are 16-byte aligned.
template <bool ALIGNED>
__device__ __forceinline__ u4a ld_codes16(const uint8_t* p, int64_t i) {
    if (ALIGNED) return reinterpret_cast<const u4a*>(p)[i];
    const U4U t = reinterpret_cast<const U4U*>(p)[i];
    return u4a{t.x, t.y, t.z, t.w};
}

template <bool ALIGNED>
__device__ __forceinline__ void st_codes16(uint8_t* p, int64_t i, u4a v) {
    if (ALIGNED) __builtin_nontemporal_store(v, reinterpret_cast<u4a*>(p) + i);
    else reinterpret_cast<U4U*>(p)[i] = U4U{v.x, v.y, v.z, v.w};
}

// Pass 1: population of each code value, one partial per workgroup.  1 byte per element.
template <bool ALIGNED, int R>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void code_count_kernel(const uint8_t* __restrict__ codes, int64_t n,
                                                                              Workspace* ws) {
    __shared__ unsigned cnt[kBins * R];
    for (int i = threadIdx.x; i < kBins * R; i += kThreads) cnt[i] = 0u;
    __syncthreads();
    const int rep = threadIdx.x & (R - 1);
    auto bump = [&](uint32_t code) {
        __hip_atomic_fetch_add(&cnt[code * R + rep], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    const int64_t nvec = n >> 4;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        u4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? ld_codes16<ALIGNED>(codes, i) : u4a{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t w = v[j][k];
                    bump(w & 255);
                    bump((w >> 8) & 255);
                    bump((w >> 16) & 255);
                    bump(w >> 24);
                }
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 15)) bump(codes[(nvec << 4) + threadIdx.x]);
    __syncthreads();
    for (int b = threadIdx.x; b < kBins; b += kThreads) {
        unsigned c = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) c += cnt[b * R + r];
        ws->code_cnt[blockIdx.x][b] = c;
    }
}

// Between the passes, first kernel: total population of each code.  Workgroup j owns codes
// 4j .. 4j+3 (16 contiguous bytes of every partial); lane (row, code) adds partials row,
// row + 256, ..., then the rows are added up.
__global__ __launch_bounds__(kFinalThreads) void code_total_kernel(Workspace* ws, int nparts) {
    constexpr int kRows = kFinalThreads / kLutBinsPerBlock;
    __shared__ unsigned long long sh_cnt[kFinalThreads];
    const int bl = threadIdx.x % kLutBinsPerBlock;
    const int row = threadIdx.x / kLutBinsPerBlock;
    const int bin = blockIdx.x * kLutBinsPerBlock + bl;
    constexpr int kIters = kMaxGrid / kRows;
    uint32_t part[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {          // all loads in flight at once
        const int p = row + k * kRows;
        part[k] = p < nparts ? ws->code_cnt[p][bin] : 0u;
    }
    unsigned long long c = 0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) c += part[k];
    // integers: every wavefront joins the rows that share a row of sixteen lanes, the totals meet in LDS
    // behind one barrier and the first wavefront adds them
    c = sum_row_mod4(c);
    if ((threadIdx.x & 15) < kLutBinsPerBlock) sh_cnt[(threadIdx.x >> 4) * kLutBinsPerBlock + bl] = c;
    __syncthreads();
    if (threadIdx.x < 64) {
        unsigned long long t = 0;
#pragma unroll
        for (int k = 0; k < kFinalThreads / 256; ++k) t += sh_cnt[threadIdx.x + 64 * k];
        t = sum_lanes_mod4(t);
        if (row == 0) ws->code_total[bin] = t;
    }
}

// Between the passes, second kernel, one workgroup: the statistics
// sum = sum_c count_c * lut_in[c] and sumsq = sum_c count_c * lut_in[c]^2 in fp64, the scale
// (compression.cpp:113-116), the map old code -> new code (:23-24 applied to lut_in[c]) and the
// new lookup table (:99-101).  Entries of lut_in whose code does not occur are ignored.
__global__ __launch_bounds__(kFinalThreads) void requant_plan_kernel(Workspace* ws, const float* __restrict__ lut_in, int64_t n,
                                                                      float* __restrict__ lut_out, prime_qparams* qp_out) {
    struct Rec {
        double term;                 // count * value
        unsigned long long count;
        int target;                  // new code, -1 when the old code does not occur
        int pad;
    };
    constexpr int kGroups = kFinalThreads / kBins;
    constexpr int kSpan = kBins / kGroups;
    __shared__ Rec rec[kBins];
    __shared__ double sh_s[kBins / 64], sh_q[kBins / 64];
    __shared__ float sh_inv;
    __shared__ double g_sum[kGroups][kBins];
    __shared__ unsigned long long g_cnt[kGroups][kBins];
    const int bin = threadIdx.x & (kBins - 1);
    float v = 0.0f;
    unsigned long long t = 0;
    if (threadIdx.x < kBins) {
        t = ws->code_total[bin];
        v = lut_in[bin];
        double s = 0.0, q = 0.0;
        if (t) {
            const double dv = v, dc = static_cast<double>(t);
            s = dc * dv;
            q = dc * (dv * dv);
        }
        rec[bin].term = s;
        rec[bin].count = t;
        s = wave_sum(s);
        q = wave_sum(q);
        if ((threadIdx.x & 63) == 0) { sh_s[threadIdx.x >> 6] = s; sh_q[threadIdx.x >> 6] = q; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kBins / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        prime_qparams qp;
        finalize_qparams(S, Q, n, &qp);
        sh_inv = qp.inv_scale;
        ws->qp = qp;
        if (qp_out) *qp_out = qp;
    }
    __syncthreads();
    int target = 0;
    if (threadIdx.x < kBins) {
        target = quantize_code(v, sh_inv, kZeroPoint);
        rec[bin].target = t ? target : -1;
    }
    __syncthreads();
    {
        // new entry `bin`: population-weighted mean of the old entries that map to it; the 256 old
        // codes are split over kGroups groups of lanes, joined in a fixed order
        const int group = threadIdx.x / kBins;
        double sum = 0.0;
        unsigned long long k = 0;
#pragma unroll 16
        for (int j = 0; j < kSpan; ++j) {
            const Rec r = rec[group * kSpan + j];
            const bool hit = r.target == bin;
            sum += hit ? r.term : 0.0;
            k += hit ? r.count : 0ull;
        }
        g_sum[group][bin] = sum;
        g_cnt[group][bin] = k;
    }
    __syncthreads();
    if (threadIdx.x < kBins) {
        double sum = g_sum[0][bin];
        unsigned long long k = g_cnt[0][bin];
#pragma unroll
        for (int g = 1; g < kGroups; ++g) { sum += g_sum[g][bin]; k += g_cnt[g][bin]; }
        lut_out[bin] = k ? static_cast<float>(sum / static_cast<double>(k)) : 0.0f;
        // four adjacent lanes pack their new codes into one word of the map
        uint32_t word = static_cast<uint32_t>(target) << (8 * (bin & 3));
        word |= __shfl_xor(word, 1, 64);
        word |= __shfl_xor(word, 2, 64);
        if ((bin & 3) == 0) ws->code_map[bin >> 2] = word;
    }
}

// Pass 2: codes_out[i] = map[codes_in[i]].  2 bytes per element.  REVERSE: from the end of the codes, where the
// last-level cache still holds what the counting pass read last.
template <bool ALIGNED, bool REVERSE = false>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void code_remap_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out,
                                                                              int64_t n, const Workspace* __restrict__ ws) {
    __shared__ uint32_t map_words[kBins / 4];
    if (threadIdx.x < kBins / 4) map_words[threadIdx.x] = ws->code_map[threadIdx.x];
    __syncthreads();
    const uint8_t* map = reinterpret_cast<const uint8_t*>(map_words);
    auto remap = [&](uint32_t w) {
        return static_cast<uint32_t>(map[w & 255]) | (static_cast<uint32_t>(map[(w >> 8) & 255]) << 8) |
               (static_cast<uint32_t>(map[(w >> 16) & 255]) << 16) | (static_cast<uint32_t>(map[w >> 24]) << 24);
    };
    const int64_t nvec = n >> 4;
    sweep_tiles<kUnroll, REVERSE>(nvec, [&](int64_t base, int64_t stride, auto full_t) {
        const int64_t i0 = base + threadIdx.x;
        constexpr bool full = decltype(full_t)::value;
        u4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? ld_codes16<ALIGNED>(in, i) : u4a{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) st_codes16<ALIGNED>(out, i, u4a{remap(v[j].x), remap(v[j].y), remap(v[j].z), remap(v[j].w)});
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 15)) {
        const int64_t i = (nvec << 4) + threadIdx.x;
        out[i] = map[in[i]];
    }
}

// K5 / K4 pass A: out = lut[codes] (collectives.cpp:16-22) or out += lut[codes] (:8-14),
// the lookup table held in LDS; with STATS the fp64 sum and sum of squares of the updated
// values are taken in the same pass (the next quantization's scale).  With DIV the updated value
// is divided by `divisor` before it is stored and counted: chunk.div_(world_size) of
// ReduceOp::AVG (collectives.cpp:155-159) folded into the last accumulation of a chunk.
// POLICY is the cache policy of the fp32 stores.
// ONESHOT (never with STATS, whose partials are per workgroup of a small grid): one workgroup of
// kShotThreads lanes per tile instead of a loop.
// SHOT_ROWS: rows of a ONESHOT workgroup's tile.  The plain set does best with four up to 2^25 elements (2^23: 6.2
// against 7.5 us, 2^24: 13.1 against 15.4 us) and with two beyond (2^26: 54 against 58 us, 2^28: 211 against 242 us).
// dequant_block is the pass for the calling workgroup as workgroup `slot` of a grid of G would run it
// (s_lut: 256 floats of LDS; the statistics partial goes to part_sum[slot] / part_sq[slot]).
template <bool ADD, bool STATS, bool ALIGNED, bool NT, bool DIV, int POLICY, bool ONESHOT, int SHOT_ROWS, int SHOT_THREADS = kShotThreads>
__device__ __forceinline__ void dequant_block(float* __restrict__ out, const float* __restrict__ lut, const uint8_t* __restrict__ codes,
                                              int64_t n, double* part_sum, double* part_sq, float divisor, int slot, int G, float* s_lut) {
    static_assert(!(ONESHOT && STATS), "statistics partials need the small grid of the looping sweep");
    using M = Mem<ALIGNED, NT>;
    constexpr int T = ONESHOT ? SHOT_THREADS : kThreads;
    // The table goes to LDS once per workgroup.  A workgroup of the plain set that lives for one tile
    // issues the tile's loads before that, so that the table's trip to L2 runs beside the codes' trip
    // to memory instead of in front of it (2^28 elements: 210 instead of 233 us; with the accumulator's
    // loads in flight as well the order makes no difference or costs 1 % there).  The looping passes do
    // the same with their first tile: on a tensor of a few million elements the table's trip would
    // otherwise stand alone at the head of the kernel.
    constexpr bool kLateFill = (ONESHOT && !ADD) || !ONESHOT;
    bool filled = false;                 // uniform over the workgroup
    auto fill_lut = [&] {
        for (int b = threadIdx.x; b < kBins; b += T) s_lut[b] = lut[b];
        __syncthreads();
        filled = true;
    };
    if (!kLateFill) fill_lut();
    const int64_t nvec = n >> 2;
    constexpr int U = ONESHOT ? SHOT_ROWS : DIV ? kDivUnroll : kUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    walk_tiles_of<T, U, ONESHOT>(nvec, slot, G, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window win(out + base * 4, (nvec - base) * 16);
        uint32_t c[U];
        f4a a[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            c[j] = ok ? Mem<ALIGNED, true>::ldu32(codes, i) : 0u;      // a message is read once: never kept in cache
            if (ADD) a[j] = ok ? M::ldf4(out, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
        if (kLateFill && !filled) fill_lut();        // the workgroup's first tile: the barrier is uniform
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            f4a v;
            v.x = s_lut[c[j] & 255];
            v.y = s_lut[(c[j] >> 8) & 255];
            v.z = s_lut[(c[j] >> 16) & 255];
            v.w = s_lut[c[j] >> 24];
            if (ADD) v += a[j];
            if (DIV) v = v / divisor;
            if (full || i < nvec) {
                if (ALIGNED) win.template st128<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 16u, v);
                else M::stf4(out, i, v, false);
                if (STATS) {
                    if (j & 1) stats_add4(v, s1, q1); else stats_add4(v, s0, q0);
                }
            }
        }
    });
    if (slot == 0 && (n & 3) && !filled) fill_lut();      // a tensor of fewer than four elements: no tile at all
    if (slot == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float v = s_lut[codes[i]];
        if (ADD) v += out[i];
        if (DIV) v = v / divisor;
        out[i] = v;
        if (STATS) {
            const double d = v;
            s0 += d;
            q0 = fma(d, d, q0);
        }
    }
    if (STATS) block_stats_store(s0 + s1, q0 + q1, part_sum, part_sq, slot);
}

template <bool ADD, bool STATS, bool ALIGNED, bool NT, bool DIV, int POLICY, bool ONESHOT = false, int SHOT_ROWS = kShotUnroll,
          int SHOT_THREADS = kShotThreads>
__global__ __launch_bounds__(ONESHOT ? SHOT_THREADS : kThreads, ONESHOT ? 8 : kWavesPerSimd)
void dequant_kernel(float* __restrict__ out, const float* __restrict__ lut, const uint8_t* __restrict__ codes, int64_t n, Workspace* ws,
                    float divisor) {
    __shared__ float s_lut[kBins];
    if (STATS && blockIdx.x == 0 && threadIdx.x == 0) ws->tile_counter = 0u;      // for the quantize pass that follows (sweep_tiles_dynamic)
    dequant_block<ADD, STATS, ALIGNED, NT, DIV, POLICY, ONESHOT, SHOT_ROWS, SHOT_THREADS>(out, lut, codes, n, STATS ? ws->part_sum : nullptr,
                                                                           STATS ? ws->part_sq : nullptr, divisor, blockIdx.x, gridDim.x, s_lut);
}
