// Quantization to uint8 codes with the 256-bin sum / count histogram, the lookup-table second
// stage, the histogram under given codes (average_buckets) and the one-workgroup-per-tensor
// kernel for many small tensors.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

// The workgroup's total of a per-lane fp64 sum and element count, in lane 0: lanes of a wavefront by
// shuffles, then the wavefronts in order.  Two barriers; every lane calls it.
__device__ __forceinline__ BinAcc block_sum_bin0(double s, unsigned long long c) {
    __shared__ double sh_s[kWaves];
    __shared__ unsigned long long sh_c[kWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    s = wave_sum(s);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_down(c, off, 64);
    if (lane == 0) { sh_s[wave] = s; sh_c[wave] = c; }
    __syncthreads();
    BinAcc acc{0.0, 0ull};
    if (threadIdx.x == 0)
        for (int w = 0; w < kWaves; ++w) { acc.sum += sh_s[w]; acc.cnt += sh_c[w]; }
    __syncthreads();
    return acc;
}

// One (sum, count) pair for bin 0 as the workgroup's whole histogram partial: every lane brings the
// fp64 sum and the number of the elements it saw.
__device__ __forceinline__ void hist_store_bin0(double s, unsigned long long c, BinAcc* __restrict__ row) {
    const BinAcc total = block_sum_bin0(s, c);
    for (int b = threadIdx.x; b < kBins; b += kThreads) row[b] = b == 0 ? total : BinAcc{0.0, 0ull};
}

// Where a workgroup of the quantize pass leaves its histogram partial: 256 bin entries (BinPart when
// the histogram is the fixed-point one, BinAcc otherwise), the far elements, and - from the workgroup
// with `first` set - the form of the partials for the kernel that reads them.
struct HistOut {
    BinAcc* row;
    FarSlot far;
    HistInfo* info;
    bool first;
    unsigned* tile_counter;     // deals the last part of the tiles on demand (sweep_tiles_dynamic); null: all round-robin
    int dyn_percent;
    int mix_rounds = 0;         // rounds of tiles at the tensor's end that the last-level cache holds (sweep_tiles_dynamic)
    bool cleared = false;       // the caller has zeroed the fixed-point histogram (all copies) ahead of a barrier
};
__device__ __forceinline__ HistOut hist_out_of(Workspace* ws, int slot, int dyn_percent) {
    return HistOut{ws ? ws->hist[slot] : nullptr, FarSlot{ws ? &ws->far_sum[0][slot] : nullptr, ws ? &ws->far_cnt[0][slot] : nullptr}, ws ? &ws->hist_info : nullptr, slot == 0,
                   ws && dyn_percent > 0 ? &ws->tile_counter : nullptr, dyn_percent};
}

// K2 (+K3 when HIST): quantize to uint8, 4 codes packed per 32-bit store, and the 256-bin
// sum / count histogram of the same elements.  5 bytes per element.  REVERSE walks the tensor from
// its end (for the pass that follows a pass over the same tensor); POLICY is the cache policy of
// the code stores.  The histogram is the fixed-point one (one LDS atomic per element, 2^copies_shift
// copies of each bin, eight when the statistics show a tensor crowded into a few bins) whenever
// 1 / scale is a finite non-zero number.  When 1 / scale is infinite or not a number (scale 0: an
// all-zero tensor) every element has code 0 and the histogram is one sum; a zero 1 / scale (an
// infinite scale: a single element) takes the fp64 histogram.
// quantize_block is the pass itself for the calling workgroup's share of the tensor, given 1 / scale
// (`narrow` is INT_MIN unless the statistics show a tensor crowded into a few codes), as workgroup
// `slot` of a grid of G would run it.
// The workgroup's histogram memory: the fixed-point histogram or, for a zero 1 / scale, the fp64 one.
constexpr int kFpCopies = 8;
union QuantHist {
    ResidualHist fixed;
    LdsHist<kFpCopies> fp;
};

template <bool ALIGNED, bool NT, bool HIST, bool REVERSE, int POLICY, int U = kUnroll>
__device__ __forceinline__ void quantize_block(const float* __restrict__ x, int64_t n, float inv, int narrow, int zero_point,
                                               uint8_t* __restrict__ codes, const HistOut out_part, int copies_shift, int slot, int G,
                                               QuantHist& hist) {
    using M = Mem<ALIGNED, NT>;
    enum { kPlain, kFixed, kFp, kBin0 };
    const int mode = !HIST ? kPlain : !(__builtin_fabsf(inv) < __builtin_inff()) ? kBin0 : inv != 0.0f ? kFixed : kFp;
    const int shift = narrow != INT_MIN ? 3 : copies_shift;        // 8 = kMaxCopies
    const int copy = threadIdx.x & ((1 << shift) - 1);
    if (HIST && !(out_part.cleared && mode == kFixed)) {      // cleared: by the caller, ahead of a barrier
        if (mode == kFixed) rhist_zero(hist.fixed, shift);
        else if (mode == kFp) hist_zero(hist.fp);
        __syncthreads();
    }
    const int64_t nvec = n >> 2;
    double lane_sum = 0.0;               // kBin0
    unsigned long long lane_cnt = 0;
    auto pass = [&](auto mode_t) {
        constexpr int kMode = decltype(mode_t)::value;
        int since_flush = 0;
        const int flush_rounds = kMode == kFixed ? ResidualHist::flush_rounds(shift) : 0;
        auto body = [&](int64_t base, int64_t stride, auto full_t) {
            constexpr bool full = decltype(full_t)::value;
            const int64_t i0 = base + threadIdx.x;
            const Window out(codes + base * 4, (nvec - base) * 4);
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
                    uint32_t word;
                    int a = 0, b = 0, c = 0, d = 0;
                    if (kMode == kFixed) {          // the histogram always has zero point 128 (compression.cpp:107)
                        word = rhist_quantize4(hist.fixed, shift, copy, v[j], inv);
                    } else {
                        a = quantize_code(v[j].x, inv, zero_point);
                        b = quantize_code(v[j].y, inv, zero_point);
                        c = quantize_code(v[j].z, inv, zero_point);
                        d = quantize_code(v[j].w, inv, zero_point);
                        word = static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) | (static_cast<uint32_t>(c) << 16) |
                               (static_cast<uint32_t>(d) << 24);
                    }
                    if (ALIGNED) out.template st32<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 4u, word);
                    else M::stu32(codes, i, word);
                    if (kMode == kFp) {
                        hist_add(hist.fp, a, v[j].x);
                        hist_add(hist.fp, b, v[j].y);
                        hist_add(hist.fp, c, v[j].z);
                        hist_add(hist.fp, d, v[j].w);
                    } else if (kMode == kBin0) {
                        lane_sum += static_cast<double>(v[j].x);
                        lane_sum += static_cast<double>(v[j].y);
                        lane_sum += static_cast<double>(v[j].z);
                        lane_sum += static_cast<double>(v[j].w);
                        lane_cnt += 4;
                    }
                }
            }
            if (kMode == kFixed && full && ++since_flush == flush_rounds) {
                rhist_flush(hist.fixed, shift);       // every lane of the workgroup runs the same rounds
                since_flush = 0;
            }
        };
        // the fixed-point histogram's partials are integers: its tiles may go to any workgroup
        if constexpr (kMode == kFixed) sweep_tiles_dynamic<U, REVERSE>(nvec, slot, G, out_part.tile_counter, out_part.dyn_percent, body, out_part.mix_rounds);
        else sweep_tiles_of<U, REVERSE>(nvec, slot, G, body);
        if (slot == 0 && threadIdx.x < (n & 3)) {
            const int64_t i = (nvec << 2) + threadIdx.x;
            const float v = x[i];
            const int a = quantize_code(v, inv, zero_point);
            codes[i] = static_cast<uint8_t>(a);
            if (kMode == kFixed) {
                const bool far = is_far(v, inv);
                if (far) rhist_add_far(hist.fixed, a, v);
                rhist_add(hist.fixed, shift, copy, a, far ? 0 : residual_fixed(v, inv, a));
            } else if (kMode == kFp) {
                hist_add(hist.fp, a, v);
            } else if (kMode == kBin0) {
                lane_sum += static_cast<double>(v);
                lane_cnt += 1;
            }
        }
    };
    if (mode == kFixed) pass(std::integral_constant<int, kFixed>{});
    else if (mode == kFp) pass(std::integral_constant<int, kFp>{});
    else if (mode == kBin0) pass(std::integral_constant<int, kBin0>{});
    else pass(std::integral_constant<int, kPlain>{});
    if (HIST) {
        if (out_part.first && threadIdx.x == 0) *out_part.info = HistInfo{inv, mode == kFixed ? kHistFixed : kHistFp};
        if (mode == kFixed) {
            rhist_store(hist.fixed, shift, reinterpret_cast<BinPart*>(out_part.row), out_part.far);
        } else if (mode == kFp) {
            __syncthreads();
            hist_store(hist.fp, out_part.row);
        } else {
            hist_store_bin0(lane_sum, lane_cnt, out_part.row);
        }
    }
}

// U = rows per tile, as for stats_kernel (2^26 elements: 46.5 against 49.7 us with 2; 2^28: 217 against 245 us with 4).
template <bool ALIGNED, bool NT, bool HIST, bool REVERSE, int POLICY, int U = kUnroll>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void quantize_kernel(const float* __restrict__ x, int64_t n, float scale_val,
                                                            int stats_parts, prime_qparams* qp_out, int zero_point,
                                                            uint8_t* __restrict__ codes, Workspace* ws, int copies_shift, int dyn_percent,
                                                            int mix_rounds) {
    // the scale: given by value, or derived here from the statistics partials of the pass before
    // (stats_parts < 0: the record a preceding kernel left in the workspace)
    int narrow = INT_MIN;                // set when the statistics show a tensor crowded into a few codes
    __shared__ std::conditional_t<HIST, QuantHist, int> hist_mem;      // no histogram memory without HIST
    // the histogram is cleared while the statistics partials are on their way (all copies: how many the pass
    // uses depends on the statistics)
    auto clear = [&]() {
        if constexpr (HIST) rhist_zero(reinterpret_cast<QuantHist&>(hist_mem).fixed, 3);
    };
    const float inv = stats_parts > 0   ? block_scale_from_partials<kThreads>(ws, stats_parts, n, qp_out, &narrow, clear)
                      : stats_parts < 0 ? ws->qp.inv_scale
                                        : 1.0f / scale_val;
    HistOut out = hist_out_of(HIST ? ws : nullptr, blockIdx.x, dyn_percent);
    out.cleared = HIST && stats_parts > 0;
    out.mix_rounds = mix_rounds;
    quantize_block<ALIGNED, NT, HIST, REVERSE, POLICY, U>(x, n, inv, narrow, zero_point, codes, out, copies_shift, blockIdx.x, gridDim.x,
                                                       reinterpret_cast<QuantHist&>(hist_mem));
}

// K2 with the scale given and no histogram (quantize_per_tensor_uint8, compression.cpp:9-43), one
// workgroup per tile: a pass that keeps nothing between tiles does not need the loop.
template <int POLICY>
__global__ __launch_bounds__(kShotThreads, 8) void quantize_shot_kernel(const float* __restrict__ x, int64_t n, float scale_val, int zero_point,
                                                                    uint8_t* __restrict__ codes) {
    using M = Mem<true, true>;
    const float inv = 1.0f / scale_val;
    const int64_t nvec = n >> 2;
    walk_tiles<kShotThreads, kShotUnroll, true>(nvec, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        const Window out(codes + base * 4, (nvec - base) * 4);
        f4a v[kShotUnroll];
#pragma unroll
        for (int j = 0; j < kShotUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < kShotUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
                const uint32_t a = quantize_code(v[j].x, inv, zero_point), b = quantize_code(v[j].y, inv, zero_point),
                               c = quantize_code(v[j].z, inv, zero_point), d = quantize_code(v[j].w, inv, zero_point);
                out.template st32<POLICY>(static_cast<uint32_t>(threadIdx.x + j * stride) * 4u, a | (b << 8) | (c << 16) | (d << 24));
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        codes[i] = static_cast<uint8_t>(quantize_code(x[i], inv, zero_point));
    }
}

// K3 alone: histogram of x under caller-supplied codes (average_buckets).  5 bytes per element.
// ALLBINS: the table has all 256 bins, so no code is left out and the additions need no predicate.
template <bool ALIGNED, int R, bool NT, bool ALLBINS>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void hist_kernel(const float* __restrict__ x, const uint8_t* __restrict__ codes,
                                                        int64_t n, int n_bins, Workspace* ws) {
    using M = Mem<ALIGNED, NT>;
    __shared__ LdsHist<R> hist;
    hist_zero(hist);
    __syncthreads();
    const int64_t nvec = n >> 2;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a v[kUnroll];
        uint32_t c[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            v[j] = ok ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
            c[j] = ok ? M::ldu32(codes, i) : 0u;
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
                const int a = c[j] & 255, b = (c[j] >> 8) & 255, cc = (c[j] >> 16) & 255, d = c[j] >> 24;
                if (ALLBINS || a < n_bins) hist_add(hist, a, v[j].x);     // compression.cpp:70
                if (ALLBINS || b < n_bins) hist_add(hist, b, v[j].y);
                if (ALLBINS || cc < n_bins) hist_add(hist, cc, v[j].z);
                if (ALLBINS || d < n_bins) hist_add(hist, d, v[j].w);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        const int a = codes[i];
        if (a < n_bins) hist_add(hist, a, x[i]);
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x == 0) ws->hist_info = HistInfo{0.0f, kHistFp};
    hist_store(hist, ws->hist[blockIdx.x]);
}

// Second stage of the lookup build.  Workgroup j owns bins 4j .. 4j+3 (64 contiguous bytes
// of every partial): lane (row, bin) adds partials row, row + THREADS / 4, ... and the rows are
// then added up.  Mean = fp64 sum / count rounded to float once; an empty bin gives 0.0f
// (compression.cpp:100).  Entries >= 256 of a longer table are 0.0f.  Fixed-point partials
// (BinPart) are added as integers, the far elements of the two clip bins beside them, and
// converted once (fixed_bin_sum).
// Two shapes: 1024 lanes for up to kMaxGrid partials, 256 lanes for up to 256 (every launch of
// the default options): with four wavefronts instead of sixteen, each on a SIMD of its own, the
// chain from the partials' arrival to the table is shorter.  fp64 partials are added in one
// order in both: as a binary tree over 256 rows that pairs rows 128 apart first and neighbours
// last (row r += row r + h for h = 128, 64, ..., 1), row r being the sum of partials r, r + 256, ...
template <int THREADS, int MAXPARTS>
__global__ __launch_bounds__(THREADS) void lut_finalize_kernel(Workspace* __restrict__ ws, int nparts,
                                                                float* __restrict__ lut, int64_t n_bins,
                                                                unsigned long long* __restrict__ counts) {
    // the fused pass of this call may have dealt tiles through the workspace's counter: left at zero for the next
    // call's (the passes that write statistics partials reset it as well)
    if (blockIdx.x == 0 && threadIdx.x == 0) ws->tile_counter = 0u;
    constexpr int kRows = THREADS / kLutBinsPerBlock;
    constexpr int kWavesHere = THREADS / 64;
    constexpr int kIters = MAXPARTS / kRows;
    static_assert((THREADS == 1024 && MAXPARTS == kMaxGrid) || (THREADS == 256 && MAXPARTS == 256), "the two shapes");
    __shared__ double sh_sum[THREADS];                       // fixed-point partials: the upper halves' total, as an integer
    __shared__ unsigned long long sh_lo[THREADS];
    __shared__ unsigned long long sh_cnt[THREADS];
    __shared__ double sh_far_s;
    __shared__ unsigned long long sh_far_n;
    const int bl = threadIdx.x % kLutBinsPerBlock;
    const int row = threadIdx.x / kLutBinsPerBlock;
    const int bin = blockIdx.x * kLutBinsPerBlock + bl;
    const HistInfo info = ws->hist_info;        // first of the loads: it is back when the partials are
    BinAcc part[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {          // all loads in flight at once
        const int p = row + k * kRows;
        part[k] = p < nparts ? ws->hist[p][bin] : BinAcc{0.0, 0ull};
    }
    // the far elements of bin 0 / 255 (fixed-point partials only; harmless to read otherwise): the last wavefront
    // of the workgroup that owns the bin adds them up, its loads in flight with everybody's
    const bool clip_block = blockIdx.x == 0 || blockIdx.x == kBins / kLutBinsPerBlock - 1;
    if (clip_block && threadIdx.x >= THREADS - 64) {
        double fs;
        unsigned long long fn;
        far_totals(ws, 0, nparts, blockIdx.x != 0, fs, fn);
        if (threadIdx.x == THREADS - 64) { sh_far_s = fs; sh_far_n = fn; }
    }
    const bool fixed = info.mode == kHistFixed;
    unsigned long long c = 0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) c += part[k].cnt;
    if (fixed) {
        // Integer partials: any order of addition gives the same totals.  Every wavefront adds the four rows
        // that share a row of sixteen lanes by data-parallel moves and leaves 16 totals (4 per bin) in LDS; one
        // barrier; the first wavefront adds them.
        long long hi = 0;
        unsigned long long lo = 0;
#pragma unroll
        for (int k = 0; k < kIters; ++k) {
            const long long u = __double_as_longlong(part[k].sum);     // BinPart::units
            hi += units_hi(u);
            lo += units_lo(u);
        }
        c = sum_row_mod4(c);
        lo = sum_row_mod4(lo);
        hi = static_cast<long long>(sum_row_mod4(static_cast<unsigned long long>(hi)));
        if ((threadIdx.x & 15) < kLutBinsPerBlock) {
            const int slot = (threadIdx.x >> 4) * kLutBinsPerBlock + bl;      // (wavefront, row of lanes, bin)
            sh_cnt[slot] = c;
            sh_lo[slot] = lo;
            sh_sum[slot] = __longlong_as_double(hi);
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            unsigned long long cc = 0, ll = 0;
            long long hh = 0;
#pragma unroll
            for (int k = 0; k < kWavesHere / 4; ++k) {        // kWavesHere * 16 slots, 64 per step; slot % 4 is the lane's bin
                cc += sh_cnt[threadIdx.x + 64 * k];
                ll += sh_lo[threadIdx.x + 64 * k];
                hh += __double_as_longlong(sh_sum[threadIdx.x + 64 * k]);
            }
            cc = sum_lanes_mod4(cc);
            ll = sum_lanes_mod4(ll);
            hh = static_cast<long long>(sum_lanes_mod4(static_cast<unsigned long long>(hh)));
            if (row == 0 && bin < n_bins) {
                const bool far_bin = bin == 0 || bin == kBins - 1;
                lut[bin] = mean_entry(fixed_bin_sum(cc, hh, ll, far_bin ? sh_far_n : 0ull, far_bin ? sh_far_s : 0.0, info.inv, bin), cc);
                if (counts) counts[bin] = cc;
            }
        }
    } else {
        // fp64 partials (rare: a zero or non-finite 1 / scale, or codes given by the caller), the fixed tree.
        // One barrier: the first wavefront, whose lane (r, bin) holds row r < 16, adds the rows r + 16 w of the
        // other wavefronts from LDS (the steps down to h = 16), then the lanes are joined by exchanges at
        // distances 32, 16, 8 and 4 (h = 8 .. 1).
        double s;
        if constexpr (THREADS == 1024) {
            s = 0.0;
#pragma unroll
            for (int k = 0; k < kIters; ++k) s += part[k].sum;
        } else {
            // row r of the tree is partial r alone here; this lane holds rows row, row + 64, row + 128, row + 192
            s = (part[0].sum + part[2].sum) + (part[1].sum + part[3].sum);      // h = 128, then h = 64
        }
        sh_cnt[threadIdx.x] = c;
        sh_sum[threadIdx.x] = s;
        __syncthreads();
        if (threadIdx.x < 64) {
            unsigned long long cw[kWavesHere];
            double sw[kWavesHere];
#pragma unroll
            for (int w = 0; w < kWavesHere; ++w) {
                cw[w] = sh_cnt[threadIdx.x + 64 * w];
                sw[w] = sh_sum[threadIdx.x + 64 * w];
            }
#pragma unroll
            for (int h = kWavesHere / 2; h > 0; h >>= 1) {
#pragma unroll
                for (int i = 0; i < h; ++i) {
                    cw[i] += cw[i + h];
                    sw[i] += sw[i + h];
                }
            }
            unsigned long long cc = cw[0];
            double sum = sw[0];
#pragma unroll
            for (int d = 32; d >= kLutBinsPerBlock; d >>= 1) {
                cc += __shfl_xor(cc, d, 64);
                sum += __shfl_xor(sum, d, 64);
            }
            if (row == 0 && bin < n_bins) {
                lut[bin] = mean_entry(sum, cc);
                if (counts) counts[bin] = cc;
            }
        }
    }
    if (blockIdx.x == 0)
        for (int64_t b = kBins + threadIdx.x; b < n_bins; b += THREADS) lut[b] = 0.0f;
}

__global__ void lut_zero_kernel(float* __restrict__ lut, int64_t n_bins, unsigned long long* __restrict__ counts) {
    for (int64_t b = threadIdx.x; b < n_bins; b += blockDim.x) {
        lut[b] = 0.0f;
        if (counts && b < kBins) counts[b] = 0ull;
    }
}

// Small tensors: one workgroup per tensor of a flat buffer does the whole of
// uniform_8bit_quantize (statistics, scale, codes, lookup) without touching the workspace.
// With VEC (flat buffer 16-byte aligned, code buffer 4-byte aligned) the part of the tensor
// between its first and last multiple-of-4 global index is read as 16-byte vectors and its
// codes stored 4 at a time; the ragged ends, which share vectors with the neighbouring
// tensors, go element by element.  The second read of a tensor comes from L2.
template <bool VEC>
__global__ __launch_bounds__(kBatchThreads) void batched_kernel(const float* __restrict__ x, const int64_t* __restrict__ offsets,
                                                                uint8_t* __restrict__ codes, float* __restrict__ luts,
                                                                prime_qparams* __restrict__ qps) {
    constexpr int R = 4;
    union Hist {
        LdsHist<R> fp;                    // a zero or non-finite 1 / scale
        ResidualHist fixed;               // everything else: one 64-bit LDS atomic per element, or none for a hot code
    };
    __shared__ Hist hist_mem;
    LdsHist<R>& hist = hist_mem.fp;
    __shared__ double sh_s[kBatchThreads / 64];
    __shared__ double sh_q[kBatchThreads / 64];
    __shared__ prime_qparams sh_qp;
    __shared__ int sh_hot_base;          // >= -1: the tensor is narrow, hot codes start here; INT_MIN: it is not
    const int64_t t = blockIdx.x;
    const int64_t lo = offsets[t];
    const int64_t hi = offsets[t + 1];
    const int64_t n = hi - lo;
    // [lo, a) and [b, hi) element by element, [a, b) as vectors
    int64_t a = VEC ? (lo + 3) & ~int64_t(3) : hi;
    int64_t b = VEC ? hi & ~int64_t(3) : hi;
    if (a > b) { a = hi; b = hi; }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    const f4a* __restrict__ x4 = reinterpret_cast<const f4a*>(x);
    constexpr int U = 4;
    for (int64_t v0 = (a >> 2) + threadIdx.x; v0 < (b >> 2); v0 += kBatchThreads * U) {
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            v[j] = i < (b >> 2) ? x4[i] : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (j & 1) stats_add4(v[j], s1, q1); else stats_add4(v[j], s0, q0);
        }
    }
    for (int64_t i = lo + threadIdx.x; i < a; i += kBatchThreads) {        // ragged head (everything without VEC)
        const double v = x[i];
        s0 += v;
        q0 = fma(v, v, q0);
    }
    for (int64_t i = b + threadIdx.x; i < hi; i += kBatchThreads) {        // ragged tail
        const double v = x[i];
        s1 += v;
        q1 = fma(v, v, q1);
    }
    double s = wave_sum(s0 + s1);
    double q = wave_sum(q0 + q1);
    if (lane == 0) { sh_s[wave] = s; sh_q[wave] = q; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kBatchThreads / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        finalize_qparams(S, Q, n, &sh_qp);
        if (qps) qps[t] = sh_qp;
        sh_hot_base = narrow_distribution(S, Q, n)
                          ? quantize_code(static_cast<float>(S / static_cast<double>(n)), sh_qp.inv_scale, kZeroPoint) - 1
                          : INT_MIN;
    }
    __syncthreads();
    const float inv = sh_qp.inv_scale;
    uint32_t* __restrict__ c4 = reinterpret_cast<uint32_t*>(codes);
    if (__builtin_fabsf(inv) < __builtin_inff() && inv != 0.0f) {
        // the fixed-point histogram (ResidualHist): one 64-bit LDS atomic per element, eight copies of each bin
        // for a tensor crowded into a few codes (measured ahead of keeping those codes' sums in registers:
        // 103 against 124 us for the 2,000 tensors of N(1, 1e-2))
        ResidualHist& h = hist_mem.fixed;
        const int shift = sh_hot_base != INT_MIN ? 3 : 2;
        const int copy = threadIdx.x & ((1 << shift) - 1);
        rhist_zero<kBatchThreads>(h, shift);
        __syncthreads();
        // a slot holds 65535 additions: a round adds at most 16 elements per lane and (kBatchThreads >> shift)
        // lanes share a slot
        constexpr int kFlushRounds = 30;
        static_assert((kBatchThreads >> 2) * 16 * (kFlushRounds + 1) < 65535, "a slot must hold the rounds between two flushes");
        int since = 0;
        for (int64_t base = a >> 2; base < (b >> 2); base += kBatchThreads * U) {      // the same trip count in every lane
            f4a v[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int64_t i = base + threadIdx.x + j * kBatchThreads;
                v[j] = i < (b >> 2) ? x4[i] : f4a{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int64_t i = base + threadIdx.x + j * kBatchThreads;
                if (i < (b >> 2)) c4[i] = rhist_quantize4(h, shift, copy, v[j], inv);
            }
            if (++since == kFlushRounds) {
                rhist_flush(h, shift);
                since = 0;
            }
        }
        for (int part = 0; part < 2; ++part) {         // the ragged ends: at most three elements each
            const int64_t from = part ? b : lo, to = part ? hi : a;
            for (int64_t i = from + threadIdx.x; i < to; i += kBatchThreads) {
                const float v = x[i];
                const int c = quantize_code(v, inv, kZeroPoint);
                codes[i] = static_cast<uint8_t>(c);
                const bool far = is_far(v, inv);
                if (far) rhist_add_far(h, c, v);
                rhist_add(h, shift, copy, c, far ? 0 : residual_fixed(v, inv, c));
            }
        }
        rhist_flush(h, shift);
        for (int bin = threadIdx.x; bin < kBins; bin += kBatchThreads) {
            unsigned long long far_n = 0;
            double far_s = 0.0;
            if (bin == 0 || bin == kBins - 1) rhist_far_side(h, bin != 0, far_n, far_s);
            const unsigned long long cnt = h.wide_cnt[bin];
            luts[t * kBins + bin] = mean_entry(fixed_bin_sum(cnt, units_hi(h.wide_sum[bin]), units_lo(h.wide_sum[bin]), far_n, far_s, inv, bin), cnt);
        }
        return;
    }
    for (int i = threadIdx.x; i < kBins * R; i += kBatchThreads) { hist.sum[i] = 0.0; hist.cnt[i] = 0u; }
    __syncthreads();
    auto second_pass = [&](auto narrow_t) {
    constexpr bool narrow = decltype(narrow_t)::value;
    HotCodes hot;
    hot.base = sh_hot_base;
    auto add = [&](int code, float xv) {
        if (narrow) hist_add_hot(hist, hot, code, xv);
        else hist_add(hist, code, xv);
    };
    for (int64_t v0 = (a >> 2) + threadIdx.x; v0 < (b >> 2); v0 += kBatchThreads * U) {
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            v[j] = i < (b >> 2) ? x4[i] : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            if (i < (b >> 2)) {
                const int ca = quantize_code(v[j].x, inv, kZeroPoint);
                const int cb = quantize_code(v[j].y, inv, kZeroPoint);
                const int cc = quantize_code(v[j].z, inv, kZeroPoint);
                const int cd = quantize_code(v[j].w, inv, kZeroPoint);
                c4[i] = static_cast<uint32_t>(ca) | (static_cast<uint32_t>(cb) << 8) | (static_cast<uint32_t>(cc) << 16) |
                        (static_cast<uint32_t>(cd) << 24);
                add(ca, v[j].x);
                add(cb, v[j].y);
                add(cc, v[j].z);
                add(cd, v[j].w);
            }
        }
    }
    for (int part = 0; part < 2; ++part) {
        const int64_t from = part ? b : lo, to = part ? hi : a;
        for (int64_t i = from + threadIdx.x; i < to; i += kBatchThreads) {
            const float v = x[i];
            const int c = quantize_code(v, inv, kZeroPoint);
            codes[i] = static_cast<uint8_t>(c);
            add(c, v);
        }
    }
    if (narrow) hist_flush_hot(hist, hot);
    };
    if (sh_hot_base != INT_MIN) second_pass(std::true_type{});
    else second_pass(std::false_type{});
    __syncthreads();
    for (int bin = threadIdx.x; bin < kBins; bin += kBatchThreads) {
        double sum = 0.0;
        unsigned long long cnt = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) { sum += hist.sum[bin * R + r]; cnt += hist.cnt[bin * R + r]; }
        luts[t * kBins + bin] = cnt ? static_cast<float>(sum / static_cast<double>(cnt)) : 0.0f;
    }
}
