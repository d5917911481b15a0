// uniform_8bit_quantize of a small tensor in one launch of one workgroup: statistics, scale,
// codes, histogram and lookup table (compression.cpp:106-125) with the results of the three-launch
// sequence bit for bit.  The three launches give a tensor of up to kSmallSlots rows (of kThreads
// 16-byte vectors) one workgroup per row; here one workgroup takes their places one after the
// other - the same additions in the same order, the same partials - so nothing is handed from one
// workgroup to another and no launch waits for the one before it.  Each lane loads its vector of
// every row once and keeps it in registers for both passes; the per-row partials stay in
// registers and LDS.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

constexpr int kSmallSlots = 4;
static_assert(kThreads >= kBins && kSmallSlots <= 4, "the table's tree is written for four rows, one bin per lane");

__device__ __forceinline__ BinAcc binacc_add(BinAcc a, BinAcc b) { return BinAcc{a.sum + b.sum, a.cnt + b.cnt}; }

// What lut_finalize_kernel makes of the partials of rows 0..3 for one bin: each first added to 0.0,
// then row r with r + 2, then r with r + 1.  (Its tree first adds rows r + 128, r + 64, ... r + 4,
// which do not exist here and count as zero: adding them changes nothing.)
__device__ __forceinline__ float lut_entry_of_rows(const BinAcc (&part)[kSmallSlots], int rows) {
    BinAcc leaf[kSmallSlots];
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) leaf[r] = r < rows ? BinAcc{0.0 + part[r].sum, part[r].cnt} : BinAcc{0.0, 0ull};
    const BinAcc t = binacc_add(binacc_add(leaf[0], leaf[2]), binacc_add(leaf[1], leaf[3]));
    return t.cnt ? static_cast<float>(t.sum / static_cast<double>(t.cnt)) : 0.0f;
}

// `rows` <= kSmallSlots is the grid the three-launch sequence uses for this tensor: one workgroup per
// row of whole vectors (the last of them may be left with the ragged end only, or with nothing).
// SRC says where the values come from: the tensor as it stands (uniform_8bit_quantize), or a ring
// step's first pass folded in - x = lut_in[codes_in] (gather step), x += lut_in[codes_in] (reduce
// step), the same divided by `divisor` (the last accumulation of an averaged chunk) - with the
// updated values written back, as dequant_kernel<.., STATS, ..> does ahead of the quantize pass.
enum SmallSource { kSmallTensor = 0, kSmallSet = 1, kSmallAdd = 2, kSmallAddDiv = 3 };

template <bool ALIGNED, int SRC>
__global__ __launch_bounds__(kThreads) void uniform_small_kernel(float* __restrict__ x, int64_t n, int rows,
                                                                 prime_qparams* qp_out, uint8_t* __restrict__ codes,
                                                                 float* __restrict__ lut, Workspace* ws, int copies_shift,
                                                                 const uint8_t* codes_in, const float* lut_in,
                                                                 float divisor) {
    using M = Mem<ALIGNED, false>;
    __shared__ QuantHist hist;
    __shared__ double sh_s[kSmallSlots][kWaves];
    __shared__ double sh_q[kSmallSlots][kWaves];
    __shared__ double sh_part_s[kSmallSlots];
    __shared__ double sh_part_q[kSmallSlots];
    __shared__ float s_lut[SRC == kSmallTensor ? 1 : kBins];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nvec = n >> 2;
    const int tail = static_cast<int>(n & 3);
    if (SRC != kSmallTensor) {
        for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut_in[b];
        __syncthreads();
    }

    // the lane's vector of every row, and its element of the ragged end
    f4a v[kSmallSlots];
    bool has[kSmallSlots];
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) {
        const int64_t i = static_cast<int64_t>(r) * kThreads + threadIdx.x;
        has[r] = r < rows && i < nvec;
        v[r] = f4a{0.f, 0.f, 0.f, 0.f};
        if (SRC == kSmallTensor || SRC == kSmallAdd || SRC == kSmallAddDiv) {
            if (has[r]) v[r] = M::ldf4(x, i);
        }
        if (SRC != kSmallTensor && has[r]) {
            const uint32_t c = M::ldu32(codes_in, i);
            f4a l;
            l.x = s_lut[c & 255];
            l.y = s_lut[(c >> 8) & 255];
            l.z = s_lut[(c >> 16) & 255];
            l.w = s_lut[c >> 24];
            if (SRC == kSmallSet) v[r] = l;
            else v[r] = l + v[r];
            if (SRC == kSmallAddDiv) v[r] = v[r] / divisor;
            M::stf4(x, i, v[r], false);
        }
    }
    const bool has_tail = static_cast<int>(threadIdx.x) < tail;
    float tail_v = 0.0f;
    if (has_tail) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        if (SRC == kSmallTensor) {
            tail_v = x[i];
        } else {
            tail_v = s_lut[codes_in[i]];
            if (SRC != kSmallSet) tail_v += x[i];
            if (SRC == kSmallAddDiv) tail_v = tail_v / divisor;
            x[i] = tail_v;
        }
    }

    // statistics: per row what stats_partial computes for the workgroup of that row
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) {
        if (r >= rows) continue;         // uniform over the workgroup
        double s = 0.0, q = 0.0;
        stats_add4(v[r], s, q);
        if (r == 0 && has_tail) {
            const double t = tail_v;
            s += t;
            q = fma(t, t, q);
        }
        s = wave_sum(s + 0.0);           // the second accumulator pair of the streaming kernel stays at zero
        q = wave_sum(q + 0.0);
        if (lane == 0) { sh_s[r][wave] = s; sh_q[r][wave] = q; }
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < rows) {
        double S = sh_s[threadIdx.x][0], Q = sh_q[threadIdx.x][0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[threadIdx.x][w]; Q += sh_q[threadIdx.x][w]; }
        sh_part_s[threadIdx.x] = S;
        sh_part_q[threadIdx.x] = Q;
    }
    __syncthreads();
    // scale: lane i of the reduction brings the partial of workgroup i
    int narrow = INT_MIN;
    const bool mine = static_cast<int>(threadIdx.x) < rows;
    const double pa = (0.0 + (mine ? sh_part_s[threadIdx.x & (kSmallSlots - 1)] : 0.0)) + 0.0;
    const double pb = (0.0 + (mine ? sh_part_q[threadIdx.x & (kSmallSlots - 1)] : 0.0)) + 0.0;
    const float inv = block_scale_reduce<kThreads>(pa, pb, ws, n, qp_out, &narrow);

    // codes and histogram, row by row; the modes are those of quantize_block
    enum { kFixed, kFp, kBin0 };
    const int mode = !(__builtin_fabsf(inv) < __builtin_inff()) ? kBin0 : inv != 0.0f ? kFixed : kFp;
    const int shift = narrow != INT_MIN ? 3 : copies_shift;
    const int copy = threadIdx.x & ((1 << shift) - 1);
    BinAcc part[kSmallSlots];
    for (int r = 0; r < kSmallSlots; ++r) part[r] = BinAcc{0.0, 0ull};
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) {
        if (r < rows) {                   // uniform over the workgroup
            const int64_t i = static_cast<int64_t>(r) * kThreads + threadIdx.x;
            const int64_t ti = (nvec << 2) + threadIdx.x;
            if (mode == kFixed) {
                rhist_zero(hist.fixed, shift);
                __syncthreads();
                if (has[r]) M::stu32(codes, i, rhist_quantize4(hist.fixed, shift, copy, v[r], inv));
                if (r == 0 && has_tail) {
                    const int a = quantize_code(tail_v, inv, kZeroPoint);
                    codes[ti] = static_cast<uint8_t>(a);
                    const bool far = is_far(tail_v, inv);
                    if (far) rhist_add_far(hist.fixed, a, tail_v);
                    rhist_add(hist.fixed, shift, copy, a, far ? 0 : residual_fixed(tail_v, inv, a));
                }
                rhist_flush(hist.fixed, shift);
                if (threadIdx.x < kBins) part[r] = rhist_bin(hist.fixed, inv, threadIdx.x);
                __syncthreads();
            } else {
                int a = 0, b = 0, c = 0, d = 0;
                if (has[r]) {
                    a = quantize_code(v[r].x, inv, kZeroPoint);
                    b = quantize_code(v[r].y, inv, kZeroPoint);
                    c = quantize_code(v[r].z, inv, kZeroPoint);
                    d = quantize_code(v[r].w, inv, kZeroPoint);
                    M::stu32(codes, i, static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) | (static_cast<uint32_t>(c) << 16) |
                                           (static_cast<uint32_t>(d) << 24));
                }
                const int ta = (r == 0 && has_tail) ? quantize_code(tail_v, inv, kZeroPoint) : 0;
                if (r == 0 && has_tail) codes[ti] = static_cast<uint8_t>(ta);
                if (mode == kFp) {
                    hist_zero(hist.fp);
                    __syncthreads();
                    if (has[r]) {
                        hist_add(hist.fp, a, v[r].x);
                        hist_add(hist.fp, b, v[r].y);
                        hist_add(hist.fp, c, v[r].z);
                        hist_add(hist.fp, d, v[r].w);
                    }
                    if (r == 0 && has_tail) hist_add(hist.fp, ta, tail_v);
                    __syncthreads();
                    if (threadIdx.x < kBins) part[r] = hist_bin(hist.fp, threadIdx.x);
                    __syncthreads();
                } else {                  // every code is 0: one sum, lanes then wavefronts in the order of hist_store_bin0
                    double ls = 0.0;
                    unsigned long long lc = 0;
                    if (has[r]) {
                        ls += static_cast<double>(v[r].x);
                        ls += static_cast<double>(v[r].y);
                        ls += static_cast<double>(v[r].z);
                        ls += static_cast<double>(v[r].w);
                        lc += 4;
                    }
                    if (r == 0 && has_tail) { ls += static_cast<double>(tail_v); lc += 1; }
                    const BinAcc total = block_sum_bin0(ls, lc);
                    if (threadIdx.x == 0) part[r] = total;
                }
            }
        }
    }
    if (threadIdx.x < kBins) lut[threadIdx.x] = lut_entry_of_rows(part, rows);
}
