/*
 * prime_hip.h - C ABI of libprime_hip.so: the int8 (uint8 code + 256-entry fp32 lookup)
 * pseudo-gradient compression path on MI355X (gfx950).
 *
 * Every entry point enqueues HIP kernels on `stream` (a hipStream_t passed as void*; NULL is
 * the default stream) and returns without synchronising.  All pointers are device pointers
 * unless a comment says otherwise.  The library never allocates or frees memory: the caller
 * owns inputs, outputs and the workspace.  Return value: 0 on success, a positive hipError_t
 * on a HIP failure, a negative PRIME_E* on a rejected argument; prime_hip_last_error() gives
 * the text for the calling thread.
 *
 * Reference interfaces these entry points stand in for (paths relative to the reference
 * checkout) are cited per function.  n_bins is 256 and zero_point 128 throughout
 * (src/zeroband/C/csrc/compression.cpp:5,107) unless passed explicitly.
 */
#ifndef PRIME_HIP_H
#define PRIME_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PRIME_HIP_ABI_VERSION 2

#define PRIME_EINVAL (-1)   /* null pointer, negative size, bad n_bins ... */
#define PRIME_EWORKSPACE (-2) /* workspace missing, too small or not initialised */

typedef void* prime_stream_t; /* hipStream_t */

/* What the statistics pass leaves on the device for the quantizer (32 bytes). */
typedef struct prime_qparams {
    float scale;      /* float(6 * std / 256), compression.cpp:116,119 */
    float inv_scale;  /* 1.0f / scale, compression.cpp:16 */
    double sum;       /* sum of x   (fp64) */
    double sumsq;     /* sum of x*x (fp64) */
    int64_t n;
} prime_qparams;

int prime_hip_abi_version(void);
const char* prime_hip_last_error(void);

/* Tuning knobs: "blocks_per_cu" (workgroups per compute unit of a streaming kernel),
 * "large_read_grid_eighths" / "large_read_min_mi_elems" (kernels that read at least as much as they
 * write use this many eighths of the compute units on tensors of at least that many Mi elements),
 * "stats_grid_eighths" (the statistics pass on such tensors: at most this many eighths; 0: the same as the others),
 * "code_store_policy", "f32_store_policy", "f32_reread_store_policy", "copy_store_policy" (cache
 * policy of the stores of codes, of fp32 outputs, of fp32 outputs the next kernel reads back, of
 * the plain copy: 0 write-back, 2 non-temporal, 16 write-through), "reverse_second_pass" (the pass
 * that re-reads a tensor walks it from its end), "hist_replicas" (copies
 * of each LDS histogram bin in the fused quantize pass: 1, 2, 4, 8), "average_replicas" (the same for
 * average_buckets' histogram: 1, 2, 4, 8, 16), "nt_load_min_mib" (tensors at least this large
 * are read with non-temporal loads in their first pass), "stats_keep_mib" (the statistics pass of
 * uniform_8bit_quantize reads the last this many MiB of the tensor without that hint and all before them with it,
 * whatever the size: what a hinted load fetches does not stay in the last-level cache, and the quantize pass
 * starts at the tensor's end; 0: nt_load_min_mib decides for the whole tensor), "mix_cached" (on tensors of at least
 * twice that size the quantize pass visits the tiles of that cached end spread evenly among the others instead of
 * first, so that cache and memory deliver side by side) and "mixed_grid_eighths" (eighths of the compute units it then
 * runs on), "nt_second_min_mib" (the same for the
 * quantize pass that reads a tensor for the last time), "one_shot" (kernels that keep nothing from
 * tile to tile - dequantize, plain quantize, divide, pseudo-gradient, outer step, copy - run as one
 * 256-lane workgroup per tile from 65536 elements up instead of a loop) and "one_shot_store_policy"
 * (cache policy of their stores), "small_max_elems" (uniform_8bit_quantize of at most this many
 * elements, and at most four rows of 4096, takes one launch of one workgroup; 0: never),
 * "two_row_below_mi_elems" (the statistics and quantize kernels take tiles of two rows of 4096
 * elements instead of four on tensors below this many Mi elements; 0: never),
 * "set_four_rows_max_mi_elems" (the one-workgroup-per-tile dequantize set takes tiles of four rows of
 * 1024 elements instead of two on tensors of at most this many Mi elements; 0: never),
 * "dynamic_tail_percent" / "dynamic_tail_min_mi_elems" (the fused quantize + lookup pass hands out this
 * share of its tiles, the last ones, on demand instead of round-robin, on tensors of at least that many
 * Mi elements; 0: never; the counter it deals them through lives in the workspace and is left at zero by
 * prime_workspace_init and by every call that uses it), "segment_blocks_per_cu" (workgroups per compute unit that the quantize pass of
 * a segmented launch shares out among its tensors), "grid_cap" (upper bound on the workgroups of a looping kernel, for
 * experiments; 0: none).
 * Cache policies, load hints, the one-workgroup-per-tile and one-launch variants, the number of LDS
 * copies, the dynamic tail and segment_blocks_per_cu never change a result.  The options that change the number of
 * workgroups of the statistics pass or its tile shape (blocks_per_cu, grid_cap, large_read_*, stats_grid_eighths,
 * two_row_below_mi_elems) change the order in which the fp64 sums are added: codes and scale have been
 * equal on all tested data, but a sum may move in its last bit and, rarely, a scale with it.
 * Returns 0 if the name is known.  The
 * options are process-wide and read at launch time: set them before work is enqueued, not
 * concurrently with it. */
int prime_hip_set_option(const char* name, int value);
int prime_hip_get_option(const char* name, int* value);

/* Per-launch timing with HIP events on the launch stream, for benchmarks: after
 * prime_hip_profile_begin every kernel the library launches is bracketed by two events;
 * prime_hip_profile_end waits for them and returns, per kernel, the number of launches, the
 * summed duration and the summed algorithmic bytes (4 B/element statistics, 5 quantize,
 * 5 / 9 dequantize set / add).  out is host memory of `capacity` entries; *count receives the
 * number of kernels seen.  No counterpart in the reference (it times with perf_counter,
 * src/zeroband/diloco.py:109-113). */
typedef struct prime_kernel_time {
    char name[40];
    int64_t launches;
    double total_ms;
    double algo_bytes;
} prime_kernel_time;
int prime_hip_profile_begin(void);
int prime_hip_profile_end(prime_kernel_time* out, int capacity, int* count);

/* Workspace: a fixed-size block of device memory (about 10 MiB) that holds every workgroup's
 * partial sums and partial 256-bin histogram between a kernel and its second stage.  The one
 * thing it carries from call to call is a tile counter that every call leaves at zero;
 * prime_workspace_init validates the block and clears its head, the scale record and that
 * counter (a fill kernel, safe under stream capture): call it once on a new workspace before
 * any other entry point sees it.  Two calls that share a workspace must be ordered on one
 * stream. */
int64_t prime_workspace_bytes(void);
int prime_workspace_init(void* ws, int64_t ws_bytes, prime_stream_t stream);

/* Sum and sum of squares in fp64 plus the quantization scale, written to *out (device).
 * Stands in for `tensor.norm()` and the scale formula of uniform_8bit_quantize,
 * src/zeroband/C/csrc/compression.cpp:113-116. */
int prime_stats_f32(const float* x, int64_t n, prime_qparams* out, void* ws, prime_stream_t stream);

/* codes[i] = clamp(int32(round(x[i] * (1.0f / scale))) + zero_point, 0, 255), round half away
 * from zero.  Stands in for quantize_per_tensor_multithreaded, compression.cpp:9-43
 * (pybind name quantize_per_tensor_uint8, compression.cpp:146-154). */
int prime_quantize_u8(const float* x, int64_t n, float scale, int32_t zero_point, uint8_t* codes,
                      prime_stream_t stream);

/* lut[b] = mean of x[i] over codes[i] == b, 0.0f for an empty bin, b < n_bins; codes >= n_bins
 * are skipped.  Stands in for average_buckets_multithread, compression.cpp:45-104 (pybind name
 * average_buckets, compression.cpp:130-138).  lut has n_bins entries; n_bins >= 1.
 * counts (optional, 256 x uint64) receives the bin populations of bins < min(n_bins, 256). */
int prime_average_buckets(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins, float* lut,
                          uint64_t* counts, void* ws, prime_stream_t stream);

/* Quantize with a caller-supplied scale and build the lookup table in the same pass
 * (compression.cpp:119 + :122 with the scale of :116 given).  lut has 256 entries. */
int prime_quantize_lookup_u8(const float* x, int64_t n, float scale, uint8_t* codes, float* lut,
                             void* ws, prime_stream_t stream);

/* The whole of uniform_8bit_quantize, compression.cpp:106-125: statistics pass, then the fused
 * quantize + lookup pass.  qparams_out (optional, device) receives scale and sums. */
int prime_uniform_8bit_quantize(const float* x, int64_t n, uint8_t* codes, float* lut,
                                prime_qparams* qparams_out, void* ws, prime_stream_t stream);

/* prime_uniform_8bit_quantize for callers that cannot allocate device memory or carry a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): no counterpart in the reference.  The per-workgroup partials live in a scratch
 * array inside the library's own device image (10.1 MiB per GPU, held until the process
 * ends; its address is looked up once per device on the first call there).  Calls no hipMalloc,
 * hipFree or other allocating routine.  Same results as prime_uniform_8bit_quantize, bit for
 * bit.  n above 2^40 is rejected with PRIME_EINVAL.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race; order them. */
int prime_uniform_8bit_quantize_noalloc(const float* x, int64_t n, uint8_t* codes, float* lut,
                                        prime_qparams* qparams_out, prime_stream_t stream);

/* The norm as the reference receives it from libtorch's CPU kernel at compression.cpp:113
 * (eight serial fp32 fused-multiply-add lanes, lanes added in order, scalar tail, sqrtf: the
 * order observed in libtorch 2.10 on x86-64 with 256-bit vectors), and the scale of :113-116
 * derived from it.  The exact entry points above differ from this value by libtorch's
 * accumulation error (-7e-4 relative at 2^24 elements, -3.7e-2 at 2^28).  The chains are
 * serial, so this runs in one workgroup at about 1.9 G elements/s: a compatibility path, for
 * bit-for-bit reproduction of the reference.  qparams_out: scale, inv_scale, n; sum is NaN and
 * sumsq the square of the norm. */
int prime_norm_literal_f32(const float* x, int64_t n, prime_qparams* qparams_out, void* ws,
                           prime_stream_t stream);

/* uniform_8bit_quantize with that norm: scale and codes equal the compiled reference's bit for
 * bit; the lookup table is the fp64 bin mean (the reference's fp32 table depends on its thread
 * count). */
int prime_uniform_8bit_quantize_literal(const float* x, int64_t n, uint8_t* codes, float* lut,
                                        prime_qparams* qparams_out, void* ws, prime_stream_t stream);

/* Large buckets, pipelined: bucket i is quantized as prime_uniform_8bit_quantize would, on
 * streams[i % n_streams] with workspaces[i % n_streams], so that the statistics pass of one
 * bucket overlaps the quantize pass and the launch ramps of its neighbours (two streams
 * give +5 % on 205 MB buckets, more of them less; a set that holds a bucket of 2^27 elements or more runs on
 * streams[0] alone: such a bucket fills the device by itself, and a neighbour on another stream would displace what
 * it keeps in the last-level cache between its passes).  This is the loop over per-layer buckets of
 * Diloco.sync_pseudo_gradient (src/zeroband/diloco.py:108-110) without the network in between.
 * xs, ns, codes, workspaces and streams are host arrays; luts is count x 256 on the device and
 * qparams_out (optional) count records.  The caller orders the streams against its own work. */
int prime_uniform_8bit_quantize_buckets(const float* const* xs, const int64_t* ns, int64_t count,
                                        uint8_t* const* codes, float* luts, prime_qparams* qparams_out,
                                        void* const* workspaces, const prime_stream_t* streams,
                                        int n_streams);

/* Many tensors in one launch: tensor t is x[offsets[t] .. offsets[t+1]) of a flat buffer, the
 * layout of the per-layer views of Diloco's flat pseudo-gradient buffer
 * (src/zeroband/diloco.py:147-201), each handled as uniform_8bit_quantize handles one tensor.
 * offsets: count+1 non-decreasing int64 on the device (not checked: they are read by the kernel).
 * x and codes may be NULL only when count is 0.  codes uses the same offsets; luts is count x 256;
 * qparams_out (optional) is count entries.  Meant for tensors of up to 65,536 elements: every tensor gets
 * exactly one workgroup, so a larger entry is still quantized correctly but on one compute unit; a
 * caller that knows its sizes on the host takes prime_uniform_8bit_quantize_segmented for such sets
 * (the Python layer does so by itself when the offsets are host-visible). */
int prime_uniform_8bit_quantize_batched(const float* x, const int64_t* offsets, int64_t count,
                                        uint8_t* codes, float* luts, prime_qparams* qparams_out,
                                        prime_stream_t stream);

/* out[i] = lut[codes[i]]: fast_index_set_omp<float>, src/zeroband/C/csrc/collectives.cpp:16-22. */
int prime_dequant_set(float* out, const float* lut, const uint8_t* codes, int64_t n,
                      prime_stream_t stream);

/* out[i] += lut[codes[i]]: fast_index_add_omp<float>, collectives.cpp:8-14. */
int prime_dequant_add(float* out, const float* lut, const uint8_t* codes, int64_t n,
                      prime_stream_t stream);

/* One hop of the ring's reduce-scatter as ring_allreduce runs it on a received chunk,
 * collectives.cpp:124-138: acc[i] += lut_in[codes_in[i]] (fast_index_add_omp), then
 * (codes_out, lut_out) = uniform_8bit_quantize(acc).  The sum of squares of the updated acc is
 * taken in the accumulate pass, so acc is read twice and written once. */
int prime_ring_reduce_step(float* acc, const uint8_t* codes_in, const float* lut_in, int64_t n,
                           uint8_t* codes_out, float* lut_out, prime_qparams* qparams_out,
                           void* ws, prime_stream_t stream);

/* The last accumulation into a rank's own chunk (reduce-scatter steps past
 * (world_size - 1) * BUFFER_COUNT, which forward nothing: collectives.cpp:124-133) together
 * with what ring_allreduce does to that chunk next (:155-162):
 * acc[i] = (acc[i] + lut_in[codes_in[i]]) / divisor  (chunk.div_(world_size) of ReduceOp::AVG;
 * pass 1.0f for SUM, which skips the division), then (codes_out, lut_out) =
 * uniform_8bit_quantize(acc).  The write-back acc = lut_out[codes_out] of :167-172 is
 * prime_dequant_set, or prime_ring_gather_step when the chunk is forwarded in the all-gather.
 * 14 bytes per element where the separate calls move 26. */
int prime_ring_reduce_div_step(float* acc, const uint8_t* codes_in, const float* lut_in, int64_t n, float divisor,
                               uint8_t* codes_out, float* lut_out, prime_qparams* qparams_out, void* ws,
                               prime_stream_t stream);

/* (codes_out, lut_out) = uniform_8bit_quantize(t) for t[i] = lut_in[codes_in[i]], without t: the
 * quantization that forwards a chunk in the all-gather (collectives.cpp:204-215) when the fp32
 * chunk itself is not needed yet.  t holds at most 256 distinct values, so the statistics
 * follow from the population of each code, codes_out[i] is a 256-entry map of codes_in[i] and
 * lut_out is the population-weighted mean of the old entries that share a new code.  Codes are
 * those of the two-pass path bit for bit; 3 bytes per element instead of 10.  codes_out must
 * not overlap codes_in. */
int prime_requantize_codes(const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out,
                           float* lut_out, prime_qparams* qparams_out, void* ws, prime_stream_t stream);

/* One hop of the ring's all-gather as ring_allreduce runs it, collectives.cpp:200-215:
 * chunk[i] = lut_in[codes_in[i]] (fast_index_set_omp), then (codes_out, lut_out) =
 * uniform_8bit_quantize(chunk) for forwarding.  The statistics are taken while the chunk is
 * written, so it is written once and read once. */
int prime_ring_gather_step(float* chunk, const uint8_t* codes_in, const float* lut_in, int64_t n,
                           uint8_t* codes_out, float* lut_out, prime_qparams* qparams_out,
                           void* ws, prime_stream_t stream);

/* ---- segmented launches: many mid-size tensors, three kernel launches in all ----
 * The ring all-reduce of one layer bucket cuts it into 2 * world_size chunks (collectives.cpp:89-90)
 * and Diloco.sync_pseudo_gradient visits one bucket after the other (src/zeroband/diloco.py:108-110),
 * so the tensors this path really sees are chunks of 1-4 M elements, where three kernel boundaries
 * per tensor cost more than the data.  These entry points take `count` tensors as host arrays of
 * device pointers and sizes, give every tensor as many workgroups as its size wants, and run the
 * whole set in three launches per group of 64 tensors: statistics (or a ring step's first pass),
 * quantize + histogram, lookup tables.  Tensor i's results (codes[i], luts + 256 * i,
 * qparams_out[i]) equal what the one-tensor entry point returns for it, bit for bit (the lookup
 * entries of a tensor whose 1 / scale is zero or not finite, and bins 0 / 255 of a tensor with
 * values beyond 628 bins in several workgroups, may differ in their last bit: they are sums of
 * fp64 values in an order that depends on the launch).  Tensors that are empty, not aligned for
 * vector access (tensor 16 bytes, codes 4), or large enough to fill the device on their own (more than
 * 2^25 elements, 2^24 for the ring steps: options "segment_max_mi_elems", "segment_ring_max_mi_elems")
 * take the one-tensor path inside the call.  The pointer
 * and size arrays are host memory and are read before the call returns; luts is count x 256 floats
 * and qparams_out (optional) count records on the device.  One workspace, as for the calls above. */
int prime_uniform_8bit_quantize_segmented(const float* const* xs, const int64_t* ns, int64_t count,
                                          uint8_t* const* codes, float* luts, prime_qparams* qparams_out,
                                          void* ws, prime_stream_t stream);

/* prime_ring_reduce_step on count chunks: what the world_size ranks of a lock-stepped ring do in one
 * step of the reduce-scatter (collectives.cpp:124-138), or one rank on the chunks of several buckets. */
int prime_ring_reduce_step_segmented(float* const* accs, const uint8_t* const* codes_in,
                                     const float* const* luts_in, const int64_t* ns, int64_t count,
                                     uint8_t* const* codes_out, float* luts_out, prime_qparams* qparams_out,
                                     void* ws, prime_stream_t stream);

/* prime_ring_reduce_div_step on count chunks, one divisor for all (collectives.cpp:124-133,155-162). */
int prime_ring_reduce_div_step_segmented(float* const* accs, const uint8_t* const* codes_in,
                                         const float* const* luts_in, const int64_t* ns, int64_t count,
                                         float divisor, uint8_t* const* codes_out, float* luts_out,
                                         prime_qparams* qparams_out, void* ws, prime_stream_t stream);

/* prime_ring_gather_step on count chunks (collectives.cpp:200-215). */
int prime_ring_gather_step_segmented(float* const* chunks, const uint8_t* const* codes_in,
                                     const float* const* luts_in, const int64_t* ns, int64_t count,
                                     uint8_t* const* codes_out, float* luts_out, prime_qparams* qparams_out,
                                     void* ws, prime_stream_t stream);

/* x[i] = x[i] / divisor in place: chunk.div_(world_size) of the ring's ReduceOp::AVG,
 * collectives.cpp:155-159. */
int prime_div_f32(float* x, int64_t n, float divisor, prime_stream_t stream);

/* ---- the callers either side of the compression path (src/zeroband/diloco.py) ---- */

/* out[i] = (outer[i] - inner[i]) / world_size: the pseudo-gradient of one bucket as
 * Diloco.sync_pseudo_gradient forms it, diloco.py:93-101 (grad = cpu_param - gpu_param, then
 * offloaded_grad_flat_tensor.div_(world_size)), with both parameter copies on the device. */
int prime_pseudo_gradient_f32(const float* outer, const float* inner, int64_t n, float world_size,
                              float* out, prime_stream_t stream);

/* A chunk's first touch in the ring with the pseudo-gradient formed on the way.  Every chunk of
 * a rank is visited exactly once in the reduce-scatter (collectives.cpp:115-116), so the pass
 * that would read the pseudo-gradient back can compute it instead:
 *   grad_out[i] = (outer[i] - inner[i]) / world_size                        (diloco.py:93-101)
 *   with codes_in:  grad_out[i] = (grad_out[i] + lut_in[codes_in[i]]) / divisor
 *                   (fast_index_add_omp, collectives.cpp:128-133; chunk.div_ for AVG on a
 *                   rank's own chunks, :155-159; 1.0f skips the division)
 *   (codes_out, lut_out) = uniform_8bit_quantize(grad_out)                  (:138 / :162)
 * codes_in == NULL is the quantization of a chunk that is sent before anything is received
 * (steps 1 and 2): prime_pseudo_gradient_f32 followed by prime_uniform_8bit_quantize, which on
 * this device beat a pass that takes the statistics along (12 + 9 bytes per element in 197 us
 * against 17 in 211 us at 2^26 elements).  With a received message the fused pass moves 18 bytes
 * per element against 12 + 14 and is 15 % faster. */
int prime_ring_first_touch(const float* outer, const float* inner, int64_t n, float world_size,
                           const uint8_t* codes_in, const float* lut_in, float divisor, float* grad_out,
                           uint8_t* codes_out, float* lut_out, prime_qparams* qparams_out, void* ws,
                           prime_stream_t stream);

/* The outer optimizer step on one bucket: torch.optim.SGD(lr, momentum, nesterov=True),
 * diloco.py:72-74 and :212-213, rounded as libtorch's CPU kernels round it
 * (buf = buf*mu + g, or g on the first step; d = fma(buf, mu, g); p = fma(d, -lr, p)),
 * followed by the copy of the new parameters to the inner model (sync_inner_model,
 * diloco.py:137-144) when inner_out is not NULL.  param and momentum_buf are updated in place. */
int prime_outer_sgd_nesterov_f32(float* param, float* momentum_buf, const float* grad, float* inner_out,
                                 int64_t n, float lr, float momentum, int first_step,
                                 prime_stream_t stream);

/* The same step with the reduced pseudo-gradient still in wire form (uint8 codes and their
 * 256-entry lookup, as the all-gather delivers them, collectives.cpp:204-209): the
 * dequantize pass is folded in. */
int prime_outer_sgd_nesterov_u8(float* param, float* momentum_buf, const uint8_t* codes, const float* lut,
                                float* inner_out, int64_t n, float lr, float momentum, int first_step,
                                prime_stream_t stream);

/* The two loops over the parameter list either side of the all-reduce as one launch per 64 tensors:
 * prime_pseudo_gradient_f32 for every parameter (the loop of diloco.py:93-99) and
 * prime_outer_sgd_nesterov_f32 for every parameter (the outer optimizer's step over its parameters
 * and sync_inner_model, diloco.py:212-215, :137-144).  Host arrays of `count` device pointers and
 * sizes, read before the call returns; inner_outs may be NULL, and so may single entries of it.
 * Elementwise arithmetic: results are those of the one-tensor calls.  Empty tensors are skipped;
 * tensors not aligned to 16 bytes take the one-tensor entry point inside the call. */
int prime_pseudo_gradient_f32_segmented(const float* const* outers, const float* const* inners,
                                        const int64_t* ns, int64_t count, float world_size,
                                        float* const* outs, prime_stream_t stream);
int prime_outer_sgd_nesterov_f32_segmented(float* const* params, float* const* momentum_bufs,
                                           const float* const* grads, float* const* inner_outs,
                                           const int64_t* ns, int64_t count, float lr, float momentum,
                                           int first_step, prime_stream_t stream);

/* A plain device copy of n bytes (16-byte vectors): the yardstick the profiler's byte
 * counters are scaled against.  No counterpart in the reference. */
int prime_copy_bytes(void* dst, const void* src, int64_t n_bytes, prime_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PRIME_HIP_H */
