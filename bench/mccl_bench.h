/*
 * mccl_bench.h -- timing loops around the C ABI of include/mccl.h (libmcclbench.so).
 * Lives beside bench.py: it is benchmark support, not part of the library's boundary.
 *
 * Benchmark support only: these loops call the product entry points unchanged and time
 * them with HIP events recorded on the launch stream, so that per-call latencies are not
 * polluted by interpreter overhead.  They have no counterpart in the reference (whose
 * timing scripts, tests/ddp_allreduce.py:86-117, time from the host).
 */
#ifndef MCCL_BENCH_H_
#define MCCL_BENCH_H_

#include "mccl.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Per-call latency of mccl_reduce_n: `iters` calls, one event pair per call, us_out[i] =
 * microseconds of call i.  `in` holds nsets*n pointers and `out` nsets pointers; call i
 * uses set i % nsets (nsets > 1 rotates buffers so the caches do not hold the inputs).
 */
int mcclb_reduce_latency(const void* const* in, int n, void* const* out, int nsets, size_t count,
                         int dtype, int op, int variant, void* stream, int warmup, int iters,
                         float* us_out);

/* Back-to-back throughput: one event pair around `iters` consecutive calls; *total_us =
 * elapsed microseconds for all of them. */
int mcclb_reduce_throughput(const void* const* in, int n, void* const* out, int nsets,
                            size_t count, int dtype, int op, int variant, void* stream, int warmup,
                            int iters, float* total_us);

/*
 * The same back-to-back loop with its set-up taken out, for a caller that times the loop with a
 * clock of its own: mcclb_loop_create makes the two events; mcclb_loop_reduce records the first,
 * enqueues `iters` calls of mccl_reduce_n and records the second, without synchronising;
 * mcclb_loop_elapsed_us waits for the second event and returns the time between the two.
 */
int mcclb_loop_create(void** loop);
int mcclb_loop_reduce(void* loop, const void* const* in, int n, void* const* out, int nsets,
                      size_t count, int dtype, int op, int variant, void* stream, int iters);
int mcclb_loop_elapsed_us(void* loop, float* total_us);
void mcclb_loop_destroy(void* loop);

/* The same two loops around mccl_reduce_scatter_n (all shards of one launch). */
int mcclb_reduce_scatter_throughput(const void* const* in, int n, void* const* out,
                                    size_t shard_count, int shard_first, int shard_num, int dtype,
                                    int op, void* stream, int warmup, int iters, float* total_us);

/* ... and around mccl_copy_segments. */
int mcclb_copy_latency(const mccl_segment_t* segs, int nseg, void* stream, int warmup, int iters,
                       float* us_out);
int mcclb_copy_throughput(const mccl_segment_t* segs, int nseg, void* stream, int warmup,
                          int iters, float* total_us);

/* ... and around mccl_alltoallv_n (all ranks). */
int mcclb_alltoallv_throughput(const void* const* in, void* const* out, int n,
                               const int64_t* split_rows, size_t row_bytes, void* stream,
                               int warmup, int iters, float* total_us);

/*
 * Machine probe (no product code): a bare streaming kernel in the launch shape of the large-message
 * reduction.  Each lane reads one 16-byte vector from each of `n_read` (0, 1, 2, 4 or 8) buffers of
 * `bytes` bytes, xors them and, if `write` is non-zero, writes the result to `out` (`bytes` bytes;
 * must be a valid buffer even when `write` is 0).  `block` is 64 or 256 lanes per workgroup;
 * `workgroups_per_cu` > 0 caps residency.  Tells what the part sustains for pure reads, pure
 * writes and a read:write mix: the practical ceiling the product kernels are compared with.
 */
int mcclb_probe_stream(const void* const* in, int n_read, void* out, int write, size_t bytes,
                       int block, int workgroups_per_cu, void* stream, int warmup, int iters,
                       float* total_us);

const char* mcclb_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* MCCL_BENCH_H_ */
