// libmcclbench: HIP-event timing loops around the C ABI (see include/mccl_bench.h).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <functional>
#include <vector>

#include "mccl_bench.h"

namespace {

thread_local char g_err[512] = "";

int fail_hip(const char* what, hipError_t e) {
  snprintf(g_err, sizeof(g_err), "%s failed: %s", what, hipGetErrorString(e));
  return MCCL_ERR_HIP;
}

int fail_mccl(int rc) {
  snprintf(g_err, sizeof(g_err), "mccl call failed (%d): %s", rc, mccl_last_error());
  return rc;
}

#define HIP_OK(expr)                                      \
  do {                                                    \
    hipError_t e_ = (expr);                               \
    if (e_ != hipSuccess) return fail_hip(#expr, e_);     \
  } while (0)

// One event pair per call.
int latency_loop(const std::function<int(int)>& call, hipStream_t s, int warmup, int iters, float* us_out) {
  if (iters <= 0 || !us_out) {
    snprintf(g_err, sizeof(g_err), "iters must be positive and us_out non-null");
    return MCCL_ERR_INVALID_ARG;
  }
  for (int i = 0; i < warmup; ++i) {
    int rc = call(i);
    if (rc != MCCL_OK) return fail_mccl(rc);
  }
  HIP_OK(hipStreamSynchronize(s));
  std::vector<hipEvent_t> e0(iters), e1(iters);
  for (int i = 0; i < iters; ++i) {
    HIP_OK(hipEventCreate(&e0[i]));
    HIP_OK(hipEventCreate(&e1[i]));
  }
  int rc = MCCL_OK;
  for (int i = 0; i < iters && rc == MCCL_OK; ++i) {
    HIP_OK(hipEventRecord(e0[i], s));
    rc = call(warmup + i);
    HIP_OK(hipEventRecord(e1[i], s));
  }
  HIP_OK(hipStreamSynchronize(s));
  if (rc == MCCL_OK) {
    for (int i = 0; i < iters; ++i) {
      float ms = 0.f;
      HIP_OK(hipEventElapsedTime(&ms, e0[i], e1[i]));
      us_out[i] = ms * 1000.f;
    }
  }
  for (int i = 0; i < iters; ++i) {
    (void)hipEventDestroy(e0[i]);
    (void)hipEventDestroy(e1[i]);
  }
  return rc == MCCL_OK ? MCCL_OK : fail_mccl(rc);
}

// One event pair around all calls.
int throughput_loop(const std::function<int(int)>& call, hipStream_t s, int warmup, int iters, float* total_us) {
  if (iters <= 0 || !total_us) {
    snprintf(g_err, sizeof(g_err), "iters must be positive and total_us non-null");
    return MCCL_ERR_INVALID_ARG;
  }
  for (int i = 0; i < warmup; ++i) {
    int rc = call(i);
    if (rc != MCCL_OK) return fail_mccl(rc);
  }
  HIP_OK(hipStreamSynchronize(s));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, s));
  int rc = MCCL_OK;
  for (int i = 0; i < iters && rc == MCCL_OK; ++i) rc = call(warmup + i);
  HIP_OK(hipEventRecord(e1, s));
  HIP_OK(hipStreamSynchronize(s));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  *total_us = ms * 1000.f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc == MCCL_OK ? MCCL_OK : fail_mccl(rc);
}

}  // namespace

extern "C" {

const char* mcclb_last_error(void) { return g_err; }

int mcclb_reduce_latency(const void* const* in, int n, void* const* out, int nsets, size_t count,
                         int dtype, int op, int variant, void* stream, int warmup, int iters,
                         float* us_out) {
  if (nsets < 1) nsets = 1;
  auto call = [&](int i) {
    const int set = i % nsets;
    return mccl_reduce_n(in + (size_t)set * n, n, out[set], count, dtype, op, variant, stream);
  };
  return latency_loop(call, (hipStream_t)stream, warmup, iters, us_out);
}

int mcclb_reduce_throughput(const void* const* in, int n, void* const* out, int nsets,
                            size_t count, int dtype, int op, int variant, void* stream, int warmup,
                            int iters, float* total_us) {
  if (nsets < 1) nsets = 1;
  auto call = [&](int i) {
    const int set = i % nsets;
    return mccl_reduce_n(in + (size_t)set * n, n, out[set], count, dtype, op, variant, stream);
  };
  return throughput_loop(call, (hipStream_t)stream, warmup, iters, total_us);
}

int mcclb_reduce_scatter_throughput(const void* const* in, int n, void* const* out,
                                    size_t shard_count, int shard_first, int shard_num, int dtype,
                                    int op, void* stream, int warmup, int iters, float* total_us) {
  auto call = [&](int) {
    return mccl_reduce_scatter_n(in, n, out, shard_count, shard_first, shard_num, dtype, op, stream);
  };
  return throughput_loop(call, (hipStream_t)stream, warmup, iters, total_us);
}

int mcclb_copy_latency(const mccl_segment_t* segs, int nseg, void* stream, int warmup, int iters,
                       float* us_out) {
  auto call = [&](int) { return mccl_copy_segments(segs, nseg, stream); };
  return latency_loop(call, (hipStream_t)stream, warmup, iters, us_out);
}

int mcclb_copy_throughput(const mccl_segment_t* segs, int nseg, void* stream, int warmup,
                          int iters, float* total_us) {
  auto call = [&](int) { return mccl_copy_segments(segs, nseg, stream); };
  return throughput_loop(call, (hipStream_t)stream, warmup, iters, total_us);
}

int mcclb_alltoallv_throughput(const void* const* in, void* const* out, int n,
                               const int64_t* split_rows, size_t row_bytes, void* stream,
                               int warmup, int iters, float* total_us) {
  auto call = [&](int) { return mccl_alltoallv_n(in, out, n, split_rows, row_bytes, stream); };
  return throughput_loop(call, (hipStream_t)stream, warmup, iters, total_us);
}

}  // extern "C"
