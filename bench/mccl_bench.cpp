// libmcclbench: HIP-event timing loops around the C ABI (see mccl_bench.h beside this file).
#include <hip/hip_runtime.h>

#include <cstdint>
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


// ---------------------------------------------------------------------------------------------
// Machine probe: a bare streaming kernel (no product code) in the launch shape of the library's
// large-message reduction: workgroups of `BLOCK` lanes, one 16-byte vector per lane per stream,
// residency capped by a dynamic-LDS reservation.  Reads NR streams, xors them, and writes the
// result (WR = 1) or keeps the store behind a compare that random data never satisfies (WR = 0).
// It tells what this part sustains for pure reads, pure writes and a given read:write mix, which
// is the ceiling the product kernels are compared with.
// ---------------------------------------------------------------------------------------------
typedef uint32_t probe_vec __attribute__((ext_vector_type(4)));
struct ProbeArgs {
  const probe_vec* in[8];
  probe_vec* out;
};

template <int NR, int WR, int BLOCK>
__global__ __launch_bounds__(BLOCK) void probe_stream_kernel(const ProbeArgs p) {
  const size_t v = (size_t)blockIdx.x * BLOCK + threadIdx.x;
  probe_vec acc = (probe_vec){1u, 2u, 3u, 4u};
  probe_vec x[NR > 0 ? NR : 1];
#pragma unroll
  for (int r = 0; r < NR; ++r) x[r] = __builtin_nontemporal_load(&p.in[r][v]);
#pragma unroll
  for (int r = 0; r < NR; ++r) acc ^= x[r];
  // the streaming store of the product kernels (write-through at agent scope), spelled as an
  // instruction so that the hint survives; the wait state after it covers the hazard the compiler
  // cannot see
  if (WR) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(&p.out[v]), "v"(acc) : "memory");
  else if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u && acc.z == 77u && acc.w == 0xfeedbeefu) p.out[v] = acc;
}

template <int NR, int WR>
void probe_launch(const ProbeArgs& p, unsigned nvec, int block, unsigned lds, hipStream_t s) {
  if (block == 256) hipLaunchKernelGGL((probe_stream_kernel<NR, WR, 256>), dim3(nvec / 256), dim3(256), lds, s, p);
  else hipLaunchKernelGGL((probe_stream_kernel<NR, WR, 64>), dim3(nvec / 64), dim3(64), lds, s, p);
}

template <int WR>
bool probe_dispatch(int n_read, const ProbeArgs& p, unsigned nvec, int block, unsigned lds, hipStream_t s) {
  switch (n_read) {
    case 0: if (!WR) return false; probe_launch<0, WR>(p, nvec, block, lds, s); return true;
    case 1: probe_launch<1, WR>(p, nvec, block, lds, s); return true;
    case 2: probe_launch<2, WR>(p, nvec, block, lds, s); return true;
    case 3: probe_launch<3, WR>(p, nvec, block, lds, s); return true;
    case 4: probe_launch<4, WR>(p, nvec, block, lds, s); return true;
    case 5: probe_launch<5, WR>(p, nvec, block, lds, s); return true;
    case 6: probe_launch<6, WR>(p, nvec, block, lds, s); return true;
    case 7: probe_launch<7, WR>(p, nvec, block, lds, s); return true;
    case 8: probe_launch<8, WR>(p, nvec, block, lds, s); return true;
    default: return false;
  }
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

// A timed loop whose set-up (the two events) happens before the caller starts its own clock.
struct TimedLoop {
  hipEvent_t e0 = nullptr, e1 = nullptr;
};

int mcclb_loop_create(void** loop) {
  if (!loop) { snprintf(g_err, sizeof(g_err), "loop must be non-null"); return MCCL_ERR_INVALID_ARG; }
  TimedLoop* t = new TimedLoop();
  hipError_t e = hipEventCreate(&t->e0);
  if (e == hipSuccess) e = hipEventCreate(&t->e1);
  if (e != hipSuccess) {
    if (t->e0) (void)hipEventDestroy(t->e0);
    delete t;
    return fail_hip("hipEventCreate", e);
  }
  *loop = t;
  return MCCL_OK;
}

int mcclb_loop_reduce(void* loop, const void* const* in, int n, void* const* out, int nsets,
                      size_t count, int dtype, int op, int variant, void* stream, int iters) {
  TimedLoop* t = static_cast<TimedLoop*>(loop);
  if (!t || iters <= 0) { snprintf(g_err, sizeof(g_err), "needs a loop and iters > 0"); return MCCL_ERR_INVALID_ARG; }
  if (nsets < 1) nsets = 1;
  hipStream_t s = (hipStream_t)stream;
  HIP_OK(hipEventRecord(t->e0, s));
  int rc = MCCL_OK;
  for (int i = 0; i < iters && rc == MCCL_OK; ++i) {
    const int set = i % nsets;
    rc = mccl_reduce_n(in + (size_t)set * n, n, out[set], count, dtype, op, variant, stream);
  }
  HIP_OK(hipEventRecord(t->e1, s));
  return rc == MCCL_OK ? MCCL_OK : fail_mccl(rc);
}

int mcclb_loop_elapsed_us(void* loop, float* total_us) {
  TimedLoop* t = static_cast<TimedLoop*>(loop);
  if (!t || !total_us) { snprintf(g_err, sizeof(g_err), "needs a loop and an output"); return MCCL_ERR_INVALID_ARG; }
  HIP_OK(hipEventSynchronize(t->e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, t->e0, t->e1));
  *total_us = ms * 1000.f;
  return MCCL_OK;
}

void mcclb_loop_destroy(void* loop) {
  TimedLoop* t = static_cast<TimedLoop*>(loop);
  if (!t) return;
  (void)hipEventDestroy(t->e0);
  (void)hipEventDestroy(t->e1);
  delete t;
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


int mcclb_probe_stream(const void* const* in, int n_read, void* out, int write, size_t bytes,
                       int block, int workgroups_per_cu, void* stream, int warmup, int iters,
                       float* total_us) {
  if (!out || (n_read > 0 && !in) || (block != 64 && block != 256) || bytes == 0 || bytes % 4096 ||
      bytes / 16 > 0xffffffffull) {
    snprintf(g_err, sizeof(g_err), "probe: needs an output buffer, a block of 64 or 256 and a size that is a multiple of 4 KiB");
    return MCCL_ERR_INVALID_ARG;
  }
  ProbeArgs p{};
  for (int r = 0; r < n_read && r < 8; ++r) {
    if (!in[r]) { snprintf(g_err, sizeof(g_err), "probe: input %d is null", r); return MCCL_ERR_INVALID_ARG; }
    p.in[r] = (const probe_vec*)in[r];
  }
  p.out = (probe_vec*)out;
  unsigned lds = 0;
  if (workgroups_per_cu > 0 && workgroups_per_cu * (block / 64) < 32) {
    lds = (unsigned)((160 * 1024 / workgroups_per_cu) & ~511);
    if (lds > 64 * 1024) lds = 64 * 1024;
  }
  const unsigned nvec = (unsigned)(bytes / 16);
  hipStream_t s = (hipStream_t)stream;
  auto call = [&](int) {
    const bool ok = write ? probe_dispatch<1>(n_read, p, nvec, block, lds, s) : probe_dispatch<0>(n_read, p, nvec, block, lds, s);
    if (!ok) return (int)MCCL_ERR_INVALID_ARG;
    return hipGetLastError() == hipSuccess ? (int)MCCL_OK : (int)MCCL_ERR_HIP;
  };
  return throughput_loop(call, s, warmup, iters, total_us);
}

}  // extern "C"
