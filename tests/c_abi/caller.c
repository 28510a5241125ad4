/*
 * A host written in plain C that drives libmi355ccl.so through include/mccl.h and the HIP runtime's
 * C API only: no C++, no torch, no Python.  It is what a maintainer of a compiled host (the
 * reference's ProcessGroupCCL is C++) would link.  Checks, with values that are exact in fp32 and
 * therefore have one right answer:
 *   - a 3-buffer fp32 SUM of an odd element count, out of place and in place,
 *   - a 2-rank bf16 SUM (fp32 accumulation, one rounding),
 *   - allgather of odd-sized byte buffers and a 2 x 2 uneven alltoallv,
 *   - an invalid call returning a status and a message instead of crashing.
 * Prints "c abi ok" and exits 0 on success.
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "mccl.h"

#define HIP_OK(x)                                                                          \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                       \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)
#define MCCL_OK_OR_DIE(x)                                                                  \
  do {                                                                                     \
    int rc_ = (x);                                                                         \
    if (rc_ != MCCL_OK) {                                                                  \
      fprintf(stderr, "%s returned %d: %s\n", #x, rc_, mccl_last_error());                 \
      return 3;                                                                            \
    }                                                                                      \
  } while (0)

static uint16_t bf16_of(float f) { /* exact for the small integers used here */
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)(u >> 16);
}

int main(void) {
  enum { N = 3 };
  const size_t count = 1000003;
  hipStream_t stream;
  HIP_OK(hipSetDevice(0));
  HIP_OK(hipStreamCreate(&stream));

  /* ---- 3-buffer fp32 sum ---- */
  float* host[N];
  void* dev[N];
  void* out = NULL;
  for (int r = 0; r < N; ++r) {
    host[r] = (float*)malloc(count * sizeof(float));
    for (size_t i = 0; i < count; ++i) host[r][i] = (float)((int)((i * 7 + (size_t)r * 13) % 201) - 100);
    HIP_OK(hipMalloc(&dev[r], count * sizeof(float)));
    HIP_OK(hipMemcpy(dev[r], host[r], count * sizeof(float), hipMemcpyHostToDevice));
  }
  HIP_OK(hipMalloc(&out, count * sizeof(float)));
  const void* in[N] = {dev[0], dev[1], dev[2]};
  MCCL_OK_OR_DIE(mccl_reduce_n(in, N, out, count, MCCL_F32, MCCL_SUM, MCCL_VARIANT_AUTO, stream));
  MCCL_OK_OR_DIE(mccl_reduce_n(in, N, dev[1], count, MCCL_F32, MCCL_SUM, MCCL_VARIANT_AUTO, stream)); /* in place */
  HIP_OK(hipStreamSynchronize(stream));
  float* got = (float*)malloc(count * sizeof(float));
  for (int pass = 0; pass < 2; ++pass) {
    HIP_OK(hipMemcpy(got, pass ? dev[1] : out, count * sizeof(float), hipMemcpyDeviceToHost));
    for (size_t i = 0; i < count; ++i) {
      const float want = host[0][i] + host[1][i] + host[2][i];
      if (got[i] != want) {
        fprintf(stderr, "fp32 sum (%s) differs at %zu: %g != %g\n", pass ? "in place" : "out of place", i, got[i], want);
        return 4;
      }
    }
  }

  /* ---- 2-rank bf16 sum ---- */
  const size_t c16 = 4099;
  uint16_t *a = (uint16_t*)malloc(c16 * 2), *b = (uint16_t*)malloc(c16 * 2), *s = (uint16_t*)malloc(c16 * 2);
  for (size_t i = 0; i < c16; ++i) {
    a[i] = bf16_of((float)(i % 64));
    b[i] = bf16_of((float)((i * 3) % 64));
  }
  void *da, *db, *ds;
  HIP_OK(hipMalloc(&da, c16 * 2));
  HIP_OK(hipMalloc(&db, c16 * 2));
  HIP_OK(hipMalloc(&ds, c16 * 2));
  HIP_OK(hipMemcpy(da, a, c16 * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(db, b, c16 * 2, hipMemcpyHostToDevice));
  const void* in16[2] = {da, db};
  MCCL_OK_OR_DIE(mccl_reduce_n(in16, 2, ds, c16, MCCL_BF16, MCCL_SUM, MCCL_VARIANT_AUTO, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(s, ds, c16 * 2, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < c16; ++i) {
    if (s[i] != bf16_of((float)(i % 64 + (i * 3) % 64))) { /* sums below 128: exact in bf16 */
      fprintf(stderr, "bf16 sum differs at %zu\n", i);
      return 5;
    }
  }

  /* ---- allgather of 3 x 1001 bytes, alltoallv of a 2 x 2 split ---- */
  const size_t nb = 1001;
  unsigned char* hb = (unsigned char*)malloc(3 * nb);
  void *g_in[3], *g_out;
  for (int r = 0; r < 3; ++r) {
    for (size_t i = 0; i < nb; ++i) hb[r * nb + i] = (unsigned char)(i * 5 + (size_t)r * 17);
    HIP_OK(hipMalloc(&g_in[r], nb));
    HIP_OK(hipMemcpy(g_in[r], hb + r * nb, nb, hipMemcpyHostToDevice));
  }
  HIP_OK(hipMalloc(&g_out, 3 * nb));
  const void* gin[3] = {g_in[0], g_in[1], g_in[2]};
  MCCL_OK_OR_DIE(mccl_allgather_n(gin, 3, g_out, nb, stream));
  HIP_OK(hipStreamSynchronize(stream));
  unsigned char* gb = (unsigned char*)malloc(3 * nb);
  HIP_OK(hipMemcpy(gb, g_out, 3 * nb, hipMemcpyDeviceToHost));
  if (memcmp(gb, hb, 3 * nb) != 0) {
    fprintf(stderr, "allgather differs\n");
    return 6;
  }
  /* rank 0 sends 2 rows to rank 0 and 1 row to rank 1; rank 1 sends 0 rows and 3 rows; rows of 7 bytes */
  const int64_t split[4] = {2, 1, 0, 3};
  const size_t row = 7;
  unsigned char h0[3 * 7], h1[3 * 7], o0[2 * 7], o1[4 * 7];
  for (size_t i = 0; i < sizeof h0; ++i) { h0[i] = (unsigned char)(10 + i); h1[i] = (unsigned char)(100 + i); }
  void *d0, *d1, *e0, *e1;
  HIP_OK(hipMalloc(&d0, sizeof h0)); HIP_OK(hipMalloc(&d1, sizeof h1));
  HIP_OK(hipMalloc(&e0, sizeof o0)); HIP_OK(hipMalloc(&e1, sizeof o1));
  HIP_OK(hipMemcpy(d0, h0, sizeof h0, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d1, h1, sizeof h1, hipMemcpyHostToDevice));
  const void* ain[2] = {d0, d1};
  void* aout[2] = {e0, e1};
  MCCL_OK_OR_DIE(mccl_alltoallv_n(ain, aout, 2, split, row, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(o0, e0, sizeof o0, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(o1, e1, sizeof o1, hipMemcpyDeviceToHost));
  if (memcmp(o0, h0, 2 * row) != 0 || memcmp(o1, h0 + 2 * row, row) != 0 || memcmp(o1 + row, h1, 3 * row) != 0) {
    fprintf(stderr, "alltoallv differs\n");
    return 7;
  }

  /* ---- errors come back as a status and a message ---- */
  if (mccl_reduce_n(in, N, out, count, 42, MCCL_SUM, MCCL_VARIANT_AUTO, stream) != MCCL_ERR_INVALID_ARG ||
      strstr(mccl_last_error(), "dtype") == NULL) {
    fprintf(stderr, "bad dtype was not refused: %s\n", mccl_last_error());
    return 8;
  }
  if (mccl_reduce_n(in, N, (char*)dev[2] + 64, count, MCCL_F32, MCCL_SUM, MCCL_VARIANT_AUTO, stream) != MCCL_ERR_INVALID_ARG) {
    fprintf(stderr, "overlapping output was not refused\n");
    return 9;
  }
  printf("c abi ok: version %d\n", mccl_version());
  return 0;
}
