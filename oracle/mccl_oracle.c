/*
 * CPU oracle for the collective data path -- TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C on host memory, what the reference's device
 * data path computes when the N "peer" buffers are N arrays.  It is the
 * checker for the HIP kernels: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may build, load or call it.  Nothing the
 * library ships may route through it.
 *
 * Reference files each function follows (paths relative to the reference):
 *   oracle_reduce           src/gpu/allreduce_small.h:289-361  (result = 0; for r in
 *                           0..N-1: result = result + buf[r]; ascending rank order,
 *                           zero start) with the accumulation type widened to fp32 for
 *                           fp16/bf16; op/dtype tables src/utils.cpp:38-58
 *   oracle_reduce_scatter   src/gpu/dpcpp_ccl.cpp:971-1019 (rank r receives the
 *                           reduction of slice [r*M,(r+1)*M) of every rank's input);
 *                           CPU twin src/cpu/cpu_ccl.cpp:819-868
 *   oracle_allgather        src/gpu/dpcpp_ccl.cpp:1147-1192 (out[k*M:(k+1)*M] = in_k)
 *   oracle_alltoall_counts  src/gpu/dpcpp_ccl.cpp:1431-1445 (send/recv counts from
 *                           split sizes; displacements = exclusive prefix sums)
 *   oracle_alltoallv        src/gpu/dpcpp_ccl.cpp:1428-1455, src/cpu/cpu_ccl.cpp:924-950
 *                           (rank d's segment r comes from rank r's segment d)
 *   oracle_pack/unpack      src/gpu/dpcpp_ccl.cpp:1505-1515, 1528-1538
 *   oracle_gather_rows / oracle_moe_dispatch / oracle_moe_combine / oracle_route_counts
 *                           no reference file: the callers' steps either side of the
 *                           all_to_all_single of src/gpu/dpcpp_ccl.cpp:1428-1455
 *
 * Parity status
 *   pinned    : indexing of every op (reference tests' closed forms, brute force on
 *               tagged tiny inputs), fp32 N=2 sum (commutative, one value possible),
 *               integer sums (associative), fp32->bf16 / fp32<->fp16 conversions
 *               (checked against numpy / torch CPU conversions).
 *               AVG (this build's addition): closed forms that a wrong order of divide and
 *               round fails (tests/test_oracle_pins.py).
 *   parity unpinned : the rounding ORDER of float reductions for N >= 3 inside the
 *               un-vendored oneCCL library, oneCCL's own bf16/fp16 arithmetic, and
 *               NaN payload / MIN,MAX-with-NaN behaviour of oneCCL.  The oracle uses the
 *               ascending-rank fp32 chain with one final round-to-nearest-even, the
 *               order the in-tree small kernel uses, and propagates NaN through MIN / MAX
 *               (what torch.min / torch.max do).
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp, no fast-math, no FMA contraction).
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* dtype and op codes: same numbering as include/mccl.h */
enum { DT_U8 = 0, DT_I8 = 1, DT_I16 = 2, DT_I32 = 3, DT_I64 = 4,
       DT_F16 = 5, DT_F32 = 6, DT_F64 = 7, DT_BF16 = 8 };
enum { OP_SUM = 0, OP_AVG = 1, OP_PROD = 2, OP_MIN = 3, OP_MAX = 4 };

static int g_threads = 1;

void oracle_set_threads(int t) { g_threads = t < 1 ? 1 : t; }
int oracle_get_threads(void) { return g_threads; }
int oracle_max_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------- scalar conversions (bit patterns in, bit patterns out) ---------- */

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 -> fp32 is exact: the 16 bits are the top half of the fp32 pattern. */
float oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; every NaN becomes the canonical 0x7FC0. */
uint16_t oracle_f32_to_bf16(float f)
{
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* fp16 -> fp32, exact (subnormals normalised by hand). */
float oracle_f16_to_f32(uint16_t h)
{
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1fu) return u2f(sign | 0x7f800000u | (man << 13));
  if (exp != 0) return u2f(sign | ((exp + 112u) << 23) | (man << 13));
  if (man == 0) return u2f(sign);
  /* subnormal: value = man * 2^-24 */
  int e = 0;
  while (!(man & 0x400u)) { man <<= 1; ++e; }
  man &= 0x3ffu;
  return u2f(sign | ((uint32_t)(113 - e) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even, gradual underflow; NaN -> canonical 0x7E00. */
uint16_t oracle_f32_to_f16(float f)
{
  uint32_t u = f2u(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return 0x7e00;
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);   /* >= 65536 (incl. inf) */
  if (a >= 0x38800000u) {                                    /* normal fp16 range */
    uint32_t r = a - 0x38000000u;                            /* rebias 127 -> 15 */
    r += 0xfffu + ((r >> 13) & 1u);                          /* may carry into inf: correct */
    return (uint16_t)(sign | (r >> 13));
  }
  if (a < 0x33000000u) return (uint16_t)sign;                /* < 2^-25 rounds to zero */
  /* subnormal result: shift the 24-bit significand right with RNE */
  uint32_t e = a >> 23;                                      /* 102..112 */
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift = 126u - e;                                 /* 14..24 */
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | q);
}

/* ---------- the N-buffer reduction ---------- */

/* One element of the chain.  SUM starts from literal +0 and adds rank 0..N-1
 * (allreduce_small.h:347-352); the other ops start from rank 0's value.
 * AVG (floats only; the reference rejects it on device, dispatch_stub.h:320-335) is the SUM
 * chain followed by ONE division by n in the accumulation type, then the single rounding to the
 * storage type.
 * MIN / MAX propagate NaN whatever the rank order: a NaN input replaces the accumulator
 * (x != x), and no later value replaces a NaN accumulator (both compares are false), so the
 * result is the NaN of the highest rank that holds one, bits untouched. */
#define REDUCE_FLOAT_CHAIN(ACC_T, LOAD, STORE)                         \
  for (size_t i = 0; i < count; ++i) {                                 \
    ACC_T acc;                                                         \
    if (op == OP_SUM || op == OP_AVG) {                                \
      acc = (ACC_T)0;                                                  \
      for (int r = 0; r < n; ++r) acc = acc + LOAD(r, i);              \
      if (op == OP_AVG) acc = acc / (ACC_T)n;                          \
    } else {                                                           \
      acc = LOAD(0, i);                                                \
      for (int r = 1; r < n; ++r) {                                    \
        ACC_T x = LOAD(r, i);                                          \
        if (op == OP_PROD) acc = acc * x;                              \
        else if (op == OP_MIN) acc = (x < acc || x != x) ? x : acc;    \
        else acc = (x > acc || x != x) ? x : acc;                      \
      }                                                                \
    }                                                                  \
    STORE(i, acc);                                                     \
  }

/* Integers: SUM / PROD wrap modulo 2^bits (done in the unsigned twin type). */
#define REDUCE_INT_CHAIN(T, UT)                                        \
  {                                                                    \
    T* o = (T*)out;                                                    \
    for (size_t i = 0; i < count; ++i) {                               \
      T acc;                                                           \
      if (op == OP_SUM) {                                              \
        UT a = 0;                                                      \
        for (int r = 0; r < n; ++r) a = (UT)(a + (UT)((const T*)in[r])[i]); \
        acc = (T)a;                                                    \
      } else if (op == OP_PROD) {                                      \
        UT a = (UT)((const T*)in[0])[i];                               \
        for (int r = 1; r < n; ++r) a = (UT)(a * (UT)((const T*)in[r])[i]); \
        acc = (T)a;                                                    \
      } else {                                                         \
        acc = ((const T*)in[0])[i];                                    \
        for (int r = 1; r < n; ++r) {                                  \
          T x = ((const T*)in[r])[i];                                  \
          if (op == OP_MIN) acc = (x < acc) ? x : acc;                 \
          else acc = (x > acc) ? x : acc;                              \
        }                                                              \
      }                                                                \
      o[i] = acc;                                                      \
    }                                                                  \
  }

static int reduce_range(const void* const* in, int n, void* out, size_t count, int dtype, int op)
{
  switch (dtype) {
    case DT_F32: {
#define LD(r, i) (((const float*)in[r])[i])
#define ST(i, v) (((float*)out)[i] = (v))
      REDUCE_FLOAT_CHAIN(float, LD, ST)
#undef LD
#undef ST
      return 0;
    }
    case DT_F64: {
#define LD(r, i) (((const double*)in[r])[i])
#define ST(i, v) (((double*)out)[i] = (v))
      REDUCE_FLOAT_CHAIN(double, LD, ST)
#undef LD
#undef ST
      return 0;
    }
    case DT_BF16: {
#define LD(r, i) oracle_bf16_to_f32(((const uint16_t*)in[r])[i])
#define ST(i, v) (((uint16_t*)out)[i] = oracle_f32_to_bf16(v))
      REDUCE_FLOAT_CHAIN(float, LD, ST)
#undef LD
#undef ST
      return 0;
    }
    case DT_F16: {
#define LD(r, i) oracle_f16_to_f32(((const uint16_t*)in[r])[i])
#define ST(i, v) (((uint16_t*)out)[i] = oracle_f32_to_f16(v))
      REDUCE_FLOAT_CHAIN(float, LD, ST)
#undef LD
#undef ST
      return 0;
    }
    case DT_U8:  REDUCE_INT_CHAIN(uint8_t, uint8_t)   return 0;
    case DT_I8:  REDUCE_INT_CHAIN(int8_t, uint8_t)    return 0;
    case DT_I16: REDUCE_INT_CHAIN(int16_t, uint16_t)  return 0;
    case DT_I32: REDUCE_INT_CHAIN(int32_t, uint32_t)  return 0;
    case DT_I64: REDUCE_INT_CHAIN(int64_t, uint64_t)  return 0;
    default: return -1;
  }
}

size_t oracle_dtype_size(int dtype)
{
  switch (dtype) {
    case DT_U8: case DT_I8: return 1;
    case DT_I16: case DT_F16: case DT_BF16: return 2;
    case DT_I32: case DT_F32: return 4;
    case DT_I64: case DT_F64: return 8;
    default: return 0;
  }
}

/* out[i] = reduce over ranks of in[r][i].  out may be one of the inputs (in place). */
int oracle_reduce(const void* const* in, int n, void* out, size_t count, int dtype, int op)
{
  size_t es = oracle_dtype_size(dtype);
  if (es == 0 || n < 1) return -1;
  if (op != OP_SUM && op != OP_AVG && op != OP_PROD && op != OP_MIN && op != OP_MAX) return -1;
  if (op == OP_AVG && !(dtype == DT_F16 || dtype == DT_F32 || dtype == DT_F64 || dtype == DT_BF16)) return -1;
  int nt = g_threads;
  if (nt <= 1 || count < 4096) return reduce_range(in, n, out, count, dtype, op);
  int rc = 0;
#ifdef _OPENMP
#pragma omp parallel num_threads(nt)
  {
    int t = omp_get_thread_num();
    int T = omp_get_num_threads();
    size_t lo = count * (size_t)t / (size_t)T;
    size_t hi = count * (size_t)(t + 1) / (size_t)T;
    const void* ptrs[256];
    for (int r = 0; r < n && r < 256; ++r) ptrs[r] = (const char*)in[r] + lo * es;
    int e = reduce_range(ptrs, n, (char*)out + lo * es, hi - lo, dtype, op);
    if (e) {
#pragma omp atomic write
      rc = e;
    }
  }
#else
  rc = reduce_range(in, n, out, count, dtype, op);
#endif
  return rc;
}

/* Shard s of every rank's input is the slice [s*M, (s+1)*M); out[s - first] receives
 * its reduction (dpcpp_ccl.cpp:971-1019: rank r's output is shard r). */
int oracle_reduce_scatter(const void* const* in, int n, void* const* out, size_t shard_count,
                          int shard_first, int shard_num, int dtype, int op)
{
  size_t es = oracle_dtype_size(dtype);
  if (es == 0 || n < 1 || n > 256) return -1;
  for (int s = 0; s < shard_num; ++s) {
    const void* ptrs[256];
    for (int r = 0; r < n; ++r)
      ptrs[r] = (const char*)in[r] + (size_t)(shard_first + s) * shard_count * es;
    int e = oracle_reduce(ptrs, n, out[s], shard_count, dtype, op);
    if (e) return e;
  }
  return 0;
}

/* out[k*bytes : (k+1)*bytes] = in[k]  (dpcpp_ccl.cpp:1147-1192) */
int oracle_allgather(const void* const* in, int n, void* out, size_t bytes_per_rank)
{
  for (int k = 0; k < n; ++k)
    memcpy((char*)out + (size_t)k * bytes_per_rank, in[k], bytes_per_rank);
  return 0;
}

/* Split-size arithmetic of alltoall_base (dpcpp_ccl.cpp:1431-1445).
 * numel / dim0 describe one rank's tensor; split == NULL means "equal split".
 * counts[i] (elements) = split ? split[i]*rowLen : numel/world; displs = exclusive scan. */
int oracle_alltoall_counts(int world, int64_t numel, int64_t dim0, const int64_t* split,
                           int64_t* counts, int64_t* displs)
{
  int64_t len = numel;
  if (len) {
    int64_t div = split ? dim0 : world;
    if (div == 0) return -1;
    len /= div;
  }
  int64_t acc = 0;
  for (int i = 0; i < world; ++i) {
    counts[i] = split ? split[i] * len : len;
    displs[i] = acc;
    acc += counts[i];
  }
  return 0;
}

/* All ranks' alltoallv at once.  split_rows is the n x n matrix S[r][d] = rows rank r
 * sends to rank d.  Rank d's output segment r (offset = sum_{r'<r} S[r'][d]) receives
 * rank r's input segment d (offset = sum_{d'<d} S[r][d']). */
int oracle_alltoallv(const void* const* in, void* const* out, int n,
                     const int64_t* split_rows, size_t row_bytes)
{
  for (int d = 0; d < n; ++d) {
    size_t roff = 0;
    for (int r = 0; r < n; ++r) {
      size_t soff = 0;
      for (int dd = 0; dd < d; ++dd) soff += (size_t)split_rows[r * n + dd];
      size_t rows = (size_t)split_rows[r * n + d];
      memcpy((char*)out[d] + roff * row_bytes, (const char*)in[r] + soff * row_bytes,
             rows * row_bytes);
      roff += rows;
    }
  }
  return 0;
}

/* pack: dst = concat(src[0..n-1]); unpack: the inverse (dpcpp_ccl.cpp:1505-1538). */
int oracle_pack(const void* const* src, const size_t* bytes, int n, void* dst)
{
  size_t off = 0;
  for (int i = 0; i < n; ++i) { memcpy((char*)dst + off, src[i], bytes[i]); off += bytes[i]; }
  return 0;
}

int oracle_unpack(const void* src, void* const* dst, const size_t* bytes, int n)
{
  size_t off = 0;
  for (int i = 0; i < n; ++i) { memcpy(dst[i], (const char*)src + off, bytes[i]); off += bytes[i]; }
  return 0;
}

/* Vectorised conversion helpers so the pins can sweep many values quickly. */
void oracle_f32_to_bf16_array(const float* in, uint16_t* out, size_t n)
{ for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16(in[i]); }
void oracle_f32_to_f16_array(const float* in, uint16_t* out, size_t n)
{ for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16(in[i]); }
void oracle_f16_to_f32_array(const uint16_t* in, float* out, size_t n)
{ for (size_t i = 0; i < n; ++i) out[i] = oracle_f16_to_f32(in[i]); }
void oracle_bf16_to_f32_array(const uint16_t* in, float* out, size_t n)
{ for (size_t i = 0; i < n; ++i) out[i] = oracle_bf16_to_f32(in[i]); }

/* ---------- the steps either side of the MoE all_to_all (BASELINE config 5) ----------
 * The reference has no MoE code; its callers build the all_to_all_single input by a row
 * gather ("token permute") and, after the experts, undo it with a second all_to_all and a
 * weighted sum over each token's top-k copies.  These restate those index maps and the fp32
 * chain; they are pinned by brute-force loops on tagged inputs and by closed-form weights. */

/* dst row j = src row idx[j]; rows whose index is outside [0, src_rows) are left untouched */
int oracle_gather_rows(const void* src, size_t src_rows, const int64_t* idx, size_t nrows,
                       size_t row_bytes, void* dst)
{
  for (size_t j = 0; j < nrows; ++j) {
    if (idx[j] < 0 || (size_t)idx[j] >= src_rows) continue;
    memcpy((char*)dst + j * row_bytes, (const char*)src + (size_t)idx[j] * row_bytes, row_bytes);
  }
  return 0;
}

/* Fused dispatch for all n ranks: rank r's send order is idx[r] (source rows grouped by
 * destination, S[r][d] rows for destination d); rank d's output segment r receives them. */
int oracle_moe_dispatch(const void* const* hidden, const size_t* hidden_rows, const int64_t* const* idx,
                        void* const* out, int n, const int64_t* split_rows, size_t row_bytes)
{
  for (int d = 0; d < n; ++d) {
    size_t roff = 0;
    for (int r = 0; r < n; ++r) {
      size_t soff = 0;
      for (int dd = 0; dd < d; ++dd) soff += (size_t)split_rows[r * n + dd];
      size_t rows = (size_t)split_rows[r * n + d];
      oracle_gather_rows(hidden[r], hidden_rows[r], idx[r] + soff, rows, row_bytes,
                         (char*)out[d] + roff * row_bytes);
      roff += rows;
    }
  }
  return 0;
}

/* y[t][c] = sum_k w[t*topk+k] * x[src_rank[t*topk+k]][src_row[t*topk+k]][c]
 * fp32 chain from +0 in ascending k; each product is rounded to fp32 before it is added
 * (no fused multiply-add); one rounding to the storage type at the end. */
int oracle_moe_combine(const void* const* x, const size_t* x_rows, int n, const int32_t* src_rank,
                       const int64_t* src_row, const float* w, size_t tokens, int topk,
                       size_t hidden, int dtype, void* y)
{
  if (dtype != DT_BF16 && dtype != DT_F16 && dtype != DT_F32) return -1;
  for (size_t t = 0; t < tokens; ++t) {
    for (size_t c = 0; c < hidden; ++c) {
      float acc = 0.0f;
      for (int k = 0; k < topk; ++k) {
        size_t e = t * (size_t)topk + (size_t)k;
        int r = src_rank[e];
        int64_t row = src_row[e];
        if (r < 0 || r >= n || row < 0 || (size_t)row >= x_rows[r]) continue;
        size_t off = (size_t)row * hidden + c;
        float xv;
        if (dtype == DT_BF16) xv = oracle_bf16_to_f32(((const uint16_t*)x[r])[off]);
        else if (dtype == DT_F16) xv = oracle_f16_to_f32(((const uint16_t*)x[r])[off]);
        else xv = ((const float*)x[r])[off];
        volatile float prod = w[e] * xv; /* rounded product, never contracted into an fma */
        acc = acc + prod;
      }
      size_t o = t * hidden + c;
      if (dtype == DT_BF16) ((uint16_t*)y)[o] = oracle_f32_to_bf16(acc);
      else if (dtype == DT_F16) ((uint16_t*)y)[o] = oracle_f32_to_f16(acc);
      else ((float*)y)[o] = acc;
    }
  }
  return 0;
}

/* Routing counts of a MoE dispatch: counts[e] = number of pairs routed to expert e; ids outside
 * [0, n_experts) are ignored.  No reference file: the caller's step before the all_to_all_single
 * of src/gpu/dpcpp_ccl.cpp:1371-1466 (its inputSplitSizes are these counts summed per rank). */
int oracle_route_counts(const int32_t* expert_ids, size_t npairs, int n_experts, int64_t* counts)
{
  if (n_experts < 1 || !counts) return -1;
  for (int e = 0; e < n_experts; ++e) counts[e] = 0;
  for (size_t i = 0; i < npairs; ++i) {
    int32_t e = expert_ids[i];
    if (e >= 0 && e < n_experts) counts[e] += 1;
  }
  return 0;
}
