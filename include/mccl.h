/*
 * mccl.h -- C ABI of libmi355ccl.so: the local-reduce and pack/permute kernels of the
 * collective data path on one MI355X (gfx950).
 *
 * The N "peer" buffers of a collective are N device pointers.  In single-GPU mode they
 * are N allocations in one GPU's HBM; on a multi-GPU node the same entry points take
 * peer-mapped pointers.  Every entry point
 *   - takes plain pointers and sizes (no torch types), and an explicit hipStream_t
 *     (passed as void*; NULL = the HIP null stream),
 *   - only enqueues work on that stream and returns; it never synchronises,
 *   - allocates no device memory,
 *   - returns MCCL_OK (0) or a negative mccl_status_t; mccl_last_error() then holds a
 *     message for the calling thread.  Nothing throws across this boundary.
 *
 * Citations (file:line) are relative to the reference tree (intel/torch-ccl).
 */
#ifndef MCCL_H_
#define MCCL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types: the entries of cclDatatypes, src/utils.cpp:46-58 (Bool travels as U8). */
typedef enum {
  MCCL_U8 = 0,
  MCCL_I8 = 1,
  MCCL_I16 = 2,
  MCCL_I32 = 3,
  MCCL_I64 = 4,
  MCCL_F16 = 5,
  MCCL_F32 = 6,
  MCCL_F64 = 7,
  MCCL_BF16 = 8
} mccl_dtype_t;

/* Reduction ops: the entries of cclOps, src/utils.cpp:38-44, numbered like
 * c10d::ReduceOp (SUM 0, AVG 1, PRODUCT 2, MIN 3, MAX 4).  AVG is this library's
 * addition (the reference rejects it on device, src/dispatch_stub.h:320-335): the
 * SUM chain followed by one division by n in the accumulation type. */
typedef enum {
  MCCL_SUM = 0,
  MCCL_AVG = 1,
  MCCL_PROD = 2,
  MCCL_MIN = 3,
  MCCL_MAX = 4
} mccl_op_t;

typedef enum {
  MCCL_OK = 0,
  MCCL_ERR_INVALID_ARG = -1, /* null pointer, bad enum, n out of range, bad alignment */
  MCCL_ERR_HIP = -2,         /* a HIP runtime call failed; message names it */
  MCCL_ERR_UNSUPPORTED = -3
} mccl_status_t;

/* Launch shape of the reduction (the reference switches at SMALL_MAX_COUNT between a
 * single-launch kernel and a persistent one, src/gpu/dpcpp_ccl.cpp:771-775). */
typedef enum {
  MCCL_VARIANT_AUTO = 0,       /* pick by size: SMALL up to MCCL_TUNE_SMALL_MAX_BYTES per rank
                                  (4 MiB), STREAM once (n+1)*bytes reaches
                                  MCCL_TUNE_STREAM_MIN_TOTAL_BYTES (112 MiB); in between
                                  PERSISTENT for 4 ranks or more, SMALL for fewer.  Whatever the
                                  shape, outputs of launches beyond those sizes are written with
                                  streaming stores, smaller ones stay cacheable */
  MCCL_VARIANT_SMALL = 1,      /* one wavefront per workgroup, one vector per lane, grid covers
                                  the message, no residency cap: lowest latency */
  MCCL_VARIANT_PERSISTENT = 2, /* fixed grid sized to the CUs, grid-stride loop */
  MCCL_VARIANT_STREAM = 3      /* SMALL's geometry with residency capped (through a dynamic-LDS
                                  reservation) so that about 14 MB of loads are in flight over the
                                  chip and no more: highest bandwidth on large messages */
} mccl_variant_t;

/* Tuning knobs for mccl_set_tuning (process-wide; meant for benchmarks and sweeps). */
typedef enum {
  MCCL_TUNE_PERSISTENT_BLOCKS_PER_CU = 0, /* grid of the PERSISTENT shape */
  MCCL_TUNE_STREAM_WAVES_PER_CU = 1,      /* resident wavefronts per CU of the STREAM shape; default 0 =
                                             chosen by the number of loads a wavefront keeps in flight
                                             (8 ranks: 8, 4 ranks: 12, 2 ranks: no cap) */
  MCCL_TUNE_SMALL_MAX_BYTES = 2,          /* per-rank bytes up to which AUTO picks SMALL */
  MCCL_TUNE_COPY_WAVES_PER_CU = 3,        /* residency cap of the segmented copy */
  MCCL_TUNE_STREAM_MIN_TOTAL_BYTES = 4,   /* (n+1)*bytes from which AUTO picks STREAM */
  MCCL_TUNE_COMBINE_PIECES_PER_WAVE = 5,  /* 1 KiB row pieces one wavefront of moe_combine walks */
  MCCL_TUNE_COMBINE_WAVES_PER_CU = 6,     /* moe_combine with top-k <= 8: default 0 = one wavefront per
                                             row chunk; > 0 = persistent grid of that many wavefronts
                                             per CU, each walking several chunks (measured slower) */
  MCCL_TUNE_XRANK_WAVES_ALL_RANKS = 7,    /* wavefronts the launches of ALL ranks of a one-launch
                                             collective (mccl_*_sync) may hold together; each
                                             rank's grid is this divided by the rank count.  A
                                             launch that waits at its start is cut further, to the
                                             rank's share of half of what the kernel's registers
                                             let the GPU hold at once (asked of the runtime per
                                             kernel), so that waiting ranks never fill the GPU */
  MCCL_TUNE_COPY_VECTORS_PER_LANE = 8,    /* segmented copy: 2 or 4 vectors of 16 bytes per lane per chunk
                                             (2 KiB or 4 KiB per wavefront); any other value = chosen by
                                             the total size of the call */
  MCCL_TUNE_COPY_STREAM_STORES = 9,       /* segmented copy, full chunks: 1 = stores written through past
                                             the caches, 2 = non-temporal stores; else chosen by size */
  MCCL_TUNE_COPY_LARGE_MIN_BYTES = 10,    /* total bytes of a copy call from which the large-copy
                                             geometry applies */
  MCCL_TUNE_GATHER_WAVES_PER_CU = 11,     /* residency cap of the row gather / fused MoE dispatch */
  MCCL_TUNE_XRANK_CACHED_LOADS = 12,      /* one-launch reductions: 1 = the peers' tensors are read
                                             through the caches after one invalidate per workgroup,
                                             0 = past the caches, access by access, 2 (default) =
                                             through the caches without an invalidate when the
                                             launch does not wait at its start (whatever the peers
                                             wrote, they wrote in kernels that had ended before this
                                             one began: its caches start clean), else as 0 */
  MCCL_TUNE_XRANK_FRESH_WAVES_PER_CU = 13, /* one-launch reductions and pushes that do not wait at their
                                             start (ready_epoch 0: the caller has ordered the ranks, e.g.
                                             with mccl_rank_barrier in front): residency cap of their
                                             single-wavefront workgroups, 32 and more = none */
  MCCL_TUNE_XRANK_FRESH_MAX_WAVES = 14,   /* the same launches: at most this many workgroups (a walk
                                             over several tiles each above it); 0 = one workgroup per
                                             tile (reductions) or per two tiles (pushes) */
  MCCL_TUNE_COUNT_ = 15
} mccl_tune_t;

#define MCCL_MAX_RANKS 64

/* One contiguous byte range to copy. */
typedef struct {
  const void* src;
  void* dst;
  size_t bytes;
} mccl_segment_t;

int mccl_version(void);

/* Message for the last non-OK status returned on this thread ("" if none). */
const char* mccl_last_error(void);

size_t mccl_dtype_size(int dtype);

/*
 * N-buffer reduction: out[i] = in[0][i] (op) in[1][i] (op) ... (op) in[n-1][i], i < count.
 * Replaces the sum loop of allreducer_small<T>::allreduce (src/gpu/allreduce_small.h:289-361)
 * and the data kernels of allreducer<T>::allreduce (src/gpu/allreduce.h:306-533), and the
 * ccl::allreduce call of src/gpu/dpcpp_ccl.cpp:781-788.
 *   - order: ascending rank; SUM starts from +0 like the reference's "result = 0".
 *   - f16 / bf16 accumulate in fp32 and round once (nearest even) on store; f32, f64 and
 *     the integer types accumulate in their own type (integers wrap).
 *   - NaN: SUM / AVG / PROD follow IEEE arithmetic.  MIN / MAX propagate NaN whatever the rank
 *     order (a NaN input replaces the accumulator, nothing replaces a NaN accumulator), like
 *     torch.min / torch.max; the result is the NaN of the highest rank that holds one.  f16 /
 *     bf16 results that are NaN are stored as the canonical quiet NaN (0x7E00 / 0x7FC0); f32 /
 *     f64 NaN payloads of arithmetic results are not part of the contract.
 *   - out may be exactly one of the inputs (in place; on large messages that is 3-5 % faster than
 *     a separate output: the write lands on DRAM pages just read); any other overlap between an output and
 *     a range the same launch reads or writes is refused with MCCL_ERR_INVALID_ARG (this holds
 *     for the shard and coalesced forms below too).
 *   - any count, any element-aligned pointers; 1 <= n <= MCCL_MAX_RANKS.
 */
int mccl_reduce_n(const void* const* in, int n, void* out, size_t count, int dtype, int op,
                  int variant, void* stream);

/*
 * Shard reduction of reduce_scatter: for s in [shard_first, shard_first + shard_num):
 *   out[s - shard_first][j] = reduce_k in[k][s * shard_count + j],  j < shard_count.
 * One launch covers all requested shards.  Replaces ccl::reduce_scatter at
 * src/gpu/dpcpp_ccl.cpp:1002-1008 (rank r calls it with shard_first = r, shard_num = 1).
 */
int mccl_reduce_scatter_n(const void* const* in, int n, void* const* out, size_t shard_count,
                          int shard_first, int shard_num, int dtype, int op, void* stream);

/*
 * Coalesced reductions: nbuf independent N-buffer reductions in one launch
 * (allreduce_coalesced, src/gpu/dpcpp_ccl.cpp:810-818).  in is laid out [nbuf][n]
 * (buffer-major), out and counts have nbuf entries.
 */
int mccl_reduce_multi(const void* const* in, int n, void* const* out, const size_t* counts,
                      int nbuf, int dtype, int op, void* stream);

/*
 * Cross-rank barrier on device flags, for ranks that are processes (or GPUs) of their own: the
 * one-thread sync kernels between the data kernels of the reference's large allreduce
 * (src/gpu/allreduce.h:731-769, 835-877).  flags[r] is the address, in the caller's own mapping,
 * of rank r's 64-bit flag word (device memory the peers can reach, e.g. opened from an IPC handle;
 * zero before the first use).  One wavefront stores `epoch` into flags[rank] and then waits until
 * every flags[r] has reached `epoch`.  Epochs must grow from call to call (the words are never
 * cleared) and all ranks must pass the same epoch for the same barrier.  Stream-ordered: what the
 * stream enqueued before the barrier is complete and visible to a peer's kernels enqueued after
 * its own barrier of the same epoch.  No host thread takes part.
 *   The wait is bounded: after timeout_us microseconds (0 = 10 s) the kernel stores 1 + the rank it
 * was waiting for into status[0] and the low half of the epoch into status[1], and returns; status
 * may be null, or two 32-bit words the GPU can write (device memory or mapped pinned host memory)
 * that the caller zeroes and reads.
 *   Callers whose ranks share one process must give every rank a stream that maps to a hardware
 * queue of its own: a waiting wavefront blocks the kernels queued behind it.
 */
int mccl_rank_barrier(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us,
                      void* status, void* stream);

/*
 * mccl_rank_barrier that also tells every rank WHERE the other ranks' buffers of the coming
 * collective are, so that no host thread has to: the reference exchanges the handles of its buffers
 * once (src/gpu/dpcpp_ccl.cpp:105-121 -> src/gpu/allreduce.h:546-594, 1208-1248) and afterwards a
 * collective is a pure enqueue; here the buffers are the callers' own tensors, which change from
 * call to call, so what is exchanged once is the ALLOCATION (mapped by every peer, on the host,
 * whenever the owner announces a new one) and what travels per collective, on the device, is which
 * allocation and where in it.
 *   Before it stores `epoch` into flags[rank], the wavefront stores *mine into offers[rank] (this
 * rank's offer slot: 32 bytes of device memory the peers can reach, 8-byte aligned; a slot may be
 * written again once every peer has started a later barrier -- two alternating slots do).  After
 * rank r's flag has arrived, lane r reads offers[r] and looks the offer up in *imports, this rank's
 * table of the peers' allocations as it has mapped them (device memory of this rank, filled by the
 * host in stream order before the launch): entry e of rank r at generation g is at
 * imports->base[r][e] when imports->generation[r][e] == g; entry MCCL_OFFER_STAGED means rank r's
 * staging buffer `slot`, imports->staging[r][slot] (slots 0 and 1: the rank's two staging buffers,
 * the same for every reader; MCCL_OFFER_SLOT_OUTBOX: the buffer rank r keeps for THIS reader
 * alone, see mccl_rank_barrier_offers_each).  The address of every rank's buffer in this
 * rank's address space -- base + offset; my_buffer for this rank itself -- goes to resolved[0..n),
 * n 64-bit words of this rank's device memory, for the kernels that follow on the stream
 * (mccl_allreduce_sync_resolved).  An offer that this rank has not mapped leaves a null pointer
 * there and is reported: status[0] = 1 + the rank, status[1] = MCCL_STATUS_UNMAPPED.  At most
 * MCCL_OFFER_RANKS ranks.  Everything else as mccl_rank_barrier.
 */
#define MCCL_OFFER_RANKS 8
#define MCCL_OFFER_ENTRIES 32
#define MCCL_OFFER_STAGED 0xffffffffu
#define MCCL_OFFER_SLOTS 4
#define MCCL_OFFER_SLOT_OUTBOX 2u
#define MCCL_STATUS_UNMAPPED 0xfffffffeu
#define MCCL_STATUS_MISMATCH 0xfffffffdu
typedef struct mccl_offer {
  uint32_t entry;      /* index in the owner's table of announced allocations, or MCCL_OFFER_STAGED */
  uint32_t slot;       /* with MCCL_OFFER_STAGED: which of the owner's staging buffers (< MCCL_OFFER_SLOTS) */
  uint64_t generation; /* of the entry: changes when the owner reuses it for another allocation */
  uint64_t offset;     /* bytes from the start of the allocation (or of the staging buffer) */
  uint64_t bytes;      /* mccl_rank_barrier_offers_each: length of the piece, which the reader checks; else 0 */
} mccl_offer_t;
typedef struct mccl_import_table {
  uint64_t base[MCCL_OFFER_RANKS][MCCL_OFFER_ENTRIES];
  uint64_t generation[MCCL_OFFER_RANKS][MCCL_OFFER_ENTRIES];
  uint64_t staging[MCCL_OFFER_RANKS][MCCL_OFFER_SLOTS];
} mccl_import_table_t;
int mccl_rank_barrier_offers(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us, void* status,
                             const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                             const mccl_import_table_t* imports, void* resolved, void* stream);

/*
 * The same for collectives in which a rank hands every peer a DIFFERENT piece (alltoall(v):
 * src/gpu/dpcpp_ccl.cpp:1371-1466): a rank publishes a row of n offers, mine[k] = where the piece
 * for rank k is and how long it is (mine[k].bytes), and reads the column addressed to it:
 * offers[r] is rank r's row (n x 32 bytes of device memory the peers can reach), of which this rank
 * reads entry `rank`.  expect_bytes[r] is what this rank expects from rank r: a piece of another
 * length is reported (status[0] = 1 + r, status[1] = MCCL_STATUS_MISMATCH) and resolves to null -- the
 * counts of an alltoallv are the callers' to keep consistent (outSplit_d[r] == inSplit_r[d]), and
 * nobody else can check them without a rendezvous.  A piece of length 0 resolves to null without
 * being looked up.  resolved[r] = where rank r's piece for this rank starts, for
 * mccl_copy_segments_sync_resolved behind it on the stream; resolved[rank] = my_source, this rank's
 * own piece.  Pieces a rank cannot offer in place it copies into a buffer it keeps for that one
 * reader (MCCL_OFFER_STAGED, slot MCCL_OFFER_SLOT_OUTBOX: imports->staging[r][2] is rank r's outbox
 * for this rank): only the two of them know the length of the piece, so only they can agree, without
 * anybody else, on when that buffer has to grow.
 */
int mccl_rank_barrier_offers_each(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us, void* status,
                                  const mccl_offer_t* mine, const uint64_t* expect_bytes, const void* my_source,
                                  void* const* offers, const mccl_import_table_t* imports, void* resolved, void* stream);

/*
 * Stream-ordered update of an import table in device memory: entry `entry` of rank `rank` is now
 * mapped at `base` at generation `generation` (base 0: not mapped any more), or staging buffer
 * `slot` of rank `rank` is at `base` (entry MCCL_OFFER_STAGED).  The values travel inside the launch, so
 * the caller's memory may change as soon as the call returns, and a barrier enqueued earlier on the
 * stream still resolves against the table as it was.  At most MCCL_IMPORT_UPDATES per call.
 */
#define MCCL_IMPORT_UPDATES 8
typedef struct mccl_import_update {
  uint32_t rank;
  uint32_t entry;       /* < MCCL_OFFER_ENTRIES: an allocation; MCCL_OFFER_STAGED: a staging buffer, `slot` (< MCCL_OFFER_SLOTS) says which */
  uint32_t slot;
  uint32_t reserved;
  uint64_t base;
  uint64_t generation;
} mccl_import_update_t;
int mccl_import_table_update(mccl_import_table_t* table, const mccl_import_update_t* updates, int n, void* stream);

/*
 * One-launch small allreduce across rank processes: copy-in, rank synchronisation and the
 * N-peer reduction in a single kernel, the structure of allreducer_small<T>::allreduce
 * (src/gpu/allreduce_small.h:166-361).  Rank `rank` contributes in[0..count) and receives the
 * reduction of all n contributions in out (out may be in).  stage[r] is rank r's staging buffer
 * (at least count elements rounded up to 16 bytes, 16-byte aligned) and tile_flags[r] its array of
 * 32-bit flags, one per MCCL_FUSED_TILE_BYTES of message (zero before the first use), both in the
 * caller's own mapping.  Every rank calls with the same count, dtype, op and epoch; epochs must
 * grow from call to call on the same staging buffers, and a staging buffer may be reused only
 * after every peer has started a later collective (two alternating sets do).  Same arithmetic and
 * bits as mccl_reduce_n over the n contributions.  At most MCCL_FUSED_MAX_RANKS ranks.  The wait
 * is bounded and reported like mccl_rank_barrier's; a tile whose peers did not arrive in time is
 * left unwritten.  The launch is one workgroup per 16 KiB of message, and a workgroup sits on one
 * compute unit: while it waits for a late rank it holds count * size / 16 KiB of the GPU's 256
 * compute units.  max_compute_units (0 = no limit) caps that: the launch is then at most that
 * many workgroups, whose wavefronts take up to four tiles each, and a message of more than
 * max_compute_units * 64 KiB is refused.  A wavefront waits for the same tile of every peer, so
 * the launches of all ranks that share a GPU must be resident together with room to spare (an
 * MI355X holds 512 such workgroups when nothing else runs): ranks that share a GPU pass a limit
 * -- at most 256 / n; 128 / n leaves half of the compute units to a late rank's other kernels.
 */
#define MCCL_FUSED_MAX_RANKS 8
#define MCCL_FUSED_TILE_BYTES 1024
int mccl_allreduce_fused(const void* in, void* out, size_t count, int dtype, int op,
                         void* const* stage, void* const* tile_flags, int n, int rank, uint32_t epoch,
                         uint64_t timeout_us, void* status, unsigned max_compute_units, void* stream);

/*
 * mccl_allreduce_fused whose epoch lives on the device, so that the launch can be recorded in a HIP
 * graph and replayed: the reference advances the index of its triple buffer on the host at every
 * call (`buffer_index`, src/gpu/allreduce_small.h:118, 139); a replayed launch
 * has no host call, so the launch reads the epoch from `state` when it starts and its last
 * wavefront stores the next one.  state: MCCL_FUSED_STATE_BYTES of THIS rank's device memory,
 * 64-byte aligned, zero before the first use, never written by the caller afterwards.  stage[r] /
 * tile_flags[r] address the first of rank r's TWO staging buffers / flag arrays; the second lies
 * stage_stride / flags_stride bytes behind it (multiples of 16 / 4; the message and its flags must
 * fit in between).  The launch with epoch e uses set (e & 1).  Everything else as
 * mccl_allreduce_fused, with the same results.  All ranks must issue the same sequence of calls on
 * the same buffers (as for any collective); eager calls and replays of recorded ones may be mixed
 * freely, in one stream order per rank.  Records no memset and allocates nothing.
 *   flags: 0, or one of the bisecting switches of the reference's small allreduce
 * (TORCH_CCL_WORK_ONLY / TORCH_CCL_SYNC_ONLY, src/gpu/dpcpp_ccl.cpp:56-85; the work_only and
 * sync_only kernels of src/gpu/allreduce_small.h:414-701, 703-999): MCCL_FUSED_WORK_ONLY runs the
 * launch without its rank waits (copy-in, flags, and the reduction of whatever the peers' buffers
 * hold at that moment), MCCL_FUSED_SYNC_ONLY runs nothing but the flags and the waits.  Both are for
 * timing what each part costs; the output of either is not a result.  All ranks pass the same flags.
 */
#define MCCL_FUSED_STATE_BYTES 128
#define MCCL_FUSED_WORK_ONLY 1u
#define MCCL_FUSED_SYNC_ONLY 2u
int mccl_allreduce_fused_replayable(const void* in, void* out, size_t count, int dtype, int op,
                                    void* const* stage, void* const* tile_flags, size_t stage_stride, size_t flags_stride,
                                    void* state, int n, int rank, uint64_t timeout_us, void* status,
                                    unsigned max_compute_units, unsigned flags, void* stream);

/*
 * One-launch collectives between rank processes that read the peers' buffers in place.  With
 * several processes on one GPU every launch of a process waits for its turn at the dispatcher, so
 * the cross-rank waits are folded into the data kernel: the launch itself publishes "this rank's
 * stream has reached the collective" (ready_epoch, in words[rank]), every workgroup waits until all
 * ranks' words have reached ready_epoch before it touches a peer's buffer, and -- when done_epoch
 * is non-zero -- the kernel does not complete before every rank has published done_epoch, i.e. has
 * finished reading (the caller's buffers may then be reused in stream order).  This replaces the
 * separate sync kernels of src/gpu/allreduce.h:731-769, 835-877 around the data kernels.
 *   words[r]: rank r's 64-bit word as for mccl_rank_barrier (the same word may serve both; epochs
 * grow: ready_epoch of a call > any epoch used before, done_epoch > ready_epoch).  done_counter:
 * MCCL_SYNC_COUNTER_BYTES of this rank's device memory, 64-byte aligned, zero before the first call
 * (the kernel leaves them zero): the workgroups count themselves out there, and the workgroup with
 * the highest index watches the counters and does the closing wait.  ready_epoch == 0: no
 * opening wait, for callers that have ordered the start of the ranks themselves -- with an
 * mccl_rank_barrier launch in front (then only the kernel's last workgroup ever waits, for the
 * closing epoch: one wavefront per rank instead of the whole grid, which matters when several
 * ranks share a GPU with other kernels), or with host barriers around the launch (done_epoch 0 as
 * well: the kernel does not wait at all; words, counters and status are then not used).
 * Waits are bounded and reported like mccl_rank_barrier's.  At most 8 ranks.  The grids of launches
 * that wait at their start are sized so that all ranks' launches are resident together
 * (MCCL_TUNE_XRANK_WAVES_ALL_RANKS); a launch without an opening wait can keep nobody out, and the
 * shard reduction and the push then run as fresh workgroups of one or two tiles each
 * (MCCL_TUNE_XRANK_FRESH_MAX_WAVES, MCCL_TUNE_XRANK_FRESH_WAVES_PER_CU).
 * max_compute_units: 0 -- single-wavefront workgroups, spread over the whole GPU, as many as the
 * budget allows (the fastest shape for large messages); k > 0 -- at most k workgroups of up to 16
 * wavefronts: a workgroup sits on one compute unit, so the launch holds at most k of the GPU's 256
 * while it waits for a late rank, and the late rank's other kernels find the rest free.  Ranks
 * that share a GPU keep the sum over all ranks at half the GPU (8 ranks: 16 each); the message
 * should then be small enough for 16 k wavefronts (a few MiB).
 */
#define MCCL_SYNC_COUNTER_BYTES 4096
typedef struct {
  void* const* words;
  int n;
  int rank;
  uint64_t ready_epoch;
  uint64_t done_epoch;
  void* done_counter;
  uint64_t timeout_us; /* 0 = 10 s */
  void* status;
  unsigned max_compute_units; /* 0 = no limit */
  unsigned reserved;          /* 0 */
} mccl_xsync_t;

/* mccl_copy_segments whose sources are peers' buffers: allgather / alltoall(v) / broadcast pulls
 * (ccl::allgatherv, ccl::alltoallv, src/gpu/dpcpp_ccl.cpp:1176-1182, 1428-1455) in one launch.
 * At most 64 segments; zero segments still take part in the waits.  flags: MCCL_COPY_SHARED_SOURCES
 * when the other ranks read the same source bytes in the same collective (allgather, broadcast):
 * the sources are then kept in the memory-side cache instead of being streamed past it. */
#define MCCL_COPY_SHARED_SOURCES 1u
int mccl_copy_segments_sync(const mccl_segment_t* segs, int nseg, unsigned flags, const mccl_xsync_t* sync,
                            void* stream);

/* allgather as pushes (ccl::allgatherv, src/gpu/dpcpp_ccl.cpp:1176-1182; stores into the peers'
 * buffers as in the gather step of src/gpu/allreduce.h:470-487): this rank's `bytes` at src are
 * written to dst[0..ndst) -- where this rank's contribution belongs in every rank's output, peers'
 * outputs through writable mappings -- read once and written through, so that a rank that has seen
 * done_epoch finds all contributions in its output.  1 to 8 destinations, any alignment; a
 * destination may be src itself (an allgather in place: nothing to copy there) but must not overlap
 * it otherwise.  With both epochs 0 it is a plain one-to-many copy. */
int mccl_fanout_sync(const void* src, void* const* dst, int ndst, size_t bytes, const mccl_xsync_t* sync,
                     void* stream);

/* mccl_reduce_n whose inputs are peers' buffers (in[r]: rank r's contribution at this rank's
 * slice): the shard reduction of reduce_scatter (ccl::reduce_scatter, src/gpu/dpcpp_ccl.cpp:1002-1008)
 * in one launch.  Same arithmetic and bits as mccl_reduce_n; out may be exactly one of the inputs
 * (a reduce_scatter in place: the output is this rank's slice of its own input, which no other rank
 * reads), and must not overlap an input otherwise. */
int mccl_reduce_sync(const void* const* in, void* out, size_t count, int dtype, int op,
                     const mccl_xsync_t* sync, void* stream);

/*
 * In-place allreduce of tensors[rank] over all ranks' tensors in one launch, for ranks whose
 * tensors are all writable by all ranks (as IPC-mapped device memory is).  Rank r reduces shard r
 * (mccl_allreduce_sync_shard(count, n) elements, the last shards may be shorter or empty) of all
 * tensors and writes the result into shard r of EVERY rank's tensor; nothing is staged and nothing
 * is copied a second time: n reads and n writes per element of a shard, where the two-shot
 * algorithm of the reference's large path (reduce-scatter through scratch, all-gather:
 * src/gpu/allreduce.h:306-533) moves n + 1 reads and 2 writes in two phases with a rank
 * synchronisation between them (its gather step stores into its peers' buffers likewise,
 * src/gpu/allreduce.h:470-487).  Only the owner of a shard touches it in any tensor while the
 * collective runs; done_epoch is required (unless ready_epoch is 0): no rank's kernel ends before
 * every rank has written its shard everywhere.  Same bits as mccl_reduce_n over the n tensors.
 */
size_t mccl_allreduce_sync_shard(size_t count, int n);
int mccl_allreduce_sync(void* const* tensors, size_t count, int dtype, int op, const mccl_xsync_t* sync,
                        void* stream);

/* mccl_allreduce_sync whose tensor addresses come from device memory: resolved[0..n) as
 * mccl_rank_barrier_offers of the same stream has just left them (the kernel reads them when it
 * starts).  The barrier in front has ordered the ranks: sync->ready_epoch must be 0 and
 * sync->done_epoch set.  A null address among them (an offer that could not be resolved, already
 * reported by the barrier) makes the launch skip its work and still take part in the closing wait. */
int mccl_allreduce_sync_resolved(const void* resolved, size_t count, int dtype, int op, const mccl_xsync_t* sync,
                                 void* stream);

/* The two in one launch, for messages small enough for a launch on few compute units: the launch
 * itself stores *mine into offers[rank] before its ready epoch, and after the opening wait every
 * wavefront resolves the peers' offers against *imports as mccl_rank_barrier_offers does (an offer
 * that does not resolve: reported, the launch only takes part in the closing wait).  sync->ready_epoch,
 * sync->done_epoch and sync->max_compute_units must be set (the packed shape: workgroups of sixteen
 * wavefronts on at most that many compute units). */
int mccl_allreduce_sync_offers(size_t count, int dtype, int op, const mccl_xsync_t* sync, const mccl_offer_t* mine,
                               const void* my_buffer, void* const* offers, const mccl_import_table_t* imports, void* stream);

/* mccl_reduce_sync and mccl_fanout_sync over addresses from the ranks' offers, in the same two
 * forms: `_resolved` behind mccl_rank_barrier_offers (sync->ready_epoch 0, done_epoch set), `_offers`
 * as one launch on few compute units that exchanges the offers itself (ready_epoch, done_epoch and
 * max_compute_units set).  What a rank offers is the buffer its peers address: for the shard
 * reduction (reduce_scatter) its whole input, of which rank r reads the `count` elements at byte
 * in_offset (its slice) of every rank's; for the push (allgather) its whole output, into which rank r
 * writes its `bytes` at byte dst_offset (its slice) of every rank's -- of its own as well, unless
 * skip_own is set (in place: the contribution already sits there). */
int mccl_reduce_sync_resolved(const void* resolved, size_t in_offset, void* out, size_t count, int dtype, int op,
                              const mccl_xsync_t* sync, void* stream);
int mccl_reduce_sync_offers(size_t in_offset, void* out, size_t count, int dtype, int op, const mccl_xsync_t* sync,
                            const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                            const mccl_import_table_t* imports, void* stream);
int mccl_fanout_sync_resolved(const void* src, const void* resolved, size_t dst_offset, size_t bytes, int skip_own,
                              const mccl_xsync_t* sync, void* stream);
int mccl_fanout_sync_offers(const void* src, size_t dst_offset, size_t bytes, int skip_own, const mccl_xsync_t* sync,
                            const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                            const mccl_import_table_t* imports, void* stream);

/*
 * mccl_copy_segments_sync whose sources come from the table a barrier with offers has resolved
 * (behind it on the stream: ready_epoch 0, done_epoch set): segment i is read from
 * resolved[src_rank[i]] + (size_t)segs[i].src -- segs[i].src is a byte offset there -- or, with
 * src_rank[i] < 0, from the address segs[i].src as it stands.  A segment whose table entry is null
 * (the barrier has reported why) is skipped.  This rank's share of an alltoall(v) as pulls
 * (ccl::alltoallv at src/gpu/dpcpp_ccl.cpp:1447-1455), with nothing about the peers' buffers known
 * on the host.
 */
int mccl_copy_segments_sync_resolved(const mccl_segment_t* segs, const int* src_rank, int nseg, const void* resolved,
                                     unsigned flags, const mccl_xsync_t* sync, void* stream);

/*
 * The all-to-all of one rank as ONE launch (ccl::alltoallv at src/gpu/dpcpp_ccl.cpp:1447-1455): what
 * mccl_rank_barrier_offers_each and mccl_copy_segments_sync_resolved do in two, plus the copies in
 * front of them, on sync->max_compute_units compute units (ready_epoch, done_epoch and
 * max_compute_units all set).  `stage` (at most MCCL_OFFER_RANKS segments) are the copies of this
 * rank's pieces into its outboxes, for the pieces it does not offer in place; when they are in memory
 * the launch publishes the row `mine` and the rank's ready epoch, waits for the peers', resolves the
 * column addressed to this rank and carries out `pulls` (at most MCCL_OFFER_RANKS; sources as in
 * mccl_copy_segments_sync_resolved, from what the launch has resolved).  Uses the word 128 bytes into
 * sync->done_counter besides the counters of the closing wait.  For messages small enough that a
 * launch costs more than the data; between rank processes that share a GPU every launch waits for
 * its process's turn.  The two-launch form and this one may be mixed among the ranks of one
 * collective.
 */
int mccl_alltoall_sync_offers(const mccl_segment_t* stage, int nstage, const mccl_segment_t* pulls, const int* src_rank, int npull,
                              const mccl_xsync_t* sync, const mccl_offer_t* mine, const uint64_t* expect_bytes, const void* my_source,
                              void* const* offers, const mccl_import_table_t* imports, void* stream);

/* Generic segmented copy: every segment is copied byte-exactly; segments must not overlap
 * each other's destinations.  The building block of the copy collectives below. */
int mccl_copy_segments(const mccl_segment_t* segs, int nseg, void* stream);

/* allgather: out[k*bytes_per_rank : (k+1)*bytes_per_rank] = in[k]
 * (ccl::allgatherv at src/gpu/dpcpp_ccl.cpp:1176-1182). */
int mccl_allgather_n(const void* const* in, int n, void* out, size_t bytes_per_rank,
                     void* stream);

/*
 * alltoall(v) for all n ranks at once.  split_rows is the n x n row-major matrix
 * S[r][d] = rows rank r sends to rank d (rank r's inputSplitSizes; rank d's
 * outputSplitSizes[r] must equal S[r][d]).  Rank d's output segment r, at row offset
 * sum_{r'<r} S[r'][d], receives rank r's input segment d, at row offset sum_{d'<d} S[r][d']
 * (count/displacement arithmetic of src/gpu/dpcpp_ccl.cpp:1431-1455).
 */
int mccl_alltoallv_n(const void* const* in, void* const* out, int n, const int64_t* split_rows,
                     size_t row_bytes, void* stream);

/* One rank's share of alltoall(v): rank `rank` pulls its n segments from the peers' input
 * buffers.  send_displ_bytes[r] = byte offset, inside rank r's input, of the segment
 * addressed to `rank`; recv_bytes[r] = its length.  Segments land back to back in out. */
int mccl_alltoallv_pull(const void* const* in, int n, void* out, const size_t* send_displ_bytes,
                        const size_t* recv_bytes, void* stream);

/* pack: dst = src[0] | src[1] | ... (src/gpu/dpcpp_ccl.cpp:1505-1515);
 * unpack: the inverse scatter (src/gpu/dpcpp_ccl.cpp:1528-1538). */
int mccl_pack(const void* const* src, const size_t* bytes, int n, void* dst, void* stream);
int mccl_unpack(const void* src, void* const* dst, const size_t* bytes, int n, void* stream);

/*
 * The callers' steps either side of the MoE all_to_all_single (no counterpart in the reference's
 * sources; its users build the send buffer with a row gather and undo it with a second
 * all_to_all plus a weighted sum).
 *
 * mccl_gather_rows: dst row j = src row row_index[j], j < nrows (the token permute).  row_index
 * is a DEVICE array of int64; rows whose index is outside [0, src_rows) are left untouched.
 *
 * mccl_moe_dispatch_n: the permute fused into the alltoallv copy, for all n ranks at once.
 * row_index[r] (device, sum_d S[r][d] entries) is rank r's send order: source rows of hidden[r]
 * grouped by destination, S[r][d] rows for destination d.  Rank d's output segment r receives
 * them directly; the permuted send buffer is never materialised (one read and one write per
 * routed row instead of two).
 *
 * mccl_moe_combine: y[t][c] = sum_k weights[t*topk+k] * x[src_rank[t*topk+k]][src_row[t*topk+k]][c]
 * for t < tokens, c < hidden_elems: the return all_to_all fused with the weighted sum over each
 * token's top-k copies.  src_rank (int32), src_row (int64) and weights (fp32) are DEVICE arrays.
 * fp32 chain from +0 in ascending k, each product rounded before it is added, one rounding to
 * the storage type on store; bf16 / f16 / f32; rows must be a multiple of 16 bytes.  Entries
 * with rank or row out of range contribute nothing.
 */
/*
 * mccl_route_counts: counts[e] = number of i < npairs with expert_ids[i] == e, for e < n_experts
 * (ids outside [0, n_experts) are ignored).  expert_ids (int32) and counts (int64, n_experts
 * entries) are DEVICE arrays.  The counts summed per destination rank are the inputSplitSizes of
 * the dispatch all_to_all_single (src/gpu/dpcpp_ccl.cpp:1436-1445); computing them on the device
 * keeps the routing decision there until the one copy of n_experts numbers the host needs.
 * workspace: n_experts 32-bit counters of device memory, 4-byte aligned, used as scratch (cleared by
 * the call, left zero).  1 <= n_experts <= MCCL_ROUTE_MAX_EXPERTS.
 */
#define MCCL_ROUTE_MAX_EXPERTS 4096
int mccl_route_counts(const int32_t* expert_ids, size_t npairs, int n_experts, void* workspace, int64_t* counts,
                      void* stream);

/*
 * mccl_route_counts without a workspace argument and without any allocation.  No counterpart in
 * the reference: it is for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid it.  The counters live in an array the
 * library holds on every GPU it runs on (MCCL_ROUTE_MAX_EXPERTS x 4 bytes = 16 KiB per GPU, until
 * the process ends); more experts than that are refused with MCCL_ERR_INVALID_ARG.  All calls on
 * one GPU share that array: calls that overlap on one GPU (different streams, different threads)
 * race and must be serialised by the caller.  Same results as mccl_route_counts.
 */
int mccl_route_counts_noalloc(const int32_t* expert_ids, size_t npairs, int n_experts, int64_t* counts,
                              void* stream);

int mccl_gather_rows(const void* src, size_t src_rows, const int64_t* row_index, size_t nrows,
                     size_t row_bytes, void* dst, void* stream);
int mccl_moe_dispatch_n(const void* const* hidden, const size_t* hidden_rows,
                        const int64_t* const* row_index, void* const* out, int n,
                        const int64_t* split_rows, size_t row_bytes, void* stream);
int mccl_moe_combine(const void* const* x, const size_t* x_rows, int n, const int32_t* src_rank,
                     const int64_t* src_row, const float* weights, size_t tokens, int topk,
                     size_t hidden_elems, int dtype, void* y, void* stream);

/* Launch geometry the library would use for mccl_reduce_n (for reports): returns the grid
 * size in workgroups (negative = mccl_status_t) and writes the workgroup size and the
 * dynamic-LDS reservation; count in elements. */
int mccl_query_launch(size_t count, int n, int dtype, int op, int variant, int* block_size,
                      int* lds_bytes);

/*
 * Advisory: 1 when n rank buffers of `bytes` bytes each sit at a spacing measured to cost 6-10 % of
 * bandwidth on large reductions (equal spacings of 256 MiB or more that are whole multiples of
 * 2 MiB, which is where a caching allocator puts equal tensors of 1 GiB and more: element i of
 * every rank then lands in the same DRAM channel and bank), else 0.  Needs no device.  The remedy
 * is the placement: a further 4 KiB per rank removes the effect.  The kernels run correctly either
 * way; the traffic is the same (counted), only the DRAM conflicts differ.
 */
int mccl_placement_check(const void* const* in, int n, size_t bytes);

/* Sets a knob of mccl_tune_t; value <= 0 restores the default. */
int mccl_set_tuning(int knob, long long value);
long long mccl_get_tuning(int knob);

#ifdef __cplusplus
}
#endif

#endif /* MCCL_H_ */
