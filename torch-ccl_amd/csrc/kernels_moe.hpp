// Row gather (token permute), fused MoE dispatch and weighted combine: the callers' steps either
// side of the all_to_all_single of src/gpu/dpcpp_ccl.cpp:1428-1455 (no kernel of the reference).
#pragma once

#include "kernels_common.hpp"

namespace {

// One gather segment: dst row j = src row idx[j], j < nrows.  Rows are row_bytes long.
struct GatherSeg {
  const char* src;
  const int64_t* idx;
  char* dst;
  uint32_t nrows;
  uint32_t src_rows;  // rows with idx outside [0, src_rows) are skipped (left untouched)
};

struct GatherArgs {
  GatherSeg seg[kMaxSegs];
  uint32_t chunk_prefix[kMaxSegs + 1];  // chunks = nrows * pieces_per_row
  int nseg;
  uint32_t row_bytes;
  uint32_t pieces_per_row;  // ceil(row_bytes / kCopyChunk)
  // 1: rows that are not a whole number of 2 KiB pieces (and are multiples of 16 bytes in 16-byte
  // aligned buffers): a chunk is a 2 KiB window of the segment's destination, whichever rows it
  // covers, instead of a piece of one row.  chunks = ceil(nrows * row_bytes / 2 KiB) then.
  uint32_t flat;
};

// One wavefront moves one 2 KiB piece of one row.  Chunks are numbered row-major within a
// segment and handed out in order, so the destination is written as a compact moving window;
// the sources are whole rows (contiguous row_bytes each).
__global__ __launch_bounds__(kWave) void gather_rows_kernel(const GatherArgs a) {
  const uint32_t total = a.chunk_prefix[a.nseg];
  const uint32_t ppr = a.pieces_per_row;
  const uint32_t row_bytes = a.row_bytes;
  for (uint32_t chunk = blockIdx.x; chunk < total; chunk += gridDim.x) {
    int lo = 0, hi = a.nseg;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (a.chunk_prefix[mid] <= chunk) lo = mid; else hi = mid;
    }
    const uint32_t lc = chunk - a.chunk_prefix[lo];
    if (a.flat) {
      // The destination rows of a segment are one contiguous range, so the wavefront writes 2 KiB
      // front to back whatever the row length (a 1 KiB row per wavefront would leave half the
      // lanes idle, a 2.5 KiB row three quarters of every second wavefront); every lane looks up
      // the source row of its own vectors (a chunk's lanes share a handful of index entries).
      const uint32_t vpr = row_bytes >> 4;               // vectors per row
      const uint32_t seg_vecs = a.seg[lo].nrows * vpr;   // the host keeps this below 2^32
      const u32x4* sbase = (const u32x4*)a.seg[lo].src;
      u32x4* dvec = (u32x4*)a.seg[lo].dst;
      u32x4 x[kCopyUnroll];
      bool ok[kCopyUnroll];
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u) {
        const uint32_t v = lc * (uint32_t)(kCopyChunk / 16) + threadIdx.x + (uint32_t)u * kWave;
        ok[u] = false;
        if (v < seg_vecs) {
          const uint32_t r = v / vpr;
          const int64_t sr = a.seg[lo].idx[r];
          if (sr >= 0 && sr < (int64_t)a.seg[lo].src_rows) {
            ok[u] = true;
            x[u] = sbase[(size_t)sr * vpr + (v - r * vpr)];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u)
        if (ok[u])
          __builtin_nontemporal_store(x[u], &dvec[lc * (uint32_t)(kCopyChunk / 16) + threadIdx.x + (uint32_t)u * kWave]);
      continue;
    }
    const uint32_t row = lc / ppr;
    const uint32_t piece = lc - row * ppr;
    const int64_t srow = a.seg[lo].idx[row];
    if (srow < 0 || srow >= (int64_t)a.seg[lo].src_rows) continue;
    const uint32_t off = piece * (uint32_t)kCopyChunk;
    const uint32_t left = row_bytes - off;
    const uint32_t len = left < (uint32_t)kCopyChunk ? left : (uint32_t)kCopyChunk;
    const char* src = a.seg[lo].src + (size_t)srow * row_bytes + off;
    char* dst = a.seg[lo].dst + (size_t)row * row_bytes + off;
    const uint32_t t = threadIdx.x;
    // 16-byte vectors aligned on the destination; bytes up to the first boundary and after the
    // last whole vector; the source is read at whatever alignment it has
    uint32_t head = (16u - (uint32_t)((uintptr_t)dst & 15u)) & 15u;
    if (head > len) head = len;
    if (t < head) dst[t] = src[t];
    const uint32_t body = len - head;
    const uint32_t nv = body >> 4;
    const u32x4_unaligned* sv = (const u32x4_unaligned*)(src + head);
    u32x4* dv = (u32x4*)(dst + head);
    if (nv == (uint32_t)(kCopyChunk / 16)) {
      u32x4 x[kCopyUnroll];
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u) x[u] = sv[t + u * kWave];  // rows are re-read (top-k): cacheable
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u) __builtin_nontemporal_store(x[u], &dv[t + u * kWave]);
    } else {
      for (uint32_t v = t; v < nv; v += kWave) __builtin_nontemporal_store((u32x4)sv[v], &dv[v]);
    }
    const uint32_t rem = body & 15u;
    if (t < rem) dst[head + (nv << 4) + t] = src[head + (nv << 4) + t];
  }
}

// Weighted combine: y[t][c] = sum_k w[t][k] * x[rank(t,k)][row(t,k)][c], fp32 chain from +0 in
// ascending k, every product rounded before it is added, one rounding on store.
struct CombineArgs {
  const char* x[MCCL_MAX_RANKS];
  uint32_t x_rows[MCCL_MAX_RANKS];
  const int32_t* src_rank;
  const int64_t* src_row;
  const float* w;
  char* y;
  uint32_t tokens;
  uint32_t topk;
  uint32_t row_vecs;        // 16-byte vectors per row
  uint32_t pieces_per_row;  // ceil(row_vecs / 64)
  uint32_t pieces_per_wave; // 1 KiB pieces one wavefront walks (routing entries are looked up once)
  uint32_t waves_per_row;   // ceil(pieces_per_row / pieces_per_wave)
  int n;
};

// GROUP > 0: top-k of at most GROUP (2, 4 or 8: one group of row loads covers a token), each a
// kernel of its own with its own register budget - a top-2 combine holds a quarter of the rows of
// a top-8 one and fits half as many registers, so that more wavefronts (and loads) are in flight.
// GROUP == 0: any top-k, entries in groups of 8.
template <int DT, int GROUP>
__global__ __launch_bounds__(kWave) void moe_combine_kernel(const CombineArgs a) {
  using A = float;
  constexpr int VE = vec_elems<DT>();
  constexpr bool FAST = GROUP > 0;
  constexpr int G = FAST ? GROUP : 8;  // row loads in flight per lane and piece
  const uint32_t total = a.tokens * a.waves_per_row;
  const size_t row_stride = (size_t)a.row_vecs * 16;
  if constexpr (FAST) {
    // The token's routing entries are looked up once for all pieces a wavefront walks: lane g
    // loads entry g (three loads in flight at once), and the values are broadcast into scalar
    // registers, so that everything derived from them (the peer pointer picked from the argument
    // block, the bounds checks, the row address) is scalar work and the row loads start after
    // one memory round trip instead of two.  With a grid smaller than the number of chunks a
    // wavefront walks several chunks and looks up the next chunk's entries while it streams the
    // rows of the current one.
    auto issue_routing = [&](uint32_t c, int& rk, int64_t& rw, float& wt) {
      rk = -1;
      rw = 0;
      wt = 0.0f;
      if (c < total && threadIdx.x < a.topk) {
        const size_t e = (size_t)(c / a.waves_per_row) * a.topk + threadIdx.x;
        rk = a.src_rank[e];
        rw = a.src_row[e];
        wt = a.w[e];
      }
    };
    int my_rank;
    int64_t my_row;
    float my_w;
    issue_routing(blockIdx.x, my_rank, my_row, my_w);
    for (uint32_t chunk = blockIdx.x; chunk < total; chunk += gridDim.x) {
      const uint32_t tok = chunk / a.waves_per_row;
      const uint32_t part = chunk - tok * a.waves_per_row;
      const uint32_t p0 = part * a.pieces_per_wave;
      const uint32_t p1 = (p0 + a.pieces_per_wave < a.pieces_per_row) ? p0 + a.pieces_per_wave : a.pieces_per_row;
      const u32x4* src[G];
      bool ok[G];
      float wk[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int rk = __builtin_amdgcn_readlane(my_rank, g);
        const uint32_t row_lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)my_row, g);
        const uint32_t row_hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)my_row >> 32), g);
        const int64_t rw = (int64_t)(((uint64_t)row_hi << 32) | row_lo);
        wk[g] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), g));
        const bool rank_ok = rk >= 0 && rk < a.n;
        const int r = rank_ok ? rk : 0;
        ok[g] = rank_ok && rw >= 0 && rw < (int64_t)a.x_rows[r];
        src[g] = (const u32x4*)(a.x[r] + (ok[g] ? (size_t)rw : 0) * row_stride);
      }
      // Double-buffered walk over the pieces: the row loads of piece i+1 are in flight while piece i
      // is weighted, summed and stored, so a wavefront never sits without memory requests.
      auto load_piece = [&](uint32_t piece, VecU<DT>(&x)[G]) {
        const uint32_t v = piece * kWave + threadIdx.x;
        const bool live = v < a.row_vecs;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          x[g].v = (u32x4){0u, 0u, 0u, 0u};
          if (ok[g] && live) x[g].v = __builtin_nontemporal_load(src[g] + v);
        }
      };
      auto finish_piece = [&](uint32_t piece, const VecU<DT>(&x)[G]) {
        const uint32_t v = piece * kWave + threadIdx.x;
        A acc[VE];
#pragma unroll
        for (int e = 0; e < VE; ++e) acc[e] = 0.0f;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          if (ok[g]) {
#pragma unroll
            for (int e = 0; e < VE; ++e) {
              const float prod = wk[g] * Elem<DT>::load(x[g].e[e]);
              acc[e] = acc[e] + prod;
            }
          }
        }
        if (v < a.row_vecs) {
          VecU<DT> r;
#pragma unroll
          for (int e = 0; e < VE; ++e) r.e[e] = Elem<DT>::store(acc[e]);
          __builtin_nontemporal_store(r.v, (u32x4*)(a.y + (size_t)tok * row_stride) + v);
        }
      };
      VecU<DT> xa[G], xb[G];
      load_piece(p0, xa);
      int next_rank;
      int64_t next_row;
      float next_w;
      issue_routing(chunk + gridDim.x, next_rank, next_row, next_w);  // behind this chunk's first rows
      for (uint32_t piece = p0; piece < p1; piece += 2) {
        if (piece + 1 < p1) load_piece(piece + 1, xb);
        finish_piece(piece, xa);
        if (piece + 1 < p1) {
          if (piece + 2 < p1) load_piece(piece + 2, xa);
          finish_piece(piece + 1, xb);
        }
      }
      my_rank = next_rank;
      my_row = next_row;
      my_w = next_w;
    }
  } else {
    for (uint32_t chunk = blockIdx.x; chunk < total; chunk += gridDim.x) {
      const uint32_t tok = chunk / a.waves_per_row;
      const uint32_t part = chunk - tok * a.waves_per_row;
      const uint32_t p0 = part * a.pieces_per_wave;
      const uint32_t p1 = (p0 + a.pieces_per_wave < a.pieces_per_row) ? p0 + a.pieces_per_wave : a.pieces_per_row;
      const size_t e0 = (size_t)tok * a.topk;
      // general top-k: groups of G entries per piece
      for (uint32_t piece = p0; piece < p1; ++piece) {
        const uint32_t v = piece * kWave + threadIdx.x;
        const bool live = v < a.row_vecs;
        A acc[VE];
#pragma unroll
        for (int e = 0; e < VE; ++e) acc[e] = 0.0f;
        for (uint32_t kb = 0; kb < a.topk; kb += G) {
          VecU<DT> x[G];
          float wk[G];
          bool ok[G];
#pragma unroll
          for (int g = 0; g < G; ++g) {
            ok[g] = false;
            wk[g] = 0.0f;
            x[g].v = (u32x4){0u, 0u, 0u, 0u};
            if (kb + g < a.topk) {
              const int r = a.src_rank[e0 + kb + g];
              const int64_t row = a.src_row[e0 + kb + g];
              if (r >= 0 && r < a.n && row >= 0 && row < (int64_t)a.x_rows[r]) {
                ok[g] = true;
                wk[g] = a.w[e0 + kb + g];
                if (live) x[g].v = __builtin_nontemporal_load((const u32x4*)(a.x[r] + (size_t)row * row_stride) + v);
              }
            }
          }
#pragma unroll
          for (int g = 0; g < G; ++g) {
            if (ok[g]) {
#pragma unroll
              for (int e = 0; e < VE; ++e) {
                const float prod = wk[g] * Elem<DT>::load(x[g].e[e]);
                acc[e] = acc[e] + prod;
              }
            }
          }
        }
        if (live) {
          VecU<DT> r;
#pragma unroll
          for (int e = 0; e < VE; ++e) r.e[e] = Elem<DT>::store(acc[e]);
          __builtin_nontemporal_store(r.v, (u32x4*)(a.y + (size_t)tok * row_stride) + v);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Routing counts: how many (token, expert) pairs go to each expert.  The caller's step before the
// all_to_all_single of src/gpu/dpcpp_ccl.cpp:1371-1466, whose inputSplitSizes are these counts
// summed per destination rank.  Two kernels: a histogram into 32-bit counters (a workgroup counts
// its share in LDS first, so the device atomics are one per expert and workgroup, not one per
// pair), and a finish that widens the counters into the caller's int64 array and leaves them
// zero for the next call.
// ------------------------------------------------------------------------------------------
constexpr int kRouteBlock = 256;
constexpr int kRouteMaxExperts = 4096;  // LDS histogram: 16 KiB

__global__ __launch_bounds__(kRouteBlock) void route_count_kernel(const int32_t* ids, uint64_t npairs, uint32_t n_experts,
                                                                  uint32_t* counters) {
  __shared__ uint32_t hist[kRouteMaxExperts];
  for (uint32_t e = threadIdx.x; e < n_experts; e += kRouteBlock) hist[e] = 0;
  __syncthreads();
  const uint64_t stride = (uint64_t)gridDim.x * kRouteBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kRouteBlock + threadIdx.x; i < npairs; i += stride) {
    const uint32_t e = (uint32_t)ids[i];  // negative ids become large and are ignored like any id out of range
    if (e < n_experts) atomicAdd(&hist[e], 1u);
  }
  __syncthreads();
  for (uint32_t e = threadIdx.x; e < n_experts; e += kRouteBlock) {
    const uint32_t c = hist[e];
    if (c) atomicAdd(&counters[e], c);
  }
}

__global__ __launch_bounds__(kRouteBlock) void route_finish_kernel(uint32_t* counters, uint32_t n_experts, int64_t* counts) {
  for (uint32_t e = blockIdx.x * kRouteBlock + threadIdx.x; e < n_experts; e += gridDim.x * kRouteBlock) {
    counts[e] = (int64_t)counters[e];
    counters[e] = 0;
  }
}

// Zeroes a workspace the caller brought (a kernel, not a memset node: callers may capture the call).
__global__ __launch_bounds__(kRouteBlock) void route_clear_kernel(uint32_t* counters, uint32_t n_experts) {
  for (uint32_t e = blockIdx.x * kRouteBlock + threadIdx.x; e < n_experts; e += gridDim.x * kRouteBlock) counters[e] = 0;
}

}  // namespace
