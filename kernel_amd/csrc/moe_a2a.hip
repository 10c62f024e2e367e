// MoE all-to-all dispatch / expert stub / combine for one MI355X (gfx950, wave64).
//
// The W destination ranks of the reference's all-to-all (all2all/reference.py:68-234) are
// partitions of one compact expert-major buffer, so an "exchange" is only the choice of a
// destination row.  The dispatch/combine path is HBM-bound integer/byte work: no MFMA, 16-byte
// vector loads and stores, LDS for counters and index tiles, ballot/popcount for ranks.  The
// expert layer that a real model runs between the two (the reference has a scalar stub there) is
// the one matrix-core kernel family: a grouped GEMM over the dispatched segments.
//
// Kernels
//   route_*            histogram, exclusive scan, stable permutation, meta rows
//   dispatch_rows      token row -> K destination rows (read once, store K times)
//   route_dispatch     both of the above in one launch for small worlds
//   dispatch_fp8       same copy with e4m3fn quantisation per 128 columns
//   stub_*             expert stand-in, one factor per row
//   combine / stub_combine   gather K rows per token, weighted sum
//   expert_gemm        y[rows of e] = x[rows of e] * W_e^T, 128 x 128 tiles (short segments)
//   expert_gemm_wide   the same on 256 x 256 tiles, software-pipelined; 16-bit or fp8 rows
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <atomic>

#include "moe_a2a.h"

namespace {

constexpr int kWave = 64;
constexpr int kRouteThreads = 1024;
constexpr int kRouteWaves = kRouteThreads / kWave;
constexpr int kRouteTilesMaxRows = 16 * kRouteThreads;  // one-launch routing up to here
constexpr int kRowMaxThreads = 512;
constexpr int kFusedIdBits = 13;
constexpr int kFusedMaxRows = 1 << kFusedIdBits;  // route_dispatch packs (expert, entry id) into one key
constexpr int kFusedMaxThreads = 1024;
#ifndef MOE_A2A_FUSED_TABLE_READS
#define MOE_A2A_FUSED_TABLE_READS (1ll << 20)
#endif
constexpr long long kFusedMaxTableReads = MOE_A2A_FUSED_TABLE_READS;  // entries read by all workgroups together

enum KernelId {
  KID_ROUTE_TILES = 0,
  KID_ROUTE_HIST,
  KID_ROUTE_SCAN,
  KID_ROUTE_RANK,
  KID_DISPATCH,
  KID_ROUTE_DISPATCH,
  KID_ROUTE_DISPATCH_TILE,
  KID_DISPATCH_FP8,
  KID_STUB,
  KID_STUB_FP8,
  KID_COMBINE,
  KID_STUB_COMBINE,
  KID_EXPERT_GEMM,
  KID_EXPERT_GEMM_WIDE,
  KID_EXPERT_GEMM_SKINNY,
  KID_EXPERT_GEMM_F8,
  KID_EXPERT_GEMM_MX,
  KID_COUNT
};
const char* const kKernelNames[KID_COUNT] = {
    "route_tiles", "route_hist", "route_scan", "route_rank",   "dispatch_rows", "route_dispatch", "route_dispatch_tile",
    "dispatch_fp8", "stub_rows",  "stub_fp8",   "combine_rows", "stub_combine", "expert_gemm",
    "expert_gemm_wide", "expert_gemm_skinny", "expert_gemm_f8", "expert_gemm_mx"};

// ---------------------------------------------------------------------------------------
// element helpers: two 16-bit values per dword, element 0 in the low half
// ---------------------------------------------------------------------------------------
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

struct Bf16 {
  static __device__ __forceinline__ float lo(uint32_t u) { return __uint_as_float(u << 16); }
  static __device__ __forceinline__ float hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
  // round-to-nearest-even; one v_cvt_pk_bf16_f32 on gfx950
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
};

struct F16 {
  static __device__ __forceinline__ float lo(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    uint32_t l = __builtin_bit_cast(uint16_t, (_Float16)a);
    uint32_t h = __builtin_bit_cast(uint16_t, (_Float16)b);
    return l | (h << 16);
  }
};

// value of x after a round trip through the 16-bit type E
template <class E>
__device__ __forceinline__ void round_pair(float& a, float& b) {
  uint32_t u = E::pack(a, b);
  a = E::lo(u);
  b = E::hi(u);
}

__device__ __forceinline__ void unpack8(const uint4& v, uint32_t (&d)[4]) {
  d[0] = v.x;
  d[1] = v.y;
  d[2] = v.z;
  d[3] = v.w;
}

__device__ __forceinline__ float stub_factor(int e, int stub_kind, int num_experts, int experts_per_rank) {
  if (stub_kind == MOE_A2A_STUB_OWNER_RANK) return (float)(1 + e / experts_per_rank);
  return (float)((double)(1 + e) / (double)num_experts);
}

// ---------------------------------------------------------------------------------------
// routing
// ---------------------------------------------------------------------------------------
struct RouteArgs {
  const int32_t* indices;
  const int32_t* rank_start;  // [W+1] or null
  int src_rank;
  int T, K, E, W, R;
  int nbits;  // bits needed for an expert id
  int pad;    // 0: compact rows; > 0: rows of expert e start at e * pad (the reference's max_recv)
  int32_t* counts;
  int32_t* offsets;
  int32_t* slot_of_entry;
  int32_t* src_of_slot;
  int32_t* meta;
  int32_t* status;
};

// expert id forced into [0, E); an id outside raises the caller's status flag
__device__ __forceinline__ int clamp_expert(const RouteArgs& a, int e) {
  if (e < 0 || e >= a.E) {
    if (a.status) *a.status = 1;  // vector store; the value is the same from every lane
    e = e < 0 ? 0 : a.E - 1;
  }
  return e;
}

__device__ __forceinline__ int load_expert(const RouteArgs& a, int i, bool valid) {
  return clamp_expert(a, valid ? a.indices[i] : 0);
}

// Lanes holding the same expert id find each other with one ballot per id bit.
// rank = number of lower lanes with the same id, cnt = size of the group.
__device__ __forceinline__ void wave_match(int e, bool valid, int nbits, int& rank, int& cnt) {
  unsigned long long m = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    bool bit = (e >> b) & 1;
    unsigned long long bal = __ballot(valid && bit);
    m &= bit ? bal : ~bal;
  }
  unsigned long long lt = (1ull << (threadIdx.x & (kWave - 1))) - 1ull;
  rank = __popcll(m & lt);
  cnt = __popcll(m);
}

__device__ __forceinline__ int wave_inclusive_scan(int v) {
  int lane = threadIdx.x & (kWave - 1);
  for (int d = 1; d < kWave; d <<= 1) {
    int n = __shfl_up(v, d, kWave);
    if (lane >= d) v += n;
  }
  return v;
}

// exclusive scan over the workgroup (blockDim.x a multiple of 64, at most 1024);
// tmp holds blockDim.x/64 + 1 ints
__device__ __forceinline__ int block_exclusive_scan(int v, int* tmp, int& total) {
  int lane = threadIdx.x & (kWave - 1);
  int w = threadIdx.x / kWave;
  int nw = blockDim.x / kWave;
  int incl = wave_inclusive_scan(v);
  if (lane == kWave - 1) tmp[w] = incl;
  __syncthreads();
  if (w == 0) {
    int x = lane < nw ? tmp[lane] : 0;
    int xi = wave_inclusive_scan(x);
    if (lane < nw) tmp[lane] = xi - x;
    if (lane == nw - 1) tmp[nw] = xi;
  }
  __syncthreads();
  int r = incl - v + tmp[w];
  total = tmp[nw];
  __syncthreads();
  return r;
}

// source rank and token-within-rank of global token t; starts is the LDS copy of rank_start
__device__ __forceinline__ void locate_token(const int* starts, int W, int src_rank, bool have_starts, int t,
                                             int& rank, int& local) {
  if (!have_starts) {
    rank = src_rank;
    local = t;
    return;
  }
  int lo = 0, hi = W;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (starts[mid] <= t) lo = mid; else hi = mid;
  }
  rank = lo;
  local = t - starts[lo];
}

// Row of the entry that is the j-th of expert e, where its compact slot is first_of_e + j.
// Padded layout: a segment holds `pad` rows; an entry beyond that is folded onto the last
// row of its segment and reported through the status flag (2) -- no access leaves the buffer.
__device__ __forceinline__ int row_of(const RouteArgs& a, int e, int slot, int first_of_e) {
  if (a.pad == 0) return slot;
  int j = slot - first_of_e;
  if (j >= a.pad) {
    if (a.status) *a.status = 2;
    j = a.pad - 1;
  }
  return e * a.pad + j;
}

__device__ __forceinline__ void emit_entry(const RouteArgs& a, const int* starts, int i, int e, int slot_compact,
                                           int first_of_e) {
  const int slot = row_of(a, e, slot_compact, first_of_e);
  a.slot_of_entry[i] = slot;
  a.src_of_slot[slot] = i;
  int t = i / a.K;
  int k = i - t * a.K;
  int sr, tl;
  locate_token(starts, a.W, a.src_rank, a.rank_start != nullptr, t, sr, tl);
  int32_t* m = a.meta + (size_t)slot * MOE_A2A_META_DIM;
  m[0] = e;
  m[1] = sr;
  m[2] = tl;
  m[3] = k;
  m[4] = 0;
}

// LDS layout shared by the routing kernels:
//   wcnt[kRouteWaves * E]   per-wave rows per expert of the current tile
//   base[E]                 running first slot per expert (single-workgroup kernel)
//   tmp[kRouteWaves + 1]    scan scratch
//   starts[W + 1]           copy of rank_start
__device__ __forceinline__ void load_starts(const RouteArgs& a, int* starts) {
  if (a.rank_start)
    for (int j = threadIdx.x; j <= a.W; j += blockDim.x) starts[j] = a.rank_start[j];
}

// per-wave counts of one tile into wcnt (zeroed first); returns this thread's in-wave rank
__device__ __forceinline__ int tile_wave_counts(int* wcnt, int E, int e, bool valid, int nbits) {
  for (int j = threadIdx.x; j < kRouteWaves * E; j += kRouteThreads) wcnt[j] = 0;
  __syncthreads();
  int rank, cnt;
  wave_match(e, valid, nbits, rank, cnt);
  if (valid && rank == 0) wcnt[(threadIdx.x / kWave) * E + e] = cnt;
  __syncthreads();
  return rank;
}

// Routing in ONE launch for up to kRouteTilesMaxRows entries.  A tile is kRouteThreads
// consecutive entries and has its own workgroup.  Every workgroup counts, in LDS, the rows of
// each expert in the tiles before its own and in the rest of the table (it reads the whole
// routing table: R * 4 bytes per workgroup, which is what replaces a histogram launch, a scan
// launch and the round trips between them), scans the totals into offsets, ranks its own
// entries stably (wave match + per-wave counts) and writes their slots and meta rows.
__global__ __launch_bounds__(kRouteThreads) void route_tiles_kernel(RouteArgs a) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  int* before = wcnt + kRouteWaves * a.E;
  int* rest = before + a.E;
  int* tmp = rest + a.E;
  int* starts = tmp + kRouteWaves + 1;
  const int tid = threadIdx.x;
  const int tile_lo = blockIdx.x * kRouteThreads;
  load_starts(a, starts);
  for (int j = tid; j < 2 * a.E; j += kRouteThreads) before[j] = 0;  // before[] and rest[] are adjacent
  __syncthreads();
#pragma unroll 4
  for (int i = tid; i < a.R; i += kRouteThreads) {
    int e = load_expert(a, i, true);
    atomicAdd(i < tile_lo ? &before[e] : &rest[e], 1);  // LDS counters; a sum does not depend on order
  }
  const int i = tile_lo + tid;
  const bool valid = i < a.R;
  const int e = load_expert(a, i, valid);
  const int rank = tile_wave_counts(wcnt, a.E, e, valid, a.nbits);  // its barriers also cover the counters
  const int all = tid < a.E ? before[tid] + rest[tid] : 0;
  int total;
  const int excl = block_exclusive_scan(all, tmp, total);
  if (blockIdx.x == 0) {
    if (tid < a.E) {
      a.counts[tid] = all;
      a.offsets[tid] = excl;
    }
    if (tid == 0) a.offsets[a.E] = total;
  }
  if (tid < a.E) {
    int run = excl + before[tid];
    for (int w = 0; w < kRouteWaves; ++w) {
      int c = wcnt[w * a.E + tid];
      wcnt[w * a.E + tid] = run;
      run += c;
    }
    rest[tid] = excl;  // rest[] is not needed any more: it now holds the first slot of each expert
  }
  __syncthreads();
  if (valid) emit_entry(a, starts, i, e, wcnt[(tid / kWave) * a.E + e] + rank, rest[e]);
}

// Routing in two or three launches for larger tables.
// step 1: rows per (tile, expert), tile-major so that lane e reads and writes coalesced.
__global__ __launch_bounds__(kRouteThreads) void route_hist_kernel(RouteArgs a, int32_t* tile_hist) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  const int tid = threadIdx.x;
  int i = blockIdx.x * kRouteThreads + tid;
  bool valid = i < a.R;
  int e = load_expert(a, i, valid);
  tile_wave_counts(wcnt, a.E, e, valid, a.nbits);
  if (tid < a.E) {
    int s = 0;
    for (int w = 0; w < kRouteWaves; ++w) s += wcnt[w * a.E + tid];
    tile_hist[(size_t)blockIdx.x * a.E + tid] = s;
  }
}

// step 2: every count becomes the number of rows of its expert in earlier tiles, and the
// column totals are scanned into counts and offsets.  One workgroup; floor(1024 / E) threads
// share a column, each walking a contiguous range of tiles eight loads at a time.
__global__ __launch_bounds__(kRouteThreads) void route_scan_kernel(int32_t* tile_hist, int E, int ntiles,
                                                                    int32_t* counts, int32_t* offsets) {
  __shared__ int part_sum[kRouteThreads];
  __shared__ int tmp[kRouteWaves + 1];
  const int tid = threadIdx.x;
  const int parts = kRouteThreads / E;  // >= 1 because E <= 1024
  const int p = tid / E, e = tid - p * E;
  const bool live = p < parts;
  const int span = (ntiles + parts - 1) / parts;
  const int lo = min(p * span, ntiles), hi = live ? min(lo + span, ntiles) : lo;
  int sum = 0;
  for (int b0 = lo; b0 < hi; b0 += 8) {
    int c[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) c[u] = b0 + u < hi ? tile_hist[(size_t)(b0 + u) * E + e] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += c[u];
  }
  part_sum[tid] = live ? sum : 0;
  __syncthreads();
  int run = 0, column = 0;
  if (live)
    for (int q = 0; q < parts; ++q) {
      int v = part_sum[q * E + e];
      if (q < p) run += v;
      column += v;
    }
  for (int b0 = lo; b0 < hi; b0 += 8) {
    int c[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) c[u] = b0 + u < hi ? tile_hist[(size_t)(b0 + u) * E + e] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (b0 + u < hi) tile_hist[(size_t)(b0 + u) * E + e] = run;
      run += c[u];
    }
  }
  const bool first = live && p == 0;  // tid == e
  int total;
  int excl = block_exclusive_scan(first ? column : 0, tmp, total);
  if (first) {
    counts[e] = column;
    offsets[e] = excl;
  }
  if (tid == 0) offsets[E] = total;
}

// step 3: stable rank inside the tile + first slot of (expert, tile) from steps 1 and 2.
__global__ __launch_bounds__(kRouteThreads) void route_rank_kernel(RouteArgs a, const int32_t* tile_hist) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  int* starts = wcnt + kRouteWaves * a.E;
  const int tid = threadIdx.x;
  load_starts(a, starts);
  int i = blockIdx.x * kRouteThreads + tid;
  bool valid = i < a.R;
  int e = load_expert(a, i, valid);
  int rank = tile_wave_counts(wcnt, a.E, e, valid, a.nbits);
  if (tid < a.E) {
    int run = a.offsets[tid] + tile_hist[(size_t)blockIdx.x * a.E + tid];
    for (int w = 0; w < kRouteWaves; ++w) {
      int c = wcnt[w * a.E + tid];
      wcnt[w * a.E + tid] = run;
      run += c;
    }
  }
  __syncthreads();
  if (valid) emit_entry(a, starts, i, e, wcnt[(tid / kWave) * a.E + e] + rank, a.pad ? a.offsets[e] : 0);
}

// steps 2 and 3 in one launch for up to kRouteFoldMaxTiles tiles: every workgroup sums the columns
// of the raw (tile, expert) counts for itself -- all tiles for the segment starts, the tiles before
// its own for its base -- instead of waiting for a one-workgroup scan launch.  The matrix is a few
// tens of KB and stays in L2; floor(1024 / E) threads share a column as in the scan kernel.
constexpr int kRouteFoldMaxTiles = 256;
__global__ __launch_bounds__(kRouteThreads) void route_rank_fold_kernel(RouteArgs a, const int32_t* tile_hist,
                                                                         int ntiles) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  int* starts = wcnt + kRouteWaves * a.E;
  __shared__ int part_all[kRouteThreads];
  __shared__ int part_before[kRouteThreads];
  __shared__ int s_first[MOE_A2A_MAX_EXPERTS];  // first slot of each expert
  __shared__ int tmp[kRouteWaves + 1];
  const int tid = threadIdx.x;
  load_starts(a, starts);
  const int i = blockIdx.x * kRouteThreads + tid;
  const bool valid = i < a.R;
  const int e = load_expert(a, i, valid);
  const int parts = kRouteThreads / a.E;  // >= 1 because E <= 1024
  const int p = tid / a.E, col = tid - p * a.E;
  const bool live = p < parts;
  const int span = (ntiles + parts - 1) / parts;
  const int lo = min(p * span, ntiles), hi = live ? min(lo + span, ntiles) : lo;
  int all = 0, before = 0;
  for (int b0 = lo; b0 < hi; b0 += 8) {
    int c[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) c[u] = b0 + u < hi ? tile_hist[(size_t)(b0 + u) * a.E + col] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      all += c[u];
      before += b0 + u < (int)blockIdx.x ? c[u] : 0;
    }
  }
  part_all[tid] = live ? all : 0;
  part_before[tid] = live ? before : 0;
  const int rank = tile_wave_counts(wcnt, a.E, e, valid, a.nbits);  // its barriers publish the partial sums
  int column = 0, bef = 0;
  if (tid < a.E)
    for (int q = 0; q < parts; ++q) {
      column += part_all[q * a.E + tid];
      bef += part_before[q * a.E + tid];
    }
  int total;
  const int excl = block_exclusive_scan(tid < a.E ? column : 0, tmp, total);
  if (tid < a.E) {
    s_first[tid] = excl;
    if (blockIdx.x == 0) {
      a.counts[tid] = column;
      a.offsets[tid] = excl;
    }
    int run = excl + bef;
    for (int w = 0; w < kRouteWaves; ++w) {
      int c = wcnt[w * a.E + tid];
      wcnt[w * a.E + tid] = run;
      run += c;
    }
  }
  if (blockIdx.x == 0 && tid == 0) a.offsets[a.E] = total;
  __syncthreads();
  if (valid) emit_entry(a, starts, i, e, wcnt[(tid / kWave) * a.E + e] + rank, a.pad ? s_first[e] : 0);
}

// ---------------------------------------------------------------------------------------
// row kernels: geometry and memory helpers
// ---------------------------------------------------------------------------------------
// A row of nvec 16-byte vectors is cut into nsplit equal column ranges of `per` vectors; one
// workgroup of round_up(per, 64) <= 512 threads moves one range, one vector per lane, so no
// lane idles when nvec is a multiple of 64 (H = 7168 -> two workgroups of 448 lanes).
//
// Cache policy of the row traffic (rows are produced by one kernel and consumed by a later
// one, never re-read by the kernel that touches them):
//   STREAM = 0  working set fits the caches: plain loads; stores write through (sc0 sc1) so
//               the lines leave L2 while the kernel runs instead of in its end-of-kernel
//               write-back;
//   STREAM = 1  working set far beyond the 256 MB Infinity Cache: non-temporal loads and
//               stores, which keep streamed rows from evicting each other.
// Scattered row stores of the dispatch always write through.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#ifndef MOE_A2A_THROUGH_POLICY
#define MOE_A2A_THROUGH_POLICY 2  // tuning aid: 0 plain store, 1 non-temporal, 2 write-through
#endif
__device__ __forceinline__ void store_through(uint4* p, const uint4& v) {
#if MOE_A2A_THROUGH_POLICY == 2
  u32x4_t t = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(t) : "memory");
#elif MOE_A2A_THROUGH_POLICY == 1
  u32x4_t t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(p));
#else
  *p = v;
#endif
}

template <int STREAM>
__device__ __forceinline__ void store_row(uint4* p, const uint4& v) {
  if (STREAM) {
    u32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(p));
  } else {
    store_through(p, v);
  }
}

template <int STREAM>
__device__ __forceinline__ uint4 load_row(const uint4* p) {
  if (STREAM) {
    u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
  }
  return *p;
}

struct RowCut {
  int t;        // row handled by this workgroup
  int c;        // vector index inside the row
  bool active;  // lane has a vector
};

__device__ __forceinline__ RowCut row_cut(int nvec, int per, int nsplit) {
  RowCut r;
  r.t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - r.t * nsplit;
  r.c = cs * per + threadIdx.x;
  r.active = (int)threadIdx.x < per && r.c < nvec;
  return r;
}

// ---------------------------------------------------------------------------------------
// dispatch: token row -> K rows
// ---------------------------------------------------------------------------------------
template <int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void dispatch_rows_kernel(const uint4* __restrict__ x,
                                                                        const int32_t* __restrict__ slot_of_entry,
                                                                        uint4* __restrict__ disp, int K, int nvec,
                                                                        int per, int nsplit) {
  const RowCut r = row_cut(nvec, per, nsplit);
  if (!r.active) return;
  const uint4 v = load_row<STREAM>(x + (size_t)r.t * nvec + r.c);
  const int32_t* sl = slot_of_entry + (size_t)r.t * K;
  for (int k = 0; k < K; ++k) store_through(disp + (size_t)sl[k] * nvec + r.c, v);
}

// Routing folded into the dispatch for R <= kFusedMaxRows.  The slot of entry i is the number
// of entries whose (expert, entry id) pair is smaller, so a workgroup can find the K slots of
// its own token by comparing every entry of the table against K keys: each lane holds EPT
// entries (all loaded in one go), a ballot + popcount per (entry, key) counts a wave's share,
// and LDS counters add the waves up.  The row load is issued first and is in flight meanwhile.
// Column split 0 of each token also writes the index arrays and meta rows; workgroup 0
// writes counts and offsets.
// EPT table entries per thread: 4 (small tables), 8, 16, 24 or 32; PAD: padded layout; VPL row
// vectors per lane: 2 for long rows (half as many waves to launch: 7.4 against 7.6 us at 256 tokens
// of 7168 columns), 1 otherwise (two were slower at 2048 columns, four at both).
template <int EPT, bool PAD, int VPL>
__global__ __launch_bounds__(kFusedMaxThreads) void route_dispatch_kernel(RouteArgs a, const uint4* __restrict__ x,
                                                                         uint4* __restrict__ disp, int nvec,
                                                                         int per, int nsplit) {
  __shared__ int s_part[kFusedMaxThreads / kWave][MOE_A2A_MAX_TOPK];  // per wave: smaller keys it holds, per key
  __shared__ int s_hist[MOE_A2A_MAX_EXPERTS];
  __shared__ int s_tmp[kFusedMaxThreads / kWave + 1];
  __shared__ int s_starts[MOE_A2A_MAX_WORLD + 1];
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int lane = tid & (kWave - 1);

  if (blockIdx.x == 0) {  // counts + offsets
    for (int j = tid; j < a.E; j += nthreads) s_hist[j] = 0;
    __syncthreads();
    for (int i = tid; i < a.R; i += nthreads) atomicAdd(&s_hist[load_expert(a, i, true)], 1);
    __syncthreads();
    const int span = (a.E + nthreads - 1) / nthreads;
    int lo = min(tid * span, a.E), hi = min(lo + span, a.E);
    int s = 0;
    for (int j = lo; j < hi; ++j) s += s_hist[j];
    int total;
    int run = block_exclusive_scan(s, s_tmp, total);
    for (int j = lo; j < hi; ++j) {
      int c = s_hist[j];
      a.counts[j] = c;
      a.offsets[j] = run;
      run += c;
    }
    if (tid == 0) a.offsets[a.E] = total;
    return;
  }

  const int t = (blockIdx.x - 1) / nsplit;
  const int cs = (blockIdx.x - 1) - t * nsplit;
  int cv[VPL];
  bool active[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    cv[j] = (cs * VPL + j) * per + tid;
    active[j] = tid < per && cv[j] < nvec;
  }
  // Raw expert ids of this lane's entries.  EPT == 4: entries 4 tid .. 4 tid + 3, indices clamped
  // into the table instead of branching, like every load below: with unconditional loads the
  // compiler can wait for the early ones while the later ones stay in flight.  Larger tables:
  // EPT / 4 vectors of four entries, vector c at entry 4 (c nthreads + tid), all issued at once
  // (one table round trip, not one per chunk); a vector that would cross the end of the table is
  // moved back to end at the last entry, and the entries it then shares with its neighbour are
  // masked out below.
  int raw[EPT];
  int pos[EPT / 4];
  if (EPT == 4) {
    pos[0] = tid * 4;
#pragma unroll
    for (int m = 0; m < 4; ++m) raw[m] = a.indices[min(pos[0] + m, a.R - 1)];
  } else {
    typedef int i32x4_t __attribute__((ext_vector_type(4), aligned(4)));  // a moved vector is only dword-aligned
#pragma unroll
    for (int ch = 0; ch < EPT / 4; ++ch) {
      pos[ch] = min((ch * nthreads + tid) * 4, a.R - 4);  // R >= 4 on this path
      const i32x4_t q = *reinterpret_cast<const i32x4_t*>(a.indices + pos[ch]);
#pragma unroll
      for (int m = 0; m < 4; ++m) raw[4 * ch + m] = q[m];
    }
  }

  // Every load goes out before the first use of a loaded value: the table, the token's own expert ids
  // (lane k of every wave holds entry k), the rank boundaries, and last the row itself, so that
  // waiting for the indices (memory operations complete in order) leaves the row in flight while
  // the slots are worked out.
  const int own = a.indices[t * a.K + min(lane, a.K - 1)];
  const bool want_starts = cs == 0 && a.rank_start != nullptr;
  const int32_t* sp = a.rank_start ? a.rank_start : a.indices;  // any readable address when unused
  const int st0 = sp[a.rank_start ? min(tid, a.W) : 0];
  const int st1 = sp[a.rank_start ? min(tid + nthreads, a.W) : 0];
  __builtin_amdgcn_sched_barrier(0);  // keep the row load behind the index loads
  uint4 v[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) v[j] = x[(size_t)t * nvec + min(cv[j], nvec - 1)];
  __builtin_amdgcn_sched_barrier(0);

  // ids outside [0, E) are clamped without branching; one flag store at the end reports them
  bool bad = false;
  auto key_of = [&](int e, int i) {
    bad |= e < 0 || e >= a.E;
    return (min(max(e, 0), a.E - 1) << kFusedIdBits) | i;
  };
  const int ownkey = lane < a.K ? key_of(own, t * a.K + lane) : 0x7fffffff;
  // count, for each of the token's K keys, the smaller keys this wave holds
  int key[EPT];
#pragma unroll
  for (int ch = 0; ch < EPT / 4; ++ch) {
    const int first = EPT == 4 ? pos[0] : (ch * nthreads + tid) * 4;  // first entry this vector owns
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = pos[ch] + m;
      key[4 * ch + m] = (i >= first && i < a.R) ? key_of(raw[4 * ch + m], i) : 0x7fffffff;
    }
  }
  for (int k = 0; k < a.K; ++k) {
    // compact: keys below mine; padded: keys below mine of my own expert (position in segment)
    const unsigned mykey = (unsigned)__builtin_amdgcn_readlane(ownkey, k);
    int cnt = 0;
    if (PAD) {
      const unsigned lo = mykey & ~((1u << kFusedIdBits) - 1u), span = mykey - lo;
#pragma unroll
      for (int m = 0; m < EPT; ++m) cnt += __popcll(__ballot((unsigned)key[m] - lo < span));
    } else {  // one compare per (entry, key): this loop is the kernel's arithmetic
#pragma unroll
      for (int m = 0; m < EPT; ++m) cnt += __popcll(__ballot((unsigned)key[m] < mykey));
    }
    if (lane == 0) s_part[tid / kWave][k] = cnt;  // plain stores: nothing to clear, one barrier in all
  }
  if (bad && a.status) *a.status = 1;
  if (want_starts) {  // W + 1 <= 257 <= 2 * nthreads
    if (tid <= a.W) s_starts[tid] = st0;
    if (tid + nthreads <= a.W) s_starts[tid + nthreads] = st1;
  }
  __syncthreads();

  // every wave adds the partial counts up for itself: lane k takes key k, lane reads hand the K
  // slots round (no second barrier, no shared result)
  int myslot = 0;
  if (lane < a.K) {
    const int nwaves = (nthreads + kWave - 1) / kWave;
    for (int wv = 0; wv < nwaves; ++wv) myslot += s_part[wv][lane];
    if (PAD) myslot = row_of(a, ownkey >> kFusedIdBits, myslot, 0);  // position in segment -> padded row
  }
  for (int k = 0; k < a.K; ++k) {
    uint4* row = disp + (size_t)__builtin_amdgcn_readlane(myslot, k) * nvec;
#pragma unroll
    for (int j = 0; j < VPL; ++j)
      if (active[j]) store_through(row + cv[j], v[j]);
  }
  if (cs == 0 && tid < a.K) {
    const int i = t * a.K + tid;
    const int slot = myslot;
    a.slot_of_entry[i] = slot;
    a.src_of_slot[slot] = i;
    int sr, tl;
    locate_token(s_starts, a.W, a.src_rank, a.rank_start != nullptr, t, sr, tl);
    int32_t* m = a.meta + (size_t)slot * MOE_A2A_META_DIM;
    m[0] = ownkey >> kFusedIdBits;
    m[1] = sr;
    m[2] = tl;
    m[3] = tid;
    m[4] = 0;
  }
}

// Routing + dispatch in ONE launch for any table size.  A workgroup owns a tile of consecutive
// tokens.  It histograms the whole routing table once into two LDS rows per expert (entries before
// the tile / from the tile on), scans the experts for the segment starts, ranks its own entries
// (at most kTileMaxOwn) against each other, and then copies its tokens' rows, a batch of vectors
// per thread at a time; the first batch of row loads is issued before the routing so that it is in
// flight meanwhile.  The table pass costs O(R / threads) per workgroup and is amortised over the
// tile's tokens, where the one-token kernel above pays O(R K / threads) per token.  Counts are
// integer sums: the result does not depend on the order of the LDS atomics.
constexpr int kTileThreads = 1024;
constexpr int kTileMaxOwn = 256;  // entries (tokens * K) of a tile
constexpr int kTileBatch = 4;     // row vectors per thread and batch

template <int STREAM>
__global__ __launch_bounds__(kTileThreads) void route_dispatch_tile_kernel(RouteArgs a, const uint4* __restrict__ x,
                                                                          uint4* __restrict__ disp, int nvec,
                                                                          int tile_tokens) {
  __shared__ int s_cnt[2 * MOE_A2A_MAX_EXPERTS];  // [0,E): entries before the tile, [E,2E): the rest
  __shared__ int s_base[MOE_A2A_MAX_EXPERTS];     // compact slot of the tile's first entry of each expert
  __shared__ int s_tmp[kTileThreads / kWave + 1];
  __shared__ int s_starts[MOE_A2A_MAX_WORLD + 1];
  __shared__ int s_own[kTileMaxOwn];   // expert of each entry of the tile
  __shared__ int s_slot[kTileMaxOwn];  // its destination row
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * tile_tokens;
  const int ntok = min(tile_tokens, a.T - t0);
  const int first = t0 * a.K, n_own = ntok * a.K;
  const int items = ntok * nvec;  // row vectors of the tile; the tile's rows are contiguous in x
  const uint4* xt = x + (size_t)t0 * nvec;

  uint4 v[kTileBatch];
#pragma unroll
  for (int b = 0; b < kTileBatch; ++b) v[b] = load_row<STREAM>(xt + min(tid + b * kTileThreads, items - 1));

  for (int j = tid; j < 2 * a.E; j += kTileThreads) s_cnt[j] = 0;
  load_starts(a, s_starts);
  __syncthreads();
  for (int i0 = 0; i0 < a.R; i0 += 4 * kTileThreads) {  // four loads in flight per thread
    int e[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) e[m] = a.indices[min(i0 + m * kTileThreads + tid, a.R - 1)];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = i0 + m * kTileThreads + tid;
      if (i < a.R) atomicAdd(&s_cnt[(i < first ? 0 : a.E) + clamp_expert(a, e[m])], 1);
    }
  }
  __syncthreads();
  const int all = tid < a.E ? s_cnt[tid] + s_cnt[a.E + tid] : 0;
  int total;
  const int run = block_exclusive_scan(all, s_tmp, total);
  if (tid < a.E) {
    s_base[tid] = run + s_cnt[tid];
    if (blockIdx.x == 0) {
      a.counts[tid] = all;
      a.offsets[tid] = run;
    }
  }
  if (blockIdx.x == 0 && tid == 0) a.offsets[a.E] = total;
  int e_own = 0;
  if (tid < n_own) {
    e_own = load_expert(a, first + tid, true);
    s_own[tid] = e_own;
  }
  __syncthreads();
  if (tid < n_own) {
    int rank = 0;  // earlier entries of the tile with the same expert (every lane reads the same word)
    for (int j = 0; j < tid; ++j) rank += s_own[j] == e_own;
    const int first_of_e = s_base[e_own] - s_cnt[e_own];
    const int slot = s_base[e_own] + rank;
    emit_entry(a, s_starts, first + tid, e_own, slot, first_of_e);
    s_slot[tid] = row_of(a, e_own, slot, first_of_e);
  }
  __syncthreads();

  for (int base = 0; base < items; base += kTileBatch * kTileThreads) {
    if (base > 0) {
#pragma unroll
      for (int b = 0; b < kTileBatch; ++b) v[b] = load_row<STREAM>(xt + min(base + tid + b * kTileThreads, items - 1));
    }
#pragma unroll
    for (int b = 0; b < kTileBatch; ++b) {
      const int item = base + tid + b * kTileThreads;
      if (item < items) {
        const int tt = item / nvec;
        const int c = item - tt * nvec;
        for (int k = 0; k < a.K; ++k) store_row<STREAM>(disp + (size_t)s_slot[tt * a.K + k] * nvec + c, v[b]);
      }
    }
  }
}

// fp8 dispatch.  8 lanes own one 128-column block (16 elements each): block amax by three
// xor-shuffles, scale = amax/448 (pow2: rounded up to a power of two, the scale format of the
// matrix instruction's block exponents), q = e4m3(x/scale) with the hardware conversion (RNE).
// Geometry is in lanes of 16 input elements: nvec = 8 * nblk, per a multiple of 8.
template <class E, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void dispatch_fp8_kernel(const uint4* __restrict__ x,
                                                                       const int32_t* __restrict__ slot_of_entry,
                                                                       uint4* __restrict__ disp_q,
                                                                       float* __restrict__ disp_scale, int K,
                                                                       int nblk, int per, int nsplit, int pow2) {
  const RowCut r = row_cut(nblk * 8, per, nsplit);
  float f[16];
  if (r.active) {
    const uint4* src = x + ((size_t)r.t * nblk * 8 + r.c) * 2;
    uint4 v0 = load_row<STREAM>(src), v1 = load_row<STREAM>(src + 1);
    uint32_t d[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      f[2 * j] = E::lo(d[j]);
      f[2 * j + 1] = E::hi(d[j]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) f[j] = 0.f;
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(f[j]));
  amax = fmaxf(amax, __shfl_xor(amax, 1, kWave));
  amax = fmaxf(amax, __shfl_xor(amax, 2, kWave));
  amax = fmaxf(amax, __shfl_xor(amax, 4, kWave));
  if (!r.active) return;
  float scale = amax == 0.f ? 1.f : amax / 448.f;
  if (pow2) {  // the next power of two at or above amax / 448, within the normal range
    const uint32_t u = __float_as_uint(scale);
    const uint32_t e = min(max((u >> 23) + ((u & 0x7fffffu) != 0 ? 1u : 0u), 1u), 254u);
    scale = __uint_as_float(e << 23);
  }
  uint32_t q[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] / scale, f[4 * j + 1] / scale, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] / scale, f[4 * j + 3] / scale, w, true);
    q[j] = (uint32_t)w;
  }
  const uint4 qv = make_uint4(q[0], q[1], q[2], q[3]);
  const int gb = r.c >> 3;
  const int32_t* sl = slot_of_entry + (size_t)r.t * K;
  for (int k = 0; k < K; ++k) {
    size_t row = (size_t)sl[k];
    store_through(disp_q + row * nblk * 8 + r.c, qv);
    if ((r.c & 7) == 0) disp_scale[row * nblk + gb] = scale;
  }
}

// ---------------------------------------------------------------------------------------
// expert stub
// ---------------------------------------------------------------------------------------
template <class In, class Out>
__device__ __forceinline__ uint4 stub_vec(const uint4& v, float s) {
  uint32_t d[4];
  unpack8(v, d);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float a = In::lo(d[j]), b = In::hi(d[j]);
    round_pair<Out>(a, b);  // .to(out_dtype); identity when In == Out
    d[j] = Out::pack(a * s, b * s);
  }
  return make_uint4(d[0], d[1], d[2], d[3]);
}

__device__ __forceinline__ void fp8x4_to_f32(uint32_t w, float (&f)[4]) {
  f[0] = __builtin_amdgcn_cvt_f32_fp8((int)w, 0);
  f[1] = __builtin_amdgcn_cvt_f32_fp8((int)w, 1);
  f[2] = __builtin_amdgcn_cvt_f32_fp8((int)w, 2);
  f[3] = __builtin_amdgcn_cvt_f32_fp8((int)w, 3);
}

// 16 fp8 values -> 16 values of Out: round_out((f32(q) * scale) * s)
template <class Out>
__device__ __forceinline__ void stub_vec_fp8(const uint4& q, float scale, float s, uint4& o0, uint4& o1) {
  const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
  uint32_t o[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float f[4];
    fp8x4_to_f32(qw[j], f);
    o[2 * j] = Out::pack((f[0] * scale) * s, (f[1] * scale) * s);
    o[2 * j + 1] = Out::pack((f[2] * scale) * s, (f[3] * scale) * s);
  }
  o0 = make_uint4(o[0], o[1], o[2], o[3]);
  o1 = make_uint4(o[4], o[5], o[6], o[7]);
}

template <class In, class Out, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void stub_rows_kernel(const uint4* __restrict__ disp,
                                                                    const int32_t* __restrict__ meta,
                                                                    uint4* __restrict__ y, int stub_kind, int E,
                                                                    int E_l, int nvec, int per, int nsplit,
                                                                    const int32_t* __restrict__ rows) {
  const RowCut r = row_cut(nvec, per, nsplit);
  if (!r.active) return;
  const size_t row = rows ? rows[r.t] : r.t;  // padded layout: visit the rows that hold entries
  const uint4 v = load_row<STREAM>(disp + row * nvec + r.c);
  const float s = stub_factor(meta[row * MOE_A2A_META_DIM], stub_kind, E, E_l);
  store_row<STREAM>(y + row * nvec + r.c, stub_vec<In, Out>(v, s));
}

// fp8 rows: each lane turns 8 bytes into 8 output elements, so a wave's stores are one
// contiguous kilobyte (a 16-byte load per lane would leave every lane two stores 32 bytes
// apart).  Geometry is that of the 16-bit output row: nvec = H / 8 lanes.
template <class Out, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void stub_fp8_kernel(const uint2* __restrict__ disp_q,
                                                                   const float* __restrict__ disp_scale,
                                                                   const int32_t* __restrict__ meta,
                                                                   uint4* __restrict__ y, int stub_kind, int E,
                                                                   int E_l, int nvec, int per, int nsplit,
                                                                   const int32_t* __restrict__ rows) {
  const RowCut r = row_cut(nvec, per, nsplit);
  if (!r.active) return;
  const size_t row = rows ? rows[r.t] : r.t;
  const uint2* src = disp_q + row * nvec + r.c;
  uint2 q;
  if (STREAM) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    u32x2_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(src));
    q = make_uint2(t.x, t.y);
  } else {
    q = *src;
  }
  const float scale = disp_scale[row * (nvec >> 4) + (r.c >> 4)];
  const float s = stub_factor(meta[row * MOE_A2A_META_DIM], stub_kind, E, E_l);
  float f0[4], f1[4];
  fp8x4_to_f32(q.x, f0);
  fp8x4_to_f32(q.y, f1);
  store_row<STREAM>(y + row * nvec + r.c,
                    make_uint4(Out::pack((f0[0] * scale) * s, (f0[1] * scale) * s),
                               Out::pack((f0[2] * scale) * s, (f0[3] * scale) * s),
                               Out::pack((f1[0] * scale) * s, (f1[1] * scale) * s),
                               Out::pack((f1[2] * scale) * s, (f1[3] * scale) * s)));
}

// ---------------------------------------------------------------------------------------
// combine
// ---------------------------------------------------------------------------------------
// The K entries of a token are folded in STRICT = ascending slot order (the order in which the
// reference's receive loop meets them) or F32 = k order.  Every wave keeps its own copy of the
// token's entries, one per lane (lane k = entry k), ranks them with lane reads, and pulls the
// entry at sorted position j into uniform registers -- no LDS, no barrier.
struct EntryLanes {
  int slot;   // lane k: slot of entry k
  float w;    // lane k: routing weight of entry k
  float f;    // lane k: stub factor of entry k (stub_combine only)
  int pos;    // lane k: position of entry k in the fold order
  int src;    // lane j: the lane whose entry has fold position j
  bool live;  // lane < K
};

template <int MODE>
__device__ __forceinline__ EntryLanes load_entries(const int32_t* __restrict__ slot_of_entry,
                                                   const float* __restrict__ weights, int t, int K) {
  const int lane = threadIdx.x & (kWave - 1);
  EntryLanes en;
  en.live = lane < K;
  en.slot = 0x7fffffff;
  en.w = 0.f;
  en.f = 1.f;
  if (en.live) {
    en.slot = slot_of_entry[(size_t)t * K + lane];
    en.w = weights[(size_t)t * K + lane];
  }
  en.pos = lane;
  en.src = lane;
  if (MODE == MOE_A2A_COMBINE_STRICT) {
    en.pos = 0;
    for (int j = 0; j < K; ++j) {
      const int sj = __builtin_amdgcn_readlane(en.slot, j);
      en.pos += sj < en.slot || (sj == en.slot && j < lane);  // ties by k keep positions distinct
    }
    // invert the permutation with one cross-lane scatter: lane pos receives this lane's number
    // (lanes >= K all land on lane K, which nobody reads)
    en.src = __builtin_amdgcn_ds_permute(en.pos << 2, lane);
  }
  return en;
}

// value of x in lane `src` (uniform), as bits: the builtin takes integers
__device__ __forceinline__ float lane_read(float x, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src));
}

// lane that holds the entry of fold position j (uniform)
template <int MODE>
__device__ __forceinline__ int entry_lane(const EntryLanes& en, int j) {
  if (MODE != MOE_A2A_COMBINE_STRICT) return j;
  return __builtin_amdgcn_readlane(en.src, j);
}

template <class E, int MODE>
__device__ __forceinline__ void accumulate8(float (&acc)[8], const uint4& v, float w) {
  uint32_t d[4];
  unpack8(v, d);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float a = acc[2 * j] + E::lo(d[j]) * w;
    float b = acc[2 * j + 1] + E::hi(d[j]) * w;
    if (MODE == MOE_A2A_COMBINE_STRICT) round_pair<E>(a, b);
    acc[2 * j] = a;
    acc[2 * j + 1] = b;
  }
}

template <class E>
__device__ __forceinline__ uint4 pack8(const float (&acc)[8]) {
  return make_uint4(E::pack(acc[0], acc[1]), E::pack(acc[2], acc[3]), E::pack(acc[4], acc[5]),
                    E::pack(acc[6], acc[7]));
}

// KT > 0: top-k known at compile time, all KT row loads of a lane are issued back to back.
// KT == 0: any K, rows in batches of four.
template <class E, int MODE, int KT, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void combine_rows_kernel(const uint4* __restrict__ y,
                                                                       const float* __restrict__ weights,
                                                                       const int32_t* __restrict__ slot_of_entry,
                                                                       uint4* __restrict__ out, int K, int nvec,
                                                                       int per, int nsplit) {
  constexpr int kBatch = KT > 0 ? KT : 4;
  const int k_rt = KT ? KT : K;
  const RowCut r = row_cut(nvec, per, nsplit);
  const EntryLanes en = load_entries<MODE>(slot_of_entry, weights, r.t, k_rt);
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int j0 = 0; j0 < k_rt; j0 += kBatch) {
    uint4 v[kBatch];
    float w[kBatch];
#pragma unroll
    for (int jj = 0; jj < kBatch; ++jj)
      if (j0 + jj < k_rt) {
        const int src = entry_lane<MODE>(en, j0 + jj);
        const int slot = __builtin_amdgcn_readlane(en.slot, src);
        w[jj] = lane_read(en.w, src);
        if (r.active) v[jj] = load_row<STREAM>(y + (size_t)slot * nvec + r.c);
      }
    if (r.active) {
#pragma unroll
      for (int jj = 0; jj < kBatch; ++jj)
        if (j0 + jj < k_rt) accumulate8<E, MODE>(acc, v[jj], w[jj]);
    }
  }
  if (r.active) store_row<STREAM>(out + (size_t)r.t * nvec + r.c, pack8<E>(acc));
}

// stub folded into the combine, 16-bit dispatched rows
template <class In, class Out, int MODE, int KT, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void stub_combine_rows_kernel(
    const uint4* __restrict__ disp, const int32_t* __restrict__ indices, const float* __restrict__ weights,
    const int32_t* __restrict__ slot_of_entry, uint4* __restrict__ out, int stub_kind, int E, int E_l, int K,
    int nvec, int per, int nsplit) {
  constexpr int kBatch = KT > 0 ? KT : 4;
  const int k_rt = KT ? KT : K;
  const RowCut r = row_cut(nvec, per, nsplit);
  EntryLanes en = load_entries<MODE>(slot_of_entry, weights, r.t, k_rt);
  if (en.live)
    en.f = stub_factor(indices[(size_t)r.t * k_rt + (threadIdx.x & (kWave - 1))], stub_kind, E, E_l);
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int j0 = 0; j0 < k_rt; j0 += kBatch) {
    uint4 v[kBatch];
    float w[kBatch], f[kBatch];
#pragma unroll
    for (int jj = 0; jj < kBatch; ++jj)
      if (j0 + jj < k_rt) {
        const int src = entry_lane<MODE>(en, j0 + jj);
        const int slot = __builtin_amdgcn_readlane(en.slot, src);
        w[jj] = lane_read(en.w, src);
        f[jj] = lane_read(en.f, src);
        if (r.active) v[jj] = load_row<STREAM>(disp + (size_t)slot * nvec + r.c);
      }
    if (r.active) {
#pragma unroll
      for (int jj = 0; jj < kBatch; ++jj)
        if (j0 + jj < k_rt) accumulate8<Out, MODE>(acc, stub_vec<In, Out>(v[jj], f[jj]), w[jj]);
    }
  }
  if (r.active) store_row<STREAM>(out + (size_t)r.t * nvec + r.c, pack8<Out>(acc));
}

// stub folded into the combine, fp8 dispatched rows (16 columns per lane)
template <class Out, int MODE, int KT, int STREAM>
__global__ __launch_bounds__(kRowMaxThreads) void stub_combine_fp8_kernel(
    const uint4* __restrict__ disp_q, const float* __restrict__ disp_scale, const int32_t* __restrict__ indices,
    const float* __restrict__ weights, const int32_t* __restrict__ slot_of_entry, uint4* __restrict__ out,
    int stub_kind, int E, int E_l, int K, int nblk, int per, int nsplit) {
  constexpr int kBatch = KT > 0 ? KT : 4;
  const int k_rt = KT ? KT : K;
  const RowCut r = row_cut(nblk * 8, per, nsplit);
  EntryLanes en = load_entries<MODE>(slot_of_entry, weights, r.t, k_rt);
  if (en.live)
    en.f = stub_factor(indices[(size_t)r.t * k_rt + (threadIdx.x & (kWave - 1))], stub_kind, E, E_l);
  float acc0[8], acc1[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc0[j] = acc1[j] = 0.f;
  for (int j0 = 0; j0 < k_rt; j0 += kBatch) {
    uint4 v[kBatch];
    float sc[kBatch], w[kBatch], f[kBatch];
#pragma unroll
    for (int jj = 0; jj < kBatch; ++jj)
      if (j0 + jj < k_rt) {
        const int src = entry_lane<MODE>(en, j0 + jj);
        const size_t row = (size_t)__builtin_amdgcn_readlane(en.slot, src);
        w[jj] = lane_read(en.w, src);
        f[jj] = lane_read(en.f, src);
        if (r.active) {
          v[jj] = load_row<STREAM>(disp_q + row * nblk * 8 + r.c);
          sc[jj] = disp_scale[row * nblk + (r.c >> 3)];
        }
      }
    if (r.active) {
#pragma unroll
      for (int jj = 0; jj < kBatch; ++jj) {
        if (j0 + jj >= k_rt) continue;
        uint4 o0, o1;
        stub_vec_fp8<Out>(v[jj], sc[jj], f[jj], o0, o1);
        accumulate8<Out, MODE>(acc0, o0, w[jj]);
        accumulate8<Out, MODE>(acc1, o1, w[jj]);
      }
    }
  }
  if (r.active) {
    uint4* dst = out + ((size_t)r.t * nblk * 8 + r.c) * 2;
    store_row<STREAM>(dst, pack8<Out>(acc0));
    store_row<STREAM>(dst + 1, pack8<Out>(acc1));
  }
}

// ---------------------------------------------------------------------------------------
// expert compute: grouped GEMM over the expert segments (the step between dispatch and combine)
// ---------------------------------------------------------------------------------------
// y[rows of e, :] = x[rows of e, :] * W_e^T with W_e[N, Kd] (both operands K-contiguous), f32
// accumulation on the matrix cores (v_mfma_f32_32x32x16), one rounding to the 16-bit output.
// A workgroup of four waves owns a 128x128 output tile (each wave 64x64 = 2x2 MFMA blocks);
// K advances 64 at a time through LDS (row stride 72 elements, so the 16-byte fragment reads
// of 16 consecutive rows fall on disjoint banks); the next K slab is fetched into registers
// while the current one is multiplied.  Tiles are numbered n-fastest, so with N/128 a multiple
// of 8 every m-tile that needs the weight slab (e, n-tile) runs on the same XCD and finds it in
// that XCD's L2.
constexpr int kGemmM = 128, kGemmN = 128, kGemmK = 64;
constexpr int kGemmLd = kGemmK + 8;  // LDS row stride in elements
constexpr int kGemmThreads = 256;

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

template <class E>
__device__ __forceinline__ f32x16_t mfma_32x32x16(const uint4& a, const uint4& b, const f32x16_t& c);
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16<Bf16>(const uint4& a, const uint4& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16<F16>(const uint4& a, const uint4& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                0, 0);
}

template <class E>
__global__ __launch_bounds__(kGemmThreads) void expert_gemm_kernel(const uint4* __restrict__ x,
                                                                    const uint4* __restrict__ w,
                                                                    const int32_t* __restrict__ offsets,
                                                                    uint16_t* __restrict__ y, int num_experts,
                                                                    int Kd, int N, int max_recv, int ntile_n) {
  __shared__ __attribute__((aligned(16))) uint16_t s_ab[(kGemmM + kGemmN) * kGemmLd];
  uint16_t* s_a = s_ab;
  uint16_t* s_b = s_ab + kGemmM * kGemmLd;
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[kGemmThreads / kWave + 1];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;

  // which (expert, m-tile, n-tile) is this workgroup?  m-tiles of all experts are numbered in
  // expert order; the prefix of ceil(count/128) is scanned here (E <= 1024: four per thread)
  const int tile_n = blockIdx.x % ntile_n;
  const int tile_m_global = blockIdx.x / ntile_n;
  {
    const int span = (num_experts + kGemmThreads - 1) / kGemmThreads;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + kGemmM - 1) / kGemmM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + kGemmM - 1) / kGemmM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    if (tile_m_global >= total) return;  // the grid is sized for the worst case
  }
  int e_lo = 0, e_hi = num_experts;  // largest e with s_pref[e] <= tile_m_global
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = e_lo;
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * kGemmM;          // first row of the tile inside the segment
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;  // its row in x and y
  const int rows = min(kGemmM, count - m0);
  const int n0 = tile_n * kGemmN;
  const int kvec = Kd / 8;  // 16-byte vectors per row

  // global -> register prefetch: a 128 x 64 slab is 1024 vectors, four per thread (8 per row)
  const uint4* xa = x + row0 * kvec;
  const uint4* wb = w + ((size_t)e * N + n0) * kvec;
  uint4 ra[4], rb[4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int v = tid + i * kGemmThreads;
      const int r = v >> 3, c = v & 7;
      ra[i] = r < rows ? xa[(size_t)r * kvec + (k0 >> 3) + c] : make_uint4(0, 0, 0, 0);
      rb[i] = n0 + r < N ? wb[(size_t)r * kvec + (k0 >> 3) + c] : make_uint4(0, 0, 0, 0);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int v = tid + i * kGemmThreads;
      const int r = v >> 3, c = v & 7;
      *reinterpret_cast<uint4*>(&s_a[r * kGemmLd + c * 8]) = ra[i];
      *reinterpret_cast<uint4*>(&s_b[r * kGemmLd + c * 8]) = rb[i];
    }
  };

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;  // this wave's 64x64 corner of the tile
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;

  fetch(0);
  for (int k0 = 0; k0 < Kd; k0 += kGemmK) {
    stash();
    __syncthreads();
    if (k0 + kGemmK < Kd) fetch(k0 + kGemmK);  // in flight during the multiplies below
#pragma unroll
    for (int kk = 0; kk < kGemmK; kk += 16) {
      uint4 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *reinterpret_cast<const uint4*>(&s_a[(wm + i * 32 + frag_row) * kGemmLd + kk + frag_k]);
        fb[i] = *reinterpret_cast<const uint4*>(&s_b[(wn + i * 32 + frag_row) * kGemmLd + kk + frag_k]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x16<E>(fa[i], fb[j], acc[i][j]);
    }
    __syncthreads();
  }

  // epilogue: each wave rounds and stores its own accumulators, no LDS staging and no barrier
  // (the staged 16-byte-store form measured 10 % slower: its two barriers idle the MFMA pipes
  // of every wave in the workgroup).  Accumulator element q of a 32x32 block sits at row
  // (q/4)*8 + (lane/32)*4 + q%4, column lane%32, so one store covers 64 contiguous bytes per
  // half wave.
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int r = wm + i * 32 + (q >> 2) * 8 + (lane >> 5) * 4 + (q & 3);
        const int c = wn + j * 32 + (lane & 31);
        if (r < rows && n0 + c < N)
          y[(row0 + r) * (size_t)N + n0 + c] = (uint16_t)(E::pack(acc[i][j][q], 0.f) & 0xffffu);
      }
}

// Wide variant for long segments: 256 x 256 output tile, four waves of 128 x 128 (a 4 x 4 grid of
// 32x32 accumulator blocks, 256 AGPRs), K slabs of 64.  One wave per SIMD and one workgroup per
// CU, so latency is hidden inside the wave: operand slabs are double-buffered in LDS (144 KB),
// the next slab travels global -> registers a whole iteration ahead, and the fragments of step
// kk+1 are read from LDS while the sixteen MFMAs of step kk issue.  Per output element a wave
// reads half the LDS bytes of the 128 x 128 kernel, which is what bounds that kernel (one
// ds_read_b128 per MFMA at 128 B/clk per CU).  The scheduling-group barriers pin the interleave;
// the scheduling barriers keep the compiler from sinking a step's fragment reads into the next
// step, where they would be waited on at once.  Accumulation order over K equals the 128 x 128
// kernel's, so both give the same bits.  Tiles with at most 128 rows take a 128 x 256 form of the
// same loop.
constexpr int kWideM = 256, kWideN = 256, kWideK = 64, kWideLd = kWideK + 8, kWideThreads = 256;
constexpr size_t kWideLdsBytes = 2 * (size_t)(kWideM + kWideN) * kWideLd * sizeof(uint16_t);
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

template <class E>
__device__ __forceinline__ f32x16_t mfma_32x32x16_v(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c);
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16_v<Bf16>(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16_v<F16>(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                0, 0);
}

// Skinny variant for short segments (a decode step: a handful of rows per expert).  The work is
// then streaming each expert's weights once: 32 x 128 output tiles (one row block, so 4x fewer
// MFMAs are spent on rows that do not exist than with 128-row tiles), four waves side by side on
// 32 x 32 each, K slabs of 128 (256 contiguous bytes of every weight row per slab: measured 6.09
// TB/s of weights at 256 experts x 8 rows, 7168 -> 2048, against 5.95 with 256 x 64 slabs and 5.84
// for the 128 x 128 kernel), weights loaded non-temporally (each is read once: 6.65 TB/s), and the
// global -> register prefetch runs TWO slabs ahead in two register sets.  Accumulation order over K equals the other kernels': same bits.
constexpr int kSkinnyM = 32, kSkinnyThreads = 256;
#ifndef MOE_A2A_SKINNY_N
#define MOE_A2A_SKINNY_N 128
#define MOE_A2A_SKINNY_K 128
#endif
constexpr int kSkinnyN = MOE_A2A_SKINNY_N, kSkinnyK = MOE_A2A_SKINNY_K;

template <class E>
__global__ __launch_bounds__(kSkinnyThreads, 3) void expert_gemm_skinny_kernel(const uint4* __restrict__ x,
                                                                            const uint4* __restrict__ w,
                                                                            const int32_t* __restrict__ offsets,
                                                                            uint16_t* __restrict__ y, int num_experts,
                                                                            int Kd, int N, int max_recv, int ntile_n) {
  constexpr int TM = kSkinnyM, TN = kSkinnyN, BK = kSkinnyK, LD = BK + 8, NT = kSkinnyThreads;  // Kd % BK == 0
  constexpr int WJ = TN / 128;  // 32-column blocks per wave
  __shared__ __attribute__((aligned(16))) uint16_t s_ab[(TM + TN) * LD];
  uint16_t* s_a = s_ab;
  uint16_t* s_b = s_ab + TM * LD;
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[NT / kWave + 1];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;

  const int tile_n = blockIdx.x % ntile_n;
  const int tile_m_global = blockIdx.x / ntile_n;
  {
    const int span = (num_experts + NT - 1) / NT;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    if (tile_m_global >= total) return;
  }
  int e_lo = 0, e_hi = num_experts;
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = e_lo;
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * TM;
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;
  const int rows = min(TM, count - m0);
  const int n0 = tile_n * TN;
  const int ncols = min(TN, N - n0);
  const int kvec = Kd / 8;
  const u32x4_t* xa = reinterpret_cast<const u32x4_t*>(x) + row0 * kvec;
  const u32x4_t* wb = reinterpret_cast<const u32x4_t*>(w) + ((size_t)e * N + n0) * kvec;

  // per slab: one vector of A (32 rows x 8) and eight of B (256 rows x 8) per thread; rows past
  // the segment / columns past N read the last valid one (they feed accumulators never stored)
  constexpr int VPR = BK / 8, NB = TN * VPR / NT;
  constexpr int NA = TM * VPR / NT > 0 ? TM * VPR / NT : 1;
  int offa[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int v = tid + i * NT;
    offa[i] = min(v / VPR, rows - 1) * kvec + v % VPR;
  }
  int offb[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int v = tid + i * NT;
    offb[i] = min(v / VPR, ncols - 1) * kvec + v % VPR;
  }
  const int st_off = (tid / VPR) * LD + (tid % VPR) * 8;
  u32x4_t ra0[NA], rb0[NB], ra1[NA], rb1[NB];
#define SKINNY_FETCH(RA, RB, K0)                                               \
  {                                                                            \
    const int kv_ = min((K0), Kd - BK) >> 3; /* past the end: the last slab again */ \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) RA[i] = xa[offa[i] + kv_];  \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) RB[i] = __builtin_nontemporal_load(wb + offb[i] + kv_); \
  }
#define SKINNY_STASH(RA, RB)                                                                          \
  {                                                                                                   \
    _Pragma("unroll") for (int i = 0; i < NA; ++i)                                                    \
        *reinterpret_cast<u32x4_t*>(&s_a[st_off + i * (NT / VPR) * LD]) = RA[i];                      \
    _Pragma("unroll") for (int i = 0; i < NB; ++i)                                                    \
        *reinterpret_cast<u32x4_t*>(&s_b[st_off + i * (NT / VPR) * LD]) = RB[i];                      \
  }
  f32x16_t acc[WJ];
#pragma unroll
  for (int j = 0; j < WJ; ++j)
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[j][q] = 0.f;
  const int wn = wave * 32 * WJ;
  const int fr_a = (lane & 31) * LD + (lane >> 5) * 8;
  const int fr_b = (wn + (lane & 31)) * LD + (lane >> 5) * 8;
#define SKINNY_SLAB()                                                                                 \
  {                                                                                                   \
    _Pragma("unroll") for (int kk = 0; kk < BK; kk += 16) {                                           \
      const u32x4_t fa = *reinterpret_cast<const u32x4_t*>(&s_a[fr_a + kk]);                          \
      _Pragma("unroll") for (int j = 0; j < WJ; ++j) {                                                 \
        const u32x4_t fb = *reinterpret_cast<const u32x4_t*>(&s_b[fr_b + j * 32 * LD + kk]);          \
        acc[j] = mfma_32x32x16_v<E>(fa, fb, acc[j]);                                                  \
      }                                                                                               \
    }                                                                                                 \
  }
  SKINNY_FETCH(ra0, rb0, 0);
  SKINNY_FETCH(ra1, rb1, BK);
  for (int k0 = 0; k0 < Kd; k0 += 2 * BK) {
    SKINNY_STASH(ra0, rb0);
    __syncthreads();
    SKINNY_FETCH(ra0, rb0, k0 + 2 * BK);
    SKINNY_SLAB();
    __syncthreads();
    if (k0 + BK >= Kd) break;
    SKINNY_STASH(ra1, rb1);
    __syncthreads();
    SKINNY_FETCH(ra1, rb1, k0 + 3 * BK);
    SKINNY_SLAB();
    __syncthreads();
  }
#undef SKINNY_FETCH
#undef SKINNY_STASH
#undef SKINNY_SLAB
#pragma unroll
  for (int j = 0; j < WJ; ++j)
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int r = (q >> 2) * 8 + (lane >> 5) * 4 + (q & 3);
      const int c = wn + j * 32 + (lane & 31);
      if (r < rows && c < ncols)
        y[(row0 + r) * (size_t)N + n0 + c] = (uint16_t)(E::pack(acc[j][q], 0.f) & 0xffffu);
    }
}

constexpr int kMaxDevices = 64;
constexpr int wide_gcd(int a, int b) { return b == 0 ? a : wide_gcd(b, a % b); }

// 16 fp8 (e4m3fn) values and their block scale -> two vectors of 8 values of E: E(f32(q) * scale)
template <class E>
__device__ __forceinline__ void wide_decode_fp8(const u32x4_t& q, float scale, u32x4_t& lo, u32x4_t& hi) {
  uint32_t o[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float f[4];
    fp8x4_to_f32(q[j], f);
    o[2 * j] = E::pack(f[0] * scale, f[1] * scale);
    o[2 * j + 1] = E::pack(f[2] * scale, f[3] * scale);
  }
  lo = u32x4_t{o[0], o[1], o[2], o[3]};
  hi = u32x4_t{o[4], o[5], o[6], o[7]};
}

// 16 fp8 (e4m3fn) values -> two vectors of 8 values of E, exactly (every e4m3fn value is a bf16 and
// an f16 value)
template <class E>
__device__ __forceinline__ void exact_fp8_to_16(const u32x4_t& q, u32x4_t& lo, u32x4_t& hi) {
  uint32_t o[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float f[4];
    fp8x4_to_f32(q[j], f);
    o[2 * j] = E::pack(f[0], f[1]);
    o[2 * j + 1] = E::pack(f[2], f[3]);
  }
  lo = u32x4_t{o[0], o[1], o[2], o[3]};
  hi = u32x4_t{o[4], o[5], o[6], o[7]};
}

// The weight-streaming kernel for quantised operands (the block format of DeepSeek-V3 checkpoints):
// weights as e4m3fn bytes with one f32 scale per 128 x 128 block, activations either 16-bit or the
// e4m3fn rows + per-(row, 128 columns) scales that dispatch_fp8 writes (AFP8).  Tile 32 x 128, K
// slabs of 128, so a workgroup meets exactly one weight scale per slab: the weight bytes go into
// LDS as exact 16-bit values, each slab is summed on the matrix cores into a partial accumulator,
// and the partial is folded into the result with one fma per element, acc += scale * partial --
// y = sum over K blocks of scale_b * (x . q_b), the scale applied in f32 after the block sum.
// Activation rows are dequantised on their way into LDS, E(f32(q) * scale) (they are a thousandth
// of the traffic here).  The weights cross HBM as one byte per element, which is what bounds a
// decode step; four slabs are in flight per workgroup in four register sets.
template <class E, bool AFP8>
__global__ __launch_bounds__(kSkinnyThreads, 3) void expert_gemm_skinny_q_kernel(
    const uint4* __restrict__ x, const float* __restrict__ x_scale, const uint4* __restrict__ w,
    const float* __restrict__ w_scale, const int32_t* __restrict__ offsets, uint16_t* __restrict__ y,
    int num_experts, int Kd, int N, int max_recv, int ntile_n) {
  constexpr int TM = kSkinnyM, TN = 128, BK = 128, LD = BK + 8, NT = kSkinnyThreads;  // Kd % 128 == 0, N % 128 == 0
  __shared__ __attribute__((aligned(16))) uint16_t s_ab[(TM + TN) * LD];
  uint16_t* s_a = s_ab;
  uint16_t* s_b = s_ab + TM * LD;
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[NT / kWave + 1];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int tile_n = blockIdx.x % ntile_n;
  const int tile_m_global = blockIdx.x / ntile_n;
  {
    const int span = (num_experts + NT - 1) / NT;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    if (tile_m_global >= total) return;
  }
  int e_lo = 0, e_hi = num_experts;
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = __builtin_amdgcn_readfirstlane(e_lo);  // the same in every lane: scales load as scalars
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * TM;
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;
  const int rows = min(TM, count - m0);
  const int n0 = tile_n * TN;
  const int kblocks = Kd / 128;
  // vectors of 16 bytes: 8 elements of a 16-bit operand, 16 of an fp8 one
  constexpr int AV = AFP8 ? BK / 16 : BK / 8, BV = BK / 16;  // per row and slab
  constexpr int NA = TM * AV / NT, NB = TN * BV / NT;         // per thread: 1 or 2, and 4
  static_assert(NA >= 1, "a slab of A holds at least one vector per thread");
  const int a_row_vecs = AFP8 ? Kd / 16 : Kd / 8, b_row_vecs = Kd / 16;
  const u32x4_t* xa = reinterpret_cast<const u32x4_t*>(x) + row0 * a_row_vecs;
  const u32x4_t* wb = reinterpret_cast<const u32x4_t*>(w) + ((size_t)e * N + n0) * b_row_vecs;
  const float* xs = AFP8 ? x_scale + row0 * kblocks : nullptr;
  const float* ws = w_scale + ((size_t)e * (N / 128) + tile_n) * kblocks;
  int offa[NA], offs[NA], sta[NA], offb[NB], stb[NB];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int v = tid + i * NT, r = v / AV, c = v % AV;
    offa[i] = min(r, rows - 1) * a_row_vecs + c;
    offs[i] = min(r, rows - 1) * kblocks;
    sta[i] = r * LD + c * (AFP8 ? 16 : 8);
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int v = tid + i * NT, r = v / BV, c = v % BV;
    offb[i] = r * b_row_vecs + c;  // N % 128 == 0: every column of the tile exists
    stb[i] = r * LD + c * 16;
  }
  struct Slab {
    u32x4_t a[NA], b[NB];
    float as[NA];
    float bs;
  };
  Slab s0, s1, s2, s3;
#define SKQ_FETCH(S, K0)                                                                              \
  {                                                                                                   \
    const int k_ = min((K0), Kd - BK); /* past the end: the last slab again */                        \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) {                                                  \
      S.a[i] = xa[offa[i] + (k_ >> (AFP8 ? 4 : 3))];                                                  \
      S.as[i] = AFP8 ? xs[offs[i] + (k_ >> 7)] : 1.f;                                                 \
    }                                                                                                 \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) S.b[i] = __builtin_nontemporal_load(wb + offb[i] + (k_ >> 4)); \
    S.bs = ws[k_ >> 7];                                                                               \
  }
#define SKQ_STASH(S)                                                                                  \
  {                                                                                                   \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) {                                                  \
      if (AFP8) {                                                                                     \
        u32x4_t lo_, hi_;                                                                             \
        wide_decode_fp8<E>(S.a[i], S.as[i], lo_, hi_);                                                \
        *reinterpret_cast<u32x4_t*>(&s_a[sta[i]]) = lo_;                                              \
        *reinterpret_cast<u32x4_t*>(&s_a[sta[i] + 8]) = hi_;                                          \
      } else {                                                                                        \
        *reinterpret_cast<u32x4_t*>(&s_a[sta[i]]) = S.a[i];                                           \
      }                                                                                               \
    }                                                                                                 \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) {                                                  \
      u32x4_t lo_, hi_;                                                                               \
      exact_fp8_to_16<E>(S.b[i], lo_, hi_);                                                           \
      *reinterpret_cast<u32x4_t*>(&s_b[stb[i]]) = lo_;                                                \
      *reinterpret_cast<u32x4_t*>(&s_b[stb[i] + 8]) = hi_;                                            \
    }                                                                                                 \
  }
  f32x16_t acc;
#pragma unroll
  for (int q = 0; q < 16; ++q) acc[q] = 0.f;
  const int wn = wave * 32;
  const int fr_a = (lane & 31) * LD + (lane >> 5) * 8;
  const int fr_b = (wn + (lane & 31)) * LD + (lane >> 5) * 8;
#define SKQ_SLAB(SCALE)                                                                               \
  {                                                                                                   \
    f32x16_t part;                                                                                    \
    _Pragma("unroll") for (int q = 0; q < 16; ++q) part[q] = 0.f;                                     \
    _Pragma("unroll") for (int kk = 0; kk < BK; kk += 16) {                                           \
      const u32x4_t fa = *reinterpret_cast<const u32x4_t*>(&s_a[fr_a + kk]);                          \
      const u32x4_t fb = *reinterpret_cast<const u32x4_t*>(&s_b[fr_b + kk]);                          \
      part = mfma_32x32x16_v<E>(fa, fb, part);                                                        \
    }                                                                                                 \
    _Pragma("unroll") for (int q = 0; q < 16; ++q) acc[q] = __builtin_fmaf(part[q], (SCALE), acc[q]); \
  }
#define SKQ_STEP(S, KNEXT)                                                                            \
  {                                                                                                   \
    SKQ_STASH(S);                                                                                     \
    const float scale_ = S.bs;                                                                        \
    __syncthreads();                                                                                  \
    SKQ_FETCH(S, (KNEXT));                                                                            \
    SKQ_SLAB(scale_);                                                                                 \
    __syncthreads();                                                                                  \
  }
  SKQ_FETCH(s0, 0);
  SKQ_FETCH(s1, BK);
  SKQ_FETCH(s2, 2 * BK);
  SKQ_FETCH(s3, 3 * BK);
  for (int k0 = 0; k0 < Kd; k0 += 4 * BK) {
    SKQ_STEP(s0, k0 + 4 * BK);
    if (k0 + BK >= Kd) break;
    SKQ_STEP(s1, k0 + 5 * BK);
    if (k0 + 2 * BK >= Kd) break;
    SKQ_STEP(s2, k0 + 6 * BK);
    if (k0 + 3 * BK >= Kd) break;
    SKQ_STEP(s3, k0 + 7 * BK);
  }
#undef SKQ_FETCH
#undef SKQ_STASH
#undef SKQ_SLAB
#undef SKQ_STEP
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int r = (q >> 2) * 8 + (lane >> 5) * 4 + (q & 3);
    const int c = wn + (lane & 31);
    if (r < rows) y[(row0 + r) * (size_t)N + n0 + c] = (uint16_t)(E::pack(acc[q], 0.f) & 0xffffu);
  }
}

// Main loop and epilogue of one wide tile.  Each wave owns WMI x WNJ accumulator blocks of 32 x 32
// at (wm, wn); AROWS rows of the A operand are staged per slab (256, or 128 when the tile holds
// no more rows than that), always 256 rows of B.
template <class E, int WMI, int WNJ, int AROWS, bool AFP8, bool BFP8, bool MX = false>
__device__ __forceinline__ void wide_tile(const u32x4_t* __restrict__ xa, const float* __restrict__ xs,
                                          const u32x4_t* __restrict__ wb, const float* __restrict__ wsc,
                                          uint16_t* __restrict__ y_tile, uint16_t* s_wide, int rows, int ncols,
                                          int Kd, int N, int wm, int wn) {
  constexpr int TM = kWideM, TN = kWideN, BK = kWideK, LD = kWideLd, NT = kWideThreads;
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int kvec = Kd / 8;
  // A slab is AROWS (A) + 256 (B) rows of 64 elements.  Rows past the segment and columns past N
  // read the last valid row instead of zeros: they only feed accumulators that are never stored,
  // and the loads stay unconditional.  A 16-bit operand: 8 vectors of 8 elements per row.  An fp8
  // operand: 4 vectors of 16 elements per row plus a scale -- for A (AFP8) the row's f32 scale of
  // that 128-column block, for B (BFP8) the scale of the 128 x 128 weight block (two column blocks
  // per tile: wsc[0..] and wsc[Kd/128..]); a vector is turned into two 16-bit vectors,
  // E(f32(q) * scale), on its way into LDS, so the LDS image and the number of LDS stores per
  // thread are those of the 16-bit case.
  // MX: both operands are fp8 bytes that go to the fp8 matrix instruction as they are, with scales
  // that are powers of two and ride along as the instruction's block exponents.  The caller passes
  // Kd = bytes per row / 2, so a row looks like a 16-bit row of half the length and everything on
  // the way into LDS is the 16-bit case; a slab of 64 such elements is one 128-wide scale block.
  // xs = the tile's first row of x_scale, wsc = the scales of this wave's 128-column block.
  static_assert(!MX || (!AFP8 && !BFP8), "MX operands are copied, not decoded");
  constexpr int VPR = BK / 8;
  constexpr int AVPR = AFP8 ? BK / 16 : VPR, BVPR = BFP8 ? BK / 16 : VPR;  // global vectors per row and slab
  constexpr int NA = AROWS * AVPR / NT, NB = TN * BVPR / NT;               // ... per thread
  constexpr int NS = AFP8 ? NA : 0;                                         // A scales per thread
  int offa[NA], offs[NS > 0 ? NS : 1], offb[NB];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int v = tid + i * NT;
    const int r = min(v / AVPR, rows - 1);
    offa[i] = r * (AFP8 ? Kd / 16 : kvec) + v % AVPR;
    if (AFP8) offs[i] = r * (Kd / 128);
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int v = tid + i * NT;
    offb[i] = min(v / BVPR, ncols - 1) * (BFP8 ? Kd / 16 : kvec) + v % BVPR;
  }
  // native vectors, not uint4: the struct type keeps the staging arrays in scratch memory
  u32x4_t ra[NA], rb[NB];
  float rs[NS > 0 ? NS : 1];
  float rsb[2] = {1.f, 1.f};  // weight scales of the tile's two column blocks for the slab in flight
  // MX: scale of each of the lane's WMI rows (row lane % 32 of every 32-row block) for the slab in flight
  int mx_off[MX ? WMI : 1];  // a tile's scales span at most 256 rows x Kd / 64 floats: an int offset
  float mx_rsa[MX ? WMI : 1];
  if (MX) {
#pragma unroll
    for (int i = 0; i < WMI; ++i) mx_off[i] = min(wm + i * 32 + (lane & 31), rows - 1) * (Kd / 64);
  }
  const int sb1 = ncols > 128 ? Kd / 128 : 0;  // a tile of one column block reads its scale twice
  const int st_off_a = (tid / AVPR) * LD + (tid % AVPR) * (AFP8 ? 16 : 8);
  const int st_off_b = (tid / BVPR) * LD + (tid % BVPR) * (BFP8 ? 16 : 8);
#define WIDE_FETCH(K0)                                                                           \
  {                                                                                              \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) ra[i] = xa[offa[i] + ((K0) >> (AFP8 ? 4 : 3))]; \
    if (AFP8) { _Pragma("unroll") for (int i = 0; i < NS; ++i) rs[i] = xs[offs[i] + ((K0) >> 7)]; } \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) rb[i] = wb[offb[i] + ((K0) >> (BFP8 ? 4 : 3))]; \
    if (BFP8) {                                                                                  \
      rsb[0] = wsc[(K0) >> 7];                                                                   \
      rsb[1] = wsc[sb1 + ((K0) >> 7)];                                                           \
    }                                                                                            \
    if (MX) {                                                                                    \
      _Pragma("unroll") for (int i = 0; i < WMI; ++i) mx_rsa[i] = xs[mx_off[i] + ((K0) >> 6)];   \
      rsb[0] = wsc[(K0) >> 6];                                                                   \
    }                                                                                            \
  }
#define WIDE_STASH(BUF)                                                                                        \
  {                                                                                                            \
    uint16_t* s_a_ = s_wide + (BUF) * (TM + TN) * LD + st_off_a;                                               \
    uint16_t* s_b_ = s_wide + (BUF) * (TM + TN) * LD + TM * LD + st_off_b;                                     \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) {                                                           \
      if (AFP8) {                                                                                              \
        u32x4_t lo_, hi_;                                                                                      \
        wide_decode_fp8<E>(ra[i], rs[i], lo_, hi_);                                                            \
        *reinterpret_cast<u32x4_t*>(&s_a_[i * (NT / AVPR) * LD]) = lo_;                                        \
        *reinterpret_cast<u32x4_t*>(&s_a_[i * (NT / AVPR) * LD + 8]) = hi_;                                    \
      } else {                                                                                                 \
        *reinterpret_cast<u32x4_t*>(&s_a_[i * (NT / AVPR) * LD]) = ra[i];                                      \
      }                                                                                                        \
    }                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) {                                                           \
      if (BFP8) { /* vector i sits in row tid / 4 + 64 i: i < NB / 2 is the first column block */              \
        u32x4_t lo_, hi_;                                                                                      \
        wide_decode_fp8<E>(rb[i], rsb[i < NB / 2 ? 0 : 1], lo_, hi_);                                          \
        *reinterpret_cast<u32x4_t*>(&s_b_[i * (NT / BVPR) * LD]) = lo_;                                        \
        *reinterpret_cast<u32x4_t*>(&s_b_[i * (NT / BVPR) * LD + 8]) = hi_;                                    \
      } else {                                                                                                 \
        *reinterpret_cast<u32x4_t*>(&s_b_[i * (NT / BVPR) * LD]) = rb[i];                                      \
      }                                                                                                        \
    }                                                                                                          \
  }

  f32x16_t acc[WMI][WNJ];
#pragma unroll
  for (int i = 0; i < WMI; ++i)
#pragma unroll
    for (int j = 0; j < WNJ; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
  const int fr_a = (wm + (lane & 31)) * LD + (lane >> 5) * 8;
  const int fr_b = (TM + wn + (lane & 31)) * LD + (lane >> 5) * 8;
  u32x4_t f0a[WMI], f0b[WNJ], f1a[WMI], f1b[WNJ];
#define WIDE_FRAGS(FA, FB, BUF, KK)                                                                            \
  {                                                                                                            \
    const uint16_t* base_ = s_wide + (BUF) * (TM + TN) * LD + (KK);                                            \
    _Pragma("unroll") for (int i = 0; i < WMI; ++i)                                                            \
        FA[i] = *reinterpret_cast<const u32x4_t*>(&base_[fr_a + i * 32 * LD]);                                 \
    _Pragma("unroll") for (int j = 0; j < WNJ; ++j)                                                            \
        FB[j] = *reinterpret_cast<const u32x4_t*>(&base_[fr_b + j * 32 * LD]);                                 \
  }
#define WIDE_MMA(FA, FB)                                                                                       \
  {                                                                                                            \
    _Pragma("unroll") for (int i = 0; i < WMI; ++i)                                                            \
    _Pragma("unroll") for (int j = 0; j < WNJ; ++j) acc[i][j] = mfma_32x32x16_v<E>(FA[i], FB[j], acc[i][j]);   \
  }
  // Instruction classes of the scheduling groups: 0x008 MFMA, 0x020 VMEM read, 0x100 LDS read,
  // 0x200 LDS write.  Per step a wave issues MM MFMAs and RD fragment reads, per slab ST stores to
  // LDS and ST global loads.
  constexpr int RD = WMI + WNJ, MM = WMI * WNJ, ST = (AFP8 ? 2 * NA : NA) + (BFP8 ? 2 * NB : NB);  // LDS stores
  constexpr int GW = wide_gcd(MM, ST), GF = wide_gcd(MM - RD, ST - RD);
  static_assert(MM >= RD && ST >= RD, "interleave patterns assume at least one MFMA and one load per read");
#define WIDE_MIX_READS() /* RD x (LDS read, MFMA), then the other MFMAs */                                      \
  {                                                                                                            \
    _Pragma("unroll") for (int s_ = 0; s_ < RD; ++s_) {                                                        \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                       \
    }                                                                                                          \
    __builtin_amdgcn_sched_group_barrier(0x008, MM - RD, 0);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                         \
  }
#define WIDE_MIX_WRITES() /* the LDS reads, then MFMAs and LDS writes in even shares */                         \
  {                                                                                                            \
    __builtin_amdgcn_sched_group_barrier(0x100, RD, 0);                                                        \
    _Pragma("unroll") for (int s_ = 0; s_ < GW; ++s_) {                                                        \
      __builtin_amdgcn_sched_group_barrier(0x008, MM / GW, 0);                                                 \
      __builtin_amdgcn_sched_group_barrier(0x200, ST / GW, 0);                                                 \
    }                                                                                                          \
    __builtin_amdgcn_sched_barrier(0);                                                                         \
  }
#define WIDE_MIX_FETCH() /* RD x (LDS read, MFMA, global load), then the rest in even shares */                 \
  {                                                                                                            \
    _Pragma("unroll") for (int s_ = 0; s_ < RD; ++s_) {                                                        \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                       \
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                                                       \
    }                                                                                                          \
    _Pragma("unroll") for (int s_ = 0; s_ < GF; ++s_) {                                                        \
      __builtin_amdgcn_sched_group_barrier(0x008, (MM - RD) / GF, 0);                                          \
      __builtin_amdgcn_sched_group_barrier(0x020, (ST - RD) / GF, 0);                                          \
    }                                                                                                          \
    __builtin_amdgcn_sched_barrier(0);                                                                         \
  }

  // The prefetches past the last slab re-read the last slab (clamped k) and land in a buffer
  // nobody reads: the loop body stays free of branches.
  if constexpr (MX) {
    // One slab = two steps of the fp8 instruction; a lane's operand is 32 bytes, read as the two
    // 16-byte fragments the 16-bit loop reads for a pair of its steps (the same bytes for both
    // operands, so the order in which the instruction walks K inside a step does not matter, and
    // all its blocks of 32 carry the same exponent here).  Step 0 multiplies while step 1's
    // fragments are read; step 1's first half while the next slab goes into the other buffer and
    // the slab after that is requested; its second half while the next slab's first fragments
    // are read.
    u32x4_t f2a[WMI], f2b[WNJ], f3a[WMI], f3b[WNJ];
    int sa_cur[WMI], sa_nxt[WMI], sb_cur, sb_nxt;
#define MX_OPERAND(LO, HI) \
  i32x8_t{(int)LO[0], (int)LO[1], (int)LO[2], (int)LO[3], (int)HI[0], (int)HI[1], (int)HI[2], (int)HI[3]}
#define MX_MMA(LOA, HIA, LOB, HIB, I0, I1)                                                             \
  {                                                                                                    \
    _Pragma("unroll") for (int i = (I0); i < (I1); ++i)                                                \
    _Pragma("unroll") for (int j = 0; j < WNJ; ++j)                                                    \
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                                   \
            MX_OPERAND(LOA[i], HIA[i]), MX_OPERAND(LOB[j], HIB[j]), acc[i][j], 0, 0, 0, sa_cur[i], 0, sb_cur); \
  }
#define MX_TAKE_SCALES() /* exponent fields of the slab that has just arrived */                       \
  {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < WMI; ++i) sa_nxt[i] = (__float_as_int(mx_rsa[i]) >> 23) & 0xff; \
    sb_nxt = (__float_as_int(rsb[0]) >> 23) & 0xff;                                                    \
  }
    constexpr int HM = WMI / 2 * WNJ;  // MFMAs of half a step
    WIDE_FETCH(0);
    WIDE_STASH(0);
    MX_TAKE_SCALES();
#pragma unroll
    for (int i = 0; i < WMI; ++i) sa_cur[i] = sa_nxt[i];
    sb_cur = sb_nxt;
    WIDE_FETCH(min(BK, Kd - BK));
    __syncthreads();
    WIDE_FRAGS(f0a, f0b, 0, 0);
    WIDE_FRAGS(f1a, f1b, 0, 16);
    int buf = 0;
    for (int k0 = 0; k0 < Kd; k0 += BK, buf ^= 1) {
      WIDE_FRAGS(f2a, f2b, buf, 32);
      WIDE_FRAGS(f3a, f3b, buf, 48);
      MX_MMA(f0a, f1a, f0b, f1b, 0, WMI);
#pragma unroll
      for (int s_ = 0; s_ < 2 * HM; ++s_) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (2 * RD + 2 * HM - 1) / (2 * HM), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();  // every wave has left the previous slab: the other buffer is free
      WIDE_STASH(buf ^ 1);
      MX_TAKE_SCALES();
      WIDE_FETCH(min(k0 + 2 * BK, Kd - BK));
      MX_MMA(f2a, f3a, f2b, f3b, 0, WMI / 2);
#pragma unroll
      for (int s_ = 0; s_ < HM / 2; ++s_) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x200, (ST + HM / 2 - 1) / (HM / 2), 0);
      }
#pragma unroll
      for (int s_ = 0; s_ < HM - HM / 2; ++s_) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, (ST + WMI + 1 + HM - HM / 2 - 1) / (HM - HM / 2), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();  // the other buffer is complete
      WIDE_FRAGS(f0a, f0b, buf ^ 1, 0);
      WIDE_FRAGS(f1a, f1b, buf ^ 1, 16);
      MX_MMA(f2a, f3a, f2b, f3b, WMI / 2, WMI);
#pragma unroll
      for (int s_ = 0; s_ < HM; ++s_) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (2 * RD + HM - 1) / HM, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < WMI; ++i) sa_cur[i] = sa_nxt[i];
      sb_cur = sb_nxt;
    }
#undef MX_OPERAND
#undef MX_MMA
#undef MX_TAKE_SCALES
  } else {
  WIDE_FETCH(0);
  WIDE_STASH(0);
  WIDE_FETCH(min(BK, Kd - BK));
  __syncthreads();
  WIDE_FRAGS(f0a, f0b, 0, 0);
  int buf = 0;
  for (int k0 = 0; k0 < Kd; k0 += BK, buf ^= 1) {
    WIDE_FRAGS(f1a, f1b, buf, 16);
    WIDE_MMA(f0a, f0b);
    WIDE_MIX_READS();
    __syncthreads();  // every wave has left the previous slab: the other buffer is free
    WIDE_FRAGS(f0a, f0b, buf, 32);
    WIDE_STASH(buf ^ 1);
    WIDE_MMA(f1a, f1b);
    WIDE_MIX_WRITES();
    WIDE_FETCH(min(k0 + 2 * BK, Kd - BK));
    WIDE_FRAGS(f1a, f1b, buf, 48);
    WIDE_MMA(f0a, f0b);
    WIDE_MIX_FETCH();
    __syncthreads();  // the other buffer is complete
    WIDE_FRAGS(f0a, f0b, buf ^ 1, 0);
    WIDE_MMA(f1a, f1b);
    WIDE_MIX_READS();
  }
  }
#undef WIDE_FETCH
#undef WIDE_STASH
#undef WIDE_FRAGS
#undef WIDE_MMA
#undef WIDE_MIX_READS
#undef WIDE_MIX_WRITES
#undef WIDE_MIX_FETCH

#pragma unroll
  for (int i = 0; i < WMI; ++i)
#pragma unroll
    for (int j = 0; j < WNJ; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int r = wm + i * 32 + (q >> 2) * 8 + (lane >> 5) * 4 + (q & 3);
        const int c = wn + j * 32 + (lane & 31);
        if (r < rows && c < ncols) y_tile[r * (size_t)N + c] = (uint16_t)(E::pack(acc[i][j][q], 0.f) & 0xffffu);
      }
}

// MX: both operands fp8 with power-of-two scales, multiplied by the fp8 instruction with the
// scales as its block exponents (see wide_tile).
template <class E, bool AFP8, bool BFP8, bool MX = false>
__global__ __launch_bounds__(kWideThreads) void expert_gemm_wide_kernel(const uint4* __restrict__ x,
                                                                         const float* __restrict__ x_scale,
                                                                         const uint4* __restrict__ w,
                                                                         const float* __restrict__ w_scale,
                                                                         const int32_t* __restrict__ offsets,
                                                                         uint16_t* __restrict__ y, int num_experts,
                                                                         int Kd, int N, int max_recv, int ntile_n) {
  constexpr int TM = kWideM, TN = kWideN, NT = kWideThreads;
  extern __shared__ __attribute__((aligned(16))) uint16_t s_wide[];  // [2][TM + TN][LD]
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[NT / kWave + 1];
  const int tid = threadIdx.x, wave = tid / kWave;

  // (expert, m-tile, n-tile) of this workgroup, as in the 128 x 128 kernel with 256-row tiles
  const int tile_n = blockIdx.x % ntile_n;
  const int tile_m_global = blockIdx.x / ntile_n;
  {
    const int span = (num_experts + NT - 1) / NT;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    if (tile_m_global >= total) return;
  }
  int e_lo = 0, e_hi = num_experts;
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = e_lo;
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * TM;
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;
  const int rows = min(TM, count - m0);
  const int n0 = tile_n * TN;
  const int ncols = min(TN, N - n0);
  const int kvec = Kd / 8;
  uint16_t* y_tile = y + row0 * (size_t)N + n0;
  if constexpr (MX) {
    // rows and weight rows are Kd bytes (Kd / 16 vectors) with Kd / 128 scales; N % 128 == 0
    const u32x4_t* xa = reinterpret_cast<const u32x4_t*>(x) + row0 * (Kd / 16);
    const u32x4_t* wb = reinterpret_cast<const u32x4_t*>(w) + ((size_t)e * N + n0) * (Kd / 16);
    const float* xs = x_scale + row0 * (Kd / 128);
    const int wn = rows > 128 ? (wave & 1) * 128 : wave * 64;  // the wave's columns lie in one scale block
    const int nblk = __builtin_amdgcn_readfirstlane(min(n0 + wn, N - 1) >> 7);
    const float* wsc = w_scale + ((size_t)e * (N / 128) + nblk) * (Kd / 128);
    if (rows > 128)
      wide_tile<E, 4, 4, 256, false, false, true>(xa, xs, wb, wsc, y_tile, s_wide, rows, ncols, Kd / 2, N, (wave >> 1) * 128, wn);
    else
      wide_tile<E, 4, 2, 128, false, false, true>(xa, xs, wb, wsc, y_tile, s_wide, rows, ncols, Kd / 2, N, 0, wn);
  } else {
    // fp8 rows are Kd bytes (Kd / 16 vectors) with Kd / 128 scales each
    const u32x4_t* xa = reinterpret_cast<const u32x4_t*>(x) + row0 * (AFP8 ? Kd / 16 : kvec);
    const float* xs = AFP8 ? x_scale + row0 * (Kd / 128) : nullptr;
    const u32x4_t* wb = reinterpret_cast<const u32x4_t*>(w) + ((size_t)e * N + n0) * (BFP8 ? Kd / 16 : kvec);
    // block-quantised weights: N % 128 == 0, the tile's first column block is n0 / 128
    const float* wsc = BFP8 ? w_scale + ((size_t)e * (N / 128) + n0 / 128) * (Kd / 128) : nullptr;
    // A segment's last tile is often less than half full (23 % of the MFMAs of a 512-rows-per-expert
    // ragged input would be spent on rows that do not exist): up to 128 rows the four waves stand
    // side by side on 128 x 64 each, and only 128 rows of A are staged.
    if (rows > 128)
      wide_tile<E, 4, 4, 256, AFP8, BFP8>(xa, xs, wb, wsc, y_tile, s_wide, rows, ncols, Kd, N, (wave >> 1) * 128, (wave & 1) * 128);
    else
      wide_tile<E, 4, 2, 128, AFP8, BFP8>(xa, xs, wb, wsc, y_tile, s_wide, rows, ncols, Kd, N, 0, wave * 64);
  }
}

// Both operands quantised: rows as the fp8 dispatch writes them (e4m3fn bytes + one f32 scale per
// row and 128 columns), weights in the checkpoint block format (e4m3fn bytes + one f32 scale per
// 128 x 128 block).  The bytes of both go to the matrix cores as they are, on
// v_mfma_f32_32x32x64_f8f6f4 (fp8 x fp8 -> f32, twice the rate of the 16-bit instruction and half
// the LDS bytes per product), and the scales are applied where the format puts them: K advances
// one 128-wide block per slab, the slab's products are summed into a partial accumulator, and the
// partial is folded into the result with one fma per element,
//   acc[r][n] += (x_scale[r][kb] * w_scale[n / 128][kb]) * partial[r][n].
// 128 x 128 output tile (one weight scale per slab and workgroup), four waves of 64 x 64, a slab is
// 128 + 128 rows of 128 bytes in LDS (row stride 144 bytes: the 16-byte reads of consecutive rows
// fall on disjoint banks), the next slab is fetched into registers while this one is multiplied.
// A lane's fragment is 32 consecutive bytes of a row, the same bytes for both operands, so the
// order in which the instruction walks K inside a fragment does not matter.  The weights are the
// instruction's first operand: the result block is transposed, every accumulator element of a lane
// belongs to the same row of x, and the fold needs one scale per lane and row block.
constexpr int kF8M = 128, kF8K = 128, kF8Ld = kF8K + 16;
constexpr int kXcds = 8;  // accelerator dies of an MI355X; workgroup b runs on die b % 8

__device__ __forceinline__ f32x16_t mfma_32x32x64_fp8(const i32x8_t& a, const i32x8_t& b, const f32x16_t& c) {
  // formats 0 / 0 = e4m3 for both operands; the block exponents of the scaled form are 127 = 2^0
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, 127);
}

template <class E, int TN>
__global__ __launch_bounds__(2 * TN, TN == 128 ? 2 : 1) void expert_gemm_f8_kernel(const uint4* __restrict__ x_q,
                                                                       const float* __restrict__ x_scale,
                                                                       const uint4* __restrict__ w_q,
                                                                       const float* __restrict__ w_scale,
                                                                       const int32_t* __restrict__ offsets,
                                                                       uint16_t* __restrict__ y, int num_experts,
                                                                       int Kd, int N, int max_recv, int ntile_n) {
  constexpr int TM = kF8M, BK = kF8K, LD = kF8Ld, NT = 2 * TN;  // a wave per 64 x 64 corner of the tile
  constexpr int NA = TM * 8 / NT, NB = TN * 8 / NT;               // vectors of a slab per thread
  __shared__ __attribute__((aligned(16))) uint8_t s_ab8[(TM + TN) * LD];  // the slab
  __shared__ __attribute__((aligned(16))) float s_sx[TM];                 // its row scales
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[NT / kWave + 1];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;

  // (expert, m-tile, n-tile) of this workgroup: m-tiles of all experts numbered in expert order.
  // Workgroups go to the chip's eight XCDs round-robin (blockIdx % 8), each with its own L2; every
  // XCD takes one contiguous eighth of the m-tiles with all their n-tiles, so the 128 rows of x
  // of an m-tile are fetched into one L2 only, and so are the weights of an expert whose m-tiles
  // are neighbours (this launch is bound by what the L2s miss, not by the matrix cores).
  const int xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
  const int tile_n = slot % ntile_n;
  const int tile_m_local = slot / ntile_n;
  int chunk;
  {
    const int span = (num_experts + NT - 1) / NT;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    chunk = (total + kXcds - 1) / kXcds;
    if (tile_m_local >= chunk || xcd * chunk + tile_m_local >= total) return;  // the grid is sized for the worst case
  }
  const int tile_m_global = xcd * chunk + tile_m_local;
  int e_lo = 0, e_hi = num_experts;  // largest e with s_pref[e] <= tile_m_global
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = e_lo;
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * TM;
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;
  const int rows = min(TM, count - m0);
  const int n0 = tile_n * TN;  // N % TN == 0
  const int kvec = Kd / 16, kblk = Kd / BK;

  // global -> register prefetch: a slab is 128 + TN rows of 8 vectors per row, one row scale for
  // each of the first 128 threads, one weight scale (uniform over the wave).  (Two register sets
  // and two LDS buffers, a slab requested two iterations ahead, measured 2 % faster and leave no
  // register for the loop specialisation below.)
  const u32x4_t* xa = reinterpret_cast<const u32x4_t*>(x_q) + row0 * kvec;
  const u32x4_t* wb = reinterpret_cast<const u32x4_t*>(w_q) + ((size_t)e * N + n0) * kvec;
  const float* xs = x_scale + (row0 + min(tid, rows - 1)) * kblk;
  const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;  // this wave's corner of the tile
  // the 128 x 128 block of the weight scales this wave's columns lie in (uniform over the wave)
  const float* ws = w_scale + ((size_t)e * (N / 128) + __builtin_amdgcn_readfirstlane((n0 + wn) >> 7)) * kblk;
  struct Slab {
    u32x4_t a[NA], b[NB];
    float sx, sw;
  };
  Slab r0;
  int offa[NA], offb[NB];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int v = tid + i * NT;
    offa[i] = min(v >> 3, rows - 1) * kvec + (v & 7);  // rows past the segment re-read its last row; their scale is 0
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int v = tid + i * NT;
    offb[i] = (v >> 3) * kvec + (v & 7);
  }
  const int st_off = (tid >> 3) * LD + (tid & 7) * 16;
  const bool row_live = tid < rows;
#define F8_FETCH(S, KB)                                                                      \
  {                                                                                          \
    const int kb_ = min((KB), kblk - 1); /* past the end: the last slab again, never used */ \
    _Pragma("unroll") for (int i = 0; i < NA; ++i) S.a[i] = xa[offa[i] + kb_ * 8];           \
    _Pragma("unroll") for (int i = 0; i < NB; ++i) S.b[i] = wb[offb[i] + kb_ * 8];           \
    S.sx = xs[kb_];                                                                          \
    S.sw = ws[kb_];                                                                          \
  }
#define F8_STASH(S, BUF)                                                                     \
  {                                                                                          \
    uint8_t* sa_ = s_ab8 + (BUF) * (TM + TN) * LD + st_off;                                  \
    _Pragma("unroll") for (int i = 0; i < NA; ++i)                                           \
        *reinterpret_cast<u32x4_t*>(&sa_[i * (NT / 8) * LD]) = S.a[i];                       \
    _Pragma("unroll") for (int i = 0; i < NB; ++i)                                           \
        *reinterpret_cast<u32x4_t*>(&sa_[TM * LD + i * (NT / 8) * LD]) = S.b[i];             \
    if (tid < TM) s_sx[(BUF) * TM + tid] = row_live ? S.sx : 0.f; /* 0 past the segment */   \
  }
  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
  const int fr_a = (wm + (lane & 31)) * LD + (lane >> 5) * 32;
  const int fr_b = (TM + wn + (lane & 31)) * LD + (lane >> 5) * 32;
  // 32-row blocks of this wave that hold rows of the segment: 0, 1 or 2 (uniform over the wave)
  const int live_blocks = __builtin_amdgcn_readfirstlane(min(2, max(0, (rows - wm + 31) / 32)));

#define F8_SLAB(BUF, S, LB)                                                                                     \
  {                                                                                                            \
    const uint8_t* sb_ = s_ab8 + (BUF) * (TM + TN) * LD;                                                       \
    f32x16_t part[2][2];                                                                                       \
    _Pragma("unroll") for (int kk = 0; kk < BK; kk += 64) {                                                    \
      i32x8_t fa[2], fb[2];                                                                                    \
      _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                          \
        const u32x4_t b0 = *reinterpret_cast<const u32x4_t*>(&sb_[fr_b + i * 32 * LD + kk]);                   \
        const u32x4_t b1 = *reinterpret_cast<const u32x4_t*>(&sb_[fr_b + i * 32 * LD + kk + 16]);              \
        fb[i] = i32x8_t{(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3],                                        \
                        (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};                                       \
      }                                                                                                        \
      _Pragma("unroll") for (int i = 0; i < 2; ++i)                                                            \
        if (i < (LB)) { /* blocks of 32 rows past the segment cost no MFMA */                                  \
          const u32x4_t a0 = *reinterpret_cast<const u32x4_t*>(&sb_[fr_a + i * 32 * LD + kk]);                 \
          const u32x4_t a1 = *reinterpret_cast<const u32x4_t*>(&sb_[fr_a + i * 32 * LD + kk + 16]);            \
          fa[i] = i32x8_t{(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3],                                      \
                          (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};                                     \
          _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                                      \
            f32x16_t zero;                                                                                     \
            _Pragma("unroll") for (int q = 0; q < 16; ++q) zero[q] = 0.f;                                      \
            part[i][j] = mfma_32x32x64_fp8(fb[j], fa[i], kk == 0 ? zero : part[i][j]); /* weights x rows^T */  \
          }                                                                                                    \
        }                                                                                                      \
    }                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < 2; ++i)                                                              \
      if (i < (LB)) {                                                                                          \
        /* the lane's row of x: one factor for all 16 elements, row scale x weight scale */                    \
        const float sc = s_sx[(BUF) * TM + wm + i * 32 + (lane & 31)] * S;                                     \
        _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                          \
        _Pragma("unroll") for (int q = 0; q < 16; ++q)                                                         \
            acc[i][j][q] = __builtin_fmaf(part[i][j][q], sc, acc[i][j][q]);                                    \
      }                                                                                                        \
  }

  // Per slab: registers -> LDS, barrier, request the next slab (in flight during the multiplies),
  // multiply and fold, barrier.  The loop exists three times, for waves with two, one and no 32-row
  // block inside the segment (a wave without rows still moves its share of every slab and meets
  // every barrier): at 128 rows per expert on average a third of all 32-row blocks are empty.
#define F8_LOOP(LB)                              \
  for (int kb = 0; kb < kblk; ++kb) {            \
    F8_STASH(r0, 0);                             \
    const float sw = r0.sw;                      \
    __syncthreads();                             \
    F8_FETCH(r0, kb + 1);                        \
    F8_SLAB(0, sw, LB);                          \
    __syncthreads();                             \
  }
  F8_FETCH(r0, 0);
  if (live_blocks == 2) {
    F8_LOOP(2)
  } else if (live_blocks == 1) {
    F8_LOOP(1)
  } else {
    F8_LOOP(0)
  }
#undef F8_LOOP
#undef F8_SLAB
#undef F8_STASH
#undef F8_FETCH

  // The product is formed transposed (weight rows x rows of x), so a lane's accumulator elements
  // all belong to one row of x -- one scale per lane in the fold above -- and element q is column
  // (q / 4) * 8 + (lane / 32) * 4 + q % 4 of the 32-column block: four consecutive columns per
  // group of four elements, one 8-byte store.
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = wm + i * 32 + (lane & 31);
    if (r < rows) {
      uint16_t* y_row = y + (row0 + r) * (size_t)N + n0 + wn + (lane >> 5) * 4;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          *reinterpret_cast<uint2*>(&y_row[j * 32 + g * 8]) =
              make_uint2(E::pack(acc[i][j][4 * g], acc[i][j][4 * g + 1]), E::pack(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]));
    }
  }
}

// Power-of-two scales, slabs travelling memory -> LDS directly.  Ablation of the register-staged
// loop above puts the cost where the slabs enter the CU: with the global loads taken out the same
// loop runs 1.7 times faster, with the LDS stores out as well twice as fast, and its registers
// leave no room to request a slab earlier.  Here a slab is 256 + 256 rows of 64 bytes (one step of
// the fp8 instruction), global_load_lds (16 bytes per lane, 1 KB = 16 rows per wave instruction)
// puts it into one of four 32 KB buffers, and slab s + 3 is requested while slab s is multiplied:
// no staging registers, no LDS store instructions, three slabs in flight.  Rows of 64 bytes cannot
// be padded, so the 16-byte chunk c of row r sits at chunk position c ^ ((r / 2) % 4): the reads
// of eight consecutive rows then fall on disjoint banks.  The four buffers are separate arrays and
// the loop is unrolled four times, so the compiler knows which buffer a read touches and does not
// wait for the loads in flight to the others.  One barrier per slab, at its top; the sixteen MFMAs
// hide the fragment reads of the next slab and the issue of the loads.
constexpr int kMxdThreads = 256, kMxdSlab = (256 + 256) * 64;

template <class E>
__global__ __launch_bounds__(kMxdThreads) void expert_gemm_mxd_kernel(const uint4* __restrict__ x_q,
                                                                      const float* __restrict__ x_scale,
                                                                      const uint4* __restrict__ w_q,
                                                                      const float* __restrict__ w_scale,
                                                                      const int32_t* __restrict__ offsets,
                                                                      uint16_t* __restrict__ y, int num_experts,
                                                                      int Kd, int N, int max_recv, int ntile_n) {
  constexpr int TM = 256, TN = 256, NT = kMxdThreads, ROWB = 64;
  __shared__ __attribute__((aligned(1024))) uint8_t s_b0[kMxdSlab];
  __shared__ __attribute__((aligned(1024))) uint8_t s_b1[kMxdSlab];
  __shared__ __attribute__((aligned(1024))) uint8_t s_b2[kMxdSlab];
  __shared__ __attribute__((aligned(1024))) uint8_t s_b3[kMxdSlab];
  __shared__ int s_pref[MOE_A2A_MAX_EXPERTS + 1];
  __shared__ int s_tmp[NT / kWave + 1];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;

  // tile of this workgroup: every XCD (workgroup b runs on XCD b % 8, each with its own L2) takes a
  // contiguous eighth of the m-tiles with all their n-tiles, so the rows of an m-tile are fetched
  // into one L2 only (with the plain n-fastest map this launch reads its operands from memory
  // nine times over)
  const int xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
  const int tile_n = slot % ntile_n;
  const int tile_m_local = slot / ntile_n;
  int tile_m_global;
  {
    const int span = (num_experts + NT - 1) / NT;
    const int lo = min(tid * span, num_experts), hi = min(lo + span, num_experts);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    int total;
    int run = block_exclusive_scan(sum, s_tmp, total);
    for (int e = lo; e < hi; ++e) {
      s_pref[e] = run;
      run += (offsets[e + 1] - offsets[e] + TM - 1) / TM;
    }
    if (tid == 0) s_pref[num_experts] = total;
    __syncthreads();
    const int chunk = (total + kXcds - 1) / kXcds;
    tile_m_global = xcd * chunk + tile_m_local;
    if (tile_m_local >= chunk || tile_m_global >= total) return;  // the grid is sized for the worst case
  }
  int e_lo = 0, e_hi = num_experts;
  while (e_hi - e_lo > 1) {
    int mid = (e_lo + e_hi) >> 1;
    if (s_pref[mid] <= tile_m_global) e_lo = mid; else e_hi = mid;
  }
  const int e = e_lo;
  const int count = offsets[e + 1] - offsets[e];
  const int m0 = (tile_m_global - s_pref[e]) * TM;
  const size_t row0 = (size_t)(max_recv > 0 ? e * max_recv : offsets[e]) + m0;
  const int rows = min(TM, count - m0);
  const int n0 = tile_n * TN;
  const int ncols = min(TN, N - n0);
  const int kvec = Kd / 16, kblk = Kd / 128, nslab = Kd / ROWB;

  // waves 0, 1 bring in the rows of x, waves 2, 3 the weight rows: eight instructions of sixteen
  // rows per wave and slab; lane l fills row l / 4, chunk position l % 4 of its kilobyte
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const u32x4_t* gsrc = wave < 2 ? reinterpret_cast<const u32x4_t*>(x_q) + row0 * kvec
                                 : reinterpret_cast<const u32x4_t*>(w_q) + ((size_t)e * N + n0) * kvec;
  const int limit = wave < 2 ? rows : ncols;  // rows past the end re-read the last one: never stored
  int goff[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int r = (wave & 1) * 128 + t * 16 + (lane >> 2);
    goff[t] = min(r, limit - 1) * kvec + ((lane & 3) ^ ((r >> 1) & 3));
  }
  const int lds_wave = wave * 8 * 1024;  // x rows are the first 16 KB of a buffer, weight rows the second
#define MXD_ISSUE(S, BUFP)                                                                                   \
  {                                                                                                          \
    const int s_ = min((S), nslab - 1); /* past the end: the last slab again, into a buffer nobody reads */  \
    _Pragma("unroll") for (int t = 0; t < 8; ++t)                                                            \
        __builtin_amdgcn_global_load_lds((gptr_t)(gsrc + goff[t] + s_ * 4), (lptr_t)(BUFP + lds_wave + t * 1024), \
                                         16, 0, 0);                                                          \
  }
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
  // Scales: the exponent fields go to the instruction.  The row scales of a 128-wide block (two
  // slabs) travel memory -> LDS as well, one float per row (a vector load into registers here
  // would make the compiler wait for every load in flight whenever its value is used): wave w
  // fetches rows 64 w .. 64 w + 63, two blocks ahead, into the array of the block's parity; a
  // lane reads the four it needs (row lane % 32 of its wave's four 32-row blocks) one step before
  // the block starts.  The weight scale is uniform over the wave: a scalar load.
  __shared__ __attribute__((aligned(256))) float s_sc0[TM];
  __shared__ __attribute__((aligned(256))) float s_sc1[TM];
  const float* xs = x_scale + (row0 + min(wave * 64 + lane, rows - 1)) * kblk;
  const float* wsc = w_scale + ((size_t)e * (N / 128) + __builtin_amdgcn_readfirstlane(min(n0 + wn, N - 1) >> 7)) * kblk;
  int sa_cur[4], sa_nxt[4], sb_cur, sb_nxt;
#define MXD_SCALES_ISSUE(KB, SCP) \
  __builtin_amdgcn_global_load_lds((gptr_t)(xs + min((KB), kblk - 1)), (lptr_t)(SCP + wave * 64), 4, 0, 0);
#define MXD_SCALES_READ(KB, SCP, SA, SB)                                                                     \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                            \
        SA[i] = (__float_as_int(SCP[wm + i * 32 + (lane & 31)]) >> 23) & 0xff;                               \
    SB = (__float_as_int(wsc[min((KB), kblk - 1)]) >> 23) & 0xff;                                            \
  }
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
  // fragment of a lane: row lane % 32 of a block, chunks 2 h and 2 h + 1 of the four, h = lane / 32,
  // at their swizzled positions ((row / 2) % 4 == (lane / 2) % 4: blocks start at multiples of 32)
  const int sw = (lane >> 1) & 3;
  const int p0 = (((lane >> 5) * 2) ^ sw) * 16, p1 = (((lane >> 5) * 2 + 1) ^ sw) * 16;
  const int fr_a = (wm + (lane & 31)) * ROWB, fr_b = (TM + wn + (lane & 31)) * ROWB;
  i32x8_t pa[4], pb[4], qa[4], qb[4];
#define MXD_LOAD8(DST, PTR)                                                                                  \
  {                                                                                                          \
    const u32x4_t lo_ = *reinterpret_cast<const u32x4_t*>(&(PTR)[p0]);                                       \
    const u32x4_t hi_ = *reinterpret_cast<const u32x4_t*>(&(PTR)[p1]);                                       \
    DST = i32x8_t{(int)lo_[0], (int)lo_[1], (int)lo_[2], (int)lo_[3], (int)hi_[0], (int)hi_[1], (int)hi_[2], (int)hi_[3]}; \
  }
#define MXD_FRAGS(FA, FB, BUFP)                                                                              \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) MXD_LOAD8(FA[i], BUFP + fr_a + i * 32 * ROWB);             \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) MXD_LOAD8(FB[j], BUFP + fr_b + j * 32 * ROWB);             \
  }
#define MXD_MMA(FA, FB, I0, I1)                                                                              \
  {                                                                                                          \
    _Pragma("unroll") for (int i = (I0); i < (I1); ++i)                                                      \
    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                            \
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FA[i], FB[j], acc[i][j], 0, 0, 0, sa_cur[i], 0, \
                                                                    sb_cur);                                 \
  }
  // One slab.  First make sure slab S + 1 has landed for every wave (vmcnt(8): at most the eight
  // load instructions of slab S + 2 are pending; then the barrier -- which also says that every wave
  // has left slab S - 1).  Then the sixteen MFMAs of slab S from the fragments FA / FB, and in their
  // shadow: the request for slab S + 3 into DBUF (the buffer of slab S - 1), one load instruction
  // behind each of the first eight MFMAs (a wave that waits for the address unit to take a load
  // issues nothing else, and an MFMA in flight covers 64 clocks of that); the fragments of slab
  // S + 1 from RBUF into GA / GB, one read behind each MFMA (spread over the whole slab the four
  // waves ask the LDS for half of what it can deliver; packed behind eight MFMAs it was all of
  // it).  PRE and POST are the scale traffic of even steps.
#define MXD_STEP(S, DBUF, RBUF, FA, FB, GA, GB, PRE, POST)                                                   \
  {                                                                                                          \
    asm volatile("" ::: "memory");                                                                           \
    __builtin_amdgcn_s_waitcnt(0x0F78); /* vmcnt(8) */                                                       \
    __builtin_amdgcn_s_barrier();                                                                            \
    asm volatile("" ::: "memory");                                                                           \
    __builtin_amdgcn_sched_barrier(0);                                                                       \
    PRE;                                                                                                     \
    MXD_ISSUE((S) + 3, DBUF);                                                                                \
    MXD_FRAGS(GA, GB, RBUF);                                                                                 \
    POST;                                                                                                    \
    MXD_MMA(FA, FB, 0, 4);                                                                                   \
    _Pragma("unroll") for (int s_ = 0; s_ < 8; ++s_) {                                                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                     \
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                                                     \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                     \
    }                                                                                                        \
    _Pragma("unroll") for (int s_ = 0; s_ < 8; ++s_) {                                                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                     \
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                                                     \
    }                                                                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                                       \
  }
  MXD_SCALES_ISSUE(0, s_sc0);
  MXD_SCALES_ISSUE(1, s_sc1);
  MXD_ISSUE(0, s_b0);
  MXD_ISSUE(1, s_b1);
  MXD_ISSUE(2, s_b2);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16): the scales of blocks 0 and 1 and slab 0 are in
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  MXD_SCALES_READ(0, s_sc0, sa_cur, sb_cur);
  MXD_FRAGS(pa, pb, s_b0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave has read the scales of block 0 ...
  __builtin_amdgcn_s_barrier();        // ... and so has every other: the first step may overwrite them
  asm volatile("" ::: "memory");
  // A 128-wide scale block is two slabs.  On the first slab of block b the scales of block b + 2
  // are requested (into the array block b used: every wave read it a barrier ago) and those of
  // block b + 1 are read (they were requested two steps earlier and have landed with this step's
  // wait); after its second slab they become current.  Kd is a multiple of 256 here, so the
  // number of slabs is a multiple of four.
#pragma clang loop unroll(disable)
  for (int s = 0; s < nslab; s += 4) {
    MXD_STEP(s, s_b3, s_b1, pa, pb, qa, qb, MXD_SCALES_ISSUE(s / 2 + 2, s_sc0),
             MXD_SCALES_READ(s / 2 + 1, s_sc1, sa_nxt, sb_nxt));
    MXD_STEP(s + 1, s_b0, s_b2, qa, qb, pa, pb, , );
#pragma unroll
    for (int i = 0; i < 4; ++i) sa_cur[i] = sa_nxt[i];
    sb_cur = sb_nxt;
    MXD_STEP(s + 2, s_b1, s_b3, pa, pb, qa, qb, MXD_SCALES_ISSUE(s / 2 + 3, s_sc1),
             MXD_SCALES_READ(s / 2 + 2, s_sc0, sa_nxt, sb_nxt));
    MXD_STEP(s + 3, s_b2, s_b0, qa, qb, pa, pb, , );
#pragma unroll
    for (int i = 0; i < 4; ++i) sa_cur[i] = sa_nxt[i];
    sb_cur = sb_nxt;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing may land after the LDS is given back
#undef MXD_ISSUE
#undef MXD_SCALES_ISSUE
#undef MXD_SCALES_READ
#undef MXD_FRAGS
#undef MXD_LOAD8
#undef MXD_MMA
#undef MXD_STEP

  uint16_t* y_tile = y + row0 * (size_t)N + n0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int r = wm + i * 32 + (q >> 2) * 8 + (lane >> 5) * 4 + (q & 3);
        const int c = wn + j * 32 + (lane & 31);
        if (r < rows && c < ncols) y_tile[r * (size_t)N + c] = (uint16_t)(E::pack(acc[i][j][q], 0.f) & 0xffffu);
      }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
struct LaunchTimer {
  bool active = false;
  int capacity = 0;
  int used = 0;
  hipEvent_t* start = nullptr;
  hipEvent_t* stop = nullptr;
  int* ids = nullptr;
};
LaunchTimer g_timer;

template <typename T>
struct same_type {
  typedef T type;
};

// Arguments are converted to the kernel's own parameter types before they are packed.
template <typename... KArgs>
int launch(int kid, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
           typename same_type<KArgs>::type... args) {
  if (g_timer.active && g_timer.used < g_timer.capacity) {
    int n = g_timer.used++;
    g_timer.ids[n] = kid;
    hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, g_timer.start[n], g_timer.stop[n], 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
  }
  return (int)hipGetLastError();
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int check_route_shape(int T, int K, int E, int W) {
  if (T < 0 || K < 1 || K > MOE_A2A_MAX_TOPK || E < 1 || E > MOE_A2A_MAX_EXPERTS || W < 1 ||
      W > MOE_A2A_MAX_WORLD || E % W != 0)
    return MOE_A2A_E_SHAPE;
  if ((long long)T * K > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  return 0;
}

int id_bits(int E) {
  int b = 0;
  while ((1 << b) < E) ++b;
  return b;
}

// column split of a row of nvec lanes; `unit` lanes must stay in one workgroup
struct RowGeom {
  int per, nsplit, threads;
};
RowGeom row_geom(int nvec, int unit = 1, int max_threads = kRowMaxThreads, int min_threads = kWave) {
  RowGeom g;
  g.nsplit = ceil_div(nvec, max_threads);
  g.per = ceil_div(ceil_div(nvec, g.nsplit), unit) * unit;
  g.threads = ceil_div(g.per, kWave) * kWave;
  if (g.threads < min_threads) g.threads = min_threads;  // extra lanes only help with index work
  return g;
}

// Combine at cache-resident sizes: about four workgroups per CU (1024 in all) finish sooner than
// fewer, wider ones (256 tokens of 896 vectors: 4 x 224 lanes 6.4 us, 2 x 448 lanes 6.7 us); a
// workgroup keeps at least 128 lanes.  Streaming sizes keep the widest workgroups (512 lanes).
RowGeom combine_geom_resident(int nvec, int T) {
  int nsplit = ceil_div(1024, T > 0 ? T : 1);
  if (nsplit > nvec / 128) nsplit = nvec / 128;
  const int least = ceil_div(nvec, kRowMaxThreads);
  if (nsplit < least) nsplit = least;
  RowGeom g;
  g.nsplit = nsplit;
  g.per = ceil_div(nvec, nsplit);
  g.threads = ceil_div(g.per, kWave) * kWave;
  return g;
}

template <typename F>
void set_max_lds(F kernel, size_t bytes) {
  if (bytes > 48 * 1024)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)bytes);
}

}  // namespace

extern "C" {

int moe_a2a_abi_version(void) { return MOE_A2A_ABI_VERSION; }

const char* moe_a2a_strerror(int code) {
  switch (code) {
    case 0: return "success";
    case MOE_A2A_E_NULL: return "moe_a2a: a required pointer is NULL";
    case MOE_A2A_E_SHAPE: return "moe_a2a: T, K, E, W or H out of range or not divisible as required";
    case MOE_A2A_E_DTYPE: return "moe_a2a: unknown element type, stub kind or combine mode";
    case MOE_A2A_E_WORKSPACE: return "moe_a2a: workspace missing or too small";
    case MOE_A2A_E_ALIGN: return "moe_a2a: row buffer not 16-byte aligned";
    case MOE_A2A_E_STATE: return "moe_a2a: launch timer used out of order";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "moe_a2a: unknown error";
}

size_t moe_a2a_workspace_bytes(int T, int K, int E) {
  if (T < 0 || K < 1 || E < 1) return 0;
  long long R = (long long)T * K;
  if (R <= kRouteTilesMaxRows) return 256;
  long long ntiles = (R + kRouteThreads - 1) / kRouteThreads;
  return align_up((size_t)ntiles * (size_t)E * sizeof(int32_t), 256);
}

int moe_a2a_route(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                  int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot,
                  int32_t* meta, int32_t* status, void* workspace, size_t workspace_bytes,
                  moe_a2a_stream_t stream_) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (max_recv < 0 || (long long)max_recv * E > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), max_recv, counts, offsets,
              slot_of_entry, src_of_slot, meta, status};
  const size_t lds_w = (size_t)kRouteWaves * E * sizeof(int);
  const size_t lds_starts = (size_t)(W + 1) * sizeof(int);
  if (a.R <= kRouteTilesMaxRows) {
    size_t lds = lds_w + 2 * (size_t)E * sizeof(int) + (kRouteWaves + 1) * sizeof(int) + lds_starts;
    set_max_lds(route_tiles_kernel, lds);
    return launch(KID_ROUTE_TILES, route_tiles_kernel, dim3(a.R ? ceil_div(a.R, kRouteThreads) : 1),
                  dim3(kRouteThreads), lds, stream, a);
  }
  if (!workspace || workspace_bytes < moe_a2a_workspace_bytes(T, K, E)) return MOE_A2A_E_WORKSPACE;
  int ntiles = ceil_div(a.R, kRouteThreads);
  int32_t* tile = (int32_t*)workspace;
  set_max_lds(route_hist_kernel, lds_w);
  if (int rc = launch(KID_ROUTE_HIST, route_hist_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w, stream, a, tile))
    return rc;
  if (ntiles <= kRouteFoldMaxTiles) {  // scan folded into the rank launch
    set_max_lds(route_rank_fold_kernel, lds_w + lds_starts);
    return launch(KID_ROUTE_RANK, route_rank_fold_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w + lds_starts,
                  stream, a, (const int32_t*)tile, ntiles);
  }
  if (int rc = launch(KID_ROUTE_SCAN, route_scan_kernel, dim3(1), dim3(kRouteThreads), 0, stream, tile, E, ntiles,
                      counts, offsets))
    return rc;
  set_max_lds(route_rank_kernel, lds_w + lds_starts);
  return launch(KID_ROUTE_RANK, route_rank_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w + lds_starts, stream, a,
                (const int32_t*)tile);
}

static int check_rows(const void* a, const void* b, int T, int K, int H, int mult) {
  if (T < 0 || K < 1 || K > MOE_A2A_MAX_TOPK || H < mult || H % mult != 0) return MOE_A2A_E_SHAPE;
  if ((long long)T * K > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  // one workgroup per (row, column split) and one more: the grid has to hold them
  if (((long long)T + 1) * (ceil_div(H / 8, kWave) + 1) > (long long)INT32_MAX) return MOE_A2A_E_SHAPE;
  if (T > 0 && (!a || !b)) return MOE_A2A_E_NULL;
  if (!aligned16(a) || !aligned16(b)) return MOE_A2A_E_ALIGN;
  return 0;
}

// bytes a row kernel moves decide its cache policy (see load_row / store_row)
#ifndef MOE_A2A_STREAM_BYTES
#define MOE_A2A_STREAM_BYTES (192ll << 20)
#endif
static bool streams(long long rows_in, long long rows_out, int H, int in_bytes, int out_bytes) {
  return (rows_in * in_bytes + rows_out * out_bytes) * (long long)H > MOE_A2A_STREAM_BYTES;
}

int moe_a2a_dispatch(const void* x, const int32_t* slot_of_entry, void* disp_x, int T, int K, int H,
                     moe_a2a_stream_t stream_) {
  if (int rc = check_rows(x, disp_x, T, K, H, 8)) return rc;
  if (T == 0) return 0;
  if (!slot_of_entry) return MOE_A2A_E_NULL;
  const int nvec = H / 8;
  const RowGeom g = row_geom(nvec);
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
  if (streams(T, (long long)T * K, H, 2, 2))
    return launch(KID_DISPATCH, dispatch_rows_kernel<1>, grid, block, 0, (hipStream_t)stream_, (const uint4*)x,
                  slot_of_entry, (uint4*)disp_x, K, nvec, g.per, g.nsplit);
  return launch(KID_DISPATCH, dispatch_rows_kernel<0>, grid, block, 0, (hipStream_t)stream_, (const uint4*)x,
                slot_of_entry, (uint4*)disp_x, K, nvec, g.per, g.nsplit);
}

int moe_a2a_fused_max_rows(void) { return INT32_MAX / 8; }

// Geometry of the fused kernel: lanes of a workgroup and row vectors per lane.
static int fused_vectors_per_lane(int nvec) { return nvec >= 768 ? 2 : 1; }
static RowGeom fused_geom(int nvec, int R = 0) {
  RowGeom g = row_geom(ceil_div(nvec, fused_vectors_per_lane(nvec)), 1, kFusedMaxThreads, 256);
  // up to two more waves (they hold table entries only) if that brings the table down to four
  // entries per thread: half the compares per wave, measured 7.3 against 7.5 us at 2048 entries
  const int want = ceil_div(ceil_div(R, 4), kWave) * kWave;
  if (want > g.threads && want <= g.threads + 2 * kWave && want <= kFusedMaxThreads) g.threads = want;
  return g;
}

// Table entries each thread of the fused kernel holds: the smallest of 4, 8, 16, 24, 32 that covers
// R entries with `threads` threads, 0 when even 32 do not.
static int fused_entries_per_thread(int R, int threads) {
  for (int ept : {4, 8, 16, 24, 32})
    if ((long long)threads * ept >= R) return ept;
  return 0;
}

// The one-token-per-workgroup kernel: small tables only.
static bool fused_small_ok(int T, int K, int H) {
  if (T < 1 || K < 1 || H < 8) return false;
  const long long R = (long long)T * K;
  if (R > kFusedMaxRows) return false;
  const RowGeom g = fused_geom(H / 8, (int)R);
  if (fused_entries_per_thread((int)R, g.threads) == 0) return false;
  // every workgroup reads the whole routing table (from L2): keep that traffic below the payload
  return R * T * g.nsplit <= kFusedMaxTableReads;
}

// Tokens per workgroup of the tile kernel: at most kTileMaxOwn entries per tile; enough tokens that
// the table passes of all workgroups together read at most a quarter of the bytes the dispatch
// writes ((T / tile) * R * 4 <= R * H * 2 / 4, i.e. tile >= 8 T / H); otherwise as few as possible
// (more workgroups).
static int tile_tokens(int T, int K, int H) {
  const int cap = kTileMaxOwn / K > 0 ? kTileMaxOwn / K : 1;
  int tile = ceil_div((int)std::min<long long>(8ll * T, INT32_MAX), H);
  if (tile < 1) tile = 1;
  return tile < cap ? tile : cap;
}

int moe_a2a_fused_ok(int T, int K, int H) {
  if (T < 1 || K < 1 || K > kTileMaxOwn || H < 8) return 0;
  if (fused_small_ok(T, K, H)) return 1;
  // Token tiles pay off while the rows stay cache-resident (measured: 26 against 35 us at 134 MB of
  // rows, 151 against 110 us at 537 MB); the streaming sizes keep separate routing and dispatch.
  if (streams(T, (long long)T * K, H, 2, 2)) return 0;
  // ... and while a tile of at most kTileMaxOwn entries still keeps the table passes of all
  // workgroups together below the bytes the dispatch writes: (T / tile) * R * 4 <= R * H * 2
  return (long long)tile_tokens(T, K, H) * H >= 2ll * T ? 1 : 0;
}

int moe_a2a_route_dispatch(const void* x, const int32_t* indices, const int32_t* rank_start, int src_rank, int T,
                           int K, int E, int W, int H, int max_recv, int32_t* counts, int32_t* offsets,
                           int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta, int32_t* status,
                           void* disp_x, moe_a2a_stream_t stream_) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (max_recv < 0 || (long long)max_recv * E > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(x, disp_x, T, K, H, 8)) return rc;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), max_recv, counts, offsets,
              slot_of_entry, src_of_slot, meta, status};
  const int nvec = H / 8;
  const char* force_tile = getenv("MOE_A2A_ROUTE_TILE");  // tuning aid: 1 forces the token-tile kernel
  if (!fused_small_ok(T, K, H) || (force_tile && atoi(force_tile) == 1)) {  // token tiles: any table size
    if (T == 0) return moe_a2a_route(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets,
                                     slot_of_entry, src_of_slot, meta, status, nullptr, 0, stream_);
    if (K > kTileMaxOwn) return MOE_A2A_E_SHAPE;
    const int tile = tile_tokens(T, K, H);
    dim3 grid((unsigned)ceil_div(T, tile)), block(kTileThreads);
    if (streams(T, (long long)T * K, H, 2, 2))
      return launch(KID_ROUTE_DISPATCH_TILE, route_dispatch_tile_kernel<1>, grid, block, 0, (hipStream_t)stream_, a,
                    (const uint4*)x, (uint4*)disp_x, nvec, tile);
    return launch(KID_ROUTE_DISPATCH_TILE, route_dispatch_tile_kernel<0>, grid, block, 0, (hipStream_t)stream_, a,
                  (const uint4*)x, (uint4*)disp_x, nvec, tile);
  }
  const RowGeom g = fused_geom(nvec, T * K);
  const int vpl = fused_vectors_per_lane(nvec);
  const int ept = fused_entries_per_thread(T * K, g.threads);
  if (ept == 0) return MOE_A2A_E_SHAPE;
  dim3 grid((unsigned)T * g.nsplit + 1), block(g.threads);
#define CALL_FUSED3(EPT, PAD, VPL)                                                                             \
  return launch(KID_ROUTE_DISPATCH, route_dispatch_kernel<EPT, PAD, VPL>, grid, block, 0, (hipStream_t)stream_, a, \
                (const uint4*)x, (uint4*)disp_x, nvec, g.per, g.nsplit)
#define CALL_FUSED(EPT)                                                                                        \
  {                                                                                                            \
    if (max_recv > 0) {                                                                                        \
      if (vpl == 2) CALL_FUSED3(EPT, true, 2);                                                                 \
      CALL_FUSED3(EPT, true, 1);                                                                               \
    }                                                                                                          \
    if (vpl == 2) CALL_FUSED3(EPT, false, 2);                                                                  \
    CALL_FUSED3(EPT, false, 1);                                                                                \
  }
  if (ept == 4) CALL_FUSED(4);
  if (ept == 8) CALL_FUSED(8);
  if (ept == 16) CALL_FUSED(16);
  if (ept == 24) CALL_FUSED(24);
  CALL_FUSED(32);
#undef CALL_FUSED3
#undef CALL_FUSED
}

int moe_a2a_dispatch_fp8(const void* x, int x_type, const int32_t* slot_of_entry, uint8_t* disp_q,
                         float* disp_scale, int T, int K, int H, int scale_mode, moe_a2a_stream_t stream_) {
  if (x_type != MOE_A2A_F16 && x_type != MOE_A2A_BF16) return MOE_A2A_E_DTYPE;
  if (scale_mode != MOE_A2A_FP8_SCALE_F32 && scale_mode != MOE_A2A_FP8_SCALE_POW2) return MOE_A2A_E_DTYPE;
  const int pow2 = scale_mode == MOE_A2A_FP8_SCALE_POW2;
  if (int rc = check_rows(x, disp_q, T, K, H, MOE_A2A_FP8_BLOCK)) return rc;
  if (T == 0) return 0;
  if (!slot_of_entry || !disp_scale) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int nblk = H / MOE_A2A_FP8_BLOCK;
  const RowGeom g = row_geom(nblk * 8, 8);
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
  const bool st = streams(T, (long long)T * K, H, 2, 1);
#define FP8_LAUNCH(EL, ST)                                                                                       \
  return launch(KID_DISPATCH_FP8, dispatch_fp8_kernel<EL, ST>, grid, block, 0, stream, (const uint4*)x, slot_of_entry, \
                (uint4*)disp_q, disp_scale, K, nblk, g.per, g.nsplit, pow2)
  if (x_type == MOE_A2A_BF16) {
    if (st) FP8_LAUNCH(Bf16, 1);
    FP8_LAUNCH(Bf16, 0);
  }
  if (st) FP8_LAUNCH(F16, 1);
  FP8_LAUNCH(F16, 0);
#undef FP8_LAUNCH
}

static bool known_type(int t) { return t == MOE_A2A_F16 || t == MOE_A2A_BF16; }

int moe_a2a_stub(const void* disp, const float* disp_scale, const int32_t* meta, const int32_t* rows, int in_type,
                 int out_type, int stub_kind, int E, int W, void* y, int R, int H, moe_a2a_stream_t stream_) {
  if (!known_type(out_type) || (!disp_scale && !known_type(in_type))) return MOE_A2A_E_DTYPE;
  if (stub_kind != MOE_A2A_STUB_OWNER_RANK && stub_kind != MOE_A2A_STUB_EXPERT_FRACTION) return MOE_A2A_E_DTYPE;
  if (E < 1 || W < 1 || E % W != 0 || R < 0) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(disp, y, R, 1, H, disp_scale ? MOE_A2A_FP8_BLOCK : 8)) return rc;
  if (R == 0) return 0;
  if (!meta) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int E_l = E / W;
  const bool st = streams(R, R, H, disp_scale ? 1 : 2, 2);
  if (disp_scale) {
    const int nvec = H / 8;
    const RowGeom g = row_geom(nvec);
    dim3 grid((unsigned)R * g.nsplit), block(g.threads);
#define STUB8_LAUNCH(OUT, ST)                                                                                   \
  return launch(KID_STUB_FP8, stub_fp8_kernel<OUT, ST>, grid, block, 0, stream, (const uint2*)disp, disp_scale, meta, \
                (uint4*)y, stub_kind, E, E_l, nvec, g.per, g.nsplit, rows)
    if (out_type == MOE_A2A_BF16) {
      if (st) STUB8_LAUNCH(Bf16, 1);
      STUB8_LAUNCH(Bf16, 0);
    }
    if (st) STUB8_LAUNCH(F16, 1);
    STUB8_LAUNCH(F16, 0);
#undef STUB8_LAUNCH
  }
  const int nvec = H / 8;
  const RowGeom g = row_geom(nvec);
  dim3 grid((unsigned)R * g.nsplit), block(g.threads);
#define STUB_LAUNCH(IN, OUT)                                                                                  \
  {                                                                                                           \
    if (st)                                                                                                   \
      return launch(KID_STUB, stub_rows_kernel<IN, OUT, 1>, grid, block, 0, stream, (const uint4*)disp, meta, \
                    (uint4*)y, stub_kind, E, E_l, nvec, g.per, g.nsplit, rows);                               \
    return launch(KID_STUB, stub_rows_kernel<IN, OUT, 0>, grid, block, 0, stream, (const uint4*)disp, meta,   \
                  (uint4*)y, stub_kind, E, E_l, nvec, g.per, g.nsplit, rows);                                 \
  }
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_BF16) STUB_LAUNCH(Bf16, Bf16)
  if (in_type == MOE_A2A_F16 && out_type == MOE_A2A_F16) STUB_LAUNCH(F16, F16)
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_F16) STUB_LAUNCH(Bf16, F16)
  STUB_LAUNCH(F16, Bf16)
#undef STUB_LAUNCH
}

// top-k values with a specialised kernel; any other K takes the generic one (KT = 0)
#define MOE_A2A_SWITCH_KT(K, CALL) \
  switch (K) {                     \
    case 2: CALL(2);               \
    case 4: CALL(4);               \
    case 6: CALL(6);               \
    case 8: CALL(8);               \
    default: CALL(0);              \
  }

int moe_a2a_combine(const void* expert_y, const float* weights, const int32_t* slot_of_entry, int mode,
                    int elem_type, void* out, int T, int K, int H, moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (mode != MOE_A2A_COMBINE_STRICT && mode != MOE_A2A_COMBINE_F32) return MOE_A2A_E_DTYPE;
  if (int rc = check_rows(expert_y, out, T, K, H, 8)) return rc;
  if (T == 0) return 0;
  if (!weights || !slot_of_entry) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int nvec = H / 8;
  const bool st = streams((long long)T * K, T, H, 2, 2);
  const RowGeom g = st ? row_geom(nvec) : combine_geom_resident(nvec, T);
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
#define COMBINE_LAUNCH(EL, MD, KT)                                                                            \
  {                                                                                                           \
    if (st)                                                                                                   \
      return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 1>, grid, block, 0, stream,                  \
                    (const uint4*)expert_y, weights, slot_of_entry, (uint4*)out, K, nvec, g.per, g.nsplit);   \
    return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 0>, grid, block, 0, stream,                    \
                  (const uint4*)expert_y, weights, slot_of_entry, (uint4*)out, K, nvec, g.per, g.nsplit);     \
  }
#define CALL_BS(KT) COMBINE_LAUNCH(Bf16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_BF(KT) COMBINE_LAUNCH(Bf16, MOE_A2A_COMBINE_F32, KT)
#define CALL_HS(KT) COMBINE_LAUNCH(F16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_HF(KT) COMBINE_LAUNCH(F16, MOE_A2A_COMBINE_F32, KT)
  const bool strict = mode == MOE_A2A_COMBINE_STRICT;
  if (elem_type == MOE_A2A_BF16) {
    if (strict) MOE_A2A_SWITCH_KT(K, CALL_BS)
    MOE_A2A_SWITCH_KT(K, CALL_BF)
  }
  if (strict) MOE_A2A_SWITCH_KT(K, CALL_HS)
  MOE_A2A_SWITCH_KT(K, CALL_HF)
#undef CALL_BS
#undef CALL_BF
#undef CALL_HS
#undef CALL_HF
#undef COMBINE_LAUNCH
}

int moe_a2a_stub_combine(const void* disp, const float* disp_scale, const int32_t* indices, const float* weights,
                         const int32_t* slot_of_entry, int mode, int in_type, int out_type, int stub_kind, int E,
                         int W, void* out, int T, int K, int H, moe_a2a_stream_t stream_) {
  if (!known_type(out_type) || (!disp_scale && !known_type(in_type))) return MOE_A2A_E_DTYPE;
  if (mode != MOE_A2A_COMBINE_STRICT && mode != MOE_A2A_COMBINE_F32) return MOE_A2A_E_DTYPE;
  if (stub_kind != MOE_A2A_STUB_OWNER_RANK && stub_kind != MOE_A2A_STUB_EXPERT_FRACTION) return MOE_A2A_E_DTYPE;
  if (E < 1 || W < 1 || E % W != 0) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(disp, out, T, K, H, disp_scale ? MOE_A2A_FP8_BLOCK : 8)) return rc;
  if (T == 0) return 0;
  if (!indices || !weights || !slot_of_entry) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int E_l = E / W;
  const bool strict = mode == MOE_A2A_COMBINE_STRICT;
  const bool st = streams((long long)T * K, T, H, disp_scale ? 1 : 2, 2);
  if (disp_scale) {
    const int nblk = H / MOE_A2A_FP8_BLOCK;
    const RowGeom g = row_geom(nblk * 8);
    dim3 grid((unsigned)T * g.nsplit), block(g.threads);
#define SC8_LAUNCH(OUT, MD, KT)                                                                                 \
  {                                                                                                             \
    if (st)                                                                                                     \
      return launch(KID_STUB_COMBINE, stub_combine_fp8_kernel<OUT, MD, KT, 1>, grid, block, 0, stream,          \
                    (const uint4*)disp, disp_scale, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, \
                    E_l, K, nblk, g.per, g.nsplit);                                                             \
    return launch(KID_STUB_COMBINE, stub_combine_fp8_kernel<OUT, MD, KT, 0>, grid, block, 0, stream,            \
                  (const uint4*)disp, disp_scale, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E,   \
                  E_l, K, nblk, g.per, g.nsplit);                                                               \
  }
#define CALL_BS(KT) SC8_LAUNCH(Bf16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_BF(KT) SC8_LAUNCH(Bf16, MOE_A2A_COMBINE_F32, KT)
#define CALL_HS(KT) SC8_LAUNCH(F16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_HF(KT) SC8_LAUNCH(F16, MOE_A2A_COMBINE_F32, KT)
    if (out_type == MOE_A2A_BF16) {
      if (strict) MOE_A2A_SWITCH_KT(K, CALL_BS)
      MOE_A2A_SWITCH_KT(K, CALL_BF)
    }
    if (strict) MOE_A2A_SWITCH_KT(K, CALL_HS)
    MOE_A2A_SWITCH_KT(K, CALL_HF)
#undef CALL_BS
#undef CALL_BF
#undef CALL_HS
#undef CALL_HF
#undef SC8_LAUNCH
  }
  const int nvec = H / 8;
  const RowGeom g = st ? row_geom(nvec) : combine_geom_resident(nvec, T);
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
#define SC_LAUNCH(IN, OUT, MD, KT)                                                                              \
  {                                                                                                             \
    if (st)                                                                                                     \
      return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD, KT, 1>, grid, block, 0, stream,     \
                    (const uint4*)disp, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, E_l, K,     \
                    nvec, g.per, g.nsplit);                                                                     \
    return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD, KT, 0>, grid, block, 0, stream,       \
                  (const uint4*)disp, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, E_l, K, nvec, \
                  g.per, g.nsplit);                                                                             \
  }
#define CALL_BS(KT) SC_LAUNCH(Bf16, Bf16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_BF(KT) SC_LAUNCH(Bf16, Bf16, MOE_A2A_COMBINE_F32, KT)
#define CALL_HS(KT) SC_LAUNCH(F16, F16, MOE_A2A_COMBINE_STRICT, KT)
#define CALL_HF(KT) SC_LAUNCH(F16, F16, MOE_A2A_COMBINE_F32, KT)
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_BF16) {
    if (strict) MOE_A2A_SWITCH_KT(K, CALL_BS)
    MOE_A2A_SWITCH_KT(K, CALL_BF)
  }
  if (in_type == MOE_A2A_F16 && out_type == MOE_A2A_F16) {
    if (strict) MOE_A2A_SWITCH_KT(K, CALL_HS)
    MOE_A2A_SWITCH_KT(K, CALL_HF)
  }
  // mixed element types: generic kernel only
  if (in_type == MOE_A2A_BF16) {
    if (strict) SC_LAUNCH(Bf16, F16, MOE_A2A_COMBINE_STRICT, 0)
    SC_LAUNCH(Bf16, F16, MOE_A2A_COMBINE_F32, 0)
  }
  if (strict) SC_LAUNCH(F16, Bf16, MOE_A2A_COMBINE_STRICT, 0)
  SC_LAUNCH(F16, Bf16, MOE_A2A_COMBINE_F32, 0)
#undef CALL_BS
#undef CALL_BF
#undef CALL_HS
#undef CALL_HF
#undef SC_LAUNCH
}
#undef MOE_A2A_SWITCH_KT

int moe_a2a_forward(const void* x, const int32_t* indices, const float* weights, const int32_t* rank_start,
                    int src_rank, int T, int K, int E, int W, int H, int max_recv, int in_type, int out_type,
                    int fp8_dispatch, int stub_kind, int combine_mode, int fuse_route, int fuse_stub,
                    int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                    int32_t* status, void* disp, float* disp_scale, void* expert_y, void* out, void* workspace,
                    size_t workspace_bytes, moe_a2a_stream_t stream) {
  if (!known_type(in_type) || !known_type(out_type)) return MOE_A2A_E_DTYPE;
  if (fp8_dispatch < 0 || fp8_dispatch > 2) return MOE_A2A_E_DTYPE;
  if (fp8_dispatch && !disp_scale) return MOE_A2A_E_NULL;
  if (!fuse_stub && T > 0 && !expert_y) return MOE_A2A_E_NULL;
  const bool fused = !fp8_dispatch && T > 0 &&
                     (fuse_route == 2 ? K <= kTileMaxOwn : (fuse_route == 1 && moe_a2a_fused_ok(T, K, H)));
  if (fused) {
    if (int rc = moe_a2a_route_dispatch(x, indices, rank_start, src_rank, T, K, E, W, H, max_recv, counts, offsets,
                                        slot_of_entry, src_of_slot, meta, status, disp, stream))
      return rc;
  } else {
    if (int rc = moe_a2a_route(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry,
                               src_of_slot, meta, status, workspace, workspace_bytes, stream))
      return rc;
    if (int rc = fp8_dispatch ? moe_a2a_dispatch_fp8(x, in_type, slot_of_entry, (uint8_t*)disp, disp_scale, T, K, H,
                                                     fp8_dispatch == 2 ? MOE_A2A_FP8_SCALE_POW2
                                                                       : MOE_A2A_FP8_SCALE_F32,
                                                     stream)
                              : moe_a2a_dispatch(x, slot_of_entry, disp, T, K, H, stream))
      return rc;
  }
  const float* scale = fp8_dispatch ? disp_scale : nullptr;
  if (fuse_stub)
    return moe_a2a_stub_combine(disp, scale, indices, weights, slot_of_entry, combine_mode, in_type, out_type,
                                stub_kind, E, W, out, T, K, H, stream);
  // padded layout: the stub visits the rows that hold entries, entry by entry
  if (int rc = moe_a2a_stub(disp, scale, meta, max_recv > 0 ? slot_of_entry : nullptr, in_type, out_type, stub_kind,
                            E, W, expert_y, T * K, H, stream))
    return rc;
  return moe_a2a_combine(expert_y, weights, slot_of_entry, combine_mode, out_type, out, T, K, H, stream);
}

// Launch of the 256 x 256 kernel; x_scale != nullptr selects fp8 rows of x, w_scale != nullptr
// block-quantised weights.
static int launch_gemm_wide(const void* x, const float* x_scale, const void* weights, const float* w_scale,
                            const int32_t* offsets, void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                            hipStream_t stream, bool mx = false) {
  const int ntile_n = ceil_div(N, kWideN);
  const long long mtiles = (long long)R / kWideM + E;  // every expert may end with a partly filled tile
  if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
  dim3 grid((unsigned)(mtiles * ntile_n)), block(kWideThreads);
  // the kernels need more dynamic LDS than the 64 KB default: raised once per device (the
  // attribute belongs to the device's copy of the function); racing first calls only repeat it
  static std::atomic<bool> lds_raised[kMaxDevices];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MOE_A2A_E_STATE;
  if (!lds_raised[dev].load(std::memory_order_acquire)) {
    const void* kernels[10] = {(const void*)expert_gemm_wide_kernel<Bf16, false, false, true>,
                              (const void*)expert_gemm_wide_kernel<F16, false, false, true>,
                              (const void*)expert_gemm_wide_kernel<Bf16, false, false>,
                              (const void*)expert_gemm_wide_kernel<F16, false, false>,
                              (const void*)expert_gemm_wide_kernel<Bf16, true, false>,
                              (const void*)expert_gemm_wide_kernel<F16, true, false>,
                              (const void*)expert_gemm_wide_kernel<Bf16, false, true>,
                              (const void*)expert_gemm_wide_kernel<F16, false, true>,
                              (const void*)expert_gemm_wide_kernel<Bf16, true, true>,
                              (const void*)expert_gemm_wide_kernel<F16, true, true>};
    for (const void* k : kernels) {
      hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLdsBytes);
      if (e != hipSuccess) return (int)e;
    }
    lds_raised[dev].store(true, std::memory_order_release);
  }
#define CALL_WIDE(ET, AF, BF)                                                                                  \
  return launch(KID_EXPERT_GEMM_WIDE, expert_gemm_wide_kernel<ET, AF, BF>, grid, block, kWideLdsBytes, stream, \
                (const uint4*)x, x_scale, (const uint4*)weights, w_scale, offsets, (uint16_t*)y, E, Kd, N,     \
                max_recv, ntile_n)
#define CALL_WIDE_E(ET)                  \
  {                                      \
    if (mx)                                                                                                    \
      return launch(KID_EXPERT_GEMM_MX, expert_gemm_wide_kernel<ET, false, false, true>, grid, block,          \
                    kWideLdsBytes, stream, (const uint4*)x, x_scale, (const uint4*)weights, w_scale, offsets,  \
                    (uint16_t*)y, E, Kd, N, max_recv, ntile_n);                                                \
    if (x_scale && w_scale) CALL_WIDE(ET, true, true);  \
    if (x_scale) CALL_WIDE(ET, true, false);            \
    if (w_scale) CALL_WIDE(ET, false, true);            \
    CALL_WIDE(ET, false, false);                        \
  }
  if (elem_type == MOE_A2A_BF16) CALL_WIDE_E(Bf16);
  CALL_WIDE_E(F16);
#undef CALL_WIDE_E
#undef CALL_WIDE
}

int moe_a2a_expert_gemm(const void* x, const void* weights, const int32_t* offsets, void* y, int R, int E, int Kd,
                        int N, int max_recv, int elem_type, moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (R < 0 || E < 1 || E > MOE_A2A_MAX_EXPERTS || Kd < kGemmK || Kd % kGemmK != 0 || N < 8 || N % 8 != 0 ||
      max_recv < 0)
    return MOE_A2A_E_SHAPE;
  if (R == 0) return 0;
  if (!x || !weights || !offsets || !y) return MOE_A2A_E_NULL;
  if (!aligned16(x) || !aligned16(weights) || !aligned16(y)) return MOE_A2A_E_ALIGN;
  hipStream_t stream = (hipStream_t)stream_;
  // Long segments take the 256 x 256 kernel: with fewer than 256 rows per expert on average most
  // of its tiles would be half empty.  MOE_A2A_GEMM_TILE=32|128|256 in the environment overrides.
  // Short segments (a decode step) take the 32 x 256 kernel, which streams the weights.
  bool wide = (long long)R >= 256ll * E && N >= kWideN;
  bool skinny = (long long)R <= 32ll * E;
  if (const char* forced = getenv("MOE_A2A_GEMM_TILE")) {
    wide = atoi(forced) == 256;
    skinny = atoi(forced) == 32;
  }
  if (Kd % kSkinnyK != 0) skinny = false;  // its K slabs are 128 wide; the 128 x 128 kernel takes the rest
  if (wide) return launch_gemm_wide(x, nullptr, weights, nullptr, offsets, y, R, E, Kd, N, max_recv, elem_type, stream);
  if (skinny) {
    const int ntile_n = ceil_div(N, kSkinnyN);
    const long long mtiles = (long long)R / kSkinnyM + E;
    if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
    dim3 grid((unsigned)(mtiles * ntile_n)), block(kSkinnyThreads);
    if (elem_type == MOE_A2A_BF16)
      return launch(KID_EXPERT_GEMM_SKINNY, expert_gemm_skinny_kernel<Bf16>, grid, block, 0, stream, (const uint4*)x,
                    (const uint4*)weights, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
    return launch(KID_EXPERT_GEMM_SKINNY, expert_gemm_skinny_kernel<F16>, grid, block, 0, stream, (const uint4*)x,
                  (const uint4*)weights, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
  }
  const int ntile_n = ceil_div(N, kGemmN);
  // worst case of m-tiles: every expert ends with a partly filled tile
  const long long mtiles = (long long)R / kGemmM + E;
  if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
  dim3 grid((unsigned)(mtiles * ntile_n)), block(kGemmThreads);
  if (elem_type == MOE_A2A_BF16)
    return launch(KID_EXPERT_GEMM, expert_gemm_kernel<Bf16>, grid, block, 0, stream, (const uint4*)x,
                  (const uint4*)weights, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
  return launch(KID_EXPERT_GEMM, expert_gemm_kernel<F16>, grid, block, 0, stream, (const uint4*)x,
                (const uint4*)weights, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
}

int moe_a2a_expert_gemm_fp8(const void* x_q, const float* x_scale, const void* weights, const int32_t* offsets,
                            void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                            moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (R < 0 || E < 1 || E > MOE_A2A_MAX_EXPERTS || Kd < MOE_A2A_FP8_BLOCK || Kd % MOE_A2A_FP8_BLOCK != 0 || N < 8 ||
      N % 8 != 0 || max_recv < 0)
    return MOE_A2A_E_SHAPE;
  if (R == 0) return 0;
  if (!x_q || !x_scale || !weights || !offsets || !y) return MOE_A2A_E_NULL;
  if (!aligned16(x_q) || !aligned16(weights) || !aligned16(y)) return MOE_A2A_E_ALIGN;
  return launch_gemm_wide(x_q, x_scale, weights, nullptr, offsets, y, R, E, Kd, N, max_recv, elem_type,
                          (hipStream_t)stream_);
}

int moe_a2a_expert_gemm_q8(const void* x, const float* x_scale, const void* w_q, const float* w_scale,
                           const int32_t* offsets, void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                           moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (R < 0 || E < 1 || E > MOE_A2A_MAX_EXPERTS || Kd < MOE_A2A_FP8_BLOCK || Kd % MOE_A2A_FP8_BLOCK != 0 ||
      N < MOE_A2A_FP8_BLOCK || N % MOE_A2A_FP8_BLOCK != 0 || max_recv < 0)
    return MOE_A2A_E_SHAPE;
  if (R == 0) return 0;
  if (!x || !w_q || !w_scale || !offsets || !y) return MOE_A2A_E_NULL;
  if (!aligned16(x) || !aligned16(w_q) || !aligned16(y)) return MOE_A2A_E_ALIGN;
  hipStream_t stream = (hipStream_t)stream_;
  // A decode step streams the weights (32-row tiles); longer segments multiply fp8 by fp8 when the
  // rows are fp8, else on the 256 x 256 kernel, which dequantises the weights on their way into LDS
  // (it needs N >= 256).  MOE_A2A_GEMM_TILE = 32 | 128 | 256 forces one where it applies.
  enum { kStream, kBothFp8, kDequant } kernel;
  if ((long long)R <= 32ll * E) kernel = kStream;
  else if (x_scale) kernel = kBothFp8;
  else kernel = N >= kWideN ? kDequant : kStream;
  if (const char* forced = getenv("MOE_A2A_GEMM_TILE")) {
    const int tile = atoi(forced);
    if (tile == 32) kernel = kStream;
    if (tile == 128 && x_scale) kernel = kBothFp8;
    if (tile == 256 && N >= kWideN) kernel = kDequant;
  }
  if (kernel == kDequant)
    return launch_gemm_wide(x, x_scale, w_q, w_scale, offsets, y, R, E, Kd, N, max_recv, elem_type, stream);
  if (kernel == kBothFp8) {
    // both operands fp8: the bytes go to the matrix cores as they are.  128 x 128 tiles: the
    // 128 x 256 form of the kernel (one workgroup of eight waves per CU) measured slower, 1160
    // against 1140 us at 128 rows per expert and 1030 against 920 us at 512.
    constexpr int tn = 128;
    const int ntile_n = N / tn;
    // worst case of m-tiles (every expert ends with a partly filled one), an eighth of them per XCD
    const long long mtiles = ((long long)R / kF8M + E + kXcds - 1) / kXcds * kXcds;
    if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
    dim3 grid((unsigned)(mtiles * ntile_n)), block(2 * tn);
    if (elem_type == MOE_A2A_BF16)
      return launch(KID_EXPERT_GEMM_F8, expert_gemm_f8_kernel<Bf16, tn>, grid, block, 0, stream, (const uint4*)x,
                    x_scale, (const uint4*)w_q, w_scale, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
    return launch(KID_EXPERT_GEMM_F8, expert_gemm_f8_kernel<F16, tn>, grid, block, 0, stream, (const uint4*)x,
                  x_scale, (const uint4*)w_q, w_scale, offsets, (uint16_t*)y, E, Kd, N, max_recv, ntile_n);
  }
  const int ntile_n = N / 128;
  const long long mtiles = (long long)R / kSkinnyM + E;
  if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
  dim3 grid((unsigned)(mtiles * ntile_n)), block(kSkinnyThreads);
#define CALL_SKQ(ET, AF)                                                                                        \
  return launch(KID_EXPERT_GEMM_SKINNY, expert_gemm_skinny_q_kernel<ET, AF>, grid, block, 0, stream,       \
                (const uint4*)x, x_scale, (const uint4*)w_q, w_scale, offsets, (uint16_t*)y, E, Kd, N, max_recv, \
                ntile_n)
  if (elem_type == MOE_A2A_BF16) {
    if (x_scale) CALL_SKQ(Bf16, true);
    CALL_SKQ(Bf16, false);
  }
  if (x_scale) CALL_SKQ(F16, true);
  CALL_SKQ(F16, false);
#undef CALL_SKQ
}

int moe_a2a_expert_gemm_mx8(const void* x_q, const float* x_scale, const void* w_q, const float* w_scale,
                            const int32_t* offsets, void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                            moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (R < 0 || E < 1 || E > MOE_A2A_MAX_EXPERTS || Kd < MOE_A2A_FP8_BLOCK || Kd % MOE_A2A_FP8_BLOCK != 0 ||
      N < MOE_A2A_FP8_BLOCK || N % MOE_A2A_FP8_BLOCK != 0 || max_recv < 0)
    return MOE_A2A_E_SHAPE;
  if (R == 0) return 0;
  if (!x_q || !x_scale || !w_q || !w_scale || !offsets || !y) return MOE_A2A_E_NULL;
  if (!aligned16(x_q) || !aligned16(w_q) || !aligned16(y)) return MOE_A2A_E_ALIGN;
  // A decode step (R <= 32 E) is bound by the weight bytes: moe_a2a_expert_gemm_q8 streams them, and
  // powers of two are f32 scales like any other.  Otherwise 256 x 256 tiles with the scales as block
  // exponents: slabs sent memory -> LDS directly when Kd is a multiple of 256 (measured against the
  // kernel that folds f32 scales on the vector units: 1022 / 1140 us at 128 rows per expert,
  // 7168 -> 2048; 735 / 923 us and 2592 / 3420 us at 512 rows per expert, 4096 -> 2048 and -> 7168),
  // the register-staged loop for other Kd on long segments (3109 us in the last case), the folding
  // kernel for what is left.  MOE_A2A_GEMM_TILE = 32 | 128 force the streaming / the folding kernel,
  // 256 the tiles; MOE_A2A_MX_STAGED = 1 the register-staged loop.
  enum { kStream, kFold, kTilesDirect, kTilesStaged } kernel;
  const bool staged_only = Kd % 256 != 0 || (getenv("MOE_A2A_MX_STAGED") && atoi(getenv("MOE_A2A_MX_STAGED")) == 1);
  if ((long long)R <= 32ll * E) kernel = kStream;
  else if (!staged_only) kernel = kTilesDirect;
  else kernel = (long long)R >= 256ll * E ? kTilesStaged : kFold;
  if (const char* forced = getenv("MOE_A2A_GEMM_TILE")) {
    const int tile = atoi(forced);
    if (tile == 32) kernel = kStream;
    if (tile == 128) kernel = kFold;
    if (tile == 256) kernel = staged_only ? kTilesStaged : kTilesDirect;
  }
  if (kernel == kStream || kernel == kFold)  // the same environment variable picks between the two there
    return moe_a2a_expert_gemm_q8(x_q, x_scale, w_q, w_scale, offsets, y, R, E, Kd, N, max_recv, elem_type, stream_);
  if (kernel == kTilesDirect) {
    const int ntile_n = ceil_div(N, 256);
    // worst case of m-tiles (every expert ends with a partly filled one), an eighth of them per XCD
    const long long mtiles = ((long long)R / 256 + E + kXcds - 1) / kXcds * kXcds;
    if (mtiles * ntile_n > INT32_MAX) return MOE_A2A_E_SHAPE;
    dim3 grid((unsigned)(mtiles * ntile_n)), block(kMxdThreads);
    if (elem_type == MOE_A2A_BF16)
      return launch(KID_EXPERT_GEMM_MX, expert_gemm_mxd_kernel<Bf16>, grid, block, 0, (hipStream_t)stream_,
                    (const uint4*)x_q, x_scale, (const uint4*)w_q, w_scale, offsets, (uint16_t*)y, E, Kd, N, max_recv,
                    ntile_n);
    return launch(KID_EXPERT_GEMM_MX, expert_gemm_mxd_kernel<F16>, grid, block, 0, (hipStream_t)stream_,
                  (const uint4*)x_q, x_scale, (const uint4*)w_q, w_scale, offsets, (uint16_t*)y, E, Kd, N, max_recv,
                  ntile_n);
  }
  return launch_gemm_wide(x_q, x_scale, w_q, w_scale, offsets, y, R, E, Kd, N, max_recv, elem_type,
                          (hipStream_t)stream_, true);
}

int moe_a2a_timer_begin(int capacity) {
  if (g_timer.active || capacity < 1) return MOE_A2A_E_STATE;
  g_timer.start = new hipEvent_t[capacity];
  g_timer.stop = new hipEvent_t[capacity];
  g_timer.ids = new int[capacity];
  for (int i = 0; i < capacity; ++i) {
    hipError_t e1 = hipEventCreate(&g_timer.start[i]);
    hipError_t e2 = e1 == hipSuccess ? hipEventCreate(&g_timer.stop[i]) : e1;
    if (e2 != hipSuccess) {  // give back what exists: events 0 .. i-1 in pairs, and start[i] if it was made
      if (e1 == hipSuccess) (void)hipEventDestroy(g_timer.start[i]);
      for (int j = 0; j < i; ++j) {
        (void)hipEventDestroy(g_timer.start[j]);
        (void)hipEventDestroy(g_timer.stop[j]);
      }
      delete[] g_timer.start;
      delete[] g_timer.stop;
      delete[] g_timer.ids;
      g_timer = LaunchTimer{};
      return (int)e2;
    }
  }
  g_timer.capacity = capacity;
  g_timer.used = 0;
  g_timer.active = true;
  return 0;
}

int moe_a2a_timer_end(int* kernel_ids, float* microseconds, int n) {
  if (!g_timer.active) return MOE_A2A_E_STATE;
  g_timer.active = false;
  int written = 0;
  for (int i = 0; i < g_timer.used; ++i) {
    (void)hipEventSynchronize(g_timer.stop[i]);
    float ms = 0.f;
    hipError_t e = hipEventElapsedTime(&ms, g_timer.start[i], g_timer.stop[i]);
    if (written < n && kernel_ids && microseconds) {
      kernel_ids[written] = g_timer.ids[i];
      microseconds[written] = e == hipSuccess ? ms * 1000.f : -1.f;
      ++written;
    }
  }
  for (int i = 0; i < g_timer.capacity; ++i) {
    (void)hipEventDestroy(g_timer.start[i]);
    (void)hipEventDestroy(g_timer.stop[i]);
  }
  delete[] g_timer.start;
  delete[] g_timer.stop;
  delete[] g_timer.ids;
  g_timer = LaunchTimer{};
  return written;
}

const char* moe_a2a_kernel_name(int kernel_id) {
  if (kernel_id < 0 || kernel_id >= KID_COUNT) return "unknown";
  return kKernelNames[kernel_id];
}

}  // extern "C"
