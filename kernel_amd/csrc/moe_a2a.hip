// MoE all-to-all dispatch / expert stub / combine for one MI355X (gfx950, wave64).
//
// The W destination ranks of the reference's all-to-all (all2all/reference.py:68-234) are
// partitions of one compact expert-major buffer, so an "exchange" is only the choice of a
// destination row.  Everything here is HBM-bound integer/byte work: no MFMA, 16-byte
// vector loads and stores, LDS for counters and index tiles, ballot/popcount for ranks.
//
// Kernels
//   route_*            histogram, exclusive scan, stable permutation, meta rows
//   dispatch_rows      token row -> K destination rows (read once, store K times)
//   route_dispatch     both of the above in one launch for small worlds
//   dispatch_fp8       same copy with e4m3fn quantisation per 128 columns
//   stub_*             expert stand-in, one factor per row
//   combine / stub_combine   gather K rows per token, weighted sum
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "moe_a2a.h"

namespace {

constexpr int kWave = 64;
constexpr int kRouteThreads = 1024;
constexpr int kRouteWaves = kRouteThreads / kWave;
constexpr int kRouteSingleMaxRows = 16 * kRouteThreads;  // one-workgroup routing up to here
constexpr int kRowThreads = 256;
constexpr int kFusedMaxRows = 4096;  // route_dispatch: 12-bit entry ids
constexpr int kFusedEntriesPerThread = 8;

enum KernelId {
  KID_ROUTE_SINGLE = 0,
  KID_ROUTE_HIST,
  KID_ROUTE_SCAN,
  KID_ROUTE_RANK,
  KID_DISPATCH,
  KID_ROUTE_DISPATCH,
  KID_DISPATCH_FP8,
  KID_STUB,
  KID_STUB_FP8,
  KID_COMBINE,
  KID_STUB_COMBINE,
  KID_COUNT
};
const char* const kKernelNames[KID_COUNT] = {
    "route_single", "route_hist", "route_scan", "route_rank",   "dispatch_rows", "route_dispatch",
    "dispatch_fp8", "stub_rows",  "stub_fp8",   "combine_rows", "stub_combine"};

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
  int32_t* counts;
  int32_t* offsets;
  int32_t* slot_of_entry;
  int32_t* src_of_slot;
  int32_t* meta;
  int32_t* status;
};

__device__ __forceinline__ int load_expert(const RouteArgs& a, int i, bool valid) {
  int e = valid ? a.indices[i] : 0;
  if (e < 0 || e >= a.E) {
    if (a.status) *a.status = 1;  // vector store; the value is the same from every lane
    e = e < 0 ? 0 : a.E - 1;
  }
  return e;
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

__device__ __forceinline__ void emit_entry(const RouteArgs& a, const int* starts, int i, int e, int slot) {
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

// Whole routing in one workgroup: pass 1 histogram + scan, pass 2 stable ranks tile by tile.
__global__ __launch_bounds__(kRouteThreads) void route_single_kernel(RouteArgs a) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  int* base = wcnt + kRouteWaves * a.E;
  int* tmp = base + a.E;
  int* starts = tmp + kRouteWaves + 1;
  const int tid = threadIdx.x;
  load_starts(a, starts);
  for (int j = tid; j < a.E; j += kRouteThreads) base[j] = 0;
  __syncthreads();
  for (int i0 = 0; i0 < a.R; i0 += kRouteThreads) {
    int i = i0 + tid;
    bool valid = i < a.R;
    int e = load_expert(a, i, valid);
    int rank, cnt;
    wave_match(e, valid, a.nbits, rank, cnt);
    if (valid && rank == 0) atomicAdd(&base[e], cnt);  // LDS counter; order does not matter for a sum
  }
  __syncthreads();
  int v = tid < a.E ? base[tid] : 0;
  int total;
  int excl = block_exclusive_scan(v, tmp, total);
  if (tid < a.E) {
    base[tid] = excl;
    a.counts[tid] = v;
    a.offsets[tid] = excl;
  }
  if (tid == 0) a.offsets[a.E] = total;
  __syncthreads();
  for (int i0 = 0; i0 < a.R; i0 += kRouteThreads) {
    int i = i0 + tid;
    bool valid = i < a.R;
    int e = load_expert(a, i, valid);
    int rank = tile_wave_counts(wcnt, a.E, e, valid, a.nbits);
    if (tid < a.E) {
      int run = base[tid];
      for (int w = 0; w < kRouteWaves; ++w) {
        int c = wcnt[w * a.E + tid];
        wcnt[w * a.E + tid] = run;
        run += c;
      }
      base[tid] = run;
    }
    __syncthreads();
    if (valid) emit_entry(a, starts, i, e, wcnt[(tid / kWave) * a.E + e] + rank);
    __syncthreads();
  }
}

// Multi-workgroup routing, step 1: rows per (expert, tile), expert-major.
__global__ __launch_bounds__(kRouteThreads) void route_hist_kernel(RouteArgs a, int32_t* tile_hist, int ntiles) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  const int tid = threadIdx.x;
  int i = blockIdx.x * kRouteThreads + tid;
  bool valid = i < a.R;
  int e = load_expert(a, i, valid);
  tile_wave_counts(wcnt, a.E, e, valid, a.nbits);
  for (int j = tid; j < a.E; j += kRouteThreads) {
    int s = 0;
    for (int w = 0; w < kRouteWaves; ++w) s += wcnt[w * a.E + j];
    tile_hist[(size_t)j * ntiles + blockIdx.x] = s;
  }
}

// step 2: exclusive scan of the (expert, tile) matrix in place, counts and offsets.
__global__ __launch_bounds__(kRouteThreads) void route_scan_kernel(int32_t* tile_hist, int n, int E, int ntiles,
                                                                    int32_t* counts, int32_t* offsets) {
  __shared__ int tmp[kRouteWaves + 1];
  const int tid = threadIdx.x;
  int per = (n + kRouteThreads - 1) / kRouteThreads;
  int lo = tid * per;
  int hi = min(lo + per, n);
  int s = 0;
  for (int j = lo; j < hi; ++j) s += tile_hist[j];
  int total;
  int run = block_exclusive_scan(s, tmp, total);
  for (int j = lo; j < hi; ++j) {
    int c = tile_hist[j];
    tile_hist[j] = run;
    run += c;
  }
  __syncthreads();
  for (int e = tid; e < E; e += kRouteThreads) {
    int first = tile_hist[(size_t)e * ntiles];
    int next = e + 1 < E ? tile_hist[(size_t)(e + 1) * ntiles] : total;
    offsets[e] = first;
    counts[e] = next - first;
  }
  if (tid == 0) offsets[E] = total;
}

// step 3: stable rank inside the tile + first slot of (expert, tile).
__global__ __launch_bounds__(kRouteThreads) void route_rank_kernel(RouteArgs a, const int32_t* tile_base,
                                                                    int ntiles) {
  extern __shared__ int smem[];
  int* wcnt = smem;
  int* starts = wcnt + kRouteWaves * a.E;
  const int tid = threadIdx.x;
  load_starts(a, starts);
  int i = blockIdx.x * kRouteThreads + tid;
  bool valid = i < a.R;
  int e = load_expert(a, i, valid);
  int rank = tile_wave_counts(wcnt, a.E, e, valid, a.nbits);
  for (int j = tid; j < a.E; j += kRouteThreads) {
    int run = tile_base[(size_t)j * ntiles + blockIdx.x];
    for (int w = 0; w < kRouteWaves; ++w) {
      int c = wcnt[w * a.E + j];
      wcnt[w * a.E + j] = run;
      run += c;
    }
  }
  __syncthreads();
  if (valid) emit_entry(a, starts, i, e, wcnt[(tid / kWave) * a.E + e] + rank);
}

// ---------------------------------------------------------------------------------------
// dispatch: token row -> K rows
// ---------------------------------------------------------------------------------------
// One workgroup copies U*256 16-byte vectors of one token row to that token's K slots.
template <int U>
__global__ __launch_bounds__(kRowThreads) void dispatch_rows_kernel(const uint4* __restrict__ x,
                                                                     const int32_t* __restrict__ slot_of_entry,
                                                                     uint4* __restrict__ disp, int K, int nvec,
                                                                     int nsplit) {
  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  const int c0 = cs * (kRowThreads * U) + threadIdx.x;
  const uint4* src = x + (size_t)t * nvec;
  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int c = c0 + u * kRowThreads;
    if (c < nvec) v[u] = src[c];
  }
  const int32_t* sl = slot_of_entry + (size_t)t * K;
  for (int k = 0; k < K; ++k) {
    uint4* dst = disp + (size_t)sl[k] * nvec;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int c = c0 + u * kRowThreads;
      if (c < nvec) dst[c] = v[u];
    }
  }
}

// Routing folded into the dispatch for R <= kFusedMaxRows.  The slot of entry i is the number
// of entries whose (expert, entry id) pair is smaller, so a workgroup can find the K slots of
// its own token by comparing every entry of the table against K keys: each lane holds
// kFusedEntriesPerThread entries, a ballot + popcount per (entry, key) counts a wave's share,
// and LDS counters add the waves up.  Column split 0 of each token also writes the index
// arrays and meta rows; one extra workgroup writes counts and offsets.
template <int U>
__global__ __launch_bounds__(kRowThreads) void route_dispatch_kernel(RouteArgs a, const uint4* __restrict__ x,
                                                                      uint4* __restrict__ disp, int nvec,
                                                                      int nsplit) {
  __shared__ int s_slot[MOE_A2A_MAX_TOPK];
  __shared__ int s_key[MOE_A2A_MAX_TOPK];
  __shared__ int s_hist[MOE_A2A_MAX_EXPERTS];
  __shared__ int s_tmp[kRowThreads / kWave + 1];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int ntok_blocks = a.T * nsplit;

  if ((int)blockIdx.x == ntok_blocks) {  // counts + offsets
    for (int j = tid; j < a.E; j += kRowThreads) s_hist[j] = 0;
    __syncthreads();
    for (int i = tid; i < a.R; i += kRowThreads) atomicAdd(&s_hist[load_expert(a, i, true)], 1);
    __syncthreads();
    const int per = (a.E + kRowThreads - 1) / kRowThreads;
    int lo = min(tid * per, a.E), hi = min(lo + per, a.E);
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

  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  const int c0 = cs * (kRowThreads * U) + tid;
  const uint4* src = x + (size_t)t * nvec;
  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {  // row loads are in flight while the slots are worked out
    int c = c0 + u * kRowThreads;
    if (c < nvec) v[u] = src[c];
  }
  if (tid < a.K) {  // keys of this token's own entries
    int ik = t * a.K + tid;
    s_key[tid] = (load_expert(a, ik, true) << 12) | ik;
    s_slot[tid] = 0;
  }
  __syncthreads();

  constexpr int kChunk = kRowThreads * kFusedEntriesPerThread;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.indices) & 15u) == 0;
  for (int i0 = 0; i0 < a.R; i0 += kChunk) {
    int key[kFusedEntriesPerThread];
    const int ibase = i0 + tid * kFusedEntriesPerThread;
    if (vec_ok && ibase + kFusedEntriesPerThread <= a.R) {
      const int4* p = reinterpret_cast<const int4*>(a.indices + ibase);
      const int4 q0 = p[0], q1 = p[1];
      const int e[kFusedEntriesPerThread] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
      for (int m = 0; m < kFusedEntriesPerThread; ++m) {
        int em = e[m];
        if (em < 0 || em >= a.E) {
          if (a.status) *a.status = 1;
          em = em < 0 ? 0 : a.E - 1;
        }
        key[m] = (em << 12) | (ibase + m);
      }
    } else {
#pragma unroll
      for (int m = 0; m < kFusedEntriesPerThread; ++m) {
        int i = ibase + m;
        bool valid = i < a.R;
        int e = load_expert(a, i, valid);
        key[m] = valid ? ((e << 12) | i) : 0x7fffffff;
      }
    }
    for (int k = 0; k < a.K; ++k) {
      const int mykey = s_key[k];
      int c = 0;
#pragma unroll
      for (int m = 0; m < kFusedEntriesPerThread; ++m) c += __popcll(__ballot(key[m] < mykey));
      if (lane == 0 && c) atomicAdd(&s_slot[k], c);
    }
  }
  __syncthreads();

  for (int k = 0; k < a.K; ++k) {
    uint4* dst = disp + (size_t)s_slot[k] * nvec;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int c = c0 + u * kRowThreads;
      if (c < nvec) dst[c] = v[u];
    }
  }
  if (cs == 0 && tid < a.K) {
    int i = t * a.K + tid;
    int e = load_expert(a, i, true);
    int slot = s_slot[tid];
    a.slot_of_entry[i] = slot;
    a.src_of_slot[slot] = i;
    int sr = a.src_rank, tl = t;
    if (a.rank_start) {
      int lo = 0, hi = a.W;
      while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (a.rank_start[mid] <= t) lo = mid; else hi = mid;
      }
      sr = lo;
      tl = t - a.rank_start[lo];
    }
    int32_t* m = a.meta + (size_t)slot * MOE_A2A_META_DIM;
    m[0] = e;
    m[1] = sr;
    m[2] = tl;
    m[3] = tid;
    m[4] = 0;
  }
}

// fp8 dispatch.  8 lanes own one 128-column block (16 elements each): block amax by three
// xor-shuffles, scale = amax/448, q = e4m3(x/scale) with the hardware conversion (RNE).
template <class E>
__global__ __launch_bounds__(kRowThreads) void dispatch_fp8_kernel(const uint4* __restrict__ x,
                                                                    const int32_t* __restrict__ slot_of_entry,
                                                                    uint4* __restrict__ disp_q,
                                                                    float* __restrict__ disp_scale, int K, int nblk,
                                                                    int nsplit) {
  constexpr int kBlocksPerWg = kRowThreads / 8;
  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  const int gb = cs * kBlocksPerWg + (threadIdx.x >> 3);
  const int sub = threadIdx.x & 7;
  const bool valid = gb < nblk;
  float f[16];
  if (valid) {
    const uint4* src = x + ((size_t)t * nblk + gb) * 16 + sub * 2;
    uint4 v0 = src[0], v1 = src[1];
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
  float scale = amax == 0.f ? 1.f : amax / 448.f;
  uint32_t q[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] / scale, f[4 * j + 1] / scale, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] / scale, f[4 * j + 3] / scale, w, true);
    q[j] = (uint32_t)w;
  }
  if (!valid) return;
  const uint4 qv = make_uint4(q[0], q[1], q[2], q[3]);
  const int32_t* sl = slot_of_entry + (size_t)t * K;
  for (int k = 0; k < K; ++k) {
    size_t row = (size_t)sl[k];
    disp_q[(row * nblk + gb) * 8 + sub] = qv;
    if (sub == 0) disp_scale[row * nblk + gb] = scale;
  }
}

// ---------------------------------------------------------------------------------------
// expert stub
// ---------------------------------------------------------------------------------------
template <class In, class Out, int U>
__global__ __launch_bounds__(kRowThreads) void stub_rows_kernel(const uint4* __restrict__ disp,
                                                                 const int32_t* __restrict__ meta,
                                                                 uint4* __restrict__ y, int stub_kind, int E,
                                                                 int E_l, int nvec, int nsplit) {
  const int row = blockIdx.x / nsplit;
  const int cs = blockIdx.x - row * nsplit;
  const int c0 = cs * (kRowThreads * U) + threadIdx.x;
  const float s = stub_factor(meta[(size_t)row * MOE_A2A_META_DIM], stub_kind, E, E_l);
  const uint4* src = disp + (size_t)row * nvec;
  uint4* dst = y + (size_t)row * nvec;
  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int c = c0 + u * kRowThreads;
    if (c < nvec) v[u] = src[c];
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int c = c0 + u * kRowThreads;
    if (c >= nvec) continue;
    uint32_t d[4];
    unpack8(v[u], d);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = In::lo(d[j]), b = In::hi(d[j]);
      round_pair<Out>(a, b);  // .to(out_dtype)
      d[j] = Out::pack(a * s, b * s);
    }
    dst[c] = make_uint4(d[0], d[1], d[2], d[3]);
  }
}

__device__ __forceinline__ void fp8x4_to_f32(uint32_t w, float (&f)[4]) {
  f[0] = __builtin_amdgcn_cvt_f32_fp8((int)w, 0);
  f[1] = __builtin_amdgcn_cvt_f32_fp8((int)w, 1);
  f[2] = __builtin_amdgcn_cvt_f32_fp8((int)w, 2);
  f[3] = __builtin_amdgcn_cvt_f32_fp8((int)w, 3);
}

// fp8 rows: each lane turns 16 bytes into 16 output elements (two 16-byte stores).
template <class Out>
__global__ __launch_bounds__(kRowThreads) void stub_fp8_kernel(const uint4* __restrict__ disp_q,
                                                                const float* __restrict__ disp_scale,
                                                                const int32_t* __restrict__ meta,
                                                                uint4* __restrict__ y, int stub_kind, int E, int E_l,
                                                                int nblk, int nsplit) {
  const int row = blockIdx.x / nsplit;
  const int cs = blockIdx.x - row * nsplit;
  const int c = cs * kRowThreads + threadIdx.x;  // 16-byte vector of the fp8 row
  if (c >= nblk * 8) return;
  const float s = stub_factor(meta[(size_t)row * MOE_A2A_META_DIM], stub_kind, E, E_l);
  const float scale = disp_scale[(size_t)row * nblk + (c >> 3)];
  const uint4 q = disp_q[(size_t)row * nblk * 8 + c];
  const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
  uint32_t o[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float f[4];
    fp8x4_to_f32(qw[j], f);
    o[2 * j] = Out::pack((f[0] * scale) * s, (f[1] * scale) * s);
    o[2 * j + 1] = Out::pack((f[2] * scale) * s, (f[3] * scale) * s);
  }
  uint4* dst = y + ((size_t)row * nblk * 8 + c) * 2;
  dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
  dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

// ---------------------------------------------------------------------------------------
// combine
// ---------------------------------------------------------------------------------------
// Order the K entries of token t for the weighted sum: STRICT = ascending slot (the order in
// which the reference's receive loop meets them), F32 = k order.
__device__ __forceinline__ void order_entries(const int32_t* __restrict__ slot_of_entry,
                                              const float* __restrict__ weights, int t, int K, int mode,
                                              int* s_slot, float* s_w, int* s_k) {
  if ((int)threadIdx.x < K) {
    const int32_t* sl = slot_of_entry + (size_t)t * K;
    int mine = sl[threadIdx.x];
    int pos = threadIdx.x;
    if (mode == MOE_A2A_COMBINE_STRICT) {
      pos = 0;
      for (int j = 0; j < K; ++j) pos += sl[j] < mine;
    }
    s_slot[pos] = mine;
    s_w[pos] = weights[(size_t)t * K + threadIdx.x];
    s_k[pos] = threadIdx.x;
  }
  __syncthreads();
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

template <class E, int MODE>
__global__ __launch_bounds__(kRowThreads) void combine_rows_kernel(const uint4* __restrict__ y,
                                                                    const float* __restrict__ weights,
                                                                    const int32_t* __restrict__ slot_of_entry,
                                                                    uint4* __restrict__ out, int K, int nvec,
                                                                    int nsplit) {
  __shared__ int s_slot[MOE_A2A_MAX_TOPK];
  __shared__ float s_w[MOE_A2A_MAX_TOPK];
  __shared__ int s_k[MOE_A2A_MAX_TOPK];
  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  order_entries(slot_of_entry, weights, t, K, MODE, s_slot, s_w, s_k);
  const int c = cs * kRowThreads + threadIdx.x;
  if (c >= nvec) return;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int j0 = 0; j0 < K; j0 += 8) {
    uint4 v[8];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj)
      if (j0 + jj < K) v[jj] = y[(size_t)s_slot[j0 + jj] * nvec + c];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj)
      if (j0 + jj < K) accumulate8<E, MODE>(acc, v[jj], s_w[j0 + jj]);
  }
  out[(size_t)t * nvec + c] = make_uint4(E::pack(acc[0], acc[1]), E::pack(acc[2], acc[3]),
                                         E::pack(acc[4], acc[5]), E::pack(acc[6], acc[7]));
}

// stub folded into the combine, 16-bit dispatched rows
template <class In, class Out, int MODE>
__global__ __launch_bounds__(kRowThreads) void stub_combine_rows_kernel(
    const uint4* __restrict__ disp, const int32_t* __restrict__ indices, const float* __restrict__ weights,
    const int32_t* __restrict__ slot_of_entry, uint4* __restrict__ out, int stub_kind, int E, int E_l, int K,
    int nvec, int nsplit) {
  __shared__ int s_slot[MOE_A2A_MAX_TOPK];
  __shared__ float s_w[MOE_A2A_MAX_TOPK];
  __shared__ int s_k[MOE_A2A_MAX_TOPK];
  __shared__ float s_f[MOE_A2A_MAX_TOPK];
  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  order_entries(slot_of_entry, weights, t, K, MODE, s_slot, s_w, s_k);
  if ((int)threadIdx.x < K)
    s_f[threadIdx.x] = stub_factor(indices[(size_t)t * K + s_k[threadIdx.x]], stub_kind, E, E_l);
  __syncthreads();
  const int c = cs * kRowThreads + threadIdx.x;
  if (c >= nvec) return;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int j0 = 0; j0 < K; j0 += 8) {
    uint4 v[8];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj)
      if (j0 + jj < K) v[jj] = disp[(size_t)s_slot[j0 + jj] * nvec + c];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      if (j0 + jj >= K) continue;
      const float s = s_f[j0 + jj];
      uint32_t d[4];
      unpack8(v[jj], d);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float a = In::lo(d[j]), b = In::hi(d[j]);
        round_pair<Out>(a, b);
        d[j] = Out::pack(a * s, b * s);
      }
      accumulate8<Out, MODE>(acc, make_uint4(d[0], d[1], d[2], d[3]), s_w[j0 + jj]);
    }
  }
  out[(size_t)t * nvec + c] = make_uint4(Out::pack(acc[0], acc[1]), Out::pack(acc[2], acc[3]),
                                         Out::pack(acc[4], acc[5]), Out::pack(acc[6], acc[7]));
}

// stub folded into the combine, fp8 dispatched rows (16 columns per lane)
template <class Out, int MODE>
__global__ __launch_bounds__(kRowThreads) void stub_combine_fp8_kernel(
    const uint4* __restrict__ disp_q, const float* __restrict__ disp_scale, const int32_t* __restrict__ indices,
    const float* __restrict__ weights, const int32_t* __restrict__ slot_of_entry, uint4* __restrict__ out,
    int stub_kind, int E, int E_l, int K, int nblk, int nsplit) {
  __shared__ int s_slot[MOE_A2A_MAX_TOPK];
  __shared__ float s_w[MOE_A2A_MAX_TOPK];
  __shared__ int s_k[MOE_A2A_MAX_TOPK];
  __shared__ float s_f[MOE_A2A_MAX_TOPK];
  const int t = blockIdx.x / nsplit;
  const int cs = blockIdx.x - t * nsplit;
  order_entries(slot_of_entry, weights, t, K, MODE, s_slot, s_w, s_k);
  if ((int)threadIdx.x < K)
    s_f[threadIdx.x] = stub_factor(indices[(size_t)t * K + s_k[threadIdx.x]], stub_kind, E, E_l);
  __syncthreads();
  const int c = cs * kRowThreads + threadIdx.x;
  if (c >= nblk * 8) return;
  float acc0[8], acc1[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc0[j] = acc1[j] = 0.f;
  for (int j0 = 0; j0 < K; j0 += 4) {
    uint4 v[4];
    float sc[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
      if (j0 + jj < K) {
        size_t row = (size_t)s_slot[j0 + jj];
        v[jj] = disp_q[row * nblk * 8 + c];
        sc[jj] = disp_scale[row * nblk + (c >> 3)];
      }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      if (j0 + jj >= K) continue;
      const float s = s_f[j0 + jj];
      const uint32_t qw[4] = {v[jj].x, v[jj].y, v[jj].z, v[jj].w};
      uint32_t o[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float f[4];
        fp8x4_to_f32(qw[j], f);
        o[2 * j] = Out::pack((f[0] * sc[jj]) * s, (f[1] * sc[jj]) * s);
        o[2 * j + 1] = Out::pack((f[2] * sc[jj]) * s, (f[3] * sc[jj]) * s);
      }
      accumulate8<Out, MODE>(acc0, make_uint4(o[0], o[1], o[2], o[3]), s_w[j0 + jj]);
      accumulate8<Out, MODE>(acc1, make_uint4(o[4], o[5], o[6], o[7]), s_w[j0 + jj]);
    }
  }
  uint4* dst = out + ((size_t)t * nblk * 8 + c) * 2;
  dst[0] = make_uint4(Out::pack(acc0[0], acc0[1]), Out::pack(acc0[2], acc0[3]), Out::pack(acc0[4], acc0[5]),
                      Out::pack(acc0[6], acc0[7]));
  dst[1] = make_uint4(Out::pack(acc1[0], acc1[1]), Out::pack(acc1[2], acc1[3]), Out::pack(acc1[4], acc1[5]),
                      Out::pack(acc1[6], acc1[7]));
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

// vectors per thread for the row kernels: fewer when the grid would otherwise be small
int pick_unroll(int rows, int nvec) {
  for (int u = 4; u > 1; u >>= 1) {
    if (nvec >= kRowThreads * u && (long long)rows * ceil_div(nvec, kRowThreads * u) >= 2048) return u;
  }
  return 1;
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
  if (R <= kRouteSingleMaxRows) return 256;
  long long ntiles = (R + kRouteThreads - 1) / kRouteThreads;
  return align_up((size_t)ntiles * (size_t)E * sizeof(int32_t), 256);
}

int moe_a2a_route(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                  int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                  int32_t* status, void* workspace, size_t workspace_bytes, moe_a2a_stream_t stream_) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), counts, offsets, slot_of_entry,
              src_of_slot, meta, status};
  const size_t lds_w = (size_t)kRouteWaves * E * sizeof(int);
  const size_t lds_starts = (size_t)(W + 1) * sizeof(int);
  if (a.R <= kRouteSingleMaxRows) {
    size_t lds = lds_w + (size_t)E * sizeof(int) + (kRouteWaves + 1) * sizeof(int) + lds_starts;
    set_max_lds(route_single_kernel, lds);
    return launch(KID_ROUTE_SINGLE, route_single_kernel, dim3(1), dim3(kRouteThreads), lds, stream, a);
  }
  if (!workspace || workspace_bytes < moe_a2a_workspace_bytes(T, K, E)) return MOE_A2A_E_WORKSPACE;
  int ntiles = ceil_div(a.R, kRouteThreads);
  int32_t* tile = (int32_t*)workspace;
  set_max_lds(route_hist_kernel, lds_w);
  if (int rc = launch(KID_ROUTE_HIST, route_hist_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w, stream, a, tile,
                      ntiles))
    return rc;
  if (int rc = launch(KID_ROUTE_SCAN, route_scan_kernel, dim3(1), dim3(kRouteThreads), 0, stream, tile, E * ntiles,
                      E, ntiles, counts, offsets))
    return rc;
  set_max_lds(route_rank_kernel, lds_w + lds_starts);
  return launch(KID_ROUTE_RANK, route_rank_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w + lds_starts, stream, a,
                (const int32_t*)tile, ntiles);
}

static int check_rows(const void* a, const void* b, int T, int K, int H, int mult) {
  if (T < 0 || K < 1 || K > MOE_A2A_MAX_TOPK || H < mult || H % mult != 0) return MOE_A2A_E_SHAPE;
  if ((long long)T * K > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (T > 0 && (!a || !b)) return MOE_A2A_E_NULL;
  if (!aligned16(a) || !aligned16(b)) return MOE_A2A_E_ALIGN;
  return 0;
}

int moe_a2a_dispatch(const void* x, const int32_t* slot_of_entry, void* disp_x, int T, int K, int H,
                     moe_a2a_stream_t stream_) {
  if (int rc = check_rows(x, disp_x, T, K, H, 8)) return rc;
  if (T == 0) return 0;
  if (!slot_of_entry) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int nvec = H / 8;
  const int U = pick_unroll(T, nvec);
  const int nsplit = ceil_div(nvec, kRowThreads * U);
  dim3 grid((unsigned)T * nsplit), block(kRowThreads);
  const uint4* xs = (const uint4*)x;
  uint4* ds = (uint4*)disp_x;
  switch (U) {
    case 4: return launch(KID_DISPATCH, dispatch_rows_kernel<4>, grid, block, 0, stream, xs, slot_of_entry, ds, K, nvec, nsplit);
    case 2: return launch(KID_DISPATCH, dispatch_rows_kernel<2>, grid, block, 0, stream, xs, slot_of_entry, ds, K, nvec, nsplit);
    default: return launch(KID_DISPATCH, dispatch_rows_kernel<1>, grid, block, 0, stream, xs, slot_of_entry, ds, K, nvec, nsplit);
  }
}

int moe_a2a_fused_max_rows(void) { return kFusedMaxRows; }

int moe_a2a_route_dispatch(const void* x, const int32_t* indices, const int32_t* rank_start, int src_rank, int T,
                           int K, int E, int W, int H, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry,
                           int32_t* src_of_slot, int32_t* meta, int32_t* status, void* disp_x,
                           moe_a2a_stream_t stream_) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if ((long long)T * K > kFusedMaxRows) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(x, disp_x, T, K, H, 8)) return rc;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), counts, offsets, slot_of_entry,
              src_of_slot, meta, status};
  const int nvec = H / 8;
  const int U = pick_unroll(T, nvec);
  const int nsplit = ceil_div(nvec, kRowThreads * U);
  dim3 grid((unsigned)T * nsplit + 1), block(kRowThreads);
  const uint4* xs = (const uint4*)x;
  uint4* ds = (uint4*)disp_x;
  switch (U) {
    case 4: return launch(KID_ROUTE_DISPATCH, route_dispatch_kernel<4>, grid, block, 0, stream, a, xs, ds, nvec, nsplit);
    case 2: return launch(KID_ROUTE_DISPATCH, route_dispatch_kernel<2>, grid, block, 0, stream, a, xs, ds, nvec, nsplit);
    default: return launch(KID_ROUTE_DISPATCH, route_dispatch_kernel<1>, grid, block, 0, stream, a, xs, ds, nvec, nsplit);
  }
}

int moe_a2a_dispatch_fp8(const void* x, int x_type, const int32_t* slot_of_entry, uint8_t* disp_q,
                         float* disp_scale, int T, int K, int H, moe_a2a_stream_t stream_) {
  if (x_type != MOE_A2A_F16 && x_type != MOE_A2A_BF16) return MOE_A2A_E_DTYPE;
  if (int rc = check_rows(x, disp_q, T, K, H, MOE_A2A_FP8_BLOCK)) return rc;
  if (T == 0) return 0;
  if (!slot_of_entry || !disp_scale) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int nblk = H / MOE_A2A_FP8_BLOCK;
  const int nsplit = ceil_div(nblk, kRowThreads / 8);
  dim3 grid((unsigned)T * nsplit), block(kRowThreads);
  if (x_type == MOE_A2A_BF16)
    return launch(KID_DISPATCH_FP8, dispatch_fp8_kernel<Bf16>, grid, block, 0, stream, (const uint4*)x, slot_of_entry,
                  (uint4*)disp_q, disp_scale, K, nblk, nsplit);
  return launch(KID_DISPATCH_FP8, dispatch_fp8_kernel<F16>, grid, block, 0, stream, (const uint4*)x, slot_of_entry,
                (uint4*)disp_q, disp_scale, K, nblk, nsplit);
}

static bool known_type(int t) { return t == MOE_A2A_F16 || t == MOE_A2A_BF16; }

int moe_a2a_stub(const void* disp, const float* disp_scale, const int32_t* meta, int in_type, int out_type,
                 int stub_kind, int E, int W, void* y, int R, int H, moe_a2a_stream_t stream_) {
  if (!known_type(out_type) || (!disp_scale && !known_type(in_type))) return MOE_A2A_E_DTYPE;
  if (stub_kind != MOE_A2A_STUB_OWNER_RANK && stub_kind != MOE_A2A_STUB_EXPERT_FRACTION) return MOE_A2A_E_DTYPE;
  if (E < 1 || W < 1 || E % W != 0 || R < 0) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(disp, y, R, 1, H, disp_scale ? MOE_A2A_FP8_BLOCK : 8)) return rc;
  if (R == 0) return 0;
  if (!meta) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int E_l = E / W;
  dim3 block(kRowThreads);
  if (disp_scale) {
    const int nblk = H / MOE_A2A_FP8_BLOCK;
    const int nsplit = ceil_div(nblk * 8, kRowThreads);
    dim3 grid((unsigned)R * nsplit);
    if (out_type == MOE_A2A_BF16)
      return launch(KID_STUB_FP8, stub_fp8_kernel<Bf16>, grid, block, 0, stream, (const uint4*)disp, disp_scale, meta,
                    (uint4*)y, stub_kind, E, E_l, nblk, nsplit);
    return launch(KID_STUB_FP8, stub_fp8_kernel<F16>, grid, block, 0, stream, (const uint4*)disp, disp_scale, meta,
                  (uint4*)y, stub_kind, E, E_l, nblk, nsplit);
  }
  const int nvec = H / 8;
  const int U = pick_unroll(R, nvec) >= 2 ? 2 : 1;
  const int nsplit = ceil_div(nvec, kRowThreads * U);
  dim3 grid((unsigned)R * nsplit);
#define STUB_LAUNCH(IN, OUT, UU)                                                                              \
  return launch(KID_STUB, stub_rows_kernel<IN, OUT, UU>, grid, block, 0, stream, (const uint4*)disp, meta, \
                (uint4*)y, stub_kind, E, E_l, nvec, nsplit)
#define STUB_TYPES(UU)                                                     \
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_BF16) STUB_LAUNCH(Bf16, Bf16, UU); \
  if (in_type == MOE_A2A_F16 && out_type == MOE_A2A_F16) STUB_LAUNCH(F16, F16, UU);     \
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_F16) STUB_LAUNCH(Bf16, F16, UU);   \
  STUB_LAUNCH(F16, Bf16, UU)
  if (U == 2) { STUB_TYPES(2); }
  STUB_TYPES(1);
#undef STUB_TYPES
#undef STUB_LAUNCH
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
  const int nsplit = ceil_div(nvec, kRowThreads);
  dim3 grid((unsigned)T * nsplit), block(kRowThreads);
#define COMBINE_LAUNCH(EL, MD)                                                                                  \
  return launch(KID_COMBINE, combine_rows_kernel<EL, MD>, grid, block, 0, stream, (const uint4*)expert_y, weights, \
                slot_of_entry, (uint4*)out, K, nvec, nsplit)
  if (elem_type == MOE_A2A_BF16) {
    if (mode == MOE_A2A_COMBINE_STRICT) COMBINE_LAUNCH(Bf16, MOE_A2A_COMBINE_STRICT);
    COMBINE_LAUNCH(Bf16, MOE_A2A_COMBINE_F32);
  }
  if (mode == MOE_A2A_COMBINE_STRICT) COMBINE_LAUNCH(F16, MOE_A2A_COMBINE_STRICT);
  COMBINE_LAUNCH(F16, MOE_A2A_COMBINE_F32);
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
  dim3 block(kRowThreads);
  const bool strict = mode == MOE_A2A_COMBINE_STRICT;
  if (disp_scale) {
    const int nblk = H / MOE_A2A_FP8_BLOCK;
    const int nsplit = ceil_div(nblk * 8, kRowThreads);
    dim3 grid((unsigned)T * nsplit);
#define SC8_LAUNCH(OUT, MD)                                                                                   \
  return launch(KID_STUB_COMBINE, stub_combine_fp8_kernel<OUT, MD>, grid, block, 0, stream, (const uint4*)disp, \
                disp_scale, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, E_l, K, nblk, nsplit)
    if (out_type == MOE_A2A_BF16) {
      if (strict) SC8_LAUNCH(Bf16, MOE_A2A_COMBINE_STRICT);
      SC8_LAUNCH(Bf16, MOE_A2A_COMBINE_F32);
    }
    if (strict) SC8_LAUNCH(F16, MOE_A2A_COMBINE_STRICT);
    SC8_LAUNCH(F16, MOE_A2A_COMBINE_F32);
#undef SC8_LAUNCH
  }
  const int nvec = H / 8;
  const int nsplit = ceil_div(nvec, kRowThreads);
  dim3 grid((unsigned)T * nsplit);
#define SC_LAUNCH(IN, OUT, MD)                                                                                     \
  return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD>, grid, block, 0, stream, (const uint4*)disp, \
                indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, E_l, K, nvec, nsplit)
#define SC_MODES(IN, OUT)                                  \
  {                                                        \
    if (strict) SC_LAUNCH(IN, OUT, MOE_A2A_COMBINE_STRICT); \
    SC_LAUNCH(IN, OUT, MOE_A2A_COMBINE_F32);               \
  }
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_BF16) SC_MODES(Bf16, Bf16)
  if (in_type == MOE_A2A_F16 && out_type == MOE_A2A_F16) SC_MODES(F16, F16)
  if (in_type == MOE_A2A_BF16 && out_type == MOE_A2A_F16) SC_MODES(Bf16, F16)
  SC_MODES(F16, Bf16)
#undef SC_MODES
#undef SC_LAUNCH
}

int moe_a2a_timer_begin(int capacity) {
  if (g_timer.active || capacity < 1) return MOE_A2A_E_STATE;
  g_timer.start = new hipEvent_t[capacity];
  g_timer.stop = new hipEvent_t[capacity];
  g_timer.ids = new int[capacity];
  for (int i = 0; i < capacity; ++i) {
    hipError_t e1 = hipEventCreate(&g_timer.start[i]);
    hipError_t e2 = hipEventCreate(&g_timer.stop[i]);
    if (e1 != hipSuccess || e2 != hipSuccess) return (int)(e1 != hipSuccess ? e1 : e2);
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
