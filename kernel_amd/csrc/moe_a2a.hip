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
//   route_dispatch_fp8 routing and that copy in one launch, a tile of tokens per workgroup
//   stub_*             expert stand-in, one factor per row
//   combine / stub_combine   gather K rows per token, weighted sum
//   forward_token / forward_tile   the whole path of a token (routing, dispatch, stub, weighted sum)
//                      in one launch: a workgroup reads back the rows it stored itself
//   dispatch_fold      dispatch, stub and weighted sum of a token behind a routing of its own
//   expert_gemm        y[rows of e] = x[rows of e] * W_e^T, 128 x 128 tiles (short segments)
//   expert_gemm_wide   the same on 256 x 256 tiles, software-pipelined; 16-bit or fp8 rows
//   gemm_rs_*          the reference's other problem on one GPU: a K-split linear layer whose
//                      reduce-scatter is the sum over the K shards held in one buffer
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <mutex>

#include "gemm_rs.h"
#include "moe_a2a.h"

// Scratch of moe_a2a_route_noalloc: the (tile, expert) count matrix of the multi-launch routing, held
// by every GPU the library runs on from load to the end of the process (4 MiB).  In host code this
// name is only a handle for hipGetSymbolAddress; kernels get the device address it resolves to.
constexpr size_t kStaticScratchInts = (size_t)1 << 20;
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

namespace {

constexpr int kWave = 64;
constexpr int kXcds = 8;  // accelerator dies of an MI355X; workgroup b runs on die b % 8
constexpr int kRouteThreads = 1024;
constexpr int kRouteWaves = kRouteThreads / kWave;
constexpr int kRouteTilesMaxRows = 32 * kRouteThreads;  // one-launch routing up to here (8.7 against 10.2 us in two
                                                        // launches at 32 K entries, 12.2 against 10.8 us at 64 K)
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
  KID_ROUTE_EMPTY,
  KID_FORWARD_TOKEN,
  KID_FORWARD_TILE,
  KID_DISPATCH_FOLD,
  KID_GEMM_RS_WIDE,
  KID_GEMM_RS_TILE,
  KID_GEMM_RS_REDUCE,
  KID_GEMM_RS_PAD,
  KID_GEMM_RS_NARROW,
  KID_ROUTE_DISPATCH_FP8,
  KID_COUNT
};
const char* const kKernelNames[KID_COUNT] = {
    "route_tiles", "route_hist", "route_scan", "route_rank",   "dispatch_rows", "route_dispatch", "route_dispatch_tile",
    "dispatch_fp8", "stub_rows",  "stub_fp8",   "combine_rows", "stub_combine", "expert_gemm",
    "expert_gemm_wide", "expert_gemm_skinny", "expert_gemm_f8", "expert_gemm_mx", "route_empty", "forward_token", "forward_tile", "dispatch_fold",
    "gemm_rs_wide", "gemm_rs_tile", "gemm_rs_reduce", "gemm_rs_pad", "gemm_rs_narrow", "route_dispatch_fp8"};

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
  // a rounded to bf16 and left where the arithmetic goes on, in f32: the conversion of the pair
  // (0, a) puts bf16(a) into the high half of the word over zeros, which IS that f32 -- one
  // instruction per element where packing two and taking them apart again costs one and a half
  static __device__ __forceinline__ float round(float a) { return __uint_as_float(pack(0.f, a)); }
};

struct F16 {
  static __device__ __forceinline__ float lo(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t u) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
  }
  // Two roundings, as torch does them: the caller's f32 arithmetic rounds to f32, the conversion
  // rounds that f32 to f16.  The empty asm hides where a and b come from: left to itself the
  // compiler merges a preceding multiply or add into v_fma_mixlo_f16, which rounds the exact
  // product or sum ONCE to f16 and gives a different last bit in a fraction of a percent of the
  // values (seen against the oracle on fp8 rows, where the f32 product is rarely exact).
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    asm("" : "+v"(a), "+v"(b));
    uint32_t l = __builtin_bit_cast(uint16_t, (_Float16)a);
    uint32_t h = __builtin_bit_cast(uint16_t, (_Float16)b);
    return l | (h << 16);
  }
  static __device__ __forceinline__ float round(float a) {
    asm("" : "+v"(a));  // as in pack: keep the multiply or add that made a out of the conversion
    return (float)(_Float16)a;
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

// (1 + e) / E as the f32 nearest the exact quotient.  The oracle divides in double and rounds the
// result to f32; for integers up to 1024 the correctly rounded f32 division gives the same value (a
// quotient of such integers is never within 2^-53 relative of an f32 rounding boundary without lying
// on it), at a quarter of the instructions.
__device__ __forceinline__ float stub_factor(int e, int stub_kind, int num_experts, int experts_per_rank) {
  if (stub_kind == MOE_A2A_STUB_OWNER_RANK) return (float)(1 + e / experts_per_rank);
  return __fdiv_rn((float)(1 + e), (float)num_experts);
}

// the kernels, in three files of their own
#include "route_kernels.inc"
#include "row_kernels.inc"
#include "expert_gemm_kernels.inc"
#include "gemm8_kernels.inc"
#include "gemm_rs_kernels.inc"

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
struct LaunchTimer {
  bool active = false;
  int capacity = 0;
  int used = 0;
  int skip = 0;  // launches still to go out untimed
  hipEvent_t* start = nullptr;
  hipEvent_t* stop = nullptr;
  int* ids = nullptr;
};
LaunchTimer g_timer;
// A launch looks at this flag only (relaxed: the timer is off in a product run and the launch path
// then touches no shared mutable state); while it is set, launches, begin, skip and end take the
// mutex, so a second caller thread's launches are recorded one at a time instead of racing.
std::atomic<bool> g_timer_on{false};
std::mutex g_timer_mutex;

template <typename T>
struct same_type {
  typedef T type;
};

// Arguments are converted to the kernel's own parameter types before they are packed.
template <typename... KArgs>
int launch(int kid, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
           typename same_type<KArgs>::type... args) {
  if (!g_timer_on.load(std::memory_order_relaxed)) {
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
    return (int)hipGetLastError();
  }
  std::lock_guard<std::mutex> hold(g_timer_mutex);
  if (g_timer.active && g_timer.skip > 0) {
    --g_timer.skip;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
  } else if (g_timer.active && g_timer.used < g_timer.capacity) {
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

// Geometry of the combine kernels: `per` lanes of a workgroup hold `vpl` row vectors each.
struct CombineGeom {
  int per, nsplit, threads, vpl;
};
// Dynamic LDS beyond the 48 KB default needs the function's attribute raised.  The attribute belongs
// to a device's copy of the function, so the largest size granted so far is kept per kernel and
// device and the runtime is only asked when a launch needs more (racing first calls repeat it).
template <auto Kernel>
int ensure_lds(size_t bytes) {
  if (bytes <= 48 * 1024) return 0;
  static std::atomic<size_t> granted[kMaxDevices];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MOE_A2A_E_STATE;
  if (granted[dev].load(std::memory_order_acquire) >= bytes) return 0;
  if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      e != hipSuccess)
    return (int)e;
  granted[dev].store(bytes, std::memory_order_release);
  return 0;
}

// Process-wide switches of moe_a2a_set_option; 0 = automatic.
std::atomic<int> g_option[MOE_A2A_OPT_COUNT];
inline int option(int which) { return g_option[which].load(std::memory_order_relaxed); }

// Combine at cache-resident sizes: about four workgroups per CU (1024 in all) finish sooner than
// fewer, wider ones (256 tokens of 896 vectors: 4 x 224 lanes 6.4 us, 2 x 448 lanes 6.7 us); a
// workgroup keeps at least 128 lanes.  Streaming sizes keep the widest workgroups (512 lanes).
// MOE_A2A_OPT_COMBINE_LANES / _VPL override both (measurements).
// The XCD-aware workgroup map of the combine (see combine_body): cache-resident sizes only.
bool combine_xcd_map(int T, int nsplit, bool streaming) {
  return !streaming && option(MOE_A2A_OPT_COMBINE_PLAIN_MAP) == 0 &&
         ((long long)T + kXcds) * nsplit < (long long)INT32_MAX;
}

CombineGeom combine_geom(int nvec, int T, bool streaming) {
  CombineGeom g;
  g.vpl = 1;
  if (const int lanes = option(MOE_A2A_OPT_COMBINE_LANES)) {
    g.vpl = option(MOE_A2A_OPT_COMBINE_VPL) == 2 && !streaming ? 2 : 1;
    g.per = std::min(std::max(lanes, 1), kRowMaxThreads);
    g.nsplit = ceil_div(nvec, g.per * g.vpl);
  } else if (streaming) {
    const RowGeom r = row_geom(nvec);
    g.per = r.per;
    g.nsplit = r.nsplit;
  } else {
    int nsplit = ceil_div(1024, T > 0 ? T : 1);
    if (nsplit > nvec / 128) nsplit = nvec / 128;
    const int least = ceil_div(nvec, kRowMaxThreads);
    if (nsplit < least) nsplit = least;
    g.nsplit = nsplit;
    g.per = ceil_div(nvec, nsplit);
  }
  g.threads = ceil_div(g.per, kWave) * kWave;
  return g;
}

// Routing of a table beyond kRouteTilesMaxRows entries: two launches (three beyond
// kRouteFoldMaxTiles tiles) around the tile-major count matrix `tile` (ceil(R / 1024) x E ints).
int route_large(const RouteArgs& a, int32_t* tile, hipStream_t stream) {
  const size_t lds_w = (size_t)kRouteWaves * a.E * sizeof(int);
  const size_t lds_starts = (size_t)(a.W + 1) * sizeof(int);
  const int ntiles = ceil_div(a.R, kRouteThreads);
  if (int rc = ensure_lds<route_hist_kernel>(lds_w)) return rc;
  if (int rc = launch(KID_ROUTE_HIST, route_hist_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w, stream, a, tile))
    return rc;
  if (ntiles <= kRouteFoldMaxTiles) {  // scan folded into the rank launch
    if (int rc = ensure_lds<route_rank_fold_kernel>(lds_w + lds_starts)) return rc;
    return launch(KID_ROUTE_RANK, route_rank_fold_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w + lds_starts,
                  stream, a, (const int32_t*)tile, ntiles);
  }
  if (int rc = launch(KID_ROUTE_SCAN, route_scan_kernel, dim3(1), dim3(kRouteThreads), 0, stream, tile, a.E, ntiles,
                      a.counts, a.offsets))
    return rc;
  if (int rc = ensure_lds<route_rank_kernel>(lds_w + lds_starts)) return rc;
  return launch(KID_ROUTE_RANK, route_rank_kernel, dim3(ntiles), dim3(kRouteThreads), lds_w + lds_starts, stream, a,
                (const int32_t*)tile);
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
    case MOE_A2A_E_CAPACITY:
      return "moe_a2a: routing table too large for the static scratch of moe_a2a_route_noalloc "
             "(ceil(T*K/1024) * E must not exceed moe_a2a_route_noalloc_max_ints())";
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

// Which kernel moe_a2a_route launches first for this shape (host logic only, no GPU needed).
static int route_first_kernel(int T, int K) {
  const long long R = (long long)T * K;
  if (R == 0) return KID_ROUTE_EMPTY;
  return R <= kRouteTilesMaxRows ? KID_ROUTE_TILES : KID_ROUTE_HIST;
}

// Device address of `scratch` on the current device, resolved once per device (each GPU holds its
// own copy of the array at its own address).
static int static_scratch(int32_t** out) {
  static std::atomic<int32_t*> resolved[kMaxDevices];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MOE_A2A_E_STATE;
  int32_t* p = resolved[dev].load(std::memory_order_acquire);
  if (!p) {
    void* addr = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)); e != hipSuccess) return (int)e;
    if (!addr) return MOE_A2A_E_STATE;
    p = static_cast<int32_t*>(addr);
    resolved[dev].store(p, std::memory_order_release);  // racing first calls resolve the same address
  }
  *out = p;
  return 0;
}

// workspace == nullptr and static_ok: the count matrix of a large table goes to the static scratch
static int route_impl(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                      int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot,
                      int32_t* meta, int32_t* status, void* workspace, size_t workspace_bytes, bool static_ok,
                      moe_a2a_stream_t stream_, int32_t* clear_status = nullptr) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (max_recv < 0 || (long long)max_recv * E > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  // No token: counts and offsets are zero and nothing else is written.  A kernel of its own, which
  // is never handed `indices` (NULL is allowed here), does that.
  if (T == 0)
    return launch(KID_ROUTE_EMPTY, route_empty_kernel, dim3(1), dim3(kRouteThreads), 0, stream, counts, offsets, E,
                  clear_status);
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), max_recv, counts, offsets,
              slot_of_entry, src_of_slot, meta, status, clear_status};
  const size_t lds_w = (size_t)kRouteWaves * E * sizeof(int);
  const size_t lds_starts = (size_t)(W + 1) * sizeof(int);
  if (a.R <= kRouteTilesMaxRows) {
    size_t lds = lds_w + (size_t)kRouteCopies * route_copy_stride(E) * sizeof(int) + (kRouteWaves + 1) * sizeof(int) +
                 lds_starts;
    if (int rc = ensure_lds<route_tiles_kernel>(lds)) return rc;
    return launch(KID_ROUTE_TILES, route_tiles_kernel, dim3(ceil_div(a.R, kRouteThreads)), dim3(kRouteThreads), lds,
                  stream, a);
  }
  if (static_ok) {
    const size_t need = (size_t)ceil_div(a.R, kRouteThreads) * (size_t)E;
    if (need > kStaticScratchInts) return MOE_A2A_E_CAPACITY;
    int32_t* tile = nullptr;
    if (int rc = static_scratch(&tile)) return rc;
    return route_large(a, tile, stream);
  }
  if (!workspace || workspace_bytes < moe_a2a_workspace_bytes(T, K, E)) return MOE_A2A_E_WORKSPACE;
  return route_large(a, (int32_t*)workspace, stream);
}

int moe_a2a_route(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                  int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot,
                  int32_t* meta, int32_t* status, void* workspace, size_t workspace_bytes,
                  moe_a2a_stream_t stream) {
  return route_impl(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry, src_of_slot,
                    meta, status, workspace, workspace_bytes, false, stream);
}

int moe_a2a_route_noalloc(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                          int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry,
                          int32_t* src_of_slot, int32_t* meta, int32_t* status, moe_a2a_stream_t stream) {
  return route_impl(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry, src_of_slot,
                    meta, status, nullptr, 0, true, stream);
}

size_t moe_a2a_route_noalloc_max_ints(void) { return kStaticScratchInts; }

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

static int route_dispatch_impl(const void* x, const int32_t* indices, const int32_t* rank_start, int src_rank, int T,
                               int K, int E, int W, int H, int max_recv, int32_t* counts, int32_t* offsets,
                               int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta, int32_t* status,
                               void* disp_x, moe_a2a_stream_t stream_, int32_t* clear_status) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (max_recv < 0 || (long long)max_recv * E > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(x, disp_x, T, K, H, 8)) return rc;
  if (!counts || !offsets) return MOE_A2A_E_NULL;
  if (T > 0 && (!indices || !slot_of_entry || !src_of_slot || !meta)) return MOE_A2A_E_NULL;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), max_recv, counts, offsets,
              slot_of_entry, src_of_slot, meta, status, clear_status};
  const int nvec = H / 8;
  if (!fused_small_ok(T, K, H) || option(MOE_A2A_OPT_ROUTE_TILE) == 1) {  // token tiles: any table size
    if (T == 0) return route_impl(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry,
                                  src_of_slot, meta, status, nullptr, 0, false, stream_, clear_status);
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

int moe_a2a_route_dispatch(const void* x, const int32_t* indices, const int32_t* rank_start, int src_rank, int T,
                           int K, int E, int W, int H, int max_recv, int32_t* counts, int32_t* offsets,
                           int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta, int32_t* status,
                           void* disp_x, moe_a2a_stream_t stream) {
  return route_dispatch_impl(x, indices, rank_start, src_rank, T, K, E, W, H, max_recv, counts, offsets, slot_of_entry,
                             src_of_slot, meta, status, disp_x, stream, nullptr);
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

// Routing and the fp8 dispatch in one launch (route_dispatch_fp8_tile_kernel), for moe_a2a_forward: any
// table a tile kernel takes.  Every workgroup counts the whole table for itself, so the launch saves the
// launch boundary and the index arrays' round trip through memory, not the table pass: 56.1 against
// 9.4 + 48.5 us at 4096 tokens, top-8, 256 experts, H = 7168.  Tokens per workgroup: tiles of at most 64
// entries keep the slot arithmetic inside one wave (8 tokens of top-8: 56.1 us; 4: 57.9, 16: 62.5, 32:
// 79.5); more tokens per tile only beyond two workgroups per CU.
static bool route_dispatch_fp8_ok(int T, int K, int H) {
  return T > 0 && K <= kTileMaxOwn && H % MOE_A2A_FP8_BLOCK == 0;
}
static int fp8_tile_tokens(int T, int K) {
  const int cap = std::max(kTileMaxOwn / K, 1), wave = std::max(kWave / K, 1);
  const int forced = option(MOE_A2A_OPT_FP8_TILE);
  if (forced > 0) return std::min(forced, cap);
  return std::min(cap, std::max(wave, ceil_div(T, 2 * 256)));
}
static int route_dispatch_fp8_impl(const void* x, int x_type, const int32_t* indices, const int32_t* rank_start,
                                   int src_rank, int T, int K, int E, int W, int H, int max_recv, int32_t* counts,
                                   int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                                   int32_t* status, void* disp_q, float* disp_scale, int pow2, hipStream_t stream,
                                   int32_t* clear_status) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (max_recv < 0 || (long long)max_recv * E > (long long)INT32_MAX / 8) return MOE_A2A_E_SHAPE;
  if (int rc = check_rows(x, disp_q, T, K, H, MOE_A2A_FP8_BLOCK)) return rc;
  if (!counts || !offsets || !indices || !slot_of_entry || !src_of_slot || !meta || !disp_scale) return MOE_A2A_E_NULL;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), max_recv, counts, offsets,
              slot_of_entry, src_of_slot, meta, status, clear_status};
  const int nblk = H / MOE_A2A_FP8_BLOCK;
  const int tile = fp8_tile_tokens(T, K);
  // workgroups of 512 lanes, three to a CU, so that one's table pass runs under another's rows (a thread
  // per expert in the scan: 1024 lanes beyond 512 experts)
  const int threads = E <= 512 ? 512 : kTileThreads;
  dim3 grid((unsigned)ceil_div(T, tile)), block(threads);
  const bool st = streams(T, (long long)T * K, H, 2, 1);
#define RDF8_T(EL, ST, TH)                                                                                       \
  return launch(KID_ROUTE_DISPATCH_FP8, route_dispatch_fp8_tile_kernel<EL, ST, TH>, grid, block, 0, stream, a,   \
                (const uint4*)x, (uint4*)disp_q, disp_scale, nblk, tile, pow2)
#define RDF8(EL, ST)                         \
  {                                          \
    if (threads == 512) RDF8_T(EL, ST, 512); \
    RDF8_T(EL, ST, kTileThreads);            \
  }
  if (x_type == MOE_A2A_BF16) {
    if (st) RDF8(Bf16, 1);
    RDF8(Bf16, 0);
  }
  if (st) RDF8(F16, 1);
  RDF8(F16, 0);
#undef RDF8_T
#undef RDF8
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

// Output stores of a streaming combine.  Non-temporal ones keep the Infinity Cache (256 MB) for the
// dispatched rows that the next step's expert reads there; once those rows exceed that cache there
// is nothing to keep and write-through stores make the combine 4-7 % faster (measured by the wall
// clock of whole steps: 388 -> 385 us at 537 MB of dispatched rows, but 248 -> 252 us at 242 MB).
// `dispatched_bytes` is what the dispatch of the same step wrote.
static int combine_impl(const void* expert_y, const float* weights, const int32_t* slot_of_entry, int mode,
                        int elem_type, void* out, int T, int K, int H, long long dispatched_bytes,
                        moe_a2a_stream_t stream_);

int moe_a2a_combine(const void* expert_y, const float* weights, const int32_t* slot_of_entry, int mode,
                    int elem_type, void* out, int T, int K, int H, moe_a2a_stream_t stream_) {
  // the dispatch is not known here: take the expert rows for 16-bit copies of fp8 rows, half their size
  return combine_impl(expert_y, weights, slot_of_entry, mode, elem_type, out, T, K, H, (long long)T * K * H, stream_);
}

static int combine_impl(const void* expert_y, const float* weights, const int32_t* slot_of_entry, int mode,
                        int elem_type, void* out, int T, int K, int H, long long dispatched_bytes,
                        moe_a2a_stream_t stream_) {
  if (!known_type(elem_type)) return MOE_A2A_E_DTYPE;
  if (mode != MOE_A2A_COMBINE_STRICT && mode != MOE_A2A_COMBINE_F32) return MOE_A2A_E_DTYPE;
  if (int rc = check_rows(expert_y, out, T, K, H, 8)) return rc;
  if (T == 0) return 0;
  if (!weights || !slot_of_entry) return MOE_A2A_E_NULL;
  hipStream_t stream = (hipStream_t)stream_;
  const int nvec = H / 8;
  const bool st = streams((long long)T * K, T, H, 2, 2);
  const bool through = dispatched_bytes > (256ll << 20);
  const CombineGeom g = combine_geom(nvec, T, st);
  const int xcd_T = combine_xcd_map(T, g.nsplit, st) ? T : 0;
  dim3 grid((unsigned)(xcd_T ? ceil_div(T, kXcds) * kXcds : T) * g.nsplit), block(g.threads);
#define COMBINE_ARGS (const uint4*)expert_y, weights, slot_of_entry, (uint4*)out, K, nvec, g.per, g.nsplit, xcd_T
#define COMBINE_LAUNCH(EL, MD, KT)                                                                             \
  {                                                                                                            \
    if (st && through)                                                                                         \
      return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 2, 1>, grid, block, 0, stream, COMBINE_ARGS); \
    if (st) return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 1, 1>, grid, block, 0, stream, COMBINE_ARGS); \
    if (g.vpl == 2)                                                                                            \
      return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 0, 2>, grid, block, 0, stream, COMBINE_ARGS); \
    return launch(KID_COMBINE, combine_rows_kernel<EL, MD, KT, 0, 1>, grid, block, 0, stream, COMBINE_ARGS);   \
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
#undef COMBINE_ARGS
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
  const CombineGeom g = combine_geom(nvec, T, st);
  const int xcd_T = combine_xcd_map(T, g.nsplit, st) ? T : 0;
  dim3 grid((unsigned)(xcd_T ? ceil_div(T, kXcds) * kXcds : T) * g.nsplit), block(g.threads);
#define SC_ARGS                                                                                              \
  (const uint4*)disp, indices, weights, slot_of_entry, (uint4*)out, stub_kind, E, E_l, K, nvec, g.per, g.nsplit, \
      xcd_T
#define SC_LAUNCH(IN, OUT, MD, KT)                                                                            \
  {                                                                                                           \
    if (st)                                                                                                   \
      return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD, KT, 1, 1>, grid, block, 0, stream, \
                    SC_ARGS);                                                                                 \
    if (g.vpl == 2)                                                                                           \
      return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD, KT, 0, 2>, grid, block, 0, stream, \
                    SC_ARGS);                                                                                 \
    return launch(KID_STUB_COMBINE, stub_combine_rows_kernel<IN, OUT, MD, KT, 0, 1>, grid, block, 0, stream,  \
                  SC_ARGS);                                                                                   \
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
#undef SC_ARGS
}
#undef MOE_A2A_SWITCH_KT

// The whole path in one launch (forward_token_kernel): small routing tables, 16-bit rows of one
// element type, compact layout, stub folded in.
// 0: no; 1: one token per workgroup (forward_token_kernel); 2: a tile of tokens per workgroup
// (forward_tile_kernel), wherever moe_a2a_route_dispatch would take its token-tile kernel by itself.
static int forward_one_launch_form(int T, int K, int H, int max_recv, int in_type, int out_type, int fp8_dispatch) {
  if (fp8_dispatch || max_recv > 0 || in_type != out_type || T < 1) return 0;
  if (option(MOE_A2A_OPT_TWO_LAUNCHES) == 1 || !moe_a2a_fused_ok(T, K, H)) return 0;
  if (fused_small_ok(T, K, H) && option(MOE_A2A_OPT_ROUTE_TILE) != 1) {
    const RowGeom g = fused_geom(H / 8, T * K);
    if (fused_entries_per_thread(T * K, g.threads) <= 8) return 1;
  }
  return K <= kTileMaxOwn ? 2 : 0;
}
static bool forward_one_launch_ok(int T, int K, int H, int max_recv, int in_type, int out_type, int fp8_dispatch) {
  return forward_one_launch_form(T, K, H, max_recv, in_type, out_type, fp8_dispatch) != 0;
}

// Routing by its own launches, then dispatch and fold of each token in one kernel (dispatch_fold_kernel):
// 16-bit rows of one element type, compact layout, stub folded in, wherever routing and dispatch
// would be separate launches anyway.
static bool dispatch_fold_ok(int T, int K, int H, int max_recv, int in_type, int out_type, int fp8_dispatch,
                             int fuse_route) {
  if (max_recv > 0 || in_type != out_type || T < 1) return false;
  if (option(MOE_A2A_OPT_TWO_LAUNCHES) == 1) return false;
  // The fold behind an fp8 dispatch is routed by a launch of its own.  It pays while the rows stay in
  // the caches (one launch boundary less); at streaming volumes two kernels (routing + dispatch in one,
  // then stub + combine) move the same bytes about 1 % faster (120.0 against 118.8 us at 16384 tokens,
  // top-8, H = 7168).
  if (fp8_dispatch) return !streams(T, 2ll * T * K, H, 2, 1);
  return !(fuse_route == 2 ? K <= kTileMaxOwn : (fuse_route == 1 && moe_a2a_fused_ok(T, K, H)));
}

static int dispatch_fold_fp8(const void* x, const int32_t* indices, const float* weights,
                             const int32_t* slot_of_entry, void* disp_q, float* disp_scale, void* out, int T, int K,
                             int E, int W, int H, int elem_type, int stub_kind, int combine_mode, int pow2,
                             hipStream_t stream) {
  if (int rc = check_rows(x, disp_q, T, K, H, MOE_A2A_FP8_BLOCK)) return rc;
  if (!aligned16(out)) return MOE_A2A_E_ALIGN;
  if (!indices || !weights || !slot_of_entry || !disp_scale || !out) return MOE_A2A_E_NULL;
  const int nblk = H / MOE_A2A_FP8_BLOCK, E_l = E / W;
  const RowGeom g = row_geom(nblk * 8, 8);  // cache-resident volumes only: see dispatch_fold_ok
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
#define DF8_ARGS                                                                                                  \
  (const uint4*)x, indices, weights, slot_of_entry, (uint4*)disp_q, disp_scale, (uint4*)out, stub_kind, E, E_l, K, \
      nblk, g.per, g.nsplit, pow2
#define DF84(EL, MD, KT) \
  return launch(KID_DISPATCH_FOLD, dispatch_fold_fp8_kernel<EL, MD, KT, 0>, grid, block, 0, stream, DF8_ARGS);
#define DF83(EL, MD)             \
  {                              \
    switch (K) {                 \
      case 8: DF84(EL, MD, 8)    \
      default: DF84(EL, MD, 0)   \
    }                            \
  }
#define DF82(EL)                                                        \
  {                                                                     \
    if (combine_mode == MOE_A2A_COMBINE_STRICT) DF83(EL, MOE_A2A_COMBINE_STRICT) \
    DF83(EL, MOE_A2A_COMBINE_F32)                                       \
  }
  if (elem_type == MOE_A2A_BF16) DF82(Bf16)
  DF82(F16)
#undef DF82
#undef DF83
#undef DF84
#undef DF8_ARGS
}

static int dispatch_fold(const void* x, const int32_t* indices, const float* weights, const int32_t* slot_of_entry,
                         void* disp, void* out, int T, int K, int E, int W, int H, int elem_type, int stub_kind,
                         int combine_mode, hipStream_t stream) {
  if (int rc = check_rows(x, disp, T, K, H, 8)) return rc;
  if (!aligned16(out)) return MOE_A2A_E_ALIGN;
  if (!indices || !weights || !slot_of_entry || !out) return MOE_A2A_E_NULL;
  const int nvec = H / 8, E_l = E / W;
  const bool st = streams(T, 2ll * T * K + T, H, 2, 2);
  const RowGeom g = row_geom(nvec);
  dim3 grid((unsigned)T * g.nsplit), block(g.threads);
#define DF_ARGS                                                                                                   \
  (const uint4*)x, indices, weights, slot_of_entry, (uint4*)disp, (uint4*)out, stub_kind, E, E_l, K, nvec, g.per, \
      g.nsplit
#define DF4(EL, MD, KT)                                                                                            \
  {                                                                                                                \
    if (st) return launch(KID_DISPATCH_FOLD, dispatch_fold_kernel<EL, MD, KT, 2>, grid, block, 0, stream, DF_ARGS); \
    return launch(KID_DISPATCH_FOLD, dispatch_fold_kernel<EL, MD, KT, 0>, grid, block, 0, stream, DF_ARGS);        \
  }
#define DF3(EL, MD)              \
  {                              \
    switch (K) {                 \
      case 4: DF4(EL, MD, 4)     \
      case 8: DF4(EL, MD, 8)     \
      default: DF4(EL, MD, 0)    \
    }                            \
  }
#define DF2(EL)                                                        \
  {                                                                    \
    if (combine_mode == MOE_A2A_COMBINE_STRICT) DF3(EL, MOE_A2A_COMBINE_STRICT) \
    DF3(EL, MOE_A2A_COMBINE_F32)                                       \
  }
  if (elem_type == MOE_A2A_BF16) DF2(Bf16)
  DF2(F16)
#undef DF2
#undef DF3
#undef DF4
#undef DF_ARGS
}

int moe_a2a_forward_launches(int T, int K, int H, int max_recv, int in_type, int out_type, int fp8_dispatch,
                             int fuse_route, int fuse_stub) {
  if (T <= 0) return 0;
  if (fuse_stub && fuse_route && forward_one_launch_ok(T, K, H, max_recv, in_type, out_type, fp8_dispatch)) return 1;
  if (fuse_stub && dispatch_fold_ok(T, K, H, max_recv, in_type, out_type, fp8_dispatch, fuse_route)) {
    const long long R = (long long)T * K;
    if (R <= kRouteTilesMaxRows) return 2;
    return ceil_div((int)std::min<long long>(R, INT32_MAX), kRouteThreads) <= kRouteFoldMaxTiles ? 3 : 4;
  }
  const bool fused = fp8_dispatch ? (fuse_route && route_dispatch_fp8_ok(T, K, H))
                                  : (fuse_route == 2 ? K <= kTileMaxOwn : (fuse_route == 1 && moe_a2a_fused_ok(T, K, H)));
  int n = fused ? 1 : 2;  // routing + dispatch
  if (!fused) {
    const long long R = (long long)T * K;
    if (R > kRouteTilesMaxRows) n += ceil_div((int)std::min<long long>(R, INT32_MAX), kRouteThreads) <= kRouteFoldMaxTiles ? 1 : 2;
  }
  return n + (fuse_stub ? 1 : 2);
}

static int forward_one_launch(const void* x, const int32_t* indices, const float* weights, const int32_t* rank_start,
                              int src_rank, int T, int K, int E, int W, int H, int elem_type, int stub_kind,
                              int combine_mode, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry,
                              int32_t* src_of_slot, int32_t* meta, int32_t* status, void* disp, void* out,
                              hipStream_t stream, int32_t* clear_status) {
  if (int rc = check_route_shape(T, K, E, W)) return rc;
  if (int rc = check_rows(x, disp, T, K, H, 8)) return rc;
  if (!aligned16(out)) return MOE_A2A_E_ALIGN;
  if (!counts || !offsets || !indices || !weights || !slot_of_entry || !src_of_slot || !meta || !out)
    return MOE_A2A_E_NULL;
  RouteArgs a{indices, rank_start, src_rank, T, K, E, W, T * K, id_bits(E), 0, counts, offsets,
              slot_of_entry, src_of_slot, meta, status, clear_status};
  const int nvec = H / 8;
  const int E_l = E / W;
  if (forward_one_launch_form(T, K, H, 0, elem_type, elem_type, 0) == 2) {
    const int tile = tile_tokens(T, K, H);
    dim3 grid((unsigned)ceil_div(T, tile)), block(kTileThreads);
#define FWT_ARGS a, (const uint4*)x, (uint4*)disp, weights, (uint4*)out, stub_kind, E_l, nvec, tile
#define FWT3(EL, MD)                                                                                              \
  {                                                                                                               \
    switch (K) {                                                                                                  \
      case 4: return launch(KID_FORWARD_TILE, forward_tile_kernel<EL, MD, 4>, grid, block, 0, stream, FWT_ARGS);  \
      case 6: return launch(KID_FORWARD_TILE, forward_tile_kernel<EL, MD, 6>, grid, block, 0, stream, FWT_ARGS);  \
      case 8: return launch(KID_FORWARD_TILE, forward_tile_kernel<EL, MD, 8>, grid, block, 0, stream, FWT_ARGS);  \
      default: return launch(KID_FORWARD_TILE, forward_tile_kernel<EL, MD, 0>, grid, block, 0, stream, FWT_ARGS); \
    }                                                                                                             \
  }
#define FWT2(EL)                                                        \
  {                                                                     \
    if (combine_mode == MOE_A2A_COMBINE_STRICT) FWT3(EL, MOE_A2A_COMBINE_STRICT) \
    FWT3(EL, MOE_A2A_COMBINE_F32)                                       \
  }
    if (elem_type == MOE_A2A_BF16) FWT2(Bf16)
    FWT2(F16)
#undef FWT2
#undef FWT3
#undef FWT_ARGS
  }
  const RowGeom g = fused_geom(nvec, T * K);
  const int vpl = fused_vectors_per_lane(nvec);
  const int ept = fused_entries_per_thread(T * K, g.threads);
  dim3 grid((unsigned)T * g.nsplit + 1), block(g.threads);
#define FWD_ARGS a, (const uint4*)x, (uint4*)disp, weights, (uint4*)out, stub_kind, E_l, nvec, g.per, g.nsplit
#define FWD4(EPT, VPL, EL, MD)                                                                                   \
  {                                                                                                              \
    if (K == 8)                                                                                                  \
      return launch(KID_FORWARD_TOKEN, forward_token_kernel<EPT, VPL, EL, MD, 8>, grid, block, 0, stream, FWD_ARGS); \
    return launch(KID_FORWARD_TOKEN, forward_token_kernel<EPT, VPL, EL, MD, 0>, grid, block, 0, stream, FWD_ARGS); \
  }
#define FWD3(EPT, VPL, EL)                                                      \
  {                                                                             \
    if (combine_mode == MOE_A2A_COMBINE_STRICT) FWD4(EPT, VPL, EL, MOE_A2A_COMBINE_STRICT) \
    FWD4(EPT, VPL, EL, MOE_A2A_COMBINE_F32)                                     \
  }
#define FWD2(EPT, VPL)                          \
  {                                             \
    if (elem_type == MOE_A2A_BF16) FWD3(EPT, VPL, Bf16) \
    FWD3(EPT, VPL, F16)                         \
  }
#define FWD1(EPT)             \
  {                           \
    if (vpl == 2) FWD2(EPT, 2) \
    FWD2(EPT, 1)              \
  }
  if (ept == 4) FWD1(4)
  FWD1(8)
#undef FWD1
#undef FWD2
#undef FWD3
#undef FWD4
#undef FWD_ARGS
}

static int forward_impl(const void* x, const int32_t* indices, const float* weights, const int32_t* rank_start,
                        int src_rank, int T, int K, int E, int W, int H, int max_recv, int in_type, int out_type,
                        int fp8_dispatch, int stub_kind, int combine_mode, int fuse_route, int fuse_stub,
                        int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                        int32_t* status, void* disp, float* disp_scale, void* expert_y, void* out, void* workspace,
                        size_t workspace_bytes, moe_a2a_stream_t stream, int32_t* clear_status) {
  if (!known_type(in_type) || !known_type(out_type)) return MOE_A2A_E_DTYPE;
  if (fp8_dispatch < 0 || fp8_dispatch > 2) return MOE_A2A_E_DTYPE;
  if (fp8_dispatch && !disp_scale) return MOE_A2A_E_NULL;
  if (!fuse_stub && T > 0 && !expert_y) return MOE_A2A_E_NULL;
  if (stub_kind != MOE_A2A_STUB_OWNER_RANK && stub_kind != MOE_A2A_STUB_EXPERT_FRACTION) return MOE_A2A_E_DTYPE;
  if (combine_mode != MOE_A2A_COMBINE_STRICT && combine_mode != MOE_A2A_COMBINE_F32) return MOE_A2A_E_DTYPE;
  if (T > 0 && fuse_stub && fuse_route &&
      forward_one_launch_ok(T, K, H, max_recv, in_type, out_type, fp8_dispatch))
    return forward_one_launch(x, indices, weights, rank_start, src_rank, T, K, E, W, H, in_type, stub_kind,
                              combine_mode, counts, offsets, slot_of_entry, src_of_slot, meta, status, disp, out,
                              (hipStream_t)stream, clear_status);
  if (T > 0 && fuse_stub && dispatch_fold_ok(T, K, H, max_recv, in_type, out_type, fp8_dispatch, fuse_route)) {
    if (int rc = route_impl(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry,
                            src_of_slot, meta, status, workspace, workspace_bytes, false, stream, clear_status))
      return rc;
    if (fp8_dispatch)
      return dispatch_fold_fp8(x, indices, weights, slot_of_entry, disp, disp_scale, out, T, K, E, W, H, in_type,
                               stub_kind, combine_mode, fp8_dispatch == 2, (hipStream_t)stream);
    return dispatch_fold(x, indices, weights, slot_of_entry, disp, out, T, K, E, W, H, in_type, stub_kind,
                         combine_mode, (hipStream_t)stream);
  }
  const bool fused = !fp8_dispatch && T > 0 &&
                     (fuse_route == 2 ? K <= kTileMaxOwn : (fuse_route == 1 && moe_a2a_fused_ok(T, K, H)));
  if (fused) {
    if (int rc = route_dispatch_impl(x, indices, rank_start, src_rank, T, K, E, W, H, max_recv, counts, offsets,
                                     slot_of_entry, src_of_slot, meta, status, disp, stream, clear_status))
      return rc;
  } else if (fp8_dispatch && fuse_route && route_dispatch_fp8_ok(T, K, H)) {
    if (int rc = route_dispatch_fp8_impl(x, in_type, indices, rank_start, src_rank, T, K, E, W, H, max_recv, counts,
                                         offsets, slot_of_entry, src_of_slot, meta, status, disp, disp_scale,
                                         fp8_dispatch == 2, (hipStream_t)stream, clear_status))
      return rc;
  } else {
    if (int rc = route_impl(indices, rank_start, src_rank, T, K, E, W, max_recv, counts, offsets, slot_of_entry,
                            src_of_slot, meta, status, workspace, workspace_bytes, false, stream, clear_status))
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
  return combine_impl(expert_y, weights, slot_of_entry, combine_mode, out_type, out, T, K, H,
                      (long long)T * K * H * (fp8_dispatch ? 1 : 2), stream);
}

int moe_a2a_forward(const void* x, const int32_t* indices, const float* weights, const int32_t* rank_start,
                    int src_rank, int T, int K, int E, int W, int H, int max_recv, int in_type, int out_type,
                    int fp8_dispatch, int stub_kind, int combine_mode, int fuse_route, int fuse_stub,
                    int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                    int32_t* status, void* disp, float* disp_scale, void* expert_y, void* out, void* workspace,
                    size_t workspace_bytes, moe_a2a_stream_t stream) {
  return forward_impl(x, indices, weights, rank_start, src_rank, T, K, E, W, H, max_recv, in_type, out_type,
                      fp8_dispatch, stub_kind, combine_mode, fuse_route, fuse_stub, counts, offsets, slot_of_entry,
                      src_of_slot, meta, status, disp, disp_scale, expert_y, out, workspace, workspace_bytes, stream,
                      nullptr);
}

int moe_a2a_forward_packed(const moe_a2a_forward_args* a) {
  if (!a) return MOE_A2A_E_NULL;
  return forward_impl(a->x, a->indices, a->weights, a->rank_start, a->src_rank, a->T, a->K, a->E, a->W, a->H,
                         a->max_recv, a->in_type, a->out_type, a->fp8_dispatch, a->stub_kind, a->combine_mode,
                         a->fuse_route, a->fuse_stub, a->counts, a->offsets, a->slot_of_entry, a->src_of_slot, a->meta,
                      a->status, a->disp, a->disp_scale, a->expert_y, a->out, a->workspace, a->workspace_bytes,
                      a->stream, a->clear_status);
}

#include "expert_gemm_entry.inc"
#include "gemm_rs_entry.inc"

const char* moe_a2a_route_plan(int T, int K) {
  if (T < 0 || K < 1) return "unknown";
  return kKernelNames[route_first_kernel(T, K)];
}

int moe_a2a_set_option(int which, int value) {
  if (which < 0 || which >= MOE_A2A_OPT_COUNT) return MOE_A2A_E_DTYPE;
  if (value < 0) return MOE_A2A_E_SHAPE;  // no option takes a negative value, so a return below zero is always an error
  return g_option[which].exchange(value, std::memory_order_relaxed);
}

int moe_a2a_get_option(int which) {
  if (which < 0 || which >= MOE_A2A_OPT_COUNT) return MOE_A2A_E_DTYPE;
  return option(which);
}

int moe_a2a_timer_begin(int capacity) {
  std::lock_guard<std::mutex> hold(g_timer_mutex);
  if (g_timer.active || capacity < 1) return MOE_A2A_E_STATE;
  g_timer.start = new hipEvent_t[capacity];
  g_timer.stop = new hipEvent_t[capacity];
  g_timer.ids = new int[capacity];
  const unsigned flags = (unsigned)option(MOE_A2A_OPT_TIMER_EVENT_FLAGS);
  for (int i = 0; i < capacity; ++i) {
    hipError_t e1 = hipEventCreateWithFlags(&g_timer.start[i], flags);
    hipError_t e2 = e1 == hipSuccess ? hipEventCreateWithFlags(&g_timer.stop[i], flags) : e1;
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
  g_timer.skip = 0;
  g_timer.active = true;
  g_timer_on.store(true, std::memory_order_release);
  return 0;
}

int moe_a2a_timer_skip(int launches) {
  std::lock_guard<std::mutex> hold(g_timer_mutex);
  if (!g_timer.active || launches < 0) return MOE_A2A_E_STATE;
  g_timer.skip = launches;
  return 0;
}

int moe_a2a_timer_end(int* kernel_ids, float* microseconds, int n) {
  std::lock_guard<std::mutex> hold(g_timer_mutex);
  if (!g_timer.active) return MOE_A2A_E_STATE;
  g_timer.active = false;
  g_timer_on.store(false, std::memory_order_release);
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
