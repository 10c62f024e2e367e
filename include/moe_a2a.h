/*
 * moe_a2a.h -- C ABI of the MI355X (gfx950) MoE all-to-all dispatch/combine library.
 *
 * One GPU holds the whole emulated world: the W destination ranks are partitions of
 * one compact, expert-major buffer.  A routed row ("entry") is the triple
 * (source rank, token, k); entries are numbered i = t*K + k over the tokens of all
 * source ranks concatenated in rank order.  Entry i lives at row
 *
 *     slot_of_entry[i] = offsets[e_i] + #{ j < i : e_j == e_i }
 *
 * of disp_x[R,H], R = T*K, which is slot (owner rank e/E_l, local expert e%E_l,
 * position j) of the reference's padded [E_l, max_recv, H] buffers
 * (all2all/reference.py:123-146).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer into caller-owned memory unless marked host;
 *   - the library allocates nothing, never synchronises, reads no environment variable and
 *     keeps no mutable state besides the opt-in launch timer and the option switches at the
 *     end of this file (both off unless the caller turns them on: a launch then reads one atomic
 *     flag and nothing else that is shared); every launch goes to the stream passed in, so a call
 *     sequence can be captured into a hipGraph;
 *   - return value: 0 success, < 0 argument error found on the host before any
 *     launch (MOE_A2A_E_*), > 0 a hipError_t reported by the launch.
 */
#ifndef MOE_A2A_H_
#define MOE_A2A_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_A2A_ABI_VERSION 5

/* element types of activations */
#define MOE_A2A_F16 0
#define MOE_A2A_BF16 1

/* expert stub flavours */
#define MOE_A2A_STUB_OWNER_RANK 0      /* y = x * (1 + e / E_l)   all2all/reference.py:262 */
#define MOE_A2A_STUB_EXPERT_FRACTION 1 /* y = x * f32((1 + e) / E)                          */

/* combine arithmetic */
#define MOE_A2A_COMBINE_STRICT 0 /* ascending slot order, round to out type after every add */
#define MOE_A2A_COMBINE_F32 1    /* k order, f32 accumulator, one final rounding            */

/* limits */
#define MOE_A2A_MAX_EXPERTS 1024
#define MOE_A2A_MAX_TOPK 32
#define MOE_A2A_MAX_WORLD 256
#define MOE_A2A_META_DIM 5
#define MOE_A2A_FP8_BLOCK 128
/* scale of an fp8 block: amax / 448 in f32, or that rounded up to a power of two */
#define MOE_A2A_FP8_SCALE_F32 0
#define MOE_A2A_FP8_SCALE_POW2 1

/* bits of the status word the routing entry points write (OR-ed into what the word holds: a call
 * that meets both conditions reports both, and the word keeps what earlier calls raised until its
 * owner clears it -- by a fill of its own, or without a launch through
 * moe_a2a_forward_args.clear_status) */
#define MOE_A2A_STATUS_BAD_EXPERT 1 /* an expert id was outside [0, E) and has been clamped      */
#define MOE_A2A_STATUS_OVERFLOW 2   /* padded layout: an expert has more than max_recv entries   */

/* argument errors */
#define MOE_A2A_E_NULL (-1)      /* a required pointer is NULL                       */
#define MOE_A2A_E_SHAPE (-2)     /* T, K, E, W or H out of range / not divisible      */
#define MOE_A2A_E_DTYPE (-3)     /* unknown element type, stub kind or combine mode   */
#define MOE_A2A_E_WORKSPACE (-4) /* workspace missing or smaller than workspace_bytes */
#define MOE_A2A_E_ALIGN (-5)     /* a row buffer is not 16-byte aligned               */
#define MOE_A2A_E_STATE (-6)     /* launch timer used out of order                    */
#define MOE_A2A_E_CAPACITY (-7)  /* table beyond the static scratch of moe_a2a_route_noalloc */

typedef void* moe_a2a_stream_t; /* hipStream_t */

int moe_a2a_abi_version(void);

/* Text for any value the functions below return (host pointer, static storage). */
const char* moe_a2a_strerror(int code);

/* Bytes of scratch moe_a2a_route needs for T tokens, top-K, E experts. */
size_t moe_a2a_workspace_bytes(int T, int K, int E);

/*
 * Routing: histogram + exclusive prefix sum + stable permutation.
 * Replaces all2all/reference.py:72-91 (bucketing, counts), :100-105 (meta rows) and
 * :123-146 (arrival-order slotting per local expert).
 *
 *   indices[T,K]         expert id of every entry, 0 <= e < E
 *   rank_start[W+1]      first token of each source rank in the concatenated world, or
 *                        NULL: then all T tokens belong to source rank `src_rank`
 *   counts[E]            rows per expert            (= expert_num_tokens of every rank)
 *   offsets[E+1]         exclusive prefix sum of counts; offsets[E] = R
 *   slot_of_entry[R]     entry -> row of the compact layout
 *   src_of_slot[R]       row -> entry (inverse permutation)
 *   meta[R,5]            per row: [e, source rank, token within its rank, k, 0]
 *                        (all2all/reference.py:85)
 *   status               optional int32[1], cleared by the caller: MOE_A2A_STATUS_BAD_EXPERT is
 *                        OR-ed in if an expert id was out of range (such ids are clamped into
 *                        [0,E) so no access goes out of bounds), MOE_A2A_STATUS_OVERFLOW as below
 *   max_recv             0: compact layout, rows of all experts back to back (R rows).
 *                        > 0: the reference's padded layout (all2all/reference.py:65,127-136):
 *                        expert e owns rows [e*max_recv, (e+1)*max_recv), its j-th entry sits at
 *                        e*max_recv + j, so disp_x / meta / src_of_slot have E*max_recv rows and,
 *                        viewed as [W, E_l, max_recv, .], are the expert_x / expert_meta of every
 *                        owner rank; rows past counts[e] are not written.  slot_of_entry then
 *                        holds these physical rows, which is all dispatch and combine follow.
 *                        An expert with more than max_recv entries raises MOE_A2A_STATUS_OVERFLOW
 *                        (the extra entries are folded onto the segment's last row; counts stay
 *                        the true numbers).
 * T == 0 (indices may then be NULL): counts and offsets are written as zeros by a kernel that is
 * never handed the routing table; nothing else is written.
 */
int moe_a2a_route(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                  int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot,
                  int32_t* meta, int32_t* status, void* workspace, size_t workspace_bytes,
                  moe_a2a_stream_t stream);

/*
 * Dispatch: disp_x[slot_of_entry[t*K+k], :] = x[t, :] for every k.  Each token row is read
 * once and stored K times.  Pure copy of 16-bit elements (H % 8 == 0).
 * Replaces all2all/reference.py:93-112 (send-buffer gather + exchange) and :144.
 */
int moe_a2a_dispatch(const void* x, const int32_t* slot_of_entry, void* disp_x, int T, int K, int H,
                     moe_a2a_stream_t stream);

/*
 * moe_a2a_route for callers that cannot allocate and have no workspace to hand in: code under hipGraph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose torch code allocates in every call).  Same arguments, kernels and results as
 * moe_a2a_route, minus the workspace: the (tile, expert) count matrix that routing of more than 32 768
 * entries needs lives in a static device array of the library instead (4 MiB per GPU, held until the
 * process ends; smaller tables need no scratch at all).  The call allocates and frees nothing.
 *   limit   ceil(T*K / 1024) * E <= moe_a2a_route_noalloc_max_ints() (2^20), else MOE_A2A_E_CAPACITY
 *           and nothing is launched
 *   sharing every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU (two
 *           streams, two threads) race on it; calls on one stream do not.  Nothing has to be cleared
 *           between calls: every cell a call reads, the same call has written.
 *   set-up  the array's address is looked up on the first call on each device (no stream work, no
 *           allocation); make that first call outside graph capture.
 */
int moe_a2a_route_noalloc(const int32_t* indices, const int32_t* rank_start, int src_rank, int T, int K, int E, int W,
                          int max_recv, int32_t* counts, int32_t* offsets, int32_t* slot_of_entry,
                          int32_t* src_of_slot, int32_t* meta, int32_t* status, moe_a2a_stream_t stream);
size_t moe_a2a_route_noalloc_max_ints(void);

/*
 * Name of the kernel moe_a2a_route launches first for T tokens of top-K ("route_empty",
 * "route_tiles" or "route_hist"): host logic only, usable without a GPU (the reference has no
 * counterpart; a caller sizing its workspace, or a test, asks which form a shape takes).
 */
const char* moe_a2a_route_plan(int T, int K);

/*
 * Routing and dispatch in ONE launch: every workgroup derives the slots of its own tokens from
 * the routing table, so no routing kernel has to finish first and no workspace is needed.
 * Outputs as moe_a2a_route + moe_a2a_dispatch.  Two kernels behind it: one token per workgroup
 * for small tables, a tile of tokens per workgroup (at most 256 entries, so K <= 256) otherwise;
 * any table size is accepted.
 */
int moe_a2a_fused_max_rows(void); /* largest R = T*K the one-launch form takes */
/* 1 if moe_a2a_route_dispatch is the faster choice for this shape: always for cache-resident
 * sizes; at streaming sizes (more than ~192 MB moved) separate routing and dispatch win. */
int moe_a2a_fused_ok(int T, int K, int H);
int moe_a2a_route_dispatch(const void* x, const int32_t* indices, const int32_t* rank_start, int src_rank, int T,
                           int K, int E, int W, int H, int max_recv, int32_t* counts, int32_t* offsets,
                           int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta, int32_t* status,
                           void* disp_x, moe_a2a_stream_t stream);

/*
 * fp8 dispatch: quantise each token row once to e4m3fn with one f32 scale per 128 columns
 * (scale = amax/448, 1 if amax == 0; q = rne_e4m3(x / scale)), then store row and scales at
 * the K slots.  x is MOE_A2A_F16 or MOE_A2A_BF16, H % 128 == 0.  The reference has no fp8
 * path; the arithmetic is the one stated here.
 *   scale_mode  MOE_A2A_FP8_SCALE_F32: scale as above.  MOE_A2A_FP8_SCALE_POW2: that value rounded
 *               up to the next power of two (exponent field clamped to 1..254), still stored as
 *               f32 -- every consumer of the rows works unchanged, and moe_a2a_expert_gemm_mx8 can
 *               hand the exponents to the matrix instruction.
 *   disp_q[R,H] uint8, disp_scale[R,H/128] f32
 */
int moe_a2a_dispatch_fp8(const void* x, int x_type, const int32_t* slot_of_entry, uint8_t* disp_q,
                         float* disp_scale, int T, int K, int H, int scale_mode, moe_a2a_stream_t stream);

/*
 * Expert stub (all2all/reference.py:262): y[row,:] = round_out(f32(round_out(x[row,:])) * s(e)),
 * e = meta[row,0].  With disp_scale != NULL the input is fp8: y = round_out((f32(q)*scale) * s(e)).
 * rows == NULL: rows 0..R-1 (compact layout).  rows != NULL: the R rows rows[0..R-1] -- pass
 * slot_of_entry for the padded layout, so that only rows holding an entry are touched (the
 * reference multiplies the whole padded buffer, uninitialised rows included).
 */
int moe_a2a_stub(const void* disp, const float* disp_scale, const int32_t* meta, const int32_t* rows, int in_type,
                 int out_type, int stub_kind, int E, int W, void* y, int R, int H, moe_a2a_stream_t stream);

/*
 * Combine: out[t,:] = sum_k weights[t,k] * expert_y[slot_of_entry[t*K+k], :]
 * (all2all/reference.py:163-232 without the regroup/exchange).  STRICT reproduces the
 * reference's order (ascending slot) and its rounding to the output type after every add;
 * F32 keeps an f32 accumulator in k order.  Multiply and add are never contracted.
 * Rows of out that belong to no token are not touched.  (Cache policy of the output stores at
 * streaming sizes: this entry point does not know what the dispatch wrote and assumes one byte
 * per element of the expert rows; moe_a2a_forward decides from the actual figure.)
 */
int moe_a2a_combine(const void* expert_y, const float* weights, const int32_t* slot_of_entry, int mode,
                    int elem_type, void* out, int T, int K, int H, moe_a2a_stream_t stream);

/*
 * Combine with the expert stub folded in: reads the dispatched rows directly and applies
 * s(e) with the stub's rounding before the weighted sum -- identical results to
 * moe_a2a_stub followed by moe_a2a_combine, without the R*H round trip through memory.
 */
int moe_a2a_stub_combine(const void* disp, const float* disp_scale, const int32_t* indices,
                         const float* weights, const int32_t* slot_of_entry, int mode, int in_type, int out_type,
                         int stub_kind, int E, int W, void* out, int T, int K, int H, moe_a2a_stream_t stream);

/*
 * The whole path in one call: routing + dispatch, expert stub, combine -- what custom_kernel
 * does between reading its inputs and returning y (submission.py:192-219 of the reference;
 * ref_kernel, all2all/reference.py:256-272).  Same kernels and results as the separate calls;
 * one host call keeps the launches back to back.
 *   fp8_dispatch  0: 16-bit rows, 1: fp8 rows with f32 scales, 2: fp8 rows with power-of-two scales
 *   fuse_stub     0: stub kernel + combine, 1: moe_a2a_stub_combine.  With fuse_stub and fuse_route on a
 *                 small routing table (what moe_a2a_route_dispatch takes one token per workgroup for:
 *                 a few thousand entries), 16-bit rows of one element type and the compact layout,
 *                 the whole path is ONE launch: a workgroup dispatches its token and then folds the
 *                 rows it has just written -- the stand-in expert is elementwise, so a token's result
 *                 depends on no other workgroup's rows; same buffers, same bits, no launch in between.
 *   fuse_route    0: moe_a2a_route + dispatch, 1: moe_a2a_route_dispatch when moe_a2a_fused_ok,
 *                 2: moe_a2a_route_dispatch at any size
 *   expert_y      [R,H] (padded layout: [E*max_recv,H]) of out_type, unused (may be NULL) when fuse_stub
 *   max_recv      0 compact layout, > 0 padded layout (see moe_a2a_route)
 */
int moe_a2a_forward(const void* x, const int32_t* indices, const float* weights, const int32_t* rank_start,
                    int src_rank, int T, int K, int E, int W, int H, int max_recv, int in_type, int out_type,
                    int fp8_dispatch, int stub_kind, int combine_mode, int fuse_route, int fuse_stub,
                    int32_t* counts, int32_t* offsets, int32_t* slot_of_entry, int32_t* src_of_slot, int32_t* meta,
                    int32_t* status, void* disp, float* disp_scale, void* expert_y, void* out, void* workspace,
                    size_t workspace_bytes, moe_a2a_stream_t stream);

/*
 * moe_a2a_forward with its arguments in a struct (same order, same meaning, plus clear_status): a
 * caller that repeats the call fills the struct once and patches the pointers that change, which
 * costs a foreign-function binding one argument instead of thirty-one.
 */
typedef struct moe_a2a_forward_args {
  const void* x;
  const int32_t* indices;
  const float* weights;
  const int32_t* rank_start;
  int src_rank, T, K, E, W, H, max_recv, in_type, out_type, fp8_dispatch, stub_kind, combine_mode, fuse_route,
      fuse_stub;
  int32_t *counts, *offsets, *slot_of_entry, *src_of_slot, *meta, *status;
  void* disp;
  float* disp_scale;
  void* expert_y;
  void* out;
  void* workspace;
  size_t workspace_bytes;
  moe_a2a_stream_t stream;
  /* NULL, or one int32 that the first kernel of the call sets to 0.  A caller that alternates
   * between two sets of buffers names the status word of the OTHER set here: the next call, which
   * runs on that set behind this one on the stream, then starts from a cleared word and its status
   * describes that call alone, with no launch spent on clearing.  Must not be this call's `status`. */
  int32_t* clear_status;
} moe_a2a_forward_args;
int moe_a2a_forward_packed(const moe_a2a_forward_args* args);

/* Kernel launches moe_a2a_forward issues for this shape and these switches (host logic only). */
int moe_a2a_forward_launches(int T, int K, int H, int max_recv, int in_type, int out_type, int fp8_dispatch,
                             int fuse_route, int fuse_stub);

/*
 * Expert compute on the dispatched layout: y[rows of e, :] = x[rows of e, :] * W_e^T for every
 * expert e, rows of e = [offsets[e], offsets[e+1]) (compact) or [e*max_recv, e*max_recv + count)
 * (padded).  The reference stands a scalar multiply in for this step (all2all/reference.py:262);
 * this is the grouped matrix product a real MoE layer runs there.
 *   x[rows, Kd], weights[E, N, Kd], y[rows, N]: 16-bit elements of elem_type, f32 accumulation,
 *   Kd % 64 == 0, N % 8 == 0, 16-byte aligned.
 * Three kernels with identical results: 256 x 256 tiles (R > 32 * E and N >= 256; for segments of
 * less than 192 rows on average in a form that requests the weight rows early,
 * MOE_A2A_OPT_GEMM_STAGED = 3 / 4 forces it on / off); 32 x 128 tiles that stream the weights when
 * segments are short (R <= 32 * E and Kd % 128 == 0); 128 x 128 output tiles for what is left.  The option MOE_A2A_OPT_GEMM_TILE = 32, 128 or 256 forces one.
 * Padded layout: a segment longer than max_recv (routing raised MOE_A2A_STATUS_OVERFLOW) is
 * multiplied over its first max_recv rows only, so no tile leaves the segment or the buffers.
 */
int moe_a2a_expert_gemm(const void* x, const void* weights, const int32_t* offsets, void* y, int R, int E, int Kd,
                        int N, int max_recv, int elem_type, moe_a2a_stream_t stream);

/*
 * The same product on rows that moe_a2a_dispatch_fp8 wrote: x_q[rows, Kd] e4m3fn bytes with
 * x_scale[rows, Kd/128] f32.  A row element enters the product as elem(f32(q) * scale), i.e.
 * dequantised and rounded once to the 16-bit type of the weights, inside the kernel (the rows
 * are read as fp8: half the operand traffic, no dequantised copy in memory).  weights[E, N, Kd]
 * and y[rows, N] are 16-bit elements of elem_type; Kd % 128 == 0, N % 8 == 0.  Always the
 * 256 x 256 kernel.  No counterpart in the reference (it has no fp8 path).
 */
int moe_a2a_expert_gemm_fp8(const void* x_q, const float* x_scale, const void* weights, const int32_t* offsets,
                            void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                            moe_a2a_stream_t stream);

/*
 * The same product with quantised weights in the block format of DeepSeek-V3 checkpoints:
 * w_q[E, N, Kd] e4m3fn bytes with w_scale[E, N/128, Kd/128] f32 (one scale per 128 x 128 block).
 * x is 16-bit (x_scale == NULL) or the e4m3fn rows + x_scale[rows, Kd/128] of moe_a2a_dispatch_fp8
 * (dequantised and rounded once to elem_type inside the kernel); y[rows, N] of elem_type.
 * Kd % 128 == 0, N % 128 == 0.  Three kernels, chosen by the mean segment length and the rows:
 *   R <= 32 * E (a decode step, bound by the weight bytes, which cross memory once at one byte per
 *     element): 32 x 128 tiles, the operand slabs travel memory -> LDS directly (the weights with
 *     non-temporal loads: they are read once).  16-bit rows: the weight bytes enter the matrix
 *     cores exactly (turned into 16-bit values in registers), each 128-wide K block is summed in
 *     f32 and scaled in f32: y = sum over K blocks of scale_b * (x . q_b).  fp8 rows: the bytes of
 *     both operands go to the fp8 matrix instruction untouched, folded per K block as below.
 *     The option MOE_A2A_OPT_GEMM_STAGED = 1 selects the register-staged form of the same
 *     arithmetic (fp8 rows are then dequantised and rounded once to elem_type first).
 *   longer segments, fp8 rows: both operands enter the fp8 matrix instruction as bytes (eight
 *     waves on 256 x 128 tiles with the 16x16x128 instruction for Kd >= 256; the option
 *     MOE_A2A_OPT_GEMM_STAGED = 2, and Kd = 128, take four waves on 128 x 128 tiles with the
 *     32x32x64 one), each 128-wide K block is summed in f32 and folded with
 *     x_scale[row][kb] * w_scale[n / 128][kb]; nothing is rounded before the output.
 *   longer segments, 16-bit rows (and N >= 256): the 256 x 256 kernel; a weight enters the matrix
 *     cores as elem(f32(q) * scale), i.e. dequantised and rounded once to elem_type on its way into
 *     LDS -- the result of dequantising the weights to 16 bits and calling moe_a2a_expert_gemm,
 *     without the 16-bit copy in memory.
 * The three differ by those roundings (2^-9 relative per operand for bf16); the option
 * MOE_A2A_OPT_GEMM_TILE = 32, 128 (fp8 rows) or 256 forces one.  No counterpart in the reference.
 */
int moe_a2a_expert_gemm_q8(const void* x, const float* x_scale, const void* w_q, const float* w_scale,
                           const int32_t* offsets, void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                           moe_a2a_stream_t stream);

/*
 * The same product for operands whose scales are all powers of two (rows from moe_a2a_dispatch_fp8
 * with MOE_A2A_FP8_SCALE_POW2, weights quantised with power-of-two block scales, the UE8M0 style
 * of newer DeepSeek checkpoints): the bytes of both operands go to the scaled fp8 matrix
 * instruction (v_mfma_scale_f32_16x16x128_f8f6f4 on eight-wave 256 x 256 tiles for Kd from 256 to
 * 8192; v_mfma_scale_f32_32x32x64_f8f6f4 on four-wave tiles otherwise) and the exponent fields of
 * the scales ride along as the instruction's block exponents, so the products of all K blocks
 * accumulate inside the matrix cores (nothing is folded on the vector units; the operand slabs
 * travel memory -> LDS directly).  y = sum over K blocks of
 * x_scale * w_scale * (q_x . q_w) in f32, one rounding to elem_type.  ONLY the exponent field of a
 * scale is used: a scale that is not a power of two is silently taken as the power of two below
 * it.  Segments of at most 32 rows on average (a decode step), and other Kd on segments shorter
 * than 256 rows, go through moe_a2a_expert_gemm_q8 (any f32 scale).  The option
 * MOE_A2A_OPT_GEMM_TILE = 256 forces the tiles, 32 / 128 the kernels of moe_a2a_expert_gemm_q8,
 * MOE_A2A_OPT_GEMM_STAGED = 1 the register-staged four-wave loop of the tiles, 2 the four-wave loop
 * with slabs sent memory -> LDS (Kd % 256 == 0), 3 / 4 the eight-wave loop with / without the early
 * requests for the weight rows that segments of less than 192 rows on average get by themselves.
 * Arguments as for
 * moe_a2a_expert_gemm_q8 with x_scale required.  No counterpart in the reference.
 */
int moe_a2a_expert_gemm_mx8(const void* x_q, const float* x_scale, const void* w_q, const float* w_scale,
                            const int32_t* offsets, void* y, int R, int E, int Kd, int N, int max_recv, int elem_type,
                            moe_a2a_stream_t stream);

/*
 * Launch timer (opt-in, process-wide).  Between begin and end every kernel the library launches,
 * from any thread, carries a pair of HIP events bound to that dispatch, so the reported time is the
 * kernel's own begin-to-end duration on the GPU; while the timer is on, launches are serialised on
 * a mutex (a measurement aid: a product run leaves it off and pays one relaxed atomic read).
 *   begin(capacity)  allocate `capacity` event pairs and start recording
 *   end(ids, us, n)  wait for the recorded launches, write up to n (kernel id, microseconds)
 *                    pairs to HOST arrays, release the events; returns the number written
 *   skip(launches)   the next `launches` launches go out without events (they cost the host a
 *                    fifth of a timed launch: a caller issues untimed steps first so that the GPU
 *                    queue stays full while the timed ones are issued)
 *   kernel_name(id)  host string for a kernel id
 */
int moe_a2a_timer_begin(int capacity);
int moe_a2a_timer_skip(int launches);
int moe_a2a_timer_end(int* kernel_ids, float* microseconds, int n);
const char* moe_a2a_kernel_name(int kernel_id);

/*
 * Option switches (opt-in, process-wide; every option starts at 0 = the library decides).  They
 * force one of several kernels that give the same results, for tests that compare the kernels with
 * each other and for measurements; they are plain integers read at launch time, so a caller that
 * never sets one pays nothing and sees no hidden behaviour.
 *   set_option(option, value)  returns the previous value (>= 0), MOE_A2A_E_DTYPE for an unknown
 *                              option or MOE_A2A_E_SHAPE for a negative value (no option takes one,
 *                              so a negative return is always an error)
 *   get_option(option)         current value, or MOE_A2A_E_DTYPE
 * A value is read when an entry point runs: a workspace size queried under one setting, or a
 * hipGraph captured under it, belongs to that setting.
 */
#define MOE_A2A_OPT_ROUTE_TILE 0    /* 1: moe_a2a_route_dispatch takes the token-tile kernel at any size   */
#define MOE_A2A_OPT_GEMM_TILE 1     /* 32 | 128 | 256: tile family of the expert GEMM entry points          */
#define MOE_A2A_OPT_GEMM_STAGED 2   /* 1: register-staged form of the weight-streaming / scaled-MFMA loops;
                                       2: four-wave forms of moe_a2a_expert_gemm_mx8 / _q8 with fp8 rows;
                                       3 | 4: moe_a2a_expert_gemm_mx8's eight-wave loop with | without early
                                       requests for the weight rows                                        */
#define MOE_A2A_OPT_COMBINE_LANES 3 /* lanes of a combine workgroup at cache-resident sizes (64 .. 512)     */
#define MOE_A2A_OPT_COMBINE_VPL 4   /* 2: two row vectors per lane in the combine at cache-resident sizes   */
#define MOE_A2A_OPT_TIMER_EVENT_FLAGS 5 /* hipEventCreateWithFlags value for the launch timer's events    */
#define MOE_A2A_OPT_COMBINE_PLAIN_MAP 6 /* 1: combine workgroups in token order, not grouped by XCD          */
#define MOE_A2A_OPT_TWO_LAUNCHES 7      /* 1: moe_a2a_forward never takes its one-launch form                */
#define MOE_A2A_OPT_FP8_TILE 8          /* tokens per workgroup of the fused routing + fp8 dispatch (0: chosen) */
#define MOE_A2A_OPT_COUNT 9
int moe_a2a_set_option(int option, int value);
int moe_a2a_get_option(int option);

#ifdef __cplusplus
}
#endif
#endif /* MOE_A2A_H_ */
