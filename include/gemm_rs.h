/* C ABI of the GEMM + reduce-scatter on one MI355X: the one-GPU share of the reference's second
 * problem, gemm_rs/ (a K-split tensor-parallel linear layer followed by reduce_scatter_tensor).
 * Same library as moe_a2a.h (libmoe_a2a.so), same conventions: device pointers in caller-owned
 * memory, kernels are only enqueued on the stream given, 0 = success, < 0 = MOE_A2A_E_* found on
 * the host before anything is launched, > 0 = the hipError_t of a launch.
 */
#ifndef GEMM_RS_H
#define GEMM_RS_H

#include <stddef.h>

#include "moe_a2a.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces ref_kernel of gemm_rs/reference.py:36-60 (and custom_kernel of gemm_rs/submission.py:5-29)
 * for a world of W ranks whose shards are partitions of one buffer on this GPU:
 *
 *   out[M, N] = sum over ranks s of  input_s[M, K/W] x weight_s[N, K/W]^T   (+ W * bias[N])
 *
 * Rank s of the reference multiplies its K-shard (reference.py:53), adds the bias (:54-55; so the
 * bias enters the sum once per rank), and reduce_scatter_tensor (:58-59) sums the W products and
 * hands rows [r M/W, (r+1) M/W) to rank r: that row block of `out` is rank r's return value.
 * Accumulation is f32 over the whole of K with one rounding to elem_type; the reference rounds each
 * rank's product and each reduction step to bf16 and checks with rtol = atol = 1e-2 (:66).
 *
 *   input   shard s at input + s * input_shard_stride elements, [M, K/W] row-major
 *   weight  shard s at weight + s * weight_shard_stride elements, [N, K/W] row-major
 *           a stride of 0 means packed shards (M*K/W, N*K/W); strides are multiples of 8 elements
 *   bias    [N] of elem_type, or NULL
 *   out     [M, N] of elem_type
 *   K % W == 0, (K/W) % 8 == 0, 16-byte aligned operands; M need not divide by W for the sum itself
 *   workspace  gemm_rs_workspace_bytes(M, N, K, W) bytes, 16-byte aligned; what it is for depends on the
 *           kernel form the shape gets:
 *             - outputs of few tiles spread the shards over groups of workgroups, one f32 partial
 *               product per group (what each rank holds before the reduce-scatter), which a second
 *               launch sums: REQUIRED, MOE_A2A_E_WORKSPACE if missing or too small;
 *             - large outputs whose local K is not a multiple of 64 (rows that start off the
 *               128-byte line grid) are first copied onto zero-padded, aligned rows: OPTIONAL --
 *               with NULL or too few bytes the product runs on the rows as they lie, about a
 *               tenth slower;
 *             - 0 bytes for every other shape.
 *           The form, and with it the size, follows MOE_A2A_OPT_GEMM_TILE at the time of the call: a
 *           size queried under one setting belongs to that setting.
 * MOE_A2A_OPT_GEMM_TILE forces a form where the shape allows it: 256 the 256 x 256 tiles, 129 the
 * 256 x 128 tiles (131 / 132: with 192 / 128 of a tile's rows in use, as the library chooses by itself
 * when that fills the CUs better), 130 those with one partial product per shard, 128 the 128 x 128
 * tiles, 32 those with one partial product per shard.  All unsplit forms give identical bits.
 */
size_t gemm_rs_workspace_bytes(int M, int N, int K, int W);
int gemm_rs_forward(const void* input, const void* weight, const void* bias, void* out, int M, int N, int K, int W,
                    long long input_shard_stride, long long weight_shard_stride, int elem_type, void* workspace,
                    size_t workspace_bytes, moe_a2a_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
