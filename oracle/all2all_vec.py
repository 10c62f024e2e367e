"""TEST INFRASTRUCTURE -- vectorised CPU restatement of the reference's MoE all-to-all.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg may
import this package; product code never does.

Same results as ``all2all_literal`` (proved bit-for-bit in tests/test_oracle_pins.py)
but built from library routines so it finishes in seconds at the large workloads:

  route      stable sort of the expert ids over the canonical entry order
             (src_rank, token, k)  -- reproduces reference.py:79-86 (entry order),
             :107-112 (chunks arrive in ascending source rank) and :140-146
             (arrival-order slotting per local expert);
  dispatch   ``index_select`` of token rows                       (reference.py:93,144);
  stub       ``(x.float() * s).to(out_dtype)``                    (reference.py:262);
  combine    per token, the K expert rows are folded in ascending slot order with
             ``acc = (acc.float() + y.float() * w).to(out_dtype)`` after every add
             (reference.py:227-232 into the ``out_dtype`` buffer of :263-268; rows
             return in (owner rank, local expert, position) order, :170-179).

fp8 dispatch has no counterpart in the reference; its arithmetic is defined here:
per (row, 128-column block) ``amax = max|f32(x)|``, ``scale = amax / 448`` in f32
(``scale = 1`` when ``amax == 0``), ``q = (f32(x) / scale).to(float8_e4m3fn)``.
PARITY UNPINNED against the reference for that function (nothing to pin against);
it is pinned against torch's own e4m3fn cast and the stated error bound only.

``expert_gemm`` / ``expert_gemm_fp8`` / ``expert_gemm_q8`` (a per-expert linear layer in place of the stub) have no
counterpart in the reference either: PARITY UNPINNED against it; they are an f32 torch matmul per
segment and serve as the tolerance reference for the HIP grouped GEMM.
"""
from __future__ import annotations

from typing import Sequence

import torch

META_DIM = 5
FP8_BLOCK = 128
FP8_MAX = 448.0


def concat_world(world: Sequence):
    """Concatenate per-rank tensors in rank order; returns x, indices, weights, starts."""
    x = torch.cat([rd.x for rd in world], 0)
    idx = torch.cat([rd.indices for rd in world], 0)
    w = torch.cat([rd.weights for rd in world], 0)
    starts = [0]
    for rd in world:
        starts.append(starts[-1] + int(rd.num_tokens))
    return x, idx, w, starts


def route(indices: torch.Tensor, starts: Sequence[int], num_experts: int):
    """Counts, offsets and the two permutations for the compact expert-major layout.

    ``indices[T,K]`` is the whole world's routing table in rank order; entry
    ``i = t*K + k`` (global token ``t``).  Slot of entry ``i`` =
    ``offsets[e_i] + #{j < i : e_j == e_i}``.
    """
    T, K = indices.shape
    R = T * K
    flat = indices.reshape(-1).to(torch.int64)
    counts = torch.bincount(flat, minlength=num_experts).to(torch.int32)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts.to(torch.int64), 0).to(torch.int32)
    _, src_of_slot = torch.sort(flat, stable=True)
    slot_of_entry = torch.empty(R, dtype=torch.int64)
    slot_of_entry[src_of_slot] = torch.arange(R, dtype=torch.int64)
    # meta rows [e, src_rank, local token, k, 0] at their slots (reference.py:85)
    tok = src_of_slot // K
    bounds = torch.tensor(list(starts[1:]), dtype=torch.int64)
    src_rank = torch.bucketize(tok, bounds, right=True)
    start_t = torch.tensor(list(starts), dtype=torch.int64)
    meta = torch.stack(
        [flat[src_of_slot], src_rank, tok - start_t[src_rank], src_of_slot % K, torch.zeros_like(tok)], dim=1
    ).to(torch.int32)
    return dict(
        counts=counts,
        offsets=offsets,
        slot_of_entry=slot_of_entry.to(torch.int32),
        src_of_slot=src_of_slot.to(torch.int32),
        meta=meta,
    )


def dispatch(x: torch.Tensor, src_of_slot: torch.Tensor, K: int) -> torch.Tensor:
    """``disp_x[slot] = x[token(src_of_slot[slot])]`` -- a pure row copy."""
    return x.index_select(0, (src_of_slot.to(torch.int64) // K))


def pow2_at_or_above(scale: torch.Tensor) -> torch.Tensor:
    """The next power of two at or above a positive f32 (exponent field clamped to 1..254): the
    power-of-two scale mode.  Done on the bits: exponent field + 1 when the mantissa is not zero."""
    u = scale.contiguous().view(torch.int32)
    e = (u >> 23) + ((u & 0x7FFFFF) != 0).to(torch.int32)
    return (e.clamp(1, 254) << 23).view(torch.float32)


def quantize_fp8(x: torch.Tensor, pow2: bool = False):
    """Per-row, per-128-column e4m3fn quantisation; returns (q as uint8 bits, scale f32).
    ``pow2``: the scale is ``amax / 448`` rounded up to a power of two."""
    T, H = x.shape
    assert H % FP8_BLOCK == 0
    xf = x.to(torch.float32).view(T, H // FP8_BLOCK, FP8_BLOCK)
    amax = xf.abs().amax(dim=-1)
    scale = amax / FP8_MAX
    scale = torch.where(amax == 0, torch.ones_like(scale), scale)
    if pow2:
        scale = pow2_at_or_above(scale)
    q = (xf / scale.unsqueeze(-1)).to(torch.float8_e4m3fn)
    return q.view(T, H).view(torch.uint8), scale


def dispatch_fp8(x: torch.Tensor, src_of_slot: torch.Tensor, K: int, pow2: bool = False):
    """Quantise each token row once, then copy rows and scales to their slots."""
    q, scale = quantize_fp8(x, pow2)
    tok = src_of_slot.to(torch.int64) // K
    return q.index_select(0, tok), scale.index_select(0, tok)


def dequantize_fp8(q_bits: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    R, H = q_bits.shape
    qf = q_bits.view(torch.float8_e4m3fn).to(torch.float32).view(R, H // FP8_BLOCK, FP8_BLOCK)
    return (qf * scale.unsqueeze(-1)).view(R, H)


def stub_scales(meta: torch.Tensor, stub_kind: int, num_experts: int, world_size: int) -> torch.Tensor:
    """f32 factor per dispatched row: ``1 + owner_rank`` or ``f32((1+e)/E)``."""
    e = meta[:, 0].to(torch.int64)
    if stub_kind == 0:
        return (1 + e // (num_experts // world_size)).to(torch.float32)
    return ((1 + e).to(torch.float64) / float(num_experts)).to(torch.float32)


def stub(disp_x: torch.Tensor, meta: torch.Tensor, stub_kind: int, num_experts: int, world_size: int,
         out_dtype: torch.dtype, scale: torch.Tensor = None) -> torch.Tensor:
    """Expert stand-in (reference.py:262).

    bf16/fp16 rows: ``round_out(f32(round_out(x)) * s)``.  fp8 rows (``scale`` given):
    ``round_out((f32(q) * scale) * s)`` -- dequantise in f32, then the same factor.
    """
    s = stub_scales(meta, stub_kind, num_experts, world_size).unsqueeze(-1)
    if scale is not None:
        return (dequantize_fp8(disp_x, scale) * s).to(out_dtype)
    return (disp_x.to(out_dtype).to(torch.float32) * s).to(out_dtype)


def expert_gemm(disp_x: torch.Tensor, offsets: torch.Tensor, weights: torch.Tensor,
                out_dtype: torch.dtype) -> torch.Tensor:
    """Per-expert linear layer on the compact rows: ``y[seg e] = x[seg e] @ W_e^T`` computed in f32
    and rounded once.  Has no counterpart in the reference (its expert is the scalar stub); the
    HIP kernel is compared with this within a tolerance, because the summation order differs."""
    R = disp_x.shape[0]
    E, N, _ = weights.shape
    y = torch.zeros(R, N, dtype=out_dtype)
    off = offsets.tolist()
    for e in range(E):
        if off[e + 1] > off[e]:
            y[off[e]:off[e + 1]] = (disp_x[off[e]:off[e + 1]].float() @ weights[e].float().t()).to(out_dtype)
    return y


def expert_gemm_fp8(q_bits: torch.Tensor, scale: torch.Tensor, offsets: torch.Tensor, weights: torch.Tensor,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """The same layer on fp8 dispatched rows: each element is dequantised, ``f32(q) * scale``, and
    rounded once to the weights' 16-bit type before it enters the product (what the HIP kernel
    stages into LDS).  No counterpart in the reference."""
    return expert_gemm(dequantize_fp8(q_bits, scale).to(weights.dtype), offsets, weights, out_dtype)


def quantize_weights_fp8(weights: torch.Tensor, pow2: bool = False):
    """Expert weights ``[E, N, Kd]`` -> e4m3fn bits and one f32 scale per 128 x 128 block
    (``scale = amax / 448``, 1 for an all-zero block; ``pow2``: rounded up to a power of two): the
    block format of DeepSeek-V3 checkpoints.  Test-side helper: the library only consumes weights
    in this format."""
    E, N, Kd = weights.shape
    assert N % FP8_BLOCK == 0 and Kd % FP8_BLOCK == 0
    wf = weights.to(torch.float32).view(E, N // FP8_BLOCK, FP8_BLOCK, Kd // FP8_BLOCK, FP8_BLOCK)
    amax = wf.abs().amax(dim=(2, 4))
    scale = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    if pow2:
        scale = pow2_at_or_above(scale)
    q = (wf / scale[:, :, None, :, None]).to(torch.float8_e4m3fn)
    return q.view(E, N, Kd).view(torch.uint8), scale


def dequantize_weights_fp8(q_bits: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    E, N, Kd = q_bits.shape
    qf = q_bits.view(torch.float8_e4m3fn).to(torch.float32).view(E, N // FP8_BLOCK, FP8_BLOCK, Kd // FP8_BLOCK, FP8_BLOCK)
    return (qf * scale[:, :, None, :, None]).view(E, N, Kd)


def expert_gemm_q8(disp_x: torch.Tensor, x_scale, w_bits: torch.Tensor, w_scale: torch.Tensor,
                   offsets: torch.Tensor, out_dtype: torch.dtype, round_rows: bool = True) -> torch.Tensor:
    """The expert layer with block-quantised weights: ``y = sum over K blocks of scale_b * (x . q_b)``,
    i.e. the weights enter exactly (``f32(q) * scale`` in f32) and everything is summed in f32, one
    rounding to ``out_dtype`` at the end.  fp8 rows (``x_scale`` given) are dequantised and, with
    ``round_rows``, rounded once to ``out_dtype`` first, as in ``expert_gemm_fp8`` (the kernels that
    multiply on the 16-bit matrix instruction do that); without it they enter as ``f32(q) * scale``
    (the kernel that multiplies fp8 by fp8 rounds nothing before the output).  No counterpart in the
    reference: PARITY UNPINNED against it."""
    w = dequantize_weights_fp8(w_bits, w_scale)  # f32
    if x_scale is None:
        x = disp_x
    else:
        x = dequantize_fp8(disp_x, x_scale)
        x = x.to(out_dtype) if round_rows else x
    R = x.shape[0]
    E, N, _ = w.shape
    y = torch.zeros(R, N, dtype=out_dtype)
    off = offsets.tolist()
    for e in range(E):
        if off[e + 1] > off[e]:
            y[off[e]:off[e + 1]] = (x[off[e]:off[e + 1]].float() @ w[e].t()).to(out_dtype)
    return y


def combine_strict(expert_y: torch.Tensor, weights: torch.Tensor, slot_of_entry: torch.Tensor,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Reference-order weighted sum with a rounding to ``out_dtype`` after every add."""
    T, K = weights.shape
    H = expert_y.shape[1]
    slots = slot_of_entry.view(T, K).to(torch.int64)
    order = torch.argsort(slots, dim=1, stable=True)  # ascending slot == reference arrival order
    s_sorted = torch.gather(slots, 1, order)
    w_sorted = torch.gather(weights.to(torch.float32), 1, order)
    acc = torch.zeros(T, H, dtype=out_dtype)
    for j in range(K):
        term = expert_y.index_select(0, s_sorted[:, j]).to(torch.float32) * w_sorted[:, j:j + 1]
        acc = (acc.to(torch.float32) + term).to(out_dtype)
    return acc


def combine_f32(expert_y: torch.Tensor, weights: torch.Tensor, slot_of_entry: torch.Tensor,
                out_dtype: torch.dtype) -> torch.Tensor:
    """f32 accumulation in k order (separate multiply and add), one final rounding."""
    T, K = weights.shape
    H = expert_y.shape[1]
    slots = slot_of_entry.view(T, K).to(torch.int64)
    acc = torch.zeros(T, H, dtype=torch.float32)
    for k in range(K):
        acc = acc + expert_y.index_select(0, slots[:, k]).to(torch.float32) * weights[:, k:k + 1].to(torch.float32)
    return acc.to(out_dtype)


def run_world(cfg, world: Sequence, stub_kind: int = 0, fp8: bool = False, combine_mode: int = 0,
              pow2: bool = False):
    """Whole path for an emulated world; returns every intermediate plus ``y[T,H]``."""
    x, idx, w, starts = concat_world(world)
    W = len(world)
    K = cfg.experts_per_token
    r = route(idx, starts, cfg.num_experts)
    out = dict(r)
    if fp8:
        q, sc = dispatch_fp8(x, r["src_of_slot"], K, pow2)
        out.update(disp_x=q, disp_scale=sc)
        ey = stub(q, r["meta"], stub_kind, cfg.num_experts, W, cfg.out_dtype, scale=sc)
    else:
        dx = dispatch(x, r["src_of_slot"], K)
        out.update(disp_x=dx)
        ey = stub(dx, r["meta"], stub_kind, cfg.num_experts, W, cfg.out_dtype)
    out["expert_y"] = ey
    comb = combine_strict if combine_mode == 0 else combine_f32
    out["y"] = comb(ey, w, r["slot_of_entry"], cfg.out_dtype)
    out["starts"] = starts
    return out


def closed_form(cfg, rank_data, stub_kind: int, world_size: int) -> torch.Tensor:
    """Dispatch-free statement of one rank's output (the stub is elementwise, so a
    rank's result depends on its own tokens only): fold the K terms of each token in
    ascending (expert id, k) order with per-step rounding."""
    x, idx, w = rank_data.x, rank_data.indices.to(torch.int64), rank_data.weights.to(torch.float32)
    T, K = idx.shape
    key = idx * K + torch.arange(K).unsqueeze(0)
    order = torch.argsort(key, dim=1)
    e_sorted = torch.gather(idx, 1, order)
    w_sorted = torch.gather(w, 1, order)
    acc = torch.zeros(T, cfg.hidden_dim, dtype=cfg.out_dtype)
    xo = x.to(cfg.out_dtype).to(torch.float32)
    for j in range(K):
        e = e_sorted[:, j]
        if stub_kind == 0:
            s = (1 + e // (cfg.num_experts // world_size)).to(torch.float32)
        else:
            s = ((1 + e).to(torch.float64) / float(cfg.num_experts)).to(torch.float32)
        y = (xo * s.unsqueeze(-1)).to(cfg.out_dtype)
        acc = (acc.to(torch.float32) + y.to(torch.float32) * w_sorted[:, j:j + 1]).to(cfg.out_dtype)
    return acc
