"""TEST INFRASTRUCTURE -- literal CPU restatement of the reference's MoE all-to-all.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg may
import this package; product code never does.

This file follows all2all/reference.py step by step for an *emulated world held in
one process*: every rank runs the reference's loops in turn, and an
``all_to_all_single`` becomes a transpose of per-(src,dst) lists (the chunk rank
``d`` receives from rank ``s`` is the chunk rank ``s`` addressed to rank ``d``,
received chunks concatenated in ascending ``s``).  Row loops and torch's own
arithmetic are kept, so the rounding is whatever torch does for the same
expressions.  It is slow by construction; use it on small cases.

Pinned by (tests/test_oracle_pins.py, tests/test_golden.py):
  * golden vectors written by the reference's own ``PyTorchAllToAll`` over gloo
    (tests/golden/), for dispatch, combine and the end-to-end output;
  * brute-force O(R^2) slot ranks, ``bincount``/stable ``sort`` library routines;
  * algebraic special cases of the combine (one-hot weights, K=1, zero weights).
"""
from __future__ import annotations

from typing import List, Sequence

import torch

META_DIM = 5  # reference.py:56


class EmulatedRank:
    """One rank's ``PyTorchAllToAll`` state (reference.py:58-65)."""

    def __init__(self, cfg, rank: int, world_size: int):
        self.cfg = cfg
        self.rank = rank
        self.world_size = world_size
        self.num_local_experts = cfg.num_experts // world_size
        self.max_recv = cfg.max_num_tokens * world_size


def _all_to_all(send: List[List[torch.Tensor]]) -> List[List[torch.Tensor]]:
    """send[s][d] -> recv[d][s]; what all_to_all_single does with split sizes."""
    W = len(send)
    return [[send[s][d] for s in range(W)] for d in range(W)]


def dispatch_world(cfg, world: Sequence, padded: bool = False):
    """reference.py:68-148 for every rank of the world.

    Returns per owner rank ``d``: ``expert_num_tokens[E_l] int32``, ``expert_x`` and
    ``expert_meta``.  With ``padded=False`` the latter two are lists (one entry per
    local expert) of ``[count, H]`` / ``[count, 5]`` tensors -- the initialised part
    of the reference's ``[E_l, max_recv, .]`` buffers; ``padded=True`` builds the
    full reference-shaped buffers (zero-filled where the reference leaves
    ``torch.empty`` garbage).
    """
    W = len(world)
    ranks = [EmulatedRank(cfg, r, W) for r in range(W)]
    E_l = ranks[0].num_local_experts
    H = cfg.hidden_dim

    send_x, send_meta, send_counts = [], [], []
    for r, rd in enumerate(world):
        # reference.py:72-86
        counts = [0] * W
        token_map = [[] for _ in range(W)]
        meta_map = [[] for _ in range(W)]
        for t, expert_list in enumerate(rd.indices.tolist()):
            for k, e in enumerate(expert_list):
                dst = e // E_l
                counts[dst] += 1
                token_map[dst].append(t)
                meta_map[dst].extend([e, r, t, k, 0])
        send_counts.append(counts)
        # reference.py:93  (kept per destination instead of concatenated)
        send_x.append([rd.x[torch.tensor(tm, dtype=torch.long)] if tm else rd.x[:0] for tm in token_map])
        send_meta.append([torch.tensor(mm, dtype=torch.int32).view(-1, META_DIM) for mm in meta_map])

    recv_x = _all_to_all(send_x)  # reference.py:107-112
    recv_meta = _all_to_all(send_meta)  # reference.py:114-120

    out = []
    for d in range(W):
        buf = torch.cat(recv_x[d], dim=0) if recv_x[d] else torch.empty(0, H, dtype=cfg.in_dtype)
        meta = torch.cat(recv_meta[d], dim=0)
        total_recv = sum(send_counts[s][d] for s in range(W))  # reference.py:88-94
        assert buf.shape[0] == total_recv == meta.shape[0]
        # reference.py:123-146: arrival-order slotting per local expert
        num = torch.zeros(E_l, dtype=torch.int32)
        rows_x = [[] for _ in range(E_l)]
        rows_m = [[] for _ in range(E_l)]
        for i in range(total_recv):
            local_eid = int(meta[i, 0].item()) % E_l
            rows_x[local_eid].append(buf[i])
            rows_m[local_eid].append(meta[i])
            num[local_eid] += 1
        ex = [torch.stack(r) if r else torch.empty(0, H, dtype=cfg.in_dtype) for r in rows_x]
        em = [torch.stack(r) if r else torch.empty(0, META_DIM, dtype=torch.int32) for r in rows_m]
        if padded:
            max_recv = ranks[d].max_recv
            px = torch.zeros(E_l, max_recv, H, dtype=cfg.in_dtype)
            pm = torch.zeros(E_l, max_recv, META_DIM, dtype=torch.int32)
            for le in range(E_l):
                px[le, : ex[le].shape[0]] = ex[le]
                pm[le, : em[le].shape[0]] = em[le]
            ex, em = px, pm
        out.append((num, ex, em))
    return out


def stub_world(cfg, dispatched, stub_kind: int):
    """reference.py:262 on the initialised rows.

    kind 0: ``expert_x.to(out_dtype) * (1 + owner_rank)``;
    kind 1: ``expert_x.to(out_dtype) * ((1 + e) / num_experts)`` with the global
    expert id ``e`` (python float scalar, as the rank factor is a python int).
    """
    W = len(dispatched)
    E_l = cfg.num_experts // W
    out = []
    for d, (num, ex, em) in enumerate(dispatched):
        ys = []
        for le in range(E_l):
            xe = ex[le][: int(num[le])]
            if stub_kind == 0:
                ys.append(xe.to(cfg.out_dtype) * (1 + d))
            else:
                e = d * E_l + le
                ys.append(xe.to(cfg.out_dtype) * ((1 + e) / cfg.num_experts))
        out.append(ys)
    return out


def combine_world(cfg, world: Sequence, dispatched, expert_y):
    """reference.py:151-234 for every rank; returns ``y[max_num_tokens, H]`` per rank."""
    W = len(world)
    E_l = cfg.num_experts // W
    H = cfg.hidden_dim
    send_y, send_meta = [], []
    for d in range(W):
        num, _, em = dispatched[d]
        y_map = [[] for _ in range(W)]
        meta_map = [[] for _ in range(W)]
        for local_eid in range(E_l):  # reference.py:170-179
            cnt = int(num[local_eid].item())
            for j in range(cnt):
                meta = em[local_eid][j]
                dst_rank = int(meta[1].item())
                y_map[dst_rank].append(expert_y[d][local_eid][j].unsqueeze(0))
                meta_map[dst_rank].extend(meta.tolist())
        send_y.append([torch.cat(s, dim=0) if s else torch.empty(0, H, dtype=cfg.out_dtype) for s in y_map])
        send_meta.append([torch.tensor(mm, dtype=torch.int32).view(-1, META_DIM) for mm in meta_map])
    recv_y = _all_to_all(send_y)  # reference.py:210-215
    recv_meta = _all_to_all(send_meta)  # reference.py:217-224

    outs = []
    for s, rd in enumerate(world):
        out_tokens = torch.zeros(max(cfg.max_num_tokens, rd.num_tokens), H, dtype=cfg.out_dtype)  # reference.py:263-268
        buf = torch.cat(recv_y[s], dim=0)
        meta = torch.cat(recv_meta[s], dim=0)
        for i in range(buf.shape[0]):  # reference.py:227-232
            src_token = int(meta[i, 2].item())
            src_k = int(meta[i, 3].item())
            w = rd.weights[src_token, src_k].to(torch.float32)
            out_tokens[src_token] += buf[i].to(torch.float32) * w
        outs.append(out_tokens)
    return outs


def ref_kernel_world(cfg, world: Sequence, stub_kind: int = 0):
    """reference.py:256-272 for every rank: list of ``y[:num_tokens]``."""
    disp = dispatch_world(cfg, world)
    ey = stub_world(cfg, disp, stub_kind)
    ys = combine_world(cfg, world, disp, ey)
    return [y[: rd.num_tokens] for y, rd in zip(ys, world)]


def compact_from_dispatched(cfg, dispatched):
    """Flatten per-rank / per-expert lists into the expert-major compact layout.

    Returns ``counts[E]``, ``offsets[E+1]``, ``disp_x[R,H]``, ``meta[R,5]`` where the
    reference slot ``(owner d, local expert le, position j)`` is row
    ``offsets[d*E_l + le] + j``.
    """
    W = len(dispatched)
    E_l = cfg.num_experts // W
    counts = torch.cat([num for num, _, _ in dispatched]).to(torch.int32)
    offsets = torch.zeros(cfg.num_experts + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts.to(torch.int64), 0).to(torch.int32)
    xs, ms = [], []
    for d, (num, ex, em) in enumerate(dispatched):
        for le in range(E_l):
            xs.append(ex[le][: int(num[le])])
            ms.append(em[le][: int(num[le])])
    return counts, offsets, torch.cat(xs, 0), torch.cat(ms, 0)
