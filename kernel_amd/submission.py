"""``custom_kernel(data)`` -- the entry point a caller of the reference imports from its
``submission`` module (eval.py:159-180; shape of the call: submission.py:192-219).

``data = (cfg, rank_data, rank, world_size)``; returns ``y[:num_tokens]`` with dtype
``cfg.out_dtype`` on the device of ``rank_data.x``.  The destination ranks are partitions
of one buffer on that GPU, so no process group is needed and every emulated rank may
call this from one process.  The expert stand-in is the reference's ``x * (1 + owner)``.
"""
from __future__ import annotations

import torch

from .all2all import HipAllToAll
from .contract import COMBINE_STRICT, STUB_OWNER_RANK

_instances = {}
_last = [None, None]  # key and instance of the previous call (a harness calls with one config many times)


def _instance(cfg, rank: int, world_size: int, device, stub_kind: int, combine_mode: int) -> HipAllToAll:
    """The host object for this configuration, made on first use and kept.

    Every field the kernels' geometry depends on is part of the key and is read from ``cfg`` at
    every call: a config changed in place between two calls finds (or makes) the instance of its
    new values, never one whose buffers were sized for the old ones.  The previous call's key is
    compared first (a tuple compare is cheaper than hashing the device and dtype objects)."""
    key = (cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim, cfg.max_num_tokens, cfg.in_dtype, cfg.out_dtype,
           rank, world_size, device, stub_kind, combine_mode)
    if _last[0] == key:
        return _last[1]
    ata = _instances.get(key)
    if ata is None:
        if len(_instances) > 64:
            _instances.clear()
        # the stub is a stand-in for expert compute: folding it into the combine gives the same
        # bits with one launch and one pass over the dispatched rows fewer
        ata = _instances[key] = HipAllToAll(cfg, rank, world_size, stub_kind=stub_kind, combine_mode=combine_mode,
                                            fuse_stub=True)
    _last[0], _last[1] = key, ata
    return ata


def custom_kernel(data, stub_kind: int = STUB_OWNER_RANK, combine_mode: int = COMBINE_STRICT,
                  check_status: bool = False) -> torch.Tensor:
    """``check_status=True`` reads the routing status back after the call (one synchronisation) and
    raises where the reference would: ``IndexError`` for an expert id outside ``[0, num_experts)``
    (``token_map[dst_rank]``, reference.py:81-86)."""
    cfg, rank_data, rank, world_size = data
    x = rank_data.x
    if not x.is_cuda:
        raise RuntimeError("custom_kernel needs its inputs on the GPU: there is no CPU implementation")
    ata = _instance(cfg, rank, world_size, x.device, stub_kind, combine_mode)
    T = x.shape[0]
    # the caller owns its result (eval.py deletes it after each run): the combine writes straight
    # into a fresh tensor instead of one of the reused buffers
    y = torch.empty((T, cfg.hidden_dim), dtype=cfg.out_dtype, device=x.device)
    idx, w = rank_data.indices, rank_data.weights
    if not (x.is_contiguous() and idx.is_contiguous() and w.is_contiguous()):
        x, idx, w = x.contiguous(), idx.contiguous(), w.contiguous()
    if x.device.index == torch.cuda.current_device():  # the usual case: no device switch to pay for
        ata.forward(x, idx, w, out=y, check_status=check_status)
    else:
        with torch.cuda.device(x.device):
            ata.forward(x, idx, w, out=y, check_status=check_status)
    n = rank_data.num_tokens
    return y if n == T else y[:n]
