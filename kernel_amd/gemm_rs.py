"""GEMM + reduce-scatter of the reference's ``gemm_rs`` problem on one MI355X.

Mirrors gemm_rs/reference.py: ``generate_input`` (:5-33), ``ref_kernel`` / ``custom_kernel``
(:36-60, submission.py:5-29).  The reference runs one process per GPU and sums the ranks' products
with ``reduce_scatter_tensor``; here the W ranks are partitions of one buffer on one GPU, so the
reduction is the sum over the K shards inside one call of the library (``gemm_rs_forward``,
include/gemm_rs.h) and rank r's result is row block r of the one output.  Everything that computes
is in ``libmoe_a2a.so``; torch supplies device memory and the current stream.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib

# the reference's test and benchmark specs (gemm_rs/task.yml:59-79)
TEST_SPECS = [
    dict(world_size=8, m=64, n=2880, k=2880, has_bias=True, seed=2035),
    dict(world_size=8, m=64, n=3584, k=14336, has_bias=True, seed=13),
    dict(world_size=8, m=512, n=3584, k=14336, has_bias=True, seed=4297),
    dict(world_size=8, m=512, n=4608, k=36864, has_bias=False, seed=1597),
    dict(world_size=8, m=2048, n=4096, k=7168, has_bias=False, seed=716),
    dict(world_size=8, m=2048, n=8192, k=30720, has_bias=False, seed=20201),
    dict(world_size=8, m=4096, n=2880, k=2880, has_bias=True, seed=136),
    dict(world_size=8, m=4096, n=8192, k=2048, has_bias=True, seed=138),
    dict(world_size=8, m=8192, n=3584, k=14336, has_bias=True, seed=748),
    dict(world_size=8, m=8192, n=4608, k=36864, has_bias=True, seed=4422),
    dict(world_size=8, m=8192, n=8192, k=28672, has_bias=False, seed=1536),
]
BENCHMARK_SPECS = [
    dict(world_size=8, m=64, n=7168, k=18432, has_bias=False, seed=1234),
    dict(world_size=8, m=512, n=4096, k=12288, has_bias=True, seed=663),
    dict(world_size=8, m=2048, n=2880, k=2880, has_bias=True, seed=166),
    dict(world_size=8, m=4096, n=4096, k=4096, has_bias=False, seed=1371),
    dict(world_size=8, m=8192, n=4096, k=14336, has_bias=True, seed=7168),
    dict(world_size=8, m=8192, n=8192, k=29568, has_bias=False, seed=42),
]

Data = Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]


def generate_input(rank: int, world_size: int, m: int, n: int, k: int, has_bias: bool, seed: int,
                   device: Optional[torch.device] = None) -> Data:
    """One rank's ``(input[M, K/W], weight[N, K/W], bias[N] or None)`` in the reference's
    distribution (uniform in +-0.01, bf16; the same bias on every rank).  The reference draws on the
    device's own generator (reference.py:19-20); this draws on the CPU generator and moves the
    result, so that the CPU oracle sees the same values."""
    assert m % world_size == 0, "m must be divisible by world_size"
    assert k % world_size == 0, "k must be divisible by world_size"
    gen = torch.Generator().manual_seed(seed + rank)
    local_k = k // world_size
    x = ((torch.rand((m, local_k), generator=gen) * 2 - 1) * 0.01).to(torch.bfloat16)
    w = ((torch.rand((n, local_k), generator=gen) * 2 - 1) * 0.01).to(torch.bfloat16)
    bias = None
    if has_bias:
        gen.manual_seed(seed)
        bias = ((torch.rand((n,), generator=gen) * 2 - 1) * 0.01).to(torch.bfloat16)
    if device is not None:
        x, w = x.to(device), w.to(device)
        bias = bias.to(device) if bias is not None else None
    return x, w, bias


def pack_world(datas: Sequence[Data], device: torch.device):
    """The W ranks' shards as partitions of one buffer: ``input[W, M, K/W]``, ``weight[W, N, K/W]``."""
    x = torch.stack([d[0] for d in datas]).to(device).contiguous()
    w = torch.stack([d[1] for d in datas]).to(device).contiguous()
    bias = datas[0][2]
    return x, w, (bias.to(device).contiguous() if bias is not None else None)


class HipGemmReduceScatter:
    """``forward(input[W, M, Kl], weight[W, N, Kl], bias)`` -> ``out[M, N]``; ``out[r*M/W:(r+1)*M/W]``
    is what rank r of the reference returns."""

    def __init__(self, world_size: int, pad_ragged: bool = True):
        self.world_size = int(world_size)
        # False: a shape whose workspace is optional (ragged shards on 256 x 256 tiles, which run faster on
        # a zero-padded, line-aligned copy of the operands) is multiplied in place, without it
        self.pad_ragged = bool(pad_ragged)
        self.lib = _lib.load()
        self._workspace = None

    def workspace_for(self, m: int, n: int, k: int, device) -> Optional[torch.Tensor]:
        need = int(self.lib.gemm_rs_workspace_bytes(m, n, k, self.world_size))
        if need == 0:
            return None
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != device:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=device)
        return self._workspace

    def forward(self, x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if not x.is_cuda:
            raise RuntimeError("HipGemmReduceScatter needs tensors on the GPU (there is no CPU path)")
        W = self.world_size
        if x.dim() != 3 or w.dim() != 3 or x.shape[0] != W or w.shape[0] != W or x.shape[2] != w.shape[2]:
            raise ValueError(f"expected input[{W}, M, K/W] and weight[{W}, N, K/W], got {tuple(x.shape)}, {tuple(w.shape)}")
        if x.dtype not in (torch.bfloat16, torch.float16) or w.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
            raise ValueError("input, weight and bias must share one 16-bit float type")
        if not (x.is_contiguous() and w.is_contiguous() and (bias is None or bias.is_contiguous())):
            raise ValueError("operands must be contiguous")
        M, Kl, N = x.shape[1], x.shape[2], w.shape[1]
        if bias is not None and bias.shape != (N,):
            raise ValueError(f"bias must be [{N}]")
        if out is None:
            out = torch.empty((M, N), dtype=x.dtype, device=x.device)
        def call(ws):
            return self.lib.gemm_rs_forward(
                x.data_ptr(), w.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, Kl * W,
                W, 0, 0, _lib.BF16 if x.dtype == torch.bfloat16 else _lib.F16, ws.data_ptr() if ws is not None else None,
                ws.numel() if ws is not None else 0, torch.cuda.current_stream(x.device).cuda_stream)

        rc = call(None) if not self.pad_ragged else -4
        if rc == -4:  # MOE_A2A_E_WORKSPACE: this shape's form needs its workspace (nothing was launched)
            rc = call(self.workspace_for(M, N, Kl * W, x.device))
        _lib.check(rc, "gemm_rs_forward")
        return out


def custom_kernel_world(datas: Sequence[Data]) -> List[torch.Tensor]:
    """The reference's ``custom_kernel`` for every rank of an emulated world at once: ``datas[r]`` is
    what rank r would pass; element r of the result is what rank r would get back, ``[M/W, N]``."""
    W = len(datas)
    x, w, bias = pack_world(datas, datas[0][0].device)
    M = x.shape[1]
    assert M % W == 0, "m must be divisible by world_size"
    out = HipGemmReduceScatter(W).forward(x, w, bias)
    return list(out.view(W, M // W, out.shape[1]).unbind(0))


def custom_kernel(data: Data) -> torch.Tensor:
    """A world of one rank: the linear layer itself (``[M, N]``)."""
    return custom_kernel_world([data])[0]
