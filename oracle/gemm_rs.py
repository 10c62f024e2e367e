"""CPU restatement of the reference's GEMM + reduce-scatter (gemm_rs/reference.py).

TEST INFRASTRUCTURE ONLY: imported by tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py``; the product path never calls it.

``ref_world`` follows ``ref_kernel`` (reference.py:36-60) for a world held in one process, with
torch's own CPU arithmetic: every rank's ``matmul(input, weight.T)`` in bf16 (:53), the bias added
on every rank (:54-55), then the sum over the ranks (:58-59) and the row block each rank receives.
The order in which ``reduce_scatter_tensor`` adds the W partial products is the backend's (a ring
in gloo and RCCL), so the reference's own result is only defined up to the rounding of that sum;
here the partial products are added in rank order in bf16.  ``exact_world`` is the same sum in f64.

Pinned by tests/golden/gemm_rs_*.npz, which the reference itself wrote in the build container over
gloo with 2, 4 and 8 local processes (tests/golden/make_golden_gemm_rs.py): ``ref_world`` equals
them bit for bit where W = 2 (one addition: no order to choose) and stays within 1/4 of the
reference's tolerance elsewhere; both lie within bf16 rounding noise of ``exact_world``.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

Data = Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]


def ref_world(datas: Sequence[Data]) -> torch.Tensor:
    """``[M, N]``: row block r is what rank r of the reference returns."""
    total = None
    for x, w, bias in datas:
        out = torch.matmul(x, w.T)  # reference.py:53
        if bias is not None:
            out = out + bias        # :54-55
        total = out if total is None else total + out  # :59, rank order
    return total


def exact_world(datas: Sequence[Data]) -> torch.Tensor:
    """The same sum without any intermediate rounding (f64)."""
    total = None
    for x, w, bias in datas:
        out = x.double() @ w.double().T
        if bias is not None:
            out = out + bias.double()
        total = out if total is None else total + out
    return total


def check_implementation(expected: torch.Tensor, output: torch.Tensor):
    """The reference's acceptance test (reference.py:63-71): rtol = atol = 1e-2."""
    if not torch.allclose(output.float(), expected.float(), rtol=1e-2, atol=1e-2):
        return False, "Output values mismatch"
    return True, ""
