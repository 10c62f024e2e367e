"""TEST INFRASTRUCTURE -- ``ref_kernel`` / ``check_implementation`` of the contract.

Restates all2all/reference.py:256-283 on top of the CPU oracle: the expected output
of ``custom_kernel(data)`` for one rank, and the comparison the reference applies to
it (device equality first, then ``torch.allclose``).  The reference's tolerance is
rtol=1e-2, atol=5e-3 (fp16); the bf16 workloads of this build use rtol=atol=1e-2.
"""
from __future__ import annotations

import torch

from . import all2all_vec

REFERENCE_TOL = dict(rtol=1e-2, atol=5e-3)  # reference.py:279
BF16_TOL = dict(rtol=1e-2, atol=1e-2)


def _world_of(cfg, rank_data, rank, world_size):
    class _Empty:
        num_tokens = 0
        indices = torch.empty(0, cfg.experts_per_token, dtype=torch.int32)
        weights = torch.empty(0, cfg.experts_per_token, dtype=torch.float32)
        x = torch.empty(0, cfg.hidden_dim, dtype=cfg.in_dtype)

    class _Cpu:
        num_tokens = rank_data.num_tokens
        indices = rank_data.indices.cpu()
        weights = rank_data.weights.cpu()
        x = rank_data.x.cpu()

    return [_Cpu if r == rank else _Empty for r in range(world_size)]


def ref_kernel(data, stub_kind: int = 0, combine_mode: int = 0) -> torch.Tensor:
    """reference.py:256-272 -- ``y[:num_tokens]`` on the device of ``rank_data.x``."""
    cfg, rank_data, rank, world_size = data
    out = all2all_vec.run_world(cfg, _world_of(cfg, rank_data, rank, world_size), stub_kind=stub_kind,
                                combine_mode=combine_mode)
    return out["y"][: rank_data.num_tokens].to(rank_data.x.device)


def check_implementation(data, output, stub_kind: int = 0, rtol=REFERENCE_TOL["rtol"], atol=REFERENCE_TOL["atol"]):
    """reference.py:275-283 -- ``(ok, message)``."""
    expected = ref_kernel(data, stub_kind=stub_kind)
    if output.device != expected.device:
        return False, f"Output device mismatch: {output.device} != {expected.device}"
    if output.dtype != expected.dtype:
        return False, f"Output dtype mismatch: {output.dtype} != {expected.dtype}"
    if output.shape != expected.shape:
        return False, f"Output shape mismatch: {tuple(output.shape)} != {tuple(expected.shape)}"
    if not torch.allclose(output, expected, rtol=rtol, atol=atol):
        diff = (output.float() - expected.float()).abs()
        bad = int((diff > atol + rtol * expected.float().abs()).sum())
        return False, f"Output values mismatch: {bad} elements out of tolerance, max abs diff {float(diff.max())}"
    return True, ""
