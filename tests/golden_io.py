"""Loader for the fixtures under tests/golden/ (data written by make_golden.py)."""
import os
import types

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GOLDEN_CASES = ("ref_w2_fp16", "ref_w4_bf16", "ref_w4_fp16_dup", "ref_w8_bf16")


def _f(arr, dtype):
    return torch.from_numpy(np.ascontiguousarray(arr)).view(dtype)


def load_golden(name):
    """Returns (cfg, world, expected) -- expected[r] holds the reference's outputs of rank r."""
    from kernel_amd.contract import MoEConfig, RankData

    z = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
    dtype = getattr(torch, str(z["dtype"]))
    W = int(z["world_size"])
    cfg = MoEConfig(int(z["num_experts"]), int(z["experts_per_token"]), int(z["hidden_dim"]),
                    int(z["max_num_tokens"]), in_dtype=dtype, out_dtype=dtype)
    world, expected = [], []
    for r in range(W):
        idx = torch.from_numpy(z[f"r{r}_indices"])
        w = torch.from_numpy(z[f"r{r}_weights"])
        x = _f(z[f"r{r}_x"], dtype)
        world.append(RankData(idx.shape[0], idx, w, x))
        expected.append(types.SimpleNamespace(
            expert_num_tokens=torch.from_numpy(z[f"r{r}_expert_num_tokens"]),
            expert_x=_f(z[f"r{r}_expert_x"], dtype).view(-1, cfg.hidden_dim),
            expert_meta=torch.from_numpy(z[f"r{r}_expert_meta"]).view(-1, 5),
            expert_y=_f(z[f"r{r}_expert_y"], dtype).view(-1, cfg.hidden_dim),
            y=_f(z[f"r{r}_y"], dtype).view(-1, cfg.hidden_dim),
        ))
    return cfg, world, expected


def golden_compact(cfg, expected):
    """Concatenate the per-owner outputs into the expert-major compact arrays."""
    counts = torch.cat([e.expert_num_tokens for e in expected]).to(torch.int32)
    return dict(
        counts=counts,
        disp_x=torch.cat([e.expert_x for e in expected], 0),
        meta=torch.cat([e.expert_meta for e in expected], 0),
        expert_y=torch.cat([e.expert_y for e in expected], 0),
        y=torch.cat([e.y for e in expected], 0),
    )


def bits(t):
    return t.contiguous().view(torch.int16) if t.dtype in (torch.float16, torch.bfloat16) else t
