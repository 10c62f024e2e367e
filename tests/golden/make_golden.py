"""Writes tests/golden/ref_*.npz by running the reference's own ``PyTorchAllToAll``.

Run in the build container only (the reference tree is not available elsewhere):

    python tests/golden/make_golden.py [/root/reference/all2all]

For each case it starts ``world_size`` local processes on the gloo backend (CPU
tensors), hands every rank a hand-built record with the attributes the reference
reads (``num_tokens, indices, weights, x`` -- its own ``RankTestData`` constructor
needs a CUDA device), and calls the reference's ``PyTorchAllToAll.dispatch``,
``.combine`` and ``ref_kernel``.  What is stored per rank: the inputs, and the
initialised part of every output (``expert_num_tokens``, ``expert_x[le,:count]``,
``expert_meta[le,:count]``, ``y``).  16-bit floats are stored as their int16 bit
patterns.  The fixtures are data only; no reference source is stored.

These vectors pin what reading alone leaves open: the row order after the
all-to-all (ascending source rank), the per-expert arrival order, the accumulation
order and per-step rounding of the weighted sum, and the stub arithmetic.
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (world_size, E, K, H, max_num_tokens, dtype, seed, allow duplicate experts in a token)
CASES = {
    "ref_w2_fp16": (2, 8, 2, 32, 6, torch.float16, 11, False),
    "ref_w4_bf16": (4, 16, 3, 64, 9, torch.bfloat16, 12, False),
    "ref_w4_fp16_dup": (4, 8, 4, 16, 7, torch.float16, 13, True),
    "ref_w8_bf16": (8, 64, 6, 128, 8, torch.bfloat16, 14, False),
}


def make_rank_inputs(case, rank):
    W, E, K, H, max_tok, dtype, seed, dup = case
    g = torch.Generator().manual_seed(seed * 1000 + rank)
    T = int(torch.randint(1, max_tok, [1], generator=g).item())
    if dup:
        idx = torch.randint(0, E, (T, K), generator=g).to(torch.int32)
    else:
        idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, K, generator=g, dtype=torch.float32)
    x = torch.randn(T, H, generator=g, dtype=torch.float32).to(dtype)
    return T, idx, w, x


def _bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.contiguous().view(torch.int16).numpy()
    return t.contiguous().numpy()


def worker(rank, name, ref_dir, port, out_dir):
    case = CASES[name]
    W, E, K, H, max_tok, dtype, seed, dup = case
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(port)
    dist.init_process_group("gloo", rank=rank, world_size=W)
    sys.path.insert(0, ref_dir)
    import reference as ref  # the reference's all2all/reference.py

    cfg = ref.MoEConfig(num_experts=E, experts_per_token=K, hidden_dim=H, max_num_tokens=max_tok, in_dtype=dtype,
                        out_dtype=dtype)
    T, idx, w, x = make_rank_inputs(case, rank)
    rd = types.SimpleNamespace(num_tokens=T, indices=idx, weights=w, x=x)

    ata = ref.PyTorchAllToAll(cfg, rank, W)
    num, ex, em = ata.dispatch(rd.x, rd.indices)
    ey = ex.to(cfg.out_dtype) * (1 + rank)
    y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype)
    ata.combine(y, rd.weights, em, ey, num)
    y = y[:T]
    y2 = ref.ref_kernel((cfg, rd, rank, W))
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))

    E_l = E // W
    rows_x = [ex[le, : int(num[le])] for le in range(E_l)]
    rows_m = [em[le, : int(num[le])] for le in range(E_l)]
    rows_y = [ey[le, : int(num[le])] for le in range(E_l)]
    np.savez(
        os.path.join(out_dir, f"{name}.rank{rank}.npz"),
        indices=idx.numpy(), weights=w.numpy(), x=_bits(x),
        expert_num_tokens=num.numpy(),
        expert_x=_bits(torch.cat(rows_x, 0)), expert_meta=torch.cat(rows_m, 0).numpy(),
        expert_y=_bits(torch.cat(rows_y, 0)), y=_bits(y),
    )
    dist.barrier()
    dist.destroy_process_group()


def main():
    ref_dir = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/all2all"
    tmp = os.path.join(HERE, "_tmp")
    os.makedirs(tmp, exist_ok=True)
    port = 29610
    for name, case in CASES.items():
        W = case[0]
        mp.spawn(worker, args=(name, ref_dir, port, tmp), nprocs=W, join=True)
        port += 1
        merged = dict(world_size=np.int64(W), num_experts=np.int64(case[1]), experts_per_token=np.int64(case[2]),
                      hidden_dim=np.int64(case[3]), max_num_tokens=np.int64(case[4]),
                      dtype=np.str_(str(case[5]).replace("torch.", "")))
        for r in range(W):
            part = np.load(os.path.join(tmp, f"{name}.rank{r}.npz"))
            for k in part.files:
                merged[f"r{r}_{k}"] = part[k]
            os.remove(os.path.join(tmp, f"{name}.rank{r}.npz"))
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **merged)
        print("wrote", name)
    os.rmdir(tmp)


if __name__ == "__main__":
    main()
