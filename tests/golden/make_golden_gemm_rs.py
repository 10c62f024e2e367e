"""Writes tests/golden/gemm_rs_*.npz by running the reference's own gemm_rs ``ref_kernel``.

Run in the build container only (the reference tree is not available elsewhere):

    python tests/golden/make_golden_gemm_rs.py [/root/reference/gemm_rs]

For each case it starts ``world_size`` local processes on the gloo backend (CPU tensors), hands
every rank its shard ``(input[M, K/W], weight[N, K/W], bias[N] or None)`` in the distribution of
the reference's ``generate_input`` (uniform in +-0.01, bf16; the reference's own generator needs a
CUDA device) and calls the reference's ``ref_kernel``: a bf16 matmul, the bias added on every rank,
then ``reduce_scatter_tensor``.  Stored per rank: the shard and the ``[M/W, N]`` result, 16-bit
floats as int16 bit patterns.  The fixtures are data only; no reference source is stored.

What these vectors pin and reading alone leaves open: that the bias enters once per rank (so W
times in the sum), which row block a rank receives, and the size of the rounding noise of the
bf16 partial products and the bf16 reduction that a result has to stay within.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (world_size, m, n, k, has_bias, seed)
CASES = {
    "gemm_rs_w2_bias": (2, 8, 24, 64, True, 21),
    "gemm_rs_w4_nobias": (4, 16, 40, 160, False, 22),
    "gemm_rs_w8_bias": (8, 64, 96, 2880, True, 23),   # local K = 360: not a multiple of 64
    "gemm_rs_w8_wide": (8, 256, 320, 1024, True, 24),
}


def make_rank_inputs(case, rank):
    W, m, n, k, has_bias, seed = case
    g = torch.Generator().manual_seed(seed + rank)
    kl = k // W
    x = ((torch.rand((m, kl), generator=g) * 2 - 1) * 0.01).to(torch.bfloat16)
    w = ((torch.rand((n, kl), generator=g) * 2 - 1) * 0.01).to(torch.bfloat16)
    bias = None
    if has_bias:
        g.manual_seed(seed)  # the same bias on every rank, as in the reference
        bias = ((torch.rand((n,), generator=g) * 2 - 1) * 0.01).to(torch.bfloat16)
    return x, w, bias


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy()


def worker(rank, name, ref_dir, port, out_dir):
    case = CASES[name]
    W = case[0]
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(port)
    dist.init_process_group("gloo", rank=rank, world_size=W)
    sys.path.insert(0, ref_dir)
    import reference as ref  # the reference's gemm_rs/reference.py

    x, w, bias = make_rank_inputs(case, rank)
    out = ref.ref_kernel((x, w, bias))
    ok, msg = ref.check_implementation((x, w, bias), out)
    assert ok, msg
    parts = dict(input=_bits(x), weight=_bits(w), out=_bits(out))
    if bias is not None:
        parts["bias"] = _bits(bias)
    np.savez(os.path.join(out_dir, f"{name}.rank{rank}.npz"), **parts)
    dist.barrier()
    dist.destroy_process_group()


def main():
    ref_dir = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/gemm_rs"
    tmp = os.path.join(HERE, "_tmp")
    os.makedirs(tmp, exist_ok=True)
    port = 29640
    for name, case in CASES.items():
        W, m, n, k, has_bias, seed = case
        mp.spawn(worker, args=(name, ref_dir, port, tmp), nprocs=W, join=True)
        port += 1
        merged = dict(world_size=np.int64(W), m=np.int64(m), n=np.int64(n), k=np.int64(k),
                      has_bias=np.int64(int(has_bias)))
        for r in range(W):
            part = np.load(os.path.join(tmp, f"{name}.rank{r}.npz"))
            for key in part.files:
                merged[f"r{r}_{key}"] = part[key]
            os.remove(os.path.join(tmp, f"{name}.rank{r}.npz"))
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **merged)
        print("wrote", name)
    os.rmdir(tmp)


if __name__ == "__main__":
    main()
