"""Seeded random shapes through the one-call forward (every form it can take) and the GEMM +
reduce-scatter, against the oracles: world sizes, expert counts, top-k, row lengths, ragged and empty
ranks, both element types, both combine modes, both stub flavours, fp8 dispatch, input scales.
Every case is small; the point is the variety of kernel instantiations and geometries."""
import random

import pytest
import torch

from kernel_amd import _lib, contract as C, gemm_rs as G
from kernel_amd.all2all import HipAllToAll, concat_world
from oracle import all2all_vec as V
from oracle import gemm_rs as O


def _bits(t):
    return t.view(torch.int16) if t.dtype in (torch.float16, torch.bfloat16) else t


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_forward_on_random_shapes(gpu_device, options, seed):
    rnd = random.Random(seed)
    for case in range(40):
        W = rnd.choice([1, 2, 4, 8])
        E = W * rnd.choice([1, 2, 4, 8, 16, 32])
        K = rnd.choice([k for k in (1, 2, 3, 4, 6, 8, 12) if k <= E])
        fp8 = rnd.random() < 0.3
        H = rnd.choice([128, 256, 384, 1024, 2048, 2816, 4096, 7168])
        if not fp8 and rnd.random() < 0.2:
            H = rnd.choice([8, 72, 2880])  # rows that are not a multiple of 64 vectors or of 128 columns
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        mode, stub = rnd.choice([0, 1]), rnd.choice([0, 1])
        toks = [rnd.choice([0, 1, 3, 17, 64, 130, 257]) for _ in range(W)]
        if sum(toks) == 0:
            toks[0] = 5
        if sum(toks) * K * H > 40e6:
            toks = [min(t, 17) for t in toks]
        g = torch.Generator().manual_seed(seed * 1000 + case)
        cfg = C.MoEConfig(E, K, H, max(toks) + 1, dtype, dtype)
        scale = rnd.choice([1.0, 1e-3, 30.0])
        world = []
        for T in toks:
            idx = (torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32) if T
                   else torch.zeros(0, K, dtype=torch.int32))
            world.append(C.RankData(T, idx, torch.rand(T, K, generator=g), (torch.randn(T, H, generator=g) * scale).to(dtype)))
        what = f"seed {seed} case {case}: W{W} E{E} K{K} H{H} tokens {toks} {dtype} fp8={fp8} mode={mode} stub={stub}"
        want = V.run_world(cfg, world, stub_kind=stub, fp8=fp8, combine_mode=mode)
        x, idx, w, rs = concat_world(world, gpu_device)
        for fuse_stub, two in ((True, 0), (True, 1), (False, 0)):
            options.set("TWO_LAUNCHES", two)
            ata = HipAllToAll(cfg, 0, W, stub_kind=stub, combine_mode=mode, fp8_dispatch=fp8, fuse_stub=fuse_stub)
            y = ata.forward(x, idx, w, rs)
            torch.cuda.synchronize()
            assert torch.equal(_bits(y.cpu()), _bits(want["y"])), (what, fuse_stub, two)
            d = ata.last
            for key, got in (("counts", d.counts), ("offsets", d.offsets), ("slot_of_entry", d.slot_of_entry),
                             ("src_of_slot", d.src_of_slot), ("meta", d.meta), ("disp_x", d.disp_x)):
                e = want[key]
                gg = _bits(got.cpu())
                ee = _bits(e) if gg.dtype != torch.uint8 else e.view(torch.uint8)
                assert gg.shape == ee.shape and torch.equal(gg, ee), (what, fuse_stub, two, key)
            assert int(d.status.item()) == 0, what


@pytest.mark.gpu
def test_gemm_rs_on_random_shapes(gpu_device, options):
    rnd = random.Random(21)
    for case in range(80):
        W = rnd.choice([1, 2, 3, 4, 8])
        kl = 8 * rnd.choice([1, 2, 7, 8, 9, 16, 45, 64, 100])
        m = rnd.choice([1, 8, 63, 64, 130, 256, 300, 513, 1024])
        n = rnd.choice([4, 8, 100, 128, 136, 256, 260, 520, 1030])
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        options.set("GEMM_TILE", rnd.choice([0, 0, 256, 128, 32]))
        g = torch.Generator().manual_seed(case)
        bias = ((torch.rand((n,), generator=g) * 2 - 1) * 0.05).to(dtype) if rnd.random() < 0.5 else None
        datas = [(((torch.rand((m, kl), generator=g) * 2 - 1) * 0.05).to(dtype),
                  ((torch.rand((n, kl), generator=g) * 2 - 1) * 0.05).to(dtype), bias) for _ in range(W)]
        x, w, b = G.pack_world(datas, gpu_device)
        out = G.HipGemmReduceScatter(W).forward(x, w, b).cpu()
        exact = O.exact_world(datas)
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11  # one rounding of the exact sum
        err = (out.double() - exact).abs()
        assert bool((err <= exact.abs() * ulp + 1e-6).all()), (case, W, m, n, kl, dtype, float(err.max()))
