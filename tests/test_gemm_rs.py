"""GEMM + reduce-scatter (the reference's gemm_rs problem) on one GPU.

CPU: the oracle against the vectors the reference itself wrote over gloo, the C ABI of
include/gemm_rs.h (symbols, host-side argument checks), the input generator.
GPU (``-m gpu``): the HIP path through the C ABI against the reference's vectors, the oracle, the
exact f64 sum on sampled rows and an f32 matrix product of the whole output, for the reference's
test and benchmark shapes at full size and for each of the three kernel forms.

Tolerances.  The reference accepts rtol = atol = 1e-2 (gemm_rs/reference.py:66).  The HIP path
accumulates in f32 over the whole of K and rounds once, so it is also held to the exact sum within
one bf16 rounding: |out - exact| <= 2^-8 |exact| + 1e-6 (2^-9 is half a unit in the last place; the
f32 accumulation adds less than 2^-15 relative over these K).
"""
import ctypes
import glob
import os
import re

import numpy as np
import pytest
import torch

from kernel_amd import _lib
from kernel_amd import gemm_rs as G
from oracle import gemm_rs as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gemm_rs.h")
GOLDEN = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "gemm_rs_*.npz")))
E_NULL, E_SHAPE, E_DTYPE, E_WORKSPACE, E_ALIGN = -1, -2, -3, -4, -5
A = 0x1000  # any non-NULL, 16-byte aligned address; never dereferenced on the host


def load_golden(path):
    d = np.load(path)
    W = int(d["world_size"])
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)
    bias = bf(d["r0_bias"]) if int(d["has_bias"]) else None
    datas = [(bf(d[f"r{r}_input"]), bf(d[f"r{r}_weight"]), bias) for r in range(W)]
    want = torch.cat([bf(d[f"r{r}_out"]) for r in range(W)], 0)
    return datas, want


def within_one_rounding(out, exact):
    err = (out.double() - exact).abs()
    return bool((err <= exact.abs() * 2.0 ** -8 + 1e-6).all()), float(err.max())


# ---------------------------------------------------------------------------------------------
# CPU
# ---------------------------------------------------------------------------------------------
def test_golden_files_exist():
    assert len(GOLDEN) == 4


@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_against_the_reference_vectors(path):
    datas, want = load_golden(path)
    got = O.ref_world(datas)
    assert got.shape == want.shape and got.dtype == want.dtype
    W = len(datas)
    if W == 2:  # one addition in the reduction: no order to choose, so the bits are defined
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # a quarter of the reference's own tolerance (a few bf16 units in the last place of the sum)
    assert torch.allclose(got.float(), want.float(), rtol=2.5e-3, atol=2.5e-3)
    ok, _ = O.check_implementation(want, got)
    assert ok
    # both are the exact sum up to the rounding of W bf16 products and W - 1 bf16 additions
    exact = O.exact_world(datas)
    bound = 2.0 ** -8 * (2 * W) * exact.abs().max().item() + 1e-6
    assert (want.double() - exact).abs().max().item() <= bound
    assert (got.double() - exact).abs().max().item() <= bound


def test_the_bias_enters_once_per_rank():
    """What the vectors pin and a reading could get wrong: W times the bias, not once."""
    datas, want = load_golden([p for p in GOLDEN if p.endswith("gemm_rs_w8_bias.npz")][0])
    W, bias = len(datas), datas[0][2]
    no_bias = O.exact_world([(x, w, None) for x, w, _ in datas])
    resid = (want.double() - no_bias).mean(0)  # per column: what the bias contributed
    assert torch.allclose(resid, W * bias.double(), atol=2e-4)
    assert not torch.allclose(resid, bias.double(), atol=2e-3)


def test_row_block_r_is_rank_r(tmp_path):
    datas, want = load_golden([p for p in GOLDEN if p.endswith("gemm_rs_w4_nobias.npz")][0])
    W, M = len(datas), want.shape[0]
    exact = O.exact_world(datas)
    d = np.load([p for p in GOLDEN if p.endswith("gemm_rs_w4_nobias.npz")][0])
    for r in range(W):
        mine = torch.from_numpy(d[f"r{r}_out"].copy()).view(torch.bfloat16)
        blk = exact[r * M // W:(r + 1) * M // W]
        assert mine.shape == blk.shape
        assert (mine.double() - blk).abs().max().item() <= 2.0 ** -8 * 2 * W * exact.abs().max().item() + 1e-6


def test_generate_input_follows_the_reference_distribution():
    x, w, b = G.generate_input(3, 8, 64, 96, 2880, True, 7)
    assert x.shape == (64, 360) and w.shape == (96, 360) and b.shape == (96,)
    assert x.dtype == w.dtype == b.dtype == torch.bfloat16
    assert x.abs().max().item() <= 0.0101 and w.abs().max().item() <= 0.0101  # bf16 rounds 0.00999.. up
    assert abs(x.float().mean().item()) < 2e-4 and abs(x.float().std().item() - 0.01 / 3 ** 0.5) < 3e-4
    x2, _, b2 = G.generate_input(4, 8, 64, 96, 2880, True, 7)
    assert not torch.equal(x, x2) and torch.equal(b, b2)  # the same bias on every rank
    assert G.generate_input(0, 8, 64, 96, 2880, False, 7)[2] is None
    assert len(G.TEST_SPECS) == 11 and len(G.BENCHMARK_SPECS) == 6


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(gemm_rs_[a-z0-9_]+)\s*\(", text)))


def test_header_binding_and_exports_agree():
    assert declared_functions() == sorted(_lib.GEMM_RS_PROTOTYPES)
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), f"{name} is declared in include/gemm_rs.h but not exported"


def test_host_side_argument_checks():
    lib = _lib.load()
    f = lib.gemm_rs_forward
    ok = dict(M=256, N=256, K=1024, W=8)
    call = lambda inp=A, wt=A, out=A, M=256, N=256, K=1024, W=8, et=_lib.BF16, ws=None, wsb=0: f(
        inp, wt, None, out, M, N, K, W, 0, 0, et, ws, wsb, None)
    assert call(K=1000) == E_SHAPE            # K not divisible by W
    assert call(K=8 * 12) == E_SHAPE          # local K not a multiple of 8
    assert call(W=0) == E_SHAPE and call(N=0) == E_SHAPE and call(M=-1) == E_SHAPE
    assert call(et=7) == E_DTYPE
    assert call(M=0) == 0                     # nothing to do, nothing launched
    assert call(inp=None) == E_NULL and call(wt=None) == E_NULL and call(out=None) == E_NULL
    assert call(inp=A + 4) == E_ALIGN
    assert f(A, A, None, A, 256, 256, 1024, 8, 100, 0, _lib.BF16, None, 0, None) == E_SHAPE  # shards would overlap
    # an output of few tiles keeps one partial product per shard and needs the workspace for them
    need = lib.gemm_rs_workspace_bytes(64, 7168, 18432, 8)
    assert need == 8 * 64 * 7168 * 4
    assert call(M=64, N=7168, K=18432) == E_WORKSPACE
    assert call(M=64, N=7168, K=18432, ws=A, wsb=need - 1) == E_WORKSPACE
    assert lib.gemm_rs_workspace_bytes(8192, 4096, 14336, 8) == 0  # whole slabs per shard, enough tiles
    # ragged shards on 256 x 256 tiles: room for both operands in rows padded to whole 64-column slabs
    # (optional: without it the product runs on the rows as they lie)
    assert lib.gemm_rs_workspace_bytes(8192, 8192, 29568, 8) == 8 * (8192 + 8192) * 3712 * 2
    # a few hundred rows: 256 x 128 tiles with the shards in four groups
    assert lib.gemm_rs_workspace_bytes(512, 4096, 12288, 8) == 4 * 512 * 4096 * 4
    assert lib.gemm_rs_workspace_bytes(64, 64, 100, 8) == 0  # invalid shape: no size


def test_no_cpu_path():
    x, w, b = G.generate_input(0, 1, 8, 8, 64, True, 1)
    with pytest.raises(RuntimeError):
        G.custom_kernel((x, w, b))


# ---------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------
def to_dev(datas, dev):
    return [(x.to(dev), w.to(dev), b.to(dev) if b is not None else None) for x, w, b in datas]


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: os.path.basename(p)[:-4])
def test_hip_against_the_reference_vectors(gpu_device, path):
    datas, want = load_golden(path)
    outs = G.custom_kernel_world(to_dev(datas, gpu_device))
    W, M = len(datas), want.shape[0]
    assert len(outs) == W and all(o.shape == (M // W, want.shape[1]) for o in outs)
    got = torch.cat(outs, 0).cpu()
    ok, msg = O.check_implementation(want, got)  # the reference's own acceptance test, on its own result
    assert ok, msg
    ok, worst = within_one_rounding(got, O.exact_world(datas))
    assert ok, worst


def spec_id(s):
    return f"m{s['m']}-n{s['n']}-k{s['k']}-{'bias' if s['has_bias'] else 'nobias'}"


@pytest.mark.gpu
@pytest.mark.parametrize("spec", G.TEST_SPECS + G.BENCHMARK_SPECS, ids=spec_id)
def test_reference_shapes_at_full_size(gpu_device, spec):
    W, m, n, k = spec["world_size"], spec["m"], spec["n"], spec["k"]
    datas = [G.generate_input(r, device=None, **spec) for r in range(W)]
    x, w, bias = G.pack_world(datas, gpu_device)
    out = G.HipGemmReduceScatter(W).forward(x, w, bias)
    torch.cuda.synchronize()
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    # (1) every element against an f32 matrix product of the concatenated shards (torch's own GEMM)
    xc = x.permute(1, 0, 2).reshape(m, k).float()
    wc = w.permute(1, 0, 2).reshape(n, k).float()
    ref = xc @ wc.T
    if bias is not None:
        ref += W * bias.float()
    assert torch.allclose(out.float(), ref, rtol=1e-2, atol=1e-2)
    err = (out.float() - ref).abs()
    assert bool((err <= ref.abs() * 2.0 ** -8 + 2e-6).all()), float(err.max())
    del xc, wc, ref, err
    # (2) sampled rows against the exact f64 sum on the CPU
    g = torch.Generator().manual_seed(spec["seed"])
    rows = torch.randperm(m, generator=g)[:16]
    sample = [(d[0][rows], d[1], d[2]) for d in datas]
    ok, worst = within_one_rounding(out[rows.to(gpu_device)].cpu(), O.exact_world(sample))
    assert ok, worst
    # (3) the whole oracle where it finishes in seconds
    if m * n * k <= 3e10:
        want = O.ref_world(datas)
        ok, msg = O.check_implementation(want, out.cpu())
        assert ok, msg


@pytest.mark.gpu
@pytest.mark.parametrize("form", [256, 129, 131, 132, 130, 128, 32])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("k", [1024, 1440, 4 * 72], ids=["k256", "k360", "k72"])
def test_each_kernel_form(gpu_device, options, form, dtype, k):
    """256 x 256 tiles, 256 x 128 tiles (129; 131 / 132: 192 / 128 of their rows in use, the former on
    the map that deals the tiles out evenly; 130: with per-shard partial products), 128 x 128 tiles and
    their per-shard partial products (32) on one shape with ragged
    edges (M and N not multiples of the tiles); local K a multiple of the 64-column slab, five slabs
    and a short one (360: the wide tiles start the last slab of a shard early and mask what it
    shares with the one before), and one slab and a bit (72)."""
    options.set("GEMM_TILE", form)
    W, m, n = 4, 392, 600
    g = torch.Generator().manual_seed(form)
    datas = [(((torch.rand((m, k // W), generator=g) * 2 - 1) * 0.05).to(dtype),
              ((torch.rand((n, k // W), generator=g) * 2 - 1) * 0.05).to(dtype),
              None) for _ in range(W)]
    bias = ((torch.rand((n,), generator=g) * 2 - 1) * 0.05).to(dtype)
    datas = [(x, w, bias) for x, w, _ in datas]
    x, w, b = G.pack_world(datas, gpu_device)
    exact = O.exact_world(datas)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    # ragged shards on the wide tiles: on the zero-padded copy of the operands (with the workspace) and
    # in place (without it: the early-starting last slab of a shard)
    for pad_ragged in (True, False):
        out = G.HipGemmReduceScatter(W, pad_ragged=pad_ragged).forward(x, w, b).cpu()
        err = (out.double() - exact).abs()
        assert bool((err <= exact.abs() * ulp + 1e-6).all()), (pad_ragged, float(err.max()))


@pytest.mark.gpu
def test_local_k_with_a_short_last_slab_and_one_rank(gpu_device):
    """Local K = 360 (five slabs of 64 and one of 40, the reference's 2880 / 8), and a world of one."""
    for W, m, n, k in ((8, 64, 2880, 2880), (1, 130, 136, 72)):
        datas = [G.generate_input(r, W, m if m % W == 0 else m, n, k, True, 5) if m % W == 0 else None for r in range(W)]
        if datas[0] is None:  # M need not divide by W for the sum itself
            g = torch.Generator().manual_seed(9)
            datas = [(((torch.rand((m, k // W), generator=g) * 2 - 1) * 0.01).to(torch.bfloat16),
                      ((torch.rand((n, k // W), generator=g) * 2 - 1) * 0.01).to(torch.bfloat16), None)
                     for _ in range(W)]
        x, w, b = G.pack_world(datas, gpu_device)
        out = G.HipGemmReduceScatter(W).forward(x, w, b).cpu()
        ok, worst = within_one_rounding(out, O.exact_world(datas))
        assert ok, worst


@pytest.mark.gpu
@pytest.mark.parametrize("form", [256, 129, 131, 130, 128, 32])
def test_shards_with_gaps_between_them(gpu_device, options, form):
    """Shard strides of the C ABI: the shards of each operand lie further apart than their size."""
    options.set("GEMM_TILE", form)
    lib = _lib.load()
    W, m, n, kl, gap_a, gap_b = 4, 264, 272, 128, 64, 200
    g = torch.Generator().manual_seed(31)
    datas = [(((torch.rand((m, kl), generator=g) * 2 - 1) * 0.05).to(torch.bfloat16),
              ((torch.rand((n, kl), generator=g) * 2 - 1) * 0.05).to(torch.bfloat16), None) for _ in range(W)]
    sa, sb = m * kl + gap_a, n * kl + gap_b
    a = torch.full((W * sa,), float("nan"), dtype=torch.bfloat16, device=gpu_device)  # the gaps hold NaN
    b = torch.full((W * sb,), float("nan"), dtype=torch.bfloat16, device=gpu_device)
    for s, (x, w, _) in enumerate(datas):
        a[s * sa:s * sa + m * kl] = x.to(gpu_device).reshape(-1)
        b[s * sb:s * sb + n * kl] = w.to(gpu_device).reshape(-1)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu_device)
    need = int(lib.gemm_rs_workspace_bytes(m, n, kl * W, W))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=gpu_device)
    rc = lib.gemm_rs_forward(a.data_ptr(), b.data_ptr(), None, out.data_ptr(), m, n, kl * W, W, sa, sb, _lib.BF16,
                             ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    ok, worst = within_one_rounding(out.cpu(), O.exact_world(datas))
    assert ok, worst


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(8, 64, 512, 8 * 256), (4, 520, 520, 4 * 128)], ids=["partial-products", "tiles"])
def test_replays_of_a_captured_graph_follow_their_inputs(gpu_device, shape):
    """The entry point only enqueues kernels (the grouped form: the tile kernel, then the reduction
    over its partial products in the caller's workspace), so a call can be captured into a hipGraph;
    every replay is checked against an eager run on the inputs of the moment, with eager work and
    synchronisations between the replays."""
    W, m, n, k = shape
    op = G.HipGemmReduceScatter(W)
    g = torch.Generator().manual_seed(77)
    fresh = lambda: (((torch.rand((W, m, k // W), generator=g) * 2 - 1) * 0.05).to(torch.bfloat16).to(gpu_device),
                     ((torch.rand((W, n, k // W), generator=g) * 2 - 1) * 0.05).to(torch.bfloat16).to(gpu_device),
                     ((torch.rand((n,), generator=g) * 2 - 1) * 0.05).to(torch.bfloat16).to(gpu_device))
    x, w, b = fresh()
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu_device)
    op.forward(x, w, b, out=out)  # allocates the workspace outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            op.forward(x, w, b, out=out)
    for _ in range(3):
        nx, nw, nb = fresh()
        x.copy_(nx), w.copy_(nw), b.copy_(nb)
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = G.HipGemmReduceScatter(W).forward(x, w, b)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16))
        ok, worst = within_one_rounding(got.cpu(), O.exact_world([(x[s].cpu(), w[s].cpu(), b.cpu()) for s in range(W)]))
        assert ok, worst
