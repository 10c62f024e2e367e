"""Pins of the CPU oracle that do not restate its formulas.

  * literal (row-loop) and vectorised forms agree bit for bit on multi-rank worlds, ragged
    and empty ranks, duplicate experts, both stub flavours;
  * route: brute-force O(R^2) slot ranks, bijection, segment invariants;
  * combine: algebraic special cases with known answers (one-hot weights give back x, K=1
    gives the stub, zero weights give zero), the dispatch-free closed form, and an f64
    reference bound for the f32 mode;
  * fp8: an independent table-driven e4m3fn encoder (nearest value, ties to even mantissa)
    against torch's cast, plus the stated per-block error bound.
"""
import numpy as np
import pytest
import torch

from golden_io import bits
from kernel_amd import contract as C
from oracle import all2all_literal as L
from oracle import all2all_vec as V
from oracle import checker


def random_world(seed, W, E, K, H, tokens, dtype=torch.bfloat16, dup=False):
    g = torch.Generator().manual_seed(seed)
    cfg = C.MoEConfig(E, K, H, max(max(tokens), 1) + 1, dtype, dtype)
    world = []
    for n in tokens:
        if dup:
            idx = torch.randint(0, E, (n, K), generator=g).to(torch.int32)
        else:
            idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32) if n else \
                torch.empty(0, K, dtype=torch.int32)
        world.append(C.RankData(n, idx, torch.rand(n, K, generator=g), torch.randn(n, H, generator=g).to(dtype)))
    return cfg, world


WORLDS = [
    dict(seed=1, W=1, E=8, K=2, H=32, tokens=[9]),
    dict(seed=2, W=4, E=16, K=4, H=24, tokens=[5, 0, 7, 2]),
    dict(seed=3, W=8, E=64, K=6, H=16, tokens=[3, 1, 4, 1, 5, 9, 2, 6], dtype=torch.float16),
    dict(seed=4, W=2, E=4, K=3, H=8, tokens=[6, 6], dup=True),
    dict(seed=5, W=4, E=8, K=8, H=8, tokens=[2, 3, 0, 4]),
]


@pytest.mark.parametrize("spec", WORLDS, ids=lambda s: f"seed{s['seed']}")
@pytest.mark.parametrize("stub_kind", [0, 1])
def test_literal_and_vectorised_forms_agree(spec, stub_kind):
    cfg, world = random_world(**spec)
    disp = L.dispatch_world(cfg, world)
    counts, offsets, dx, meta = L.compact_from_dispatched(cfg, disp)
    ey = L.stub_world(cfg, disp, stub_kind)
    ys = L.combine_world(cfg, world, disp, ey)
    o = V.run_world(cfg, world, stub_kind=stub_kind)
    assert torch.equal(o["counts"], counts) and torch.equal(o["offsets"], offsets)
    assert torch.equal(o["meta"], meta)
    assert torch.equal(bits(o["disp_x"]), bits(dx))
    assert torch.equal(bits(o["expert_y"]), bits(torch.cat([torch.cat(r, 0) for r in ey], 0)))
    st = o["starts"]
    for r, rd in enumerate(world):
        assert torch.equal(bits(o["y"][st[r]:st[r + 1]]), bits(ys[r][: rd.num_tokens]))


@pytest.mark.parametrize("spec", WORLDS, ids=lambda s: f"seed{s['seed']}")
def test_route_against_brute_force(spec):
    cfg, world = random_world(**spec)
    x, idx, w, starts = V.concat_world(world)
    r = V.route(idx, starts, cfg.num_experts)
    flat = idx.flatten().tolist()
    R, K = len(flat), cfg.experts_per_token
    for i, e in enumerate(flat):  # slot = rows of smaller experts + earlier rows of the same expert
        want = sum(1 for f in flat if f < e) + sum(1 for j in range(i) if flat[j] == e)
        assert int(r["slot_of_entry"][i]) == want
    assert sorted(r["slot_of_entry"].tolist()) == list(range(R))
    assert torch.equal(r["src_of_slot"][r["slot_of_entry"].long()], torch.arange(R, dtype=torch.int32))
    assert int(r["counts"].sum()) == R and int(r["offsets"][-1]) == R
    meta = r["meta"]
    for e in range(cfg.num_experts):
        seg = meta[int(r["offsets"][e]):int(r["offsets"][e + 1])]
        assert bool((seg[:, 0] == e).all()) and bool((seg[:, 4] == 0).all())
        keys = [(int(m[1]), int(m[2]), int(m[3])) for m in seg]
        assert keys == sorted(keys)  # arrival order: source rank, token, k
    for slot in range(R):  # meta names the entry that lives in the slot
        e, sr, tl, k, _ = meta[slot].tolist()
        i = int(r["src_of_slot"][slot])
        assert flat[i] == e and i % K == k and i // K == starts[sr] + tl and tl < world[sr].num_tokens


def test_dispatch_is_a_pure_row_copy():
    cfg, world = random_world(seed=7, W=4, E=16, K=4, H=24, tokens=[5, 0, 7, 2])
    o = V.run_world(cfg, world)
    x, idx, w, starts = V.concat_world(world)
    tok = o["src_of_slot"].long() // cfg.experts_per_token
    assert torch.equal(bits(o["disp_x"]), bits(x)[tok])


def test_combine_one_hot_weights_returns_the_token():
    cfg, world = random_world(seed=8, W=1, E=8, K=4, H=40, tokens=[11])  # W=1: stub factor is 1
    rd = world[0]
    hot = torch.randint(0, 4, (11,), generator=torch.Generator().manual_seed(0))
    rd.weights = torch.nn.functional.one_hot(hot, 4).float()
    for mode in (0, 1):
        y = V.run_world(cfg, world, stub_kind=0, combine_mode=mode)["y"]
        assert torch.equal(y.float(), rd.x.float())
    ys = L.ref_kernel_world(cfg, world, 0)
    assert torch.equal(ys[0].float(), rd.x.float())


def test_combine_top1_is_the_stub_and_zero_weights_give_zero():
    cfg, world = random_world(seed=9, W=4, E=8, K=1, H=16, tokens=[3, 2, 4, 1])
    for rd in world:
        rd.weights = torch.ones_like(rd.weights)
    o = V.run_world(cfg, world, stub_kind=0)
    x, idx, w, starts = V.concat_world(world)
    owner = (idx[:, 0] // 2).float().unsqueeze(1)
    assert torch.equal(o["y"].float(), (x.float() * (1 + owner)).to(torch.bfloat16).float())
    for rd in world:
        rd.weights = torch.zeros_like(rd.weights)
    assert float(V.run_world(cfg, world)["y"].float().abs().max()) == 0.0


@pytest.mark.parametrize("stub_kind", [0, 1])
def test_closed_form_per_rank(stub_kind):
    cfg, world = random_world(seed=10, W=8, E=64, K=6, H=32, tokens=[4, 2, 7, 1, 3, 5, 2, 6])
    o = V.run_world(cfg, world, stub_kind=stub_kind)
    st = o["starts"]
    for r, rd in enumerate(world):
        assert torch.equal(bits(V.closed_form(cfg, rd, stub_kind, 8)), bits(o["y"][st[r]:st[r + 1]]))
        # ref_kernel of the contract: one rank alone gives the same rows
        y1 = checker.ref_kernel((cfg, rd, r, 8), stub_kind=stub_kind)
        assert torch.equal(bits(y1), bits(o["y"][st[r]:st[r + 1]]))


def test_f32_mode_is_close_to_exact_arithmetic():
    wl = C.generate_workload("dsv3_rank", tokens_scale=1 / 8)
    o = V.run_world(wl.cfg, wl.world, stub_kind=1, combine_mode=1)
    x, idx, w, starts = V.concat_world(wl.world)
    s = ((1 + idx.double()) / wl.cfg.num_experts)
    exact = (x.double().unsqueeze(1) * s.unsqueeze(-1) * w.double().unsqueeze(-1)).sum(1)
    err = (o["y"].double() - exact).abs()
    assert float((err / (exact.abs() + 1e-2)).max()) < 2.0 ** -6  # a few bf16 roundings
    strict = V.run_world(wl.cfg, wl.world, stub_kind=1, combine_mode=0)["y"]
    assert torch.allclose(strict.float(), o["y"].float(), rtol=1e-2, atol=1e-2)


# ---- fp8 ------------------------------------------------------------------------------------
def e4m3fn_table():
    """All finite e4m3fn values by bit pattern: 1 sign, 4 exponent (bias 7), 3 mantissa bits."""
    vals = np.zeros(256, dtype=np.float64)
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            vals[b] = np.nan
        elif e == 0:
            vals[b] = (m / 8.0) * 2.0 ** -6
        else:
            vals[b] = (1 + m / 8.0) * 2.0 ** (e - 7)
        if s:
            vals[b] = -vals[b]
    return vals


def encode_e4m3fn_nearest_even(x: np.ndarray) -> np.ndarray:
    """Nearest representable value, ties to the even bit pattern; inputs within +-448."""
    tab = e4m3fn_table()
    pos = tab[:127]  # 0x00..0x7e ascending magnitudes
    mag = np.abs(x.astype(np.float64))
    hi = np.searchsorted(pos, mag, side="left").clip(1, 126)
    lo = hi - 1
    dlo, dhi = mag - pos[lo], pos[hi] - mag
    pick = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    return (pick | np.where(np.signbit(x), 0x80, 0)).astype(np.uint8)


def test_fp8_cast_against_independent_encoder():
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(4096, generator=g) * 100, torch.randn(4096, generator=g),
                   torch.randn(4096, generator=g) * 1e-2, torch.tensor([0.0, -0.0, 448.0, -448.0, 2.0 ** -9,
                                                                        2.0 ** -10, 3 * 2.0 ** -10, 464.0 - 1e-3])])
    x = x.clamp(-448, 448)
    got = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    want = encode_e4m3fn_nearest_even(x.numpy())
    assert np.array_equal(got, want)


def test_fp8_quantisation_definition_and_bound():
    wl = C.generate_workload("fp8_dispatch", tokens_scale=32 / 4096)
    x = wl.world[0].x
    q, scale = V.quantize_fp8(x)
    T, H = x.shape
    xf = x.float().view(T, H // 128, 128)
    assert torch.equal(scale, xf.abs().amax(-1) / 448.0)
    ratio = (xf / scale.unsqueeze(-1)).numpy()
    assert np.array_equal(q.view(T, H // 128, 128).numpy(), encode_e4m3fn_nearest_even(ratio))
    deq = V.dequantize_fp8(q, scale).view(T, H // 128, 128)
    bound = torch.maximum(xf.abs() * 2.0 ** -4, scale.unsqueeze(-1) * 2.0 ** -10) * (1 + 1e-6)
    assert bool(((deq - xf).abs() <= bound).all())
    z = torch.zeros(2, 128, dtype=torch.bfloat16)  # all-zero block: scale 1, q 0
    qz, sz = V.quantize_fp8(z)
    assert float(sz.min()) == 1.0 and int(qz.max()) == 0


def test_fp8_power_of_two_scales():
    """Scale mode 2: the scale is the least power of two >= amax / 448 (so nothing saturates and at
    most one bit of the e4m3 range is given up), the cast is the same, the error bound holds with
    the block's own scale."""
    wl = C.generate_workload("fp8_dispatch", tokens_scale=32 / 4096)
    x = wl.world[0].x
    q, scale = V.quantize_fp8(x, pow2=True)
    T, H = x.shape
    xf = x.float().view(T, H // 128, 128)
    exact = xf.abs().amax(-1) / 448.0
    mant, _ = torch.frexp(scale)
    assert bool((mant == 0.5).all())                       # a power of two
    assert bool((scale >= exact).all()) and bool((scale < 2 * exact).all())
    ratio = (xf / scale.unsqueeze(-1)).numpy()
    assert float(np.abs(ratio).max()) <= 448.0
    assert np.array_equal(q.view(T, H // 128, 128).numpy(), encode_e4m3fn_nearest_even(ratio))
    deq = V.dequantize_fp8(q, scale).view(T, H // 128, 128)
    bound = torch.maximum(xf.abs() * 2.0 ** -4, scale.unsqueeze(-1) * 2.0 ** -10) * (1 + 1e-6)
    assert bool(((deq - xf).abs() <= bound).all())
    # closed cases of the rounding: powers of two stay, anything above moves up, the ends clamp
    s = torch.tensor([1.0, 1.0 + 2.0 ** -23, 1.5, 2.0 ** -126, 1e-40, 3e38], dtype=torch.float32)
    assert V.pow2_at_or_above(s).tolist() == [1.0, 2.0, 2.0, 2.0 ** -126, 2.0 ** -126, 2.0 ** 127]
    wq, ws = V.quantize_weights_fp8(torch.randn(2, 128, 256), pow2=True)
    assert bool((torch.frexp(ws)[0] == 0.5).all())


def test_fp8_path_output_within_tolerance_of_bf16_path():
    wl = C.generate_workload("fp8_dispatch", tokens_scale=64 / 4096)
    a = V.run_world(wl.cfg, wl.world, stub_kind=1, fp8=True)["y"].float()
    b = V.run_world(wl.cfg, wl.world, stub_kind=1, fp8=False)["y"].float()
    assert float((a - b).abs().max()) < 2.0 ** -4 * float(b.abs().max())


# ---- expert GEMM helpers (no counterpart in the reference: pinned by explicit loops) -----------
def test_weight_quantisation_and_q8_gemm_against_explicit_loops():
    """quantize_weights_fp8 / dequantize_weights_fp8 / expert_gemm_q8 on 2 x 128 x 128 integer-valued
    weights, against plain Python loops over blocks and the independent e4m3fn encoder: the block
    scale is amax / 448, the bits are the nearest-even e4m3fn code of w / scale, dequantisation is
    code value x scale, and the product is the sum over K of x x dequantised weight, rounded once."""
    g = torch.Generator().manual_seed(21)
    E, N, Kd = 2, 128, 256  # one block row, two K blocks per expert
    w = torch.randint(-40, 41, (E, N, Kd), generator=g).to(torch.float32)
    w[1, :, 128:] = 0.0  # an all-zero block: scale 1, codes 0
    q, s = V.quantize_weights_fp8(w)
    assert q.dtype == torch.uint8 and tuple(q.shape) == (E, N, Kd) and tuple(s.shape) == (E, 1, 2)
    tab = e4m3fn_table()
    deq_loop = np.zeros((E, N, Kd), dtype=np.float64)
    for e in range(E):
        for kb in range(2):
            blk = w[e, :, 128 * kb:128 * (kb + 1)].numpy()
            amax = np.float32(np.abs(blk).max())
            scale = np.float32(1.0) if amax == 0 else np.float32(amax / np.float32(448.0))
            assert np.float32(s[e, 0, kb]) == scale
            codes = encode_e4m3fn_nearest_even((blk / scale).astype(np.float32))
            assert np.array_equal(q[e, :, 128 * kb:128 * (kb + 1)].numpy(), codes)
            deq_loop[e, :, 128 * kb:128 * (kb + 1)] = tab[codes].astype(np.float32) * scale
    deq = V.dequantize_weights_fp8(q, s)
    assert np.array_equal(deq.numpy(), deq_loop.astype(np.float32))
    # integer-valued rows keep every partial sum exact in f32, so the loop below has ONE right answer
    x = torch.randint(-3, 4, (6, Kd), generator=g).to(torch.bfloat16)
    offsets = torch.tensor([0, 4, 6], dtype=torch.int32)
    y = V.expert_gemm_q8(x, None, q, s, offsets, torch.float32)
    for r in range(6):
        e = 0 if r < 4 else 1
        for n in range(0, N, 17):
            acc = 0.0
            for k in range(Kd):
                acc += float(x[r, k]) * float(deq_loop[e, n, k])
            assert abs(float(y[r, n]) - acc) <= 1e-4 * max(1.0, abs(acc)), (r, n)
    # fp8 rows: dequantised with their own scales; round_rows rounds them once to the output type first
    xq, xs = V.quantize_fp8(x)
    xd = V.dequantize_fp8(xq, xs)
    for round_rows in (False, True):
        y8 = V.expert_gemm_q8(xq, xs, q, s, offsets, torch.bfloat16, round_rows=round_rows)
        rows = xd.to(torch.bfloat16).float() if round_rows else xd
        for r in (0, 5):
            e = 0 if r < 4 else 1
            want = (rows[r].double() @ torch.from_numpy(deq_loop[e]).t()).to(torch.float32).to(torch.bfloat16)
            assert torch.equal(bits(y8[r]), bits(want)), (round_rows, r)


def test_stub_factor_f32_division_equals_the_double_quotient_rounded_to_f32():
    """The kernels divide (1 + e) by E in f32 (correctly rounded); the oracle divides in double and
    rounds to f32.  Equal for every expert count the library accepts."""
    for E in range(1, 1025):
        e = np.arange(E, dtype=np.int64)
        via_double = ((1 + e).astype(np.float64) / np.float64(E)).astype(np.float32)
        via_f32 = (1 + e).astype(np.float32) / np.float32(E)
        assert np.array_equal(via_double, via_f32), E
