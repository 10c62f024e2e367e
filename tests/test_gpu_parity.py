"""HIP path against the CPU oracle, through the C ABI, on seeded inputs.  Needs a GPU.

Bar: counts, offsets, permutations, meta, dispatched rows, stub rows and the combine output
are compared BIT FOR BIT (both combine modes follow a stated operation order, so they are
exact too); fp8 rows are compared bit for bit against torch's e4m3fn cast.
"""
import pytest
import torch

from golden_io import GOLDEN_CASES, bits, golden_compact, load_golden
from kernel_amd import _lib, contract as C
from kernel_amd.all2all import HipAllToAll, concat_world
from oracle import all2all_vec as V

pytestmark = pytest.mark.gpu


def run_hip(cfg, world, dev, stub_kind, combine_mode=0, fp8=False, fuse_route=True, rank=0):
    W = len(world)
    x, idx, w, rs = concat_world(world, dev)
    ata = HipAllToAll(cfg, rank, W, stub_kind=stub_kind, combine_mode=combine_mode, fp8_dispatch=fp8,
                      fuse_route=fuse_route)
    d = ata.dispatch(x, idx, rs)
    ey = ata.expert_stub(d)
    y = ata.combine(None, w, d, ey)
    y2 = ata.stub_combine(torch.empty_like(y), w, idx, d)
    torch.cuda.synchronize()
    return d, ey, y, y2


def assert_same(name, got, want):
    got = got.cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert got.dtype == want.dtype, f"{name}: dtype {got.dtype} != {want.dtype}"
    g, w = bits(got), bits(want)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        raise AssertionError(f"{name}: {bad.shape[0]} mismatches, first at {bad[0].tolist()}: "
                             f"{got[tuple(bad[0])]} != {want[tuple(bad[0])]}")


def compare(cfg, world, dev, stub_kind, combine_mode=0, fp8=False, fuse_route=True):
    o = V.run_world(cfg, world, stub_kind=stub_kind, fp8=bool(fp8), combine_mode=combine_mode, pow2=fp8 == "pow2")
    d, ey, y, y2 = run_hip(cfg, world, dev, stub_kind, combine_mode, fp8, fuse_route)
    assert int(d.status.item()) == 0
    assert_same("counts", d.counts, o["counts"])
    assert_same("offsets", d.offsets, o["offsets"])
    assert_same("slot_of_entry", d.slot_of_entry, o["slot_of_entry"])
    assert_same("src_of_slot", d.src_of_slot, o["src_of_slot"])
    assert_same("meta", d.meta, o["meta"])
    assert_same("disp_x", d.disp_x, o["disp_x"])
    if fp8:
        assert_same("disp_scale", d.disp_scale, o["disp_scale"])
    assert_same("expert_y", ey, o["expert_y"])
    assert_same("y", y, o["y"])
    assert_same("y (stub folded into combine)", y2, o["y"])
    return o, d


@pytest.mark.parametrize("name", GOLDEN_CASES)
@pytest.mark.parametrize("fuse_route", ["always", False])
def test_reference_vectors(gpu_device, name, fuse_route):
    """Against the outputs the reference's own PyTorchAllToAll wrote (tests/golden/)."""
    cfg, world, expected = load_golden(name)
    g = golden_compact(cfg, expected)
    d, ey, y, y2 = run_hip(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=fuse_route)
    assert_same("counts", d.counts, g["counts"])
    assert_same("meta", d.meta, g["meta"])
    assert_same("disp_x", d.disp_x, g["disp_x"])
    assert_same("expert_y", ey, g["expert_y"])
    assert_same("y", y, g["y"])
    assert_same("y2", y2, g["y"])
    # the reference's own return value of dispatch for every owner rank
    for r, exp in enumerate(expected):
        num, ex, em = d.padded(r)
        assert_same("expert_num_tokens", num, exp.expert_num_tokens)
        rows = torch.cat([ex[le, : int(num[le])] for le in range(num.numel())], 0)
        assert_same("expert_x", rows, exp.expert_x)


@pytest.mark.parametrize("spec", C.REFERENCE_TESTS, ids=lambda s: f"E{s['num_experts']}K{s['experts_per_token']}"
                                                                     f"H{s['hidden_dim']}T{s['max_num_tokens']}")
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_reference_specs_whole_world(gpu_device, spec, dtype):
    """The reference's 9 test specs (all2all/task.yml:59-68), all 8 ranks resident at once."""
    cfg, world = C.generate_world(**spec, dtype=dtype)
    for fuse in ("always", True, False):
        compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=fuse)


@pytest.mark.parametrize("name,scale", [("tiny", 1.0), ("dsv3_rank", 1.0), ("skew_world", 1.0)])
@pytest.mark.parametrize("mode", [C.COMBINE_STRICT, C.COMBINE_F32], ids=["strict", "f32"])
def test_named_workloads(gpu_device, name, scale, mode):
    wl = C.generate_workload(name, tokens_scale=scale)
    for fuse in ("always", True, False):
        o, d = compare(wl.cfg, wl.world, gpu_device, wl.stub_kind, combine_mode=mode, fuse_route=fuse)
    if name == "skew_world":
        assert int(o["counts"].max()) <= wl.total_tokens  # one row per token and expert at most


def test_multi_workgroup_routing(gpu_device):
    """R = 40960: histogram launch + rank launch, 8 source ranks."""
    wl = C.generate_workload("prefill_graph", tokens_scale=10240 / 16384)
    cfg = wl.cfg
    # spread the tokens over 8 uneven source ranks
    x, idx, w = wl.world[0].x, wl.world[0].indices, wl.world[0].weights
    cuts = [0, 7, 7, 3000, 3001, 6000, 9000, 10239, 10240]
    world = [C.RankData(cuts[i + 1] - cuts[i], idx[cuts[i]:cuts[i + 1]], w[cuts[i]:cuts[i + 1]],
                        x[cuts[i]:cuts[i + 1]]) for i in range(8)]
    compare(cfg, world, gpu_device, C.STUB_EXPERT_FRACTION)


@pytest.mark.parametrize("name,scale", [("tiny", 1.0), ("dsv3_rank", 1.0), ("skew_world", 1.0), ("prefill_graph", 1 / 16)])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
def test_token_tile_kernel_on_every_size(gpu_device, options, name, scale, padded):
    """The one-launch routing + dispatch with a tile of tokens per workgroup, forced for shapes the
    library would give to the one-token kernel or to separate launches: same bits everywhere."""
    options.set("ROUTE_TILE", 1)
    wl = C.generate_workload(name, tokens_scale=scale)
    cfg = wl.cfg
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    T = x.shape[0]
    ata = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind, fuse_route="always", padded=padded,
                      max_recv=T if padded else None)
    lib = ata.lib
    import ctypes
    assert lib.moe_a2a_timer_begin(8) == 0
    d = ata.dispatch(x, idx, rs)
    torch.cuda.synchronize()
    ids, us = (ctypes.c_int * 8)(), (ctypes.c_float * 8)()
    assert lib.moe_a2a_timer_end(ids, us, 8) == 1
    assert lib.moe_a2a_kernel_name(ids[0]) == b"route_dispatch_tile"
    o = V.run_world(cfg, wl.world, stub_kind=wl.stub_kind)
    assert int(d.status.item()) == 0
    assert_same("counts", d.counts, o["counts"])
    assert_same("offsets", d.offsets, o["offsets"])
    soe = o["slot_of_entry"].long()
    if padded:
        e = o["meta"][:, 0].long()
        want_rows = e * T + (torch.arange(soe.numel()) - o["offsets"].long()[e])  # row of compact slot s
        assert_same("slot_of_entry", d.slot_of_entry, want_rows[soe].to(torch.int32))
        rows = d.slot_of_entry.long()
        assert_same("meta", d.meta[rows], o["meta"][soe])
        assert_same("disp_x", d.disp_x[rows], o["disp_x"][soe])
    else:
        assert_same("slot_of_entry", d.slot_of_entry, o["slot_of_entry"])
        assert_same("src_of_slot", d.src_of_slot, o["src_of_slot"])
        assert_same("meta", d.meta, o["meta"])
        assert_same("disp_x", d.disp_x, o["disp_x"])
    y = ata.combine(None, w, d, ata.expert_stub(d))
    assert_same("y", y, o["y"])


def test_launch_timer_skips_the_launches_it_is_told_to(gpu_device):
    """Launches skipped by moe_a2a_timer_skip go out without events: they are not reported, the
    ones after them are, and every result is what it would be without the timer."""
    import ctypes
    wl = C.generate_workload("dsv3_rank", tokens_scale=0.25)
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind)
    lib = ata.lib
    o = V.run_world(wl.cfg, wl.world, stub_kind=wl.stub_kind)
    assert lib.moe_a2a_timer_begin(16) == 0
    assert lib.moe_a2a_timer_skip(-1) != 0
    assert lib.moe_a2a_timer_skip(3) == 0  # one forward: route_dispatch, stub, combine
    y1 = ata.forward(x, idx, w, rs).clone()
    y2 = ata.forward(x, idx, w, rs).clone()
    torch.cuda.synchronize()
    ids, us = (ctypes.c_int * 16)(), (ctypes.c_float * 16)()
    assert lib.moe_a2a_timer_end(ids, us, 16) == 3
    assert [lib.moe_a2a_kernel_name(ids[i]) for i in range(3)] == [b"route_dispatch", b"stub_rows", b"combine_rows"]
    assert all(0.5 < us[i] < 1000 for i in range(3))
    assert_same("y (skipped)", y1, o["y"])
    assert_same("y (timed)", y2, o["y"])


@pytest.mark.parametrize("T,K", [(1001, 3), (2731, 6), (10921, 3), (16383, 3)])
def test_routing_table_not_a_multiple_of_four(gpu_device, T, K):
    """The one-launch routing reads the table four entries at a time: R % 4 = 3, 2, 3 (the largest
    table it takes) and 1 (two launches), separate routing and the fused forms."""
    g = torch.Generator().manual_seed(T)
    E, H = 64, 64
    cfg = C.MoEConfig(E, K, H, T + 1, torch.bfloat16, torch.bfloat16)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    cuts = [0, T // 3, T // 3, T - 5, T]
    world = [C.RankData(cuts[i + 1] - cuts[i], idx[cuts[i]:cuts[i + 1]], torch.rand(cuts[i + 1] - cuts[i], K, generator=g),
                        torch.randn(cuts[i + 1] - cuts[i], H, generator=g).to(torch.bfloat16)) for i in range(4)]
    for fuse in (False, True):
        compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=fuse)


@pytest.mark.parametrize("T", [12000, 33000])
def test_huge_routing_table(gpu_device, T):
    """R = 96000 routed rows: histogram launch + rank launch that scans the tile counts itself;
    R = 264000: more tiles than the rank kernel sums by itself, so the column-scan kernel runs too."""
    g = torch.Generator().manual_seed(9)
    K, E, H = 8, 32, 64
    cfg = C.MoEConfig(E, K, H, T + 1, torch.float16, torch.float16)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    world = [C.RankData(T, idx, torch.rand(T, K, generator=g), torch.randn(T, H, generator=g).to(torch.float16))]
    world += [C.RankData.empty(cfg) for _ in range(7)]
    compare(cfg, world, gpu_device, C.STUB_OWNER_RANK)


def test_fp8_dispatch(gpu_device):
    wl = C.generate_workload("fp8_dispatch", tokens_scale=512 / 4096)
    compare(wl.cfg, wl.world, gpu_device, wl.stub_kind, fp8=True)
    compare(wl.cfg, wl.world, gpu_device, wl.stub_kind, fp8=True, combine_mode=C.COMBINE_F32)


def test_fp8_dispatch_power_of_two_scales(gpu_device):
    """The same path with scales rounded up to powers of two: bytes, scales and every later step
    bit for bit, through the separate calls and through the one-call forward."""
    wl = C.generate_workload("fp8_dispatch", tokens_scale=512 / 4096)
    o, d = compare(wl.cfg, wl.world, gpu_device, wl.stub_kind, fp8="pow2")
    assert bool((torch.frexp(d.disp_scale.cpu())[0] == 0.5).all())
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    ata = HipAllToAll(wl.cfg, 0, len(wl.world), stub_kind=wl.stub_kind, fp8_dispatch="pow2")
    y = ata.forward(x, idx, w, rs)
    torch.cuda.synchronize()
    assert_same("y (forward)", y, o["y"])


@pytest.mark.parametrize("H,T,K,E", [(128, 37, 2, 8), (384, 300, 3, 16), (8320, 64, 4, 32), (16384, 33, 8, 64),
                                     (2048, 1500, 6, 64)])
@pytest.mark.parametrize("fp8", [True, "pow2"], ids=["f32scales", "pow2scales"])
def test_fp8_dispatch_row_lengths(gpu_device, H, T, K, E, fp8):
    """fp8 dispatch on rows of one block, of a few blocks, of more blocks than one workgroup holds
    (65 and 128: the row is cut in two, each part writes its own scales) and on a table that takes the
    multi-workgroup routing; ragged world of four ranks."""
    g = torch.Generator().manual_seed(H + T)
    cfg = C.MoEConfig(E, K, H, T + 1, torch.bfloat16, torch.bfloat16)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    x = (torch.randn(T, H, generator=g) * torch.rand(T, 1, generator=g) * 8).to(torch.bfloat16)
    x[::7, : H // 2] = 0  # whole blocks of zeros: scale 1
    cuts = [0, T // 4, T // 4, T - 1, T]
    world = [C.RankData(cuts[i + 1] - cuts[i], idx[cuts[i]:cuts[i + 1]], torch.rand(cuts[i + 1] - cuts[i], K, generator=g),
                        x[cuts[i]:cuts[i + 1]]) for i in range(4)]
    compare(cfg, world, gpu_device, C.STUB_EXPERT_FRACTION, fp8=fp8)
    compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fp8=fp8, combine_mode=C.COMBINE_F32, fuse_route=False)


def test_duplicate_experts_and_ragged_world(gpu_device):
    """A token may name the same expert twice; ranks may be empty; H not a multiple of 256 lanes."""
    g = torch.Generator().manual_seed(5)
    cfg = C.MoEConfig(16, 4, 2880, 9, torch.bfloat16, torch.bfloat16)
    world = []
    for n in [3, 0, 8, 1]:
        world.append(C.RankData(n, torch.randint(0, 16, (n, 4), generator=g).to(torch.int32),
                                torch.rand(n, 4, generator=g), torch.randn(n, 2880, generator=g).to(torch.bfloat16)))
    for fuse in ("always", True, False):
        compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=fuse)


@pytest.mark.parametrize("E,K,T,H", [(1024, 3, 300, 128), (64, 32, 40, 256), (8, 1, 17, 64), (48, 5, 700, 1032)])
def test_limits_and_generic_topk(gpu_device, E, K, T, H):
    """Largest expert count (LDS beyond 64 KB), largest top-k, K without a specialised kernel,
    H that is not a multiple of 64 lanes."""
    g = torch.Generator().manual_seed(E + K)
    cfg = C.MoEConfig(E, K, H, T + 1, torch.bfloat16, torch.bfloat16)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    world = [C.RankData.empty(cfg) for _ in range(8)]
    world[3] = C.RankData(T, idx, torch.rand(T, K, generator=g), torch.randn(T, H, generator=g).to(torch.bfloat16))
    for fuse in ("always", False):
        for mode in (C.COMBINE_STRICT, C.COMBINE_F32):
            compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, combine_mode=mode, fuse_route=fuse)


def _random_shapes(n, seed):
    """Seeded sweep of routing shapes around the limits that pick a kernel: entries per thread of the
    one-token kernel (4..32), its table-read budget, tile sizes of the token-tile kernel, one
    workgroup vs. several routing tiles, ragged worlds, duplicate-free and duplicated expert ids."""
    g = torch.Generator().manual_seed(seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    out = []
    for _ in range(n):
        W = pick([1, 2, 4, 8])
        E = W * pick([1, 2, 3, 8, 16, 32])
        K = pick([1, 2, 3, 4, 6, 8, 12])
        H = 8 * pick([1, 3, 8, 32, 96, 129, 256, 512])
        T = pick([1, 2, 5, 31, 64, 129, 300, 777, 1500, 2500])
        out.append((W, E, K, H, T, bool(pick([0, 0, 1])), int(torch.randint(0, 1 << 30, (1,), generator=g))))
    return out


@pytest.mark.parametrize("W,E,K,H,T,dup,seed", _random_shapes(24, 2024))
def test_random_shapes_all_routing_kernels(gpu_device, options, W, E, K, H, T, dup, seed):
    """Every routing implementation (one-token, token-tile, separate launches) on the same random
    world, compact and through the library's own choice: all bit-identical to the oracle."""
    g = torch.Generator().manual_seed(seed)
    K = min(K, E) if not dup else K
    cfg = C.MoEConfig(E, K, H, T + 1, torch.bfloat16, torch.bfloat16)
    cuts = sorted(int(v) for v in torch.randint(0, T + 1, (W - 1,), generator=g)) if W > 1 else []
    cuts = [0] + cuts + [T]
    world = []
    for r in range(W):
        n = cuts[r + 1] - cuts[r]
        if dup:
            idx = torch.randint(0, E, (n, K), generator=g).to(torch.int32)
        else:
            idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32) if n else \
                torch.empty(0, K, dtype=torch.int32)
        world.append(C.RankData(n, idx, torch.rand(n, K, generator=g), torch.randn(n, H, generator=g).to(torch.bfloat16)))
    options.set("ROUTE_TILE", 0)
    compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=True)       # the library's choice
    compare(cfg, world, gpu_device, C.STUB_EXPERT_FRACTION, fuse_route=False)  # separate launches
    options.set("ROUTE_TILE", 1)
    compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route="always")   # token tiles
    options.set("ROUTE_TILE", 0)
    compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route="always")   # one-token kernel when it applies


@pytest.mark.parametrize("name", ["tiny", "dsv3_rank", "skew_world"])
def test_forward_single_call_equals_separate_calls(gpu_device, name):
    wl = C.generate_workload(name)
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    want = V.run_world(wl.cfg, wl.world, stub_kind=wl.stub_kind)
    for fuse_route in ("always", True, False):
        for fuse_stub in (False, True):
            ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, fuse_route=fuse_route,
                              fuse_stub=fuse_stub)
            for _ in range(3):  # both buffer sets, and the first one again
                y = ata.forward(x, idx, w, rs)
                assert_same("y", y, want["y"])
                assert_same("meta", ata.last.meta, want["meta"])
                assert_same("disp_x", ata.last.disp_x, want["disp_x"])
            step = ata.plan(x, idx, w, rs)
            for _ in range(3):
                assert_same("y (planned)", step(), want["y"])
                assert_same("slot_of_entry (planned)", ata.last.slot_of_entry, want["slot_of_entry"])


@pytest.mark.parametrize("W,E,K,H,tokens", [
    (1, 8, 2, 256, [64]),                        # tiny: K without a specialised fold
    (8, 256, 8, 7168, [256, 0, 0, 0, 0, 0, 0, 0]),  # headline shape: one token per workgroup
    (2, 16, 3, 2880, [100, 37]),                 # rows of 360 vectors (not whole waves), odd K
    (8, 64, 6, 2048, [128] * 8),                 # a tile of tokens per workgroup
    (4, 32, 4, 4096, [700, 0, 123, 9]),          # ragged ranks, tiles
    (1, 4, 1, 64, [5]),                          # K = 1
    (2, 64, 32, 512, [40, 41]),                  # K = 32: every lane group of the fold is used
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("mode", [C.COMBINE_STRICT, C.COMBINE_F32], ids=["strict", "f32"])
def test_one_launch_forward_equals_the_oracle_and_the_two_launch_form(gpu_device, options, W, E, K, H, tokens,
                                                                      dtype, mode):
    """forward with the stub folded in runs in ONE launch for these shapes (a workgroup dispatches
    its tokens and then folds the rows it wrote): the dispatched buffers and the output are bit for
    bit those of the oracle and of the two-launch form of the same call."""
    g = torch.Generator().manual_seed(sum(tokens) + E + K)
    cfg = C.MoEConfig(E, K, H, max(tokens) + 1, dtype, dtype)
    world = []
    for n in tokens:
        idx = (torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32) if n
               else torch.empty(0, K, dtype=torch.int32))
        world.append(C.RankData(n, idx, torch.rand(n, K, generator=g), torch.randn(n, H, generator=g).to(dtype)))
    x, idx, w, rs = concat_world(world, gpu_device)
    T = x.shape[0]
    lib = _lib.load()
    assert lib.moe_a2a_forward_launches(T, K, H, 0, _lib.BF16, _lib.BF16, 0, 1, 1) == 1
    for stub_kind in (C.STUB_OWNER_RANK, C.STUB_EXPERT_FRACTION):
        want = V.run_world(cfg, world, stub_kind=stub_kind, combine_mode=mode)
        got = {}
        for two in (0, 1):
            options.set("TWO_LAUNCHES", two)
            ata = HipAllToAll(cfg, 0, W, stub_kind=stub_kind, combine_mode=mode, fuse_stub=True)
            for _ in range(2):
                y = ata.forward(x, idx, w, rs)
            torch.cuda.synchronize()
            d = ata.last
            assert int(d.status.item()) == 0
            for key, val in (("counts", d.counts), ("offsets", d.offsets), ("slot_of_entry", d.slot_of_entry),
                             ("src_of_slot", d.src_of_slot), ("meta", d.meta), ("disp_x", d.disp_x), ("y", y)):
                assert_same(f"{key} ({'two launches' if two else 'one launch'})", val, want[key])
            got[two] = y.clone()
        assert torch.equal(bits(got[0]), bits(got[1]))
    # the launch timer names the kernel that ran
    options.set("TWO_LAUNCHES", 0)
    ata = HipAllToAll(cfg, 0, W, combine_mode=mode, fuse_stub=True)
    ata.forward(x, idx, w, rs)
    torch.cuda.synchronize()
    import ctypes
    assert lib.moe_a2a_timer_begin(4) == 0
    ata.forward(x, idx, w, rs)
    ids, us = (ctypes.c_int * 4)(), (ctypes.c_float * 4)()
    assert lib.moe_a2a_timer_end(ids, us, 4) == 1
    assert lib.moe_a2a_kernel_name(ids[0]) in (b"forward_token", b"forward_tile")


@pytest.mark.parametrize("W,E,K,H,tokens", [
    (1, 8, 2, 256, [64]),
    (8, 256, 8, 7168, [40, 0, 3, 0, 17, 0, 0, 1]),
    (2, 16, 3, 384, [100, 37]),          # three 128-column blocks, K without a specialised fold
    (4, 32, 4, 4096, [300, 0, 123, 9]),
])
@pytest.mark.parametrize("fp8", [True, "pow2"], ids=["f32scales", "pow2scales"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("mode", [C.COMBINE_STRICT, C.COMBINE_F32], ids=["strict", "f32"])
def test_forward_with_fp8_dispatch_and_folded_stub(gpu_device, options, W, E, K, H, tokens, fp8, dtype, mode):
    """forward with an fp8 dispatch and the stub folded in quantises, stores and folds a token in one
    kernel behind the routing launch: rows, scales and output bit for bit those of the oracle and of
    the separate dispatch_fp8 + stub_combine launches."""
    g = torch.Generator().manual_seed(sum(tokens) + E + K)
    cfg = C.MoEConfig(E, K, H, max(tokens) + 1, dtype, dtype)
    world = []
    for n in tokens:
        idx = (torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32) if n
               else torch.empty(0, K, dtype=torch.int32))
        world.append(C.RankData(n, idx, torch.rand(n, K, generator=g), torch.randn(n, H, generator=g).to(dtype)))
    x, idx, w, rs = concat_world(world, gpu_device)
    want = V.run_world(cfg, world, stub_kind=C.STUB_EXPERT_FRACTION, fp8=True, combine_mode=mode, pow2=fp8 == "pow2")
    for two in (1, 0):
        options.set("TWO_LAUNCHES", two)  # 1: routing, dispatch_fp8 and stub_combine as separate launches
        ata = HipAllToAll(cfg, 0, W, stub_kind=C.STUB_EXPERT_FRACTION, combine_mode=mode, fp8_dispatch=fp8,
                          fuse_stub=True)
        for _ in range(2):
            y = ata.forward(x, idx, w, rs)
        torch.cuda.synchronize()
        d = ata.last
        for key, val in (("counts", d.counts), ("slot_of_entry", d.slot_of_entry), ("meta", d.meta),
                         ("disp_x", d.disp_x), ("disp_scale", d.disp_scale), ("y", y)):
            assert_same(f"{key} ({'separate launches' if two else 'one kernel'})", val, want[key])


@pytest.mark.parametrize("W,E,K,H,tokens", [
    (1, 8, 2, 128, [1]),                              # one token, one block
    (8, 256, 8, 7168, [40, 0, 3, 0, 17, 0, 0, 1]),
    (2, 16, 3, 384, [2001, 1000]),                    # 9003 entries: past the first table batch, R % 4 = 3
    (4, 64, 8, 1024, [1200, 0, 900, 1011]),           # 24888 entries: the vector pass over the table
    (2, 32, 5, 2048, [33, 20]),                       # K = 5: tiles of 12 tokens, the last one short
])
@pytest.mark.parametrize("fp8", [True, "pow2"], ids=["f32scales", "pow2scales"])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
def test_forward_routes_and_quantises_in_one_launch(gpu_device, options, W, E, K, H, tokens, fp8, padded):
    """forward with an fp8 dispatch routes and quantises in one launch (a tile of tokens per
    workgroup): index arrays, rows, scales and output bit for bit those of the oracle and of the
    routing launch followed by dispatch_fp8, at the chosen tile and at forced tiles of 1, 5 and 32 tokens."""
    g = torch.Generator().manual_seed(sum(tokens) + E + K)
    dtype = torch.bfloat16 if K % 2 else torch.float16
    cfg = C.MoEConfig(E, K, H, max(tokens) + 1, dtype, dtype)
    world = []
    for n in tokens:
        idx = (torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32) if n
               else torch.empty(0, K, dtype=torch.int32))
        world.append(C.RankData(n, idx, torch.rand(n, K, generator=g), torch.randn(n, H, generator=g).to(dtype)))
    x, idx, w, rs = concat_world(world, gpu_device)
    T = x.shape[0]
    want = V.run_world(cfg, world, stub_kind=C.STUB_EXPERT_FRACTION, fp8=True, pow2=fp8 == "pow2")
    lib = _lib.load()
    elem = _lib.BF16 if dtype == torch.bfloat16 else _lib.F16
    assert lib.moe_a2a_forward_launches(T, K, H, 0, elem, elem, 1, 1, 0) == 3
    assert lib.moe_a2a_forward_launches(T, K, H, 0, elem, elem, 1, 0, 0) == (4 if T * K <= 32768 else 5)
    ref = None
    for fuse_route, tile in ((False, 0), (True, 0), (True, 1), (True, 5), (True, 32)):
        options.set("FP8_TILE", tile)
        ata = HipAllToAll(cfg, 0, W, stub_kind=C.STUB_EXPERT_FRACTION, fp8_dispatch=fp8, fuse_route=fuse_route,
                          fuse_stub=False, padded=padded)
        for _ in range(2):
            y = ata.forward(x, idx, w, rs)
        torch.cuda.synchronize()
        d = ata.last
        assert int(d.status.item()) == 0
        what = f"route_dispatch_fp8, tile {tile}" if fuse_route else "separate launches"
        got = dict(counts=d.counts, offsets=d.offsets, slot_of_entry=d.slot_of_entry, src_of_slot=d.src_of_slot,
                   meta=d.meta, disp_x=d.disp_x, disp_scale=d.disp_scale, y=y)
        if not padded:
            for key, val in got.items():
                assert_same(f"{key} ({what})", val, want[key])
        else:  # the padded layout against the compact one: entry by entry, and the output
            assert_same(f"counts ({what})", d.counts, want["counts"])
            assert_same(f"y ({what})", y, want["y"])
            slots, wslots = d.slot_of_entry.cpu().long().flatten(), want["slot_of_entry"].long().flatten()
            assert torch.equal(d.disp_x.cpu()[slots], want["disp_x"][wslots])
            assert torch.equal(bits(d.disp_scale.cpu()[slots]), bits(want["disp_scale"][wslots]))
            assert torch.equal(d.meta.cpu()[slots], want["meta"][wslots])
        if ref is None:
            ref = {k: v.clone() for k, v in got.items()}
        else:  # rows no entry owns are not written by either form: compare what the entries own
            for key in ("counts", "offsets", "slot_of_entry", "y"):
                assert torch.equal(bits(got[key]), bits(ref[key])), f"{key} ({what})"
    # the launch timer names the kernel
    import ctypes
    options.set("FP8_TILE", 0)
    assert lib.moe_a2a_timer_begin(8) == 0
    ata.forward(x, idx, w, rs)
    ids, us = (ctypes.c_int * 8)(), (ctypes.c_float * 8)()
    assert lib.moe_a2a_timer_end(ids, us, 8) == 3
    assert lib.moe_a2a_kernel_name(ids[0]) == b"route_dispatch_fp8"


def test_one_launch_fp8_routing_reports_a_bad_expert_id(gpu_device):
    cfg = C.MoEConfig(16, 2, 256, 64, torch.bfloat16, torch.bfloat16)
    g = torch.Generator().manual_seed(5)
    idx = torch.stack([torch.randperm(16, generator=g)[:2] for _ in range(64)]).to(torch.int32)
    idx[17, 1] = 16
    x = torch.randn(64, 256, generator=g).to(torch.bfloat16).to(gpu_device)
    ata = HipAllToAll(cfg, 0, 1, fp8_dispatch=True, fuse_stub=False)
    with pytest.raises(IndexError):
        ata.forward(x, idx.to(gpu_device), torch.rand(64, 2, generator=g).to(gpu_device), check_status=True)


@pytest.mark.parametrize("name", GOLDEN_CASES)
@pytest.mark.parametrize("fuse_route", ["always", False])
def test_padded_layout_is_the_reference_dispatch_return_value(gpu_device, name, fuse_route):
    """padded=True lays the rows out as the reference's [E_l, max_recv, .] buffers: the views
    handed out per owner rank equal what the reference's own dispatch returned, and the final
    output is unchanged."""
    cfg, world, expected = load_golden(name)
    W = len(world)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, padded=True, fuse_route=fuse_route)
    d = ata.dispatch(x, idx, rs)
    ey = ata.expert_stub(d)
    y = ata.combine(None, w, d, ey)
    assert int(d.status.item()) == 0
    E_l = cfg.num_experts // W
    assert d.disp_x.shape[0] == cfg.num_experts * ata.max_recv and ata.max_recv == cfg.max_num_tokens * W
    for r, exp in enumerate(expected):
        num, ex, em = d.padded(r)
        assert ex.shape == (E_l, ata.max_recv, cfg.hidden_dim) and ex.data_ptr() >= d.disp_x.data_ptr()  # a view
        assert_same("expert_num_tokens", num, exp.expert_num_tokens)
        assert_same("expert_x", torch.cat([ex[le, : int(num[le])] for le in range(E_l)], 0), exp.expert_x)
        assert_same("expert_meta", torch.cat([em[le, : int(num[le])] for le in range(E_l)], 0), exp.expert_meta)
        ey_r = ey.view(W, E_l, ata.max_recv, cfg.hidden_dim)[r]
        assert_same("expert_y", torch.cat([ey_r[le, : int(num[le])] for le in range(E_l)], 0), exp.expert_y)
    assert_same("y", y, golden_compact(cfg, expected)["y"])
    assert_same("y (single call)", ata.forward(x, idx, w, rs), golden_compact(cfg, expected)["y"])


def test_padded_layout_larger_worlds_and_overflow_flag(gpu_device):
    wl = C.generate_workload("skew_world")
    want = V.run_world(wl.cfg, wl.world, stub_kind=wl.stub_kind)
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    for fuse_route, max_recv in ((False, 1024), ("always", 1024), (False, None)):
        ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, padded=True, fuse_route=fuse_route,
                          max_recv=max_recv)
        y = ata.forward(x, idx, w, rs)
        assert_same("y", y, want["y"])
        d = ata.last
        assert int(d.status.item()) == 0
        off = want["offsets"].tolist()
        rows = d.slot_of_entry.cpu().long()
        e = idx.flatten().cpu().long()
        j = want["slot_of_entry"].long() - want["offsets"][e].long()
        assert torch.equal(rows, e * ata.max_recv + j)  # row = expert * max_recv + position
        assert_same("rows hold the tokens", d.disp_x[rows.to(gpu_device)], want["disp_x"][want["slot_of_entry"].long()])
    # the hottest expert receives far more than 64 rows: too small a segment must be flagged
    for fuse_route in (False, "always"):
        small = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, padded=True, max_recv=64,
                            fuse_route=fuse_route)
        small.forward(x, idx, w, rs)
        torch.cuda.synchronize()
        assert int(small.last.status.item()) == 2


@pytest.mark.parametrize("E,K,T,H,W", [(1, 1, 1, 8, 1), (2, 2, 1, 16, 2), (4, 2, 3, 8, 1), (256, 8, 1, 7168, 8),
                                         (8, 8, 2049, 64, 8)])
def test_degenerate_shapes(gpu_device, E, K, T, H, W):
    """One expert, one token, the narrowest rows (a single 16-byte vector), every expert chosen
    by every token, a table one entry past a tile boundary."""
    g = torch.Generator().manual_seed(T + H)
    cfg = C.MoEConfig(E, K, H, T + 1, torch.float16, torch.float16)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    world = [C.RankData.empty(cfg) for _ in range(W)]
    world[W - 1] = C.RankData(T, idx, torch.rand(T, K, generator=g), torch.randn(T, H, generator=g).to(torch.float16))
    for fuse in ("always", False):
        compare(cfg, world, gpu_device, C.STUB_OWNER_RANK, fuse_route=fuse)


def test_unaligned_index_slices_and_out_of_range_ids(gpu_device):
    """indices / weights that start 4 bytes into an allocation; an expert id outside [0, E) is
    clamped (nothing is written out of bounds) and raises the status flag."""
    wl = C.generate_workload("tiny")
    cfg = wl.cfg
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    T, K = idx.shape
    idx_store = torch.zeros(T * K + 1, dtype=torch.int32, device=gpu_device)
    w_store = torch.zeros(T * K + 1, dtype=torch.float32, device=gpu_device)
    idx_u, w_u = idx_store[1:].view(T, K), w_store[1:].view(T, K)
    idx_u.copy_(idx)
    w_u.copy_(w)
    assert idx_u.data_ptr() % 16 == 4
    want = V.run_world(cfg, wl.world, stub_kind=1)
    for fuse in ("always", False):
        ata = HipAllToAll(cfg, 0, 1, stub_kind=1, fuse_route=fuse)
        assert_same("y", ata.forward(x, idx_u, w_u), want["y"])
        assert int(ata.last.status.item()) == 0
    bad = idx.clone()
    bad[5, 1] = 99
    bad[9, 0] = -3
    clamped = bad.clamp(0, cfg.num_experts - 1)
    want = V.run_world(cfg, [C.RankData(T, clamped.cpu(), w.cpu(), x.cpu())], stub_kind=1)
    for fuse in ("always", False):
        for fuse_stub in (False, True):  # the folded stub takes its factor from the clamped id as well
            ata = HipAllToAll(cfg, 0, 1, stub_kind=1, fuse_route=fuse, fuse_stub=fuse_stub)
            y = ata.forward(x, bad, w)
            assert int(ata.last.status.item()) == _lib.STATUS_BAD_EXPERT
            assert_same("slot_of_entry", ata.last.slot_of_entry, want["slot_of_entry"])
            assert_same("disp_x", ata.last.disp_x, want["disp_x"])
            assert_same("y", y, want["y"])


def test_status_reports_both_conditions(gpu_device):
    """A call that meets an expert id out of range AND a padded segment that overflows reports both
    bits, whichever lane gets there first; the record of a later call describes that call alone."""
    wl = C.generate_workload("skew_world")
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    bad = idx.clone()
    bad[3, 0] = wl.cfg.num_experts + 5
    bad[700, 2] = -1
    for fuse_route in (False, "always"):
        ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, padded=True, max_recv=64,
                          fuse_route=fuse_route)
        ata.forward(x, bad, w, rs)
        torch.cuda.synchronize()
        assert int(ata.last.status.item()) == _lib.STATUS_BAD_EXPERT | _lib.STATUS_OVERFLOW
        for _ in range(3):  # clean ids on the other buffer set, then on the first one again: only the overflow
            ata.forward(x, idx, w, rs)
            torch.cuda.synchronize()
            assert int(ata.last.status.item()) == _lib.STATUS_OVERFLOW


@pytest.mark.parametrize("name,fp8,fuse_route", [("tiny", False, True), ("dsv3_rank", False, True),
                                                 ("skew_world", False, True), ("skew_world", False, False),
                                                 ("skew_world", True, True), ("prefill_graph", False, True)])
def test_status_describes_the_call_that_produced_it(gpu_device, name, fp8, fuse_route):
    """The status word belongs to a reused buffer set and the kernels only set bits in it: every call
    clears the word of the OTHER set (no launch of its own), so a clean call after a bad one reads 0
    whichever set it lands on, through every form of the one-call forward and through the
    phase-by-phase dispatch; `check_status` raises as the reference does (reference.py:81-86)."""
    wl = C.generate_workload(name, tokens_scale=1 / 8 if name == "prefill_graph" else 1.0)
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    bad = idx.clone()
    bad[0, 0] = wl.cfg.num_experts
    ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, fp8_dispatch=fp8, fuse_route=fuse_route,
                      fuse_stub=True)
    want = ata.forward(x, idx, w, rs).clone()
    seen = []
    for ids in (bad, idx, idx, bad, bad, idx, idx):
        y = ata.forward(x, ids, w, rs)
        seen.append(int(ata.last.status.item()))
        if ids is idx:
            assert torch.equal(bits(y.cpu()), bits(want.cpu()))
    assert seen == [1, 0, 0, 1, 1, 0, 0]
    with pytest.raises(IndexError, match="expert id"):
        ata.forward(x, bad, w, rs, check_status=True)
    ata.forward(x, idx, w, rs, check_status=True)  # and the clean call behind it passes
    ata.forward(x, idx, w, rs, check_status=True)
    # phase by phase: the record of a dispatch describes that dispatch
    for ids, bits_want in ((bad, 1), (idx, 0), (idx, 0)):
        assert int(ata.dispatch(x, ids, rs).status.item()) == bits_want


def test_custom_kernel_check_status_and_config_changed_in_place(gpu_device):
    """`custom_kernel(data, check_status=True)` raises on an id the reference would fail on; a config
    object changed in place between two calls gets the instance of its new values."""
    from kernel_amd.submission import custom_kernel
    from oracle.checker import ref_kernel

    spec = dict(C.REFERENCE_TESTS[1])
    W = spec.pop("world_size")
    cfg, rd, rank, world = C.generate_input(**spec, rank=2, world_size=W, device=gpu_device)
    out = custom_kernel((cfg, rd, rank, world), check_status=True)
    assert torch.equal(bits(out.cpu()), bits(ref_kernel((cfg, rd, rank, world)).cpu()))
    bad = C.RankData(rd.num_tokens, rd.indices.clone(), rd.weights, rd.x)
    bad.indices[0, 0] = cfg.num_experts + 1
    with pytest.raises(IndexError):
        custom_kernel((cfg, bad, rank, world), check_status=True)
    custom_kernel((cfg, bad, rank, world))  # default: clamped, no error
    # same object, other geometry: half the hidden size and another top-k
    T = rd.num_tokens
    cfg.hidden_dim //= 2
    cfg.experts_per_token -= 1
    rd2 = C.RankData(T, rd.indices[:, :cfg.experts_per_token].contiguous(),
                     rd.weights[:, :cfg.experts_per_token].contiguous(), rd.x[:, :cfg.hidden_dim].contiguous())
    out2 = custom_kernel((cfg, rd2, rank, world), check_status=True)
    assert out2.shape == (T, cfg.hidden_dim)
    assert torch.equal(bits(out2.cpu()), bits(ref_kernel((cfg, rd2, rank, world)).cpu()))


def test_dispatch_of_an_empty_rank(gpu_device):
    """No token at all: counts and offsets are zeros, nothing else is touched, and the routing
    table (an empty tensor, whose address is not readable) is never read."""
    cfg = C.MoEConfig(64, 6, 2048, 16, torch.bfloat16, torch.bfloat16)
    x = torch.empty(0, cfg.hidden_dim, dtype=torch.bfloat16, device=gpu_device)
    idx = torch.empty(0, cfg.experts_per_token, dtype=torch.int32, device=gpu_device)
    w = torch.empty(0, cfg.experts_per_token, dtype=torch.float32, device=gpu_device)
    for fuse_route in (True, False, "always"):
        ata = HipAllToAll(cfg, 3, 8, fuse_route=fuse_route)
        d = ata.dispatch(x, idx)
        torch.cuda.synchronize()
        assert d.num_rows == 0 and int(d.status.item()) == 0
        assert torch.equal(d.counts.cpu(), torch.zeros(64, dtype=torch.int32))
        assert torch.equal(d.offsets.cpu(), torch.zeros(65, dtype=torch.int32))
        y = ata.combine(None, w, d, ata.expert_stub(d))
        assert tuple(y.shape) == (0, cfg.hidden_dim)
        assert tuple(ata.forward(x, idx, w).shape) == (0, cfg.hidden_dim)
    # the same through the C entry points with NULL for everything that holds no element
    lib = _lib.load()
    counts = torch.full((64,), -1, dtype=torch.int32, device=gpu_device)
    offsets = torch.full((65,), -1, dtype=torch.int32, device=gpu_device)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.moe_a2a_route(None, None, 0, 0, 6, 64, 8, 0, counts.data_ptr(), offsets.data_ptr(), None, None, None,
                             None, None, 0, st) == 0
    torch.cuda.synchronize()
    assert int(counts.abs().sum()) == 0 and int(offsets.abs().sum()) == 0
    counts.fill_(-1)
    offsets.fill_(-1)
    assert lib.moe_a2a_route_dispatch(None, None, None, 0, 0, 6, 64, 8, 2048, 0, counts.data_ptr(),
                                      offsets.data_ptr(), None, None, None, None, None, st) == 0
    torch.cuda.synchronize()
    assert int(counts.abs().sum()) == 0 and int(offsets.abs().sum()) == 0


def test_custom_kernel_contract(gpu_device):
    """custom_kernel(data) per rank == oracle ref_kernel, checked with the reference's tolerance."""
    from kernel_amd.submission import custom_kernel
    from oracle.checker import check_implementation, ref_kernel

    spec = dict(C.REFERENCE_TESTS[5])
    W = spec.pop("world_size")
    for rank in range(W):
        data = C.generate_input(**spec, rank=rank, world_size=W, device=gpu_device)
        out = custom_kernel(data)
        assert out.dtype == data[0].out_dtype and out.shape == (data[1].num_tokens, data[0].hidden_dim)
        ok, msg = check_implementation(data, out)
        assert ok, msg
        assert torch.equal(bits(out.cpu()), bits(ref_kernel(data).cpu()))


@pytest.mark.gpu
def test_buffer_sets_alternate_and_old_token_counts_are_dropped(gpu_device):
    """Two buffer sets per token count alternate (a result stays valid until the second-next call with
    that count), both are allocated on the first call, and only the most recently used counts are kept."""
    E, K, H = 16, 2, 64
    cfg = C.MoEConfig(E, K, H, 64, torch.bfloat16, torch.bfloat16)
    ata = HipAllToAll(cfg, 0, 1, fuse_stub=True)
    g = torch.Generator().manual_seed(5)

    def inputs(T):
        idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
        world = [C.RankData(T, idx, torch.rand(T, K, generator=g), torch.randn(T, H, generator=g).to(torch.bfloat16))]
        return world, concat_world(world, gpu_device)

    worlds = {}
    for T in range(1, ata.MAX_CACHED_SHAPES + 4):  # more token counts than the cache keeps
        world, (x, idx, w, rs) = inputs(T)
        y = ata.forward(x, idx, w, rs)
        torch.cuda.synchronize()
        want = V.run_world(cfg, world, stub_kind=ata.stub_kind)["y"]
        assert torch.equal(bits(y.cpu()), bits(want)), T
        worlds[T] = (world, x, idx, w, rs, y, want)
    assert len(ata._bufs) == ata.MAX_CACHED_SHAPES
    kept = [key[0] for key in ata._bufs]
    assert kept == list(range(4, ata.MAX_CACHED_SHAPES + 4))  # the oldest counts went first
    assert all(s is not None for ring in ata._bufs.values() for s in ring["sets"])  # both sets exist at once
    # the result of a call survives the next call with the same count and is reused by the one after
    T = kept[-1]
    world, x, idx, w, rs, y1, want = worlds[T]
    y2 = ata.forward(x, idx, w, rs)
    assert y2.data_ptr() != y1.data_ptr()
    torch.cuda.synchronize()
    assert torch.equal(bits(y1.cpu()), bits(want)) and torch.equal(bits(y2.cpu()), bits(want))
    y3 = ata.forward(x, idx, w, rs)
    assert y3.data_ptr() == y1.data_ptr()
    # a dropped count comes back with fresh buffers and the right answer
    world, x, idx, w, rs, _, want = worlds[1]
    y = ata.forward(x, idx, w, rs)
    torch.cuda.synchronize()
    assert torch.equal(bits(y.cpu()), bits(want))
    assert len(ata._bufs) == ata.MAX_CACHED_SHAPES
