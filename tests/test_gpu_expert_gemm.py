"""Grouped expert GEMM (matrix cores) against an f32 torch reference of the same product.

The summation order differs from torch's, so the comparison is a tolerance, stated here:
|got - want| <= 1e-2 * |want| + 1e-2 * rms(want) (one bf16 ulp is 0.4-0.8 %; fp16 is tighter).
"""
import pytest
import torch

from kernel_amd import contract as C
from kernel_amd.all2all import HipAllToAll, concat_world
from oracle import all2all_vec as V

pytestmark = pytest.mark.gpu


def close(got, want):
    got, want = got.float().cpu(), want.float()
    tol = 1e-2 * want.abs() + 1e-2 * want.pow(2).mean().sqrt()
    bad = (got - want).abs() > tol
    assert not bool(bad.any()), f"{int(bad.sum())} of {bad.numel()} out of tolerance, worst " \
                                f"{float(((got - want).abs() / tol).max()):.2f}x"


def make(E, K, T, H, N, W, dtype, seed, zipf=False):
    g = torch.Generator().manual_seed(seed)
    cfg = C.MoEConfig(E, K, H, T + 1, dtype, dtype)
    if zipf:
        p = (torch.arange(E, dtype=torch.float64) + 1).pow(-1.2)
        idx = torch.multinomial((p / p.sum()).float().expand(T, E), K, generator=g).to(torch.int32)
    else:
        idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    world = [C.RankData(T, idx, torch.rand(T, K, generator=g), torch.randn(T, H, generator=g).to(dtype))]
    world += [C.RankData.empty(cfg) for _ in range(W - 1)]
    weights = (torch.randn(E, N, H, generator=g) / H ** 0.5).to(dtype)
    return cfg, world, weights


@pytest.mark.parametrize("E,K,T,H,N,W,zipf", [
    (8, 2, 40, 64, 64, 1, False),      # one K slab, tiles mostly empty
    (8, 2, 700, 128, 200, 2, False),   # several m-tiles per expert, N not a multiple of 128
    (16, 4, 300, 192, 136, 4, True),   # skewed: empty experts and long segments
    (64, 6, 1024, 2048, 2048, 8, True),
    (256, 8, 256, 7168, 512, 8, False),  # headline routing shape, 8 rows per expert on average
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
@pytest.mark.parametrize("tile", ["32", "128", "256"], ids=["tile32", "tile128", "tile256"])
def test_expert_gemm_matches_f32_reference(gpu_device, options, E, K, T, H, N, W, zipf, dtype, padded, tile):
    # every kernel on every shape (the 32-row kernel needs H % 128 == 0; the library takes the
    # 128 x 128 kernel for the other hidden sizes)
    options.set("GEMM_TILE", tile)
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=E + T, zipf=zipf)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, padded=padded, max_recv=T if padded else None)
    d = ata.dispatch(x, idx, rs)
    y = ata.expert_gemm(d, weights.to(gpu_device))
    torch.cuda.synchronize()
    o = V.run_world(cfg, world)
    want = V.expert_gemm(o["disp_x"], o["offsets"], weights, dtype)
    rows = d.slot_of_entry.long() if padded else o["slot_of_entry"].long().to(gpu_device)
    close(y[rows], want[o["slot_of_entry"].long()])
    if not padded:
        close(y, want)


@pytest.mark.parametrize("E,K,T,H,N,zipf", [
    (8, 2, 1200, 384, 264, False),   # 300 rows per expert: the library itself picks the 256 x 256 kernel
    (16, 4, 1500, 256, 512, True),   # skewed, segments from empty to well past one tile
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_both_tile_sizes_give_the_same_bits(gpu_device, options, E, K, T, H, N, zipf, dtype):
    """The two kernels accumulate over K in the same order, so their outputs are identical; the
    default choice for these shapes (R > 32 E) is the wide one."""
    cfg, world, weights = make(E, K, T, H, N, 1, dtype, seed=7 * E + T, zipf=zipf)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, 1)
    d = ata.dispatch(x, idx, rs)
    wd = weights.to(gpu_device)
    lib = ata.lib
    outs = {}
    for tile in ("default", "32", "128", "256"):
        if tile == "default":
            options.set("GEMM_TILE", 0)
        else:
            options.set("GEMM_TILE", tile)
        assert lib.moe_a2a_timer_begin(4) == 0
        outs[tile] = ata.expert_gemm(d, wd).clone()
        torch.cuda.synchronize()
        import ctypes
        ids, us = (ctypes.c_int * 4)(), (ctypes.c_float * 4)()
        assert lib.moe_a2a_timer_end(ids, us, 4) == 1
        name = lib.moe_a2a_kernel_name(ids[0]).decode()
        assert name == {"32": "expert_gemm_skinny", "128": "expert_gemm"}.get(tile, "expert_gemm_wide")
    assert torch.equal(outs["128"].view(torch.int16), outs["256"].view(torch.int16))
    assert torch.equal(outs["32"].view(torch.int16), outs["256"].view(torch.int16))
    assert torch.equal(outs["default"].view(torch.int16), outs["256"].view(torch.int16))
    o = V.run_world(cfg, world)
    close(outs["256"], V.expert_gemm(o["disp_x"], o["offsets"], weights, dtype))


@pytest.mark.parametrize("E,K,T,H,N,W,zipf", [
    (8, 2, 40, 128, 64, 1, False),      # one scale block, tiles mostly empty
    (8, 2, 1200, 256, 264, 2, False),   # full 256-row tiles and 128-row tails, ragged N
    (16, 4, 300, 384, 136, 4, True),    # skewed: empty experts and long segments
    (32, 4, 2048, 1024, 512, 8, False),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
def test_expert_gemm_on_fp8_rows(gpu_device, E, K, T, H, N, W, zipf, dtype, padded):
    """fp8 dispatch -> expert GEMM.  The dispatched bytes and scales are bit-exact (checked here
    again), and the product is compared with an f32 matmul of the dequantised rows, each element
    rounded once to the weights' type as the kernel does."""
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=3 * E + T, zipf=zipf)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, fp8_dispatch=True, padded=padded, max_recv=T if padded else None)
    d = ata.dispatch(x, idx, rs)
    y = ata.expert_gemm(d, weights.to(gpu_device))
    torch.cuda.synchronize()
    o = V.run_world(cfg, world, fp8=True)
    rows = d.slot_of_entry.long() if padded else o["slot_of_entry"].long().to(gpu_device)
    soe = o["slot_of_entry"].long()
    assert torch.equal(d.disp_x[rows].cpu(), o["disp_x"][soe])
    assert torch.equal(d.disp_scale[rows].cpu(), o["disp_scale"][soe])
    want = V.expert_gemm_fp8(o["disp_x"], o["disp_scale"], o["offsets"], weights, dtype)
    close(y[rows], want[soe])


def test_fp8_gemm_feeds_combine(gpu_device):
    """fp8 dispatch -> expert GEMM (H -> H) -> f32 combine against the same chain on the CPU."""
    cfg, world, weights = make(32, 4, 1024, 256, 256, 8, torch.bfloat16, seed=5)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, 8, fp8_dispatch=True, combine_mode=C.COMBINE_F32)
    d = ata.dispatch(x, idx, rs)
    y = ata.combine(None, w, d, ata.expert_gemm(d, weights.to(gpu_device)))
    o = V.run_world(cfg, world, fp8=True)
    ey = V.expert_gemm_fp8(o["disp_x"], o["disp_scale"], o["offsets"], weights, torch.bfloat16)
    want = V.combine_f32(ey, w.cpu(), o["slot_of_entry"], torch.bfloat16)
    close(y, want)


def test_decode_shape_takes_the_skinny_kernel(gpu_device, options):
    """Eight rows per expert on average (the headline routing shape): the library picks the
    32 x 256 kernel by itself, and its bits equal the 128 x 128 kernel's."""
    options.set("GEMM_TILE", 0)
    cfg, world, weights = make(256, 8, 256, 1024, 520, 8, torch.bfloat16, seed=11)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, 8)
    d = ata.dispatch(x, idx, rs)
    wd = weights.to(gpu_device)
    import ctypes
    assert ata.lib.moe_a2a_timer_begin(4) == 0
    y = ata.expert_gemm(d, wd).clone()
    torch.cuda.synchronize()
    ids, us = (ctypes.c_int * 4)(), (ctypes.c_float * 4)()
    assert ata.lib.moe_a2a_timer_end(ids, us, 4) == 1
    assert ata.lib.moe_a2a_kernel_name(ids[0]) == b"expert_gemm_skinny"
    options.set("GEMM_TILE", "128")
    y128 = ata.expert_gemm(d, wd)
    assert torch.equal(y.view(torch.int16), y128.view(torch.int16))
    o = V.run_world(cfg, world)
    close(y, V.expert_gemm(o["disp_x"], o["offsets"], weights, torch.bfloat16))


@pytest.mark.parametrize("E,K,T,H,N,W,zipf", [
    (8, 2, 40, 128, 128, 1, False),      # one block each way
    (64, 4, 128, 512, 384, 8, False),    # decode-like: 8 rows per expert
    (16, 4, 300, 384, 256, 4, True),     # skewed: empty experts and long segments
    (8, 2, 1200, 256, 256, 2, False),    # 300 rows per expert
    (4, 2, 1100, 1024, 384, 1, True),    # eight K blocks, three 128-column tiles, long ragged segments
    (3, 1, 700, 640, 128, 1, False),     # five K blocks: the three-buffer loop ends on its second tail step
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("fp8_rows", [False, True], ids=["rows16", "rows8"])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
@pytest.mark.parametrize("tile", ["32", "32r", "128", "128f", "256"],
                         ids=["tile32", "tile32staged", "tile128", "tile128fourwaves", "tile256"])
def test_expert_gemm_block_quantised_weights(gpu_device, options, E, K, T, H, N, W, zipf, dtype, fp8_rows,
                                             padded, tile):
    """Weights as e4m3fn bytes with one scale per 128 x 128 block, rows 16-bit or from the fp8
    dispatch, against an f32 matmul of the dequantised operands (each rounded once to the 16-bit
    type, as two of the kernels do), through the weight-streaming kernel, the fp8 x fp8 kernel (tile
    128, fp8 rows only: 16-bit rows keep the default choice) and the 256 x 256 kernel (which needs
    N >= 256; the one N == 128 case stays on the other).  The weight-streaming form exists twice:
    slabs sent memory -> LDS directly (tile32) and staged through registers (tile32staged)."""
    options.set("GEMM_TILE", tile[:2] if tile.startswith("32") else tile[:3])
    if tile == "32r":
        options.set("GEMM_STAGED", 1)
    if tile == "128f":  # the four-wave 128 x 128 form of the fp8 x fp8 kernel (eight waves on 256 x 128 otherwise)
        options.set("GEMM_STAGED", 2)
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=5 * E + T, zipf=zipf)
    wq, ws = V.quantize_weights_fp8(weights)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, fp8_dispatch=fp8_rows, padded=padded, max_recv=T if padded else None)
    d = ata.dispatch(x, idx, rs)
    y = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device))
    torch.cuda.synchronize()
    o = V.run_world(cfg, world, fp8=fp8_rows)
    # fp8 rows on segments of more than 32 rows take the fp8 x fp8 kernel unless another is forced: no
    # rounding of the rows there
    f8_kernel = fp8_rows and (tile in ("128", "128f") or (tile == "256" and N < 256 and d.num_rows > 32 * E))
    want = V.expert_gemm_q8(o["disp_x"], o["disp_scale"] if fp8_rows else None, wq, ws, o["offsets"], dtype,
                            round_rows=not f8_kernel)
    rows = d.slot_of_entry.long() if padded else o["slot_of_entry"].long().to(gpu_device)
    close(y[rows], want[o["slot_of_entry"].long()])


@pytest.mark.parametrize("E,K,T,H,N,W,zipf", [
    (8, 2, 40, 128, 128, 1, False),      # 10 rows per expert: half tiles, one 128-column block
    (4, 2, 300, 256, 256, 1, False),     # 150 rows per expert: half tiles
    (16, 4, 300, 384, 384, 4, True),     # skewed: empty experts, long segments, a 128-column tail tile
    (8, 2, 1200, 256, 512, 2, False),    # 300 rows per expert
    (3, 1, 1000, 1024, 256, 1, False),   # 333 rows per expert, eight K blocks
    (5, 2, 700, 768, 640, 1, True),      # twelve slabs of 64 bytes, a 128-column tail tile, ragged
    (2, 1, 300, 8192, 256, 1, False),    # 64 scale blocks per row: the eight-wave form's exponent table is full
    (2, 1, 300, 8448, 256, 1, False),    # 66: beyond it (the four-wave forms run)
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("padded", [False, True], ids=["compact", "padded"])
@pytest.mark.parametrize("form", [4, 3, 2, 1], ids=["eight", "eight-early-b", "direct", "staged"])
def test_expert_gemm_power_of_two_scales(gpu_device, options, E, K, T, H, N, W, zipf, dtype, padded, form):
    """fp8 rows and fp8 weights whose scales are powers of two, multiplied by the fp8 matrix
    instruction with the scales as its block exponents, against the f32 matmul of the
    dequantised operands; the fp8 x fp8 kernel with the fold on the vector units, which takes
    any f32 scale, has to agree with it to f32 summation order.  All forms of the tiled kernel:
    eight waves on slabs of 128 columns (hidden sizes from 256; with and without the early requests for the
    rows of the weights that short segments get by themselves), four waves with slabs of 64 columns
    sent memory -> LDS directly (multiples of 256) and staged through registers (every hidden size)."""
    options.set("GEMM_TILE", "256")  # the tiles at every segment length
    options.set("GEMM_STAGED", form)
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=7 * E + T, zipf=zipf)
    wq, ws = V.quantize_weights_fp8(weights, pow2=True)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, fp8_dispatch="pow2", padded=padded, max_recv=T if padded else None)
    d = ata.dispatch(x, idx, rs)
    y = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device), scales_pow2=True)
    options.set("GEMM_TILE", 0)
    y_auto = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device), scales_pow2=True)  # library's choice
    y_fold = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device))
    torch.cuda.synchronize()
    o = V.run_world(cfg, world, fp8=True, pow2=True)
    want = V.expert_gemm_q8(o["disp_x"], o["disp_scale"], wq, ws, o["offsets"], dtype, round_rows=False)
    rows = d.slot_of_entry.long() if padded else o["slot_of_entry"].long().to(gpu_device)
    close(y[rows], want[o["slot_of_entry"].long()])
    close(y[rows], y_fold[rows].cpu())
    close(y_auto[rows], want[o["slot_of_entry"].long()])


@pytest.mark.parametrize("form", ["16bit-32", "16bit-128", "16bit-256", "q8-32", "q8-32staged", "q8-128", "q8-256",
                                  "mx-eight", "mx-early", "mx-direct", "mx-staged"])
def test_padded_overflow_stays_inside_the_buffers(gpu_device, options, form):
    """Padded layout with a LAST expert that receives more rows than max_recv (routing folds the
    surplus onto the segment's last row and raises the overflow bit; counts stay the true numbers):
    every GEMM form multiplies only the max_recv rows the segment holds.  Guard rows behind the
    output keep their sentinel, the rows of the other experts and the unfolded rows of the full
    expert equal the reference."""
    from kernel_amd import _lib

    E, K, T, H, N, W, max_recv = 8, 2, 300, 256, 256, 2, 96
    dtype = torch.bfloat16
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=11)
    world[0].indices[:, 1] = E - 1  # every token also goes to the last expert: 300 rows for 96 places
    world[0].indices[:, 0] %= E - 1
    kind, tile = form.split("-")
    options.set("GEMM_TILE", int(tile[:3].rstrip("sd")) if tile[0].isdigit() else 256)
    if tile in ("32staged", "staged"):
        options.set("GEMM_STAGED", 1)
    if tile == "direct":
        options.set("GEMM_STAGED", 2)
    if tile in ("eight", "early"):  # the eight-wave loop without / with the early requests for the weight rows
        options.set("GEMM_STAGED", 4 if tile == "eight" else 3)
    fp8 = {"16bit": False, "q8": True, "mx": "pow2"}[kind]
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, fp8_dispatch=fp8, padded=True, max_recv=max_recv)
    d = ata.dispatch(x, idx, rs)
    rows = E * max_recv
    guard = 2 * max_recv + 300  # more than the surplus of the overflowing expert
    buf = torch.full((rows + guard, N), 7.0, dtype=dtype, device=gpu_device)
    if kind == "16bit":
        ata.expert_gemm(d, weights.to(gpu_device), out=buf[:rows])
    else:
        wq, ws = V.quantize_weights_fp8(weights, pow2=kind == "mx")
        ata.expert_gemm(d, wq.to(gpu_device), out=buf[:rows], w_scale=ws.to(gpu_device), scales_pow2=kind == "mx")
    torch.cuda.synchronize()
    assert int(d.status.item()) == _lib.STATUS_OVERFLOW
    assert int(d.counts[E - 1]) == T  # the true number, beyond the segment
    assert bool((buf[rows:] == 7.0).all()), "rows behind the output buffer were written"
    # reference: the same product on the rows the padded buffers hold
    dx = d.disp_x.cpu()
    sc = d.disp_scale.cpu() if fp8 else None
    counts = d.counts.cpu().clamp(max=max_recv)
    for e in range(E):
        n = int(counts[e]) - (1 if e == E - 1 else 0)  # the folded entries race for the full segment's last row
        lo = e * max_recv
        seg = torch.tensor([0, n], dtype=torch.int32)
        if kind == "16bit":
            want = V.expert_gemm(dx[lo:lo + n], seg, weights[e:e + 1], dtype)
        else:
            want = V.expert_gemm_q8(dx[lo:lo + n], sc[lo:lo + n], wq[e:e + 1], ws[e:e + 1], seg, dtype,
                                    round_rows=False)
        close(buf[lo:lo + n], want)


def test_dispatch_gemm_combine_end_to_end(gpu_device):
    """dispatch -> expert GEMM (H -> H) -> combine against the same chain on the CPU."""
    cfg, world, weights = make(32, 4, 512, 256, 256, 8, torch.bfloat16, seed=3)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, 8, combine_mode=C.COMBINE_F32)
    d = ata.dispatch(x, idx, rs)
    y = ata.combine(None, w, d, ata.expert_gemm(d, weights.to(gpu_device)))
    o = V.run_world(cfg, world)
    ey = V.expert_gemm(o["disp_x"], o["offsets"], weights, torch.bfloat16)
    want = V.combine_f32(ey, w.cpu(), o["slot_of_entry"], torch.bfloat16)
    close(y, want)


@pytest.mark.parametrize("T,E", [(2048, 8), (96, 32)], ids=["wide", "skinny"])
def test_dispatch_gemm_combine_graph_replay(gpu_device, options, T, E):
    """dispatch -> expert GEMM -> combine captured once into a hipGraph; every replay, with eager
    work and synchronisation between the replays and fresh inputs each time, equals the eager
    result bit for bit (no launch of the chain allocates, clears memory or reads a value back)."""
    options.set("GEMM_TILE", 0)
    cfg, world, weights = make(E, 2, T, 256, 256, 4, torch.bfloat16, seed=T)
    x, idx, w, rs = concat_world(world, gpu_device)
    wd = weights.to(gpu_device)

    def chain(a, xx, ii, ww, out_gemm, out):
        d = a.dispatch(xx, ii, rs)
        return a.combine(out, ww, d, a.expert_gemm(d, wd, out=out_gemm))

    ata = HipAllToAll(cfg, 0, 4, combine_mode=C.COMBINE_F32)
    sx, sidx, sw = x.clone(), idx.clone(), w.clone()  # static inputs of the graph
    R = T * 2
    g_gemm = torch.empty(R, 256, dtype=torch.bfloat16, device=gpu_device)
    g_out = torch.empty(T, 256, dtype=torch.bfloat16, device=gpu_device)
    for _ in range(2):  # both buffer sets of the host class exist, first-call set-up is done
        chain(ata, sx, sidx, sw, g_gemm, g_out)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(ata, sx, sidx, sw, g_gemm, g_out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = chain(ata, sx, sidx, sw, g_gemm, g_out)
    eager = HipAllToAll(cfg, 0, 4, combine_mode=C.COMBINE_F32)
    gen = torch.Generator().manual_seed(3)
    for it in range(4):
        perm = torch.randperm(T, generator=gen).to(gpu_device)
        nx, nidx, nw = x[perm].contiguous(), idx[perm].contiguous(), w[perm].contiguous()
        e_gemm = torch.empty_like(g_gemm)
        want = chain(eager, nx, nidx, nw, e_gemm, None).clone()  # eager work between replays
        torch.cuda.synchronize()
        sx.copy_(nx)
        sidx.copy_(nidx)
        sw.copy_(nw)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static.view(torch.int16), want.view(torch.int16)), f"replay {it}"


def test_expert_gemm_argument_checks(gpu_device):
    cfg, world, weights = make(8, 2, 16, 64, 64, 1, torch.bfloat16, seed=1)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, 1)
    d = ata.dispatch(x, idx)
    with pytest.raises(ValueError):
        ata.expert_gemm(d, weights[:, :, :32].contiguous().to(gpu_device))
    bad = HipAllToAll(C.MoEConfig(8, 2, 72, 17, torch.bfloat16, torch.bfloat16), 0, 1)
    xb = torch.randn(16, 72, device=gpu_device).to(torch.bfloat16)
    db = bad.dispatch(xb, idx)
    from kernel_amd._lib import MoeA2AError
    with pytest.raises(MoeA2AError):  # hidden size must be a multiple of 64
        bad.expert_gemm(db, torch.zeros(8, 64, 72, dtype=torch.bfloat16, device=gpu_device))


@pytest.mark.parametrize("seed", range(20))
def test_random_shapes_every_expert_gemm_form(gpu_device, options, seed):
    """Seeded sweep: random expert counts, segment lengths (empty experts, segments that end a
    row or two past a tile), hidden and output sizes, layouts, element types, and every operand
    format (16-bit, fp8 rows, fp8 block-quantised weights, both) through whichever kernel the
    library picks for the shape and, on odd seeds, through a forced one."""
    g = torch.Generator().manual_seed(1000 + seed)

    def pick(choices):
        return choices[int(torch.randint(len(choices), (1,), generator=g))]

    E = pick([1, 3, 8, 9, 24, 40])
    K = pick([1, 2, 4])
    K = min(K, E)
    T = pick([1, 7, 33, 129, 260, 600, 1100])
    H = pick([128, 256, 384, 640])
    N = pick([128, 256, 384, 512, 640])
    W = pick([w for w in (1, 2, 4, 8) if E % w == 0])
    dtype = pick([torch.bfloat16, torch.float16])
    zipf = pick([False, True])
    padded = pick([False, True])
    fp8_rows = pick([False, True])
    q8 = pick([False, True])
    pow2 = pick([False, True]) and fp8_rows and q8  # scales as the matrix instruction's block exponents
    if seed % 2:
        options.set("GEMM_TILE", pick(["32", "128", "256"]))
    else:
        options.set("GEMM_TILE", 0)
    cfg, world, weights = make(E, K, T, H, N, W, dtype, seed=seed, zipf=zipf)
    x, idx, w, rs = concat_world(world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, fp8_dispatch="pow2" if pow2 else fp8_rows, padded=padded,
                      max_recv=T if padded else None)
    d = ata.dispatch(x, idx, rs)
    o = V.run_world(cfg, world, fp8=fp8_rows, pow2=pow2)
    if q8:
        wq, ws = V.quantize_weights_fp8(weights, pow2=pow2)
        y = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device), scales_pow2=pow2)
        # which of the q8 kernels ran decides whether fp8 rows were rounded to 16 bits first; both
        # readings of the rows differ by far less than the tolerance, so the unrounded one serves
        want = V.expert_gemm_q8(o["disp_x"], o["disp_scale"] if fp8_rows else None, wq, ws, o["offsets"], dtype,
                                round_rows=False)
    elif fp8_rows:
        y = ata.expert_gemm(d, weights.to(gpu_device))
        want = V.expert_gemm_fp8(o["disp_x"], o["disp_scale"], o["offsets"], weights, dtype)
    else:
        y = ata.expert_gemm(d, weights.to(gpu_device))
        want = V.expert_gemm(o["disp_x"], o["offsets"], weights, dtype)
    torch.cuda.synchronize()
    rows = d.slot_of_entry.long() if padded else o["slot_of_entry"].long().to(gpu_device)
    close(y[rows], want[o["slot_of_entry"].long()])


def make_counts(counts, H, N, dtype, seed):
    """One rank, one expert per token, expert e receiving exactly counts[e] rows (shuffled)."""
    g = torch.Generator().manual_seed(seed)
    E = len(counts)
    ids = torch.repeat_interleave(torch.arange(E), torch.tensor(counts))
    ids = ids[torch.randperm(ids.numel(), generator=g)].to(torch.int32).reshape(-1, 1)
    T = ids.shape[0]
    cfg = C.MoEConfig(E, 1, H, T + 1, dtype, dtype)
    world = [C.RankData(T, ids, torch.rand(T, 1, generator=g), torch.randn(T, H, generator=g).to(dtype))]
    weights = (torch.randn(E, N, H, generator=g) / H ** 0.5).to(dtype)
    return cfg, world, weights


def walk_cases():
    lone = [0, 0, 0, 3500, 0]                       # fourteen m-tiles of one expert: several groups of four
    gaps = [0] * 64
    for e, n in ((1, 256), (2, 257), (17, 1025), (18, 1), (40, 255), (63, 513)):
        gaps[e] = n                                 # tile-exact, one past a tile, one row, runs of empty experts
    many = [0] * 1024
    for e in range(0, 1024, 3):
        many[e] = 1 + (e * 7) % 5                   # the largest expert count: a few rows on every third
    many[1023] = 700
    ends = [300] + [0] * 30 + [300]                 # rows only on the first and the last expert
    return [("lone", lone), ("gaps", gaps), ("many", many), ("ends", ends)]


@pytest.mark.parametrize("name,counts", walk_cases(), ids=[c[0] for c in walk_cases()])
@pytest.mark.parametrize("fmt", ["16bit", "16bit-early-b", "mx", "mx-early-b", "f32scale"])
@pytest.mark.parametrize("N", [256, 640])
def test_eight_wave_tile_walk_on_odd_segment_tables(gpu_device, options, name, counts, fmt, N):
    """The eight-wave kernels give every expert's m-tiles to one die's workgroups, in groups of at
    most four.  Segment tables that stress that walk: one expert with many tiles, tile-exact and
    one-row segments between runs of empty experts, the largest expert count, rows only at the two
    ends; one n-tile and a ragged last n-tile; each operand format's eight-wave kernel forced, the two with
    two slab buffers in both forms (the rows of the weights requested before the slab's last quarter, or
    early, behind a second barrier, as short segments get them by default)."""
    dtype, H = torch.bfloat16, 256
    fmt, _, early = fmt.partition("-")
    options.set("GEMM_TILE", "128" if fmt == "f32scale" else "256")
    if fmt != "f32scale":
        options.set("GEMM_STAGED", 3 if early else 4)
    cfg, world, weights = make_counts(counts, H, N, dtype, seed=len(counts) + N)
    x, idx, w, rs = concat_world(world, gpu_device)
    fp8 = {"16bit": False, "mx": "pow2", "f32scale": True}[fmt]
    ata = HipAllToAll(cfg, 0, 1, fp8_dispatch=fp8)
    d = ata.dispatch(x, idx, rs)
    o = V.run_world(cfg, world, fp8=bool(fp8), pow2=fmt == "mx")
    assert o["offsets"].tolist() == torch.tensor([0] + counts).cumsum(0).tolist()
    if fmt == "16bit":
        y = ata.expert_gemm(d, weights.to(gpu_device))
        want = V.expert_gemm(o["disp_x"], o["offsets"], weights, dtype)
    else:
        wq, ws = V.quantize_weights_fp8(weights, pow2=fmt == "mx")
        y = ata.expert_gemm(d, wq.to(gpu_device), w_scale=ws.to(gpu_device), scales_pow2=fmt == "mx")
        want = V.expert_gemm_q8(o["disp_x"], o["disp_scale"], wq, ws, o["offsets"], dtype, round_rows=False)
    torch.cuda.synchronize()
    close(y, want)
