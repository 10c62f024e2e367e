"""The five named workloads at their full sizes, plus size-independent properties and the
hipGraph-captured launch sequence.  Needs a GPU.

Bit-exact against the vectorised CPU oracle (seconds of CPU time per workload), and
through properties that need no oracle: a permutation round trip (one-hot weights and a
unit stub give back the tokens), an integer checksum of checksums of the dispatched rows,
and idempotence of the routing outputs.
"""
import pytest
import torch

from golden_io import bits
from kernel_amd import contract as C
from kernel_amd.all2all import HipAllToAll, concat_world
from oracle import all2all_vec as V

pytestmark = pytest.mark.gpu


def gpu_run(wl, dev, combine_mode=0, fp8=None, fuse_stub=False):
    fp8 = wl.fp8_dispatch if fp8 is None else fp8
    x, idx, w, rs = concat_world(wl.world, dev)
    ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, combine_mode=combine_mode, fp8_dispatch=fp8,
                      fuse_stub=fuse_stub)
    d = ata.dispatch(x, idx, rs)
    if fuse_stub:
        y = ata.stub_combine(None, w, idx, d)
    else:
        y = ata.combine(None, w, d, ata.expert_stub(d))
    torch.cuda.synchronize()
    return ata, d, y, (x, idx, w, rs)


@pytest.mark.parametrize("name", C.WORKLOAD_NAMES)
def test_full_size_against_oracle(gpu_device, name):
    wl = C.generate_workload(name)
    want = V.run_world(wl.cfg, wl.world, stub_kind=wl.stub_kind, fp8=wl.fp8_dispatch)
    ata, d, y, _ = gpu_run(wl, gpu_device)
    assert int(d.status.item()) == 0
    for key in ("counts", "offsets", "slot_of_entry", "src_of_slot", "meta", "disp_x"):
        assert torch.equal(bits(getattr(d, key).cpu()), bits(want[key])), key
    if wl.fp8_dispatch:
        assert torch.equal(d.disp_scale.cpu(), want["disp_scale"])
    assert torch.equal(bits(y.cpu()), bits(want["y"]))
    # tolerance stated by the contract for the final output (trivially met when bit-exact)
    assert torch.allclose(y.cpu().float(), want["y"].float(), rtol=1e-2, atol=1e-2)
    # the stub folded into the combine gives the same bits
    _, _, y2, _ = gpu_run(wl, gpu_device, fuse_stub=True)
    assert torch.equal(bits(y2.cpu()), bits(want["y"]))
    # the one-call forward knows what the dispatch wrote and may pick other cache policies for the
    # combine (write-through output stores beyond 256 MB of dispatched rows): same bits, both modes
    # ... and with the stub folded in it is what custom_kernel and bench.py run (for fp8_dispatch in
    # f32 mode: the streaming stub_combine over fp8 rows that the bench line of that workload times)
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    folded = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, fp8_dispatch=wl.fp8_dispatch,
                         fuse_stub=True)
    want32 = None
    for mode in (C.COMBINE_STRICT, C.COMBINE_F32):
        for host in (ata, folded):
            host.combine_mode = mode
            y3 = host.forward(x, idx, w, rs)
            torch.cuda.synchronize()
            assert int(host.last.status.item()) == 0
            if mode == C.COMBINE_STRICT:
                assert torch.equal(bits(y3.cpu()), bits(want["y"]))
            else:
                if want32 is None:
                    want32 = V.run_world(wl.cfg, wl.world, stub_kind=wl.stub_kind, fp8=wl.fp8_dispatch,
                                         combine_mode=mode)["y"]
                assert torch.equal(bits(y3.cpu()), bits(want32))


@pytest.mark.parametrize("fp8", [True, "pow2"], ids=["f32scales", "pow2scales"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_fp8_forward_routes_and_quantises_in_one_launch_at_full_size(gpu_device, fp8, dtype):
    """The fp8 workload through forward (routing + fp8 dispatch in one launch, then stub + combine): index
    arrays, rows, scales and output bit for bit the oracle's, for both scale modes and both element types."""
    import dataclasses

    from kernel_amd import _lib

    wl = C.generate_workload("fp8_dispatch")
    cfg = dataclasses.replace(wl.cfg, in_dtype=dtype, out_dtype=dtype)
    world = [C.RankData(r.num_tokens, r.indices, r.weights, r.x.to(dtype)) for r in wl.world]
    want = V.run_world(cfg, world, stub_kind=wl.stub_kind, fp8=True, pow2=fp8 == "pow2", combine_mode=C.COMBINE_F32)
    x, idx, w, rs = concat_world(world, gpu_device)
    T, K, H = x.shape[0], cfg.experts_per_token, cfg.hidden_dim
    elem = _lib.BF16 if dtype == torch.bfloat16 else _lib.F16
    assert _lib.load().moe_a2a_forward_launches(T, K, H, 0, elem, elem, 2 if fp8 == "pow2" else 1, 1, 1) == 2
    ata = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind, combine_mode=C.COMBINE_F32, fp8_dispatch=fp8,
                      fuse_stub=True)
    for _ in range(2):  # both buffer sets
        y = ata.forward(x, idx, w, rs)
        torch.cuda.synchronize()
        d = ata.last
        assert int(d.status.item()) == 0
        for key in ("counts", "offsets", "slot_of_entry", "src_of_slot", "meta", "disp_x"):
            assert torch.equal(bits(getattr(d, key).cpu()), bits(want[key])), key
        assert torch.equal(bits(d.disp_scale.cpu()), bits(want["disp_scale"]))
        assert torch.equal(bits(y.cpu()), bits(want["y"]))


def test_fp8_rows_within_stated_bound_at_full_size(gpu_device):
    """After dequantisation: |q*scale - x| <= max(2^-4 |x|, 2^-10 scale) for every element."""
    wl = C.generate_workload("fp8_dispatch")
    ata, d, y, (x, idx, w, rs) = gpu_run(wl, gpu_device)
    K = wl.cfg.experts_per_token
    R, H = d.disp_x.shape
    tok = (d.src_of_slot.long() // K)
    worst = 0.0
    for lo in range(0, R, 4096):  # chunks keep the f32 temporaries small
        hi = min(lo + 4096, R)
        q = d.disp_x[lo:hi].view(torch.float8_e4m3fn).float().view(hi - lo, H // 128, 128)
        sc = d.disp_scale[lo:hi].unsqueeze(-1)
        xs = x[tok[lo:hi]].float().view(hi - lo, H // 128, 128)
        bound = torch.maximum(xs.abs() * 2.0 ** -4, sc * 2.0 ** -10) * (1 + 1e-6)
        assert bool(((q * sc - xs).abs() <= bound).all())
        worst = max(worst, float(((q * sc - xs).abs() / bound).max()))
    assert worst <= 1.0


@pytest.mark.parametrize("name", ["dsv3_rank", "prefill_graph"])
def test_round_trip_and_checksums(gpu_device, name):
    """No oracle involved: permutation round trip and integer checksums at full size."""
    wl = C.generate_workload(name)
    cfg = wl.cfg
    K = cfg.experts_per_token
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    T = x.shape[0]
    # (1) unit stub: with one emulated rank the owner-rank factor is 1 for every expert
    ata = HipAllToAll(cfg, 0, 1, stub_kind=C.STUB_OWNER_RANK)
    hot = torch.randint(0, K, (T,), generator=torch.Generator().manual_seed(1))
    w1 = torch.nn.functional.one_hot(hot, K).float().to(gpu_device)
    for mode in (C.COMBINE_STRICT, C.COMBINE_F32):
        ata.combine_mode = mode
        y = ata.forward(x, idx, w1)
        assert torch.equal(y.float(), x.float())  # dispatch -> combine is the identity
    d = ata.dispatch(x, idx)
    # (2) routing invariants
    R = T * K
    assert int(d.counts.sum()) == R and int(d.offsets[-1]) == R
    assert torch.equal(torch.sort(d.slot_of_entry).values, torch.arange(R, dtype=torch.int32, device=gpu_device))
    assert torch.equal(d.src_of_slot[d.slot_of_entry.long()], torch.arange(R, dtype=torch.int32, device=gpu_device))
    seg_expert = torch.repeat_interleave(torch.arange(cfg.num_experts, device=gpu_device), d.counts.long())
    assert torch.equal(d.meta[:, 0].long(), seg_expert)  # rows are grouped by expert, in order
    assert torch.equal(d.meta[:, 0], idx.flatten()[d.src_of_slot.long()])
    inside = d.src_of_slot[1:] > d.src_of_slot[:-1]
    same = d.meta[1:, 0] == d.meta[:-1, 0]
    assert bool((inside | ~same).all())  # stable: entry ids ascend inside an expert's segment
    # (3) checksum of checksums: every token row appears K times among the dispatched rows
    row_sum = x.view(torch.int16).long().sum(dim=1)
    disp_sum = d.disp_x.view(torch.int16).long().sum(dim=1)
    assert torch.equal(disp_sum, row_sum[d.src_of_slot.long() // K])
    assert int(disp_sum.sum()) == K * int(row_sum.sum())
    # (4) idempotence: a second call reproduces every output bit for bit
    first = {k: getattr(d, k).clone() for k in ("counts", "offsets", "slot_of_entry", "src_of_slot", "meta", "disp_x")}
    d2 = ata.dispatch(x, idx)
    for k, v in first.items():
        assert torch.equal(bits(getattr(d2, k)), bits(v)), k


def test_buffers_beyond_four_gigabytes(gpu_device):
    """304 000 routed rows of 7168 columns: 2.2e9 elements, 4.4 GB per row buffer, so element and
    byte offsets leave the 32-bit range (and the table takes the three-launch routing).  No oracle:
    round trip with one-hot weights, routing invariants, checksum of checksums, fp8 bound on the
    last rows."""
    T, K, E, H = 38000, 8, 64, 7168
    cfg = C.MoEConfig(E, K, H, T + 1, torch.bfloat16, torch.bfloat16)
    g = torch.Generator(device=gpu_device).manual_seed(5)
    x = torch.randn(T, H, generator=g, device=gpu_device).to(torch.bfloat16)
    idx = torch.rand(T, E, generator=g, device=gpu_device).topk(K, dim=1).indices.to(torch.int32)  # distinct per token
    hot = torch.randint(0, K, (T,), generator=g, device=gpu_device)
    w1 = torch.nn.functional.one_hot(hot, K).float()
    ata = HipAllToAll(cfg, 0, 1, stub_kind=C.STUB_OWNER_RANK)  # one emulated rank: the stub factor is 1
    R = T * K
    assert R * H > 2 ** 31
    for mode in (C.COMBINE_STRICT, C.COMBINE_F32):
        ata.combine_mode = mode
        y = ata.forward(x, idx, w1)
        assert torch.equal(y.view(torch.int16), x.view(torch.int16))
    d = ata.last
    assert int(d.status.item()) == 0
    assert int(d.counts.sum()) == R and int(d.offsets[-1]) == R
    assert torch.equal(d.src_of_slot[d.slot_of_entry.long()], torch.arange(R, dtype=torch.int32, device=gpu_device))
    assert torch.equal(d.meta[:, 0], idx.flatten()[d.src_of_slot.long()])
    row_sum = x.view(torch.int16).sum(dim=1, dtype=torch.int64)
    disp_sum = d.disp_x.view(torch.int16).sum(dim=1, dtype=torch.int64)
    assert torch.equal(disp_sum, row_sum[d.src_of_slot.long() // K])
    ata.release_buffers()
    del y, d
    # fp8 dispatch of the same rows: the last 4096 rows of the buffer (beyond 2^31 bytes) obey the bound
    ata8 = HipAllToAll(cfg, 0, 1, stub_kind=C.STUB_OWNER_RANK, fp8_dispatch=True)
    d8 = ata8.dispatch(x, idx)
    torch.cuda.synchronize()
    rows = torch.arange(R - 4096, R, device=gpu_device)
    q = d8.disp_x[rows].view(torch.float8_e4m3fn).float().view(4096, H // 128, 128)
    sc = d8.disp_scale[rows].view(4096, H // 128, 1)
    xs = x[d8.src_of_slot[rows].long() // K].float().view(4096, H // 128, 128)
    bound = torch.maximum(xs.abs() * 2.0 ** -4, sc * 2.0 ** -10) * (1 + 1e-6)
    assert bool(((q * sc - xs).abs() <= bound).all())
    ata8.release_buffers()


def test_linearity_of_combine_in_the_weights(gpu_device):
    """f32-mode combine is linear in the weights up to rounding: y(w) + y(w') ~ y(w + w')."""
    wl = C.generate_workload("skew_world")
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, combine_mode=C.COMBINE_F32)
    w2 = torch.rand_like(w)
    ya = ata.forward(x, idx, w, rs).float().clone()
    yb = ata.forward(x, idx, w2, rs).float().clone()
    yc = ata.forward(x, idx, w + w2, rs).float()
    assert torch.allclose(ya + yb, yc, rtol=2e-2, atol=2e-2)


def test_graph_replay_matches_eager(gpu_device):
    """route -> dispatch -> stub -> combine captured once into a hipGraph; every replay, with
    eager work and synchronisation in between and fresh inputs each time, equals the eager
    result bit for bit."""
    wl = C.generate_workload("prefill_graph", tokens_scale=1 / 8)
    cfg = wl.cfg
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    ata = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind)
    sx, sidx, sw = x.clone(), idx.clone(), w.clone()  # static inputs of the graph
    ata.forward(sx, sidx, sw, rs)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ata.forward(sx, sidx, sw, rs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = ata.forward(sx, sidx, sw, rs)
    eager = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind)
    g = torch.Generator().manual_seed(3)
    T = x.shape[0]
    for it in range(4):
        perm = torch.randperm(T, generator=g).to(gpu_device)
        nx, nidx, nw = x[perm].contiguous(), idx[perm].contiguous(), w[perm].contiguous()
        want = eager.forward(nx, nidx, nw, rs).clone()  # eager work between replays
        torch.cuda.synchronize()
        sx.copy_(nx)
        sidx.copy_(nidx)
        sw.copy_(nw)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(y_static), bits(want)), f"replay {it}"
    want_cpu = V.run_world(cfg, [C.RankData(T, nidx.cpu(), nw.cpu(), nx.cpu())] +
                           [C.RankData.empty(cfg) for _ in range(7)], stub_kind=wl.stub_kind)["y"]
    assert torch.equal(bits(y_static.cpu()), bits(want_cpu))


@pytest.mark.parametrize("name,fuse_stub", [("prefill_graph", False), ("prefill_graph", True), ("fp8_dispatch", True)])
def test_full_size_graph_replay_against_the_oracle(gpu_device, name, fuse_stub):
    """The two streaming workloads at FULL size, the whole path captured once into a hipGraph: two
    replays with eager work, a synchronisation and fresh inputs between them; the second replay's
    dispatched rows, counts and output are compared bit for bit with the CPU oracle run on the same
    inputs (the first with an eager run of the library)."""
    wl = C.generate_workload(name)
    cfg, W = wl.cfg, wl.world_size
    fp8 = wl.fp8_dispatch
    x, idx, w, rs = concat_world(wl.world, gpu_device)
    ata = HipAllToAll(cfg, 0, W, stub_kind=wl.stub_kind, fp8_dispatch=fp8, fuse_stub=fuse_stub)
    sx, sidx, sw = x.clone(), idx.clone(), w.clone()  # static inputs of the graph
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ata.forward(sx, sidx, sw, rs)
        ata.forward(sx, sidx, sw, rs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = ata.forward(sx, sidx, sw, rs)
    rec = ata.last
    eager = HipAllToAll(cfg, 0, W, stub_kind=wl.stub_kind, fp8_dispatch=fp8, fuse_stub=fuse_stub)
    T = x.shape[0]
    # replay 1: the tokens in reverse order inside every rank's range stays a valid world only if whole
    # ranks are kept, so the permutation moves tokens inside their rank
    g = torch.Generator().manual_seed(5)
    starts = rs.cpu().tolist()
    perm = torch.cat([starts[r] + torch.randperm(starts[r + 1] - starts[r], generator=g) for r in range(W)])
    permd = perm.to(gpu_device)
    nx, nidx, nw = x[permd].contiguous(), idx[permd].contiguous(), w[permd].contiguous()
    want = eager.forward(nx, nidx, nw, rs).clone()  # eager work between capture and replay
    torch.cuda.synchronize()
    sx.copy_(nx)
    sidx.copy_(nidx)
    sw.copy_(nw)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(bits(y_static), bits(want)), "replay 1 differs from the eager run"
    # replay 2: the original inputs again, against the CPU oracle
    eager.forward(x, idx, w, rs)
    torch.cuda.synchronize()
    sx.copy_(x)
    sidx.copy_(idx)
    sw.copy_(w)
    graph.replay()
    torch.cuda.synchronize()
    o = V.run_world(cfg, wl.world, stub_kind=wl.stub_kind, fp8=bool(fp8))
    assert torch.equal(rec.counts.cpu(), o["counts"]) and torch.equal(rec.slot_of_entry.cpu(), o["slot_of_entry"])
    assert torch.equal(bits(rec.disp_x.cpu()), bits(o["disp_x"]))
    if fp8:
        assert torch.equal(rec.disp_scale.cpu(), o["disp_scale"])
    assert torch.equal(bits(y_static.cpu()), bits(o["y"]))
    ata.release_buffers()
    eager.release_buffers()
