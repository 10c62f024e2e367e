"""Host-side logic that needs no GPU: the contract module and the refusal to run on the CPU."""
import pytest
import torch

from kernel_amd import contract as C
from kernel_amd.all2all import HipAllToAll, concat_world


def test_generate_input_matches_reference_distribution():
    for spec in C.REFERENCE_TESTS + C.REFERENCE_BENCHMARKS:
        s = dict(spec)
        W = s.pop("world_size")
        cfg, rd, rank, world = C.generate_input(**s, rank=3, world_size=W)
        assert (rank, world) == (3, W)
        assert cfg.in_dtype == cfg.out_dtype == torch.float16  # all2all/reference.py:249-250
        assert 1 <= rd.num_tokens <= cfg.max_num_tokens - 1  # randint upper bound is exclusive
        assert rd.indices.dtype == torch.int32 and rd.indices.shape == (rd.num_tokens, cfg.experts_per_token)
        assert rd.weights.dtype == torch.float32 and float(rd.weights.min()) >= 0 and float(rd.weights.max()) < 1
        assert rd.x.shape == (rd.num_tokens, cfg.hidden_dim) and rd.x.dtype == torch.float16
        assert int(rd.indices.min()) >= 0 and int(rd.indices.max()) < cfg.num_experts
        srt = rd.indices.sort(dim=1).values
        assert bool((srt[:, 1:] != srt[:, :-1]).all())  # distinct experts per token


def test_generate_input_is_seeded_per_rank():
    a = C.generate_input(64, 6, 64, 8, 542, 1, 8)[1]
    b = C.generate_input(64, 6, 64, 8, 542, 1, 8)[1]
    c = C.generate_input(64, 6, 64, 8, 542, 2, 8)[1]
    assert torch.equal(a.x, b.x) and torch.equal(a.indices, b.indices)
    assert a.num_tokens != c.num_tokens or not torch.equal(a.x, c.x)


@pytest.mark.parametrize("name,T,E,K,H,W", [("tiny", 64, 8, 2, 256, 1), ("dsv3_rank", 256, 256, 8, 7168, 8),
                                            ("skew_world", 1024, 64, 6, 2048, 8)])
def test_named_workloads_have_their_shapes(name, T, E, K, H, W):
    wl = C.generate_workload(name)
    assert (wl.total_tokens, wl.cfg.num_experts, wl.cfg.experts_per_token, wl.cfg.hidden_dim, wl.world_size) == \
        (T, E, K, H, W)
    x, idx, w, rs = concat_world(wl.world)
    assert x.dtype == torch.bfloat16 and idx.dtype == torch.int32 and rs.tolist()[-1] == T
    assert torch.allclose(w.sum(-1), torch.ones(T), atol=1e-5)  # softmax weights
    srt = idx.sort(dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())
    again = C.generate_workload(name)
    assert torch.equal(again.world[0].x.view(torch.int16), wl.world[0].x.view(torch.int16))


def test_skewed_workload_is_skewed_but_within_capacity():
    wl = C.generate_workload("skew_world")
    idx = torch.cat([r.indices for r in wl.world])
    counts = torch.bincount(idx.flatten().long(), minlength=64)
    assert int(counts.max()) <= wl.total_tokens  # at most one row per token and expert
    assert int(counts[:8].sum()) > 3 * int(counts[-8:].sum())  # Zipf: low ids are hot


def test_scaled_workloads_and_outliers():
    wl = C.generate_workload("prefill_graph", tokens_scale=1 / 16)
    assert wl.total_tokens == 1024 and wl.graph
    mags = wl.world[0].x.float().abs().amax(dim=1)
    assert int((mags > 50).sum()) == 1024 // 100  # 1 % of the rows were multiplied by 100
    f8 = C.generate_workload("fp8_dispatch", tokens_scale=1 / 64)
    assert f8.fp8_dispatch and f8.total_tokens == 64


def test_algorithmic_bytes_match_the_published_table():
    ab = C.algorithmic_bytes(256, 8, 7168)
    assert ab["dispatch"] == ab["combine"] == 33_030_144  # 66.06 MB together
    ab3 = C.algorithmic_bytes(1024, 6, 2048)
    assert ab3["dispatch"] + ab3["combine"] == 58_720_256
    ab4 = C.algorithmic_bytes(4096, 8, 7168, fp8=True)
    assert round(ab4["dispatch"] / 1e6, 2) == 300.94 and round(ab4["combine"] / 1e6, 2) == 528.48
    ab5 = C.algorithmic_bytes(16384, 4, 4096)
    assert round((ab5["dispatch"] + ab5["combine"]) / 1e6, 2) == 1342.18
    assert round((ab5["dispatch"] + ab5["combine"] + ab5["stub"]) / 1e6, 2) == 2415.92


def test_product_path_refuses_cpu_tensors():
    wl = C.generate_workload("tiny")
    x, idx, w, rs = concat_world(wl.world)
    ata = HipAllToAll(wl.cfg, 0, 1)
    with pytest.raises(RuntimeError, match="GPU"):
        ata.dispatch(x, idx)
    from kernel_amd.submission import custom_kernel
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        custom_kernel((wl.cfg, wl.world[0], 0, 1))


def test_constructor_checks_expert_split():
    with pytest.raises(ValueError):
        HipAllToAll(C.MoEConfig(10, 2, 64, 8), 0, 4)


def test_custom_kernel_instance_follows_the_config_values(monkeypatch):
    """The memo of `custom_kernel` is keyed by the config's VALUES, read at every call: a config
    changed in place never meets an instance (and buffers) built for its old values, and the
    instance keeps a copy of the config it was built for."""
    from kernel_amd import submission as S

    made = []

    class Recorder:
        def __init__(self, cfg, rank, world_size, **kw):
            self.key = (cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim)
            made.append(self)

    monkeypatch.setattr(S, "HipAllToAll", Recorder)
    monkeypatch.setattr(S, "_instances", {})
    monkeypatch.setattr(S, "_last", [None, None])
    cfg = C.MoEConfig(64, 6, 2048, 32)
    a = S._instance(cfg, 0, 8, "cuda:0", 0, 0)
    assert S._instance(cfg, 0, 8, "cuda:0", 0, 0) is a and len(made) == 1
    cfg.hidden_dim = 4096  # in place
    b = S._instance(cfg, 0, 8, "cuda:0", 0, 0)
    assert b is not a and b.key == (64, 6, 4096)
    cfg.experts_per_token = 4
    c = S._instance(cfg, 0, 8, "cuda:0", 0, 0)
    assert c is not a and c is not b and c.key == (64, 4, 4096)
    cfg.hidden_dim, cfg.experts_per_token = 2048, 6  # back to the first values: the first instance again
    assert S._instance(cfg, 0, 8, "cuda:0", 0, 0) is a and len(made) == 3
    other = C.MoEConfig(64, 6, 2048, 32)  # an equal config in another object shares it
    assert S._instance(other, 0, 8, "cuda:0", 0, 0) is a
    assert S._instance(other, 1, 8, "cuda:0", 0, 0) is not a  # another rank does not


def test_host_object_keeps_its_own_copy_of_the_config():
    cfg = C.MoEConfig(64, 6, 2048, 32)
    ata = HipAllToAll(cfg, 0, 8)
    cfg.hidden_dim = 64
    assert ata.cfg.hidden_dim == 2048 and ata.cfg is not cfg
