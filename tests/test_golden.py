"""The oracle against vectors the reference's own PyTorchAllToAll produced (tests/golden/)."""
import pytest
import torch

from golden_io import GOLDEN_CASES, bits, golden_compact, load_golden
from oracle import all2all_literal as L
from oracle import all2all_vec as V


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_literal_oracle_matches_reference_vectors(name):
    cfg, world, expected = load_golden(name)
    disp = L.dispatch_world(cfg, world)
    ey = L.stub_world(cfg, disp, 0)
    ys = L.combine_world(cfg, world, disp, ey)
    E_l = cfg.num_experts // len(world)
    for d, exp in enumerate(expected):
        num, ex, em = disp[d]
        assert torch.equal(num, exp.expert_num_tokens)
        assert torch.equal(bits(torch.cat(ex, 0)), bits(exp.expert_x))
        assert torch.equal(torch.cat(em, 0), exp.expert_meta)
        assert torch.equal(bits(torch.cat(ey[d], 0)), bits(exp.expert_y))
        assert torch.equal(bits(ys[d][: world[d].num_tokens]), bits(exp.y))
        assert len(ex) == E_l


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_vectorised_oracle_matches_reference_vectors(name):
    cfg, world, expected = load_golden(name)
    g = golden_compact(cfg, expected)
    o = V.run_world(cfg, world, stub_kind=0)
    assert torch.equal(o["counts"], g["counts"])
    assert torch.equal(o["meta"], g["meta"])
    assert torch.equal(bits(o["disp_x"]), bits(g["disp_x"]))
    assert torch.equal(bits(o["expert_y"]), bits(g["expert_y"]))
    assert torch.equal(bits(o["y"]), bits(g["y"]))


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_f32_combine_is_within_reference_tolerance_of_vectors(name):
    cfg, world, expected = load_golden(name)
    g = golden_compact(cfg, expected)
    o = V.run_world(cfg, world, stub_kind=0, combine_mode=1)
    assert torch.allclose(o["y"].float(), g["y"].float(), rtol=1e-2, atol=1e-2)
