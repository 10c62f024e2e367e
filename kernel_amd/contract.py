"""Problem contract of the MoE all-to-all dispatch/combine path.

Mirrors the types a caller of ``custom_kernel(data)`` hands over
(all2all/reference.py:10-51, 237-253; all2all/task.py:8-17):

    data = (cfg: MoEConfig, rank_data, rank: int, world_size: int)

``rank_data`` exposes ``num_tokens``, ``indices[T,K] int32``, ``weights[T,K] f32``
and ``x[T,H] in_dtype``.  The reference draws them from a CUDA generator on
``cuda:{rank}``; here every draw comes from a CPU generator and is then moved to
the requested device, so a seed produces identical inputs with and without a GPU.

Two input families are produced:

* ``generate_input``       the reference's own distribution (fp16 by default,
                           ``num_tokens`` in [1, max_num_tokens), uniform weights,
                           distinct experts per token) -- reference.py:21-51.
* ``generate_workload(i)`` the five named workloads of this build (bf16, fixed
                           token counts, softmax weights, ``(1+e)/E`` expert stub).

A *world* is the list of the ``world_size`` per-rank records; a single-rank call
is a world in which every other rank holds zero tokens.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence, Tuple, TypedDict

import torch

META_DIM = 5  # [global_expert, src_rank, src_token, src_k, 0]   reference.py:56
FP8_BLOCK = 128  # columns per fp8 scale
FP8_MAX = 448.0  # largest finite e4m3fn

# expert stub flavours (reference.py:262 and the named workloads)
STUB_OWNER_RANK = 0  # y = x * (1 + owner_rank),  owner_rank = e // experts_per_rank
STUB_EXPERT_FRACTION = 1  # y = x * (1 + e) / num_experts

# combine arithmetic
COMBINE_STRICT = 0  # round to out_dtype after every add, ascending slot order
COMBINE_F32 = 1  # f32 accumulate in k order, one final rounding


@dataclasses.dataclass
class MoEConfig:
    """reference.py:10-17 -- same field names, same defaults."""

    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    in_dtype: torch.dtype = torch.float16
    out_dtype: torch.dtype = torch.float16


class TestSpec(TypedDict):
    """all2all/task.py:12-17."""

    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    seed: int


TestSpec.__test__ = False  # not a pytest class


class RankData:
    """Per-rank inputs; attribute names follow reference.py:21-51."""

    def __init__(self, num_tokens: int, indices: torch.Tensor, weights: torch.Tensor, x: torch.Tensor):
        self.num_tokens = int(num_tokens)
        self.indices = indices
        self.weights = weights
        self.x = x

    def to(self, device) -> "RankData":
        return RankData(self.num_tokens, self.indices.to(device), self.weights.to(device), self.x.to(device))

    @staticmethod
    def empty(cfg: MoEConfig, device="cpu") -> "RankData":
        K, H = cfg.experts_per_token, cfg.hidden_dim
        return RankData(
            0,
            torch.empty(0, K, dtype=torch.int32, device=device),
            torch.empty(0, K, dtype=torch.float32, device=device),
            torch.empty(0, H, dtype=cfg.in_dtype, device=device),
        )


def draw_rank_data(cfg: MoEConfig, rng: torch.Generator, device="cpu") -> RankData:
    """The reference's per-rank distribution (reference.py:21-51), CPU generator.

    Draw order is the reference's: num_tokens, one randperm per token, weights, x.
    ``randint(1, max_num_tokens)`` excludes its upper bound, hence
    ``1 <= num_tokens <= max_num_tokens - 1``.
    """
    T = int(torch.randint(1, cfg.max_num_tokens, [1], generator=rng).item())
    idx = torch.empty(T, cfg.experts_per_token, dtype=torch.int32)
    for t in range(T):
        idx[t] = torch.randperm(cfg.num_experts, generator=rng)[: cfg.experts_per_token]
    w = torch.rand(T, cfg.experts_per_token, dtype=torch.float32, generator=rng)
    x = torch.randn(T, cfg.hidden_dim, dtype=torch.float32, generator=rng).to(cfg.in_dtype)
    return RankData(T, idx, w, x).to(device)


def generate_input(
    num_experts: int,
    experts_per_token: int,
    hidden_dim: int,
    max_num_tokens: int,
    seed: int,
    rank: int,
    world_size: int,
    device="cpu",
    dtype: torch.dtype = torch.float16,
):
    """reference.py:237-253: ``(cfg, rank_data, rank, world_size)`` seeded ``seed + rank``."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed + rank)
    cfg = MoEConfig(num_experts, experts_per_token, hidden_dim, max_num_tokens, in_dtype=dtype, out_dtype=dtype)
    return cfg, draw_rank_data(cfg, gen, device), rank, world_size


def generate_world(num_experts, experts_per_token, hidden_dim, max_num_tokens, seed, world_size, device="cpu",
                   dtype: torch.dtype = torch.float16):
    """All ``world_size`` ranks of one reference test case: ``(cfg, [RankData]*W)``."""
    world = []
    cfg = None
    for r in range(world_size):
        cfg, rd, _, _ = generate_input(num_experts, experts_per_token, hidden_dim, max_num_tokens, seed, r,
                                       world_size, device, dtype)
        world.append(rd)
    return cfg, world


# Spec lists of all2all/task.yml:59-76 (the YAML itself is malformed, so they are
# written out here).  Every spec runs with world_size 8.
REFERENCE_TESTS: Tuple[dict, ...] = (
    dict(num_experts=8, experts_per_token=2, hidden_dim=6144, max_num_tokens=4, seed=1236, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=4, seed=1234, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=8, seed=542, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=16, seed=347, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=32, seed=51, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=64, seed=175, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=128, seed=534, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=64, seed=897, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=128, seed=4, world_size=8),
)
REFERENCE_BENCHMARKS: Tuple[dict, ...] = (
    dict(num_experts=8, experts_per_token=2, hidden_dim=6144, max_num_tokens=16, seed=6635, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=32, seed=1234, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=128, seed=51, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=256, seed=175, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=256, seed=4, world_size=8),
)


# ---------------------------------------------------------------------------
# Named workloads
# ---------------------------------------------------------------------------
@dataclasses.dataclass
class Workload:
    """One named workload: a whole emulated world resident in one process."""

    name: str
    cfg: MoEConfig
    world_size: int
    world: List[RankData]  # len == world_size; ranks without tokens hold empty tensors
    stub_kind: int = STUB_EXPERT_FRACTION
    fp8_dispatch: bool = False
    graph: bool = False

    @property
    def total_tokens(self) -> int:
        return sum(r.num_tokens for r in self.world)

    def to(self, device) -> "Workload":
        return dataclasses.replace(self, world=[r.to(device) for r in self.world])


_WORKLOADS = {
    # name: (W, E, K, H, tokens per source rank (list or int on rank 0 only), flavour)
    "tiny": dict(W=1, E=8, K=2, H=256, tokens=[64]),
    "dsv3_rank": dict(W=8, E=256, K=8, H=7168, tokens=[256] + [0] * 7),
    "skew_world": dict(W=8, E=64, K=6, H=2048, tokens=[128] * 8, zipf=1.2),
    "fp8_dispatch": dict(W=8, E=256, K=8, H=7168, tokens=[4096] + [0] * 7, fp8=True),
    "prefill_graph": dict(W=8, E=128, K=4, H=4096, tokens=[16384] + [0] * 7, outliers=0.01, graph=True),
}
WORKLOAD_NAMES = tuple(_WORKLOADS)


def generate_workload(name: str, seed: int = 0, device="cpu", dtype: torch.dtype = torch.bfloat16,
                      tokens_scale: float = 1.0) -> Workload:
    """Build one named workload from a CPU generator seeded ``seed``.

    Draw order (fixed, part of the contract): all activations ``randn(T,H)``, then
    the expert ids, then the routing logits ``randn(T,K)``; ``T`` is the token count
    of the whole world and the per-rank records are consecutive slices of it.

    * expert ids: uniform without replacement per token (one ``randperm(E)[:K]`` per
      token) or, for ``skew_world``, ``multinomial(p, K, replacement=False)`` with
      ``p(e) ~ (e+1)^-1.2``;
    * weights: ``softmax(logits, -1)`` in f32;
    * ``prefill_graph``: 1 % of the rows (``randperm(T)[:T//100]``) are multiplied by
      100 before the cast to ``dtype``.

    ``tokens_scale`` shrinks every rank's token count (tests use it to get a
    same-shaped but smaller case); 1.0 is the named size.
    """
    if isinstance(name, int):
        name = WORKLOAD_NAMES[name]
    spec = _WORKLOADS[name]
    W, E, K, H = spec["W"], spec["E"], spec["K"], spec["H"]
    tokens = [int(round(t * tokens_scale)) if t else 0 for t in spec["tokens"]]
    T = sum(tokens)
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    x32 = torch.randn(T, H, dtype=torch.float32, generator=g)
    if "zipf" in spec:
        p = (torch.arange(E, dtype=torch.float64) + 1.0).pow(-spec["zipf"])
        p = (p / p.sum()).to(torch.float32)
        idx = torch.multinomial(p.expand(T, E), K, replacement=False, generator=g).to(torch.int32)
    else:
        idx = torch.empty(T, K, dtype=torch.int32)
        for t in range(T):
            idx[t] = torch.randperm(E, generator=g)[:K]
    logits = torch.randn(T, K, dtype=torch.float32, generator=g)
    w = torch.softmax(logits, dim=-1)
    if "outliers" in spec:
        rows = torch.randperm(T, generator=g)[: int(T * spec["outliers"])]
        x32[rows] *= 100.0
    x = x32.to(dtype)
    del x32
    cfg = MoEConfig(E, K, H, max_num_tokens=max(max(tokens), 2), in_dtype=dtype, out_dtype=dtype)
    world, lo = [], 0
    for n in tokens:
        world.append(RankData(n, idx[lo:lo + n], w[lo:lo + n], x[lo:lo + n]).to(device))
        lo += n
    return Workload(name, cfg, W, world, STUB_EXPERT_FRACTION, bool(spec.get("fp8")), bool(spec.get("graph")))


# ---------------------------------------------------------------------------
# helpers shared by host code and tests
# ---------------------------------------------------------------------------
def world_of_single_rank(cfg: MoEConfig, rank_data, rank: int, world_size: int) -> List[RankData]:
    """A world in which only ``rank`` holds tokens."""
    dev = rank_data.x.device
    return [rank_data if r == rank else RankData.empty(cfg, dev) for r in range(world_size)]


def rank_starts(world: Sequence) -> List[int]:
    """``start[s]`` = index of rank ``s``'s first token in the concatenated world."""
    out = [0]
    for rd in world:
        out.append(out[-1] + int(rd.num_tokens))
    return out


def algorithmic_bytes(T: int, K: int, H: int, in_bytes: int = 2, out_bytes: int = 2, fp8: bool = False,
                      stub_folded: bool = False) -> dict:
    """HBM bytes the path must move.  Index, weight and meta traffic is left out.

    dispatch: read ``x`` once, write ``R`` rows (plus ``4*H/128`` scale bytes per row
    for fp8); combine: read ``R`` expert rows, write ``T`` rows; stub: read the
    dispatched rows, write ``R`` rows.  ``stub_folded``: the combine reads the dispatched rows
    themselves (fp8 bytes and scales for an fp8 dispatch) and there is no stub pass.
    """
    R = T * K
    b_d = 1 if fp8 else in_bytes
    S = 4 * H // FP8_BLOCK if fp8 else 0
    dispatch = T * H * in_bytes + R * (H * b_d + S)
    if stub_folded:
        return dict(dispatch=dispatch, combine=R * (H * b_d + S) + T * H * out_bytes, stub=0)
    combine = R * H * out_bytes + T * H * out_bytes
    stub = R * (H * b_d + S) + R * H * out_bytes
    return dict(dispatch=dispatch, combine=combine, stub=stub)
