"""Host side of the MoE all-to-all: same roles as the reference's ``PyTorchAllToAll``
(all2all/reference.py:55-234), every step a HIP kernel behind the C ABI.

``HipAllToAll(cfg, rank, world_size)`` offers ``dispatch`` -> ``expert_stub`` ->
``combine``.  Differences from the reference that a caller sees:

* one GPU holds every destination rank, so ``dispatch`` returns the rows of ALL
  ``num_experts`` experts in one expert-major buffer (``Dispatched``): compact by default
  (rows back to back), or with ``padded=True`` exactly the reference's ``[E_l, max_recv, .]``
  buffers of every owner rank laid end to end; ``Dispatched.padded(owner)`` hands out the
  reference's ``(expert_num_tokens, expert_x, expert_meta)`` triple of one owner rank
  (views in the padded layout, a copy in the compact one);
* there is no process group: the three exchanges per phase are gone;
* ``combine`` writes ``out[:T]`` (it does not add into what ``out`` held before).

torch is used for device memory and the current stream only.
"""
from __future__ import annotations

import collections
import copy
import ctypes
import dataclasses
from typing import Optional, Sequence

import torch

from . import _lib
from .contract import (COMBINE_F32, COMBINE_STRICT, FP8_BLOCK, META_DIM, STUB_EXPERT_FRACTION, STUB_OWNER_RANK,
                       MoEConfig)

_ELEM = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _elem(dtype: torch.dtype) -> int:
    try:
        return _ELEM[dtype]
    except KeyError:
        raise TypeError(f"activations must be float16 or bfloat16, got {dtype}") from None


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device_index: Optional[int] = None) -> int:
    """Handle of torch's current stream on the current device (or the one named).  The raw query is
    one C call; the public one builds a Stream object and resolves the device twice (8 us of a 19 us
    forward)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device() if device_index is None else device_index)
    return torch.cuda.current_stream(device_index).cuda_stream


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: the HIP library is the only implementation")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


@dataclasses.dataclass
class Dispatched:
    """Result of ``dispatch``: the compact expert-major layout of the whole world."""

    cfg: MoEConfig
    world_size: int
    num_tokens: int  # T, tokens of all source ranks
    counts: torch.Tensor  # [E]   int32 rows per expert (= expert_num_tokens of every rank, concatenated)
    offsets: torch.Tensor  # [E+1] int32 first row of each expert
    slot_of_entry: torch.Tensor  # [R] int32
    src_of_slot: torch.Tensor  # [R] int32
    meta: torch.Tensor  # [R,5] int32: e, source rank, token in rank, k, 0
    disp_x: torch.Tensor  # [R,H] in_dtype, or uint8 e4m3fn bits for fp8 dispatch
    disp_scale: Optional[torch.Tensor] = None  # [R,H/128] f32 (fp8 only)
    # [1] int32, bits: 1 an expert id was out of range, 2 a padded segment overflowed.  It describes
    # the call that produced this record and stays readable until the next call on the same
    # ``HipAllToAll`` is enqueued (that call clears the word for the call after it: the host class
    # alternates between two buffer sets, and each call clears the other set's word)
    status: Optional[torch.Tensor] = None
    max_recv: int = 0  # > 0: padded layout, expert e owns rows [e*max_recv, (e+1)*max_recv)

    @property
    def num_rows(self) -> int:
        return self.slot_of_entry.numel()

    def padded(self, owner_rank: int, max_recv: Optional[int] = None):
        """``(expert_num_tokens, expert_x, expert_meta)`` of one owner rank in the reference's
        padded shape (all2all/reference.py:123-148); rows past the count are zero."""
        cfg, W = self.cfg, self.world_size
        E_l = cfg.num_experts // W
        lo, hi = owner_rank * E_l, (owner_rank + 1) * E_l
        if self.max_recv > 0 and max_recv in (None, self.max_recv):
            # already laid out that way: views, no copy (rows past the counts are uninitialised,
            # as they are in the reference)
            H = self.disp_x.shape[1]
            return (self.counts[lo:hi], self.disp_x.view(W, E_l, self.max_recv, H)[owner_rank],
                    self.meta.view(W, E_l, self.max_recv, META_DIM)[owner_rank])
        if self.max_recv > 0:
            raise ValueError("this record is padded with a different max_recv")
        max_recv = max_recv if max_recv is not None else cfg.max_num_tokens * W
        num = self.counts[lo:hi].clone()
        off = self.offsets[lo:hi + 1].tolist()
        ex = torch.zeros(E_l, max_recv, self.disp_x.shape[1], dtype=self.disp_x.dtype, device=self.disp_x.device)
        em = torch.zeros(E_l, max_recv, META_DIM, dtype=torch.int32, device=self.meta.device)
        for le in range(E_l):
            n = off[le + 1] - off[le]
            if n > max_recv:
                raise ValueError(f"expert {lo + le} holds {n} rows, more than max_recv={max_recv}")
            ex[le, :n] = self.disp_x[off[le]:off[le + 1]]
            em[le, :n] = self.meta[off[le]:off[le + 1]]
        return num, ex, em


class HipAllToAll:
    """MoE dispatch / expert stub / combine on one MI355X."""

    META_DIM = META_DIM
    MAX_CACHED_SHAPES = 8  # token counts whose buffers are kept (two sets each)

    def __init__(self, cfg: MoEConfig, rank: int, world_size: int, stub_kind: int = STUB_OWNER_RANK,
                 combine_mode: int = COMBINE_STRICT, fp8_dispatch: bool = False, fuse_route: bool = True,
                 fuse_stub: bool = False, padded: bool = False, max_recv: Optional[int] = None):
        if cfg.num_experts % world_size:
            raise ValueError("num_experts must be a multiple of world_size")
        # a copy: buffers and checks belong to the values the instance was built for, also when the
        # caller changes its config object in place afterwards
        self.cfg = cfg = copy.copy(cfg)
        self.rank = rank
        self.world_size = world_size
        self.num_local_experts = cfg.num_experts // world_size
        self.max_recv = max_recv if max_recv is not None else cfg.max_num_tokens * world_size
        self.padded = padded  # rows laid out as the reference's [E_l, max_recv, .] buffers of every owner rank
        self.stub_kind = stub_kind
        self.combine_mode = combine_mode
        # False: 16-bit rows; True: fp8 rows with f32 scales (amax / 448); "pow2": fp8 rows whose scales
        # are that rounded up to a power of two (what expert_gemm(..., scales_pow2=True) needs)
        if fp8_dispatch not in (False, True, "pow2"):
            raise ValueError("fp8_dispatch is False, True or 'pow2'")
        self.fp8_dispatch = fp8_dispatch
        self.fuse_route = fuse_route
        self.fuse_stub = fuse_stub
        self.lib = _lib.load()
        self._fused_max_rows = self.lib.moe_a2a_fused_max_rows()
        self._bufs = collections.OrderedDict()  # (T, device) -> two buffer sets; least recently used goes first

    # ---- buffers ---------------------------------------------------------------------
    def _buffers(self, T: int, device, advance: bool = False) -> dict:
        """Device buffers for T tokens, kept between calls.

        Two sets alternate (``advance=True`` at the start of a dispatch flips to the other
        one).  Rows a kernel has just read are slow to overwrite from the next kernel, so a
        step never writes what the step before it read; it also means the result of a call
        stays valid until the second-next call.
        """
        key = (T, device)
        ring = self._bufs.get(key)
        if ring is None:
            while len(self._bufs) >= self.MAX_CACHED_SHAPES:  # a caller with many token counts keeps the recent ones
                self._bufs.popitem(last=False)
            ring = self._bufs[key] = dict(sets=[None, None], cur=0)
        else:
            self._bufs.move_to_end(key)
        if advance:
            ring["cur"] ^= 1
        b = ring["sets"][ring["cur"]]
        if b is not None:
            return b
        # both sets of a new shape are allocated together, so that the second call with this shape
        # does not meet an allocation either
        for i in (0, 1):
            ring["sets"][i] = self._allocate(T, device)
        for i in (0, 1):  # a call on one set clears the status word of the other (see Dispatched.status)
            ring["sets"][i]["partner_status"] = ring["sets"][i ^ 1]["status"]
        return ring["sets"][ring["cur"]]

    def _allocate(self, T: int, device) -> dict:
        cfg = self.cfg
        K, H, E = cfg.experts_per_token, cfg.hidden_dim, cfg.num_experts
        R = T * K
        rows = E * self.max_recv if self.padded else R  # rows of the dispatched buffers
        i32 = dict(dtype=torch.int32, device=device)
        b = dict(
            counts=torch.empty(E, **i32),
            offsets=torch.empty(E + 1, **i32),
            slot_of_entry=torch.empty(R, **i32),
            src_of_slot=torch.empty(rows, **i32),
            meta=torch.empty(rows, META_DIM, **i32),
            status=torch.zeros(1, **i32),
            workspace=torch.empty(max(self.lib.moe_a2a_workspace_bytes(T, K, E), 256), dtype=torch.uint8,
                                  device=device),
            # the stub's output rows exist only where the stub is a launch of its own (expert_stub
            # allocates them on first use otherwise)
            expert_y=None if self.fuse_stub else torch.empty(rows, H, dtype=cfg.out_dtype, device=device),
            out=torch.empty(T, H, dtype=cfg.out_dtype, device=device),
        )
        if self.fp8_dispatch:
            b["disp_x"] = torch.empty(rows, H, dtype=torch.uint8, device=device)
            b["disp_scale"] = torch.empty(rows, H // FP8_BLOCK, dtype=torch.float32, device=device)
        else:
            b["disp_x"] = torch.empty(rows, H, dtype=cfg.in_dtype, device=device)
            b["disp_scale"] = None
        return b

    def release_buffers(self) -> None:
        self._bufs.clear()

    # ---- dispatch --------------------------------------------------------------------
    def dispatch(self, dp_x: torch.Tensor, indices: torch.Tensor,
                 rank_start: Optional[torch.Tensor] = None) -> Dispatched:
        """all2all/reference.py:68-148.

        ``dp_x[T,H]`` and ``indices[T,K]`` are the tokens of this rank, or of the whole world
        concatenated in rank order when ``rank_start[W+1]`` (int32, on the GPU) is given.
        """
        cfg = self.cfg
        _require_gpu(dp_x, "dp_x")
        _require_gpu(indices, "indices")
        if indices.dtype != torch.int32:
            raise TypeError("indices must be int32")
        T, H = dp_x.shape
        K, E, W = cfg.experts_per_token, cfg.num_experts, self.world_size
        if H != cfg.hidden_dim or tuple(indices.shape) != (T, K) or dp_x.dtype != cfg.in_dtype:
            raise ValueError("dp_x / indices do not match the MoEConfig")
        if rank_start is not None:
            _require_gpu(rank_start, "rank_start")
            if rank_start.dtype != torch.int32 or rank_start.numel() != W + 1:
                raise ValueError("rank_start must be int32[world_size + 1]")
        b = self._buffers(T, dp_x.device, advance=True)
        b["status"].zero_()  # the phase-by-phase entry points only ever set bits: the record describes this call
        lib, st = self.lib, _stream()
        pad = self.max_recv if self.padded else 0
        route_out = (_ptr(b["counts"]), _ptr(b["offsets"]), _ptr(b["slot_of_entry"]), _ptr(b["src_of_slot"]),
                     _ptr(b["meta"]), _ptr(b["status"]))
        if self.fuse_route and not self.fp8_dispatch and (
                self.fuse_route == "always" and 0 < T * K <= self._fused_max_rows
                or self.lib.moe_a2a_fused_ok(T, K, H)):
            _lib.check(lib.moe_a2a_route_dispatch(_ptr(dp_x), _ptr(indices), _ptr(rank_start), self.rank, T, K, E, W,
                                                  H, pad, *route_out, _ptr(b["disp_x"]), st), "moe_a2a_route_dispatch")
        else:
            _lib.check(lib.moe_a2a_route(_ptr(indices), _ptr(rank_start), self.rank, T, K, E, W, pad, *route_out,
                                         _ptr(b["workspace"]), b["workspace"].numel(), st), "moe_a2a_route")
            if self.fp8_dispatch:
                _lib.check(lib.moe_a2a_dispatch_fp8(_ptr(dp_x), _elem(cfg.in_dtype), _ptr(b["slot_of_entry"]),
                                                    _ptr(b["disp_x"]), _ptr(b["disp_scale"]), T, K, H,
                                                    _lib.FP8_SCALE_POW2 if self.fp8_dispatch == "pow2"
                                                    else _lib.FP8_SCALE_F32, st),
                           "moe_a2a_dispatch_fp8")
            else:
                _lib.check(lib.moe_a2a_dispatch(_ptr(dp_x), _ptr(b["slot_of_entry"]), _ptr(b["disp_x"]), T, K, H, st),
                           "moe_a2a_dispatch")
        return Dispatched(cfg, W, T, b["counts"], b["offsets"], b["slot_of_entry"], b["src_of_slot"], b["meta"],
                          b["disp_x"], b["disp_scale"], b["status"], pad)

    # ---- expert stub -----------------------------------------------------------------
    def expert_stub(self, d: Dispatched) -> torch.Tensor:
        """all2all/reference.py:262 on the compact rows -> ``expert_y[R,H]`` out_dtype."""
        cfg = self.cfg
        R, H = d.num_rows, d.disp_x.shape[1]
        b = self._buffers(d.num_tokens, d.disp_x.device)
        if b["expert_y"] is None:
            b["expert_y"] = torch.empty(d.disp_x.shape[0], H, dtype=cfg.out_dtype, device=d.disp_x.device)
        y = b["expert_y"]
        in_type = _lib.BF16 if d.disp_scale is not None else _elem(d.disp_x.dtype)
        rows = d.slot_of_entry if d.max_recv > 0 else None  # padded: only rows that hold an entry
        _lib.check(self.lib.moe_a2a_stub(_ptr(d.disp_x), _ptr(d.disp_scale), _ptr(d.meta), _ptr(rows), in_type,
                                         _elem(cfg.out_dtype), self.stub_kind, cfg.num_experts, self.world_size,
                                         _ptr(y), R, H, _stream()), "moe_a2a_stub")
        return y

    def expert_gemm(self, d: Dispatched, weights: torch.Tensor, out: Optional[torch.Tensor] = None,
                    w_scale: Optional[torch.Tensor] = None, scales_pow2: bool = False) -> torch.Tensor:
        """Real expert compute in place of the stub: ``y[rows of e] = disp_x[rows of e] @ weights[e].T``
        for every expert, on the matrix cores (f32 accumulation, one rounding to ``out_dtype``).

        ``weights[E, N, H]`` of ``out_dtype``; returns ``y[rows, N]`` with the row layout of the
        dispatched buffer (rows that hold no entry are not written).  ``N == H`` feeds ``combine``.
        16-bit dispatched rows must have the weights' type; fp8 dispatched rows (``d.disp_scale``
        set) are dequantised inside the kernel, each element rounded once to the weights' type.

        Block-quantised weights: ``weights`` as e4m3fn bits (``uint8`` or ``float8_e4m3fn``) with
        ``w_scale[E, N/128, H/128]`` f32, the format of DeepSeek-V3 checkpoints; ``N % 128 == 0``.

        ``scales_pow2``: the caller states that every scale of both operands is a power of two
        (rows from ``fp8_dispatch="pow2"``, weights quantised that way); the library then hands the
        scales' exponents to the matrix instruction (``moe_a2a_expert_gemm_mx8``).  Only the exponent
        field of a scale is used there, so the statement has to be true.
        """
        cfg = self.cfg
        _require_gpu(weights, "weights")
        rows, H = d.disp_x.shape
        E = cfg.num_experts
        quant = w_scale is not None
        want_w = (torch.uint8, torch.float8_e4m3fn) if quant else (cfg.out_dtype,)
        if weights.dim() != 3 or weights.shape[0] != E or weights.shape[2] != H or weights.dtype not in want_w \
                or not weights.is_contiguous():
            raise ValueError("weights must be out_dtype[E, N, H] (or e4m3fn bits with w_scale), contiguous")
        fp8 = d.disp_scale is not None
        if not fp8 and cfg.out_dtype != d.disp_x.dtype:
            raise ValueError("expert_gemm keeps the element type of 16-bit dispatched rows")
        N = weights.shape[1]
        if quant:
            _require_gpu(w_scale, "w_scale")
            if H % 128 or N % 128 or tuple(w_scale.shape) != (E, N // 128, H // 128) or w_scale.dtype != torch.float32 \
                    or not w_scale.is_contiguous():
                raise ValueError("w_scale must be float32[E, N/128, H/128], contiguous, with N and H multiples of 128")
        if out is None:
            out = torch.empty(rows, N, dtype=cfg.out_dtype, device=weights.device)
        elif tuple(out.shape) != (rows, N) or out.dtype != cfg.out_dtype or not out.is_contiguous():
            raise ValueError("out must be out_dtype[rows, N], contiguous")
        common = (_ptr(d.offsets), _ptr(out), d.num_rows, E, H, N, d.max_recv, _elem(cfg.out_dtype), _stream())
        if scales_pow2:
            if not (quant and fp8):
                raise ValueError("scales_pow2 needs fp8 dispatched rows and block-quantised weights")
            _lib.check(self.lib.moe_a2a_expert_gemm_mx8(_ptr(d.disp_x), _ptr(d.disp_scale), _ptr(weights),
                                                        _ptr(w_scale), *common), "moe_a2a_expert_gemm_mx8")
        elif quant:
            _lib.check(self.lib.moe_a2a_expert_gemm_q8(_ptr(d.disp_x), _ptr(d.disp_scale) if fp8 else None,
                                                       _ptr(weights), _ptr(w_scale), *common),
                       "moe_a2a_expert_gemm_q8")
        elif fp8:
            _lib.check(self.lib.moe_a2a_expert_gemm_fp8(_ptr(d.disp_x), _ptr(d.disp_scale), _ptr(weights), *common),
                       "moe_a2a_expert_gemm_fp8")
        else:
            _lib.check(self.lib.moe_a2a_expert_gemm(_ptr(d.disp_x), _ptr(weights), *common), "moe_a2a_expert_gemm")
        return out

    # ---- combine ---------------------------------------------------------------------
    def combine(self, out_tokens: Optional[torch.Tensor], weights: torch.Tensor, d: Dispatched,
                expert_y: torch.Tensor) -> torch.Tensor:
        """all2all/reference.py:151-234: weighted sum of each token's K expert rows into
        ``out_tokens[:T]`` (allocated here when None)."""
        cfg = self.cfg
        T, K, H = d.num_tokens, cfg.experts_per_token, cfg.hidden_dim
        _require_gpu(weights, "weights")
        _require_gpu(expert_y, "expert_y")
        if weights.dtype != torch.float32 or tuple(weights.shape) != (T, K):
            raise ValueError("weights must be float32[T,K]")
        if expert_y.dtype != cfg.out_dtype or tuple(expert_y.shape) != (d.disp_x.shape[0], H):
            raise ValueError("expert_y must be out_dtype[rows,H] with the rows of the dispatched buffer")
        if out_tokens is None:
            out_tokens = self._buffers(T, expert_y.device)["out"]
        else:
            _require_gpu(out_tokens, "out_tokens")
            if out_tokens.dtype != cfg.out_dtype or out_tokens.shape[0] < T or out_tokens.shape[1] != H:
                raise ValueError("out_tokens must be out_dtype[>=T,H]")
        _lib.check(self.lib.moe_a2a_combine(_ptr(expert_y), _ptr(weights), _ptr(d.slot_of_entry), self.combine_mode,
                                            _elem(cfg.out_dtype), _ptr(out_tokens), T, K, H, _stream()),
                   "moe_a2a_combine")
        return out_tokens

    def stub_combine(self, out_tokens: Optional[torch.Tensor], weights: torch.Tensor, indices: torch.Tensor,
                     d: Dispatched) -> torch.Tensor:
        """Expert stub folded into the combine (same results, no ``expert_y`` buffer)."""
        cfg = self.cfg
        T, K, H = d.num_tokens, cfg.experts_per_token, cfg.hidden_dim
        _require_gpu(weights, "weights")
        _require_gpu(indices, "indices")
        if out_tokens is None:
            out_tokens = self._buffers(T, weights.device)["out"]
        in_type = _lib.BF16 if d.disp_scale is not None else _elem(d.disp_x.dtype)
        _lib.check(self.lib.moe_a2a_stub_combine(_ptr(d.disp_x), _ptr(d.disp_scale), _ptr(indices), _ptr(weights),
                                                 _ptr(d.slot_of_entry), self.combine_mode, in_type,
                                                 _elem(cfg.out_dtype), self.stub_kind, cfg.num_experts,
                                                 self.world_size, _ptr(out_tokens), T, K, H, _stream()),
                   "moe_a2a_stub_combine")
        return out_tokens

    # ---- whole path ------------------------------------------------------------------
    def _forward_args(self, b: dict, x, indices, weights, rank_start, stream: int) -> tuple:
        cfg = self.cfg
        T, H = x.shape
        fuse_route = 2 if self.fuse_route == "always" else int(bool(self.fuse_route))
        return (_ptr(x), _ptr(indices), _ptr(weights), _ptr(rank_start), self.rank, T, cfg.experts_per_token,
                cfg.num_experts, self.world_size, H, self.max_recv if self.padded else 0, _elem(cfg.in_dtype), _elem(cfg.out_dtype), 2 if self.fp8_dispatch == "pow2" else int(self.fp8_dispatch),
                self.stub_kind, self.combine_mode, fuse_route, int(self.fuse_stub), _ptr(b["counts"]),
                _ptr(b["offsets"]), _ptr(b["slot_of_entry"]), _ptr(b["src_of_slot"]), _ptr(b["meta"]),
                _ptr(b["status"]), _ptr(b["disp_x"]), _ptr(b["disp_scale"]), _ptr(b["expert_y"]), _ptr(b["out"]),
                _ptr(b["workspace"]), b["workspace"].numel(), stream, _ptr(b["partner_status"]))

    def _check_inputs(self, x, indices, weights, rank_start) -> None:
        cfg = self.cfg
        if not (x.is_cuda and indices.is_cuda and weights.is_cuda and x.is_contiguous() and indices.is_contiguous()
                and weights.is_contiguous()):
            for name, t in (("x", x), ("indices", indices), ("weights", weights)):
                _require_gpu(t, name)  # raises, naming the tensor
        T, H = x.shape
        K = cfg.experts_per_token
        si, sw = indices.shape, weights.shape
        if (H != cfg.hidden_dim or len(si) != 2 or si[0] != T or si[1] != K or len(sw) != 2 or sw[0] != T or sw[1] != K
                or x.dtype != cfg.in_dtype or indices.dtype != torch.int32 or weights.dtype != torch.float32):
            raise ValueError("x / indices / weights do not match the MoEConfig")
        if rank_start is not None:
            _require_gpu(rank_start, "rank_start")
            if rank_start.dtype != torch.int32 or rank_start.numel() != self.world_size + 1:
                raise ValueError("rank_start must be int32[world_size + 1]")

    def _record(self, b: dict, T: int) -> Dispatched:
        return Dispatched(self.cfg, self.world_size, T, b["counts"], b["offsets"], b["slot_of_entry"],
                          b["src_of_slot"], b["meta"], b["disp_x"], b["disp_scale"], b["status"],
                          self.max_recv if self.padded else 0)

    def forward(self, x: torch.Tensor, indices: torch.Tensor, weights: torch.Tensor,
                rank_start: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                check_status: bool = False) -> torch.Tensor:
        """dispatch -> stub -> combine in one library call; returns ``y[T,H]``: ``out`` if given
        (``out_dtype[>=T,H]``, contiguous), else a buffer the second-next call reuses.
        ``self.last`` holds the ``Dispatched`` record of the call.

        ``check_status=True`` reads the call's status word back (this synchronises) and raises where
        the reference would: ``IndexError`` for an expert id outside ``[0, num_experts)`` (the
        reference indexes ``token_map[dst_rank]``, all2all/reference.py:81-86), ``RuntimeError`` for
        a padded segment with more than ``max_recv`` rows (reference.py:140-146 would write past
        ``expert_x[local_eid]``).  Without it such ids are clamped and the bits stay in
        ``self.last.status`` until the next call."""
        cfg = self.cfg
        T = x.shape[0]
        if T == 0:
            return torch.empty(0, cfg.hidden_dim, dtype=cfg.out_dtype, device=x.device)
        self._check_inputs(x, indices, weights, rank_start)
        if out is not None:
            _require_gpu(out, "out")
            if out.dtype != cfg.out_dtype or out.dim() != 2 or out.shape[0] < T or out.shape[1] != cfg.hidden_dim:
                raise ValueError("out must be out_dtype[>=T,H]")
        b = self._buffers(T, x.device, advance=True)
        # the argument struct of a buffer set is built once; a call patches the caller's pointers in
        a = b.get("_args")
        if a is None:
            a = b["_args"] = _lib.ForwardArgs(*self._forward_args(b, x, indices, weights, rank_start, 0))
            b["_argp"] = ctypes.pointer(a)
            b["_record"] = self._record(b, T)
        a.x, a.indices, a.weights = x.data_ptr(), indices.data_ptr(), weights.data_ptr()
        a.out = b["out"].data_ptr() if out is None else out.data_ptr()
        # what rarely changes between two calls is written only when it does (a field of a foreign
        # struct costs a quarter of a microsecond to set)
        rs = None if rank_start is None else rank_start.data_ptr()
        st = _stream(x.device.index)
        switches = (rs, st, self.stub_kind, self.combine_mode, self.fuse_route, self.fuse_stub)
        if b.get("_switches") != switches:
            b["_switches"] = switches
            a.rank_start, a.stream = rs, st
            a.stub_kind, a.combine_mode = self.stub_kind, self.combine_mode
            a.fuse_route = 2 if self.fuse_route == "always" else int(bool(self.fuse_route))
            a.fuse_stub = int(self.fuse_stub)
        rc = self.lib.moe_a2a_forward_packed(b["_argp"])
        if rc:
            raise _lib.MoeA2AError(rc, "moe_a2a_forward")
        self.last = b["_record"]
        if check_status:
            self.raise_on_status(b["status"])
        return b["out"] if out is None else out

    @staticmethod
    def raise_on_status(status: torch.Tensor) -> None:
        """Read a status word back (synchronises); clear it and raise if a bit is set."""
        bits = int(status.item())
        if not bits:
            return
        status.zero_()
        if bits & _lib.STATUS_BAD_EXPERT:
            raise IndexError("an expert id lies outside [0, num_experts): the reference fails on it at "
                             "token_map[dst_rank] (all2all/reference.py:81-86); the kernels clamped it")
        raise RuntimeError("a padded expert segment holds more than max_recv rows (status bit "
                           f"{_lib.STATUS_OVERFLOW}): the extra entries were folded onto its last row")

    def plan(self, x: torch.Tensor, indices: torch.Tensor, weights: torch.Tensor,
             rank_start: Optional[torch.Tensor] = None, stream: Optional[torch.cuda.Stream] = None):
        """Pre-marshalled ``forward`` for a serving loop that reuses its input tensors.

        Checks shapes once and returns ``step()``: every call launches the whole path on
        ``stream`` (default: the stream that is current NOW -- under hipGraph capture pass the
        capturing stream), reading whatever the input tensors hold at that moment, and returns
        ``y[T,H]``; calls alternate between the two buffer sets.  The per-call host cost is one
        foreign call.
        """
        if x.shape[0] == 0:
            raise ValueError("plan() needs at least one token")
        self._check_inputs(x, indices, weights, rank_start)
        T, dev = x.shape[0], x.device
        st = stream.cuda_stream if stream is not None else _stream()
        sets = [self._buffers(T, dev, advance=True), self._buffers(T, dev, advance=True)]
        args = [self._forward_args(b, x, indices, weights, rank_start, st) for b in sets]
        outs = [b["out"] for b in sets]
        records = [self._record(b, T) for b in sets]
        fn = self.lib.moe_a2a_forward_packed
        structs = [_lib.ForwardArgs(*a) for a in args]
        ptrs = [ctypes.pointer(st_) for st_ in structs]
        keep = (x, indices, weights, rank_start, structs)  # the raw pointers above must stay valid
        state = [0]

        def step() -> torch.Tensor:
            i = state[0]
            state[0] = i ^ 1
            rc = fn(ptrs[i])
            if rc:
                raise _lib.MoeA2AError(rc, "moe_a2a_forward")
            self.last = records[i]
            return outs[i]

        step.inputs = keep
        step.args = args  # the two argument tuples of moe_a2a_forward, for callers with their own loop
        return step


def concat_world(world: Sequence, device=None):
    """Concatenate per-rank records in rank order -> x, indices, weights, rank_start (int32)."""
    x = torch.cat([rd.x for rd in world], 0)
    idx = torch.cat([rd.indices for rd in world], 0)
    w = torch.cat([rd.weights for rd in world], 0)
    starts = [0]
    for rd in world:
        starts.append(starts[-1] + int(rd.num_tokens))
    rs = torch.tensor(starts, dtype=torch.int32)
    if device is not None:
        x, idx, w, rs = x.to(device), idx.to(device), w.to(device), rs.to(device)
    else:
        rs = rs.to(x.device)
    return x.contiguous(), idx.contiguous(), w.contiguous(), rs
