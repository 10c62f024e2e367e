"""TEST INFRASTRUCTURE -- one-GPU counterpart of the reference's evaluation harness (eval.py).

    POPCORN_FD=<fd> [POPCORN_SEED=<n>] python -m oracle.eval_harness <mode> <tests-file>

Modes, tests-file syntax, log protocol and exit codes follow eval.py so that the same tests
files and log readers work:

  tests file   one case per line, ``key: value; key: value`` (eval.py:60-93); the public seed
               of a case is mixed with the secret POPCORN_SEED by Cantor pairing (:49-57)
  log          ``key: value`` lines on the inherited descriptor POPCORN_FD (:25-40):
               test-count, test.i.spec/status/error, benchmark-count,
               benchmark.i.{spec,runs,mean,std,err,best,worst} in ns, check: pass|fail
  modes        test | benchmark | leaderboard | profile  (:527-574)
  exit codes   0 ok, 2 usage or unknown mode, 111 no POPCORN_FD, 112 a check failed,
               113 unreadable or malformed tests file

What differs, because one GPU holds the whole emulated world: there is no process pool and no
process group; the ``world_size`` ranks of a case run one after the other on ``cuda:0`` (each is
an independent call, because a rank's output depends on its own tokens only), and a case's
duration is the slowest rank's, which is what the reference's barrier-to-barrier wall clock
measures when the ranks run side by side.  The result of every rank is checked with the CPU
oracle (``oracle.checker.check_implementation``); the cache flush before a timed call overwrites
1 GiB, four times the Infinity Cache (the reference's 256 MB would fit in it).  ``profile``
reports the library's per-kernel launch timer instead of torch.profiler.
"""
from __future__ import annotations

import base64
import dataclasses
import math
import os
import re
import sys
import time
from typing import Callable, List, Optional

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

EXIT_USAGE, EXIT_NO_FD, EXIT_CHECK_FAILED, EXIT_BAD_TESTS = 2, 111, 112, 113
MAX_REPEATS = 100
WALL_LIMIT_NS = 120e9


class HarnessError(Exception):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


@dataclasses.dataclass
class Case:
    spec: str
    args: dict


@dataclasses.dataclass
class Stats:
    runs: int
    mean: float
    std: float
    err: float
    best: float
    worst: float


def mix_seed(public: int, secret: int) -> int:
    """Cantor pairing of the public per-case seed with the secret one (eval.py:49-57)."""
    s = public + secret
    return public + s * (s + 1) // 2


_PAIR = re.compile(r"\s*([a-zA-Z_]+):\s*([a-zA-Z]+|[+-]?[0-9]+)\s*")


def parse_cases(text: str, secret_seed: Optional[int] = None) -> List[Case]:
    cases = []
    for line in text.splitlines():
        args = {}
        for part in line.split(";"):
            m = _PAIR.fullmatch(part)
            if m is None:
                raise HarnessError(EXIT_BAD_TESTS, f"invalid test case: '{line}': '{part}'")
            key, val = m.group(1), m.group(2)
            args[key] = int(val) if re.fullmatch(r"[+-]?[0-9]+", val) else val
        if secret_seed is not None and "seed" in args:
            args["seed"] = mix_seed(args["seed"], secret_seed)
        cases.append(Case(line, args))
    return cases


def read_cases(path: str, secret_seed: Optional[int]) -> List[Case]:
    try:
        with open(path) as f:
            text = f.read()
    except OSError as e:
        raise HarnessError(EXIT_BAD_TESTS, f"could not open tests file '{path}': {e}") from None
    return parse_cases(text, secret_seed)


def summarise(durations_ns: List[float]) -> Stats:
    """runs / mean / sample std / standard error / best / worst (eval.py:106-124)."""
    n = len(durations_ns)
    mean = sum(durations_ns) / n
    var = sum((d - mean) ** 2 for d in durations_ns) / (n - 1) if n > 1 else 0.0
    std = math.sqrt(var)
    return Stats(n, mean, std, std / math.sqrt(n), float(min(durations_ns)), float(max(durations_ns)))


def should_stop(durations_ns: List[float], max_time_ns: float, wall_ns: float) -> bool:
    """After at least three runs: relative error of the mean below 0.1 %, or the time budget
    of the case used up, or two minutes of wall clock (eval.py:298-306, 383-391)."""
    if len(durations_ns) < 3:
        return False
    st = summarise(durations_ns)
    return st.err / st.mean < 0.001 or st.mean * st.runs > max_time_ns or wall_ns > WALL_LIMIT_NS


class KeyValueLog:
    def __init__(self, fd: int):
        self.file = os.fdopen(fd, "w")

    def log(self, key, value) -> None:
        print(f"{key}: {value}", file=self.file, flush=True)

    def close(self) -> None:
        self.file.close()


class Harness:
    """Runs cases against ``kernel(data)``.  ``device`` is where inputs are generated; the GPU
    run uses ``cuda:0``, the CPU tests pass a stand-in kernel and ``cpu``."""

    def __init__(self, kernel: Callable, device: str = "cuda:0", log: Optional[KeyValueLog] = None):
        import torch

        from kernel_amd import contract
        from oracle import checker

        self.torch = torch
        self.contract = contract
        self.checker = checker
        self.kernel = kernel
        self.device = torch.device(device)
        self.on_gpu = self.device.type == "cuda"
        self.out = log
        self._flush = None

    # -- plumbing ---------------------------------------------------------------------------
    def _sync(self) -> None:
        if self.on_gpu:
            self.torch.cuda.synchronize()

    def _flush_caches(self) -> None:
        if not self.on_gpu:
            return
        if self._flush is None:
            self._flush = self.torch.empty(1 << 30, dtype=self.torch.uint8, device=self.device)
        self._flush.fill_(42)

    def _inputs(self, case: Case, rank: int):
        a = dict(case.args)
        world = a.pop("world_size", 1)
        return self.contract.generate_input(**a, rank=rank, world_size=world, device=self.device)

    def _clone(self, data):
        cfg, rd, rank, world = data
        return cfg, self.contract.RankData(rd.num_tokens, rd.indices.clone(), rd.weights.clone(), rd.x.clone()), \
            rank, world

    def _log(self, key, value) -> None:
        if self.out is not None:
            self.out.log(key, value)

    # -- one case ---------------------------------------------------------------------------
    def check_case(self, case: Case):
        """Every rank of the case once; ``(ok, message)`` like eval.py:187-205."""
        world = case.args.get("world_size", 1)
        errors = []
        for rank in range(world):
            data = self._inputs(case, rank)
            self._sync()
            out = self.kernel(self._clone(data))
            self._sync()
            ok, msg = self.checker.check_implementation(data, out)
            if not ok:
                errors.append(f"rank {rank} - {msg}")
        return not errors, "\n".join(errors)

    def time_case(self, case: Case, recheck: bool, max_repeats: int, max_time_ns: float):
        """Stats of the case, or an error string (eval.py:311-410)."""
        world = case.args.get("world_size", 1)
        case = Case(case.spec, dict(case.args))
        datas = [self._inputs(case, r) for r in range(world)]
        for data in datas:  # one obligatory correctness check
            ok, msg = self.checker.check_implementation(data, self.kernel(self._clone(data)))
            if not ok:
                return msg
        durations: List[float] = []
        t_begin = time.perf_counter_ns()
        for _ in range(max_repeats):
            if recheck:  # fresh inputs every repeat (leaderboard mode)
                if "seed" in case.args:
                    case.args["seed"] += 13
                datas = [self._inputs(case, r) for r in range(world)]
            slowest = 0.0
            for data in datas:
                self._flush_caches()
                self._sync()
                t0 = time.perf_counter_ns()
                out = self.kernel(self._clone(data))  # the input clone is inside the timed region
                self._sync()
                slowest = max(slowest, float(time.perf_counter_ns() - t0))
                if recheck:
                    ok, msg = self.checker.check_implementation(data, out)
                    if not ok:
                        return msg
                del out
            durations.append(slowest)
            if should_stop(durations, max_time_ns, time.perf_counter_ns() - t_begin):
                break
        return summarise(durations)

    def profile_case(self, case: Case) -> str:
        """Per-kernel GPU durations of rank 0's call, from the library's launch timer."""
        import ctypes

        from kernel_amd import _lib

        lib = _lib.load()
        data = self._inputs(case, 0)
        self.kernel(self._clone(data))
        self._sync()
        cap = 64
        lib.moe_a2a_timer_begin(cap)
        self.kernel(self._clone(data))
        self._sync()
        ids, us = (ctypes.c_int * cap)(), (ctypes.c_float * cap)()
        n = lib.moe_a2a_timer_end(ids, us, cap)
        rows = [f"{lib.moe_a2a_kernel_name(ids[i]).decode():<20s} {us[i]:10.2f} us" for i in range(n)]
        return "\n".join(["kernel                 GPU time"] + rows)

    # -- modes ------------------------------------------------------------------------------
    def run_tests(self, cases: List[Case]) -> int:
        self._log("test-count", len(cases))
        passed = True
        for i, case in enumerate(cases):
            self._log(f"test.{i}.spec", case.spec)
            ok, msg = self.check_case(case)
            self._log(f"test.{i}.status", "pass" if ok else "fail")
            if not ok:
                self._log(f"test.{i}.error", msg)
                passed = False
        self._log("check", "pass" if passed else "fail")
        return 0 if passed else EXIT_CHECK_FAILED

    def run_benchmarks(self, cases: List[Case], leaderboard: bool = False) -> int:
        self.time_case(cases[0], False, MAX_REPEATS, 1e7 if leaderboard else 1e8)  # warm-up
        self._log("benchmark-count", len(cases))
        passed = True
        for i, case in enumerate(cases):
            self._log(f"benchmark.{i}.spec", case.spec)
            result = self.time_case(case, leaderboard, MAX_REPEATS, 30e9 if leaderboard else 10e9)
            if isinstance(result, Stats):
                for f in dataclasses.fields(Stats):
                    self._log(f"benchmark.{i}.{f.name}", getattr(result, f.name))
            else:
                passed = False
                self._log(f"benchmark.{i}.status", "fail")
                self._log(f"benchmark.{i}.error", result)
                if leaderboard:
                    break
        self._log("check", "pass" if passed else "fail")
        return 0 if passed else EXIT_CHECK_FAILED

    def run_profiles(self, cases: List[Case]) -> int:
        self._log("benchmark-count", len(cases))
        for i, case in enumerate(cases):
            self._log(f"benchmark.{i}.spec", case.spec)
            report = self.profile_case(case)
            self._log(f"benchmark.{i}.report", base64.b64encode(report.encode("utf-8"), b"+*").decode("utf-8"))
        self._log("check", "pass")
        return 0


def main(argv: Optional[List[str]] = None) -> int:
    argv = sys.argv if argv is None else argv
    fd = os.getenv("POPCORN_FD")
    if not fd:
        return EXIT_NO_FD
    if len(argv) < 3:
        return EXIT_USAGE
    mode = argv[1]
    if mode not in ("test", "benchmark", "leaderboard", "profile"):
        return EXIT_USAGE
    seed = os.getenv("POPCORN_SEED")
    os.environ.pop("POPCORN_SEED", None)
    try:
        cases = read_cases(argv[2], int(seed) if seed else None)
    except HarnessError as e:
        print(str(e), file=sys.stderr)
        return e.code
    from kernel_amd.submission import custom_kernel

    log = KeyValueLog(int(fd))
    try:
        h = Harness(custom_kernel, "cuda:0", log)
        if mode == "test":
            return h.run_tests(cases)
        if mode == "profile":
            return h.run_profiles(cases)
        return h.run_benchmarks(cases, leaderboard=(mode == "leaderboard"))
    finally:
        log.close()


if __name__ == "__main__":
    sys.exit(main())
