"""The one-GPU evaluation harness: tests-file syntax, seed mixing, statistics, log protocol and
exit codes of the reference's eval.py; CPU runs use the oracle as a stand-in kernel."""
import base64
import math
import os
import subprocess
import sys

import pytest
import torch

from kernel_amd import contract as C
from oracle import checker
from oracle import eval_harness as EH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def spec_line(s):
    return "; ".join(f"{k}: {v}" for k, v in s.items())


def test_tests_file_syntax_and_seed_mixing():
    cases = EH.parse_cases("num_experts: 8; experts_per_token: 2; hidden_dim: 64; max_num_tokens: 4; seed: 7; "
                           "world_size: 2\nmode: fast; seed: -3")
    assert cases[0].args == dict(num_experts=8, experts_per_token=2, hidden_dim=64, max_num_tokens=4, seed=7,
                                 world_size=2)
    assert cases[1].args == dict(mode="fast", seed=-3)
    assert cases[0].spec.startswith("num_experts: 8")
    # Cantor pairing: a + (a+b)(a+b+1)/2
    assert EH.mix_seed(4, 10) == 4 + 14 * 15 // 2 == 109
    mixed = EH.parse_cases("seed: 4; n: 1", secret_seed=10)
    assert mixed[0].args["seed"] == 109
    for bad in ("seed 4", "seed: 4; ; n: 1", "seed: 4.5", "seed: a1"):
        with pytest.raises(EH.HarnessError) as e:
            EH.parse_cases(bad)
        assert e.value.code == EH.EXIT_BAD_TESTS


def test_statistics_and_stopping_rule():
    st = EH.summarise([1.0, 2.0, 3.0, 4.0])
    assert (st.runs, st.mean, st.best, st.worst) == (4, 2.5, 1.0, 4.0)
    assert math.isclose(st.std, math.sqrt(5 / 3)) and math.isclose(st.err, st.std / 2)
    assert not EH.should_stop([5.0, 5.0], 1e9, 0)  # at least three runs
    assert EH.should_stop([5.0, 5.0, 5.0], 1e9, 0)  # relative error below 0.1 %
    assert not EH.should_stop([1.0, 9.0, 5.0], 1e9, 0)
    assert EH.should_stop([1.0, 9.0, 5.0], 10.0, 0)  # budget of the case used up
    assert EH.should_stop([1.0, 9.0, 5.0], 1e9, 121e9)  # two minutes of wall clock


def run_cli(args, env_extra, pass_fd=True):
    r, w = os.pipe()
    env = dict(os.environ, **env_extra)
    env.pop("POPCORN_SEED", None)
    env.update(env_extra)
    if pass_fd:
        env["POPCORN_FD"] = str(w)
    else:
        env.pop("POPCORN_FD", None)
    p = subprocess.run([sys.executable, "-m", "oracle.eval_harness", *args], cwd=ROOT, env=env,
                       pass_fds=(w,) if pass_fd else (), capture_output=True, text=True, timeout=600)
    os.close(w)
    with os.fdopen(r) as f:
        log = f.read()
    return p.returncode, log, p.stderr


def test_exit_codes_without_a_gpu(tmp_path):
    good = tmp_path / "t.txt"
    good.write_text("seed: 1")
    assert run_cli(["test", str(good)], {}, pass_fd=False)[0] == EH.EXIT_NO_FD
    assert run_cli(["test"], {})[0] == EH.EXIT_USAGE
    assert run_cli(["frobnicate", str(good)], {})[0] == EH.EXIT_USAGE
    assert run_cli(["test", str(tmp_path / "missing.txt")], {})[0] == EH.EXIT_BAD_TESTS
    bad = tmp_path / "bad.txt"
    bad.write_text("seed = 1")
    code, _, err = run_cli(["test", str(bad)], {})
    assert code == EH.EXIT_BAD_TESTS and "invalid test case" in err


class ListLog:
    def __init__(self):
        self.lines = []

    def log(self, k, v):
        self.lines.append(f"{k}: {v}")


SMALL = [dict(num_experts=8, experts_per_token=2, hidden_dim=64, max_num_tokens=4, seed=1236, world_size=4),
         dict(num_experts=16, experts_per_token=4, hidden_dim=32, max_num_tokens=6, seed=5, world_size=2)]


def test_modes_end_to_end_on_cpu_with_the_oracle_as_kernel():
    cases = EH.parse_cases("\n".join(spec_line(s) for s in SMALL))
    log = ListLog()
    h = EH.Harness(lambda data: checker.ref_kernel(data), "cpu", log)
    assert h.run_tests(cases) == 0
    assert log.lines[0] == "test-count: 2" and log.lines[-1] == "check: pass"
    assert "test.1.status: pass" in log.lines and f"test.0.spec: {spec_line(SMALL[0])}" in log.lines
    log.lines.clear()
    assert h.run_benchmarks(cases[:1]) == 0
    keys = [l.split(":")[0] for l in log.lines]
    assert keys == ["benchmark-count", "benchmark.0.spec"] + [f"benchmark.0.{f}" for f in
                                                             ("runs", "mean", "std", "err", "best", "worst")] + ["check"]
    assert 3 <= int(log.lines[2].split(": ")[1]) <= EH.MAX_REPEATS
    log.lines.clear()
    assert h.run_benchmarks(cases[:1], leaderboard=True) == 0 and log.lines[-1] == "check: pass"


def test_wrong_results_are_reported_and_fail_the_run():
    cases = EH.parse_cases(spec_line(SMALL[0]))
    log = ListLog()

    def wrong(data):
        return torch.zeros_like(checker.ref_kernel(data))

    h = EH.Harness(wrong, "cpu", log)
    assert h.run_tests(cases) == EH.EXIT_CHECK_FAILED
    assert "test.0.status: fail" in log.lines and log.lines[-1] == "check: fail"
    assert any(l.startswith("test.0.error: rank 0 - Output values mismatch") for l in log.lines)
    log.lines.clear()
    assert h.run_benchmarks(cases) == EH.EXIT_CHECK_FAILED and "benchmark.0.status: fail" in log.lines

    def wrong_dtype(data):
        return checker.ref_kernel(data).float()

    assert EH.Harness(wrong_dtype, "cpu", ListLog()).run_tests(cases) == EH.EXIT_CHECK_FAILED


@pytest.mark.gpu
def test_reference_test_specs_pass_on_the_gpu(gpu_device, tmp_path):
    """`test` mode over the reference's nine specs (task.yml:59-68), a secret seed mixed in."""
    f = tmp_path / "tests.txt"
    f.write_text("\n".join(spec_line(s) for s in C.REFERENCE_TESTS))
    code, log, err = run_cli(["test", str(f)], {"POPCORN_SEED": "4242"})
    assert code == 0, err + log
    lines = log.splitlines()
    assert lines[0] == "test-count: 9" and lines[-1] == "check: pass"
    assert sum(l.endswith(".status: pass") for l in lines) == 9


@pytest.mark.gpu
def test_benchmark_and_profile_modes_on_the_gpu(gpu_device, tmp_path):
    f = tmp_path / "bench.txt"
    f.write_text("\n".join(spec_line(s) for s in C.REFERENCE_BENCHMARKS[:2]))
    code, log, err = run_cli(["benchmark", str(f)], {})
    assert code == 0, err + log
    vals = dict(l.split(": ", 1) for l in log.splitlines())
    assert vals["benchmark-count"] == "2" and vals["check"] == "pass"
    assert float(vals["benchmark.1.best"]) <= float(vals["benchmark.1.mean"]) <= float(vals["benchmark.1.worst"])
    code, log, err = run_cli(["profile", str(f)], {})
    assert code == 0, err + log
    report = [l for l in log.splitlines() if l.startswith("benchmark.0.report: ")][0].split(": ", 1)[1]
    text = base64.b64decode(report, b"+*").decode()
    assert "forward_token" in text  # custom_kernel: dispatch and combine of a token in one launch at these sizes


@pytest.mark.gpu
def test_leaderboard_mode_on_the_gpu(gpu_device, tmp_path):
    """`leaderboard` mode (eval.py:340-346, 369-372 of the reference): the inputs are generated anew
    with seed + 13 for every repeat and EVERY run's output is checked, not only the first."""
    f = tmp_path / "bench.txt"
    f.write_text("\n".join(spec_line(s) for s in C.REFERENCE_BENCHMARKS[:2]))
    code, log, err = run_cli(["leaderboard", str(f)], {"POPCORN_SEED": "99"})
    assert code == 0, err + log
    vals = dict(l.split(": ", 1) for l in log.splitlines())
    assert vals["benchmark-count"] == "2" and vals["check"] == "pass"
    for i in (0, 1):
        assert int(vals[f"benchmark.{i}.runs"]) >= 3
        assert float(vals[f"benchmark.{i}.best"]) <= float(vals[f"benchmark.{i}.mean"])
