"""The bench + verify driver (tests/driver/flash_driver, counterpart of the reference's main(), src/main.cu:38-251).

CPU: the binary exists, links against the library and the oracle, and rejects bad flags.
GPU: reference-compatible runs (U(0,10) fill with engine seed 26, verfiy with the 0.06 relative bound of
src/main.cu:224) must end with "finish,error:0" -- the line the reference prints for a correct kernel.
"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "driver", "flash_driver")


def _run(*args, timeout=120):
    return subprocess.run([DRIVER, *args], capture_output=True, text=True, timeout=timeout)


def test_driver_is_built_and_prints_usage():
    assert os.path.exists(DRIVER), "run `make -C tests/driver` (or __graft_entry__.build())"
    r = _run("--help")
    assert r.returncode == 2
    for flag in ("--batch", "--causal", "--window", "--alibi", "--dropout", "--splits", "--iters", "--fill", "--tol"):
        assert flag in r.stdout
    assert _run("--no-such-flag").returncode == 2
    assert _run("--seq", "0").returncode == 2


def test_driver_is_not_older_than_the_header():
    """A driver built against an older flash_params would hand the library a short struct; `make -q` says whether the
    binary is up to date with flash_driver.cpp and the public header.  (The binary also checks flash_params_size().)"""
    r = subprocess.run(["make", "-q", "-C", os.path.join(ROOT, "tests", "driver"), "flash_driver"], capture_output=True)
    assert r.returncode == 0, "tests/driver/flash_driver is stale: run `make -C tests/driver`"


def test_driver_and_python_harness_draw_the_same_normal_inputs(tmp_path):
    """`--fill normal --seed S` fills Q, K, V from the portable generator with seeds S, S + 1, S + 2: the same fp16 bits
    as tests/helpers.py draws for those seeds (no GPU needed: --dump-inputs stops before the first HIP call)."""
    import numpy as np
    import sys

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from oracle import cpu_oracle

    B, H, N, d = 2, 3, 37, 31
    n = B * H * N * d
    for seed in (1, 77):
        f = tmp_path / f"inputs_{seed}.bin"
        r = _run("--fill", "normal", "--seed", str(seed), "--batch", str(B), "--heads", str(H), "--seq", str(N),
                 "--head-dim", str(d), "--dump-inputs", str(f))
        assert r.returncode == 0, r.stderr
        bits = np.fromfile(f, dtype=np.uint16)
        assert bits.size == 3 * n
        for t in range(3):
            want = cpu_oracle.normal_f16((B, H, N, d), seed + t).view(np.uint16).ravel()
            assert np.array_equal(bits[t * n:(t + 1) * n], want), (seed, t)
    # the harness's device tensors are copies of exactly these arrays
    import inspect
    import helpers
    assert "cpu_oracle.normal_f16" in inspect.getsource(helpers.randn_f16_gpu)


def test_mfma_rate_probe_is_built():
    assert os.path.exists(os.path.join(ROOT, "tests", "driver", "mfma_rate")), "run `make -C tests/driver`"


@pytest.mark.gpu
def test_mfma_rate_probe_reports_its_rates():
    import json

    r = subprocess.run([os.path.join(ROOT, "tests", "driver", "mfma_rate")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    rates = json.loads(r.stdout.strip().splitlines()[-1])
    assert rates["unit"] == "TFLOP/s"
    # nothing can run above the published dense fp16 peak; random operands never run faster than zeros (+5 % noise)
    assert 100.0 < rates["random"] <= rates["zeros"] * 1.05 <= 2500.0 * 1.05
    # LDS reads and softmax arithmetic beside every MFMA can only cost
    assert 100.0 < rates["random_attention_mix"] <= rates["random"] * 1.05


def _check(out):
    assert re.search(r"^split_num: \d+$", out, re.M), out
    assert re.search(r"^kernel time: [0-9.]+ us$", out, re.M), out
    assert "Verify the result of kernel function" in out
    assert "===================start verfiy===================" in out
    m = re.search(r"==================finish,error:(\d+)==================", out)
    assert m, out
    return int(m.group(1))


@pytest.mark.gpu
@pytest.mark.parametrize(
    "args",
    [
        (),  # the reference's own configuration: B1 H8 N1021 d31, split count from the library's rule, ragged N and d
        ("--splits", "4"),  # the same in four splits, the count the reference's rule takes
        ("--causal",),
        ("--window", "128"),
        ("--alibi",),
        ("--causal", "--splits", "1"),
        ("--batch", "2", "--heads", "4", "--seq", "640", "--head-dim", "128", "--causal"),
        ("--batch", "2", "--heads", "4", "--seq", "512", "--head-dim", "64", "--fill", "normal", "--tol", "1e9"),
    ],
    ids=["reference_default", "reference_default_4_splits", "causal", "window128", "alibi", "causal_nosplit", "d128_causal", "normal_fill"],
)
def test_driver_reference_compatible_runs(args):
    r = _run("--iters", "5", *args)
    assert r.returncode == 0, r.stdout + r.stderr
    assert _check(r.stdout) == 0


@pytest.mark.gpu
def test_driver_dropout_skips_the_check():
    # src/main.cu:222: with dropout the CPU result cannot match, so the reference does not verify
    r = _run("--iters", "3", "--dropout", "0.1", "--seq", "256", "--head-dim", "64")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "kernel time" in r.stdout and "start verfiy" not in r.stdout
