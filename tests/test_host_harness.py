"""The C++ host harnesses (tests/host): the reference's test/test_correctness.cu and
test/benchmark.cu flows -- pack() on the host, hipMalloc/hipMemcpy, linear_vN_launch or the
C ABI, CPU comparison / event timing -- as plain host programs linked against the library."""
import re
import subprocess
from pathlib import Path

import pytest

HOST = Path(__file__).resolve().parent / "host"
BIN = HOST / "bin"


def _binary(name: str) -> Path:
    exe = BIN / name
    if not exe.exists():  # built by __graft_entry__.build(); build here only if nothing is there
        subprocess.run(["make", "-C", str(HOST)], check=True, capture_output=True, text=True)
    assert exe.exists(), exe
    return exe


def test_harness_binaries_link_against_the_library():
    for name in ("correctness", "benchmark", "vendor_compare"):  # (stream_ceiling does not use the library)
        out = subprocess.run(["ldd", str(_binary(name))], check=True, capture_output=True, text=True).stdout
        assert "libint4linear.so" in out and "not found" not in out, out


def test_harness_usage_errors_without_a_device():
    r = subprocess.run([str(_binary("correctness")), "--entry", "v99", "16x16x128"], capture_output=True, text=True)
    assert r.returncode == 2
    r = subprocess.run([str(_binary("benchmark")), "--kernel", "nope"], capture_output=True, text=True)
    assert r.returncode == 2


@pytest.mark.gpu
@pytest.mark.parametrize("entry", ["v21", "v20", "v11", "v10", "v2", "v1", "v0", "c"])
def test_correctness_harness_every_entry_point(gpu, entry):
    r = subprocess.run([str(_binary("correctness")), "--entry", entry, "--seed", "7",
                        "300x520x512", "16x1024x1024", "33x70x72"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("TEST PASSED!") == 3 and "FAILED" not in r.stdout


@pytest.mark.gpu
def test_correctness_harness_benchmark_configs(gpu):
    # cfg1 in full; one large square and one long-K shape on sampled rows; decode shapes with
    # normal(0, 2) activations.
    r = subprocess.run([str(_binary("correctness")), "--threads", "16", "1024x1024x1024"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "TEST PASSED!" in r.stdout, r.stdout + r.stderr
    r = subprocess.run([str(_binary("correctness")), "--threads", "16", "--rows", "24", "4096x4096x4096", "2048x2048x4096"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.count("TEST PASSED!") == 2, r.stdout + r.stderr
    r = subprocess.run([str(_binary("correctness")), "--threads", "16", "--dist", "normal",
                        "16x14336x4096", "1x4096x14336", "64x4096x4096"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.count("TEST PASSED!") == 3, r.stdout + r.stderr


@pytest.mark.gpu
def test_benchmark_harness_reports_tops(gpu):
    r = subprocess.run([str(_binary("benchmark")), "--iters", "5", "--warmup", "2", "2048x2048x2048", "16x4096x4096"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = re.findall(r"\[PERF\] (\d+)x(\d+)x(\d+) kernel=(\w+) epilogue=\w+ median ([\d.]+) ms .* ([\d.]+) TOPS", r.stdout)
    assert len(lines) == 2 and all(float(l[5]) > 0 for l in lines), r.stdout


@pytest.mark.gpu
def test_vendor_comparison_agrees_bit_for_bit(gpu):
    """hipBLASLt's int8 GEMM on the widened operands is an independent implementation of the
    same product: the harness exits non-zero if any output differs."""
    r = subprocess.run([str(_binary("vendor_compare")), "--iters", "3", "--warmup", "1",
                        "1024x1024x1024", "300x520x512", "16x4096x4096", "2048x2048x2048"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = [l for l in r.stdout.splitlines() if l.startswith("[VENDOR]")]
    assert len(lines) == 4, r.stdout
    for l in lines:
        assert "results identical" in l or "offers no int8" in l, l


def test_stream_ceiling_usage_error_without_a_device():
    r = subprocess.run([str(_binary("stream_ceiling"))], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr
    r = subprocess.run([str(_binary("stream_ceiling")), "16x4096x100"], capture_output=True, text=True)
    assert r.returncode == 2


@pytest.mark.gpu
def test_stream_ceiling_reports_a_rate(gpu):
    r = subprocess.run([str(_binary("stream_ceiling")), "--steps", "50", "16x4096x4096", "16x14336x4096"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    rates = re.findall(r"\[CEILING\] \d+x\d+x\d+ ([\d.]+) us ([\d.]+) GB/s", r.stdout)
    assert len(rates) == 2 and all(0.5 < float(us) < 100 and float(gbs) > 100 for us, gbs in rates), r.stdout


def test_mfma_ceiling_usage_error_without_a_device():
    r = subprocess.run([str(_binary("mfma_ceiling")), "--bogus"], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
def test_mfma_ceiling_reports_rates(gpu):
    r = subprocess.run([str(_binary("mfma_ceiling")), "--iters", "500"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    rows = re.findall(r"\[MFMA\] (int8|fp6|bf6) .*? ([\d.]+) TOPS +([\d.]+) GHz", r.stdout)
    assert len(rows) == 12 and all(float(t) > 500 and 0.5 < float(g) < 3.0 for _, t, g in rows), r.stdout


def test_fp6_ablation_usage_error_without_a_device():
    r = subprocess.run([str(_binary("fp6_ablation")), "--bogus"], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
def test_fp6_ablation_reports_every_build(gpu):
    """The FP6 kernel with parts left out: every build runs and reports a time (a small shape;
    the figures that matter come from 8192^3, and a bound on them here would only measure how
    busy the box is)."""
    r = subprocess.run([str(_binary("fp6_ablation")), "2048x2048x4096", "--iters", "10", "--warmup", "5"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    rows = re.findall(r"\[ABLATION\] (.*?) +([\d.]+) us +([\d.]+) TOPS", r.stdout)
    assert len(rows) == 16 and rows[0][0] == "whole kernel", r.stdout
    assert r.stdout.count("[SPREAD]") == 3, r.stdout
    assert all(float(us) > 0 and float(tops) > 0 for _, us, tops in rows), r.stdout


def test_int8_ablation_usage_error_without_a_device():
    r = subprocess.run([str(_binary("int8_ablation")), "--bogus"], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
def test_int8_ablation_reports_every_build(gpu):
    """The int8 kernel with parts left out: every build runs and reports a time."""
    r = subprocess.run([str(_binary("int8_ablation")), "2048x2048x4096", "--iters", "10", "--warmup", "5"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    rows = re.findall(r"\[ABLATION\] (.*?) +([\d.]+) us +([\d.]+) TOPS", r.stdout)
    assert len(rows) == 13 and rows[0][0] == "whole kernel", r.stdout
    assert all(float(us) > 0 and float(tops) > 0 for _, us, tops in rows), r.stdout
    assert r.stdout.count("[SPREAD]") == 2, r.stdout
