"""The process / stdout protocol of the reference's drivers (the process-level boundary):
parsing rules on the CPU, the real mains on the GPU."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "harness"))
import driver  # noqa: E402


def test_bench_stream_parses_with_the_reference_slicing():
    # what bench.cu prints: every value carries a spare trailing zero
    warm = ["10.0000", "11.0000", "12.0000", "13.0000", "14.0000"]
    timed = ["5.1230", "5.4560", "6.7890"]
    stream = ", ".join(warm) + ", End of warmup, " + ", ".join(timed) + ", "
    bench_ts, warmup_ts = driver.parse_bench_output(stream)
    assert sorted(bench_ts) == [5.123, 5.456, 6.789]        # the last value lost only its spare zero
    assert warmup_ts == [13.0, 14.0]                         # the first three fields are dropped
    s = driver.stats(bench_ts)
    assert abs(s["median"] - 5.456) < 1e-12 and abs(s["mean"] - (5.123 + 5.456 + 6.789) / 3) < 1e-12


def test_test_stream_parses_json_and_bare_nan():
    assert driver.parse_test_output('{"max_delta": 0.03125, "total_delta": 12.5}') == (0.03125, 12.5)
    mx, tot = driver.parse_test_output('{"max_delta": nan, "total_delta": nan}')
    assert mx != mx and tot != tot


def test_skip_rules():
    base = {"B_LANES_": 1, "OPS_": 4, "A_PRODUCERS_": 0, "B_PRODUCERS_": 0, "CONSUMERS_": 1, "QSIZE_": 8, "SK_": 1, "OP_M_": 8}
    assert not driver.skip(base)
    assert driver.skip(dict(base, A_PRODUCERS_=8, B_PRODUCERS_=8, CONSUMERS_=1))            # 17 waves
    assert driver.skip(dict(base, A_PRODUCERS_=1, B_PRODUCERS_=4, CONSUMERS_=3, QSIZE_=2))  # qsize < consumers
    assert not driver.skip(dict(base, A_PRODUCERS_=1, B_PRODUCERS_=4, CONSUMERS_=3, QSIZE_=6, B_LANES_=2))
    assert driver.skip(dict(base, B_LANES_=4, CONSUMERS_=8, QSIZE_=8))                      # LDS over budget


def test_core_rewrite_touches_only_define_lines(tmp_path):
    core = os.path.join(ROOT, "tests", "harness", "projects", "skinny_gemm", "core.cu")
    original = open(core).readlines()
    for name in ("B_LANES_", "QSIZE_", "OP_M_", "OPS_", "A_PRODUCERS_", "B_PRODUCERS_", "CONSUMERS_", "SK_"):
        assert any(line.startswith("#define %s " % name) for line in original), name
    p = tmp_path / "core.cu"
    driver.rewrite_core(str(p), original, {"QSIZE_": 4, "SK_": 2})
    new = p.read_text().splitlines(keepends=True)
    changed = [(a, b) for a, b in zip(original, new) if a != b]
    assert [b for _, b in changed] == ["#define QSIZE_ 4\n", "#define SK_ 2\n"]


def test_mains_compile_for_gfx950():
    """Single translation unit per main, kernels included as source, for every project the reference's drivers name
    with -p: skinny_gemm, the three async_gemm_* ancestors, tiled_sum_reduce and its _async variant."""
    for exe in driver.compile_all():
        assert os.path.exists(exe)
    for p in driver.PROJECTS:
        for f in ("test.cu", "bench.cu"):
            assert os.path.exists(os.path.join(ROOT, "tests", "harness", "projects", p, f)), (p, f)


@pytest.mark.gpu
def test_protocol_end_to_end():
    data = driver.main(["bench", "-p", "skinny_gemm", "-a", "8 512 4096", "-t", "2"])
    worst = float(data["max_deltas"].split()[0])
    assert worst <= 0.05                      # bf16 outputs of magnitude ~1: one ulp is 2^-8
    assert 0.5 < data["median"] < 200.0       # microseconds per GEMM


@pytest.mark.gpu
@pytest.mark.parametrize("project", ["tiled_sum_reduce", "tiled_sum_reduce_async"])
def test_protocol_tiled_sum_reduce(project):
    """argv = b m n (tiled_sum_reduce/test.cu:28-33); the batch sum is bit-identical to the host loop, so both deltas are 0."""
    data = driver.main(["bench", "-p", project, "-a", "5 256 2050", "-t", "2"])
    assert data["max_deltas"].split()[0] == "0.0000" and data["sum_deltas"].split()[0] == "0.0000"
    assert 0.5 < data["median"] < 500.0


@pytest.mark.gpu
@pytest.mark.parametrize("project,args", [("async_gemm_sparse", "8 512 1024"), ("async_gemm_blanes", "16 1000 2048"),
                                          ("async_gemm_16x16x64", "24 256 512")])
def test_protocol_async_gemm(project, args):
    """argv = m n k (async_gemm_sparse/test.cu:44-48); fp32 output of U[-1, 1) operands against the host's sequential
    fp32 sum: what is left is summation order and the instruction's in-run cut, far below 1e-2 at these sizes."""
    data = driver.main(["bench", "-p", project, "-a", args, "-t", "2"])
    assert float(data["max_deltas"].split()[0]) <= 1e-2
    assert 0.5 < data["median"] < 500.0
