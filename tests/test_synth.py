"""The device-side seeded generator (rocm_dev_amd.synth) is the oracle's counter generator: same integers, same
normals, same E4M3 codes - so a benchmark buffer and a test buffer with the same (seed, stream) hold the same data."""
import importlib.util
import os

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _synth():
    # loaded by path: importing the package would load libsgemm.so, which this CPU test does not need
    spec = importlib.util.spec_from_file_location("sg_synth", os.path.join(ROOT, "rocm_dev_amd", "synth.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_counter_stream_is_the_oracles(oracle):
    synth = _synth()
    for seed, stream in ((0, 1), (5, 3), (123456789, 1 << 33)):
        i = torch.tensor([0, 1, 2, 7, 1000, (1 << 40) + 3], dtype=torch.int64)
        got = synth.rng_u64(seed, stream, i).numpy().view(np.uint64)
        want = np.array([oracle._lib.orc_rng_u64(seed, stream, int(j)) for j in i], np.uint64)
        assert np.array_equal(got, want)


def test_normals_and_codes_are_the_oracles(oracle):
    synth = _synth()
    x = synth.normal_f32((48, 4096), 0, 1, device="cpu", chunk=50000).numpy()     # several chunks, a ragged last one
    y = oracle.normal_f32((48, 4096), 0, 1)
    assert (x == y).mean() > 0.99999 and np.abs(x - y).max() <= 2.0 ** -22
    a8, b8, s = synth.gemm_operands(8, 256, 512, seed=0, device="cpu")
    ra, rb, rs = oracle.make_gemm_operands(8, 256, 512, seed=0)
    assert (a8.numpy() == ra).mean() > 0.9999 and (b8.numpy() == rb).mean() > 0.9999
    assert abs(float(s) - float(rs)) <= 1e-6 * float(rs)


@pytest.mark.gpu
def test_device_generation_matches_the_oracle(oracle):
    synth = _synth()
    x = synth.normal_f32((64, 4096), 3, 2, device="cuda").cpu().numpy()
    y = oracle.normal_f32((64, 4096), 3, 2)
    assert (x == y).mean() > 0.9999 and np.abs(x - y).max() <= 2.0 ** -20
    a8, b8, s = synth.gemm_operands(8, 512, 1024, seed=0, device="cuda")
    ra, rb, rs = oracle.make_gemm_operands(8, 512, 1024, seed=0)
    assert (a8.cpu().numpy() == ra).mean() > 0.999 and (b8.cpu().numpy() == rb).mean() > 0.999
    assert abs(float(s) - float(rs)) <= 1e-6 * float(rs)
