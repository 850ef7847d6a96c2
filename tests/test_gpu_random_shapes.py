"""Seeded random shapes through every GEMM entry point against the oracle: m, n, k, row stride and - for the
tuned entry - records drawn from the tuner's search space that no hand-written case lists."""
import random

import numpy as np
import pytest
import torch

from gpu_util import GEMM_TOL, bits, dev, gemm_reference, rowcol_reference, scale_tensor, sparse_reference
from rocm_dev_amd import autotune

pytestmark = pytest.mark.gpu

KINDS = ["fast", "stride", "rowcol", "tuned", "sparse", "mid", "async"]


@pytest.fixture(scope="module")
def sg():
    import rocm_dev_amd
    rocm_dev_amd.tuning_clear()
    return rocm_dev_amd


def _shape(rng, kind):
    m = rng.randint(33, 300) if kind == "mid" else rng.choice([1, 2, 3, 5, 8, 9, 15, 16, 17, 24, 31, 32, rng.randint(1, 80)])
    n = 2 * rng.randint(1, 1500)
    if kind == "sparse":
        k = 512 * rng.randint(1, 8)
    elif kind == "mid":
        k = 128 * rng.randint(1, 40)
    elif kind == "async":
        k = 64 * rng.randint(1, 80)
    elif kind == "tuned" and rng.random() < 0.6:
        k = 256 * rng.randint(1, 20)
    else:
        k = 16 * rng.randint(1, 300)
    return m, n, k


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("case", range(8))
def test_random_shape(sg, oracle, kind, case):
    rng = random.Random(1000 * KINDS.index(kind) + case)
    m, n, k = _shape(rng, kind)
    seed = rng.randint(0, 1 << 20)
    D = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    if kind == "sparse":
        a8, vals, meta, _, scale = oracle.make_sparse24_operands(m, n, k, seed=seed)
        assert sg.sparse24_gemm(dev(a8), dev(vals), dev(meta), D, scale_tensor(scale)) == 0
        torch.cuda.synchronize()
        assert oracle.max_rel_err_bf16(bits(D), sparse_reference(oracle, a8, vals, meta, scale)) <= GEMM_TOL, (m, n, k)
        return
    if kind == "async":
        a8, b8, _ = oracle.make_gemm_operands(m, n, k, seed=seed)
        if case % 2:
            D = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        assert sg.async_gemm(dev(a8), dev(b8), D) == 0
        torch.cuda.synchronize()
        if case % 2:
            ref32 = oracle.gemm_f32(a8, b8, 1.0)
            assert np.abs(D.cpu().numpy() - ref32).max() <= 5e-4 * np.abs(ref32).max(), (m, n, k)
        else:
            assert oracle.max_rel_err_bf16(bits(D), gemm_reference(oracle, a8, b8, 1.0)) <= GEMM_TOL, (m, n, k)
        return
    pad = 16 * rng.randint(1, 3) if kind == "stride" else 0
    a8, b8, scale = oracle.make_gemm_operands(m, n, k, seed=seed, b_stride=(k + pad) if pad else None)
    A, S = dev(a8), scale_tensor(scale)
    B = dev(b8)[:, :k]
    dense = np.ascontiguousarray(b8[:, :k])
    if kind == "rowcol":
        rs = np.random.default_rng(seed).uniform(0.5, 2.0, size=m).astype(np.float32)
        cs = np.random.default_rng(seed + 1).uniform(0.5, 2.0, size=n).astype(np.float32)
        assert sg.skinny_gemm_rowcol(A, B, D, S, dev(rs), dev(cs)) == 0
        torch.cuda.synchronize()
        assert oracle.max_rel_err_bf16(bits(D), rowcol_reference(oracle, a8, dense, scale, rs, cs)) <= GEMM_TOL, (m, n, k)
        return
    ref = gemm_reference(oracle, a8, dense, scale)
    if kind != "tuned":
        assert sg.skinny_gemm_fastpath(A, B, D, S) == 0
        torch.cuda.synchronize()
        assert oracle.max_rel_err_bf16(bits(D), ref) <= GEMM_TOL, (m, n, k, pad)
        return
    space = autotune.search_space(m, n, k)
    ran = 0
    for rec in rng.sample(space, min(len(space), 20)):
        D.fill_(float("nan"))
        rc = sg.skinny_gemm_tuned(A, B, D, S, **rec)
        torch.cuda.synchronize()
        if rc != 0:
            assert rc in (3, 4, 6, 10), (rc, rec)          # rejected before launch
            continue
        ran += 1
        assert oracle.max_rel_err_bf16(bits(D), ref) <= GEMM_TOL, (m, n, k, rec)
    assert ran >= 1
