"""The oracle's GEMM and batch-sum restatements against the reference's OWN host loops, compiled from the
reference sources where they lie into oracle/_ref/libref_host.so (oracle/ref_host_loops.cpp, `make -C oracle ref`):
host_skinny_gemm (skinny_gemm/test.cu:7-39) and host_tiled_sum_reduce (tiled_sum_reduce/test.cu:5-26).

The reference decodes E4M3 *FNUZ* (exponent bias 8, no infinities, 0x80 = NaN) and this build's oracle decodes
OCP E4M3 (bias 7), so for every code other than 0x80, 0x7f and 0xff the reference's operand is exactly half
the oracle's.  Products are exact in both (fp16 holds any product of two FNUZ values, fp32 any product of two
OCP values), the K sums run in the same order in fp32, and scaling by a power of two is exact: the
reference's fp32 result must be the oracle's times 1/4, bit for bit.  A different loop order, a scale applied
inside the sum, or a rounding of the products would break the equality."""
import ctypes as C
import os

import numpy as np
import pytest

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libref_host.so")

pytestmark = pytest.mark.skipif(not os.path.exists(LIB), reason="oracle/_ref not built (needs the reference tree: make -C oracle ref)")


@pytest.fixture(scope="module")
def ref():
    lib = C.CDLL(LIB)
    vp = C.c_void_p
    lib.ref_host_skinny_gemm_f32.argtypes = [vp, vp, vp, C.c_float, C.c_int, C.c_int, C.c_int]
    lib.ref_host_skinny_gemm_f16.argtypes = [vp, vp, vp, C.c_float, C.c_int, C.c_int, C.c_int]
    lib.ref_host_tiled_sum_reduce.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int]
    return lib


def _codes(rng, shape):
    q = rng.integers(0, 256, size=shape, dtype=np.uint8)
    q[(q == 0x80) | ((q & 0x7F) == 0x7F)] = 0x38      # the three codes the two formats read differently
    return q


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (8, 64, 256), (5, 37, 640), (32, 48, 4096), (3, 2, 16)])
@pytest.mark.parametrize("scale", [1.0, 0.37, 2.0 ** -9, 1234.5])
def test_gemm_loop_matches_the_reference_host_loop(ref, oracle, m, n, k, scale):
    rng = np.random.default_rng(m * 1000 + k)
    A, B = _codes(rng, (m, k)), _codes(rng, (n, k))
    got = np.empty((m, n), np.float32)
    ref.ref_host_skinny_gemm_f32(_ptr(A), _ptr(B), _ptr(got), np.float32(scale), m, n, k)
    mine = oracle.gemm_f32(A, B, np.float32(scale))
    assert np.array_equal(got, mine * np.float32(0.25))
    # the reference's own output type: one more rounding, to fp16 (numpy's float16 cast rounds to nearest even too)
    half = np.empty((m, n), np.uint16)
    ref.ref_host_skinny_gemm_f16(_ptr(A), _ptr(B), _ptr(half), np.float32(scale), m, n, k)
    with np.errstate(over="ignore"):
        want = (mine * np.float32(0.25)).astype(np.float16).view(np.uint16)
    assert np.array_equal(half, want)


def test_the_formats_differ_where_expected(ref, oracle):
    """0x7f is 240 in FNUZ and NaN in OCP; 0x80 is NaN in FNUZ and -0 in OCP: the oracle follows OCP (what gfx950's
    MFMA decodes), so on these codes - and only on these - the two loops disagree."""
    A = np.full((1, 16), 0x38, np.uint8)           # 1.0 (OCP) / 0.5 (FNUZ)
    B = np.full((2, 16), 0x38, np.uint8)
    B[0, 3] = 0x7F
    B[1, 5] = 0x80
    got = np.empty((1, 2), np.float32)
    ref.ref_host_skinny_gemm_f32(_ptr(A), _ptr(B), _ptr(got), np.float32(1.0), 1, 2, 16)
    mine = oracle.gemm_f32(A, B, np.float32(1.0))
    assert got[0, 0] == 15 * 0.25 + 0.5 * 240.0 and np.isnan(mine[0, 0])
    assert np.isnan(got[0, 1]) and mine[0, 1] == 15.0


@pytest.mark.parametrize("b,m,n", [(1, 8, 64), (3, 8, 64), (7, 16, 128), (4, 5, 33)])
def test_batch_sum_matches_the_reference_host_loop(ref, oracle, b, m, n):
    rng = np.random.default_rng(b)
    A = (rng.standard_normal((b, m, n)) * 1e3).astype(np.float32)
    B = rng.standard_normal((b, m, n)).astype(np.float32)
    got = np.empty((m, n), np.float32)
    ref.ref_host_tiled_sum_reduce(_ptr(A), _ptr(B), _ptr(got), b, m, n)
    assert np.array_equal(got, oracle.tiled_sum_reduce(A, B))
