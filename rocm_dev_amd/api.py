"""Host-side mirror of the reference's launcher and torch-binding surface.

Reference interfaces mirrored (paths below the reference's projects/ directory):
  skinny_gemm(...)            skinny_gemm/skinny_gemm_caller.cu:20-43
  skinny_gemm_fastpath(...)   skinny_gemm/skinny_gemm_caller.cu:343-346
  HFRK_skinny_gemm            skinny_gemm/skinny_gemm_binding.cu:64-100
  async_gemm(...)             async_gemm_sparse/sparse_k.cu:45-69
  tiled_sum_reduce(...)       tiled_sum_reduce/src.cu:52-73, tiled_sum_reduce_async/src.cu:179-200 (lds_queue=True)
Every function returns the integer return code of the C ABI (0 = success), as the
reference's launchers do; ``check=True`` raises SgError instead.  Tensors are torch CUDA
tensors used purely as device buffers: fp8 operands are uint8 or float8_e4m3fn, outputs
bfloat16 (or float32 for async_gemm), and everything is enqueued on torch's current stream.
"""
import ctypes as C
import enum

import torch

from ._lib import lib


class SgReturnCode(enum.IntEnum):
    SUCCESS = 0
    M_ABOVE_WARPTILE_M = 1
    N_NOT_EVEN = 2
    K_NOT_DIVISIBLE_BY_WARPTILE_K = 3
    TOO_MANY_WARPS = 4
    QSIZE_TOO_SMALL = 5
    INVALID_CONFIG = 6
    LAUNCH_FAILED = 7
    BAD_ALIGNMENT = 8
    BAD_ARGUMENT = 9
    WORKSPACE_TOO_SMALL = 10
    NO_DEVICE = 11


class SgError(RuntimeError):
    def __init__(self, code):
        self.code = int(code)
        super().__init__("libsgemm: %s (code %d)" % (strerror(code), code))


def strerror(code):
    return lib.sg_strerror(int(code)).decode()


def _done(rc, check):
    if check and rc != 0:
        raise SgError(rc)
    return rc


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dev(t, *dtypes):
    if not t.is_cuda:
        raise ValueError("expected a CUDA (HIP) tensor")
    if dtypes and t.dtype not in dtypes:
        raise ValueError("expected dtype in %s, got %s" % (dtypes, t.dtype))
    return t.data_ptr()


_FP8 = (torch.uint8, torch.float8_e4m3fn)


def skinny_gemm(A, B, D, scale_tensor, split_k, A_producers, B_producers, consumers, b_lanes, qsize, op_m, ops,
                b_stride=None, check=False):
    """D[m,n] = bf16(scale * A[m,k] @ B[n,k]^T) with explicit tunables.  B is [n, k] with row stride b_stride."""
    m, k = A.shape
    n = B.shape[0]
    if b_stride is None:
        b_stride = B.stride(0)
    with torch.cuda.device(A.device):
        rc = lib.sg_skinny_gemm(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                _dev(scale_tensor, torch.float32), m, n, k, b_stride, split_k, A_producers,
                                B_producers, consumers, b_lanes, qsize, op_m, ops, _stream())
    return _done(rc, check)


def skinny_gemm_fastpath(A, B, D, scale_tensor, check=False):
    """Library-chosen configuration; B is [n, k] (row stride taken from the tensor)."""
    m, k = A.shape
    n = B.shape[0]
    with torch.cuda.device(A.device):
        rc = lib.sg_skinny_gemm_auto(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                     _dev(scale_tensor, torch.float32), m, n, k, B.stride(0), _stream())
    return _done(rc, check)


class SgTuning(C.Structure):
    """Mirror of the C struct SgTuning (include/sgemm.h)."""
    _fields_ = [(name, C.c_int) for name in
                ("engine", "split_k", "waves", "row_tiles", "m_blocks", "depth", "k_chunks", "non_temporal",
                 "persistent_wgs_per_cu", "wave_tiles")]


ENGINE_AUTO, ENGINE_DIRECT, ENGINE_LDS, ENGINE_MID = 0, 1, 2, 4
TUNING_FIELDS = tuple(name for name, _ in SgTuning._fields_)


def tuning_as_dict(t):
    return {name: getattr(t, name) for name in TUNING_FIELDS}


def skinny_gemm_rowcol(A, B, D, scale_tensor=None, row_scales=None, col_scales=None, check=False):
    """D = bf16(((A @ B^T) * scale) * row_scales[:, None] * col_scales[None, :]); any factor may be None."""
    m, k = A.shape
    n = B.shape[0]
    if row_scales is not None and tuple(row_scales.shape) != (m,):
        raise ValueError("row_scales must have shape (m,)")
    if col_scales is not None and tuple(col_scales.shape) != (n,):
        raise ValueError("col_scales must have shape (n,)")
    with torch.cuda.device(A.device):
        rc = lib.sg_skinny_gemm_rowcol(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                       None if scale_tensor is None else _dev(scale_tensor, torch.float32),
                                       None if row_scales is None else _dev(row_scales, torch.float32),
                                       None if col_scales is None else _dev(col_scales, torch.float32),
                                       m, n, k, B.stride(0), _stream())
    return _done(rc, check)


def skinny_gemm_bf16act(X, B, D, scale_tensor=None, col_scales=None, row_scales_out=None, tuning=None, check=False):
    """The rowcol GEMM on bf16 activations X [m, k]: rows quantised to E4M3 inside the GEMM (as fp8_encode_rows would),
    D = bf16(((q(X) @ B^T) * scale) * row_scale[:, None] * col_scales[None, :]); row_scales_out, if given, receives the
    row scales.  One launch where the fused kernel pays (skinny_gemm_bf16act_choice), two inside the library otherwise;
    with `tuning` (an SgTuning; engine 0 = the library's record for the shape) always the fused kernel."""
    m, k = X.shape
    n = B.shape[0]
    if col_scales is not None and tuple(col_scales.shape) != (n,):
        raise ValueError("col_scales must have shape (n,)")
    if row_scales_out is not None and tuple(row_scales_out.shape) != (m,):
        raise ValueError("row_scales_out must have shape (m,)")
    args = (_dev(X, torch.bfloat16), _dev(B, *_FP8), _dev(D, torch.bfloat16),
            None if scale_tensor is None else _dev(scale_tensor, torch.float32),
            None if col_scales is None else _dev(col_scales, torch.float32),
            None if row_scales_out is None else _dev(row_scales_out, torch.float32), m, n, k, B.stride(0))
    with torch.cuda.device(X.device):
        if tuning is None:
            rc = lib.sg_skinny_gemm_bf16act(*args, _stream())
        else:
            rc = lib.sg_skinny_gemm_bf16act_tuned(*args, C.byref(tuning), _stream())
    return _done(rc, check)


def skinny_gemm_bf16act_choice(m, n, k):
    """(record, fused): the SgTuning skinny_gemm_bf16act launches for the shape and whether it is the fused kernel."""
    t, fused = SgTuning(), C.c_int(0)
    rc = lib.sg_skinny_gemm_bf16act_choice(m, n, k, C.byref(t), C.byref(fused))
    if rc != 0:
        raise SgError(rc)
    return t, bool(fused.value)


def skinny_gemm_tuned(A, B, D, scale_tensor, engine=ENGINE_AUTO, split_k=1, waves=4, row_tiles=1, m_blocks=None,
                      depth=2, k_chunks=4, non_temporal=1, persistent_wgs_per_cu=0, wave_tiles=0, check=False):
    """The library-native tuning entry (no reference counterpart): pick the engine and its shape."""
    m, k = A.shape
    n = B.shape[0]
    if m_blocks is None:
        m_blocks = 1 if m <= 16 else 2
    t = SgTuning(engine, split_k, waves, row_tiles, m_blocks, depth, k_chunks, non_temporal, persistent_wgs_per_cu, wave_tiles)
    with torch.cuda.device(A.device):
        rc = lib.sg_skinny_gemm_tuned(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                      _dev(scale_tensor, torch.float32), m, n, k, B.stride(0), C.byref(t), _stream())
    return _done(rc, check)


def skinny_gemm_tuned_noalloc(A, B, D, scale_tensor, engine=ENGINE_AUTO, split_k=1, waves=4, row_tiles=1, m_blocks=None,
                              depth=2, k_chunks=4, non_temporal=1, persistent_wgs_per_cu=0, wave_tiles=0, check=False):
    """skinny_gemm_tuned with the split-K partials in the library's fixed device array: allocates nothing, refuses
    configurations whose partials exceed 8 MB or 4096 tiles with WORKSPACE_TOO_SMALL (no reference counterpart)."""
    m, k = A.shape
    n = B.shape[0]
    if m_blocks is None:
        m_blocks = 1 if m <= 16 else 2
    t = SgTuning(engine, split_k, waves, row_tiles, m_blocks, depth, k_chunks, non_temporal, persistent_wgs_per_cu, wave_tiles)
    with torch.cuda.device(A.device):
        rc = lib.sg_skinny_gemm_tuned_noalloc(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                              _dev(scale_tensor, torch.float32), m, n, k, B.stride(0), C.byref(t),
                                              _stream())
    return _done(rc, check)


def init_stream(stream=None, partial_bytes=64 << 20, check=True):
    """Create the split-K workspace of `stream` (torch stream; None = torch's current stream) ahead of time."""
    handle = _stream() if stream is None else stream.cuda_stream
    return _done(lib.sg_init_stream(handle, partial_bytes), check)


def workspace_bytes():
    return lib.sg_workspace_bytes()


def skinny_gemm_pick(m, n, k):
    """The tunables the fastpath would use: dict with the reference's parameter names."""
    out = (C.c_int * 8)()
    rc = lib.sg_skinny_gemm_pick(m, n, k, C.byref(out))
    if rc != 0:
        raise SgError(rc)
    names = ("split_k", "A_producers", "B_producers", "consumers", "b_lanes", "qsize", "op_m", "ops")
    return dict(zip(names, list(out)))


def skinny_gemm_choice(m, n, k):
    """(record, from_table): the complete SgTuning the fastpath would launch for the shape, and whether it comes
    from the tuning table rather than the built-in heuristics."""
    t, from_table = SgTuning(), C.c_int(0)
    rc = lib.sg_skinny_gemm_choice(m, n, k, C.byref(t), C.byref(from_table))
    if rc != 0:
        raise SgError(rc)
    return t, bool(from_table.value)


def tuning_set(m, n, k, tuning):
    """Store `tuning` (an SgTuning, or None to remove the entry) as the record the fastpath uses for the shape."""
    return _done(lib.sg_tuning_set(m, n, k, None if tuning is None else C.byref(tuning)), True)


def tuning_get(m, n, k):
    """The table's SgTuning for the shape, or None."""
    t = SgTuning()
    return t if lib.sg_tuning_get(m, n, k, C.byref(t)) == 0 else None


def tuning_count():
    return lib.sg_tuning_count()


def tuning_clear():
    return _done(lib.sg_tuning_clear(), True)


def tuning_load(path):
    """Merge a tuning file (written by tuning_save or rocm_dev_amd.autotune) into the table."""
    return _done(lib.sg_tuning_load(str(path).encode()), True)


def tuning_save(path):
    return _done(lib.sg_tuning_save(str(path).encode()), True)


class HFRK_skinny_gemm:
    """Same constructor and method as the reference's torch extension class.

    ``B`` is passed as the reference passes it: a (k, n) *view* of an n x k, K-contiguous
    weight, so n = B.size(1) and b_stride = B.stride(1) (skinny_gemm_binding.cu:36-39).
    op_m follows m: 8, 16 or 32 (skinny_gemm_binding.cu:42-45).  D is bfloat16 and is
    overwritten.
    """

    def __init__(self, world_size):
        self.world_size = world_size  # unused, as in the reference

    def skinny_gemm_torch_binding(self, A, B, D, scale_tensor, split_k, A_producers, B_producers, consumers,
                                  b_lanes, qsize, ops):
        m, k = A.size(0), A.size(1)
        n = B.size(1)
        b_stride = B.stride(1)
        op_m = 8 if m <= 8 else (16 if m <= 16 else 32)
        with torch.cuda.device(A.device):
            return lib.sg_skinny_gemm(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16),
                                      _dev(scale_tensor, torch.float32), m, n, k, b_stride, split_k, A_producers,
                                      B_producers, consumers, b_lanes, qsize, op_m, ops, _stream())


def sparse24_gemm(A, B_vals, B_meta, D, scale_tensor, tuning=None, check=False):
    """2:4 sparse weights: B_vals [n, k/2] kept codes, B_meta [n, k/8] position nibbles (include/sgemm.h)."""
    m, k = A.shape
    n = B_vals.shape[0]
    with torch.cuda.device(A.device):
        if tuning is None:
            rc = lib.sg_sparse24_gemm(_dev(A, *_FP8), _dev(B_vals, *_FP8), _dev(B_meta, torch.uint8),
                                      _dev(D, torch.bfloat16), _dev(scale_tensor, torch.float32), m, n, k, _stream())
        else:
            rc = lib.sg_sparse24_gemm_tuned(_dev(A, *_FP8), _dev(B_vals, *_FP8), _dev(B_meta, torch.uint8),
                                            _dev(D, torch.bfloat16), _dev(scale_tensor, torch.float32), m, n, k,
                                            C.byref(tuning), _stream())
    return _done(rc, check)


def sparse24_compress(B, B_vals, B_meta, check=False):
    """Prune dense E4M3 weights B [n, k] to 2:4 (two largest magnitudes per group of four) and compress them
    into B_vals [n, k/2] and B_meta [n, k/8] (format of include/sgemm.h)."""
    n, k = B.shape
    with torch.cuda.device(B.device):
        rc = lib.sg_sparse24_compress(_dev(B, *_FP8), _dev(B_vals, *_FP8), _dev(B_meta, torch.uint8), n, k, B.stride(0),
                                      _stream())
    return _done(rc, check)


def async_gemm(A, B, D, check=False):
    """D = A @ B^T without a scale on the default stream; D is float32 or bfloat16."""
    m, k = A.shape
    n = B.shape[0]
    with torch.cuda.device(A.device):
        if D.dtype == torch.float32:
            rc = lib.sg_async_gemm_f32(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D), m, n, k)
        else:
            rc = lib.sg_async_gemm_bf16(_dev(A, *_FP8), _dev(B, *_FP8), _dev(D, torch.bfloat16), m, n, k)
    return _done(rc, check)


def tiled_sum_reduce(A, B, D, check=False, lds_queue=False):
    """D[m,n] = sum_b (A[b,m,n] + B[b,m,n]) in fp32, batch order.  lds_queue=True runs the variant that stages the
    batches through a queue in LDS (tiled_sum_reduce_async/src.cu:179-200); the result bits are the same."""
    b, m, n = A.shape
    fn = lib.sg_tiled_sum_reduce_async if lds_queue else lib.sg_tiled_sum_reduce
    with torch.cuda.device(A.device):
        rc = fn(_dev(A, torch.float32), _dev(B, torch.float32), _dev(D, torch.float32), b, m, n, _stream())
    return _done(rc, check)


def fp8_encode_rows(X, Q, scales, check=False):
    rows, cols = X.shape
    with torch.cuda.device(X.device):
        rc = lib.sg_fp8_encode_rows(_dev(X, torch.bfloat16), _dev(Q, *_FP8), _dev(scales, torch.float32),
                                    rows, cols, _stream())
    return _done(rc, check)


def fp8_decode_rows(Q, scales, Y, check=False):
    rows, cols = Q.shape
    with torch.cuda.device(Q.device):
        rc = lib.sg_fp8_decode_rows(_dev(Q, *_FP8), _dev(scales, torch.float32), _dev(Y, torch.bfloat16),
                                    rows, cols, _stream())
    return _done(rc, check)


def fp8_reduce_rows(Q, scales, Y, check=False):
    """Q [nbuf, rows, cols], scales [nbuf, rows] -> Y [rows, cols] bfloat16."""
    nbuf, rows, cols = Q.shape
    with torch.cuda.device(Q.device):
        rc = lib.sg_fp8_reduce_rows(_dev(Q, *_FP8), _dev(scales, torch.float32), _dev(Y, torch.bfloat16),
                                    nbuf, Q.stride(0), rows, cols, _stream())
    return _done(rc, check)
