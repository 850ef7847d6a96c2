"""MI355X (gfx950) FP8 skinny-GEMM library: Python host side over the C ABI of libsgemm.so.

The names mirror the reference's launchers (``skinny_gemm``, ``skinny_gemm_fastpath``,
``async_gemm``, ``tiled_sum_reduce``) and its torch binding class ``HFRK_skinny_gemm``;
torch is used only for device memory and streams.
"""
from .api import (  # noqa: F401
    HFRK_skinny_gemm,
    SgError,
    SgReturnCode,
    async_gemm,
    fp8_decode_rows,
    fp8_encode_rows,
    fp8_reduce_rows,
    skinny_gemm,
    sparse24_compress,
    sparse24_gemm,
    SgTuning,
    skinny_gemm_fastpath,
    skinny_gemm_choice,
    skinny_gemm_pick,
    skinny_gemm_rowcol,
    skinny_gemm_bf16act,
    skinny_gemm_bf16act_choice,
    skinny_gemm_tuned,
    skinny_gemm_tuned_noalloc,
    init_stream,
    workspace_bytes,
    workspace_query,
    workspace_init,
    skinny_gemm_auto_ws,
    release_stream,
    release_workspaces,
    strerror,
    tiled_sum_reduce,
    tuning_clear,
    tuning_count,
    tuning_get,
    tuning_load,
    tuning_save,
    tuning_set,
)
from . import synth  # noqa: F401
from .build import build  # noqa: F401
