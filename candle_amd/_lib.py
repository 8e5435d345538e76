"""ctypes binding of libcandle_hip_quant.so (the C ABI declared in include/candle_hip_quant.h and
include/candle_hip_nn.h).

The library must be built first (``python -m candle_amd.build`` or ``__graft_entry__.build()``);
loading fails loudly when it is missing — there is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcandle_hip_quant.so")

_i64 = ctypes.c_int64
_int = ctypes.c_int
_vp = ctypes.c_void_p
_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors the two headers under include/ one to one
SIGNATURES = {
    "cq_status_string": (ctypes.c_char_p, [_int]),
    "cq_block_size": (_i64, [_int]),
    "cq_type_size": (_i64, [_int]),
    "cq_storage_bytes": (_i64, [_int, _i64]),
    "cq_dequantize": (_int, [_int, _vp, _vp, _i64, _int, _vp]),
    "cq_embedding": (_int, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "cq_quantize": (_int, [_int, _vp, _vp, _i64, _vp]),
    "cq_act_scratch_bytes": (_i64, [_int, _i64, _i64]),
    "cq_quantize_act": (_int, [_int, _vp, _int, _vp, _i64, _i64, _vp]),
    "cq_matvec": (_int, [_int, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp]),
    "cq_matmul": (_int, [_int, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "cq_qmatmul_workspace_bytes": (_i64, [_int, _i64, _i64, _i64]),
    "cq_qmatmul_stream_step_bytes": (_i64, [_int, _i64, _i64]),
    "cq_qmatmul_forward": (_int, [_int, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp, _i64, _vp]),
    "cq_static_workspace_bytes": (_i64, []),
    "cq_qmatmul_forward_static": (_int, [_int, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp]),
    "cq_indexed_moe_workspace_bytes": (_i64, [_int, _i64, _i64, _i64, _i64, _i64, _i64]),
    "cq_indexed_moe_forward": (_int, [_int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "cq_moe_gemm_workspace_bytes": (_i64, [_int, _i64, _i64, _i64, _i64, _i64, _int]),
    "cq_moe_gemm_gguf_swiglu": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "cq_moe_gemm_gguf_down_after_pair": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    "cq_moe_direct_pairs": (_int, [_int, _i64, _i64, _i64]),
    "cq_moe_gemm_gguf_pair": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _vp]),
    "cq_moe_gemm_gguf": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _i64, _vp]),
    # include/candle_hip_nn.h
    "cq_nn_embedding": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "cq_nn_qmatmul_norm": (_int, [_int, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]),
    "cq_nn_qmatmul_residual": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "cq_nn_qmatmul_norm_swiglu": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]),
    "cq_nn_qmatmul_norm_pair": (_int, [_int, _vp, _i64, _vp, _int, _vp, _i64, _vp, _vp, _vp, _vp, _f32, _i64, _vp]),
    "cq_nn_qmatmul_split_planes": (_i64, [_int, _i64]),
    "cq_nn_qmatmul_split": (_int, [_int, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "cq_nn_qmatmul_norm_merge": (_int, [_int, _vp, _vp, _vp, _i64, _vp, _f32, _vp, _i64, _i64, _vp]),
    "cq_nn_qmatmul_norm_pair_merge": (_int, [_int, _vp, _i64, _vp, _int, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _f32, _i64, _vp]),
    "cq_nn_qmatmul_residual_merge": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "cq_nn_qmatmul_residual_attn_merge": (_int, [_int, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "cq_nn_qmatmul_residual_attn": (_int, [_int, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp]),
    "cq_nn_moe_route": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "cq_nn_moe_sort": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "cq_nn_moe_sum": (_int, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "cq_nn_rms_norm": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _vp]),
    "cq_nn_rope_i_kv": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "cq_nn_attention_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "cq_nn_attention": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp, _i64, _vp]),
    "cq_nn_attention_decode_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "cq_nn_attention_decode_splits": (_i64, [_i64]),
    "cq_nn_attention_decode": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp, _i64, _vp, _i64,
                                      _i64, _vp]),
    "cq_nn_coop_sync_bytes": (_i64, []),
    "cq_nn_decode_mlp": (_int, [_int, _vp, _vp, _int, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp, _vp]),
    "cq_nn_silu_mul": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "cq_nn_qmatmul_swiglu_rows": (_int, [_int, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "cq_nn_argmax": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "cq_nn_argmax_embed": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp]),
}

_lib = None


class CqError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""

    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed: {text} (status {status})")
        self.fn = fn
        self.status = status


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP extension first (python -m candle_amd.build). "
                "There is no fallback path."
            )
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


BENCH_LIB_PATH = os.path.join(_HERE, "libcq_bench.so")
_bench = None


def bench_lib():
    """libcq_bench.so, the benchmark's plain-read yardstick kernel (candle_amd/csrc/cq_bench.hip): a measurement aid that is
    not part of the C ABI.  None when it has not been built."""
    global _bench
    if _bench is None and os.path.exists(BENCH_LIB_PATH):
        B = ctypes.CDLL(BENCH_LIB_PATH)
        B.cq_bench_read.restype = _int
        B.cq_bench_read.argtypes = [_vp, _i64, _vp, _vp]
        B.cq_bench_read_best.restype = _int
        B.cq_bench_read_best.argtypes = [_vp, _i64, _vp, _vp]
        _bench = B
    return _bench


def status_string(status: int) -> str:
    return lib().cq_status_string(status).decode()


def check(fn: str, status: int) -> None:
    if status != 0:
        raise CqError(fn, status, status_string(status))
