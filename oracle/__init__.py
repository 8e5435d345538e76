"""ctypes loader for the CPU oracle (TEST INFRASTRUCTURE ONLY).

The oracle is a scalar C restatement of candle's CPU quantized-matmul path
(candle-core/src/quantized/{k_quants.rs,utils.rs,mod.rs}).  Only tests/, the smoke check and the
cpu_baseline leg of the benchmark may import this package; the shipped library never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

# GGUF type codes (candle-core/src/quantized/mod.rs:300-342)
Q4_0, Q8_0, Q4K, Q5K, Q6K, Q8K = 2, 8, 12, 13, 14, 15
Q4_1, Q5_0, Q5_1, Q8_1, Q2K, Q3K = 3, 6, 7, 9, 10, 11        # to_float / from_float only
DTYPES = {"q4_0": Q4_0, "q8_0": Q8_0, "q4k": Q4K, "q5k": Q5K, "q6k": Q6K, "q8k": Q8K}

_f32p = ctypes.POINTER(ctypes.c_float)
_i64 = ctypes.c_int64
_vp = ctypes.c_void_p


def build(force: bool = False) -> None:
    """Compile the oracle libraries with the Makefile next to this file."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load(name: str) -> ctypes.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return ctypes.CDLL(path)


_lib = None
_fast = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        L = _load("libcq_oracle.so")
        L.cqo_block_size.restype = _i64
        L.cqo_block_size.argtypes = [ctypes.c_int]
        L.cqo_type_size.restype = _i64
        L.cqo_type_size.argtypes = [ctypes.c_int]
        L.cqo_vec_dot_type.restype = ctypes.c_int
        L.cqo_vec_dot_type.argtypes = [ctypes.c_int]
        L.cqo_f16_to_f32.restype = ctypes.c_float
        L.cqo_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.cqo_f32_to_f16.restype = ctypes.c_uint16
        L.cqo_f32_to_f16.argtypes = [ctypes.c_float]
        L.cqo_to_float.argtypes = [ctypes.c_int, _vp, _vp, _i64]
        L.cqo_from_float.argtypes = [ctypes.c_int, _vp, _vp, _i64]
        L.cqo_vec_dot.argtypes = [ctypes.c_int, _i64, _vp, _vp, _f32p]
        L.cqo_matmul.argtypes = [ctypes.c_int, _i64, _i64, _i64, _vp, _vp, _vp]
        L.cqo_indexed_moe_forward.argtypes = [ctypes.c_int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64]
        L.cqo_moe_gemm_gguf.argtypes = [ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64]
        _lib = L
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_vp)


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise ValueError(f"oracle {what} failed with code {rc}")


def block_size(dtype: int) -> int:
    return int(lib().cqo_block_size(dtype))


def type_size(dtype: int) -> int:
    return int(lib().cqo_type_size(dtype))


def vec_dot_type(dtype: int) -> int:
    return int(lib().cqo_vec_dot_type(dtype))


def f16_to_f32(h: int) -> float:
    return float(lib().cqo_f16_to_f32(h))


def f32_to_f16(f: float) -> int:
    return int(lib().cqo_f32_to_f16(np.float32(f)))


def from_float(dtype: int, x: np.ndarray) -> np.ndarray:
    """GgmlType::from_float on a flat f32 array -> raw block bytes (uint8)."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    bs = block_size(dtype)
    if bs == 0 or x.size % bs:
        raise ValueError(f"size {x.size} not divisible by block size {bs}")
    out = np.zeros(x.size // bs * type_size(dtype), dtype=np.uint8)
    _check(lib().cqo_from_float(dtype, _ptr(x), _ptr(out), x.size), "from_float")
    return out


def to_float(dtype: int, blocks: np.ndarray, k: int | None = None) -> np.ndarray:
    """GgmlType::to_float on raw block bytes -> f32 array of k elements."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    ts, bs = type_size(dtype), block_size(dtype)
    if k is None:
        k = blocks.size // ts * bs
    if blocks.size < k // bs * ts:
        raise ValueError("block buffer too small")
    out = np.empty(k, dtype=np.float32)
    _check(lib().cqo_to_float(dtype, _ptr(blocks), _ptr(out), k), "to_float")
    return out


def vec_dot(dtype: int, n: int, xs: np.ndarray, ys: np.ndarray) -> float:
    """GgmlType::vec_dot_unopt: xs blocks of `dtype`, ys blocks of its VecDotType."""
    xs = np.ascontiguousarray(xs, dtype=np.uint8)
    ys = np.ascontiguousarray(ys, dtype=np.uint8)
    out = ctypes.c_float(0)
    _check(lib().cqo_vec_dot(dtype, n, _ptr(xs), _ptr(ys), ctypes.byref(out)), "vec_dot")
    return float(np.float32(out.value))


def matmul(dtype: int, lhs: np.ndarray, rhs_blocks: np.ndarray, n: int) -> np.ndarray:
    """k_quants::matmul: lhs f32 [m,k], rhs_blocks = n rows of k/blk blocks -> f32 [m,n]."""
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8).reshape(-1)
    need = n * (k // block_size(dtype)) * type_size(dtype)
    if rhs_blocks.size < need:
        raise ValueError(f"weight buffer has {rhs_blocks.size} bytes, need {need}")
    dst = np.empty((m, n), dtype=np.float32)
    _check(lib().cqo_matmul(dtype, m, k, n, _ptr(lhs), _ptr(rhs_blocks), _ptr(dst)), "matmul")
    return dst


def indexed_moe_forward(dtype: int, w_blocks: np.ndarray, shape_enk, x: np.ndarray, ids: np.ndarray) -> np.ndarray:
    """out[b,t,:] = W[ids[b,t]] . x[b, t or 0, :];  w [E,n,k], x [batch, topk or 1, k], ids [batch, topk]."""
    E, n, k = shape_enk
    x = np.ascontiguousarray(x, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    batch, input_dim1, kk = x.shape
    assert kk == k and ids.shape[0] == batch
    topk = ids.shape[1]
    w_blocks = np.ascontiguousarray(w_blocks, dtype=np.uint8).reshape(-1)
    out = np.zeros((batch, topk, n), dtype=np.float32)
    _check(lib().cqo_indexed_moe_forward(dtype, _ptr(w_blocks), _ptr(x), _ptr(ids), _ptr(out), E, n, k, batch, topk, input_dim1),
           "indexed_moe_forward")
    return out


def moe_gemm_gguf(dtype: int, x: np.ndarray, w_blocks: np.ndarray, shape_enk, sorted_token_ids: np.ndarray,
                  expert_ids: np.ndarray, topk_weights, topk: int) -> np.ndarray:
    """candle_nn::moe::moe_gemm_gguf decode semantics with CPU-path activation quantization."""
    E, n, k = shape_enk
    x = np.ascontiguousarray(x, dtype=np.float32)
    size_m = x.shape[0] * (topk if topk_weights is None else 1)
    sorted_token_ids = np.ascontiguousarray(sorted_token_ids, dtype=np.int32)
    expert_ids = np.ascontiguousarray(expert_ids, dtype=np.int32)
    assert sorted_token_ids.size == size_m and expert_ids.size == size_m
    w_blocks = np.ascontiguousarray(w_blocks, dtype=np.uint8).reshape(-1)
    out = np.zeros((size_m, n), dtype=np.float32)
    tw = None
    if topk_weights is not None:
        tw = np.ascontiguousarray(topk_weights, dtype=np.float32).reshape(-1)
    _check(lib().cqo_moe_gemm_gguf(dtype, _ptr(x), _ptr(w_blocks), _ptr(sorted_token_ids), _ptr(expert_ids),
                                   _ptr(tw) if tw is not None else None, _ptr(out), E, topk, size_m, n, k), "moe_gemm_gguf")
    return out


# ---- timed baseline: AVX2 + pthreads variant (same arithmetic as candle's avx.rs path) ----
def fast() -> ctypes.CDLL:
    global _fast
    if _fast is None:
        L = _load("libcq_oracle_fast.so")
        L.cqf_matmul.argtypes = [ctypes.c_int, _i64, _i64, _i64, _vp, _vp, _vp, ctypes.c_int]
        L.cqf_matmul.restype = ctypes.c_int
        _fast = L
    return _fast


def matmul_fast(dtype: int, lhs: np.ndarray, rhs_blocks: np.ndarray, n: int, threads: int) -> np.ndarray:
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8).reshape(-1)
    dst = np.empty((m, n), dtype=np.float32)
    _check(fast().cqf_matmul(dtype, m, k, n, _ptr(lhs), _ptr(rhs_blocks), _ptr(dst), threads), "matmul_fast")
    return dst
