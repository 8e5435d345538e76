"""Host-side mirror of candle's quantized API over the HIP C ABI.

Mirrors candle-core/src/quantized/mod.rs — ``GgmlDType`` (:281-421), ``QStorage`` (:87-278, the
``Cuda`` arm with the method set of cuda.rs:586-898), ``QTensor`` (:532-805) and ``QMatMul`` (:808-897,
:1020-1043) — with the same names, argument meaning and error behaviour, for tensors that live on the
MI355X.  PyTorch only provides device memory and the current stream; every computation goes through
libcandle_hip_quant.so.  There is no CPU storage arm here: that is candle's own k_quants path.
"""
from __future__ import annotations

import enum
import os
import threading
from typing import Optional, Sequence

import numpy as np
import torch

from . import _lib


class GgmlDType(enum.IntEnum):
    """GGUF type codes (mod.rs:300-342)."""
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q2K = 10
    Q3K = 11
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Q8K = 15
    BF16 = 30

    @classmethod
    def from_u32(cls, u: int) -> "GgmlDType":
        try:
            return cls(u)
        except ValueError:
            raise ValueError(f"unknown dtype for tensor {u}") from None

    def to_u32(self) -> int:
        return int(self)

    def type_size(self) -> int:
        return _TYPE_SIZE[self]

    def block_size(self) -> int:
        return _BLOCK_SIZE[self]


_TYPE_SIZE = {GgmlDType.F32: 4, GgmlDType.F16: 2, GgmlDType.BF16: 2, GgmlDType.Q4_0: 18, GgmlDType.Q4_1: 20,
              GgmlDType.Q5_0: 22, GgmlDType.Q5_1: 24, GgmlDType.Q8_0: 34, GgmlDType.Q8_1: 36, GgmlDType.Q2K: 84,
              GgmlDType.Q3K: 110, GgmlDType.Q4K: 144, GgmlDType.Q5K: 176, GgmlDType.Q6K: 210, GgmlDType.Q8K: 292}
_BLOCK_SIZE = {d: (1 if d in (GgmlDType.F32, GgmlDType.F16, GgmlDType.BF16) else
                   32 if d in (GgmlDType.Q4_0, GgmlDType.Q4_1, GgmlDType.Q5_0, GgmlDType.Q5_1, GgmlDType.Q8_0, GgmlDType.Q8_1)
                   else 256) for d in GgmlDType}

# every block format can be stored, quantized, dequantized and used as an embedding table
_KERNEL_DTYPES = (GgmlDType.Q4_0, GgmlDType.Q8_0, GgmlDType.Q4K, GgmlDType.Q5K, GgmlDType.Q6K, GgmlDType.Q8K)
_DEQUANT_DTYPES = _KERNEL_DTYPES + (GgmlDType.Q4_1, GgmlDType.Q5_0, GgmlDType.Q5_1, GgmlDType.Q8_1, GgmlDType.Q2K, GgmlDType.Q3K)
# QMatMul weights: each has a matvec kernel (up to 8 activation rows) and a matrix-core (prefill) kernel
_MATMUL_DTYPES = (GgmlDType.Q4_0, GgmlDType.Q8_0, GgmlDType.Q4K, GgmlDType.Q5K, GgmlDType.Q6K,
                  GgmlDType.Q4_1, GgmlDType.Q5_0, GgmlDType.Q5_1, GgmlDType.Q2K, GgmlDType.Q3K)
# expert formats of the two MoE entry points: the reference's (cuda.rs:543-548 + moe.rs:210-215) plus Q4_0
_MOE_DTYPES = (GgmlDType.Q8_0, GgmlDType.Q2K, GgmlDType.Q3K, GgmlDType.Q4K, GgmlDType.Q5K, GgmlDType.Q6K, GgmlDType.Q4_0)
_TORCH_TO_CQ = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 30}
_TORCH_PLAIN = {GgmlDType.F32: torch.float32, GgmlDType.F16: torch.float16, GgmlDType.BF16: torch.bfloat16}


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{what} must be a tensor on the GPU, got {t.device}")


# ---------------------------------------------------------------------------------------------
# Scratch memory of the library calls: one grow-only buffer per (device, stream), handed out under a lock that is held
# until the call that uses it has been enqueued, like the Mutex-guarded scratch of fast_mmvq.rs:44-81 (the guard lives
# as long as the launch).  Calls on one stream run in enqueue order, so they may share a buffer; calls on different
# streams may overlap on the GPU and get different buffers.  A buffer that is outgrown is kept alive for the life of
# the process (a HIP graph captured earlier may still replay into it), and growing while the stream is being captured
# is refused: the caller runs the call once eagerly first, which sizes the buffer.
# ---------------------------------------------------------------------------------------------
class _Workspace:
    def __init__(self):
        self.lock = threading.Lock()
        self.buf = None
        self.retired = []

    def reserve(self, nbytes: int, alloc, capturing) -> torch.Tensor:
        """The buffer of at least ``nbytes`` bytes; the caller holds ``self.lock``."""
        if self.buf is None or self.buf.numel() < nbytes:
            if capturing():
                raise RuntimeError("the workspace of this stream must grow while the stream is being captured into a graph; "
                                   "run the call once outside the capture first")
            if self.buf is not None:
                self.retired.append(self.buf)
            self.buf = alloc(max(nbytes, 1 << 20, 2 * self.buf.numel() if self.buf is not None else 0))
        return self.buf


_ws_lock = threading.Lock()
_workspaces: dict = {}


class _workspace:
    """``with _workspace(device, nbytes) as ws:`` — the stream's scratch buffer, locked until the block (the enqueue) ends."""

    def __init__(self, device: torch.device, nbytes: int):
        self.device = device
        self.nbytes = int(nbytes)
        self.slot = None

    def _key(self):
        idx = self.device.index if self.device.index is not None else torch.cuda.current_device()
        return (idx, torch.cuda.current_stream(idx).cuda_stream)

    def _alloc(self, n: int) -> torch.Tensor:
        return torch.empty(n, dtype=torch.uint8, device=self.device)

    def _capturing(self) -> bool:
        return torch.cuda.is_current_stream_capturing()

    def __enter__(self) -> torch.Tensor:
        key = self._key()
        with _ws_lock:
            slot = _workspaces.get(key)
            if slot is None:
                slot = _workspaces[key] = _Workspace()
        slot.lock.acquire()
        try:
            buf = slot.reserve(self.nbytes, self._alloc, self._capturing)
        except BaseException:
            slot.lock.release()
            raise
        self.slot = slot
        return buf

    def __exit__(self, *exc) -> None:
        self.slot.lock.release()
        self.slot = None


def check_shape(shape: Sequence[int], block_size: int) -> None:
    """mod.rs:518-530."""
    dims = tuple(shape)
    if len(dims) == 0:
        raise ValueError(f"scalar tensor cannot be quantized {dims}")
    if dims[-1] % block_size != 0:
        raise ValueError(f"quantized tensor must have their last dim divisible by block size {dims} {block_size}")


class QStorage:
    """Raw GGUF blocks in HBM (``QStorage::Cuda`` / ``QCudaStorage``, cuda.rs:586-898)."""

    def __init__(self, data: torch.Tensor, dtype: GgmlDType):
        _require_cuda(data, "QStorage data")
        if data.dtype != torch.uint8 or data.dim() != 1 or not data.is_contiguous():
            raise ValueError("QStorage data must be a contiguous 1-D uint8 tensor")
        self._data = data
        self._dtype = GgmlDType(dtype)

    @staticmethod
    def from_data(data, device, dtype: GgmlDType) -> "QStorage":
        """mod.rs:94-133 -> cuda::load_quantized (cuda.rs:989-1008): upload raw block bytes."""
        dtype = GgmlDType(dtype)
        if isinstance(data, torch.Tensor):
            host = data.detach().cpu().contiguous().view(torch.uint8).reshape(-1)
        else:
            host = torch.from_numpy(np.frombuffer(bytes(data) if not isinstance(data, np.ndarray) else data.tobytes(), dtype=np.uint8).copy())
        if host.numel() % dtype.type_size() != 0:
            raise ValueError("Data length must be a multiple of T's size")
        return QStorage(host.to(device), dtype)

    @staticmethod
    def zeros(device, elem_count: int, dtype: GgmlDType) -> "QStorage":
        """QCudaStorage::zeros (cuda.rs:624-637), without the 512-element tail padding the HIP kernels do not need."""
        dtype = GgmlDType(dtype)
        nblocks = -(-elem_count // dtype.block_size())
        return QStorage(torch.zeros(nblocks * dtype.type_size(), dtype=torch.uint8, device=device), dtype)

    def block_size(self) -> int:
        return self._dtype.block_size()

    def dtype(self) -> GgmlDType:
        return self._dtype

    def device(self) -> torch.device:
        return self._data.device

    def size_in_bytes(self) -> int:
        return self._data.numel()

    storage_size_in_bytes = size_in_bytes

    def data(self) -> bytes:
        """QCudaStorage::data (cuda.rs:880-885): device -> host copy of the block bytes."""
        return self._data.cpu().numpy().tobytes()

    def device_ptr(self) -> int:
        return self._data.data_ptr()

    def quantize(self, src: torch.Tensor) -> None:
        """QCudaStorage::quantize (cuda.rs:704-725); runs GgmlType::from_float on the GPU."""
        _require_cuda(src, "src")
        if self._dtype not in _DEQUANT_DTYPES:
            raise NotImplementedError(f"quantize is not implemented for {self._dtype.name}")
        src = src.to(torch.float32).contiguous().reshape(-1)
        if src.numel() // self.block_size() * self._dtype.type_size() != self._data.numel():
            raise ValueError("quantize: size mismatch between source and storage")
        L = _lib.lib()
        _lib.check("cq_quantize", L.cq_quantize(int(self._dtype), src.data_ptr(), self._data.data_ptr(), src.numel(), _stream_ptr()))

    def quantize_onto(self, src: torch.Tensor) -> None:
        """QCudaStorage::quantize_onto (cuda.rs:784-806): the source is on the host."""
        if src.is_cuda:
            raise ValueError("Invalid quantize source storage locations: not on cpu")
        self.quantize(src.to(self._data.device))

    def dequantize(self, elem_count: int, f16: bool = False) -> torch.Tensor:
        """QCudaStorage::dequantize / dequantize_f16 (cuda.rs:639-702)."""
        if self._dtype in _TORCH_PLAIN:
            # plain arrays (norm weights, unquantized embeddings of a file): a reinterpretation and a dtype cast, no blocks
            if elem_count * self._dtype.type_size() > self._data.numel():
                raise ValueError("dequantize: elem_count exceeds the storage")
            t = self._data[:elem_count * self._dtype.type_size()].view(_TORCH_PLAIN[self._dtype])
            return t.to(torch.float16 if f16 else torch.float32).clone()
        if self._dtype not in _DEQUANT_DTYPES:
            raise NotImplementedError(f"dequantize is not implemented for {self._dtype.name}")
        if elem_count // self.block_size() * self._dtype.type_size() > self._data.numel():
            raise ValueError("dequantize: elem_count exceeds the storage")
        out = torch.empty(elem_count, dtype=torch.float16 if f16 else torch.float32, device=self._data.device)
        L = _lib.lib()
        _lib.check("cq_dequantize", L.cq_dequantize(int(self._dtype), self._data.data_ptr(), out.data_ptr(), elem_count,
                                                    1 if f16 else 0, _stream_ptr()))
        return out


class QTensor:
    """mod.rs:59-66, 532-805."""

    def __init__(self, storage: QStorage, shape: Sequence[int]):
        shape = tuple(int(s) for s in shape)
        check_shape(shape, storage.block_size())
        self.storage = storage
        self._shape = shape

    @staticmethod
    def new(storage: QStorage, shape: Sequence[int]) -> "QTensor":
        return QTensor(storage, shape)

    @staticmethod
    def quantize(src: torch.Tensor, dtype: GgmlDType) -> "QTensor":
        """mod.rs:543-562."""
        dtype = GgmlDType(dtype)
        shape = tuple(src.shape)
        block_size = dtype.block_size()
        check_shape(shape, block_size)
        elem_count = src.numel()
        if elem_count % block_size != 0:
            raise ValueError(f"tensor size ({shape}) is not divisible by block size {block_size}")
        _require_cuda(src, "src")
        storage = QStorage.zeros(src.device, elem_count, dtype)
        storage.quantize(src)
        return QTensor(storage, shape)

    @staticmethod
    def quantize_onto(src: torch.Tensor, dtype: GgmlDType, dev) -> "QTensor":
        """mod.rs:645-671."""
        if src.is_cuda:
            raise ValueError(f"`quantize_onto` expects a `src` to be on the cpu, got {src.device}.")
        return QTensor.quantize(src.to(dev), dtype)

    def dtype(self) -> GgmlDType:
        return self.storage.dtype()

    def device(self) -> torch.device:
        return self.storage.device()

    def rank(self) -> int:
        return len(self._shape)

    def shape(self) -> tuple:
        return self._shape

    def elem_count(self) -> int:
        n = 1
        for s in self._shape:
            n *= s
        return n

    def dequantize(self, device=None) -> torch.Tensor:
        """mod.rs:689-693."""
        t = self.storage.dequantize(self.elem_count()).reshape(self._shape)
        return t if device is None else t.to(device)

    def dequantize_f16(self, device=None) -> torch.Tensor:
        """mod.rs:695-710: the GPU has a dedicated f16 kernel."""
        t = self.storage.dequantize(self.elem_count(), f16=True).reshape(self._shape)
        return t if device is None else t.to(device)

    def embedding(self, ids: torch.Tensor) -> torch.Tensor:
        """mod.rs:712-748: rows ``ids`` of a [rows, hidden] tensor, dequantized -> ids.shape + (hidden,) in f32."""
        if len(self._shape) != 2:
            raise ValueError(f"embedding expects a rank-2 tensor, got shape {self._shape}")
        rows, hidden = self._shape
        dt = self.dtype()
        if hidden % dt.block_size():
            raise ValueError(f"quantized embedding hidden size {hidden} is not divisible by block size {dt.block_size()}")
        dev = self.device()
        flat = ids.to(dev).reshape(-1).to(torch.int64)
        if flat.numel() and (int(flat.max()) >= rows or int(flat.min()) < 0):
            bad = int(flat[(flat >= rows) | (flat < 0)][0])
            raise ValueError(f"embedding id {bad} is out of range for {rows} rows")
        out_shape = tuple(ids.shape) + (hidden,)
        if dt in _TORCH_PLAIN:                                   # plain arrays: an index_select on the typed view
            w = self.storage._data[:rows * hidden * dt.type_size()].view(_TORCH_PLAIN[dt]).reshape(rows, hidden)
            return w.index_select(0, flat).to(torch.float32).reshape(out_shape)
        if dt not in _DEQUANT_DTYPES:
            raise NotImplementedError(f"embedding is not implemented for {dt.name}")
        ids32 = flat.to(torch.int32).contiguous()                # u32 values
        out = torch.empty((flat.numel(), hidden), dtype=torch.float32, device=dev)
        L = _lib.lib()
        _lib.check("cq_embedding", L.cq_embedding(int(dt), self.storage.device_ptr(), ids32.data_ptr(), out.data_ptr(), flat.numel(), rows, hidden,
                                                  _stream_ptr()))
        return out.reshape(out_shape)

    def storage_size_in_bytes(self) -> int:
        return self.storage.size_in_bytes()

    def data(self) -> bytes:
        return self.storage.data()

    def device_ptr(self) -> int:
        return self.storage.device_ptr()

    # ---- CustomOp1 for QTensor ("qmatmul"): cuda_fwd -> QCudaStorage::fwd (mod.rs:1007-1017, cuda.rs:846-878)
    def fwd(self, xs: torch.Tensor) -> torch.Tensor:
        _require_cuda(xs, "xs")
        if not xs.is_contiguous():
            raise ValueError(f"input tensor is not contiguous {tuple(xs.shape)}")
        if len(self._shape) != 2:
            raise ValueError(f"unexpected rank, expected: 2, got: {len(self._shape)} ({self._shape})")
        n, k = self._shape
        if xs.dim() < 2:
            raise ValueError(f"input tensor has only one dimension {tuple(xs.shape)}")
        if xs.shape[-1] != k:
            raise ValueError(f"input tensor {tuple(xs.shape)} incompatible with {self._shape}")
        if xs.dtype not in _TORCH_TO_CQ:
            raise ValueError("Expected f32/f16/bf16")
        if self.dtype() not in _MATMUL_DTYPES:
            raise NotImplementedError(f"qmatmul is not implemented for {self.dtype().name} weights")
        m = xs.numel() // k
        dst = torch.empty((*xs.shape[:-1], n), dtype=xs.dtype, device=xs.device)
        L = _lib.lib()
        need = L.cq_qmatmul_workspace_bytes(int(self.dtype()), m, k, n)
        cq = _TORCH_TO_CQ[xs.dtype]
        with _workspace(xs.device, need) as ws:
            _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(int(self.dtype()), self.device_ptr(), xs.data_ptr(), cq,
                                                                  dst.data_ptr(), cq, m, k, n, ws.data_ptr(), ws.numel(), _stream_ptr()))
        return dst

    def indexed_moe_forward(self, x: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """mod.rs:758-784 -> cuda.rs:587-622.  self [E, n, k]; x [batch, topk or 1, k] f32; ids [batch, topk] u32."""
        if not (x.is_cuda and ids.is_cuda):
            raise RuntimeError("Non-cuda indexed_moe_forward is not implemented!")
        if self.dtype() not in _MOE_DTYPES:
            raise ValueError(f"The given quantized dtype {self.dtype().name} is not supported for indexed_moe_forward!")
        if len(self._shape) != 3 or x.dim() != 3 or ids.dim() != 2:
            raise ValueError("indexed_moe_forward expects weights [E,n,k], x [batch, topk or 1, k], ids [batch, topk]")
        E, n, k = self._shape
        batch, input_dim1, kk = x.shape
        topk = ids.shape[1]
        assert batch == ids.shape[0], "batch dim not match!"
        if kk != k:
            raise ValueError(f"input {tuple(x.shape)} incompatible with {self._shape}")
        if x.dtype != torch.float32:
            raise ValueError("indexed_moe_forward expects f32 input")
        x = x.contiguous()
        ids32 = ids.contiguous().to(torch.int64).to(torch.int32) if ids.dtype not in (torch.int32, torch.uint32) else ids.contiguous()
        out = torch.empty((batch, topk, n), dtype=torch.float32, device=x.device)
        L = _lib.lib()
        need = L.cq_indexed_moe_workspace_bytes(int(self.dtype()), E, n, k, batch, topk, input_dim1)
        if need < 0:
            raise ValueError("indexed_moe_forward: unsupported shape (input dim 1 must be topk or 1)")
        with _workspace(x.device, need) as ws:
            _lib.check("cq_indexed_moe_forward", L.cq_indexed_moe_forward(int(self.dtype()), self.device_ptr(), x.data_ptr(), ids32.data_ptr(),
                                                                          out.data_ptr(), E, n, k, batch, topk, input_dim1,
                                                                          ws.data_ptr(), ws.numel(), _stream_ptr()))
        return out

    def __repr__(self) -> str:
        return f"QTensor[{self._shape}; {self.dtype().name}]"


def _env_flag(name: str) -> bool:
    s = os.environ.get(name)
    return s is not None and s != "" and s != "0"


class QMatMul:
    """mod.rs:807-897, 1020-1043: QTensor / Tensor / TensorF16 variants."""

    def __init__(self, kind: str, value):
        self.kind = kind      # "QTensor" | "Tensor" | "TensorF16"
        self.value = value

    @staticmethod
    def from_arc(qtensor: QTensor) -> "QMatMul":
        dequantize = qtensor.dtype() in (GgmlDType.F32, GgmlDType.F16, GgmlDType.BF16) or _env_flag("CANDLE_DEQUANTIZE_ALL")
        if dequantize:
            return QMatMul("Tensor", qtensor.dequantize())
        if _env_flag("CANDLE_DEQUANTIZE_ALL_F16"):
            return QMatMul("TensorF16", qtensor.dequantize_f16())
        return QMatMul("QTensor", qtensor)

    from_qtensor = from_arc

    def dequantize_f16(self) -> torch.Tensor:
        if self.kind == "QTensor":
            return self.value.dequantize_f16()
        if self.kind == "Tensor":
            return self.value.to(torch.float16)
        return self.value

    def forward_via_f16(self, xs: torch.Tensor) -> torch.Tensor:
        w = self.dequantize_f16()
        return (xs.to(torch.float16) @ w.t()).to(xs.dtype)

    def forward(self, xs: torch.Tensor) -> torch.Tensor:
        if self.kind == "QTensor":
            return self.value.fwd(xs)
        if self.kind == "Tensor":
            return xs @ self.value.t()
        return (xs.to(torch.float16) @ self.value.t()).to(xs.dtype)

    __call__ = forward

    def indexed_moe_forward(self, x: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        if self.kind != "QTensor":
            raise RuntimeError("Not implemented!")
        return self.value.indexed_moe_forward(x, ids)


def moe_gemm_gguf(input: torch.Tensor, weights: QTensor, topk_weights: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
                  experts_ids: torch.Tensor, topk: int, is_prefill: bool, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """candle_nn::moe::moe_gemm_gguf (candle-nn/src/moe.rs:169-337).

    input [tokens or tokens*topk, k] f32; weights [E, n, k]; sorted_token_ids / experts_ids [size_m]
    (u32 in candle, int32 here); topk_weights [size_m] f32 or None.  Returns [size_m, n] f32.
    ``dtype`` is the reference's prefill compute dtype and is unused: both paths quantize the
    activations like candle's CPU path.
    """
    if input.dtype != torch.float32:
        raise ValueError("moe_gemm_gguf only accepts f32 inputs")
    _require_cuda(input, "input")
    size_m, size_k = input.shape
    if topk_weights is None:
        size_m *= topk
    E, size_n, size_k1 = weights.shape()
    assert size_k == size_k1, f"input {size_k} and weight {size_k1} last dim mismatch!"
    if weights.dtype() not in _MOE_DTYPES:
        raise ValueError("moe_gemm_gguf `ISQ` only accept q2k, q3k, q4k, q5k, q6k or q8_0 weights!")
    assert size_k % 8 == 0, "size_k must divisible by 8"
    for name, t in (("sorted_token_ids", sorted_token_ids), ("experts_ids", experts_ids)):
        if not t.is_cuda:
            raise ValueError(f"{name} must be a cuda tensor")
    if topk_weights is not None and not topk_weights.is_cuda:
        raise ValueError("topk_weights must be a cuda tensor")
    input = input.contiguous()
    sti = sorted_token_ids.contiguous().to(torch.int32)
    eid = experts_ids.contiguous().to(torch.int32)
    tw = topk_weights.contiguous().to(torch.float32).reshape(-1) if topk_weights is not None else None
    out = torch.empty((size_m, size_n), dtype=torch.float32, device=input.device)
    L = _lib.lib()
    need = L.cq_moe_gemm_workspace_bytes(int(weights.dtype()), E, topk, size_m, size_n, size_k, 0 if tw is None else 1)
    if need < 0:
        raise ValueError("moe_gemm_gguf: unsupported shape")
    with _workspace(input.device, need) as ws:
        _lib.check("cq_moe_gemm_gguf", L.cq_moe_gemm_gguf(int(weights.dtype()), input.data_ptr(), weights.device_ptr(), sti.data_ptr(),
                                                          eid.data_ptr(), tw.data_ptr() if tw is not None else None, out.data_ptr(),
                                                          E, topk, size_m, size_n, size_k, 1 if is_prefill else 0,
                                                          ws.data_ptr(), ws.numel(), _stream_ptr()))
    return out
