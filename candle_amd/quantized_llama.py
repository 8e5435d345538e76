"""Host-side mirror of candle's quantized llama decoder over the HIP C ABI.

Mirrors candle-transformers/src/models/quantized_llama.rs: ``LayerWeights`` (:150-266), ``Mlp`` (:49-63),
``ModelWeights::forward`` (:568-596) and ``precomput_freqs_cis`` (:284-300), for the dense (non-MoE) llama
architecture with interleaved RoPE.  Every computation is a call into libcandle_hip_quant.so
(quantized matmuls from candle_hip_quant.h, f32 glue from candle_hip_nn.h); PyTorch only provides device
memory, the stream and HIP-graph capture.

Differences from the reference that do not change results:
  * the KV cache is preallocated ([n_kv_head, ctx, head_dim] per layer) instead of grown by Tensor::cat;
  * attention_wq|attention_wk and feed_forward_w1|feed_forward_w3 are stored back to back, so when their
    formats agree each pair runs as one matmul over the concatenated rows (rows are independent);
  * a greedy decode step can be captured once in a HIP graph and replayed: the next token and the
    position live in device memory (``generate_greedy``).
"""
from __future__ import annotations

import dataclasses
import math
import time
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from . import _lib
from .quantized import GgmlDType, QStorage, QTensor, _MATMUL_DTYPES


@dataclasses.dataclass
class Config:
    n_layer: int = 32
    hidden: int = 4096
    n_head: int = 32
    n_kv_head: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    rope_theta: float = 500000.0      # llama.rope.freq_base of Llama-3 files (quantized_llama.rs:455-458 reads it)
    rms_eps: float = 1e-5             # llama.attention.layer_norm_rms_epsilon
    ctx: int = 2048                   # rows of the cos/sin tables and of the KV cache (MAX_SEQ_LEN in the reference)

    @staticmethod
    def llama3_8b() -> "Config":
        return Config()


def precomput_freqs_cis(head_dim: int, freq_base: float, max_seq_len: int):
    """cos/sin tables [max_seq_len, head_dim/2] in f32 (quantized_llama.rs:284-300)."""
    i = np.arange(0, head_dim, 2, dtype=np.float32)
    theta = (np.float32(1.0) / np.power(np.float32(freq_base), i / np.float32(head_dim))).astype(np.float32)
    idx = np.arange(max_seq_len, dtype=np.float32).reshape(-1, 1)
    idx_theta = (idx * theta.reshape(1, -1)).astype(np.float32)
    return np.cos(idx_theta).astype(np.float32), np.sin(idx_theta).astype(np.float32)


# tensor order inside one layer's slab: pairs that can be fused are adjacent
_LAYER_ORDER = ("attention_wq", "attention_wk", "attention_wv", "attention_wo", "feed_forward_w1", "feed_forward_w3", "feed_forward_w2")


def _layer_shapes(cfg: Config) -> Dict[str, tuple]:
    qd, kvd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim
    return {"attention_wq": (qd, cfg.hidden), "attention_wk": (kvd, cfg.hidden), "attention_wv": (kvd, cfg.hidden),
            "attention_wo": (cfg.hidden, qd), "feed_forward_w1": (cfg.ffn, cfg.hidden), "feed_forward_w3": (cfg.ffn, cfg.hidden),
            "feed_forward_w2": (cfg.hidden, cfg.ffn)}


Q4_K_M = {"attention_wq": GgmlDType.Q4K, "attention_wk": GgmlDType.Q4K, "attention_wv": GgmlDType.Q6K, "attention_wo": GgmlDType.Q4K,
          "feed_forward_w1": GgmlDType.Q4K, "feed_forward_w3": GgmlDType.Q4K, "feed_forward_w2": GgmlDType.Q6K, "output": GgmlDType.Q4K}


class _W:
    """One quantized weight inside the model's slab: device pointer, format, shape."""
    __slots__ = ("ptr", "dtype", "n", "k", "nbytes")

    def __init__(self, ptr: int, dtype: GgmlDType, n: int, k: int, nbytes: int):
        self.ptr, self.dtype, self.n, self.k, self.nbytes = ptr, dtype, n, k, nbytes


class LayerWeights:
    def __init__(self):
        self.w: Dict[str, _W] = {}
        self.attention_norm: Optional[torch.Tensor] = None
        self.ffn_norm: Optional[torch.Tensor] = None
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None
        self.prefetch_span = 0       # bytes from attention_wo to the end of this layer's weights


class ModelWeights:
    """quantized_llama::ModelWeights for one GPU.  Build with ``random_init`` or ``from_blocks``."""

    def __init__(self, cfg: Config, device="cuda:0"):
        if cfg.hidden % 256 or cfg.ffn % 256 or (cfg.n_head * cfg.head_dim) % 256:
            raise ValueError("hidden, ffn and n_head*head_dim must be multiples of 256 (K-quant super-blocks)")
        if cfg.n_head % cfg.n_kv_head:
            raise ValueError("n_head must be a multiple of n_kv_head")
        self.cfg = cfg
        self.device = torch.device(device)
        self.L = _lib.lib()
        self.layers: List[LayerWeights] = []
        self.tok_embeddings: Optional[torch.Tensor] = None     # f32 [vocab, hidden] (the reference dequantizes token_embd)
        self.norm: Optional[torch.Tensor] = None
        self.output: Optional[_W] = None
        self._slab: Optional[torch.Tensor] = None
        self._graph = None
        self._graph_key = None
        self.fuse_decode = True            # single-token steps use the fused matvec prologues / epilogues
        self.split_w2 = False              # ... and feed_forward_w2 as a K-split matvec (planes merged by its consumers) where the shapes allow it;
                                           # off: with every format of a Q4_K_M file on the streaming kernel the unsplit step is as fast (8B shape: 608 vs 603 tok/s)
        self.merge_in_wo = False           # merge the attention key splits in the prologue of attention_wo (else: in the attention kernel)
        # Bytes of the weights behind attention (wo, w1, w3, w2 are contiguous) that the attention launch's idle CUs read ahead of
        # the kernels that stream them, each piece on the XCD whose L2 its consumer will look in.  Measured on the 8B shape
        # (tok/s at 0 / 4 / 9.4 / 14 / 18 / 28 / 40 MB): 672 / 676 / 680 / 684 / 682 / 649 / 605, read linearly 672 / - / 675 / - / 677 /
        # 673 / 656: all of attention_wo and the head of feed_forward_w1 pay, beyond what the L2s hold (8 x 4 MB) the time moves
        # into the attention launch.
        self.prefetch_bytes = 14 << 20
        # Single-token steps can run the two matvecs of the feed-forward as one cooperative launch (cq_nn_decode_mlp) where a kernel
        # exists for the formats and shapes; every such step is valid only while coop_error() is False (checked by forward and
        # generate_greedy).  Off: measured on the 8B shape the launch takes 26.4 us against 24.2 us for the two launches it replaces
        # (672 against 705 tok/s): the barrier and the acknowledged stores cost more than the kernel boundary they replace, and the
        # weights requested ahead of the barrier do not make up for it.
        self.coop = False
        self.coop_sync = None
        self.tap = None                    # tests: called as tap(stage, layer) after each launch of an eager forward

    # ------------------------------------------------------------------------------------------ construction
    def _alloc(self, dtypes: Dict[str, GgmlDType]):
        cfg, L = self.cfg, self.L
        shapes = _layer_shapes(cfg)
        total, plan = 0, []
        # a format per tensor role, which "blk.{i}.{role}" entries override for single layers (files mix formats per layer)
        dt_of = lambda li, name: GgmlDType(dtypes.get(f"blk.{li}.{name}", dtypes[name]))
        for li in range(cfg.n_layer):
            for name in _LAYER_ORDER:
                n, k = shapes[name]
                nb = L.cq_storage_bytes(int(dt_of(li, name)), n * k)
                if nb < 0:
                    raise ValueError(f"{name}: {n}x{k} is not a whole number of {dt_of(li, name).name} blocks")
                plan.append((li, name, total, nb, n, k, dt_of(li, name)))
                total += (nb + 255) // 256 * 256
        nb = L.cq_storage_bytes(int(dtypes["output"]), cfg.vocab * cfg.hidden)
        plan.append((-1, "output", total, nb, cfg.vocab, cfg.hidden, GgmlDType(dtypes["output"])))
        total += (nb + 255) // 256 * 256
        self._slab = torch.empty(total, dtype=torch.uint8, device=self.device)
        base = self._slab.data_ptr()
        self.layers = [LayerWeights() for _ in range(cfg.n_layer)]
        for li, name, off, nb, n, k, dt in plan:
            w = _W(base + off, dt, n, k, nb)
            if li < 0:
                self.output = w
            else:
                self.layers[li].w[name] = w
        f32 = dict(dtype=torch.float32, device=self.device)
        for lw in self.layers:
            w2 = lw.w["feed_forward_w2"]
            lw.prefetch_span = (w2.ptr + w2.nbytes - lw.w["attention_wo"].ptr) // 16 * 16
            lw.k_cache = torch.zeros((cfg.n_kv_head, cfg.ctx, cfg.head_dim), **f32)
            lw.v_cache = torch.zeros((cfg.n_kv_head, cfg.ctx, cfg.head_dim), **f32)
        cos, sin = precomput_freqs_cis(cfg.head_dim, cfg.rope_theta, cfg.ctx)
        self.cos = torch.from_numpy(cos).to(self.device)
        self.sin = torch.from_numpy(sin).to(self.device)
        self._alloc_activations(max_rows=1)
        # device-side decode state for graph replay
        self.token_dev = torch.zeros(1, dtype=torch.int32, device=self.device)
        self.pos_dev = torch.zeros(1, dtype=torch.int32, device=self.device)
        self.counter_dev = torch.zeros(1, dtype=torch.int32, device=self.device)
        self.history_dev = torch.zeros(cfg.ctx, dtype=torch.int32, device=self.device)
        self.argmax_ws = torch.zeros(1024, dtype=torch.uint8, device=self.device)      # CQ_NN_ARGMAX_WORKSPACE
        return plan

    def _alloc_activations(self, max_rows: int):
        cfg, L = self.cfg, self.L
        qd, kvd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim
        f32 = dict(dtype=torch.float32, device=self.device)
        self.max_rows = max_rows
        self._graph = None                 # a captured step holds the old buffer addresses
        self.x = torch.empty((max_rows, cfg.hidden), **f32)
        self.planes = torch.empty((4, cfg.hidden), **f32)       # decode: K-slice planes of a split feed_forward_w2 (CQ_NN_MAX_PLANES)
        self.xn = torch.empty((max_rows, cfg.hidden), **f32)
        self.qk = torch.empty((max_rows, qd + kvd), **f32)
        self.v = torch.empty((max_rows, kvd), **f32)
        self.att = torch.empty((max_rows, qd), **f32)
        self.delta = torch.empty((max_rows, cfg.hidden), **f32)
        self.gu = torch.empty((max_rows, 2 * cfg.ffn), **f32)
        self.h = torch.empty((max_rows, cfg.ffn), **f32)
        self.logits = torch.empty((1, cfg.vocab), **f32)
        self.partials = torch.zeros(256, **f32)          # CQ_NN_PARTIALS: sum(x^2) of the residual row, in partial sums
        need = 0
        for (n, k) in list(_layer_shapes(cfg).values()) + [(qd + kvd, cfg.hidden), (2 * cfg.ffn, cfg.hidden)]:
            for dt in (GgmlDType.Q4K, GgmlDType.Q8_0):      # K-quant and Q*_0 scratch layouts
                need = max(need, L.cq_qmatmul_workspace_bytes(int(dt), max_rows, k, n))
        need = max(need, L.cq_qmatmul_workspace_bytes(int(GgmlDType.Q4K), 1, cfg.hidden, cfg.vocab))
        self.ws = torch.empty(max(need, 256), dtype=torch.uint8, device=self.device)
        att_ws = L.cq_nn_attention_workspace_bytes(max_rows, cfg.n_head, cfg.head_dim, cfg.ctx)
        self.att_ws = torch.empty(max(att_ws, 256), dtype=torch.uint8, device=self.device)
        # single-token attention: per-split partials
        attd = L.cq_nn_attention_decode_workspace_bytes(cfg.n_head, cfg.head_dim, min(cfg.ctx, 4096))
        self.attd_ws = torch.zeros(attd, dtype=torch.uint8, device=self.device)

    @classmethod
    def random_init(cls, cfg: Config, seed: int = 0, device="cuda:0", dtypes: Optional[Dict[str, GgmlDType]] = None,
                    weight_scale: float = 0.02) -> "ModelWeights":
        """Random-init weights ~N(0, weight_scale) quantized on the device (norm weights = 1, f32 embedding table).
        ``dtypes`` maps a tensor role to its format; a ``"blk.{i}.{role}"`` entry overrides the role's format for layer i."""
        self = cls(cfg, device)
        dtypes = dict(Q4_K_M if dtypes is None else dtypes)
        plan = self._alloc(dtypes)
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        base = self._slab.data_ptr()
        for li, name, off, nb, n, k, dt in plan:
            wf = torch.randn((n, k), generator=gen, device=self.device, dtype=torch.float32) * weight_scale
            _lib.check("cq_quantize", self.L.cq_quantize(int(dt), wf.data_ptr(), base + off, n * k, None))
            torch.cuda.synchronize(self.device)
            del wf
        self.tok_embeddings = torch.randn((cfg.vocab, cfg.hidden), generator=gen, device=self.device, dtype=torch.float32) * weight_scale
        ones = torch.ones(cfg.hidden, dtype=torch.float32, device=self.device)
        for lw in self.layers:
            lw.attention_norm, lw.ffn_norm = ones, ones
        self.norm = ones
        return self

    @classmethod
    def from_blocks(cls, cfg: Config, tensors: dict, device="cuda:0") -> "ModelWeights":
        """Build from host data: ``tensors[name] = (GgmlDType, block bytes)`` for ``output`` and
        ``blk.{i}.{attention_wq,...}``, f32 arrays for ``tok_embeddings``, ``norm``, ``blk.{i}.attention_norm``,
        ``blk.{i}.ffn_norm`` (the tensors ModelWeights::from_gguf reads, quantized_llama.rs:470-540)."""
        self = cls(cfg, device)
        dtypes = {name: GgmlDType(tensors[f"blk.0.{name}"][0]) for name in _LAYER_ORDER}
        dtypes["output"] = GgmlDType(tensors["output"][0])
        for li in range(cfg.n_layer):
            for name in _LAYER_ORDER:
                dtypes[f"blk.{li}.{name}"] = GgmlDType(tensors[f"blk.{li}.{name}"][0])
        for key, dt in dtypes.items():
            if dt not in _MATMUL_DTYPES:
                raise NotImplementedError(f"{key}: no matmul kernel for {dt.name} weights")
        plan = self._alloc(dtypes)
        for li, name, off, nb, n, k, _ in plan:
            dt, blocks = tensors["output" if li < 0 else f"blk.{li}.{name}"]
            raw = np.frombuffer(bytes(blocks), dtype=np.uint8)
            if raw.size != nb:
                raise ValueError(f"{name}: expected {nb} bytes of blocks, got {raw.size}")
            self._slab[off:off + nb].copy_(torch.from_numpy(raw.copy()))
        as_dev = lambda a: (a.to(device=self.device, dtype=torch.float32).contiguous() if isinstance(a, torch.Tensor)
                            else torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(self.device))
        self.tok_embeddings = as_dev(tensors["tok_embeddings"])
        self.norm = as_dev(tensors["norm"])
        for i, lw in enumerate(self.layers):
            lw.attention_norm = as_dev(tensors[f"blk.{i}.attention_norm"])
            lw.ffn_norm = as_dev(tensors[f"blk.{i}.ffn_norm"])
        torch.cuda.synchronize(self.device)
        return self

    # architectures whose rope pairs (i, i + d/2) instead of (2i, 2i + 1) (quantized_llama.rs:396-428)
    _NEOX_ARCHS = ("qwen", "qwen2", "qwen2moe", "qwen3", "qwen3moe", "falcon", "grok", "dbrx", "phi2", "phi3", "phimoe", "stablelm",
                   "starcoder2", "bert", "nomic-bert", "jina-bert-v2", "olmo2", "olmoe", "codeshell", "plamo")

    @classmethod
    def from_gguf(cls, ct, reader, device="cuda:0", ctx: int = 4096) -> "ModelWeights":
        """ModelWeights::from_gguf (quantized_llama.rs:367-540): hyper-parameters from the metadata, tensors by their
        GGUF names, the matmul weights uploaded as the raw blocks of the file.  ``ct`` is a ``gguf_file.Content``,
        ``reader`` the open file; ``ctx`` stands for MAX_SEQ_LEN (rows of the rope tables and of the KV cache)."""
        from .gguf_file import GgufError

        def md_get(key):
            v = ct.metadata.get(key)
            if v is None:
                raise GgufError(f"cannot find {key} in metadata")
            return v

        def md_u32_or(key, default):
            v = ct.metadata.get(key)
            try:
                return default if v is None else v.to_u32()
            except GgufError:
                return default

        if md_u32_or("llama.expert_count", 0) > 1:
            raise NotImplementedError("mixture-of-experts llama files: the expert layer is candle_amd.fused_moe.FusedMoeGGUF")
        head_count = md_get("llama.attention.head_count").to_u32()
        head_count_kv = md_get("llama.attention.head_count_kv").to_u32()
        block_count = md_get("llama.block_count").to_u32()
        embedding_length = md_get("llama.embedding_length").to_u32()
        rope_dim = md_get("llama.rope.dimension_count").to_u32()
        rms_norm_eps = md_get("llama.attention.layer_norm_rms_epsilon").to_f32()
        fb = ct.metadata.get("llama.rope.freq_base")
        try:
            rope_freq_base = 10000.0 if fb is None else fb.to_f32()
        except GgufError:
            rope_freq_base = 10000.0
        arch = ct.metadata.get("general.architecture")
        arch = arch.v if arch is not None and isinstance(arch.v, str) else ""
        if arch in cls._NEOX_ARCHS:
            raise NotImplementedError(f"architecture {arch!r} uses the non-interleaved rope, which this decoder does not implement")
        head_dim = embedding_length // head_count
        if rope_dim != head_dim:
            raise NotImplementedError(f"rope over {rope_dim} of {head_dim} head dimensions is not implemented")

        tok_embeddings_q = ct.tensor(reader, "token_embd.weight", device)
        tensors = {"tok_embeddings": tok_embeddings_q.dequantize(),
                   "norm": ct.tensor(reader, "output_norm.weight", device).dequantize()}
        out_name = "output.weight" if "output.weight" in ct.tensor_infos else "token_embd.weight"      # tied embeddings
        info, raw = ct.tensor_bytes(reader, out_name)
        tensors["output"] = (info.ggml_dtype, raw)
        names = {"attention_wq": "attn_q", "attention_wk": "attn_k", "attention_wv": "attn_v", "attention_wo": "attn_output",
                 "feed_forward_w1": "ffn_gate", "feed_forward_w2": "ffn_down", "feed_forward_w3": "ffn_up"}
        ffn = None
        for i in range(block_count):
            for mine, theirs in names.items():
                info, raw = ct.tensor_bytes(reader, f"blk.{i}.{theirs}.weight")
                tensors[f"blk.{i}.{mine}"] = (info.ggml_dtype, raw)
                if mine == "feed_forward_w1":
                    ffn = info.shape[0]
            tensors[f"blk.{i}.attention_norm"] = ct.tensor(reader, f"blk.{i}.attn_norm.weight", device).dequantize()
            tensors[f"blk.{i}.ffn_norm"] = ct.tensor(reader, f"blk.{i}.ffn_norm.weight", device).dequantize()
        cfg = Config(n_layer=block_count, hidden=embedding_length, n_head=head_count, n_kv_head=head_count_kv, head_dim=head_dim, ffn=ffn,
                     vocab=tok_embeddings_q.shape()[0], rope_theta=float(rope_freq_base), rms_eps=float(rms_norm_eps), ctx=ctx)
        return cls.from_blocks(cfg, tensors, device)

    def weight_bytes_per_token(self) -> int:
        """Quantized weight bytes one decode step streams (every matmul weight once)."""
        return sum(w.nbytes for lw in self.layers for w in lw.w.values()) + self.output.nbytes

    def clear_kv_cache(self):
        """quantized_llama.rs:558-566 — with a preallocated cache only the position matters."""
        self.pos_dev.zero_()

    # ------------------------------------------------------------------------------------------ forward
    def _mm(self, w: _W, n: int, src: torch.Tensor, dst_ptr: int, rows: int, sp):
        """QMatMul::forward of `rows` f32 rows of `src` with weight rows [w.ptr, +n rows) into dst_ptr."""
        L = self.L
        _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(int(w.dtype), w.ptr, src.data_ptr(), 0, dst_ptr, 0, rows, w.k, n,
                                                              self.ws.data_ptr(), self.ws.numel(), sp))

    def _enqueue(self, ids_ptr: Optional[int], rows: int, pos: int, pos_dev_ptr: Optional[int], max_kv_len: int, sp) -> None:
        """All kernels of ModelWeights::forward (quantized_llama.rs:568-596) for `rows` new tokens; logits of the last.
        ids_ptr None (fused single-token step only): the token's embedding row and its partial sums of squares are already in
        self.x / self.partials (cq_nn_argmax_embed of the previous step put them there)."""
        cfg, L = self.cfg, self.L
        qd, kvd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim
        scale = float(np.float32(1.0 / math.sqrt(cfg.head_dim)))
        ck = _lib.check
        x, xn, qk, v, att, delta, gu, h = self.x, self.xn, self.qk, self.v, self.att, self.delta, self.gu, self.h
        if rows == 1 and self.fuse_decode and self.L.cq_nn_attention_decode_splits(max_kv_len) > 0:
            return self._enqueue_decode_fused(ids_ptr, pos, pos_dev_ptr, max_kv_len, sp)
        if ids_ptr is None:
            raise ValueError("a step without token ids needs the fused single-token path")
        tap = self.tap if self.tap is not None else (lambda stage, li: None)
        ck("cq_nn_embedding", L.cq_nn_embedding(self.tok_embeddings.data_ptr(), ids_ptr, x.data_ptr(), rows, cfg.hidden, cfg.vocab, None, sp))
        tap("embedding", -1)
        for li, lw in enumerate(self.layers):
            w = lw.w
            # x (+= mlp output of the previous layer); xn = attention_norm(x)          :579-583, :590-592
            ck("cq_nn_rms_norm", L.cq_nn_rms_norm(x.data_ptr(), delta.data_ptr() if li else None, lw.attention_norm.data_ptr(),
                                                 x.data_ptr() if li else None, xn.data_ptr(), rows, cfg.hidden, cfg.rms_eps, sp))
            tap("attention_norm", li)
            # q, k, v projections                                                         :200-202
            wq, wk, wv = w["attention_wq"], w["attention_wk"], w["attention_wv"]
            if wq.dtype == wk.dtype and wk.ptr == wq.ptr + wq.nbytes:
                self._mm(wq, qd + kvd, xn, qk.data_ptr(), rows, sp)
                q_ptr, k_ptr, qs, ks = qk.data_ptr(), qk.data_ptr() + 4 * qd, qd + kvd, qd + kvd
            else:
                self._mm(wq, qd, xn, qk.data_ptr(), rows, sp)
                self._mm(wk, kvd, xn, qk.data_ptr() + 4 * rows * qd, rows, sp)
                q_ptr, k_ptr, qs, ks = qk.data_ptr(), qk.data_ptr() + 4 * rows * qd, qd, kvd
            self._mm(wv, kvd, xn, v.data_ptr(), rows, sp)
            tap("qkv", li)
            # rope on q and k, append k and v to the cache                                :217-233
            ck("cq_nn_rope_i_kv", L.cq_nn_rope_i_kv(q_ptr, k_ptr, v.data_ptr(), lw.k_cache.data_ptr(), lw.v_cache.data_ptr(),
                                                   self.cos.data_ptr(), self.sin.data_ptr(), pos_dev_ptr, pos, rows, cfg.n_head, cfg.n_kv_head,
                                                   cfg.head_dim, cfg.ctx, qs, ks, kvd, sp))
            tap("rope", li)
            # softmax(q k^T / sqrt(d) + causal mask) v                                    :246-261
            ck("cq_nn_attention", L.cq_nn_attention(q_ptr, qs, lw.k_cache.data_ptr(), lw.v_cache.data_ptr(), att.data_ptr(), pos_dev_ptr, pos,
                                                   rows, cfg.n_head, cfg.n_kv_head, cfg.head_dim, cfg.ctx, max_kv_len, scale,
                                                   self.att_ws.data_ptr(), self.att_ws.numel(), sp))
            tap("attention", li)
            self._mm(w["attention_wo"], cfg.hidden, att, delta.data_ptr(), rows, sp)    # :264
            tap("attention_wo", li)
            # x += attn; xn = ffn_norm(x)                                                 :584-589
            ck("cq_nn_rms_norm", L.cq_nn_rms_norm(x.data_ptr(), delta.data_ptr(), lw.ffn_norm.data_ptr(), x.data_ptr(), xn.data_ptr(), rows,
                                                 cfg.hidden, cfg.rms_eps, sp))
            tap("ffn_norm", li)
            # w2(silu(w1 x) * w3 x)                                                       :56-63
            w1, w3 = w["feed_forward_w1"], w["feed_forward_w3"]
            if w1.dtype == w3.dtype and w3.ptr == w1.ptr + w1.nbytes:
                self._mm(w1, 2 * cfg.ffn, xn, gu.data_ptr(), rows, sp)
                g_ptr, u_ptr, gs = gu.data_ptr(), gu.data_ptr() + 4 * cfg.ffn, 2 * cfg.ffn
            else:
                self._mm(w1, cfg.ffn, xn, gu.data_ptr(), rows, sp)
                self._mm(w3, cfg.ffn, xn, gu.data_ptr() + 4 * rows * cfg.ffn, rows, sp)
                g_ptr, u_ptr, gs = gu.data_ptr(), gu.data_ptr() + 4 * rows * cfg.ffn, cfg.ffn
            tap("w13", li)
            w2 = w["feed_forward_w2"]
            if rows > 2 and cfg.ffn % 256 == 0:
                # silu(w1 x) * w3 x goes straight into the activation quantizer of w2
                ck("cq_nn_qmatmul_swiglu_rows", L.cq_nn_qmatmul_swiglu_rows(int(w2.dtype), w2.ptr, g_ptr, u_ptr, gs, gs, delta.data_ptr(), rows,
                                                                            w2.k, cfg.hidden, self.ws.data_ptr(), self.ws.numel(), sp))
            else:
                ck("cq_nn_silu_mul", L.cq_nn_silu_mul(g_ptr, u_ptr, h.data_ptr(), rows, cfg.ffn, gs, gs, sp))
                self._mm(w2, cfg.hidden, h, delta.data_ptr(), rows, sp)
            tap("w2", li)
        # last token only: x += mlp; final norm; output head                              :593-596
        last = 4 * (rows - 1) * cfg.hidden
        ck("cq_nn_rms_norm", L.cq_nn_rms_norm(x.data_ptr() + last, delta.data_ptr() + last, self.norm.data_ptr(), None, xn.data_ptr(), 1,
                                             cfg.hidden, cfg.rms_eps, sp))
        self._mm(self.output, cfg.vocab, xn, self.logits.data_ptr(), 1, sp)
        tap("head", -1)

    def _enqueue_decode_fused(self, ids_ptr: Optional[int], pos: int, pos_dev_ptr: Optional[int], max_kv_len: int, sp) -> None:
        """The same single-token step with the glue folded into the matvec kernels: the residual add is the
        epilogue of attention_wo / feed_forward_w2 (which also leaves sum(x^2) as partial sums), rms_norm and
        silu(w1 x) * w3 x are the prologues of the matvecs that consume them.  A long feed_forward_w2 row is split
        along K into planes; the next rms_norm prologue reads the residual row plus the planes, and the next residual
        add (attention_wo) folds them into the row."""
        cfg, L = self.cfg, self.L
        qd, kvd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim
        scale = float(np.float32(1.0 / math.sqrt(cfg.head_dim)))
        ck = _lib.check
        qk, v, att, gu, part, planes = self.qk, self.v, self.att, self.gu, self.partials, self.planes
        kq = (GgmlDType.Q4K, GgmlDType.Q5K, GgmlDType.Q6K)
        # formats with every decode fusion; the others (Q4_1, Q5_0, Q5_1, Q2K, Q3K) have the rms_norm prologue and the residual
        # epilogue only: no paired launches, no attention merge inside attention_wo, no K-split planes anywhere in the model
        full = kq + (GgmlDType.Q4_0, GgmlDType.Q8_0)
        all_full = all(w.dtype in full for lw in self.layers for w in lw.w.values()) and self.output.dtype in full
        cur = self.x.data_ptr()                                    # the residual row
        pending = 0                                                # planes of the previous feed_forward_w2 not yet added to it
        tap = self.tap if self.tap is not None else (lambda stage, li: None)
        if ids_ptr is not None:
            ck("cq_nn_embedding", L.cq_nn_embedding(self.tok_embeddings.data_ptr(), ids_ptr, cur, 1, cfg.hidden, cfg.vocab, part.data_ptr(), sp))
        tap("embedding", -1)

        def one_step(w: _W) -> bool:
            return w.k <= (4096 if w.dtype in kq + (GgmlDType.Q2K, GgmlDType.Q3K) else 2048)

        def norm_mm(w: _W, n: int, norm_w: torch.Tensor, dst_ptr: int):
            if pending:
                ck("cq_nn_qmatmul_norm_merge", L.cq_nn_qmatmul_norm_merge(int(w.dtype), w.ptr, cur, planes.data_ptr(), pending,
                                                                          norm_w.data_ptr(), cfg.rms_eps, dst_ptr, w.k, n, sp))
            else:
                ck("cq_nn_qmatmul_norm", L.cq_nn_qmatmul_norm(int(w.dtype), w.ptr, cur, part.data_ptr(), norm_w.data_ptr(), cfg.rms_eps,
                                                              dst_ptr, w.k, n, sp))

        def resid_mm(w: _W, src_ptr: int, up_ptr: Optional[int]):
            ck("cq_nn_qmatmul_residual_merge", L.cq_nn_qmatmul_residual_merge(int(w.dtype), w.ptr, src_ptr, up_ptr, cur, part.data_ptr(),
                                                                              planes.data_ptr() if pending else None, pending, w.k,
                                                                              cfg.hidden, sp))

        for li, lw in enumerate(self.layers):
            w = lw.w
            wq, wk, wv = w["attention_wq"], w["attention_wk"], w["attention_wv"]
            if wq.dtype == wk.dtype and wk.ptr == wq.ptr + wq.nbytes and wq.dtype in kq and wv.dtype in kq:
                # q|k and v in one launch even though their formats differ
                if pending:
                    ck("cq_nn_qmatmul_norm_pair_merge", L.cq_nn_qmatmul_norm_pair_merge(
                        int(wq.dtype), wq.ptr, qd + kvd, qk.data_ptr(), int(wv.dtype), wv.ptr, kvd, v.data_ptr(), cur, planes.data_ptr(),
                        pending, lw.attention_norm.data_ptr(), cfg.rms_eps, cfg.hidden, sp))
                else:
                    ck("cq_nn_qmatmul_norm_pair", L.cq_nn_qmatmul_norm_pair(int(wq.dtype), wq.ptr, qd + kvd, qk.data_ptr(), int(wv.dtype), wv.ptr,
                                                                            kvd, v.data_ptr(), cur, part.data_ptr(),
                                                                            lw.attention_norm.data_ptr(), cfg.rms_eps, cfg.hidden, sp))
            elif wq.dtype == wk.dtype and wk.ptr == wq.ptr + wq.nbytes:
                norm_mm(wq, qd + kvd, lw.attention_norm, qk.data_ptr())
                norm_mm(wv, kvd, lw.attention_norm, v.data_ptr())
            else:
                norm_mm(wq, qd, lw.attention_norm, qk.data_ptr())
                norm_mm(wk, kvd, lw.attention_norm, qk.data_ptr() + 4 * qd)
                norm_mm(wv, kvd, lw.attention_norm, v.data_ptr())
            tap("qkv", li)
            q_ptr, k_ptr = qk.data_ptr(), qk.data_ptr() + 4 * qd
            # rope, cache append, attention and the merge of the key splits in one kernel          :217-261
            wo = w["attention_wo"]
            # the attention kernel merges its key splits itself (the last workgroup of a kv head does it once); merging in
            # the prologue of attention_wo instead makes every workgroup of that matvec read every partial
            merge_in_wo = self.merge_in_wo and wo.dtype in full and qd <= (4096 if wo.dtype in kq else 2048) and \
                (cfg.head_dim & (cfg.head_dim - 1)) == 0 and L.cq_nn_attention_decode_splits(max_kv_len) <= 16
            ck("cq_nn_attention_decode", L.cq_nn_attention_decode(q_ptr, k_ptr, v.data_ptr(), lw.k_cache.data_ptr(), lw.v_cache.data_ptr(),
                                                                  self.cos.data_ptr(), self.sin.data_ptr(),
                                                                  None if merge_in_wo else att.data_ptr(), pos_dev_ptr, pos,
                                                                  cfg.n_head, cfg.n_kv_head, cfg.head_dim, cfg.ctx, max_kv_len, scale,
                                                                  self.attd_ws.data_ptr(), self.attd_ws.numel(),
                                                                  wo.ptr if self.prefetch_bytes else None,
                                                                  min(self.prefetch_bytes, lw.prefetch_span) // 16 * 16,
                                                                  L.cq_qmatmul_stream_step_bytes(int(wo.dtype), wo.k, wo.n), sp))
            tap("attention", li)
            # attention_wo adds to the residual row, and folds the pending planes into it
            if merge_in_wo:
                ck("cq_nn_qmatmul_residual_attn_merge", L.cq_nn_qmatmul_residual_attn_merge(
                    int(wo.dtype), wo.ptr, self.attd_ws.data_ptr() + 256, L.cq_nn_attention_decode_splits(max_kv_len), cfg.head_dim, cur,
                    part.data_ptr(), planes.data_ptr() if pending else None, pending, wo.k, cfg.hidden, sp))
            else:
                resid_mm(wo, att.data_ptr(), None)
            pending = 0
            tap("attention_wo", li)
            w1, w3, w2 = w["feed_forward_w1"], w["feed_forward_w3"], w["feed_forward_w2"]
            # the consumers of this layer's residual row: the next layer's q / k / v projections, or the output head
            nxt = self.layers[li + 1].w if li + 1 < len(self.layers) else None
            consumers = [nxt["attention_wq"], nxt["attention_wk"], nxt["attention_wv"]] if nxt else [self.output]
            n_split = L.cq_nn_qmatmul_split_planes(int(w2.dtype), w2.k) if self.split_w2 and all_full and cfg.hidden <= 4096 and \
                all(one_step(c) for c in consumers) else 0
            if self.coop and not n_split and w1.dtype == w3.dtype and self.tap is None:
                # both matvecs of the feed-forward in one cooperative launch (CQ_ERR_RANGE: no kernel for these formats / shapes)
                rc = L.cq_nn_decode_mlp(int(w1.dtype), w1.ptr, w3.ptr, int(w2.dtype), w2.ptr, cur, part.data_ptr(), lw.ffn_norm.data_ptr(),
                                        cfg.rms_eps, self.h.data_ptr(), cfg.hidden, cfg.ffn, self._coop_sync().data_ptr(), sp)
                if rc == 0:
                    continue
                if rc != -6:
                    ck("cq_nn_decode_mlp", rc)
            if w1.dtype == w3.dtype and w1.dtype in full and one_step(w1):
                # h = silu(w1 xn) * (w3 xn) straight out of the paired-row matvec                    :56-63
                ck("cq_nn_qmatmul_norm_swiglu", L.cq_nn_qmatmul_norm_swiglu(int(w1.dtype), w1.ptr, w3.ptr, cur, part.data_ptr(),
                                                                            lw.ffn_norm.data_ptr(), cfg.rms_eps, self.h.data_ptr(), cfg.hidden,
                                                                            cfg.ffn, sp))
                src_ptr, up_ptr = self.h.data_ptr(), None
            else:
                norm_mm(w1, cfg.ffn, lw.ffn_norm, gu.data_ptr())
                norm_mm(w3, cfg.ffn, lw.ffn_norm, gu.data_ptr() + 4 * cfg.ffn)
                src_ptr, up_ptr = gu.data_ptr(), gu.data_ptr() + 4 * cfg.ffn
            tap("w13", li)
            if n_split:
                ck("cq_nn_qmatmul_split", L.cq_nn_qmatmul_split(int(w2.dtype), w2.ptr, src_ptr, up_ptr, planes.data_ptr(), w2.k, cfg.hidden, sp))
                pending = n_split
            else:
                resid_mm(w2, src_ptr, up_ptr)
            tap("w2", li)
        norm_mm(self.output, cfg.vocab, self.norm, self.logits.data_ptr())
        tap("head", -1)

    def _coop_sync(self) -> torch.Tensor:
        if self.coop_sync is None:
            self.coop_sync = torch.zeros(self.L.cq_nn_coop_sync_bytes() // 4, dtype=torch.int32, device=self.device)
        return self.coop_sync

    def coop_error(self) -> bool:
        """Whether a cooperative launch since the last call gave up waiting (synchronizes).  The steps enqueued since then are
        invalid; the sync words are cleared so that cooperative launches can be used again."""
        if self.coop_sync is None:
            return False
        bad = bool(int(self.coop_sync[1056]) != 0)          # CQ_NN_COOP_ERR_WORD
        if bad:
            self.coop_sync.zero_()
            torch.cuda.synchronize(self.device)
        return bad

    def forward(self, x: torch.Tensor, index_pos: int) -> torch.Tensor:
        """ModelWeights::forward: token ids [1, seq_len] at positions index_pos.. -> logits [1, vocab] of the last token."""
        if x.dim() != 2 or x.shape[0] != 1:
            raise ValueError(f"expected token ids of shape (1, seq_len), got {tuple(x.shape)}")
        rows = int(x.shape[1])
        if rows == 0 or index_pos < 0 or index_pos + rows > self.cfg.ctx:
            raise ValueError(f"positions {index_pos}..{index_pos + rows} outside the context of {self.cfg.ctx}")
        if rows > self.max_rows:
            self._alloc_activations(rows)
        ids = x.to(device=self.device, dtype=torch.int32).contiguous()
        sp = torch.cuda.current_stream(self.device).cuda_stream
        self._enqueue(ids.data_ptr(), rows, index_pos, None, index_pos + rows, sp)
        if rows == 1 and self.coop and self.coop_sync is not None and self.coop_error():
            # a cooperative launch gave up waiting (the GPU is shared, or fewer compute units than workgroups were free):
            # the same step through the chain of launches
            self.coop = False
            try:
                self._enqueue(ids.data_ptr(), rows, index_pos, None, index_pos + rows, sp)
            finally:
                self.coop = True
        return self.logits.clone()

    # ------------------------------------------------------------------------------------------ greedy decode
    def _chain_embedding(self, max_kv_len: int) -> bool:
        """Whether the greedy steps hand the next token's embedding row over in place (the fused single-token path)."""
        return bool(self.fuse_decode and self.L.cq_nn_attention_decode_splits(max_kv_len) > 0)

    def _argmax_dev(self, logits_ptr: int, embed: bool, sp) -> None:
        """Sampling::ArgMax into token_dev / history_dev, the position advanced; with `embed` the chosen token's embedding row
        and its partial sums of squares go to self.x / self.partials in the same launch."""
        L, cfg = self.L, self.cfg
        if embed:
            _lib.check("cq_nn_argmax_embed", L.cq_nn_argmax_embed(logits_ptr, cfg.vocab, self.token_dev.data_ptr(), self.history_dev.data_ptr(),
                                                                 self.counter_dev.data_ptr(), self.pos_dev.data_ptr(), self.argmax_ws.data_ptr(),
                                                                 self.tok_embeddings.data_ptr(), self.x.data_ptr(), cfg.hidden, cfg.vocab,
                                                                 self.partials.data_ptr(), sp))
        else:
            _lib.check("cq_nn_argmax", L.cq_nn_argmax(logits_ptr, cfg.vocab, self.token_dev.data_ptr(), self.history_dev.data_ptr(),
                                                     self.counter_dev.data_ptr(), self.pos_dev.data_ptr(), self.argmax_ws.data_ptr(), sp))

    def _decode_step_dev(self, max_kv_len: int, sp) -> None:
        """One greedy step driven entirely from device state: token_dev at position pos_dev -> next token_dev, pos_dev + 1.
        On the fused path the step starts from the embedding row the previous arg-max left in self.x and leaves the next one."""
        chain = self._chain_embedding(max_kv_len)
        self._enqueue(None if chain else self.token_dev.data_ptr(), 1, 0, self.pos_dev.data_ptr(), max_kv_len, sp)
        self._argmax_dev(self.logits.data_ptr(), chain, sp)

    def generate_greedy(self, prompt: Sequence[int], n_new: int, use_graph: bool = True, max_kv: Optional[int] = None) -> dict:
        """The loop of candle-examples/examples/quantized/main.rs:616-690 with temperature <= 0 (Sampling::ArgMax):
        prefill the prompt in one forward, pick the arg-max token, then n_new - 1 single-token steps.
        Returns the generated tokens and the wall-clock split prompt / decode, as the example prints them.
        max_kv: the number of cache positions the captured step is laid out for (its attention split count follows from
        it); by default exactly prompt + n_new, a server that captures one step for every request passes the context."""
        cfg = self.cfg
        prompt = [int(t) for t in prompt]
        if len(prompt) + n_new > cfg.ctx:
            raise ValueError("prompt + generated tokens exceed the context")
        if max_kv is not None and not len(prompt) + n_new <= max_kv <= cfg.ctx:
            raise ValueError("max_kv must cover prompt + generated tokens and fit the context")
        dev = self.device
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        logits = self.forward(torch.tensor([prompt], dtype=torch.int32, device=dev), 0)
        stream = torch.cuda.current_stream(dev)
        self.counter_dev.zero_()
        self.pos_dev.fill_(len(prompt) - 1)       # argmax advances it to the position of the token it emits
        steps = n_new - 1
        if max_kv is None:
            max_kv = len(prompt) + n_new
        self._argmax_dev(logits.data_ptr(), steps > 0 and self._chain_embedding(max_kv), stream.cuda_stream)
        torch.cuda.synchronize(dev)
        t1 = time.perf_counter()
        prompt_seconds = t1 - t0
        if steps > 0:
            if use_graph:
                key = max_kv
                if self._graph is None or self._graph_key != key:
                    side = torch.cuda.Stream(device=dev)
                    # capture must not disturb the live decode state: save and restore it around the warm-up run
                    saved = (self.token_dev.clone(), self.pos_dev.clone(), self.counter_dev.clone(), self.x[:1].clone(), self.partials.clone())
                    with torch.cuda.stream(side):
                        self._decode_step_dev(max_kv, side.cuda_stream)
                        side.synchronize()
                        g = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(g, stream=side):
                            self._decode_step_dev(max_kv, torch.cuda.current_stream(dev).cuda_stream)
                    torch.cuda.synchronize(dev)
                    self.token_dev.copy_(saved[0]); self.pos_dev.copy_(saved[1]); self.counter_dev.copy_(saved[2])
                    self.x[:1].copy_(saved[3]); self.partials.copy_(saved[4])
                    torch.cuda.synchronize(dev)
                    self._graph, self._graph_key = g, key
                t1 = time.perf_counter()
                for _ in range(steps):
                    self._graph.replay()
            else:
                for _ in range(steps):
                    self._decode_step_dev(max_kv, stream.cuda_stream)
        torch.cuda.synchronize(dev)
        t2 = time.perf_counter()
        if self.coop and self.coop_error():
            # a cooperative launch gave up waiting for workgroups that were not running (a shared GPU): its tokens are invalid.
            # The whole generation again through the chains of launches, which this model then keeps to.
            import warnings
            warnings.warn("a cooperative decode launch timed out; falling back to one launch per matvec")
            self.coop = False
            self._graph = None
            return self.generate_greedy(prompt, n_new, use_graph)
        tokens = self.history_dev[:n_new].cpu().tolist()
        return {"tokens": tokens, "prompt_seconds": prompt_seconds, "decode_seconds": t2 - t1, "decode_steps": steps}
