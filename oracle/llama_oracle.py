"""CPU restatement (numpy, f32) of candle's quantized llama decoder and of the f32 ops around its quantized
matmuls.  TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke test and the benchmark's checker, never
by the product path.

Follows, function by function:
  rms_norm            candle-nn/src/ops.rs:499-510 (CPU kernel of candle_nn::ops::rms_norm)
  softmax_last_dim    candle-nn/src/ops.rs:270-300 (max, exp, sum, divide)
  silu                candle-core/src/op.rs, Silu::f32: v / (1 + exp(-v))
  rope_i              candle-nn/src/rotary_emb.rs:52-70 (interleaved pairs)
  precomput_freqs_cis candle-transformers/src/models/quantized_llama.rs:284-300
  LlamaOracle.forward quantized_llama.rs:568-596 with LayerWeights::forward_attn :191-266 and Mlp :56-63;
                      every QMatMul::forward is the C oracle's k_quants matmul (oracle.matmul)

Pinned by tests/test_oracle_llama.py: the reference's known answers for softmax and rms_norm
(candle-nn/tests/ops.rs:9-78, 191-196), rope_i against the independent reshape formulation of
rope_i_slow (rotary_emb.rs:290-308) on the seeded inputs of ops.rs:199-216, rotation invariants, and for
the decoder the properties the architecture fixes (prefill == token-by-token decode, a single-token
sequence attends only itself, zeroed output projections reduce the model to head(norm(embedding))).
The reference holds no golden logits for this model (its tests need downloaded GGUF files), so the
decoder's absolute outputs are pinned only through those properties and the pinned parts.
"""
from __future__ import annotations

import math

import numpy as np

import oracle

f32 = np.float32


def rms_norm(x: np.ndarray, alpha: np.ndarray, eps: float) -> np.ndarray:
    x = np.asarray(x, dtype=f32)
    out = np.empty_like(x)
    flat, oflat = x.reshape(-1, x.shape[-1]), out.reshape(-1, x.shape[-1])
    n = x.shape[-1]
    for r in range(flat.shape[0]):
        sum2 = f32(0)
        sq = flat[r] * flat[r]
        for v in sq:                      # sequential f32 sum, as Iterator::sum
            sum2 = f32(sum2 + v)
        m = f32(np.sqrt(f32(f32(sum2 / f32(n)) + f32(eps))))
        oflat[r] = (flat[r] / m) * alpha.astype(f32)
    return out


def softmax_last_dim(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=f32)
    m = np.max(x, axis=-1, keepdims=True)
    e = np.exp((x - m).astype(f32)).astype(f32)
    s = np.sum(e, axis=-1, keepdims=True, dtype=f32)
    return (e / s).astype(f32)


def silu(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=f32)
    return (x / (f32(1) + np.exp(-x).astype(f32))).astype(f32)


def rope_i(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [b, h, t, d]; cos, sin [t, d/2]; pairs (2i, 2i+1)."""
    x = np.asarray(x, dtype=f32)
    out = np.empty_like(x)
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out[..., 0::2] = x0 * cos - x1 * sin
    out[..., 1::2] = x0 * sin + x1 * cos
    return out


def precomput_freqs_cis(head_dim: int, freq_base: float, max_seq_len: int):
    i = np.arange(0, head_dim, 2, dtype=f32)
    theta = (f32(1.0) / np.power(f32(freq_base), i / f32(head_dim))).astype(f32)
    idx = np.arange(max_seq_len, dtype=f32).reshape(-1, 1)
    idx_theta = (idx * theta.reshape(1, -1)).astype(f32)
    return np.cos(idx_theta).astype(f32), np.sin(idx_theta).astype(f32)


class LlamaOracle:
    """tensors: the dictionary candle_amd.quantized_llama.ModelWeights.from_blocks takes."""

    def __init__(self, cfg, tensors: dict, threads: int = 0):
        self.cfg, self.t, self.threads = cfg, tensors, threads
        self.cos, self.sin = precomput_freqs_cis(cfg.head_dim, cfg.rope_theta, cfg.ctx)
        self.kv = [None] * cfg.n_layer

    def qmatmul(self, name: str, x: np.ndarray, n: int) -> np.ndarray:
        dt, blocks = self.t[name]
        blocks = np.frombuffer(bytes(blocks), dtype=np.uint8)
        x = np.ascontiguousarray(x, dtype=f32)
        if self.threads:
            return oracle.matmul_fast(int(dt), x, blocks, n, self.threads)
        return oracle.matmul(int(dt), x, blocks, n)

    def forward(self, tokens, index_pos: int) -> np.ndarray:
        cfg = self.cfg
        tokens = np.asarray(tokens).reshape(-1)
        seq = tokens.shape[0]
        H, KV, D = cfg.n_head, cfg.n_kv_head, cfg.head_dim
        x = np.asarray(self.t["tok_embeddings"])[np.asarray(tokens, dtype=np.int64)].astype(f32)                        # [seq, hidden]
        cos, sin = self.cos[index_pos:index_pos + seq], self.sin[index_pos:index_pos + seq]
        scale = f32(1.0 / math.sqrt(D))
        for li in range(cfg.n_layer):
            p = f"blk.{li}."
            residual = x
            xn = rms_norm(x, self.t[p + "attention_norm"], cfg.rms_eps)
            q = self.qmatmul(p + "attention_wq", xn, H * D).reshape(seq, H, D).transpose(1, 0, 2)      # [H, seq, D]
            k = self.qmatmul(p + "attention_wk", xn, KV * D).reshape(seq, KV, D).transpose(1, 0, 2)
            v = self.qmatmul(p + "attention_wv", xn, KV * D).reshape(seq, KV, D).transpose(1, 0, 2)
            q = rope_i(q[None], cos, sin)[0]
            k = rope_i(k[None], cos, sin)[0]
            if index_pos > 0 and self.kv[li] is not None:
                k = np.concatenate([self.kv[li][0], k], axis=1)
                v = np.concatenate([self.kv[li][1], v], axis=1)
            self.kv[li] = (k, v)
            rep = H // KV
            kr, vr = np.repeat(k, rep, axis=0), np.repeat(v, rep, axis=0)                             # repeat_kv
            att = (np.matmul(q, kr.transpose(0, 2, 1)).astype(f32) * scale).astype(f32)                # [H, seq, kv_len]
            if seq > 1:
                kv_len = k.shape[1]
                i = np.arange(seq).reshape(-1, 1)
                j = np.arange(kv_len).reshape(1, -1)
                att = np.where(j > i + index_pos, f32(-np.inf), att)                                  # build_causal_mask
            att = softmax_last_dim(att)
            y = np.matmul(att, vr).astype(f32).transpose(1, 0, 2).reshape(seq, H * D)
            attn = self.qmatmul(p + "attention_wo", y, cfg.hidden)
            x = (attn + residual).astype(f32)
            residual = x
            xn = rms_norm(x, self.t[p + "ffn_norm"], cfg.rms_eps)
            w1 = self.qmatmul(p + "feed_forward_w1", xn, cfg.ffn)
            w3 = self.qmatmul(p + "feed_forward_w3", xn, cfg.ffn)
            mlp = self.qmatmul(p + "feed_forward_w2", (silu(w1) * w3).astype(f32), cfg.hidden)
            x = (mlp + residual).astype(f32)
        xn = rms_norm(x, self.t["norm"], cfg.rms_eps)
        return self.qmatmul("output", xn[-1:], cfg.vocab)                                             # [1, vocab]


def random_tensors(cfg, seed: int, dtypes: dict, weight_scale: float = 0.02, norm_jitter: float = 0.1) -> dict:
    """Seeded synthetic weights quantized by the C oracle's from_float (names as ModelWeights.from_blocks expects)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    qd, kvd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim
    shapes = {"attention_wq": (qd, cfg.hidden), "attention_wk": (kvd, cfg.hidden), "attention_wv": (kvd, cfg.hidden),
              "attention_wo": (cfg.hidden, qd), "feed_forward_w1": (cfg.ffn, cfg.hidden), "feed_forward_w3": (cfg.ffn, cfg.hidden),
              "feed_forward_w2": (cfg.hidden, cfg.ffn)}
    t = {}
    for li in range(cfg.n_layer):
        for name, (n, k) in shapes.items():
            w = (rng.standard_normal((n, k), dtype=f32) * f32(weight_scale)).astype(f32)
            t[f"blk.{li}.{name}"] = (int(dtypes[name]), oracle.from_float(int(dtypes[name]), w.reshape(-1)).tobytes())
        t[f"blk.{li}.attention_norm"] = (1.0 + norm_jitter * rng.standard_normal(cfg.hidden, dtype=f32)).astype(f32)
        t[f"blk.{li}.ffn_norm"] = (1.0 + norm_jitter * rng.standard_normal(cfg.hidden, dtype=f32)).astype(f32)
    w = (rng.standard_normal((cfg.vocab, cfg.hidden), dtype=f32) * f32(weight_scale)).astype(f32)
    t["output"] = (int(dtypes["output"]), oracle.from_float(int(dtypes["output"]), w.reshape(-1)).tobytes())
    t["tok_embeddings"] = rng.standard_normal((cfg.vocab, cfg.hidden), dtype=f32).astype(f32)
    t["norm"] = (1.0 + norm_jitter * rng.standard_normal(cfg.hidden, dtype=f32)).astype(f32)
    return t
