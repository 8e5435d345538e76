"""CPU restatement (numpy, f32) of candle's fused MoE layer over GGUF experts.  TEST INFRASTRUCTURE ONLY: imported by
tests/ and the benchmark's checker, never by the product path.

Follows candle-transformers/src/fused_moe.rs:222-301 (FusedMoeGGUF::forward) step by step:
  :233      router_logits = gate.forward(xs)            bias-free f32 Linear, weight [num_experts, hidden]
  :235-236  routing_weights = softmax_last_dim(logits)  candle-nn/src/ops.rs:270-300 (llama_oracle.softmax_last_dim)
  :238-241  topk_ids = arg_sort_last_dim(descending)[:topk]   candle-core/src/sort.rs:48-53: a stable sort_by with the
            comparison reversed, so equal probabilities keep their index order (lower expert first)
  :243      topk_weights = routing_weights.gather(topk_ids)
  :245-247  norm_topk_prob: topk_weights / topk_weights.sum(-1)
  :249-260  (expert_ids, sorted_token_ids) = topk_ids.flatten().sort_last_dim(ascending); candle's sort is unstable
            (sort.rs:282-297): the order inside an expert's segment is unspecified, a stable one is used here
  :263-294  gate = moe_gemm_gguf(xs, gate_experts, None), up likewise, down = moe_gemm_gguf(up * silu(gate),
            down_experts, topk_weights): oracle.moe_gemm_gguf (candle-nn/src/moe.rs:169-337 with the CPU path's
            activation quantization)
  :296      ys.reshape(tokens, topk, hidden).sum(-2)

Pinned by tests/test_oracle_fused_moe.py: the routing against closed forms (a one-hot router gives known logits, the
softmax and top-k of small hand-made rows, ties, renormalised weights summing to one), and the whole layer against the
dense definition sum_j w_j * down_e(silu(gate_e x) * up_e x) evaluated expert by expert with the pinned oracle.matmul,
plus invariance under any reordering of the pairs inside an expert's segment.  The reference holds no golden outputs
for this layer (its only callers need downloaded GGUF files).
"""
from __future__ import annotations

import numpy as np

import oracle
from oracle.llama_oracle import silu, softmax_last_dim

f32 = np.float32


def route(xs: np.ndarray, router_w: np.ndarray, topk: int, norm_topk_prob: bool):
    """fused_moe.rs:233-247 -> (topk_ids u32 [tokens, topk], topk_weights f32 [tokens, topk])."""
    xs = np.asarray(xs, dtype=f32)
    logits = np.matmul(xs, np.asarray(router_w, dtype=f32).T).astype(f32)
    probs = softmax_last_dim(logits)
    # descending, equal values in index order: a stable ascending sort of the negated values
    order = np.argsort(-probs, axis=-1, kind="stable")
    topk_ids = np.ascontiguousarray(order[:, :topk]).astype(np.uint32)
    topk_weights = np.take_along_axis(probs, topk_ids.astype(np.int64), axis=-1).astype(f32)
    if norm_topk_prob:
        s = np.zeros((xs.shape[0], 1), dtype=f32)
        for j in range(topk):                       # sum_keepdim over the last dim, in slot order
            s = (s + topk_weights[:, j:j + 1]).astype(f32)
        topk_weights = (topk_weights / s).astype(f32)
    return topk_ids, topk_weights


def sort_pairs(topk_ids: np.ndarray):
    """fused_moe.rs:249-260 -> (expert_ids int32 [n_pairs], sorted_token_ids int32 [n_pairs])."""
    flat = np.asarray(topk_ids, dtype=np.uint32).reshape(-1)
    idx = np.argsort(flat, kind="stable")
    return flat[idx].astype(np.int32), idx.astype(np.int32)


class FusedMoeOracle:
    """gate_w f32 [E, hidden]; *_blocks uint8 GGUF blocks of [E, inter, hidden] (gate, up) and [E, hidden, inter] (down)."""

    def __init__(self, dtype: int, gate_w, gate_blocks, up_blocks, down_blocks, num_experts: int, hidden: int, inter: int, topk: int,
                 norm_topk_prob: bool):
        self.dtype, self.E, self.hidden, self.inter, self.topk, self.norm = int(dtype), num_experts, hidden, inter, topk, norm_topk_prob
        self.gate_w = np.asarray(gate_w, dtype=f32)
        self.gate_blocks, self.up_blocks, self.down_blocks = gate_blocks, up_blocks, down_blocks

    def forward(self, xs: np.ndarray, pair_order=None) -> np.ndarray:
        """xs [batch, seq, hidden] f32 -> [batch, seq, hidden].  pair_order(expert_ids, sorted_token_ids) may permute the
        pairs inside the expert segments (to show that nothing depends on that order)."""
        xs = np.asarray(xs, dtype=f32)
        batch, seq, hidden = xs.shape
        x2 = xs.reshape(-1, hidden)
        tokens = x2.shape[0]
        topk_ids, topk_weights = route(x2, self.gate_w, self.topk, self.norm)
        expert_ids, sorted_token_ids = sort_pairs(topk_ids)
        if pair_order is not None:
            expert_ids, sorted_token_ids = pair_order(expert_ids, sorted_token_ids)
        gate = oracle.moe_gemm_gguf(self.dtype, x2, self.gate_blocks, (self.E, self.inter, hidden), sorted_token_ids, expert_ids, None, self.topk)
        up = oracle.moe_gemm_gguf(self.dtype, x2, self.up_blocks, (self.E, self.inter, hidden), sorted_token_ids, expert_ids, None, self.topk)
        down_in = (up * silu(gate)).astype(f32)
        down = oracle.moe_gemm_gguf(self.dtype, down_in, self.down_blocks, (self.E, hidden, self.inter), sorted_token_ids, expert_ids,
                                    topk_weights.reshape(-1), self.topk)
        ys = down.reshape(tokens, self.topk, hidden)
        acc = ys[:, 0, :].copy()
        for j in range(1, self.topk):
            acc = (acc + ys[:, j, :]).astype(f32)
        return acc.reshape(batch, seq, hidden)
