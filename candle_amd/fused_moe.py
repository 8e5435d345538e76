"""Host-side mirror of candle's fused MoE layer over GGUF experts (candle-transformers/src/fused_moe.rs:163-303,
``FusedMoeGGUF``) on the HIP library: router + softmax + top-k, the sort of the (token, slot) pairs by expert, three
expert-grouped quantized matmuls, ``silu(gate) * up`` and the sum over the top-k slots.

Everything runs on the caller's stream from preallocated buffers (sized for the largest token count seen so far), so a
forward can be captured in a HIP graph.  The HIP extension is required: there is no CPU or torch fallback.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .quantized import GgmlDType, QTensor


class FusedMoeGGUF:
    """fused_moe.rs:163-175.  gate: router weight f32 [num_experts, hidden] (``ffn_gate_inp``, dequantized at load time
    like :186-190); gate_experts / up_experts: QTensor [num_experts, moe_intermediate, hidden]; down_experts: QTensor
    [num_experts, hidden, moe_intermediate]."""

    def __init__(self, gate: torch.Tensor, gate_experts: QTensor, up_experts: QTensor, down_experts: QTensor, norm_topk_prob: bool,
                 num_experts_per_tok: int, act: str = "silu"):
        if act != "silu":
            raise ValueError("only the silu activation of the reference's MoE configurations is implemented")
        if not gate.is_cuda or gate.dtype != torch.float32 or gate.dim() != 2:
            raise ValueError("gate must be an f32 [num_experts, hidden] tensor on the GPU")
        E, hidden = gate.shape
        ge, ue, de = gate_experts.shape(), up_experts.shape(), down_experts.shape()
        if len(ge) != 3 or ge != ue or ge[0] != E or ge[2] != hidden or de != (E, hidden, ge[1]):
            raise ValueError(f"expert shapes {ge}, {ue}, {de} do not fit a router of shape {tuple(gate.shape)}")
        if not (gate_experts.dtype() == up_experts.dtype() == down_experts.dtype()):
            raise ValueError("gate, up and down experts must share one block format")
        if not 0 < num_experts_per_tok <= E:
            raise ValueError("num_experts_per_tok out of range")
        self.gate = gate.contiguous()
        self.gate_experts, self.up_experts, self.down_experts = gate_experts, up_experts, down_experts
        self.norm_topk_prob = bool(norm_topk_prob)
        self.num_experts_per_tok = int(num_experts_per_tok)
        self.num_experts, self.hidden, self.inter = int(E), int(hidden), int(ge[1])
        self.w_dtype = gate_experts.dtype()
        self.L = _lib.lib()
        self._cap = 0
        # hundreds of pairs: the down projection reuses the grouping of the gate / up call and folds up * silu(gate) into its
        # activation quantizer (False: silu_mul and a moe_gemm_gguf call of its own; the same bits)
        self.share_grouping = True
        self.sort_pairs = False

    def _reserve(self, tokens: int) -> None:
        if tokens <= self._cap:
            return
        dev, topk = self.gate.device, self.num_experts_per_tok
        pairs = tokens * topk
        f32 = dict(dtype=torch.float32, device=dev)
        self.topk_ids = torch.empty((tokens, topk), dtype=torch.int32, device=dev)        # u32 values
        self.topk_weights = torch.empty((tokens, topk), **f32)
        self.router_logits = torch.empty((tokens, self.num_experts), **f32)
        self.expert_ids = torch.empty(pairs, dtype=torch.int32, device=dev)
        self.sorted_token_ids = torch.empty(pairs, dtype=torch.int32, device=dev)
        self.pair_iota = torch.arange(pairs, dtype=torch.int32, device=dev)
        self.gate_out = torch.empty((pairs, self.inter), **f32)
        self.up_out = torch.empty((pairs, self.inter), **f32)
        self.down_in = torch.empty((pairs, self.inter), **f32)
        self.down_out = torch.empty((pairs, self.hidden), **f32)
        L, dt, E = self.L, int(self.w_dtype), self.num_experts
        need = max(L.cq_moe_gemm_workspace_bytes(dt, E, topk, pairs, self.inter, self.hidden, 0),
                   L.cq_moe_gemm_workspace_bytes(dt, E, topk, pairs, self.hidden, self.inter, 1))
        if need < 0:
            raise ValueError("unsupported expert shape")
        self.ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        self._cap = tokens

    def forward(self, xs: torch.Tensor, is_prefill: bool, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fused_moe.rs:222-301.  xs [batch, seq_len, hidden] -> [batch, seq_len, hidden] in the dtype of xs."""
        if xs.dim() != 3 or xs.shape[2] != self.hidden:
            raise ValueError(f"expected [batch, seq_len, {self.hidden}], got {tuple(xs.shape)}")
        if not xs.is_cuda:
            raise ValueError("xs must be on the GPU")
        batch, seq_len, hidden = xs.shape
        original_dtype = xs.dtype
        x2 = xs.reshape(-1, hidden).to(torch.float32).contiguous()
        tokens, topk = x2.shape[0], self.num_experts_per_tok
        pairs = tokens * topk
        ys = out if out is not None else torch.empty((tokens, hidden), dtype=torch.float32, device=xs.device)
        if tokens == 0:
            return ys.reshape(batch, seq_len, hidden).to(original_dtype)
        self._reserve(tokens)
        L, ck, dt, E = self.L, _lib.check, int(self.w_dtype), self.num_experts
        sp = torch.cuda.current_stream(xs.device).cuda_stream
        for t0 in range(0, tokens, 65535):
            t = min(65535, tokens - t0)
            ck("cq_nn_moe_route", L.cq_nn_moe_route(x2.data_ptr() + 4 * t0 * hidden, self.gate.data_ptr(), self.topk_ids.data_ptr() + 4 * t0 * topk,
                                                    self.topk_weights.data_ptr() + 4 * t0 * topk, self.router_logits.data_ptr() + 4 * t0 * E,
                                                    t, hidden, E, topk, 1 if self.norm_topk_prob else 0, sp))
        # (expert_ids, sorted_token_ids) of fused_moe.rs:249-260.  Every path of the expert matmuls gives each pair a row of its
        # own whatever the order of the pair list (decode-sized calls run each pair as its own matvec launch block, larger ones
        # bucket the pairs by expert themselves), so the layer does not sort: the pairs are taken in token order
        # (expert_ids = topk_ids, sorted_token_ids = 0, 1, 2, ...).  sort_pairs = True runs candle's sort (cq_nn_moe_sort) anyway;
        # the results are the same bits.
        direct = bool(L.cq_moe_direct_pairs(dt, E, pairs, max(hidden, self.inter)))
        if not self.sort_pairs:
            eid_ptr, sti_ptr = self.topk_ids.data_ptr(), self.pair_iota.data_ptr()
        else:
            ck("cq_nn_moe_sort", L.cq_nn_moe_sort(self.topk_ids.data_ptr(), self.expert_ids.data_ptr(), self.sorted_token_ids.data_ptr(), pairs, E,
                                                  sp))
            eid_ptr, sti_ptr = self.expert_ids.data_ptr(), self.sorted_token_ids.data_ptr()

        def gemm(x_ptr, w: QTensor, tw_ptr, out_t, n, k):
            ck("cq_moe_gemm_gguf", L.cq_moe_gemm_gguf(dt, x_ptr, w.device_ptr(), sti_ptr, eid_ptr, tw_ptr, out_t.data_ptr(), E, topk, pairs, n, k,
                                                      1 if is_prefill else 0, self.ws.data_ptr(), self.ws.numel(), sp))

        # decode-sized calls: gate, up and the activation in one launch
        fused = -6
        if direct:
            fused = L.cq_moe_gemm_gguf_swiglu(dt, x2.data_ptr(), self.gate_experts.device_ptr(), self.up_experts.device_ptr(), sti_ptr, eid_ptr,
                                              self.down_in.data_ptr(), E, topk, pairs, self.inter, hidden, sp)
            if fused != -6:
                ck("cq_moe_gemm_gguf_swiglu", fused)
        down_done = False
        if fused == -6:                                          # CQ_ERR_RANGE: not a shape of the fused launch
            # gate and up share x and the pairs: one grouping pass and one activation quantization for both
            ck("cq_moe_gemm_gguf_pair", L.cq_moe_gemm_gguf_pair(dt, x2.data_ptr(), self.gate_experts.device_ptr(), self.up_experts.device_ptr(),
                                                                sti_ptr, eid_ptr, self.gate_out.data_ptr(), self.up_out.data_ptr(), E, topk, pairs,
                                                                self.inter, hidden, 1 if is_prefill else 0, self.ws.data_ptr(), self.ws.numel(), sp))
            # the down projection on the grouping that call left in the workspace, up * silu(gate) inside its activation quantizer
            rc = -6 if not self.share_grouping else L.cq_moe_gemm_gguf_down_after_pair(dt, self.gate_out.data_ptr(), self.up_out.data_ptr(), self.down_experts.device_ptr(),
                                                    self.topk_weights.data_ptr(), self.down_out.data_ptr(), E, topk, pairs, hidden, self.inter,
                                                    hidden, self.ws.data_ptr(), self.ws.numel(), sp)
            if rc != -6:
                ck("cq_moe_gemm_gguf_down_after_pair", rc)
                down_done = True
            else:
                # up * silu(gate), in chunks of rows the elementwise launch takes
                for r0 in range(0, pairs, 65535):
                    r = min(65535, pairs - r0)
                    off = 4 * r0 * self.inter
                    ck("cq_nn_silu_mul", L.cq_nn_silu_mul(self.gate_out.data_ptr() + off, self.up_out.data_ptr() + off, self.down_in.data_ptr() + off,
                                                          r, self.inter, self.inter, self.inter, sp))
        if not down_done:
            gemm(self.down_in.data_ptr(), self.down_experts, self.topk_weights.data_ptr(), self.down_out, hidden, self.inter)
        for t0 in range(0, tokens, 65535):
            t = min(65535, tokens - t0)
            ck("cq_nn_moe_sum", L.cq_nn_moe_sum(self.down_out.data_ptr() + 4 * t0 * topk * hidden, ys.data_ptr() + 4 * t0 * hidden, t, topk, hidden, sp))
        ys = ys.reshape(batch, seq_len, hidden)
        return ys if original_dtype == torch.float32 else ys.to(original_dtype)
