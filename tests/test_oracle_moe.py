"""Pins the oracle's MoE compositions by brute force against per-pair calls of the pinned matmul.

The reference has no CPU implementation of indexed_moe_forward / moe_gemm_gguf (mod.rs:776-782
panics off-GPU), so the semantics are taken from the GPU host code (cuda.rs:505-584,
candle-nn/src/moe.rs:169-337, moe_gguf.cu:55-132) and checked here index by index.
"""
import numpy as np
import pytest

import oracle
from tests.util import normal


def expert_slice(blocks, dtype, e, n, k):
    eb = n * (k // oracle.block_size(dtype)) * oracle.type_size(dtype)
    return blocks[e * eb:(e + 1) * eb]


@pytest.mark.parametrize("dtype", [oracle.Q8_0, oracle.Q4K, oracle.Q6K])
@pytest.mark.parametrize("dim1_one", [True, False])
def test_indexed_moe_forward_brute_force(dtype, dim1_one):
    E, n, k, batch, topk = 5, 6, 256, 3, 2
    blocks = oracle.from_float(dtype, normal(1, E * n * k, 0.02))
    ids = np.array([[4, 0], [2, 2], [1, 3]], dtype=np.uint32)
    x = normal(2, (batch, 1 if dim1_one else topk, k), 1.0)
    out = oracle.indexed_moe_forward(dtype, blocks, (E, n, k), x, ids)
    for b in range(batch):
        for t in range(topk):
            row = x[b, 0 if dim1_one else t].reshape(1, k)
            want = oracle.matmul(dtype, row, expert_slice(blocks, dtype, int(ids[b, t]), n, k), n)
            assert np.array_equal(out[b, t], want[0])


@pytest.mark.parametrize("dtype", [oracle.Q8_0, oracle.Q4K, oracle.Q5K])
def test_moe_gemm_brute_force(dtype):
    E, n, k, topk, tokens = 4, 5, 256, 2, 3
    blocks = oracle.from_float(dtype, normal(3, E * n * k, 0.02))
    expert_ids = np.array([0, 0, 1, 3, 3, 9], dtype=np.int32)          # 9 is outside [0, E): skipped
    sorted_token_ids = np.array([4, 1, 0, 5, 2, 3], dtype=np.int32)
    # without topk_weights: input row = tok / topk, scale 1
    x = normal(4, (tokens, k), 1.0)
    out = oracle.moe_gemm_gguf(dtype, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    for m in range(6):
        tok, e = int(sorted_token_ids[m]), int(expert_ids[m])
        if e >= E:
            assert np.all(out[tok] == 0.0)
            continue
        want = oracle.matmul(dtype, x[tok // topk].reshape(1, k), expert_slice(blocks, dtype, e, n, k), n)
        assert np.array_equal(out[tok], want[0])
    # with topk_weights: input row = tok, scale = topk_weights[tok]
    x2 = normal(5, (tokens * topk, k), 1.0)
    tw = normal(6, tokens * topk, 1.0)
    out2 = oracle.moe_gemm_gguf(dtype, x2, blocks, (E, n, k), sorted_token_ids, expert_ids, tw, topk)
    for m in range(6):
        tok, e = int(sorted_token_ids[m]), int(expert_ids[m])
        if e >= E:
            continue
        want = oracle.matmul(dtype, x2[tok].reshape(1, k), expert_slice(blocks, dtype, e, n, k), n)[0] * tw[tok]
        assert np.array_equal(out2[tok], want.astype(np.float32))
