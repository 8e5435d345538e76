"""Pins oracle/fused_moe_oracle.py (the restatement of FusedMoeGGUF::forward, candle-transformers/src/fused_moe.rs:222-301).

The reference holds no golden outputs for the layer, so the routing is checked against closed forms and hand-made
rows, and the whole layer against its dense definition evaluated expert by expert with the already pinned matmul."""
import numpy as np
import pytest

import oracle
from oracle import fused_moe_oracle as fm
from oracle.llama_oracle import silu
from tests.util import normal


def test_route_one_hot_router_closed_form():
    # router row e = unit vector of coordinate e: logits are the first E coordinates of x
    E, hidden, topk = 6, 8, 3
    router = np.zeros((E, hidden), dtype=np.float32)
    router[np.arange(E), np.arange(E)] = 1.0
    x = np.array([[0.5, 2.0, -1.0, 2.0, 0.0, 1.0, 9.0, 9.0]], dtype=np.float32)      # coordinates 6, 7 are not routed on
    ids, w = fm.route(x, router, topk, norm_topk_prob=False)
    # logits [0.5, 2, -1, 2, 0, 1]: the two equal maxima keep their index order (stable descending arg_sort)
    assert ids.tolist() == [[1, 3, 5]]
    z = np.exp(np.array([0.5, 2.0, -1.0, 2.0, 0.0, 1.0]) - 2.0)
    p = z / z.sum()
    assert np.allclose(w[0], p[[1, 3, 5]], rtol=1e-6)
    ids_n, w_n = fm.route(x, router, topk, norm_topk_prob=True)
    assert ids_n.tolist() == [[1, 3, 5]]
    assert np.allclose(w_n[0], p[[1, 3, 5]] / p[[1, 3, 5]].sum(), rtol=1e-6) and abs(float(w_n.sum()) - 1.0) < 1e-6


def test_route_matches_brute_force_on_random_rows():
    E, hidden, topk, tokens = 16, 32, 4, 9
    router, x = normal(1, (E, hidden), 0.3), normal(2, (tokens, hidden), 1.0)
    ids, w = fm.route(x, router, topk, norm_topk_prob=True)
    for t in range(tokens):
        logits = (router.astype(np.float64) @ x[t].astype(np.float64))
        p = np.exp(logits - logits.max())
        p /= p.sum()
        best = sorted(range(E), key=lambda e: (-p[e], e))[:topk]
        assert ids[t].tolist() == best
        assert np.allclose(w[t], p[best] / p[best].sum(), rtol=1e-5)
    assert ids.dtype == np.uint32 and w.dtype == np.float32


def test_sort_pairs_groups_by_expert():
    ids = np.array([[3, 0], [1, 3], [0, 2]], dtype=np.uint32)
    e, s = fm.sort_pairs(ids)
    assert e.tolist() == [0, 0, 1, 2, 3, 3]
    assert sorted(s.tolist()) == list(range(6)) and all(ids.reshape(-1)[s[i]] == e[i] for i in range(6))


def expert_slice(blocks, dtype, e, n, k):
    eb = n * (k // oracle.block_size(dtype)) * oracle.type_size(dtype)
    return blocks[e * eb:(e + 1) * eb]


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q8_0])
@pytest.mark.parametrize("norm", [True, False])
def test_layer_equals_dense_definition_and_ignores_pair_order(dtype, norm):
    E, hidden, inter, topk, tokens = 6, 256, 512, 2, 5
    router = normal(3, (E, hidden), 0.2)
    gate_b = oracle.from_float(dtype, normal(4, E * inter * hidden, 0.05))
    up_b = oracle.from_float(dtype, normal(5, E * inter * hidden, 0.05))
    down_b = oracle.from_float(dtype, normal(6, E * hidden * inter, 0.05))
    x = normal(7, (1, tokens, hidden), 1.0)
    layer = fm.FusedMoeOracle(dtype, router, gate_b, up_b, down_b, E, hidden, inter, topk, norm)
    got = layer.forward(x)
    ids, w = fm.route(x[0], router, topk, norm)
    want = np.zeros((tokens, hidden), dtype=np.float32)
    for t in range(tokens):
        row = x[0, t:t + 1]
        acc = None
        for j in range(topk):
            e = int(ids[t, j])
            g = oracle.matmul(dtype, row, expert_slice(gate_b, dtype, e, inter, hidden), inter)
            u = oracle.matmul(dtype, row, expert_slice(up_b, dtype, e, inter, hidden), inter)
            d = oracle.matmul(dtype, (u * silu(g)).astype(np.float32), expert_slice(down_b, dtype, e, hidden, inter), hidden)
            term = (d * w[t, j]).astype(np.float32)
            acc = term if acc is None else (acc + term).astype(np.float32)
        want[t] = acc[0]
    assert np.array_equal(got[0], want)

    def reversed_segments(expert_ids, sorted_token_ids):
        order = np.lexsort((-np.arange(expert_ids.size), expert_ids))       # same experts, pairs of a segment reversed
        return expert_ids[order], sorted_token_ids[order]

    assert np.array_equal(layer.forward(x, pair_order=reversed_segments), got)


def test_layer_shapes_and_batch_flattening():
    dtype, E, hidden, inter, topk = oracle.Q4K, 4, 256, 256, 2
    router = normal(8, (E, hidden), 0.2)
    blocks = [oracle.from_float(dtype, normal(9 + i, E * inter * hidden, 0.05)) for i in range(3)]
    layer = fm.FusedMoeOracle(dtype, router, blocks[0], blocks[1], blocks[2], E, hidden, inter, topk, True)
    x = normal(12, (2, 3, hidden), 1.0)
    y = layer.forward(x)
    assert y.shape == (2, 3, hidden)
    # tokens are independent: the same rows as one batch of six
    assert np.array_equal(y.reshape(6, hidden), layer.forward(x.reshape(1, 6, hidden))[0])
