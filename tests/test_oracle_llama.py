"""Pins the numpy restatement of the decoder glue and of the quantized llama forward (oracle/llama_oracle.py)
against the reference's own known answers and against what the mathematics fixes.  CPU only."""
import types

import numpy as np
import pytest

import oracle
from oracle import llama_oracle as lo
from tests import stdrng
from tests.util import rel_l2

DATA = np.array([[[3.0, 1.0, 4.0], [1.0, 5.0, 9.0]], [[2.0, 1.0, 7.0], [8.0, 2.0, 8.0]]], dtype=np.float32)


def round4(a):
    return np.round(np.asarray(a, dtype=np.float64) * 1e4) / 1e4


def test_softmax_last_dim_kat():
    # candle-nn/tests/ops.rs:9-52: softmax of log(data) over the last dim = data / row sum
    got = lo.softmax_last_dim(np.log(DATA))
    want = [[[0.375, 0.125, 0.5], [0.0667, 0.3333, 0.6]], [[0.2, 0.1, 0.7], [0.4444, 0.1111, 0.4444]]]
    assert round4(got).tolist() == want


def test_softmax_numerical_stability_kat():
    # candle-nn/tests/ops.rs:191-196
    assert lo.softmax_last_dim(np.array([1234.0, 0.0], dtype=np.float32)).tolist() == [1.0, 0.0]


def test_rms_norm_kat():
    # candle-nn/tests/ops.rs:55-66
    got = lo.rms_norm(DATA, np.array([1.0, 2.0, 3.0], dtype=np.float32), 1e-5)
    want = [[[1.019, 0.6794, 4.0762], [0.1674, 1.6744, 4.521]], [[0.4714, 0.4714, 4.9497], [1.206, 0.603, 3.6181]]]
    assert round4(got).tolist() == want


def test_silu_closed_form():
    x = np.array([-20.0, -1.0, 0.0, 0.5, 3.0, 30.0], dtype=np.float32)
    want = x.astype(np.float64) / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.allclose(lo.silu(x), want, rtol=1e-6, atol=1e-12)
    assert lo.silu(np.float32(0.0)) == 0.0 and abs(lo.silu(np.float32(30.0)) - 30.0) < 1e-5


def test_rope_i_matches_slow_formulation_on_reference_inputs():
    # candle-nn/tests/ops.rs:199-219: StdRng(299792458) inputs, fast kernel == rope_i_slow exactly on the CPU.
    # The slow formulation (rotary_emb.rs:290-308) is restated here independently: reshape to pairs,
    # y0 = x0 cos - x1 sin, y1 = x0 sin + x1 cos, concatenate on a new last axis, flatten.
    b, h, t, d = 2, 5, 10, 16
    n = b * h * t * d
    r = stdrng.random_f32(299792458, n + t * d)
    src = r[:n].reshape(b, h, t, d)
    cos = r[n:n + t * d // 2].reshape(t, d // 2)
    sin = r[n + t * d // 2:].reshape(t, d // 2)
    got = lo.rope_i(src, cos, sin)
    x = src.reshape(b, h, t, d // 2, 2)
    c, s = cos.reshape(1, 1, t, d // 2, 1), sin.reshape(1, 1, t, d // 2, 1)
    x0, x1 = x[..., 0:1], x[..., 1:2]
    slow = np.concatenate([x0 * c - x1 * s, x0 * s + x1 * c], axis=-1).reshape(b, h, t, d)
    assert np.array_equal(got, slow)


def test_rope_i_is_a_rotation_with_real_tables():
    cos, sin = lo.precomput_freqs_cis(64, 500000.0, 128)
    assert cos.shape == (128, 32) and np.all(cos[0] == 1.0) and np.all(sin[0] == 0.0)
    # theta_0 = 1 -> angle of pair 0 at position p is p radians
    assert np.allclose(cos[:, 0], np.cos(np.arange(128)), atol=1e-5) and np.allclose(sin[:, 0], np.sin(np.arange(128)), atol=1e-5)
    # last pair: theta = base^(-(d-2)/d)
    assert np.isclose(sin[1, -1], np.sin(500000.0 ** (-62.0 / 64.0)), rtol=1e-5)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 3, 128, 64)).astype(np.float32)
    y = lo.rope_i(x, cos, sin)
    assert np.array_equal(y[:, :, 0], x[:, :, 0])                        # position 0: identity
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
    # relative-position property: <rope(q, p1), rope(k, p2)> depends on p1 - p2 only
    q, k = x[0, 0, 0], x[0, 1, 0]
    tile = lambda v: np.broadcast_to(v, (1, 1, 128, 64)).copy()
    rq, rk = lo.rope_i(tile(q), cos, sin)[0, 0], lo.rope_i(tile(k), cos, sin)[0, 0]
    assert np.isclose(rq[10] @ rk[3], rq[50] @ rk[43], rtol=1e-3, atol=1e-3)


# ------------------------------------------------------------------------------------------- decoder
def tiny_cfg(**kw):
    base = dict(n_layer=2, hidden=256, n_head=4, n_kv_head=2, head_dim=64, ffn=512, vocab=320, rope_theta=10000.0, rms_eps=1e-5, ctx=64)
    base.update(kw)
    return types.SimpleNamespace(**base)


MIX = {"attention_wq": oracle.Q4K, "attention_wk": oracle.Q4K, "attention_wv": oracle.Q6K, "attention_wo": oracle.Q4K,
       "feed_forward_w1": oracle.Q4K, "feed_forward_w3": oracle.Q4K, "feed_forward_w2": oracle.Q6K, "output": oracle.Q4K}


@pytest.fixture(scope="module")
def tiny():
    cfg = tiny_cfg()
    return cfg, lo.random_tensors(cfg, seed=5, dtypes=MIX, weight_scale=0.05)


def test_prefill_equals_token_by_token_decode(tiny):
    cfg, t = tiny
    toks = [3, 17, 250, 9, 100, 42]
    whole = lo.LlamaOracle(cfg, t).forward(toks, 0)
    inc = lo.LlamaOracle(cfg, t)
    for i, tok in enumerate(toks):
        last = inc.forward([tok], i)
    assert whole.shape == (1, cfg.vocab)
    # per-row activation quantization makes the two paths agree to summation order only
    assert rel_l2(last, whole) < 1e-5
    # and a split prefill (4 tokens, then 2 with a rectangular causal mask) as well
    sp = lo.LlamaOracle(cfg, t)
    sp.forward(toks[:4], 0)
    assert rel_l2(sp.forward(toks[4:], 4), whole) < 1e-5


def test_causality(tiny):
    cfg, t = tiny
    a = lo.LlamaOracle(cfg, t)
    a.forward([5, 6, 7, 8], 0)
    la = a.forward([9], 4)
    b = lo.LlamaOracle(cfg, t)
    b.forward([5, 6, 7, 8], 0)
    lb = b.forward([9], 4)
    assert np.array_equal(la, lb)
    c = lo.LlamaOracle(cfg, t)
    c.forward([5, 6, 99, 8], 0)                 # a different past token must change the result
    assert rel_l2(c.forward([9], 4), la) > 1e-3


def test_zeroed_projections_reduce_to_head_of_normed_embedding(tiny):
    cfg, t = tiny
    t2 = dict(t)
    for li in range(cfg.n_layer):
        for name, n, k in (("attention_wo", cfg.hidden, cfg.n_head * cfg.head_dim), ("feed_forward_w2", cfg.hidden, cfg.ffn)):
            dt = t[f"blk.{li}.{name}"][0]
            t2[f"blk.{li}.{name}"] = (dt, oracle.from_float(dt, np.zeros(n * k, dtype=np.float32)).tobytes())
    got = lo.LlamaOracle(cfg, t2).forward([11, 12, 13], 0)
    emb = t["tok_embeddings"][13:14]
    xn = lo.rms_norm(emb, t["norm"], cfg.rms_eps)
    dt, blocks = t["output"]
    want = oracle.matmul(dt, xn, np.frombuffer(blocks, dtype=np.uint8), cfg.vocab)
    assert np.array_equal(got, want)


def test_single_token_attention_returns_its_own_value(tiny):
    # one key -> softmax weight 1 -> attention output = v of that token, independent of q and of the rotation
    cfg, t = tiny
    m = lo.LlamaOracle(cfg, t)
    m.forward([7], 0)
    k, v = m.kv[0]
    assert k.shape == (cfg.n_kv_head, 1, cfg.head_dim)
    xn = lo.rms_norm(t["tok_embeddings"][7:8], t["blk.0.attention_norm"], cfg.rms_eps)
    dt, blocks = t["blk.0.attention_wv"]
    want_v = oracle.matmul(dt, xn, np.frombuffer(blocks, dtype=np.uint8), cfg.n_kv_head * cfg.head_dim)
    assert np.array_equal(v.reshape(-1), want_v.reshape(-1))
