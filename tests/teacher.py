"""Op-level teacher forcing for the decoder tests: every launch of an eager forward is checked against the CPU restatement
of the SAME op applied to the GPU's OWN input (read back after the launch), so each op of a model of any width is held to
the per-op bar without the amplification a chain of activation quantizers adds to an end-to-end comparison.

Bars: f32 glue ops <= 1e-5, quantized matmuls <= 2e-6 relative L2 per row.  A matmul whose activation row is formed inside the
kernel (rms_norm / silu prologues) quantizes values that may differ from the CPU's in the last bit; an element that lies
within 2e-4 of a rounding boundary of the activation quantizer may then round the other way.  Such a row is accepted only
if flipping some of those boundary elements in the CPU evaluation reproduces it to the same 2e-6."""
import itertools
import math

import numpy as np
import torch

import oracle
from oracle import llama_oracle as lo
from tests.util import rel_l2

f32 = np.float32
TOL_MM = 2e-6
TOL_GLUE = 1e-5
K_QUANTS = (oracle.Q4K, oracle.Q5K, oracle.Q6K, 10, 11)        # + Q2K, Q3K: Q8_K activations; the others Q8_0 / Q8_1 blocks


def _boundary_elements(dtype: int, x: np.ndarray, width: float = 2e-4):
    """Indices of the elements of one activation row that the quantizer of `dtype`'s vec_dot type rounds from within `width`
    of a half-integer, each with the factor that pushes it across."""
    x = np.asarray(x, dtype=f32)
    span = 256 if dtype in K_QUANTS else 32
    out = []
    for s in range(0, x.size, span):
        seg = x[s:s + span].astype(np.float64)
        amax = np.abs(seg).max()
        if amax == 0:
            continue
        t = np.abs(seg) * (127.0 / amax)
        frac = t - np.floor(t)
        for j in np.nonzero(np.abs(frac - 0.5) < width * np.maximum(t, 1.0))[0]:
            if abs(seg[j]) == amax:
                continue                                       # the scale element itself: always +-127
            out.append((s + int(j), 1.0 + 4.0 * width if frac[j] < 0.5 else 1.0 - 4.0 * width))
    return out


def matmul_rows_checked(dtype: int, x: np.ndarray, w_blocks: np.ndarray, n: int, got: np.ndarray, what: str, exact_input: bool, threads: int = 8,
                        slack=None):
    """got [rows, n] against the CPU matmul of x [rows, k]; returns the number of rows that needed boundary flips.
    slack [rows]: added to the bar of a row (the rounding of a residual add the result was read back through)."""
    x = np.ascontiguousarray(x, dtype=f32)
    want = oracle.matmul_fast(dtype, x, w_blocks, n, threads)
    flipped = 0
    for r in range(x.shape[0]):
        TOL_MM = 2e-6 + (float(slack[r]) if slack is not None else 0.0)
        if rel_l2(got[r], want[r]) <= TOL_MM:
            continue
        assert not exact_input, f"{what} row {r}: {rel_l2(got[r], want[r]):.3e} on identical f32 input"
        cands = _boundary_elements(dtype, x[r])
        assert 0 < len(cands) <= 10, f"{what} row {r}: {rel_l2(got[r], want[r]):.3e} and {len(cands)} boundary elements"
        ok = False
        for m in range(1, len(cands) + 1):
            for sub in itertools.combinations(cands, m):
                xr = x[r:r + 1].copy()
                for j, fac in sub:
                    xr[0, j] = f32(xr[0, j] * fac)
                if rel_l2(got[r], oracle.matmul_fast(dtype, xr, w_blocks, n, threads)[0]) <= TOL_MM:
                    ok = True
                    break
            if ok:
                break
        assert ok, f"{what} row {r}: {rel_l2(got[r], want[r]):.3e}, not explained by its {len(cands)} boundary elements"
        flipped += 1
    return flipped


def _residual_checked(dtype, act, w_blocks, n, x_before, x_after, what, exact_input):
    """x_after = x_before + matmul(act): the matmul is read back through the f32 add, whose rounding (half an ulp of x_after
    per element) is added to the bar."""
    delta = (x_after.astype(np.float64) - x_before.astype(np.float64)).astype(f32)
    dn = np.linalg.norm(delta.astype(np.float64), axis=1)
    slack = 1.2e-7 * np.linalg.norm(x_after.astype(np.float64), axis=1) / np.where(dn > 0, dn, 1.0)
    return matmul_rows_checked(dtype, act, w_blocks, n, delta, what, exact_input, slack=slack)


class Tap:
    """Snapshots of the model's buffers after every launch of one eager forward."""

    BUFS = ("x", "xn", "qk", "v", "att", "delta", "gu", "h", "partials", "logits")

    def __init__(self, model):
        self.model, self.snaps = model, {}

    def __call__(self, stage, li):
        torch.cuda.synchronize(self.model.device)
        s = {b: getattr(self.model, b).detach().cpu().numpy().copy() for b in self.BUFS}
        if li >= 0:
            lw = self.model.layers[li]
            s["k_cache"], s["v_cache"] = lw.k_cache.cpu().numpy().copy(), lw.v_cache.cpu().numpy().copy()
        self.snaps[(stage, li)] = s

    def __enter__(self):
        self.model.tap = self
        return self

    def __exit__(self, *exc):
        self.model.tap = None


def _blocks(t, name):
    dt, blocks = t[name]
    return int(dt), np.frombuffer(bytes(blocks), dtype=np.uint8)


def _attention(q_rot, kc, vc, pos, rows, H, KV, D):
    """softmax(q k^T / sqrt(d) + causal mask) v for `rows` rotated queries [rows, H*D] at positions pos.. over the caches."""
    kv_len = pos + rows
    q = q_rot.reshape(rows, H, D).transpose(1, 0, 2)
    rep = H // KV
    kr, vr = np.repeat(kc[:, :kv_len], rep, axis=0), np.repeat(vc[:, :kv_len], rep, axis=0)
    att = (np.matmul(q, kr.transpose(0, 2, 1)).astype(f32) * f32(1.0 / math.sqrt(D))).astype(f32)
    i, j = np.arange(rows).reshape(-1, 1), np.arange(kv_len).reshape(1, -1)
    att = np.where(j > i + pos, f32(-np.inf), att)
    att = lo.softmax_last_dim(att)
    return np.matmul(att, vr).astype(f32).transpose(1, 0, 2).reshape(rows, H * D)


def check_forward_ops(model, t, cfg, tokens, pos: int, fused: bool):
    """One eager ModelWeights.forward of `tokens` at position `pos`, every op checked against the CPU op on the GPU's own input.
    fused=False: one kernel per op (any number of rows).  fused=True: the single-token path with the glue inside the matvecs.
    Returns (logits, number of matmul rows accepted through boundary flips)."""
    rows = len(tokens)
    H, KV, D = cfg.n_head, cfg.n_kv_head, cfg.head_dim
    qd, kvd = H * D, KV * D
    assert not fused or rows == 1
    old = model.fuse_decode
    model.fuse_decode = fused
    try:
        with Tap(model) as tap:
            logits = model.forward(torch.tensor([list(tokens)], dtype=torch.int32), pos).cpu().numpy()
    finally:
        model.fuse_decode = old
    S = tap.snaps
    cos, sin = lo.precomput_freqs_cis(D, cfg.rope_theta, cfg.ctx)
    cs, sn = cos[pos:pos + rows], sin[pos:pos + rows]
    flips = 0
    emb = np.asarray(t["tok_embeddings"])[np.asarray(tokens, dtype=np.int64)].astype(f32)
    assert np.array_equal(S[("embedding", -1)]["x"][:rows], emb)
    x_in = emb                                                  # the residual rows entering the layer
    prev_delta = None
    for li in range(cfg.n_layer):
        p = f"blk.{li}."
        dq, wq = _blocks(t, p + "attention_wq")
        dk, wk = _blocks(t, p + "attention_wk")
        dv, wv = _blocks(t, p + "attention_wv")
        do, wo = _blocks(t, p + "attention_wo")
        d1, w1 = _blocks(t, p + "feed_forward_w1")
        d3, w3 = _blocks(t, p + "feed_forward_w3")
        d2, w2 = _blocks(t, p + "feed_forward_w2")
        mw = model.layers[li].w
        joined_qk = mw["attention_wq"].dtype == mw["attention_wk"].dtype and mw["attention_wk"].ptr == mw["attention_wq"].ptr + mw["attention_wq"].nbytes
        joined_13 = mw["feed_forward_w1"].dtype == mw["feed_forward_w3"].dtype and \
            mw["feed_forward_w3"].ptr == mw["feed_forward_w1"].ptr + mw["feed_forward_w1"].nbytes

        def split_qk(buf):
            if joined_qk or fused:
                m = buf[:rows, :qd + kvd]
                return m[:, :qd], m[:, qd:]
            flat = buf.reshape(-1)
            return flat[:rows * qd].reshape(rows, qd), flat[rows * qd:rows * (qd + kvd)].reshape(rows, kvd)

        if not fused:
            a = S[("attention_norm", li)]
            if prev_delta is not None:
                x_in = (x_in + prev_delta).astype(f32)
                assert np.array_equal(a["x"][:rows], x_in), f"layer {li}: residual add"
            xn = a["xn"][:rows]
            assert rel_l2(xn, lo.rms_norm(x_in, t[p + "attention_norm"], cfg.rms_eps)) <= TOL_GLUE, f"layer {li}: attention_norm"
            exact = True
        else:
            xn = lo.rms_norm(x_in, t[p + "attention_norm"], cfg.rms_eps)
            exact = False
        b = S[("qkv", li)]
        gq, gk = split_qk(b["qk"])
        gv = b["v"][:rows]
        flips += matmul_rows_checked(dq, xn, wq, qd, gq, f"layer {li} attention_wq", exact)
        flips += matmul_rows_checked(dk, xn, wk, kvd, gk, f"layer {li} attention_wk", exact)
        flips += matmul_rows_checked(dv, xn, wv, kvd, gv, f"layer {li} attention_wv", exact)
        want_q = lo.rope_i(gq.reshape(rows, H, D).transpose(1, 0, 2)[None], cs, sn)[0].transpose(1, 0, 2).reshape(rows, qd)
        want_k = lo.rope_i(gk.reshape(rows, KV, D).transpose(1, 0, 2)[None], cs, sn)[0]                 # [KV, rows, D]
        c = S[("attention", li)]
        if not fused:
            r_ = S[("rope", li)]
            assert rel_l2(split_qk(r_["qk"])[0], want_q) <= TOL_GLUE, f"layer {li}: rope q"
        assert rel_l2(c["k_cache"][:, pos:pos + rows], want_k) <= TOL_GLUE, f"layer {li}: rope k / cache append"
        assert np.array_equal(c["v_cache"][:, pos:pos + rows], gv.reshape(rows, KV, D).transpose(1, 0, 2)), f"layer {li}: v cache append"
        q_for_att = split_qk(S[("rope", li)]["qk"])[0] if not fused else want_q
        want_att = _attention(q_for_att, c["k_cache"], c["v_cache"], pos, rows, H, KV, D)
        g_att = c["att"][:rows]
        assert rel_l2(g_att, want_att) <= TOL_GLUE, f"layer {li}: attention {rel_l2(g_att, want_att):.3e}"
        d = S[("attention_wo", li)]
        if not fused:
            flips += matmul_rows_checked(do, g_att, wo, cfg.hidden, d["delta"][:rows], f"layer {li} attention_wo", True)
            e = S[("ffn_norm", li)]
            x_mid = (x_in + d["delta"][:rows]).astype(f32)
            assert np.array_equal(e["x"][:rows], x_mid), f"layer {li}: residual add after attention"
            xn2 = e["xn"][:rows]
            assert rel_l2(xn2, lo.rms_norm(x_mid, t[p + "ffn_norm"], cfg.rms_eps)) <= TOL_GLUE, f"layer {li}: ffn_norm"
        else:
            x_mid = d["x"][:1]
            flips += _residual_checked(do, g_att, wo, cfg.hidden, x_in, x_mid, f"layer {li} attention_wo + residual", True)
            assert np.isclose(float(d["partials"].astype(np.float64).sum()), float((x_mid.astype(np.float64) ** 2).sum()), rtol=1e-5)
            xn2 = lo.rms_norm(x_mid, t[p + "ffn_norm"], cfg.rms_eps)
        g_ = S[("w13", li)]
        kq = (oracle.Q4K, oracle.Q5K, oracle.Q6K)
        paired = fused and d1 == d3 and d1 in kq + (oracle.Q4_0, oracle.Q8_0) and cfg.hidden <= (4096 if d1 in kq else 2048)
        if paired:
            # h = silu(w1 xn) * (w3 xn) straight out of the paired-row matvec: checked through both products
            a1 = oracle.matmul_fast(d1, np.ascontiguousarray(xn2), w1, cfg.ffn, 8)
            a3 = oracle.matmul_fast(d3, np.ascontiguousarray(xn2), w3, cfg.ffn, 8)
            want_h = (lo.silu(a1) * a3).astype(f32)
            gh = g_["h"][:1]
            if rel_l2(gh, want_h) > TOL_GLUE:
                # a boundary element of the normalized row rounded the other way: find it through feed_forward_w1 alone
                cands = _boundary_elements(d1, xn2[0])
                assert 0 < len(cands) <= 10, f"layer {li}: swiglu {rel_l2(gh, want_h):.3e}, {len(cands)} boundary elements"
                ok = False
                for m in range(1, len(cands) + 1):
                    for sub in itertools.combinations(cands, m):
                        xr = xn2.copy()
                        for j, fac in sub:
                            xr[0, j] = f32(xr[0, j] * fac)
                        hh = (lo.silu(oracle.matmul_fast(d1, xr, w1, cfg.ffn, 8)) * oracle.matmul_fast(d3, xr, w3, cfg.ffn, 8)).astype(f32)
                        if rel_l2(gh, hh) <= TOL_GLUE:
                            ok = True
                            break
                    if ok:
                        break
                assert ok, f"layer {li}: swiglu {rel_l2(gh, want_h):.3e} not explained by boundary elements"
                flips += 1
            act = gh
        else:
            gu = g_["gu"]
            if joined_13:
                m = gu[:rows, :2 * cfg.ffn]
                gg, uu = m[:, :cfg.ffn], m[:, cfg.ffn:]
            else:
                flat = gu.reshape(-1)
                gg, uu = flat[:rows * cfg.ffn].reshape(rows, cfg.ffn), flat[rows * cfg.ffn:2 * rows * cfg.ffn].reshape(rows, cfg.ffn)
            flips += matmul_rows_checked(d1, xn2, w1, cfg.ffn, gg, f"layer {li} feed_forward_w1", not fused)
            flips += matmul_rows_checked(d3, xn2, w3, cfg.ffn, uu, f"layer {li} feed_forward_w3", not fused)
            act = (lo.silu(gg) * uu).astype(f32)
        h_ = S[("w2", li)]
        if not fused:
            if rows > 2 and cfg.ffn % 256 == 0:
                flips += matmul_rows_checked(d2, act, w2, cfg.hidden, h_["delta"][:rows], f"layer {li} feed_forward_w2 (swiglu rows)", False)
            else:
                assert rel_l2(h_["h"][:rows], act) <= TOL_GLUE, f"layer {li}: silu * up"
                flips += matmul_rows_checked(d2, h_["h"][:rows], w2, cfg.hidden, h_["delta"][:rows], f"layer {li} feed_forward_w2", True)
            prev_delta = h_["delta"][:rows].copy()
            x_in = x_mid
        else:
            x_out = h_["x"][:1]
            # on the paired path the kernel quantizes exactly the f32 row read back here; otherwise silu(gate) * up is its prologue
            flips += _residual_checked(d2, act, w2, cfg.hidden, x_mid, x_out, f"layer {li} feed_forward_w2 + residual", paired)
            assert np.isclose(float(h_["partials"].astype(np.float64).sum()), float((x_out.astype(np.float64) ** 2).sum()), rtol=1e-5)
            x_in = x_out
            prev_delta = None
    dh, wh = _blocks(t, "output")
    z = S[("head", -1)]
    if not fused:
        x_last = (x_in[-1:] + prev_delta[-1:]).astype(f32)
        xn3 = z["xn"][:1]
        assert rel_l2(xn3, lo.rms_norm(x_last, t["norm"], cfg.rms_eps)) <= TOL_GLUE, "final norm"
        flips += matmul_rows_checked(dh, xn3, wh, cfg.vocab, z["logits"], "output head", True)
    else:
        xn3 = lo.rms_norm(x_in, t["norm"], cfg.rms_eps)
        flips += matmul_rows_checked(dh, xn3, wh, cfg.vocab, z["logits"], "output head", False)
    return logits, flips
