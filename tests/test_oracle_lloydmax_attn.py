"""Pins the parts of the oracle the reference has no code for: Lloyd-Max tables, the table-driven coder with a
residual sign bit and a row scale, and single-query attention over a quantized cache.

The reference holds no vector for any of these (its tests never touch attention or the quantizer), so they are
pinned by textbook tables, fixed-point properties checked by quadrature, brute-force search and float64 numpy.
"""
import os
import re

import numpy as np
import pytest

from oracle import lloyd_max as lm

HERE = os.path.dirname(os.path.abspath(__file__))
INC = os.path.join(HERE, "..", "weed_amd", "csrc", "lloyd_tables.inc")


def load_tables():
    """Parse the product's generated table file (text only; nothing is imported from the product)."""
    tables = {}
    with open(INC) as f:
        for line in f:
            m = re.match(r"static const float WEED_LM_(\w+)_(\d)\[\d+\] = \{ (.*) \};", line)
            if m:
                vals = [float.fromhex(tok.strip().rstrip("f")) for tok in m.group(3).split(",")]
                tables[(m.group(1), int(m.group(2)))] = np.array(vals, dtype=np.float64)
    return tables


TABLES = load_tables()


def coder_spec(oracle, d, bits, sign):
    levels = TABLES[("LEVELS", bits)]
    bounds = TABLES[("BOUNDS", bits)]
    recon = TABLES[("REFINED", bits)] if sign else levels
    return oracle.CoderSpec(1, d, bits, sign=sign, bounds=bounds, levels=levels, recon=recon)


@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_tables_are_lloyd_max(bits):
    levels = TABLES[("LEVELS", bits)]
    bounds = TABLES[("BOUNDS", bits)]
    refined = TABLES[("REFINED", bits)]
    n = 1 << bits
    assert len(levels) == n and len(bounds) == n - 1 and len(refined) == 2 * n
    # exactly representable in binary16, antisymmetric, ascending
    for t in (levels, refined):
        np.testing.assert_array_equal(t.astype(np.float16).astype(np.float64), t)
        np.testing.assert_array_equal(t, -t[::-1])
        assert np.all(np.diff(t) > 0)
    # textbook values (4 significant digits) + binary16 rounding (2^-11 relative)
    pos = levels[n // 2:]
    np.testing.assert_allclose(pos, lm.TEXTBOOK_LEVELS[bits], rtol=6e-4, atol=1e-4)
    # thresholds are the exact midpoints of the stored centroids
    np.testing.assert_array_equal(bounds, 0.5 * (levels[:-1] + levels[1:]))
    np.testing.assert_array_equal(bounds.astype(np.float32).astype(np.float64), bounds)
    # Lloyd's fixed point: every centroid is the conditional mean of its cell
    edges = np.concatenate([[-np.inf], bounds, [np.inf]])
    for k in range(n):
        assert abs(levels[k] - lm.conditional_mean(edges[k], edges[k + 1])) < 1e-3 * max(1.0, abs(levels[k]))
    # distortion matches the textbook value
    assert lm.quantiser_mse(bounds, levels) == pytest.approx(lm.TEXTBOOK_MSE[bits], rel=2e-3)
    # sign-refined levels: conditional means of the half cells; the law of total expectation ties them to the centroid
    for k in range(n):
        lo_mean = lm.conditional_mean(edges[k], levels[k])
        hi_mean = lm.conditional_mean(levels[k], edges[k + 1])
        assert abs(refined[2 * k] - lo_mean) < 1e-3 * max(1.0, abs(lo_mean))
        assert abs(refined[2 * k + 1] - hi_mean) < 1e-3 * max(1.0, abs(hi_mean))
        p_lo, p_hi = lm.cell_mass(edges[k], levels[k]), lm.cell_mass(levels[k], edges[k + 1])
        mixed = (p_lo * refined[2 * k] + p_hi * refined[2 * k + 1]) / (p_lo + p_hi)
        assert abs(mixed - levels[k]) < 1.5e-3 * max(1.0, abs(levels[k]))
    # the extra bit must buy distortion
    split_bounds = np.sort(np.concatenate([bounds, levels]))
    assert lm.quantiser_mse(split_bounds, refined) < 0.5 * lm.quantiser_mse(bounds, levels)


@pytest.mark.parametrize("bits,sign", [(2, 1), (3, 0), (3, 1), (4, 0), (4, 1)])
def test_lloydmax_coder_brute_force(oracle, bits, sign):
    rng = np.random.default_rng(10 * bits + sign)
    d = 64
    y = (rng.normal(size=(96, d)) * rng.uniform(0.3, 4.0, size=(96, 1))).astype(np.float32)
    spec = coder_spec(oracle, d, bits, sign)
    fields, alpha = oracle.encode_rows(spec, y)
    y64 = y.astype(np.float64)
    norm = np.sqrt((y64 ** 2).sum(axis=1))
    np.testing.assert_allclose(alpha, norm / np.sqrt(d), rtol=2e-6)
    u = y64 * (np.sqrt(d) / norm)[:, None]
    levels = TABLES[("LEVELS", bits)]
    codes = fields >> 1 if sign else fields
    want = lm.brute_force_codes(u, levels)
    # fp32 vs float64 normalisation can differ only for values within rounding of a threshold
    bounds = TABLES[("BOUNDS", bits)]
    near = np.min(np.abs(u[..., None] - bounds), axis=-1) < 1e-5
    assert np.array_equal(codes[~near], want[~near])
    assert near.mean() < 1e-3
    if sign:
        s_want = (u >= levels[want]).astype(np.uint8)
        near_c = np.abs(u - levels[want]) < 1e-5
        ok = ~(near | near_c)
        assert np.array_equal((fields & 1)[ok], s_want[ok])
    # reconstruction: alpha * table[field]; relative error of the row bounded by the quantiser's distortion
    recon = TABLES[("REFINED", bits)] if sign else levels
    back = oracle.decode_rows(spec, fields, alpha)
    np.testing.assert_allclose(back, alpha[:, None].astype(np.float64) * recon[fields], rtol=1e-6, atol=1e-7)
    rel = ((back - y64) ** 2).sum() / (y64 ** 2).sum()
    expect = lm.TEXTBOOK_MSE[bits] * (0.4 if sign else 1.0)
    assert rel < 1.25 * expect


def test_lloydmax_zero_row(oracle):
    spec = coder_spec(oracle, 32, 3, 1)
    fields, alpha = oracle.encode_rows(spec, np.zeros((1, 32), dtype=np.float32))
    assert alpha[0] == 0.0
    # u = 0 sits on the middle threshold: code 4, and 0 < centroid(4) so sign 0
    assert np.all(fields == (4 << 1))
    assert not oracle.decode_rows(spec, fields, alpha).any()


def _dense_attention_f64(K, V, q, lens, gqa_weed, Rk=None, Rv=None):
    """Textbook attention in float64 on dequantised tensors: K, V [S, Hkv, T, d], q [S, Hq, d]."""
    S, Hkv, T, d = K.shape
    Hq = q.shape[1]
    out = np.zeros((S, Hq, d))
    for s in range(S):
        L = lens[s]
        for h in range(Hq):
            kvh = (h % Hkv) if gqa_weed else (h // (Hq // Hkv))
            qq = q[s, h].astype(np.float64)
            if Rk is not None:
                qq = qq @ Rk
            sc = K[s, kvh, :L].astype(np.float64) @ qq / np.sqrt(d)
            w = np.exp(sc - sc.max())
            w /= w.sum()
            o = w @ V[s, kvh, :L].astype(np.float64)
            if Rv is not None:
                o = o @ Rv.T
            out[s, h] = o
    return out


@pytest.mark.parametrize("mode", ["uniform", "lloydmax"])
@pytest.mark.parametrize("gqa_weed", [True, False])
def test_decode_attention_against_float64(oracle, mode, gqa_weed):
    rng = np.random.default_rng(5)
    S, Hq, Hkv, T, d = 3, 4, 2, 37, 32
    lens = [37, 5, 20]
    Kx = rng.normal(size=(S, Hkv, T, d)).astype(np.float32)
    Vx = rng.normal(size=(S, Hkv, T, d)).astype(np.float32)
    q = rng.normal(size=(S, Hq, d)).astype(np.float32)
    Rk = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Rv = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Ky = oracle.apply_rotation(Kx.reshape(-1, d), Rk)
    Vy = oracle.apply_rotation(Vx.reshape(-1, d), Rv)
    if mode == "uniform":
        kspec = oracle.CoderSpec(0, d, 4, block_scale=oracle.block_scale(Ky))
        vspec = oracle.CoderSpec(0, d, 4, block_scale=oracle.block_scale(Vy))
    else:
        kspec = coder_spec(oracle, d, 3, 1)
        vspec = coder_spec(oracle, d, 4, 0)
    kf, ka = oracle.encode_rows(kspec, Ky)
    vf, va = oracle.encode_rows(vspec, Vy)
    Kd = oracle.decode_rows(kspec, kf, ka).reshape(S, Hkv, T, d)
    Vd = oracle.decode_rows(vspec, vf, va).reshape(S, Hkv, T, d)
    got, scores = oracle.decode_attn(kspec, vspec, kf.reshape(S, Hkv, T, d), ka.reshape(S, Hkv, T),
                                     vf.reshape(S, Hkv, T, d), va.reshape(S, Hkv, T), q, lens, gqa_weed=gqa_weed, Rk=Rk,
                                     Rv=Rv, want_scores=True)
    Rkm = Rk.reshape(d, d).T.astype(np.float64)
    Rvm = Rv.reshape(d, d).T.astype(np.float64)
    want = _dense_attention_f64(Kd, Vd, q, lens, gqa_weed, Rkm, Rvm)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-6)
    # the scaled scores themselves (before softmax)
    kvh = 1 if gqa_weed else 0
    sc = Kd[0, kvh].astype(np.float64) @ (q[0, 1].astype(np.float64) @ Rkm) / np.sqrt(d)
    np.testing.assert_allclose(scores[0, 1, :37], sc, rtol=1e-4, atol=2e-6)
    # quantized attention stays close to exact attention on the unquantized tensors
    exact = _dense_attention_f64(Kx, Vx, q, lens, gqa_weed)
    assert np.abs(got - exact).max() < 0.6
    # the two head mappings really differ when Hq != Hkv
    other = oracle.decode_attn(kspec, vspec, kf.reshape(S, Hkv, T, d), ka.reshape(S, Hkv, T), vf.reshape(S, Hkv, T, d),
                               va.reshape(S, Hkv, T), q, lens, gqa_weed=not gqa_weed, Rk=Rk, Rv=Rv)
    assert np.abs(other - got).max() > 1e-3


def test_decode_attention_empty_and_single_token(oracle):
    rng = np.random.default_rng(6)
    d = 32
    spec = oracle.CoderSpec(0, d, 4, block_scale=1.0)
    y = rng.normal(size=(2, d)).astype(np.float32)
    f, a = oracle.encode_rows(spec, y)
    kf = f.reshape(2, 1, 1, d)
    q = rng.normal(size=(2, 1, d)).astype(np.float32)
    out = oracle.decode_attn(spec, spec, kf, None, kf, None, q, [0, 1])
    assert not out[0].any()  # empty sequence -> zeros
    # one token: softmax weight is 1, output is the dequantised V row
    np.testing.assert_allclose(out[1, 0], oracle.decode_rows(spec, f[1:2], a[1:2])[0], rtol=1e-6)
