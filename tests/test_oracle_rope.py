"""What pins the CPU checker's rotary embedding (oracle/weed_oracle.c: wo_rope_tables, wo_rope_forward).

The reference has no test of RoPE (test/tests.cpp never names it), so these are closed forms and special cases of
the definition in src/modules/rope.cpp:18-98: tables in float64, the identity at position 0, linearity, and the
per-coordinate formula written independently in numpy.  Parity with the reference's bits is therefore unpinned.
"""
import numpy as np


def test_tables_match_float64_closed_form(oracle):
    d, L, base = 64, 300, 10000.0
    cos_t, sin_t = oracle.rope_tables(d, L, base)
    cos_m = cos_t.reshape(d, L).T  # logical [pos, j]; stored column-major
    sin_m = sin_t.reshape(d, L).T
    pos = np.arange(L, dtype=np.float64)[:, None]
    i = (np.arange(d) // 2).astype(np.float64)[None, :]  # coordinates 2i and 2i+1 share an angle
    theta = base ** (-2.0 * i / d)
    # fp32 angles grow to ~300 rad: cos/sin of an angle rounded to fp32 differ from the float64 value by ~ulp(angle)
    np.testing.assert_allclose(cos_m, np.cos(pos * theta), atol=4e-5)
    np.testing.assert_allclose(sin_m, np.sin(pos * theta), atol=4e-5)
    assert np.all(cos_m[0] == 1.0) and np.all(sin_m[0] == 0.0)
    assert np.array_equal(cos_m[:, 0::2], cos_m[:, 1::2]) and np.array_equal(sin_m[:, 0::2], sin_m[:, 1::2])
    # theta_0 = 1: the first pair turns by one radian per position
    np.testing.assert_allclose(cos_m[:, 0], np.cos(np.arange(L)), atol=4e-5)


def test_forward_special_cases_and_formula(oracle):
    rng = np.random.default_rng(3)
    B, H, T, d, L = 2, 3, 7, 32, 40
    x = rng.standard_normal((B, H, T, d)).astype(np.float32)
    cos_t, sin_t = oracle.rope_tables(d, L)
    y = oracle.rope_forward(x, cos_t, sin_t, L)
    # position 0 is the identity
    np.testing.assert_array_equal(y[:, :, 0], x[:, :, 0])
    # the definition, coordinate by coordinate, in float64
    cos_m = cos_t.reshape(d, L).T.astype(np.float64)
    sin_m = sin_t.reshape(d, L).T.astype(np.float64)
    rot = np.concatenate([-x[..., d // 2:], x[..., :d // 2]], axis=-1).astype(np.float64)
    want = x.astype(np.float64) * cos_m[None, None, :T] + rot * sin_m[None, None, :T]
    np.testing.assert_allclose(y, want, rtol=0, atol=2e-6)
    # a position offset selects later table rows: token t at offset p equals token t + p of a longer call
    x2 = np.concatenate([np.zeros((B, H, 5, d), np.float32), x], axis=2)
    y2 = oracle.rope_forward(x2, cos_t, sin_t, L)
    np.testing.assert_array_equal(oracle.rope_forward(x, cos_t, sin_t, L, pos0=5), y2[:, :, 5:])
    # linear in x
    np.testing.assert_allclose(oracle.rope_forward(2 * x, cos_t, sin_t, L), 2 * y, rtol=0, atol=0)
