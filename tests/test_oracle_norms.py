"""What pins the CPU checker's activations and norms (oracle/weed_oracle.c: wo_unary, wo_silu_mul, wo_rms_norm,
wo_layer_norm), the pieces of the two modules that call the attention module
(src/modules/transformer_encoder_layer.cpp:63-125, include/modules/qwen_decoder_layer.hpp:104-115).

Held by the reference's own tests: relu(2) = 2, relu(-2) = 0 (test/tests.cpp:230-244), sigmoid(0) = 0.5 (284-291),
tanh(0) = 0 (314-321), mean(1, 2, 3) = 2 (111-120).  The reference has no test of GeLU, SwiGLU, RMSNorm or LayerNorm,
so those are pinned by float64 closed forms and by what the mathematics fixes; parity with the reference's bits is
unpinned for them.
"""
import numpy as np


def test_reference_known_answers(oracle):
    assert oracle.unary(oracle.RELU, np.array([2.0, -2.0], np.float32)).tolist() == [2.0, 0.0]
    assert oracle.unary(oracle.SIGMOID, np.array([0.0], np.float32))[0] == 0.5
    assert oracle.unary(oracle.TANH, np.array([0.0], np.float32))[0] == 0.0
    # the axis mean both norms are built from: mean(1, 2, 3) = 2, so the centred row is (-1, 0, 1)
    y = oracle.layer_norm(np.array([[1.0, 2.0, 3.0]], np.float32), np.ones(3, np.float32), np.zeros(3, np.float32))
    np.testing.assert_allclose(y[0], [-np.sqrt(1.5), 0.0, np.sqrt(1.5)], rtol=3e-7, atol=0)
    assert y[0, 1] == 0.0


def test_activations_against_float64(oracle):
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(4000) * 3, [0.0, -0.0, 1e-8, -1e-8, 30.0, -30.0, 88.0, -88.0]]).astype(np.float32)
    xd = x.astype(np.float64)
    np.testing.assert_array_equal(oracle.unary(oracle.RELU, x), np.maximum(x, 0))
    np.testing.assert_allclose(oracle.unary(oracle.SIGMOID, x), 1.0 / (1.0 + np.exp(-xd)), rtol=3e-7, atol=1e-38)
    np.testing.assert_allclose(oracle.unary(oracle.TANH, x), np.tanh(xd), rtol=3e-7, atol=0)
    gelu = 0.5 * xd * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (xd + 0.044715 * xd ** 3)))
    np.testing.assert_allclose(oracle.unary(oracle.GELU, x), gelu, rtol=2e-6, atol=2e-7)
    # the tanh form stays within 5e-4 of the exact Gaussian GeLU x * Phi(x): a wrong constant or a dropped cubic
    # term would not
    from math import erf
    exact = np.array([0.5 * v * (1.0 + erf(v / np.sqrt(2.0))) for v in xd])
    assert np.max(np.abs(oracle.unary(oracle.GELU, x) - exact)) < 5e-4
    # limits: gelu(x) -> x for large x, -> 0 for very negative x; sigmoid(-x) = 1 - sigmoid(x)
    assert oracle.unary(oracle.GELU, np.array([30.0], np.float32))[0] == 30.0
    assert oracle.unary(oracle.GELU, np.array([-30.0], np.float32))[0] == 0.0
    s = oracle.unary(oracle.SIGMOID, x)
    np.testing.assert_allclose(s + oracle.unary(oracle.SIGMOID, -x), 1.0, rtol=0, atol=2e-7)
    up = rng.standard_normal(x.size).astype(np.float32)
    np.testing.assert_allclose(oracle.silu_mul(x, up), xd / (1.0 + np.exp(-xd)) * up.astype(np.float64), rtol=1e-6,
                               atol=1e-30)
    # operand order: the gate goes through the sigmoid, not `up`
    assert oracle.silu_mul(np.array([0.0], np.float32), np.array([5.0], np.float32))[0] == 0.0
    assert oracle.silu_mul(np.array([5.0], np.float32), np.array([0.0], np.float32))[0] == 0.0
    assert abs(oracle.silu_mul(np.array([1.0], np.float32), np.array([2.0], np.float32))[0] - 2.0 / (1.0 + np.exp(-1.0))) < 1e-6


def test_rms_norm(oracle):
    rng = np.random.default_rng(6)
    eps = oracle.norm_epsilon()
    assert eps == np.float32(np.finfo(np.float32).eps / 4)  # FP_NORM_EPSILON, weed_types.hpp:213-214
    for rows, n in ((5, 8), (3, 4096), (2, 1000)):
        x = (rng.standard_normal((rows, n)) * rng.uniform(0.1, 30, (rows, 1))).astype(np.float32)
        w = rng.uniform(0.5, 2.0, n).astype(np.float32)
        y = oracle.rms_norm(x, w)
        xd = x.astype(np.float64)
        want = xd / np.sqrt(np.mean(xd * xd, axis=1, keepdims=True) + eps) * w
        np.testing.assert_allclose(y, want, rtol=3e-6, atol=1e-7)
        # before the weight, every row has unit mean square
        np.testing.assert_allclose(np.mean((y.astype(np.float64) / w) ** 2, axis=1), 1.0, rtol=2e-5)
        # scaling a row by a power of two changes nothing but the eps term
        np.testing.assert_allclose(oracle.rms_norm(4 * x, w), y, rtol=1e-6, atol=0)
    # a constant row is its sign times the weight; eps only matters near zero: a zero row stays zero
    w = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    np.testing.assert_allclose(oracle.rms_norm(np.full((1, 4), -7.0, np.float32), w)[0], -w, rtol=3e-7)
    assert not oracle.rms_norm(np.zeros((1, 4), np.float32), w).any()
    # eps is inside the root: a row far below sqrt(eps) is scaled by 1 / sqrt(eps), not normalised
    tiny = np.full((1, 4), 1e-7, np.float32)
    np.testing.assert_allclose(oracle.rms_norm(tiny, np.ones(4, np.float32))[0], 1e-7 / np.sqrt(1e-14 + eps), rtol=1e-5)


def test_layer_norm(oracle):
    rng = np.random.default_rng(7)
    eps = oracle.norm_epsilon()
    for rows, n in ((4, 8), (3, 4096), (2, 777)):
        x = (rng.standard_normal((rows, n)) * rng.uniform(0.5, 10, (rows, 1)) + rng.uniform(-1, 1, (rows, 1))).astype(np.float32)
        gamma = rng.uniform(0.5, 2.0, n).astype(np.float32)
        beta = rng.standard_normal(n).astype(np.float32)
        y = oracle.layer_norm(x, gamma, beta)
        xd = x.astype(np.float64)
        xc = xd - xd.mean(axis=1, keepdims=True)
        want = xc / np.sqrt(np.mean(xc * xc, axis=1, keepdims=True) + eps) * gamma + beta
        np.testing.assert_allclose(y, want, rtol=2e-5, atol=2e-5)
        # before the affine step: zero mean, unit variance (biased, as mean(xc * xc) is)
        z = (y.astype(np.float64) - beta) / gamma
        np.testing.assert_allclose(z.mean(axis=1), 0.0, atol=2e-5)
        np.testing.assert_allclose((z * z).mean(axis=1), 1.0, rtol=1e-4)
        # a shift of the row leaves the result unchanged up to the rounding of the shifted values and of the mean
        # (one-after-the-other fp32 sums, as the reference adds), a row of equal values maps to beta
        np.testing.assert_allclose(oracle.layer_norm(x + np.float32(2.0), gamma, beta), y, rtol=0, atol=1e-4)
    c = np.full((1, 6), 3.25, np.float32)
    b = np.arange(6, dtype=np.float32)
    np.testing.assert_array_equal(oracle.layer_norm(c, np.ones(6, np.float32), b)[0], b)
