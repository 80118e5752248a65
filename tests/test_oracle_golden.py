"""Pins the CPU oracle: the reference's known answers and unit tests, closed forms, invariants, brute force.

No GPU is involved.  Each block names the reference lines the vectors come from.
"""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _words(hexes):
    return np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.int32)


@pytest.fixture(scope="module")
def kat():
    with open(os.path.join(HERE, "golden", "weed_uniform_kat.json")) as f:
        return json.load(f)


# ---- QuantizedKVCache::write_row / read_row (src/modules/multihead_attention.cpp:43-79) ----------------------

def test_write_row_known_answers(oracle, kat):
    for case in kat["write_row"]:
        vals = np.array([case["vals"]], dtype=np.float32)
        packed = oracle.uniform_write_rows(vals, case["bits"], case["block_scale"])
        assert packed.shape == (1, len(case["words"]))
        np.testing.assert_array_equal(packed[0], _words(case["words"]))
        spec = oracle.CoderSpec(0, vals.shape[1], case["bits"], block_scale=case["block_scale"])
        fields, _ = oracle.encode_rows(spec, vals)
        np.testing.assert_array_equal(fields[0], np.array(case["codes"], dtype=np.uint8))


def test_read_row_known_answers(oracle, kat):
    for case in kat["read_row"]:
        packed = _words(case["words"]).reshape(1, -1)
        vals = oracle.uniform_read_rows(packed, case["d"], case["bits"], case["block_scale"])
        # the recorded decimals are 8 significant digits of fp32 values
        np.testing.assert_allclose(vals[0], np.array(case["vals"], dtype=np.float32), rtol=0, atol=6e-8)


def test_write_row_ors_into_existing_words(oracle):
    # write_row never clears (cpp:61): writing twice ORs the codes together
    import ctypes
    lib = oracle.lib()
    packed = np.zeros(1, dtype=np.int32)
    fn = lib.wo_uniform_write_row
    fn.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float]
    a = np.array([-1.0] * 8, dtype=np.float32)  # code 5 at 4 bits, s = 1
    b = np.array([0.5] * 8, dtype=np.float32)   # code 9
    fn(packed.ctypes.data, 0, a.ctypes.data, 8, 4, ctypes.c_float(1.0))
    fn(packed.ctypes.data, 0, b.ctypes.data, 8, 4, ctypes.c_float(1.0))
    assert packed.view(np.uint32)[0] == 0xDDDDDDDD  # 5 | 9 = 13


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_uniform_codes_interval_property(oracle, bits):
    # brute force: code c means lo + c*step <= clamp(v) < lo + (c+1)*step, up to one rounding of the division
    rng = np.random.default_rng(bits)
    s = 0.8371
    x = rng.normal(0, 1.3, size=(64, 48)).astype(np.float32)
    spec = oracle.CoderSpec(0, 48, bits, block_scale=s)
    fields, _ = oracle.encode_rows(spec, x)
    lo, hi = np.float32(-3.0) * np.float32(s), np.float32(3.0) * np.float32(s)
    step = (hi - lo) / np.float32(1 << bits)
    exact = np.floor((np.clip(x.astype(np.float64), float(lo), float(hi - step)) - float(lo)) / float(step))
    exact = np.clip(exact, 0, (1 << bits) - 1)
    diff = fields.astype(np.int64) - exact.astype(np.int64)
    # fp32 rounding can move a value sitting within an ulp of a cell edge by one cell at most
    assert np.all(np.abs(diff) <= 1)
    assert np.mean(diff != 0) < 1e-3
    # pack -> unpack round trip and the dequantised value is the cell midpoint
    packed = oracle.uniform_write_rows(x, bits, s)
    back = oracle.uniform_read_rows(packed, 48, bits, s)
    mid = float(lo) + (fields.astype(np.float64) + 0.5) * float(step)
    np.testing.assert_allclose(back, mid, rtol=1e-6, atol=1e-6)
    assert packed.shape[1] == (48 + 32 // bits - 1) // (32 // bits)


def test_uniform_degenerate_scale_gives_zero_codes(oracle):
    # step <= 1e-8 -> every bucket is 0 (cpp:52)
    spec = oracle.CoderSpec(0, 8, 4, block_scale=1e-10)
    fields, _ = oracle.encode_rows(spec, np.ones((1, 8), dtype=np.float32))
    assert not fields.any()


def test_block_scale_closed_form(oracle):
    rng = np.random.default_rng(0)
    x = rng.normal(0, 2.0, size=4096).astype(np.float32)
    want = np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-8)
    assert abs(oracle.block_scale(x) - want) < 1e-5 * want
    assert oracle.block_scale(np.zeros(16, dtype=np.float32)) == pytest.approx(1e-4, rel=1e-6)


# ---- rotation (cpp:84-140): no vectors exist (unseeded), invariants only ----------------------------------------

@pytest.mark.parametrize("d", [8, 64, 128])
def test_rotation_invariants(oracle, d):
    rng = np.random.default_rng(d)
    g = rng.normal(size=d * d).astype(np.float32)
    R = oracle.orthonormalize_columns(g)
    Rm = R.reshape(d, d).T.astype(np.float64)  # column-major buffer -> matrix
    np.testing.assert_allclose(Rm.T @ Rm, np.eye(d), atol=3e-4)  # fp32 Gram-Schmidt
    np.testing.assert_allclose(Rm @ Rm.T, np.eye(d), atol=3e-4)
    # column 0 is the normalised first Gaussian column; later columns stay in the span order (Gram-Schmidt)
    g0 = g[:d].astype(np.float64)
    np.testing.assert_allclose(Rm[:, 0], g0 / np.linalg.norm(g0), atol=1e-6)
    G = g.reshape(d, d).T.astype(np.float64)
    Q, _ = np.linalg.qr(G)
    Q = Q * np.sign(np.sum(Q * Rm, axis=0))  # QR is unique up to column signs
    np.testing.assert_allclose(Rm, Q, atol=2e-3)
    # y = x . R, and R^T undoes it
    x = rng.normal(size=(5, d)).astype(np.float32)
    y = oracle.apply_rotation(x, R)
    np.testing.assert_allclose(y, x.astype(np.float64) @ Rm, atol=1e-5)
    # the column-major buffer of R^T is the row-major buffer of R
    back = oracle.apply_rotation(y, np.ascontiguousarray(Rm).reshape(-1).astype(np.float32))
    np.testing.assert_allclose(back, x, atol=1e-3)


# ---- Weed::matmul (src/ops/matmul.cpp:34-47); reference tests test/tests.cpp:1020-1041, 1327-1360 --------------

def test_matmul_reference_cases(oracle):
    # 1x2 . 2x1 = 23 (tests.cpp:1020-1029); column-major contiguous strides, size-1 dims have stride 0
    A = np.array([2, 3], dtype=np.float32)
    B = np.array([4, 5], dtype=np.float32)
    C = np.zeros(1, dtype=np.float32)
    oracle.matmul(1, 1, 2, A, (0, 0, 1), B, (0, 1, 0), C, (0, 0, 0))
    assert C[0] == 23
    # 2x1 . 1x2 outer product (tests.cpp:1031-1040): z[0][0]=8, z[0][1]=12, z[1][0]=10, z[1][1]=15 where z[i] is
    # column i of the column-major result, so storage is [8, 12, 10, 15]
    C = np.zeros(4, dtype=np.float32)
    oracle.matmul(2, 2, 1, A, (0, 1, 0), B, (0, 0, 1), C, (0, 1, 2))
    np.testing.assert_array_equal(C, [8, 12, 10, 15])
    # 2x3 . 3x2 of tests.cpp:1327-1341, column-major: A = [[1,3,5],[2,4,6]], B = [[7,10],[8,11],[9,12]]
    A = np.arange(1, 7, dtype=np.float32)
    B = np.arange(7, 13, dtype=np.float32)
    C = np.zeros(4, dtype=np.float32)
    oracle.matmul(2, 2, 3, A, (0, 1, 2), B, (0, 1, 3), C, (0, 1, 2))
    want = np.array([[1, 3, 5], [2, 4, 6]]) @ np.array([[7, 10], [8, 11], [9, 12]])
    np.testing.assert_array_equal(C.reshape(2, 2).T, want)


def test_matmul_strided_against_float64(oracle):
    rng = np.random.default_rng(1)
    M, N, K = 7, 5, 11
    buf_a = rng.normal(size=300).astype(np.float32)
    buf_b = rng.normal(size=300).astype(np.float32)
    C = np.zeros(200, dtype=np.float32)
    ag, bg, cg = (3, 2, 17), (5, 9, 1), (1, 11, 2)
    oracle.matmul(M, N, K, buf_a, ag, buf_b, bg, C, cg)
    Am = np.array([[buf_a[ag[0] + i * ag[1] + k * ag[2]] for k in range(K)] for i in range(M)], dtype=np.float64)
    Bm = np.array([[buf_b[bg[0] + k * bg[1] + j * bg[2]] for j in range(N)] for k in range(K)], dtype=np.float64)
    got = np.array([[C[cg[0] + i * cg[1] + j * cg[2]] for j in range(N)] for i in range(M)])
    np.testing.assert_allclose(got, Am @ Bm, rtol=1e-5, atol=1e-5)


# ---- Weed::softmax (src/ops/softmax.cpp:82-103); reference tests test/tests.cpp:1110-1171, 1206-1221 -----------

def _softmax1d(oracle, v):
    a = np.array(v, dtype=np.float32)
    out = np.zeros_like(a)
    return oracle.softmax([len(v)], 0, a, 0, [1], out, 0, [1])


def test_softmax_reference_cases(oracle):
    y = _softmax1d(oracle, [1, 2, 3])
    assert abs(float(y.sum()) - 1.0) < 0.01
    y = _softmax1d(oracle, [1, 3, 2])
    assert y[1] > y[2] > y[0]
    y = _softmax1d(oracle, [1000, 1001, 1002])
    assert np.isfinite(y).all() and abs(float(y.sum()) - 1.0) < 0.01
    y = _softmax1d(oracle, [2, 2, 2])
    np.testing.assert_allclose(y, 1.0 / 3.0, atol=1e-7)
    y = _softmax1d(oracle, [0, 1])
    denom = 1.0 + np.exp(1.0)
    np.testing.assert_allclose(y, [1.0 / denom, np.exp(1.0) / denom], atol=1e-7)
    # axis 1 of a 2x3 column-major matrix: rows are storage indices (0,2,4) and (1,3,5) (tests.cpp:1206-1221)
    a = np.arange(1, 7, dtype=np.float32)
    out = np.zeros_like(a)
    oracle.softmax([2, 3], 1, a, 0, [1, 2], out, 0, [1, 2])
    assert abs(out[[0, 2, 4]].sum() - 1.0) < 1e-6 and abs(out[[1, 3, 5]].sum() - 1.0) < 1e-6
    e = np.exp(np.array([1.0, 3.0, 5.0]) - 5.0)
    np.testing.assert_allclose(out[[0, 2, 4]], e / e.sum(), atol=1e-7)


def test_softmax_strided_rank4(oracle):
    rng = np.random.default_rng(2)
    shape = [2, 3, 4, 5]
    x = rng.normal(size=shape).astype(np.float32)
    # column-major storage of x
    stride = [1, 2, 6, 24]
    flat = np.asfortranarray(x).reshape(-1, order="F").copy()
    for axis in range(4):
        out = np.zeros_like(flat)
        oracle.softmax(shape, axis, flat, 0, stride, out, 0, stride)
        got = out.reshape(shape, order="F")
        e = np.exp(x.astype(np.float64) - x.max(axis=axis, keepdims=True))
        np.testing.assert_allclose(got, e / e.sum(axis=axis, keepdims=True), rtol=1e-6, atol=1e-7)


# ---- Weed::reduce / max / min (src/ops/reduce.cpp:33-58); reference tests test/tests.cpp:177-228 ----------------

def test_reduce_reference_cases(oracle):
    out = np.zeros(1, dtype=np.float32)
    assert oracle.reduce(0, [2], 0, np.array([1, 1], dtype=np.float32), 0, [1], out, 0, [0])[0] == 2
    assert oracle.reduce(1, [2], 0, np.array([0, 1], dtype=np.float32), 0, [1], out, 0, [0])[0] == 1
    assert oracle.reduce(2, [2], 0, np.array([0, 1], dtype=np.float32), 0, [1], out, 0, [0])[0] == 0


def test_reduce_strided_rank3(oracle):
    rng = np.random.default_rng(3)
    shape = [4, 3, 5]
    x = rng.normal(size=shape).astype(np.float32)
    flat = x.reshape(-1, order="F").copy()
    stride = [1, 4, 12]
    for axis in range(3):
        oshape = [s for i, s in enumerate(shape) if i != axis]
        ostride_full = [0, 0, 0]
        acc = 1
        for i in range(3):
            if i != axis:
                ostride_full[i] = acc
                acc *= shape[i]
        for op, fn in ((0, np.sum), (1, np.max), (2, np.min)):
            out = np.zeros(acc, dtype=np.float32)
            oracle.reduce(op, shape, axis, flat, 0, stride, out, 0, ostride_full)
            np.testing.assert_allclose(out.reshape(oshape, order="F"), fn(x.astype(np.float64), axis=axis), rtol=1e-6,
                                       atol=1e-6)


def test_triu_fill_rule(oracle):
    # src/ops/triu_fill.cpp:52-58: fill where i + diagonal <= j
    rows, cols = 5, 7
    for diag in (0, 1, 2):
        a = np.zeros(rows * cols, dtype=np.float32)
        oracle.triu_fill(a, 0, rows, cols, 1, rows, -7.0, diag)
        m = a.reshape(rows, cols, order="F")
        for i in range(rows):
            for j in range(cols):
                assert m[i, j] == (-7.0 if i + diag <= j else 0.0)
