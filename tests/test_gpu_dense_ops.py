"""GPU parity of the strided fp32 matmul, softmax and axis reductions, through the C ABI.

The reference pins these ops with tiny known-answer tests (test/tests.cpp:177-228, 1020-1041, 1110-1171, 1206-1221);
they are repeated here on the device, followed by strided / larger cases against the CPU checker.
Tolerance: fp32 sums in a different order than the checker's sequential loop -> rtol 2e-5 (atol scaled to the data);
max/min are exact.
"""
import numpy as np
import pytest

from gpu_helpers import col_major, dev
from weed_amd import workloads

pytestmark = pytest.mark.gpu


def test_matmul_reference_cases(gpu):
    import torch
    # 1x2 . 2x1 = 23 and the 2x1 . 1x2 outer product (tests.cpp:1020-1040), column-major operands
    x = col_major(np.array([[2, 3]], dtype=np.float32))
    y = col_major(np.array([[4], [5]], dtype=np.float32))
    z = col_major(np.zeros((1, 1), dtype=np.float32))
    gpu.matmul(x, y, z)
    assert z.cpu().item() == 23
    x = col_major(np.array([[2], [3]], dtype=np.float32))
    y = col_major(np.array([[4, 5]], dtype=np.float32))
    z = col_major(np.zeros((2, 2), dtype=np.float32))
    gpu.matmul(x, y, z)
    np.testing.assert_array_equal(z.cpu().numpy(), [[8, 10], [12, 15]])
    # tests.cpp:1327-1341
    A = col_major(np.array([[1, 3, 5], [2, 4, 6]], dtype=np.float32))
    B = col_major(np.array([[7, 10], [8, 11], [9, 12]], dtype=np.float32))
    C = col_major(np.zeros((2, 2), dtype=np.float32))
    gpu.matmul(A, B, C)
    np.testing.assert_array_equal(C.cpu().numpy(), np.array([[1, 3, 5], [2, 4, 6]]) @ np.array([[7, 10], [8, 11],
                                                                                                [9, 12]]))


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (7, 5, 11), (64, 64, 64), (130, 70, 33), (1, 300, 128), (257, 1, 1000),
                                   (512, 384, 256)])
def test_matmul_strided_against_checker(gpu, oracle, M, N, K):
    import torch
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32)
    want = np.zeros(M * N, dtype=np.float32)
    oracle.matmul(M, N, K, A.reshape(-1), (0, K, 1), B.reshape(-1), (0, N, 1), want, (0, N, 1))
    tol = dict(rtol=2e-5, atol=2e-5 * np.sqrt(K))
    # row-major, column-major, and views with offsets / non-unit strides
    for mk in (dev, col_major):
        C = mk(np.zeros((M, N), dtype=np.float32))
        gpu.matmul(mk(A), mk(B), C)
        np.testing.assert_allclose(C.cpu().numpy(), want.reshape(M, N), **tol)
    big_a = torch.zeros((M + 3, 2 * K + 1), device="cuda")
    big_a[2:2 + M, 1:1 + 2 * K:2] = dev(A)
    big_c = torch.full((2 * M, N + 5), -1.0, device="cuda")
    gpu.matmul(big_a[2:2 + M, 1:1 + 2 * K:2], dev(B).t().contiguous().t(), big_c[::2, 3:3 + N])
    np.testing.assert_allclose(big_c[::2, 3:3 + N].cpu().numpy(), want.reshape(M, N), **tol)
    assert torch.all(big_c[1::2] == -1.0) and torch.all(big_c[:, :3] == -1.0)  # nothing outside the view is written


@pytest.mark.parametrize("a_col,b_col,o_col", [(True, True, True), (True, False, False), (False, True, True),
                                                 (False, False, False), (True, True, False)])
@pytest.mark.parametrize("fp32_instruction,K", [(False, 160), (True, 160), (False, 144)])
def test_matmul_matrix_core_layouts(gpu, oracle, a_col, b_col, o_col, fp32_instruction, K):
    """Full 128 x 128 tiles with every combination of contiguous dimension (the four instances of the kernel on the
    bfloat16 instruction with split operands, of the one on the fp32 instruction when that is asked for, and of the
    latter for a k that is a multiple of 16 but not of 32) against the checker's sequential fp32 sums."""
    M, N = 256, 384
    rng = np.random.default_rng(M + N + K + a_col * 4 + b_col * 2 + o_col)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32)
    want = np.zeros(M * N, dtype=np.float32)
    oracle.matmul(M, N, K, A.reshape(-1), (0, K, 1), B.reshape(-1), (0, N, 1), want, (0, N, 1))
    C = (col_major if o_col else dev)(np.zeros((M, N), dtype=np.float32))
    gpu.matmul_tuning(fp32_instruction)
    try:
        gpu.matmul((col_major if a_col else dev)(A), (col_major if b_col else dev)(B), C)
    finally:
        gpu.matmul_tuning(False)
    np.testing.assert_allclose(C.cpu().numpy(), want.reshape(M, N), rtol=2e-5, atol=2e-5 * np.sqrt(K))


@pytest.mark.parametrize("M,N,K", [(128, 128, 32), (256, 384, 64), (132, 136, 36), (128, 256, 2048), (1000, 260, 1028)])
@pytest.mark.parametrize("wide_range", [False, True])
def test_matmul_split_products_keep_fp32_accuracy(gpu, M, N, K, wide_range):
    """Products that run on the bfloat16 matrix instruction (both operands split exactly into three parts, six of
    the nine products of parts kept) are as accurate as the same products on the fp32 instruction: against float64
    and relative to sum |a||b| per element, the largest error is at most 1.5 times the fp32 instruction's (+ 5e-8) and
    the mean error at most 1.25 times, for whole tiles, ragged sizes and k ranges, every layout, and operands whose
    magnitudes span 2^-20 .. 2^20.  A part's product left out or mis-paired would show as 2^-16 of a term: at k = 32
    and 64 that is ten times the errors seen."""
    rng = np.random.default_rng(M + 3 * N + 7 * K + wide_range)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32)
    if wide_range:
        A = (A * np.exp2(rng.integers(-20, 21, size=A.shape))).astype(np.float32)
        B = (B * np.exp2(rng.integers(-20, 21, size=B.shape))).astype(np.float32)
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    want = A64 @ B64
    scale = np.abs(A64) @ np.abs(B64)
    for mk_a, mk_b in ((col_major, col_major), (dev, dev), (col_major, dev), (dev, col_major)):
        err = {}
        for fp32_instruction in (True, False):
            C = col_major(np.zeros((M, N), dtype=np.float32))
            gpu.matmul_tuning(fp32_instruction)
            try:
                gpu.matmul(mk_a(A), mk_b(B), C)
            finally:
                gpu.matmul_tuning(False)
            err[fp32_instruction] = np.abs(C.cpu().numpy().astype(np.float64) - want) / scale
        assert err[True].max() <= 1.5e-6  # (the yardstick itself is sane)
        assert err[False].max() <= 1.5 * err[True].max() + 5e-8, (mk_a.__name__, mk_b.__name__, err[False].max(), err[True].max())
        assert err[False].mean() <= 1.25 * err[True].mean(), (mk_a.__name__, mk_b.__name__, err[False].mean(), err[True].mean())


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_matmul_random_shapes_through_the_dispatch(gpu, seed):
    """Forty random products per seed -- sizes that are and are not multiples of the tile or of 4, few and many rows,
    short and long k, either contiguous dimension per operand, padded (and so unaligned) views, with and without a
    bias, on either matrix instruction -- against the float64 product: the error stays below 2e-6 of sum |a||b| per
    element, and nothing outside a padded output view is written.  (What the launch code chooses between: whole
    tiles, checked 16-byte loads, element-wise guards, an interior with strips, k ranges, the streaming kernels.)"""
    import random
    import torch
    rnd = random.Random(seed)

    def dim():
        c = rnd.random()
        if c < 0.3:
            return rnd.choice([128, 256, 384, 512, 1024])
        if c < 0.6:
            return 4 * rnd.randint(5, 400)
        return rnd.randint(17, 1500)

    for _ in range(40):
        M, N = dim(), dim()
        K = rnd.choice([32, 64, 96, 128, 1024, 2048, 4096, 4100, 1000, 36, 999, 8 * rnd.randint(1, 300)])
        if M * N * K > 2 ** 32:
            K = max(8, K // 8)
        if rnd.random() < 0.15:
            M = rnd.randint(1, 70)
        la, lb, lo = rnd.choice("ik"), rnd.choice("kj"), rnd.choice("ij")
        pad = rnd.choice([0, 0, 4, 1])

        def view(rows, cols, contiguous_rows):
            if contiguous_rows:
                base = torch.randn((cols, rows + pad), device="cuda")
                return (base[:, :rows].t() if pad else base.t()), base
            base = torch.randn((rows, cols + pad), device="cuda")
            return (base[:, :cols] if pad else base), base

        A, _ = view(M, K, la == "i")
        B, _ = view(K, N, lb == "k")
        C, c_base = view(M, N, lo == "i")
        c_base.fill_(-7.0)
        bias = torch.randn(N, device="cuda") if rnd.random() < 0.3 else None
        fp32_instruction = rnd.random() < 0.3
        case = (M, N, K, la, lb, lo, pad, bias is not None, fp32_instruction)
        gpu.matmul_tuning(fp32_instruction)
        try:
            if bias is not None:
                gpu.linear(A, B, bias, C)
            else:
                gpu.matmul(A, B, C)
        finally:
            gpu.matmul_tuning(False)
        want = A.double() @ B.double()
        scale = A.double().abs() @ B.double().abs()
        if bias is not None:
            want = want + bias.double()
            scale = scale + bias.double().abs()
        err = ((C.double() - want).abs() / scale).max().item()
        assert err < 2e-6, (case, err)
        if pad:
            assert bool((c_base[:, (M if lo == "i" else N):] == -7.0).all()), case


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (40, 640, 1024), (132, 260, 68)])
def test_matmul_on_the_fp32_instruction_keeps_tiny_operands(gpu, M, N, K):
    """What weed_hip_matmul_tuning(1) is for: operands around 2^-120 against operands around 2^120.  On the fp32
    instruction the product keeps fp32 accuracy (whole tiles, the 17-64-row projection, ragged sizes); split into
    bfloat16 parts, the small operands' second and third parts would fall below bfloat16's normal range."""
    rng = np.random.default_rng(M + N + K)
    A = (rng.standard_normal((M, K)) * 2.0 ** -120).astype(np.float32)
    B = (rng.standard_normal((K, N)) * 2.0 ** 120).astype(np.float32)
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    want = A64 @ B64
    scale = np.abs(A64) @ np.abs(B64)
    C = col_major(np.zeros((M, N), dtype=np.float32))
    gpu.matmul_tuning(True)
    try:
        gpu.matmul(col_major(A), col_major(B), C)
    finally:
        gpu.matmul_tuning(False)
    err = np.abs(C.cpu().numpy().astype(np.float64) - want) / scale
    assert err.max() <= 1e-6, err.max()


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (1, 100, 260), (5, 33, 1000), (16, 48, 256), (17, 16, 4100),
                                   (33, 250, 516), (64, 512, 1024), (24, 600, 1100), (50, 1040, 772)])
def test_matmul_decode_projections(gpu, oracle, M, N, K):
    """Few rows against a tall column-major weight (y = x.W at decode time, the matrix-core streaming kernel):
    row counts on both sides of the 16-row tiles, column counts that are not multiples of 16, k ranges that do not
    fill the last 64-step, activations column-major, row-major and as a strided view; nothing outside the output
    view may be written."""
    import torch
    rng = np.random.default_rng(M * 11 + N * 5 + K)
    A = rng.standard_normal((M, K), dtype=np.float32)
    W = (rng.standard_normal((K, N), dtype=np.float32) * 0.05).astype(np.float32)
    want = (A.astype(np.float64) @ W.astype(np.float64))
    if M * N * K <= 5_000_000:
        chk = np.zeros(M * N, dtype=np.float32)
        oracle.matmul(M, N, K, A.reshape(-1), (0, K, 1), W.reshape(-1), (0, N, 1), chk, (0, N, 1))
        np.testing.assert_allclose(chk.reshape(M, N), want, rtol=2e-5, atol=2e-5 * np.sqrt(K))
    tol = dict(rtol=2e-5, atol=2e-6 * np.sqrt(K))
    Wd = col_major(W)
    for mk in (col_major, dev):
        C = mk(np.zeros((M, N), dtype=np.float32))
        gpu.matmul(mk(A), Wd, C)
        np.testing.assert_allclose(C.cpu().numpy(), want, **tol)
    big_a = torch.zeros((M + 2, 3 * K + 2), device="cuda")
    big_a[1:1 + M, 2:2 + 3 * K:3] = dev(A)
    big_c = torch.full((M + 4, 2 * N + 3), -7.0, device="cuda")
    gpu.matmul(big_a[1:1 + M, 2:2 + 3 * K:3], Wd, big_c[2:2 + M, 1:1 + 2 * N:2])
    np.testing.assert_allclose(big_c[2:2 + M, 1:1 + 2 * N:2].cpu().numpy(), want, **tol)
    assert torch.all(big_c[:2] == -7.0) and torch.all(big_c[2 + M:] == -7.0) and torch.all(big_c[:, 0::2] == -7.0)


@pytest.mark.parametrize("M,N,K", [(200, 300, 4096), (128, 128, 2048), (130, 70, 1030), (17, 17, 8), (257, 129, 33),
                                   (1000, 1000, 100), (1000, 1100, 512), (300, 4136, 1024), (129, 128, 2048),
                                   (260, 4100, 4096), (512, 4096, 1024), (760, 4096, 1024), (1000, 1000, 1028)])
@pytest.mark.parametrize("fp32_instruction", [False, True])
def test_matmul_matrix_core_edges(gpu, M, N, K, fp32_instruction):
    """Shapes that are not multiples of the 128 x 128 x 16 tiles, unaligned and doubly strided views, and few tiles with
    a long k (split over workgroups, summed by a second kernel), also 128 and 192 tiles, which split in two and four:
    against float64, and nothing outside the output view may be written.  Sizes that are multiples of 4 run the
    instances whose 16-byte loads are checked as a whole, the others the element-wise ones."""
    import torch
    rng = np.random.default_rng(M + 2 * N + 3 * K)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tol = dict(rtol=2e-5, atol=4e-6 * np.sqrt(K) * 3)
    gpu.matmul_tuning(fp32_instruction)
    try:
        _matrix_core_edges(gpu, M, N, K, A, B, want, tol)
    finally:
        gpu.matmul_tuning(False)


def _matrix_core_edges(gpu, M, N, K, A, B, want, tol):
    import torch
    for mk_a, mk_b in ((col_major, col_major), (dev, dev), (col_major, dev), (dev, col_major)):
        C = col_major(np.zeros((M, N), dtype=np.float32))
        gpu.matmul(mk_a(A), mk_b(B), C)
        np.testing.assert_allclose(C.cpu().numpy(), want, **tol)
    # views strided in both dimensions, with odd offsets; the output is a padded slice
    big_a = torch.zeros((2 * M + 1, 3 * K + 1), device="cuda")
    big_a[1::2, 1::3] = dev(A)
    big_b = torch.zeros((2 * K + 3, 2 * N + 1), device="cuda")
    big_b[3::2, 1::2] = dev(B)
    big_c = torch.full((M + 3, N + 5), -7.0, device="cuda")
    gpu.matmul(big_a[1::2, 1::3], big_b[3::2, 1::2], big_c[1:1 + M, 2:2 + N])
    got = big_c.cpu().numpy()
    np.testing.assert_allclose(got[1:1 + M, 2:2 + N], want, **tol)
    inner = np.zeros_like(got, dtype=bool)
    inner[1:1 + M, 2:2 + N] = True
    assert (got[~inner] == -7.0).all()


@pytest.mark.parametrize("M,N,K", [(3, 5, 7), (8, 4096, 1024), (16, 100, 260), (40, 640, 1024), (64, 250, 516),
                                   (128, 256, 64), (70, 33, 19), (132, 260, 68), (256, 256, 2048)])
def test_linear_equals_product_then_broadcast_add(gpu, M, N, K):
    """The bias added in the product's last step gives the bits of the two separate ops of Linear::forward
    (matmul, then the broadcast add), on every product kernel (generic, matrix-core tiles, both streaming kernels);
    the bias may be a strided view, and a null bias gives the plain product."""
    import torch
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    A = col_major(rng.standard_normal((M, K), dtype=np.float32))
    W = col_major(rng.standard_normal((K, N), dtype=np.float32) * 0.05)
    bias_store = dev(rng.standard_normal(2 * N + 1, dtype=np.float32))
    bias = bias_store[1:1 + 2 * N:2]
    plain = col_major(np.zeros((M, N), dtype=np.float32))
    gpu.matmul(A, W, plain)
    want = col_major(np.zeros((M, N), dtype=np.float32))
    gpu.elementwise(gpu.EW_ADD, plain, bias.reshape(1, N), want)
    got = col_major(np.full((M, N), 9.0, dtype=np.float32))
    gpu.linear(A, W, bias, got)
    assert torch.equal(got, want)
    assert torch.equal(want, plain + bias.reshape(1, N))
    gpu.linear(A, W, None, got)
    assert torch.equal(got, plain)


@pytest.mark.parametrize("M,N,K", [(7, 5, 11), (64, 300, 128), (128, 256, 64), (4, 32, 512)])
def test_matmul_batched_equals_the_loop(gpu, M, N, K):
    """(batch x heads) products in one launch give what the 2-D entry point gives product by product (bit for bit:
    the same kernel instance runs either way), for contiguous batches and for permuted / strided views, on the
    generic, the matrix-core and the streaming kernel."""
    import torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(M + N + K)
    B0, B1 = 3, 4
    a = torch.randn((B0, B1, M, K), generator=gen, device="cuda")
    b = torch.randn((B0, B1, K, N), generator=gen, device="cuda")
    views = [(a, b, torch.zeros((B0, B1, M, N), device="cuda")),
             # [B0, M, B1, K] storage seen as [B0, B1, M, K]; b column-major per product; out with padding
             (a.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3),
              b.transpose(2, 3).contiguous().transpose(2, 3),
              torch.zeros((B0, B1, M, N + 4), device="cuda")[..., :N])]
    for av, bv, out in views:
        gpu.matmul_batched(av, bv, out)
        for i in range(B0):
            for j in range(B1):
                one = torch.zeros_like(out[i, j])
                gpu.matmul(av[i, j], bv[i, j], one)
                assert torch.equal(out[i, j], one)
        ref = (a.double() @ b.double()).float()
        torch.testing.assert_close(out, ref, rtol=2e-5, atol=2e-5 * K ** 0.5)


def test_matmul_cfg5_sampled(gpu):
    """Configuration 5b at full size ([4096 x 1024] . [1024 x 4096], column-major): the scalar checker would need
    minutes, so 4096 sampled outputs are compared with float64 dot products, plus the column sums identity
    1^T (A W) = (1^T A) W."""
    A, W = workloads.matmul_config()
    M, K = A.shape
    N = W.shape[1]
    Ad, Wd = col_major(A), col_major(W)
    C = col_major(np.zeros((M, N), dtype=np.float32))
    gpu.matmul(Ad, Wd, C)
    Ch = C.cpu().numpy()
    rng = np.random.default_rng(0)
    ii, jj = rng.integers(0, M, 4096), rng.integers(0, N, 4096)
    want = np.einsum("ik,ki->i", A[ii].astype(np.float64), W[:, jj].astype(np.float64))
    np.testing.assert_allclose(Ch[ii, jj], want, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(Ch.astype(np.float64).sum(axis=0), A.astype(np.float64).sum(axis=0) @ W.astype(np.float64),
                               rtol=1e-4, atol=1e-3)


def test_softmax_reference_cases(gpu):
    import torch

    def sm(v):
        a = dev(np.array(v, dtype=np.float32))
        out = torch.zeros_like(a)
        gpu.softmax(a, out, 0)
        return out.cpu().numpy()

    assert abs(sm([1, 2, 3]).sum() - 1.0) < 1e-6
    y = sm([1, 3, 2])
    assert y[1] > y[2] > y[0]
    y = sm([1000, 1001, 1002])
    assert np.isfinite(y).all() and abs(y.sum() - 1.0) < 1e-6
    np.testing.assert_allclose(sm([2, 2, 2]), 1.0 / 3.0, atol=1e-7)
    denom = 1.0 + np.exp(1.0)
    np.testing.assert_allclose(sm([0, 1]), [1.0 / denom, np.exp(1.0) / denom], atol=1e-7)
    # axis 1 of the 2x3 column-major matrix (tests.cpp:1206-1221)
    a = col_major(np.array([[1, 3, 5], [2, 4, 6]], dtype=np.float32))
    out = torch.zeros_like(a)
    gpu.softmax(a, out, 1)
    e = np.exp(np.array([1.0, 3.0, 5.0]) - 5.0)
    np.testing.assert_allclose(out.cpu().numpy(), np.stack([e / e.sum()] * 2), atol=1e-7)


@pytest.mark.parametrize("shape", [(5,), (3, 1000), (1000, 3), (2, 3, 4, 5), (1, 32, 1, 2048), (4, 7, 33, 65)])
def test_softmax_and_reduce_strided_against_checker(gpu, oracle, shape):
    import torch
    rng = np.random.default_rng(len(shape) * 100 + shape[-1])
    x = (rng.standard_normal(shape, dtype=np.float32) * 3.0)
    flat = np.transpose(x).reshape(-1).copy()  # column-major storage
    stride = [int(np.prod(shape[:i])) for i in range(len(shape))]
    for mk in (col_major, dev):
        xd = mk(x)
        for axis in range(len(shape)):
            out = torch.zeros_like(xd)
            gpu.softmax(xd, out, axis)
            want = np.zeros_like(flat)
            oracle.softmax(list(shape), axis, flat, 0, stride, want, 0, stride)
            want = np.transpose(want.reshape(shape[::-1]))
            np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-5, atol=1e-7)
            oshape = [s for i, s in enumerate(shape) if i != axis] or [1]
            for op, fn in ((gpu.REDUCE_SUM, np.sum), (gpu.REDUCE_MAX, np.max), (gpu.REDUCE_MIN, np.min)):
                r = torch.zeros(oshape, device="cuda")
                if len(shape) == 1:
                    gpu.check(gpu.load().weed_hip_reduce_f32(op, 1, gpu.u32(shape), 0, xd.data_ptr(), 0,
                                                             gpu.u32(xd.stride()), r.data_ptr(), 0, gpu.u32([0])))
                else:
                    gpu.reduce(op, xd, r, axis)
                ref = fn(x.astype(np.float64), axis=axis).reshape(oshape)
                if op == gpu.REDUCE_SUM:
                    np.testing.assert_allclose(r.cpu().numpy(), ref, rtol=2e-5, atol=2e-5 * np.sqrt(shape[axis]))
                else:
                    np.testing.assert_array_equal(r.cpu().numpy(), ref.astype(np.float32))


@pytest.mark.parametrize("shape,axis", [((9004, 40), 0), ((40000, 24), 1), ((64, 8, 1, 700), 3), ((260, 3, 5), 0),
                                        ((192, 1100), 0), ((2044, 1030), 0), ((67, 1500), 0), ((1101, 1200), 0),
                                        ((300, 9000), 1), ((2060, 5000), 1),
                                        ((8200, 300), 1), ((12300, 1100), 1),
                                        ((16, 5000), 0), ((40, 3000), 0), ((7, 2000), 0), ((500, 1100), 0), ((29, 1500), 0),
                                        ((256, 1030), 0), ((64, 40000), 1), ((300, 20000), 1), ((2048, 4100), 1), ((4000, 4200), 1),
                                        ((32768, 5), 0), ((20000, 4), 0), ((40004, 3), 0),
                                        ((15, 100000), 1), ((8, 32768), 1), ((5, 40000), 1), ((3600, 16400), 1)])
def test_softmax_and_reduce_launch_shapes(gpu, shape, axis):
    """One case per way the threads are spread: a contiguous row longer than what the registers keep between the
    passes, enough rows for 32 per workgroup, few long strided rows (decode-time scores), a short aligned row, and
    many short contiguous rows (one wavefront each: aligned, longer than a wavefront's registers, unaligned lengths),
    few strided rows of 9000 and 5000 elements, which 4 and 8 neighbouring rows per workgroup keep in registers,
    and many strided rows of 300 (kept in 32 registers per thread) and of 1100 elements (two passes); many contiguous
    rows of 7 to 500 elements, which share a wavefront (4 to 32 lanes per row); few rows with a strided axis of 20000
    and 40000 elements, which is cut into bands (three launches); few contiguous rows of 20000 to 40004 elements
    (sixteen wavefronts per row, one pass up to 32768 elements); fewer than 16 long strided rows and 3600 rows of 16400,
    which go by bands as well (the sums from 2^18 elements on).
    Some positions are masked with -inf, one row of the decode case entirely (its softmax is NaN, as in numpy)."""
    import torch
    rng = np.random.default_rng(shape[0] + axis)
    x = rng.standard_normal(shape, dtype=np.float32) * 4.0
    x[rng.random(shape) < 0.1] = -np.inf
    if len(shape) == 4:
        x[3, 2, 0, :] = -np.inf
    xd = col_major(x)
    out = torch.zeros_like(xd)
    gpu.softmax(xd, out, axis)
    x64 = x.astype(np.float64)
    with np.errstate(invalid="ignore"):
        e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
        want = e / e.sum(axis=axis, keepdims=True)
    got = out.cpu().numpy()
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_allclose(np.nan_to_num(got), np.nan_to_num(want), rtol=2e-5, atol=1e-7)
    oshape = [s for i, s in enumerate(shape) if i != axis]
    finite = np.where(np.isinf(x), 0.0, x).astype(np.float32)
    fd = col_major(finite)
    for op, fn, src, srcd in ((gpu.REDUCE_SUM, np.sum, finite, fd), (gpu.REDUCE_MAX, np.max, x, xd),
                              (gpu.REDUCE_MIN, np.min, finite, fd)):
        r = col_major(np.zeros(oshape, dtype=np.float32))
        gpu.reduce(op, srcd, r, axis)
        ref = fn(src.astype(np.float64), axis=axis)
        if op == gpu.REDUCE_SUM:
            np.testing.assert_allclose(r.cpu().numpy(), ref, rtol=2e-5, atol=2e-5 * np.sqrt(shape[axis]))
        else:
            np.testing.assert_array_equal(r.cpu().numpy(), ref.astype(np.float32))


def test_reduce_reference_cases(gpu):
    import torch
    # tests.cpp:177-228: sum([1,1]) = 2, max([0,1]) = 1, min([0,1]) = 0
    for op, v, want in ((gpu.REDUCE_SUM, [1, 1], 2), (gpu.REDUCE_MAX, [0, 1], 1), (gpu.REDUCE_MIN, [0, 1], 0)):
        a = dev(np.array(v, dtype=np.float32))
        r = torch.zeros(1, device="cuda")
        gpu.check(gpu.load().weed_hip_reduce_f32(op, 1, gpu.u32([2]), 0, a.data_ptr(), 0, gpu.u32([1]), r.data_ptr(), 0,
                                                 gpu.u32([0])))
        assert r.cpu().item() == want


def test_softmax_on_a_view_with_offset(gpu, oracle):
    import torch
    rng = np.random.default_rng(8)
    big = dev(rng.standard_normal((6, 40), dtype=np.float32))
    view = big[1:5, 3:35:2]
    out = torch.full((6, 40), 7.0, device="cuda")
    gpu.softmax(view, out[1:5, 3:35:2], 1)
    x = view.cpu().numpy().astype(np.float64)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    np.testing.assert_allclose(out[1:5, 3:35:2].cpu().numpy(), e / e.sum(axis=1, keepdims=True), rtol=2e-5, atol=1e-7)
    assert torch.all(out[0] == 7.0) and torch.all(out[:, 4::2] == 7.0)


@pytest.mark.parametrize("shape,perm", [((130, 67), (1, 0)), ((5, 33, 70), (2, 1, 0)), ((5, 33, 70), (1, 0, 2)),
                                        ((3, 17, 4, 32), (0, 2, 1, 3)), ((3, 17, 4, 32), (3, 1, 2, 0)),
                                        ((64, 200), (1, 0)), ((16, 16), (1, 0))])
def test_copy_of_permuted_views(gpu, shape, perm):
    """A permuted view made contiguous (what follows every transpose in the attention module): exact copies, with
    ragged tiles, extra dimensions on either side and a destination that is itself a slice of a larger tensor."""
    import torch
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape, dtype=np.float32)
    view = col_major(x).permute(*perm)
    want = np.transpose(x, perm)
    out = col_major(np.zeros(want.shape, dtype=np.float32))
    gpu.elementwise(gpu.EW_COPY, view, None, out)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    big = col_major(np.full((want.shape[0] + 3,) + want.shape[1:], 7.0, dtype=np.float32))
    gpu.elementwise(gpu.EW_COPY, view, None, big[2:-1])
    got = big.cpu().numpy()
    np.testing.assert_array_equal(got[2:-1], want)
    assert (got[:2] == 7.0).all() and (got[-1:] == 7.0).all()


def test_elementwise_broadcast_and_gather(gpu):
    """add / sub / mul / div are single IEEE operations, so they must equal numpy bit for bit, including with a
    broadcast (stride 0) operand, transposed views and an output that aliases the first operand."""
    import torch
    rng = np.random.default_rng(9)
    a = rng.standard_normal((5, 7, 3), dtype=np.float32)
    b = rng.standard_normal((1, 7, 1), dtype=np.float32) + 3.0
    ad, bd = col_major(a), dev(b)
    for op, fn in ((gpu.EW_ADD, np.add), (gpu.EW_SUB, np.subtract), (gpu.EW_MUL, np.multiply), (gpu.EW_DIV, np.divide)):
        out = torch.zeros((5, 7, 3), device="cuda")
        gpu.elementwise(op, ad, bd, out)
        np.testing.assert_array_equal(out.cpu().numpy(), fn(a, b))
    # strided gather: a transposed view copied into a contiguous tensor (Tensor::contiguous)
    out = torch.zeros((3, 5, 7), device="cuda")
    gpu.elementwise(gpu.EW_COPY, ad.permute(2, 0, 1), None, out)
    np.testing.assert_array_equal(out.cpu().numpy(), a.transpose(2, 0, 1))
    # in place: a += b
    acc = dev(a.copy())
    gpu.elementwise(gpu.EW_ADD, acc, bd, acc)
    np.testing.assert_array_equal(acc.cpu().numpy(), a + b)
    # scalar division as attention uses it: scores / sqrt(d)
    s = dev(np.array([np.sqrt(np.float32(128.0))], dtype=np.float32))
    out = torch.zeros((5, 7, 3), device="cuda")
    gpu.elementwise(gpu.EW_DIV, ad, s.reshape(1, 1, 1), out)
    np.testing.assert_array_equal(out.cpu().numpy(), a / np.sqrt(np.float32(128.0)))


@pytest.mark.parametrize("rows,cols,diag", [(1, 1, 1), (4, 4, 1), (5, 9, 1), (9, 5, 0), (6, 6, 3)])
def test_triu_fill_against_checker(gpu, oracle, rows, cols, diag):
    rng = np.random.default_rng(10)
    a = rng.standard_normal((rows, cols), dtype=np.float32)
    ad = col_major(a)
    gpu.triu_fill(ad, -1.701411835e38, diag)
    want = np.asfortranarray(a).ravel(order="F").copy()
    oracle.triu_fill(want, 0, rows, cols, 1, rows, -1.701411835e38, diag)
    np.testing.assert_array_equal(ad.cpu().numpy(), want.reshape((rows, cols), order="F"))


@pytest.mark.parametrize("pos0", [0, 11])
def test_rope_bit_exact_against_checker(gpu, oracle, pos0):
    """x * cos + rotate_half(x) * sin is two rounded products and one add: bit-exact against the checker, on the
    (B, heads, T, head_dim) view of a column-major (B, T, heads, head_dim) tensor as the attention module forms it."""
    import torch
    rng = np.random.default_rng(12)
    B, H, T, d, L = 2, 3, 5, 64, 32
    x = rng.standard_normal((B, H, T, d)).astype(np.float32)
    cos_t, sin_t = oracle.rope_tables(d, L)
    want = oracle.rope_forward(x, cos_t, sin_t, L, pos0=pos0)
    xd = col_major(np.ascontiguousarray(x.transpose(0, 2, 1, 3))).permute(0, 2, 1, 3)  # logical [B, H, T, d]
    out = torch.zeros((B, H, T, d), device="cuda")
    gpu.rope(xd, dev(cos_t), dev(sin_t), L, out, pos0=pos0)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    with pytest.raises(gpu.WeedHipError):
        gpu.rope(xd, dev(cos_t), dev(sin_t), L, out, pos0=L - T + 1)  # positions past the table


def test_device_memory_blocks_are_reused_in_stream_order(gpu):
    """weed_hip_free keeps a block, weed_hip_malloc hands it out again for a request of about the same size (no driver
    call, no wait), a much smaller or larger request gets its own block, and weed_hip_release_cached empties the
    cache.  Reuse is safe without a wait because all work goes to one stream: a copy queued before the free is still
    read back intact after the block's next owner overwrote it later in the stream."""
    from ctypes import byref, c_void_p
    lib = gpu.load()

    def malloc(n):
        p = c_void_p()
        gpu.check(lib.weed_hip_malloc(byref(p), n))
        return p.value

    gpu.check(lib.weed_hip_release_cached())
    a = malloc(3 << 20)
    gpu.check(lib.weed_hip_free(c_void_p(a)))
    b = malloc((3 << 20) - 4096)
    assert b == a
    c = malloc(3 << 20)
    assert c != a
    small = malloc(1000)
    assert small not in (a, c)
    big = malloc(64 << 20)
    assert big not in (a, c)
    # stream order: fill b, copy it out, free it, let the next owner overwrite it, then look at the copy
    src = np.arange(1 << 18, dtype=np.float32)
    keep = malloc(src.nbytes)
    gpu.check(lib.weed_hip_memcpy_h2d(c_void_p(b), src.ctypes.data_as(c_void_p), src.nbytes))
    gpu.check(lib.weed_hip_memcpy_d2d(c_void_p(keep), c_void_p(b), src.nbytes))
    gpu.check(lib.weed_hip_free(c_void_p(b)))
    again = malloc(3 << 20)
    assert again == a
    gpu.check(lib.weed_hip_memset(c_void_p(again), 0, 3 << 20))
    back = np.empty_like(src)
    gpu.check(lib.weed_hip_memcpy_d2h(back.ctypes.data_as(c_void_p), c_void_p(keep), src.nbytes))
    np.testing.assert_array_equal(back, src)
    for p in (again, c, small, big, keep):
        gpu.check(lib.weed_hip_free(c_void_p(p)))
    gpu.check(lib.weed_hip_release_cached())
    fresh = malloc(3 << 20)
    gpu.check(lib.weed_hip_free(c_void_p(fresh)))
    gpu.check(lib.weed_hip_release_cached())


def test_degenerate_shapes(gpu):
    """Axes of length one, single rows, one very long row (contiguous and strided), rank-8 broadcasting with size-1
    dimensions everywhere, transposed copies smaller than a tile, rotations of width 1, 2, 3 and 129."""
    import torch
    rng = np.random.default_rng(123)
    for shape, axis in [((1,), 0), ((5, 1), 1), ((1, 5), 0), ((1, 1, 1), 1), ((3000, 1), 1), ((1, 3000), 0),
                        ((1, 300000), 1), ((300000, 1), 0)]:
        x = rng.standard_normal(shape, dtype=np.float32)
        for mk in (col_major, dev):
            xd = mk(x)
            out = torch.zeros_like(xd)
            gpu.softmax(xd, out, axis)
            x64 = x.astype(np.float64)
            e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
            np.testing.assert_allclose(out.cpu().numpy(), e / e.sum(axis=axis, keepdims=True), rtol=3e-5, atol=1e-12)
            if len(shape) > 1:
                r = mk(np.zeros([n for i, n in enumerate(shape) if i != axis], dtype=np.float32))
                gpu.reduce(gpu.REDUCE_MAX, xd, r, axis)
                np.testing.assert_array_equal(r.cpu().numpy(), x.max(axis=axis))
                gpu.reduce(gpu.REDUCE_SUM, xd, r, axis)
                np.testing.assert_allclose(r.cpu().numpy(), x64.sum(axis=axis), rtol=2e-5, atol=2e-5 * np.sqrt(shape[axis]))
    x = rng.standard_normal((2, 1, 3, 1, 4, 1, 5, 2), dtype=np.float32)
    y = rng.standard_normal((1, 1, 3, 1, 1, 1, 5, 1), dtype=np.float32)
    out = col_major(np.zeros(x.shape, dtype=np.float32))
    gpu.elementwise(gpu.EW_MUL, col_major(x), dev(y), out)
    np.testing.assert_array_equal(out.cpu().numpy(), x * y)
    for shape in [(16, 16), (17, 33), (1, 64), (64, 1), (15, 100)]:
        x = rng.standard_normal(shape, dtype=np.float32)
        out = col_major(np.zeros(shape[::-1], dtype=np.float32))
        gpu.elementwise(gpu.EW_COPY, col_major(x).t(), None, out)
        np.testing.assert_array_equal(out.cpu().numpy(), x.T)
    for d in (1, 2, 3, 129):
        x = rng.standard_normal((7, d), dtype=np.float32)
        r = rng.standard_normal((d, d), dtype=np.float32)  # element (i, j) of the column-major matrix: r.T.flat[i + d*j]
        out = dev(np.zeros((7, d), dtype=np.float32))
        gpu.apply_rotation(dev(x), col_major(r), out)
        np.testing.assert_allclose(out.cpu().numpy(), x.astype(np.float64) @ r.astype(np.float64), rtol=1e-5, atol=1e-5)


def test_random_shapes_and_layouts(gpu):
    """Seeded random shapes, each operand row-major, column-major or a strided slice of a larger tensor: products
    (with and without the fused bias: every kernel the dispatcher can pick), softmax, the three reductions and layout
    changing copies against float64 numpy."""
    import torch
    rng = np.random.default_rng(5)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)

    def view(shape, kind):
        if kind == 0:
            return torch.randn(shape, generator=gen, device="cuda")
        if kind == 1:
            return torch.randn(shape[::-1], generator=gen, device="cuda").permute(*reversed(range(len(shape))))
        big = torch.randn(tuple(2 * n + 1 for n in shape), generator=gen, device="cuda")
        return big[tuple(slice(1, 1 + 2 * n, 2) for n in shape)]

    def f64(t):
        return t.cpu().numpy().astype(np.float64)

    for _ in range(80):
        M = int(rng.choice([1, 2, 7, 16, 17, 33, 64, 65, 100, 128, 200, 256, 300]))
        N = int(rng.choice([1, 5, 16, 17, 48, 100, 128, 250, 512, 640, 1024]))
        K = int(rng.choice([1, 3, 8, 16, 33, 64, 100, 256, 260, 512, 1030, 2048, 4096]))
        a, b = view((M, K), int(rng.integers(3))), view((K, N), int(rng.integers(3)))
        out = view((M, N), int(rng.integers(3)))
        bias = torch.randn(N, generator=gen, device="cuda") if rng.integers(2) else None
        gpu.linear(a, b, bias, out)
        want = f64(a) @ f64(b) + (f64(bias) if bias is not None else 0.0)
        np.testing.assert_allclose(f64(out), want, rtol=2e-5, atol=1.2e-5 * np.sqrt(K),
                                   err_msg="%d x %d x %d, strides %s %s %s" % (M, K, N, a.stride(), b.stride(), out.stride()))
    for _ in range(80):
        rank = int(rng.integers(1, 5))
        shape = tuple(int(rng.choice([1, 2, 3, 5, 16, 33, 64, 130, 300])) for _ in range(rank))
        if np.prod(shape) > 2_000_000:
            continue
        axis = int(rng.integers(rank))
        x, out = view(shape, int(rng.integers(3))), view(shape, int(rng.integers(3)))
        what = "shape %s axis %d, strides %s -> %s" % (shape, axis, x.stride(), out.stride())
        gpu.softmax(x, out, axis)
        x64 = f64(x)
        e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
        np.testing.assert_allclose(f64(out), e / e.sum(axis=axis, keepdims=True), rtol=3e-5, atol=1e-9, err_msg=what)
        if rank > 1:
            r = view(tuple(n for i, n in enumerate(shape) if i != axis), int(rng.integers(3)))
            for op, fn in ((gpu.REDUCE_SUM, np.sum), (gpu.REDUCE_MAX, np.max), (gpu.REDUCE_MIN, np.min)):
                gpu.reduce(op, x, r, axis)
                np.testing.assert_allclose(f64(r), fn(x64, axis=axis), rtol=2e-5, atol=2e-5 * np.sqrt(shape[axis]),
                                           err_msg=what)
        y = view(shape, int(rng.integers(3)))
        gpu.elementwise(gpu.EW_COPY, x, None, y)
        assert torch.equal(x, y), what


# ---- activations and norms of the attention module's callers ---------------------------------------------------

def test_activations_reference_cases_and_checker(gpu, oracle):
    """Weed::relu / sigmoid / tanh (src/ops/real_unary.cpp:80,135,191), Tensor::gelu (src/tensors/tensor.cpp:841-851)
    and SwiGLU's gate (include/modules/swiglu.hpp:71-77).  The reference's own cases (test/tests.cpp:230-244, 284-291,
    314-321) exactly, then seeded values against the CPU checker: relu bit for bit, the others to a few ulp (they go
    through exp / tanh, whose last bit differs between math libraries)."""
    import torch

    def run(op, v, b=None):
        a = dev(np.asarray(v, dtype=np.float32))
        out = torch.zeros_like(a)
        gpu.elementwise(op, a, dev(np.asarray(b, dtype=np.float32)) if b is not None else None, out)
        return out.cpu().numpy()

    assert run(gpu.EW_RELU, [2.0, -2.0]).tolist() == [2.0, 0.0]
    assert run(gpu.EW_SIGMOID, [0.0])[0] == 0.5
    assert run(gpu.EW_TANH, [0.0])[0] == 0.0
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(100000) * 3, [0.0, -0.0, 30.0, -30.0, 88.0, -88.0]]).astype(np.float32)
    up = rng.standard_normal(x.size).astype(np.float32)
    np.testing.assert_array_equal(run(gpu.EW_RELU, x), oracle.unary(oracle.RELU, x))
    np.testing.assert_allclose(run(gpu.EW_SIGMOID, x), oracle.unary(oracle.SIGMOID, x), rtol=1e-6, atol=1e-37)
    np.testing.assert_allclose(run(gpu.EW_TANH, x), oracle.unary(oracle.TANH, x), rtol=1e-6, atol=1e-37)
    np.testing.assert_allclose(run(gpu.EW_GELU, x), oracle.unary(oracle.GELU, x), rtol=2e-6, atol=3e-7)
    np.testing.assert_allclose(run(gpu.EW_SILU_MUL, x, up), oracle.silu_mul(x, up), rtol=2e-6, atol=1e-37)
    # strided and broadcast operands: a column-major (B, T, d_ff) gate against an `up` that repeats over T
    g3 = rng.standard_normal((5, 3, 70)).astype(np.float32)
    u3 = rng.standard_normal((5, 1, 70)).astype(np.float32)
    gd, ud = col_major(g3), col_major(u3)
    out = torch.zeros_like(gd)
    gpu.elementwise(gpu.EW_SILU_MUL, gd, ud, out)
    want = oracle.silu_mul(g3, np.broadcast_to(u3, g3.shape))
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-6, atol=1e-37)


@pytest.mark.parametrize("shape,axis", [((3,), 0), ((64, 1, 4096), 2), ((4, 6, 8), 2), ((16, 6, 8), 2), ((3, 5, 4096), 2),
                                        ((2, 700, 96), 2), ((4096, 3), 0), ((20000, 40), 1), ((7, 20000), 1),
                                        ((33, 4, 5000), 2), ((5, 9, 11), 1)])
def test_norms_against_checker(gpu, oracle, shape, axis):
    """RMSNorm::forward (include/modules/rms_norm.hpp:34-38) and LayerNorm::forward (src/modules/layernorm.cpp:29-42)
    as one kernel each, on column-major tensors (the layout the modules see: a decode step's (B, 1, d_model) has the
    batch index fastest) and on row-major ones (the axis contiguous), against the CPU checker.  The checker adds a
    row one element after the other in fp32 as the reference does; the kernels add as trees, so the comparison allows
    the rounding of a sum of that length, and a float64 evaluation has to lie within the same distance."""
    import torch
    rng = np.random.default_rng(shape[0] * 7 + len(shape))
    n = shape[axis]
    x = (rng.standard_normal(shape) * rng.uniform(0.5, 8.0) + rng.uniform(-1, 1)).astype(np.float32)
    w = rng.uniform(0.5, 2.0, n).astype(np.float32)
    beta = rng.standard_normal(n).astype(np.float32)
    eps = oracle.norm_epsilon()
    rows = np.moveaxis(x, axis, -1).reshape(-1, n)
    back = lambda y: np.moveaxis(y.reshape(np.moveaxis(x, axis, -1).shape), -1, axis)
    want_rms, want_ln = back(oracle.rms_norm(rows, w)), back(oracle.layer_norm(rows, w, beta))
    x64 = x.astype(np.float64)
    bshape = [1] * len(shape)
    bshape[axis] = n
    w64, b64 = w.astype(np.float64).reshape(bshape), beta.astype(np.float64).reshape(bshape)
    f64_rms = x64 / np.sqrt(np.mean(x64 * x64, axis=axis, keepdims=True) + eps) * w64
    xc = x64 - x64.mean(axis=axis, keepdims=True)
    f64_ln = xc / np.sqrt(np.mean(xc * xc, axis=axis, keepdims=True) + eps) * w64 + b64
    tol = dict(rtol=2e-5, atol=2e-5)
    wd, bd = dev(w), dev(beta)
    for mk in (col_major, dev):
        xd = mk(x)
        out = torch.zeros_like(xd)
        gpu.rms_norm(xd, wd, eps, out, axis)
        np.testing.assert_allclose(out.cpu().numpy(), want_rms, **tol)
        np.testing.assert_allclose(out.cpu().numpy(), f64_rms, **tol)
        out2 = torch.zeros_like(xd)
        gpu.layer_norm(xd, wd, bd, eps, out2, axis)
        np.testing.assert_allclose(out2.cpu().numpy(), want_ln, **tol)
        np.testing.assert_allclose(out2.cpu().numpy(), f64_ln, **tol)
        # in place (the modules never do, the entry points allow it)
        gpu.rms_norm(xd, wd, eps, xd, axis)
        np.testing.assert_array_equal(xd.cpu().numpy(), out.cpu().numpy())
    # a strided weight: every second element of a longer vector
    w2 = dev(np.repeat(w, 2))[::2]
    xd = col_major(x)
    out = torch.zeros_like(xd)
    gpu.rms_norm(xd, w2, eps, out, axis)
    np.testing.assert_allclose(out.cpu().numpy(), want_rms, **tol)
