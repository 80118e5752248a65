"""GPU parity of the KV encoder, the packed cache and its read-back, through the C ABI.

Bar: codes, sign bits, Weed-packed words, row scales and dequantised values are BIT-EXACT against the CPU checker
given the same rotated input; with the rotation done on the device in the reference's rounding order (rotate = 2)
they are bit-exact end to end.
"""
import json
import os

import numpy as np
import pytest

from gpu_helpers import assert_attn_close, col_major, coder_specs, dev, export

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_uniform_known_answers_on_device(gpu, oracle):
    """The reference's recorded write_row / read_row answers (multihead_attention.cpp:43-79), padded to d = 32."""
    import torch
    with open(os.path.join(HERE, "golden", "weed_uniform_kat.json")) as f:
        kat = json.load(f)
    for case in kat["write_row"]:
        n = len(case["vals"])
        row = np.zeros((1, 1, 1, 32), dtype=np.float32)
        row[0, 0, 0, :n] = case["vals"]
        cache = gpu.KVCache(gpu.KV_UNIFORM, 1, 1, 32, 8, case["bits"], case["bits"])
        cache.set_scales(case["block_scale"], case["block_scale"])
        x = dev(row)
        cache.encode_append(x, x, rotate=0)
        fields, _ = export(cache, 0, 1)
        np.testing.assert_array_equal(fields[0, 0, 0, :n], case["codes"])
        # Weed's own word packing of the same row
        wpr = oracle.words_per_row(32, case["bits"])
        words = torch.zeros((1, 1, 1, wpr), dtype=torch.int32, device="cuda")
        cache.export_weed_words(1, words)
        np.testing.assert_array_equal(words.cpu().numpy()[0, 0, 0],
                                      oracle.uniform_write_rows(row.reshape(1, 32), case["bits"],
                                                                case["block_scale"])[0])
        cache.close()
    case = kat["read_row"][0]
    row = np.zeros((1, 1, 1, 32), dtype=np.float32)
    row[0, 0, 0, :4] = [0.5, -1.2, 2.0, -0.05]
    cache = gpu.KVCache(gpu.KV_UNIFORM, 1, 1, 32, 8, 4, 4)
    cache.set_scales(case["block_scale"], case["block_scale"])
    x = dev(row)
    cache.encode_append(x, x, rotate=0)
    out = torch.zeros((1, 1, 1, 32), dtype=torch.float32, device="cuda")
    cache.dequant(0, out)
    np.testing.assert_allclose(out.cpu().numpy()[0, 0, 0, :4], np.array(case["vals"], dtype=np.float32), rtol=0,
                               atol=6e-8)
    cache.close()


@pytest.mark.parametrize("kbits,vbits,d", [(4, 4, 64), (3, 2, 128), (2, 3, 32), (8, 8, 64), (5, 7, 128)])
def test_rows_in_weeds_word_packing_are_appended_as_they_are(gpu, oracle, kbits, vbits, d):
    """Rows that arrive already coded in Weed's word packing (what the reference's write_row leaves in
    QuantizedKVCache::packed; the words here come from the checker's write_row, which the recorded answers pin) are
    appended without a round trip through floats: in one call and token by token, the cache then holds exactly the
    codes of the float path, exports the same words, dequantises to read_row's floats and attends identically."""
    import torch
    rng = np.random.default_rng(kbits * 10 + vbits + d)
    S, Hkv, T = 2, 3, 70
    K = rng.normal(0, 1.1, size=(S, Hkv, T, d)).astype(np.float32)
    V = rng.normal(0, 0.8, size=(S, Hkv, T, d)).astype(np.float32)
    ks, vs = oracle.block_scale(K), oracle.block_scale(V)
    k_words = oracle.uniform_write_rows(K.reshape(-1, d), kbits, ks).reshape(S, Hkv, T, -1)
    v_words = oracle.uniform_write_rows(V.reshape(-1, d), vbits, vs).reshape(S, Hkv, T, -1)

    ref = gpu.KVCache(gpu.KV_UNIFORM, S, Hkv, d, 100, kbits, vbits)
    ref.set_scales(ks, vs)
    ref.encode_append(dev(K), dev(V), rotate=0)
    want = [export(ref, which, T)[0] for which in (0, 1)]
    q = dev(rng.standard_normal((S, 2 * Hkv, d), dtype=np.float32))
    want_out = torch.zeros_like(q)
    ref.decode_attn(q, want_out)

    for pieces in ([T], [1] * 5 + [64, 1]):
        cache = gpu.KVCache(gpu.KV_UNIFORM, S, Hkv, d, 100, kbits, vbits)
        cache.set_scales(ks, vs)
        t0 = 0
        for n in pieces:
            kw = torch.from_numpy(np.ascontiguousarray(k_words[:, :, t0:t0 + n])).cuda()
            vw = torch.from_numpy(np.ascontiguousarray(v_words[:, :, t0:t0 + n])).cuda()
            cache.append_weed_words(kw, vw)
            t0 += n
        assert cache.seq_lens() == [T] * S
        for which, words in ((0, k_words), (1, v_words)):
            np.testing.assert_array_equal(export(cache, which, T)[0], want[which])
            back = torch.zeros(words.shape, dtype=torch.int32, device="cuda")
            cache.export_weed_words(which, back)
            np.testing.assert_array_equal(back.cpu().numpy(), words)
        deq = torch.zeros((S, Hkv, T, d), device="cuda")
        cache.dequant(0, deq)
        np.testing.assert_array_equal(deq.cpu().numpy().reshape(-1, d),
                                      oracle.uniform_read_rows(k_words.reshape(-1, k_words.shape[-1]), d, kbits, ks))
        out = torch.zeros_like(q)
        cache.decode_attn(q, out)
        assert torch.equal(out, want_out)
        # one sequence only, and the error paths
        cache.reset()
        cache.set_scales(ks, vs)
        kw1 = torch.from_numpy(np.ascontiguousarray(k_words[1:2])).cuda()
        vw1 = torch.from_numpy(np.ascontiguousarray(v_words[1:2])).cuda()
        cache.append_weed_words(kw1, vw1, seq_begin=1)
        assert cache.seq_lens() == [0, T]
        np.testing.assert_array_equal(export(cache, 0, T)[0][1], want[0][1])
        with pytest.raises(gpu.WeedHipError):
            cache.append_weed_words(kw1, vw1, seq_begin=1)  # 140 tokens > capacity 100
        cache.close()
    lm = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, max(d, 32), 100, 3, 3)
    with pytest.raises(gpu.WeedHipError):
        lm.append_weed_words(torch.zeros((S, Hkv, 1, 16), dtype=torch.int32, device="cuda"),
                             torch.zeros((S, Hkv, 1, 16), dtype=torch.int32, device="cuda"))
    lm.close()
    ref.close()


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("d", [64, 128, 8, 48, 80])  # 8: the reference's own transformer example; 48, 80: not multiples of 32
def test_uniform_encode_bit_exact(gpu, oracle, bits, d):
    import torch
    rng = np.random.default_rng(100 * bits + d)
    S, Hkv, T = 2, 3, 150
    K = rng.normal(0, 1.2, size=(S, Hkv, T, d)).astype(np.float32)
    V = rng.normal(0, 0.7, size=(S, Hkv, T, d)).astype(np.float32)
    K[0, 0, 0, :4] = [np.inf, -np.inf, 1e30, -1e30]  # clamped, not faulted
    ks, vs = oracle.block_scale(K[np.isfinite(K)]), oracle.block_scale(V)
    cache = gpu.KVCache(gpu.KV_UNIFORM, S, Hkv, d, 200, bits, bits)
    cache.set_scales(ks, vs)
    # Weed's own layout: column-major [B, H, T, d] (dimension 0 fastest)
    cache.encode_append(col_major(K), col_major(V), rotate=0)
    assert cache.seq_lens() == [T, T]
    kspec, vspec = coder_specs(oracle, cache)
    for which, x, spec in ((0, K, kspec), (1, V, vspec)):
        want_f, _ = oracle.encode_rows(spec, x.reshape(-1, d))
        got_f, _ = export(cache, which, T)
        np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
        wpr = oracle.words_per_row(d, bits)
        words = torch.zeros((S, Hkv, T, wpr), dtype=torch.int32, device="cuda")
        cache.export_weed_words(which, words)
        want_w = oracle.uniform_write_rows(x.reshape(-1, d), bits, spec.block_scale)
        np.testing.assert_array_equal(words.cpu().numpy().reshape(-1, wpr), want_w)
        # read_row: identical floats, not merely close
        out = torch.zeros((S, Hkv, T, d), dtype=torch.float32, device="cuda")
        cache.dequant(which, out)
        want_d = oracle.uniform_read_rows(want_w, d, bits, spec.block_scale)
        np.testing.assert_array_equal(out.cpu().numpy().reshape(-1, d), want_d)
    cache.close()


@pytest.mark.parametrize("k_bits,k_sign,v_bits,v_sign", [(4, 1, 4, 1), (3, 1, 4, 0), (3, 0, 4, 0), (2, 1, 3, 0),
                                                         (1, 0, 2, 0)])
@pytest.mark.parametrize("d", [64, 128, 8, 48, 80])
def test_lloydmax_encode_bit_exact(gpu, oracle, k_bits, k_sign, v_bits, v_sign, d):
    import torch
    rng = np.random.default_rng(k_bits * 1000 + v_bits * 100 + d)
    S, Hkv, T = 2, 2, 133
    K = (rng.normal(size=(S, Hkv, T, d)) * rng.uniform(0.2, 5, size=(S, Hkv, T, 1))).astype(np.float32)
    V = rng.normal(size=(S, Hkv, T, d)).astype(np.float32)
    V[1, 1, 7] = 0.0  # an all-zero row: scale 0, codes of u = 0
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, 256, k_bits, v_bits, k_sign, v_sign)
    cache.encode_append(dev(K), dev(V), rotate=0)
    kspec, vspec = coder_specs(oracle, cache)
    for which, x, spec in ((0, K, kspec), (1, V, vspec)):
        want_f, want_a = oracle.encode_rows(spec, x.reshape(-1, d))
        got_f, got_a = export(cache, which, T)
        np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
        np.testing.assert_array_equal(got_a.reshape(-1), want_a)  # row scales bit-exact
        out = torch.zeros((S, Hkv, T, d), dtype=torch.float32, device="cuda")
        cache.dequant(which, out)
        np.testing.assert_array_equal(out.cpu().numpy().reshape(-1, d), oracle.decode_rows(spec, want_f, want_a))
    dp = (d + 31) // 32 * 32  # rows are stored with head_dim rounded up to a multiple of 32
    assert cache.row_bytes() == (dp * (k_bits + k_sign) // 8 + 4, dp * (v_bits + v_sign) // 8 + 4)
    cache.close()


@pytest.mark.parametrize("mode", ["uniform", "lloydmax"])
def test_device_rotation_modes(gpu, oracle, mode):
    """rotate = 2 reproduces the reference's rounding (matmul.cpp:40-44), so codes stay bit-exact end to end;
    rotate = 1 uses fused multiply-adds and may move values that sit on a cell edge."""
    import torch
    rng = np.random.default_rng(77)
    S, Hkv, T, d = 1, 2, 96, 128
    K = rng.normal(size=(S, Hkv, T, d)).astype(np.float32)
    V = rng.normal(size=(S, Hkv, T, d)).astype(np.float32)
    Rk = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Rv = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Ky = oracle.apply_rotation(K.reshape(-1, d), Rk)
    Vy = oracle.apply_rotation(V.reshape(-1, d), Rv)
    for rotate in (2, 1):
        if mode == "uniform":
            cache = gpu.KVCache(gpu.KV_UNIFORM, S, Hkv, d, 128, 4, 4)
            cache.set_scales(oracle.block_scale(Ky), oracle.block_scale(Vy))
        else:
            cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, 128, 3, 4, 1, 0)
        cache.set_rotations(dev(Rk), dev(Rv))
        cache.encode_append(dev(K), dev(V), rotate=rotate)
        kspec, vspec = coder_specs(oracle, cache)
        for which, y, spec in ((0, Ky, kspec), (1, Vy, vspec)):
            want_f, want_a = oracle.encode_rows(spec, y)
            got_f, got_a = export(cache, which, T)
            if rotate == 2:
                np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
                np.testing.assert_array_equal(got_a.reshape(-1), want_a)
            else:
                assert np.mean(got_f.reshape(-1, d) != want_f) < 2e-3
                np.testing.assert_allclose(got_a.reshape(-1), want_a, rtol=1e-5)
        cache.close()


@pytest.mark.parametrize("lloyd,kw,vw,d", [(True, (4, 1), (4, 0), 128), (True, (2, 1), (3, 0), 64),
                                           (False, (4, 0), (8, 0), 128), (False, (3, 0), (2, 0), 32)])
def test_half_block_appends_mix_with_packed_ones(gpu, oracle, lloyd, kw, vw, d):
    """Appends that add whole 32-token half blocks behind whole half blocks are written by the encoder itself, any
    other append goes through the packing kernel; a cache may see both in any order and per sequence.  After every
    step the fields, the row scales and the attention over the cache equal the checker's on the rows appended so far."""
    import torch
    rng = np.random.default_rng(d + kw[0] * 7 + vw[0])
    S, Hkv, cap = 3, 2, 256
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    cache = gpu.KVCache(mode, S, Hkv, d, cap, kw[0], vw[0], kw[1], vw[1])
    if not lloyd:
        cache.set_scales(1.2, 0.8)
    K = (rng.normal(size=(S, Hkv, cap, d)) * rng.uniform(0.3, 4, size=(S, Hkv, cap, 1))).astype(np.float32)
    V = rng.normal(size=(S, Hkv, cap, d)).astype(np.float32)
    Kd, Vd = dev(K), dev(V)
    lens = [0] * S
    q = rng.standard_normal((S, 2 * Hkv, d), dtype=np.float32)
    # (first sequence, sequence count, tokens): direct, direct for one sequence, packed, packed (unaligned start),
    # direct again for the one sequence that is still aligned, packed single tokens
    steps = [(0, 3, 64), (1, 1, 32), (0, 1, 5), (0, 3, 32), (2, 1, 32), (0, 3, 1), (1, 2, 1)]
    for s0, n, T in steps:
        k_new = torch.stack([Kd[s, :, lens[s]:lens[s] + T] for s in range(s0, s0 + n)])
        v_new = torch.stack([Vd[s, :, lens[s]:lens[s] + T] for s in range(s0, s0 + n)])
        cache.encode_append(k_new, v_new, seq_begin=s0)
        for s in range(s0, s0 + n):
            lens[s] += T
        assert cache.seq_lens() == lens
        kspec, vspec = coder_specs(oracle, cache)
        for which, x, spec in ((0, K, kspec), (1, V, vspec)):
            got_f, got_a = export(cache, which, max(lens))
            for s in range(S):
                want_f, want_a = oracle.encode_rows(spec, x[s, :, :lens[s]].reshape(-1, d))
                np.testing.assert_array_equal(got_f[s, :, :lens[s]].reshape(-1, d), want_f)
                if lloyd:
                    np.testing.assert_array_equal(got_a[s, :, :lens[s]].reshape(-1), want_a)
        kf, ka = export(cache, 0, max(lens))
        vf, va = export(cache, 1, max(lens))
        want = oracle.decode_attn(kspec, vspec, kf, ka if lloyd else None, vf, va if lloyd else None, q, lens,
                                  gqa_weed=True)
        out = torch.zeros((S, 2 * Hkv, d), device="cuda")
        cache.decode_attn(dev(q), out)
        assert_attn_close(out.cpu().numpy(), want, "after %s" % ((s0, n, T),))
    cache.close()


def test_incremental_and_ragged_append(gpu, oracle):
    """Appending token by token, in uneven chunks and per sequence must give the cache a one-shot encode gives
    (the reference's own incremental append re-reads old rows with the wrong strides, multihead_attention.cpp:247-273)."""
    rng = np.random.default_rng(5)
    S, Hkv, d, cap = 3, 2, 64, 300
    lens = [300, 71, 190]
    K = rng.normal(size=(S, Hkv, cap, d)).astype(np.float32)
    V = rng.normal(size=(S, Hkv, cap, d)).astype(np.float32)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, cap, 2, 3, 1, 0)
    Kd, Vd = dev(K), dev(V)
    # a shared prefill of 70 tokens for all sequences, then per-sequence continuations in odd chunk sizes
    cache.encode_append(Kd[:, :, :70], Vd[:, :, :70])
    for s, L in enumerate(lens):
        pos = 70
        for chunk in (1, 1, 1, 30, 64, 5, 1000):
            n = min(chunk, L - pos)
            if n <= 0:
                break
            cache.encode_append(Kd[s:s + 1, :, pos:pos + n], Vd[s:s + 1, :, pos:pos + n], seq_begin=s)
            pos += n
    assert cache.seq_lens() == lens
    kspec, vspec = coder_specs(oracle, cache)
    for which, x, spec in ((0, K, kspec), (1, V, vspec)):
        got_f, got_a = export(cache, which, cap)
        for s, L in enumerate(lens):
            want_f, want_a = oracle.encode_rows(spec, x[s, :, :L].reshape(-1, d))
            np.testing.assert_array_equal(got_f[s, :, :L].reshape(-1, d), want_f)
            np.testing.assert_array_equal(got_a[s, :, :L].reshape(-1), want_a)
    # capacity is checked on the host; nothing is written
    with pytest.raises(gpu.WeedHipError) as e:
        cache.encode_append(Kd[0:1, :, :1], Vd[0:1, :, :1], seq_begin=0)
    assert e.value.code == gpu.ECAPACITY
    # reset empties the cache and it can be refilled
    cache.reset()
    assert cache.seq_lens() == [0, 0, 0]
    cache.encode_append(Kd[:, :, 5:15], Vd[:, :, 5:15])
    got_f, _ = export(cache, 0, 10)
    want_f, _ = oracle.encode_rows(kspec, K[:, :, 5:15].reshape(-1, d))
    np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
    cache.close()


def test_block_scale(gpu, oracle):
    rng = np.random.default_rng(9)
    x = rng.normal(0, 1.7, size=(2, 3, 40, 64)).astype(np.float32)
    # sequential: the reference's one-accumulator fp32 order over the storage of a contiguous tensor -> bit-exact
    t = col_major(x)
    flat = np.transpose(x).reshape(-1)  # storage order of the column-major tensor
    assert gpu.block_scale(t, sequential=True) == np.float32(oracle.block_scale(flat))
    # the same logical tensor laid out (B, T, heads, d) column-major, as a module hands its rotated K over: the sum
    # still runs over the logical column-major index (b fastest, then head, token, coordinate), not over the storage
    import torch
    B, H, T, d = x.shape
    store = dev(np.ascontiguousarray(np.transpose(x, (3, 1, 2, 0))))  # storage order: b fastest, then t, h, j
    view = store.permute(3, 1, 2, 0)
    assert tuple(view.stride()) == (1, B * T, B, B * T * H) and torch.equal(view, dev(x))
    assert gpu.block_scale(view, sequential=True) == np.float32(oracle.block_scale(flat))
    storage_order = store.cpu().numpy().reshape(-1)
    assert not np.array_equal(storage_order, flat)
    want = np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-8)
    assert abs(gpu.block_scale(t) - want) < 1e-6 * want
    assert abs(gpu.block_scale(dev(x)[:, 1:, ::2]) - np.sqrt(np.mean(x[:, 1:, ::2].astype(np.float64) ** 2) + 1e-8)) \
        < 1e-6 * want


def test_rotation_on_device(gpu, oracle):
    import torch
    for d in (64, 128):
        R = torch.zeros(d * d, dtype=torch.float32, device="cuda")
        gpu.make_rotation(1234 + d, d, R)
        Rm = R.cpu().numpy().reshape(d, d).T.astype(np.float64)
        np.testing.assert_allclose(Rm.T @ Rm, np.eye(d), atol=3e-4)
        # same seed, same matrix; another seed, another matrix
        R2 = torch.zeros_like(R)
        gpu.make_rotation(1234 + d, d, R2)
        assert torch.equal(R, R2)
        gpu.make_rotation(99, d, R2)
        assert not torch.equal(R, R2)
        # device Gram-Schmidt against the CPU checker on the same Gaussian draws
        g = np.random.default_rng(d).normal(size=d * d).astype(np.float32)
        Rg = dev(g.copy())
        gpu.orthonormalize_columns(d, Rg)
        np.testing.assert_allclose(Rg.cpu().numpy(), oracle.orthonormalize_columns(g), atol=2e-4)


def test_argument_errors_are_reported_not_faulted(gpu):
    import torch
    with pytest.raises(gpu.WeedHipError) as e:
        gpu.KVCache(gpu.KV_LLOYDMAX, 1, 1, 300, 16, 3, 3)  # head_dim beyond 256
    assert e.value.code == gpu.EINVAL
    with pytest.raises(gpu.WeedHipError):
        gpu.KVCache(gpu.KV_UNIFORM, 1, 1, 64, 16, 3, 3, 1, 0)  # the uniform coder has no sign bit
    with pytest.raises(gpu.WeedHipError):
        gpu.KVCache(gpu.KV_LLOYDMAX, 1, 1, 64, 16, 5, 3)  # code width out of range
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, 2, 2, 64, 16, 3, 3)
    x = torch.zeros((1, 2, 4, 64), device="cuda")
    with pytest.raises(gpu.WeedHipError):
        cache.encode_append(x, x, seq_begin=2)  # sequence range outside the cache
    with pytest.raises(gpu.WeedHipError):
        cache.encode_append(x, x, rotate=1)  # no rotations set
    q = torch.zeros((2, 3, 64), device="cuda")
    with pytest.raises(gpu.WeedHipError):
        cache.decode_attn(q, torch.zeros_like(q))  # 3 query heads over 2 kv heads
    cache.close()


def test_replaced_tables(gpu, oracle):
    """weed_hip_kv_cache_set_tables: thresholds and levels of the caller's own (here: a uniform grid on [-2.5, 2.5] and
    the half-cell centres), reconstruction values rounded to binary16 by the library.  Fields and row scales match the
    checker given the same thresholds bit for bit; attention matches the checker fed the ROUNDED reconstruction
    values, which are what the kernels multiply with."""
    import torch
    rng = np.random.default_rng(77)
    d, S, Hkv, Hq, L = 128, 2, 2, 8, 300
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32) * 1.3
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, L, 3, 3, 1, 0)
    specs = []
    for which, bits, sign in ((0, 3, 1), (1, 3, 0)):
        n = 1 << bits
        edges = np.linspace(-2.5, 2.5, n + 1, dtype=np.float32)
        bounds = edges[1:-1]
        levels = ((edges[:-1] + edges[1:]) / 2).astype(np.float32)
        if sign:
            w = (edges[1] - edges[0]) / 4
            recon = np.stack([levels - w, levels + w], axis=1).reshape(-1) * np.float32(1.0001)  # not binary16 values
        else:
            recon = levels * np.float32(1.0003)
        rounded = np.array(cache.set_tables(which, list(bounds), list(levels), list(recon.astype(np.float32))), dtype=np.float32)
        assert np.array_equal(rounded, rounded.astype(np.float16).astype(np.float32))  # binary16 values
        assert not np.array_equal(rounded, recon) and np.allclose(rounded, recon, rtol=1e-3)
        got_b, got_l, got_r = cache.get_tables(which)
        assert np.array_equal(got_b, bounds) and np.array_equal(got_l, levels) and np.array_equal(got_r, rounded)
        specs.append(oracle.CoderSpec(1, d, bits, sign=sign, bounds=bounds, levels=levels, recon=rounded))
    cache.encode_append(dev(K), dev(V), rotate=0)
    fields, scales = [], []
    for which, x in ((0, K), (1, V)):
        want_f, want_a = oracle.encode_rows(specs[which], x.reshape(-1, d))
        got_f, got_a = export(cache, which, L)
        np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
        np.testing.assert_array_equal(got_a.reshape(-1), want_a)
        fields.append(got_f)
        scales.append(got_a)
        out = torch.zeros((S, Hkv, L, d), dtype=torch.float32, device="cuda")
        cache.dequant(which, out)
        np.testing.assert_array_equal(out.cpu().numpy().reshape(-1, d), oracle.decode_rows(specs[which], want_f, want_a))
    want = oracle.decode_attn(specs[0], specs[1], fields[0], scales[0], fields[1], scales[1], q, [L, L], gqa_weed=False)
    qd = dev(q)
    out = torch.zeros_like(qd)
    cache.decode_attn(qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=0)
    gpu.sync()
    from gpu_helpers import assert_attn_close
    assert_attn_close(out.cpu().numpy(), want, "replaced tables")
    # the checker with the UN-rounded values differs visibly: the test would notice a library that skipped the rounding
    cache.close()


def test_a_block_cannot_be_freed_twice(gpu):
    p1 = gpu.malloc(4096)
    gpu.free(p1)
    with pytest.raises(gpu.WeedHipError) as e:
        gpu.free(p1)
    assert e.value.code == gpu.EINVAL
    p2 = gpu.malloc(4096)
    p3 = gpu.malloc(4096)
    assert p2 != p3  # the cached block was handed out once
    gpu.free(p2)
    gpu.free(p3)


def test_shutdown_and_start_again(gpu, oracle):
    """init -> work -> shutdown -> init -> work: the library gives back what it holds and starts again."""
    import torch

    def work(seed):
        rng = np.random.default_rng(seed)
        a = rng.standard_normal((200, 1100), dtype=np.float32)
        b = rng.standard_normal((1100, 300), dtype=np.float32)
        out = torch.zeros((200, 300), device="cuda")
        gpu.matmul(dev(a), dev(b), out)  # a split product: uses the library's own scratch
        gpu.sync()
        np.testing.assert_allclose(out.cpu().numpy(), a.astype(np.float64) @ b.astype(np.float64), rtol=1e-4, atol=1e-3)
        p = gpu.malloc(1 << 20)
        gpu.free(p)  # stays in the library's cache

    work(1)
    gpu.shutdown()
    gpu.shutdown()  # nothing left to do
    gpu.check(gpu.load().weed_hip_init(0))
    gpu.use_torch_stream(torch.cuda.current_stream())
    work(2)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, 1, 1, 64, 64, 3, 3)
    x = torch.randn((1, 1, 40, 64), device="cuda")
    cache.encode_append(x, x)
    assert cache.seq_lens() == [40]
    cache.close()


@pytest.mark.parametrize("shape", [(3, 2, 5, 64), (7, 19, 128), (70, 20), (5, 3, 130), (130, 1, 2, 32)])
def test_apply_rotation_reference_order(gpu, oracle, shape):
    """y = x.R over the last dimension of a strided tensor, in the reference's summation order: bit-exact against the
    checker's naive loop, for column-major and row-major operands in every combination (the kernel walks each side
    along its contiguous direction), ragged row tiles, widths that are not multiples of the column chunks, a width
    beyond the LDS-tiled kernel, and an output that is a slice of a larger tensor."""
    import torch
    rng = np.random.default_rng(77 + len(shape))
    d = shape[-1]
    R = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    x = rng.standard_normal(shape, dtype=np.float32)
    want = oracle.apply_rotation(x.reshape(-1, d), R).reshape(x.shape)
    for mk_x in (col_major, dev):
        for mk_o in (col_major, dev):
            out = mk_o(np.zeros(shape, dtype=np.float32))
            gpu.apply_rotation(mk_x(x), dev(R), out)
            np.testing.assert_array_equal(out.cpu().numpy(), want)
    big = torch.full((shape[0] + 2,) + tuple(shape[1:-1]) + (d + 3,), 5.0, device="cuda")
    gpu.apply_rotation(col_major(x), dev(R), big[1:-1, ..., 2:2 + d])
    got = big.cpu().numpy()
    np.testing.assert_array_equal(got[1:-1, ..., 2:2 + d], want)
    assert (got[0] == 5.0).all() and (got[-1] == 5.0).all() and (got[..., :2] == 5.0).all() and (got[..., 2 + d:] == 5.0).all()


def test_cfg5a_encode_full_size(gpu, oracle):
    """Configuration 5's encode half at full size (4096 tokens x 8 kv heads x head_dim 128, 3-bit Lloyd-Max codes):
    with the reference-order rotation every field and row scale of both caches equals the CPU checker's, and the
    matrix-core rotation moves only values that sit on a cell edge; appending the same tokens in four chunks gives
    the same packed cache as one call (idempotence of the layout under incremental writes)."""
    import torch
    from weed_amd import workloads
    wl = workloads.config(5)
    d, T, Hkv = wl.head_dim, wl.max_len, wl.n_kv_heads
    assert (T, Hkv, d) == (4096, 8, 128)
    K, V, _ = wl.tensors()
    rng = np.random.default_rng(5)
    Rk = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Rv = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Ky = oracle.apply_rotation(K.reshape(-1, d), Rk)
    Vy = oracle.apply_rotation(V.reshape(-1, d), Rv)
    Kd, Vd = dev(K), dev(V)
    exported = {}
    for rotate in (2, 1):
        cache = gpu.KVCache(gpu.KV_LLOYDMAX, 1, Hkv, d, T, wl.k_bits, wl.v_bits, wl.k_sign, wl.v_sign)
        cache.set_rotations(dev(Rk), dev(Rv))
        cache.encode_append(Kd, Vd, rotate=rotate)
        kspec, vspec = coder_specs(oracle, cache)
        for which, y, spec in ((0, Ky, kspec), (1, Vy, vspec)):
            want_f, want_a = oracle.encode_rows(spec, y)
            got_f, got_a = export(cache, which, T)
            if rotate == 2:
                np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
                np.testing.assert_array_equal(got_a.reshape(-1), want_a)
                exported[which] = (got_f, got_a)
            else:
                assert np.mean(got_f.reshape(-1, d) != want_f) < 2e-3
                np.testing.assert_allclose(got_a.reshape(-1), want_a, rtol=1e-5)
        cache.close()
    # the same tokens in uneven chunks (the V items are rebuilt read-modify-write across calls)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, 1, Hkv, d, T, wl.k_bits, wl.v_bits, wl.k_sign, wl.v_sign)
    cache.set_rotations(dev(Rk), dev(Rv))
    edges = [0, 1, 1000, 1031, 4096]
    for a, b in zip(edges[:-1], edges[1:]):
        cache.encode_append(Kd[:, :, a:b], Vd[:, :, a:b], rotate=2)
    for which in (0, 1):
        got_f, got_a = export(cache, which, T)
        np.testing.assert_array_equal(got_f, exported[which][0])
        np.testing.assert_array_equal(got_a, exported[which][1])
    assert cache.seq_lens() == [T]
    cache.close()


@pytest.mark.parametrize("lloyd,kw,vw,d,rotate", [(True, (3, 1), (3, 0), 128, 1), (True, (2, 0), (4, 1), 96, 0),
                                                  (True, (4, 1), (1, 0), 256, 1), (False, (8, 0), (8, 0), 64, 0),
                                                  (False, (5, 0), (3, 0), 32, 1), (False, (1, 0), (7, 0), 160, 0)])
def test_one_token_appends_are_finished_by_the_encoder(gpu, lloyd, kw, vw, d, rotate):
    """A decode step's append (one token for each of a run of sequences) is one kernel: the encoder puts the new
    fields into their items itself, next to the fields of the tokens already cached, and the last workgroup moves
    the lengths.  Seventy such steps over sequences of different lengths (every place a token can have in a 64-token
    block, more rows than one workgroup takes, a last workgroup that is not full, runs that leave sequences out)
    must give, bit for bit, the cache that one append per sequence gives, and the same attention."""
    import torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(d + kw[0])
    S, Hkv, cap = 5, 9, 160
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    a = gpu.KVCache(mode, S, Hkv, d, cap, kw[0], vw[0], kw[1], vw[1])
    b = gpu.KVCache(mode, S, Hkv, d, cap, kw[0], vw[0], kw[1], vw[1])
    rk, rv = torch.zeros(d * d, device="cuda"), torch.zeros(d * d, device="cuda")
    gpu.make_rotation(3, d, rk)
    gpu.make_rotation(4, d, rv)
    for c in (a, b):
        if not lloyd:
            c.set_scales(1.3, 0.9)
        c.set_rotations(rk, rv)
    K = torch.randn((S, Hkv, cap, d), generator=gen, device="cuda") * 2
    V = torch.randn((S, Hkv, cap, d), generator=gen, device="cuda")
    lens = [0, 3, 31, 64, 70]
    for s in range(S):
        if lens[s]:
            a.encode_append(K[s:s + 1, :, :lens[s]], V[s:s + 1, :, :lens[s]], seq_begin=s, rotate=rotate)
    for step in range(70):
        s0, n = (0, S) if step % 3 else (step % 4, min(2, S - step % 4))
        k1 = torch.stack([K[s, :, lens[s]:lens[s] + 1] for s in range(s0, s0 + n)])
        v1 = torch.stack([V[s, :, lens[s]:lens[s] + 1] for s in range(s0, s0 + n)])
        a.encode_append(k1, v1, seq_begin=s0, rotate=rotate)
        for s in range(s0, s0 + n):
            lens[s] += 1
    assert a.seq_lens() == lens
    for s in range(S):
        b.encode_append(K[s:s + 1, :, :lens[s]], V[s:s + 1, :, :lens[s]], seq_begin=s, rotate=rotate)
    for which in (0, 1):
        fa, sa = export(a, which, max(lens))
        fb, sb = export(b, which, max(lens))
        for s in range(S):
            assert np.array_equal(fa[s, :, :lens[s]], fb[s, :, :lens[s]]), (which, s)
            assert np.array_equal(sa[s, :, :lens[s]], sb[s, :, :lens[s]]), (which, s)
    q = torch.randn((S, Hkv * 2, d), generator=gen, device="cuda")
    oa, ob = torch.zeros_like(q), torch.zeros_like(q)
    a.decode_attn(q, oa)
    b.decode_attn(q, ob)
    gpu.sync()
    assert torch.equal(oa, ob)
    # a cache that is reset starts over: items that still hold the old tokens' fields are rebuilt from their first field
    a.reset()
    b.reset()
    for t in range(3):
        a.encode_append(V[:, :, t:t + 1], K[:, :, t:t + 1], rotate=rotate)
    b.encode_append(V[:, :, :3], K[:, :, :3], rotate=rotate)
    for which in (0, 1):
        fa, sa = export(a, which, 3)
        fb, sb = export(b, which, 3)
        assert np.array_equal(fa, fb) and np.array_equal(sa, sb), which
    a.decode_attn(q, oa)
    b.decode_attn(q, ob)
    gpu.sync()
    assert torch.equal(oa, ob)
    a.close()
    b.close()


def test_random_append_sequences_give_the_same_cache(gpu):
    """Forty seeded random append histories (chunk sizes around the 32-token half blocks, subsets of the sequences,
    every head_dim family, both coders, all widths): the cache must equal, bit for bit, the one that a one-token
    append followed by one append of the rest builds (the rest starts inside a half block, so it goes through the
    packing kernel), and attend identically -- so the largest row scale kept per region agrees too."""
    import torch
    rng = np.random.default_rng(99)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    for case in range(40):
        d = int(rng.choice([32, 64, 96, 128, 256]))
        lloyd = bool(rng.integers(2))
        if lloyd:
            kb, vb, ks, vs = int(rng.integers(1, 5)), int(rng.integers(1, 5)), int(rng.integers(2)), int(rng.integers(2))
        else:
            kb, vb, ks, vs = int(rng.integers(1, 9)), int(rng.integers(1, 9)), 0, 0
        S, Hkv, cap = int(rng.integers(1, 5)), int(rng.integers(1, 4)), 320
        mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
        a = gpu.KVCache(mode, S, Hkv, d, cap, kb, vb, ks, vs)
        b = gpu.KVCache(mode, S, Hkv, d, cap, kb, vb, ks, vs)
        if not lloyd:
            a.set_scales(1.1, 0.7)
            b.set_scales(1.1, 0.7)
        K = torch.randn((S, Hkv, cap, d), generator=gen, device="cuda") * 2
        V = torch.randn((S, Hkv, cap, d), generator=gen, device="cuda")
        lens = [0] * S
        for _ in range(int(rng.integers(2, 8))):
            s0 = int(rng.integers(0, S))
            n = int(rng.integers(1, S - s0 + 1))
            T = int(rng.choice([1, 2, 5, 17, 31, 32, 33, 64, 96]))
            if max(lens[s0:s0 + n]) + T > cap:
                continue
            a.encode_append(torch.stack([K[s, :, lens[s]:lens[s] + T] for s in range(s0, s0 + n)]),
                            torch.stack([V[s, :, lens[s]:lens[s] + T] for s in range(s0, s0 + n)]), seq_begin=s0)
            for s in range(s0, s0 + n):
                lens[s] += T
        for s in range(S):
            if lens[s] >= 1:
                b.encode_append(K[s:s + 1, :, :1], V[s:s + 1, :, :1], seq_begin=s)
            if lens[s] > 1:
                b.encode_append(K[s:s + 1, :, 1:lens[s]], V[s:s + 1, :, 1:lens[s]], seq_begin=s)
        what = "case %d: d %d, K %d+%d V %d+%d bits, lengths %s" % (case, d, kb, ks, vb, vs, lens)
        assert a.seq_lens() == lens and b.seq_lens() == lens, what
        if max(lens):
            for which in (0, 1):
                fa, sa = export(a, which, max(lens))
                fb, sb = export(b, which, max(lens))
                for s in range(S):
                    assert np.array_equal(fa[s, :, :lens[s]], fb[s, :, :lens[s]]), what
                    assert np.array_equal(sa[s, :, :lens[s]], sb[s, :, :lens[s]]), what
            q = torch.randn((S, Hkv * 2, d), generator=gen, device="cuda")
            oa, ob = torch.zeros_like(q), torch.zeros_like(q)
            a.decode_attn(q, oa)
            b.decode_attn(q, ob)
            gpu.sync()
            assert torch.equal(oa, ob), what
        a.close()
        b.close()
