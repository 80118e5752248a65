"""GPU parity of fused decode attention over the packed cache, through the C ABI.

Bar (fp32): |gpu - checker| <= 1e-4 + 1e-3 * |checker| per output element, where the checker is the CPU restatement
of the reference's path run on the same codes.  Full-size configurations that the scalar checker cannot finish in
seconds are covered by size-independent properties.
"""
import numpy as np
import pytest

from gpu_helpers import assert_attn_close, col_major, coder_specs, dev, export
from weed_amd import workloads

pytestmark = pytest.mark.gpu


def build_cache(gpu, wl, mode, K, V, rotations=None, scales=None, rotate=0):
    cache = gpu.KVCache(mode, wl.n_seq, wl.n_kv_heads, wl.head_dim, wl.max_len, wl.k_bits, wl.v_bits,
                        wl.k_sign if mode == gpu.KV_LLOYDMAX else 0, wl.v_sign if mode == gpu.KV_LLOYDMAX else 0)
    if rotations is not None:
        cache.set_rotations(dev(rotations[0]), dev(rotations[1]))
    if scales is not None:
        cache.set_scales(*scales)
    Kd, Vd = dev(K), dev(V)
    if len(set(wl.lens)) == 1:
        cache.encode_append(Kd, Vd, rotate=rotate)
    else:
        for s, L in enumerate(wl.lens):
            cache.encode_append(Kd[s:s + 1, :, :L], Vd[s:s + 1, :, :L], seq_begin=s, rotate=rotate)
    return cache


def checker_output(oracle, gpu, cache, wl, q, gqa_weed, Rk=None, Rv=None):
    """Run the CPU checker on the fields the device cache actually holds."""
    kspec, vspec = coder_specs(oracle, cache)
    kf, ka = export(cache, 0, wl.max_len)
    vf, va = export(cache, 1, wl.max_len)
    lloyd = cache.cfg.mode == gpu.KV_LLOYDMAX
    return oracle.decode_attn(kspec, vspec, kf, ka if lloyd else None, vf, va if lloyd else None, q, wl.lens,
                              gqa_weed=gqa_weed, Rk=Rk, Rv=Rv)


def run_decode(gpu, cache, q, gqa, flags, col_major_io=False):
    import torch
    qd = col_major(q) if col_major_io else dev(q)
    out = torch.zeros_like(qd)
    cache.decode_attn(qd, out, gqa_mapping=gqa, flags=flags)
    gpu.sync()
    return out.cpu().numpy()


def rotations(oracle, d, seed):
    rng = np.random.default_rng(seed)
    return (oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32)),
            oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32)))


def test_cfg1_weed_uniform_end_to_end(gpu, oracle):
    """Configuration 1 in Weed's own coder: rotation, global block scale, 4-bit uniform codes, one head, ctx 512.
    The whole chain runs on the device (rotate = 2 keeps the reference's rounding order) and is compared with the
    checker fed the raw inputs."""
    wl = workloads.config(1)
    K, V, q = wl.tensors()
    d = wl.head_dim
    Rk, Rv = rotations(oracle, d, 1)
    Ky = oracle.apply_rotation(K.reshape(-1, d), Rk)
    Vy = oracle.apply_rotation(V.reshape(-1, d), Rv)
    scales = (oracle.block_scale(Ky), oracle.block_scale(Vy))
    cache = build_cache(gpu, wl, gpu.KV_UNIFORM, K, V, (Rk, Rv), scales, rotate=2)
    kspec, vspec = coder_specs(oracle, cache)
    kf, _ = oracle.encode_rows(kspec, Ky)
    vf, _ = oracle.encode_rows(vspec, Vy)
    got_kf, _ = export(cache, 0, wl.max_len)
    got_vf, _ = export(cache, 1, wl.max_len)
    np.testing.assert_array_equal(got_kf.reshape(-1, d), kf)
    np.testing.assert_array_equal(got_vf.reshape(-1, d), vf)
    want = oracle.decode_attn(kspec, vspec, kf.reshape(1, 1, -1, d), None, vf.reshape(1, 1, -1, d), None, q, wl.lens,
                              Rk=Rk, Rv=Rv)
    got = run_decode(gpu, cache, q, gpu.GQA_WEED, gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT, col_major_io=True)
    assert_attn_close(got, want, "cfg1 uniform")
    cache.close()


@pytest.mark.parametrize("index", [1, 2, 3])
def test_configs_lloydmax(gpu, oracle, index):
    """Configurations 1-3 at full size with the Lloyd-Max coder (config 3: 32 query / 8 kv heads, ctx 8192)."""
    wl = workloads.config(index)
    K, V, q = wl.tensors()
    Rk, Rv = rotations(oracle, wl.head_dim, index)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V, (Rk, Rv), rotate=1)
    for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
        want = checker_output(oracle, gpu, cache, wl, q, weed, Rk, Rv)
        got = run_decode(gpu, cache, q, gqa, gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT)
        assert_attn_close(got, want, "cfg%d mapping %d" % (index, gqa))
        if wl.n_q_heads == wl.n_kv_heads:
            break
    cache.close()


def test_cfg4_ragged_batch_reduced(gpu, oracle):
    """Configuration 4 (16 ragged sequences, 2-bit keys + sign, 3-bit values, split-context combine) with lengths
    scaled down 16x so that the scalar checker finishes in seconds."""
    wl = workloads.config(4, scale=1.0 / 16)
    assert min(wl.lens) >= 128 and max(wl.lens) <= 2048 and len(set(wl.lens)) > 8
    K, V, q = wl.tensors()
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, True)
    got = run_decode(gpu, cache, q, gpu.GQA_WEED, 0)
    assert_attn_close(got, want, "cfg4 reduced")
    # 32 query heads over the same 8 kv heads (the GQA variant of this configuration)
    rng = np.random.default_rng(3)
    q32 = rng.standard_normal((wl.n_seq, 32, wl.head_dim), dtype=np.float32)
    want = checker_output(oracle, gpu, cache, wl, q32, False)
    got = run_decode(gpu, cache, q32, gpu.GQA_BLOCKED, 0)
    assert_attn_close(got, want, "cfg4 reduced, 32 query heads")
    cache.close()


def test_cfg4_full_size_properties(gpu, oracle):
    """Configuration 4 at full size (lengths up to 32768): properties that do not need the scalar checker.
      * identical V rows: the softmax weights sum to one, so every output equals that row's dequantised value;
      * one sequence checked against the checker in full;
      * permutation: swapping two sequences' queries and caches swaps the outputs."""
    import torch
    wl = workloads.config(4)
    assert max(wl.lens) > 30000
    d, Hkv, S = wl.head_dim, wl.n_kv_heads, wl.n_seq
    rng = np.random.default_rng(11)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, wl.max_len, wl.k_bits, wl.v_bits, wl.k_sign, wl.v_sign)
    v_row = rng.standard_normal((1, Hkv, 1, d), dtype=np.float32)
    short = int(np.argmin(wl.lens))
    K_short = None
    for s, L in enumerate(wl.lens):
        Ks = rng.standard_normal((1, Hkv, L, d), dtype=np.float32)
        if s == short:
            K_short = Ks
        Kd = dev(Ks)
        Vd = dev(v_row).expand(1, Hkv, L, d)  # stride 0 along tokens: every row is the same vector
        cache.encode_append(Kd, Vd, seq_begin=s)
        del Kd
    assert cache.seq_lens() == wl.lens
    q = rng.standard_normal((S, wl.n_q_heads, d), dtype=np.float32)
    got = run_decode(gpu, cache, q, gpu.GQA_WEED, 0)
    kspec, vspec = coder_specs(oracle, cache)
    vf, va = oracle.encode_rows(vspec, v_row.reshape(-1, d))
    v_hat = oracle.decode_rows(vspec, vf, va)  # [Hkv, d]
    for s in range(S):
        assert_attn_close(got[s], v_hat, "constant-V property, sequence %d" % s)
    # the shortest sequence in full against the checker
    L = wl.lens[short]
    kf, ka = oracle.encode_rows(kspec, K_short.reshape(-1, d))
    vf_full = np.broadcast_to(vf.reshape(1, Hkv, 1, d), (1, Hkv, L, d))
    va_full = np.broadcast_to(va.reshape(1, Hkv, 1), (1, Hkv, L))
    want = oracle.decode_attn(kspec, vspec, kf.reshape(1, Hkv, L, d), ka.reshape(1, Hkv, L), vf_full, va_full,
                              q[short:short + 1], [L])
    assert_attn_close(got[short:short + 1], want, "cfg4 full size, shortest sequence")
    cache.close()


def test_split_context_matches_single_pass(gpu, oracle):
    """The split-context merge equals one pass over the whole context: a long single sequence (many splits) and the
    same tokens as the tail of a batch (few splits) give the same answer as the checker's one-pass softmax, including
    when one split holds a score far above all others."""
    rng = np.random.default_rng(21)
    d, Hkv, Hq, L = 64, 2, 4, 5000
    K = rng.standard_normal((1, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((1, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((1, Hq, d), dtype=np.float32)
    K[0, :, 4321] = 6.0 * q[0, :Hkv]  # a key aligned with the query: dominates the softmax
    wl = workloads.Workload("split", 1, Hq, Hkv, d, [L], 4, 4, 0, 0, 0)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, True)
    got = run_decode(gpu, cache, q, gpu.GQA_WEED, 0)
    assert_attn_close(got, want, "split context")
    cache.close()


def test_one_long_region_keeps_within_the_slot_limit(gpu, oracle):
    """A single sequence with one kv head and more 64-token blocks (1032) than the merge kernel has partial slots per
    head: the launch must lengthen its runs instead of failing, and still match the checker."""
    rng = np.random.default_rng(23)
    d, Hkv, Hq, L = 64, 1, 2, 66000
    K = rng.standard_normal((1, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((1, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((1, Hq, d), dtype=np.float32)
    wl = workloads.Workload("long", 1, Hq, Hkv, d, [L], 2, 2, 0, 0, 0)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, True)
    got = run_decode(gpu, cache, q, gpu.GQA_WEED, 0)
    assert_attn_close(got, want, "one long region")
    cache.close()


def test_run_geometry_knobs_do_not_change_the_answer(gpu, oracle):
    """The launch cuts the block list into per-wavefront runs whose lengths are skewed by wavefront age; whatever
    the skew and the number of runs, every block must be attended exactly once: ragged batch (runs straddle regions,
    empty sequence in the middle) against the checker under several settings of the two tuning variables."""
    rng = np.random.default_rng(29)
    d, Hkv, Hq = 128, 2, 8
    lens = [700, 0, 64, 3000, 129, 1]
    S = len(lens)
    wl = workloads.Workload("knobs", S, Hq, Hkv, d, lens, 3, 4, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, False)
    try:
        for waves, skew in ((0, -1), (16, 0), (16, 45), (7, 90), (40, 30), (100000, 16)):
            gpu.decode_tuning(waves, skew)
            got = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
            assert_attn_close(got, want, "waves=%d skew=%d" % (waves, skew))
    finally:
        gpu.decode_tuning()
    cache.close()


def test_equal_contexts_with_and_without_the_region_search(gpu, oracle):
    """A batch of equal contexts finds each wavefront's first region by division; the search used for ragged batches
    must give the same bits."""
    rng = np.random.default_rng(31)
    d, Hkv, Hq, S, L = 128, 2, 8, 5, 1500
    wl = workloads.Workload("equal", S, Hq, Hkv, d, [L] * S, 3, 4, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, False)
    try:
        fast = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
        # (with the merge left to the second kernel and one contiguous piece per wavefront on both sides: the kernel's
        # own merge, and wavefronts that take their blocks in turns, add in another order)
        gpu.decode_tuning(separate_merge=True, contiguous_runs=True)
        divided = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
        gpu.decode_tuning(always_search=True)
        searched = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
    finally:
        gpu.decode_tuning()
    assert_attn_close(fast, want, "equal contexts")
    assert_attn_close(divided, want, "equal contexts, separate merge")
    assert np.array_equal(divided, searched)
    cache.close()


@pytest.mark.parametrize("lloyd,d,Hkv,Hq,S,L,kb,vb,waves,rot", [
    (True, 128, 2, 8, 4, 1024, 3, 4, 32, True),     # two regions per workgroup, four wavefronts each
    (True, 128, 1, 4, 5, 1024, 3, 4, 20, True),     # the last workgroup holds one region of its two
    (True, 128, 2, 16, 2, 1024, 3, 4, 16, False),   # groups of 8, no rotations
    (False, 64, 2, 16, 4, 768, 4, 4, 48, True),     # uniform coder, head_dim 64, groups of 8, three age classes
    (True, 128, 2, 8, 2, 768, 2, 2, 24, True),      # three wavefronts per SIMD: three age classes
    (True, 64, 4, 4, 8, 768, 3, 3, 96, True),       # groups of one, four regions per workgroup
    (False, 128, 1, 2, 8, 2048, 8, 8, 64, True),    # 8-bit uniform codes (no lookup tables)
    (True, 128, 2, 32, 4, 1024, 3, 4, 32, True),    # groups of 16 (the sixteen-column instance), 32 rows per workgroup
    (False, 64, 1, 16, 6, 768, 4, 4, 0, True),      # groups of 16 at head_dim 64, whatever the natural geometry gives
    # regions of several workgroups' shares: the workgroup that arrives last at a region merges it
    (True, 128, 1, 16, 1, 2048, 3, 4, 16, True),    # groups of 16, two workgroups per region
    (True, 128, 2, 8, 1, 2048, 3, 4, 32, True),     # two workgroups per region
    (True, 128, 1, 4, 1, 8192, 3, 4, 128, True),    # sixteen workgroups per region
    (True, 128, 2, 8, 2, 1536, 2, 2, 96, True),     # three wavefronts per SIMD
    (False, 64, 2, 16, 3, 1536, 4, 4, 144, False),  # uniform coder, head_dim 64, groups of 8, no rotations
    # longer runs, which neighbouring wavefronts work through in turns
    (True, 128, 2, 8, 4, 4096, 3, 4, 64, True),     # runs of 8 +- 1 blocks, all eight of a workgroup's region in turns
    (True, 128, 2, 8, 2, 4096, 3, 4, 64, True),     # runs of 4 +- 1, two workgroups per region
    (True, 128, 2, 8, 4, 2048, 3, 4, 16, True),     # runs of 16 +- 3, four regions of one cycle per workgroup
    (True, 64, 2, 4, 2, 3072, 3, 4, 48, True),      # three age classes: runs of 5, 4 and 3, twelve in turns
    (True, 64, 2, 4, 4, 1536, 3, 4, 48, True),      # three age classes, two regions per workgroup, six in turns
    # head_dim 96 (and 80, which is stored as 96): a workgroup's 768 threads are eight rows of 96
    (True, 96, 2, 8, 4, 768, 3, 4, 48, True),       # two regions per workgroup
    (True, 96, 2, 16, 4, 1536, 4, 4, 96, False),    # groups of 8, one region per workgroup, no rotations
    (True, 80, 2, 8, 4, 768, 3, 4, 48, True),       # head_dim 80
    (False, 96, 1, 4, 8, 768, 4, 4, 96, True),      # uniform coder, four regions per workgroup
    (True, 96, 2, 8, 1, 3072, 3, 4, 48, True),      # head_dim 96, two workgroups per region
    (True, 96, 1, 4, 1, 6144, 3, 4, 96, True),      # head_dim 96, eight workgroups per region
    (True, 80, 2, 16, 2, 3072, 3, 4, 96, False),    # head_dim 80, groups of 8, two workgroups per region, no rotations
    # head_dim 32 (and below, stored as 32): two rows per wavefront
    (True, 32, 2, 8, 4, 768, 3, 4, 48, True),       # two regions per workgroup
    (True, 8, 1, 1, 8, 1536, 4, 4, 96, True),       # head_dim 8 (the reference example's), one head
    (False, 32, 2, 16, 1, 3072, 4, 4, 48, True),    # uniform coder, groups of 8, two workgroups per region
    (True, 24, 1, 4, 1, 6144, 2, 2, 96, False),     # head_dim 24, eight workgroups per region, no rotations
    # head_dim 256: a wavefront takes two of the sixteen tiles of the small rotations; at most 16 rows per workgroup
    (True, 256, 2, 8, 4, 1024, 3, 4, 32, True),     # two regions per workgroup
    (False, 256, 2, 16, 2, 1024, 4, 4, 16, False),  # uniform coder, groups of 8, two regions = 16 rows, no rotations
    (False, 256, 2, 16, 2, 1024, 4, 4, 16, True),   # ... with rotations: two passes of eight rows each
    (True, 256, 1, 4, 1, 4096, 3, 4, 64, True),     # eight workgroups per region
    (True, 240, 2, 16, 1, 2048, 3, 4, 32, True),    # head_dim 240, groups of 8, two workgroups per region
    # head_dims 160, 192 and 224: the workgroup's 512 threads are not whole rows, those behind the last whole row idle
    (True, 192, 2, 8, 4, 1024, 3, 4, 32, True),     # head_dim 192, two regions per workgroup
    (True, 160, 2, 16, 2, 1024, 3, 4, 16, True),    # head_dim 160, groups of 8, 16 rows per workgroup
    (False, 224, 1, 4, 1, 4096, 4, 4, 64, True),    # head_dim 224, uniform coder, eight workgroups per region
    (True, 200, 2, 8, 1, 2048, 3, 4, 32, False),    # head_dim 200 (stored as 224), two workgroups per region, no rotations
    (True, 176, 1, 4, 5, 1024, 2, 3, 40, True),     # head_dim 176 (stored as 192), the last workgroup holds one region of its two
    (True, 256, 2, 8, 2, 1024, 2, 2, 16, True),     # head_dim 256, 2-bit codes on both sides
    (False, 256, 2, 4, 2, 2048, 4, 2, 32, False),   # head_dim 256, uniform 4-bit K and 2-bit V, no rotations
])
def test_workgroups_that_merge_their_own_regions(gpu, oracle, lloyd, d, Hkv, Hq, S, L, kb, vb, waves, rot):
    """When every workgroup of the matrix-core kernel holds whole regions, or every region a whole number of
    workgroups' shares, the kernel rotates its queries and merges its partials itself and the call is a single kernel;
    the same call with the kernels ahead and behind must agree to rounding, and both with the checker.  Also with
    per-sequence prefix lengths, zero among them, and twice in a row (the arrival counters are back at zero)."""
    import torch
    rng = np.random.default_rng(53)
    wl = workloads.Workload("merge", S, Hq, Hkv, d, [L] * S, kb, vb, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, 7) if rot else (None, None)
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    cache = build_cache(gpu, wl, mode, K, V, rotations=(Rk, Rv) if rot else None,
                        scales=None if lloyd else (1.0, 1.0), rotate=1 if rot else 0)
    flags = (gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT) if rot else 0
    want = checker_output(oracle, gpu, cache, wl, q, False, Rk=Rk, Rv=Rv)
    prefix = [L - 1 - 37 * s for s in range(S)]
    prefix[S // 2] = 0
    wl_p = workloads.Workload("merge", S, Hq, Hkv, d, prefix, kb, vb, 0, 0, 0)
    want_p = checker_output(oracle, gpu, cache, wl_p, q, False, Rk=Rk, Rv=Rv)
    lens_dev = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    try:
        gpu.profile_reset()
        gpu.profile_enable(True)
        gpu.decode_tuning(waves)
        one_kernel = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        again = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        qd = dev(q)
        out = torch.zeros_like(qd)
        cache.decode_attn_prefix(lens_dev, qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
        gpu.sync()
        one_kernel_p = out.cpu().numpy()
        # the merging kernel ran: the timing scope of the second kernel saw no launch
        assert gpu.profile_read("kv_decode_attn")[1] == 3 and gpu.profile_read("kv_decode_combine")[1] == 0
        gpu.decode_tuning(waves, separate_query=True)
        own_merge = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        gpu.decode_tuning(waves, separate_merge=True)
        own_queries = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        gpu.decode_tuning(waves, separate_merge=True, separate_query=True)
        three_kernels = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        assert gpu.profile_read("kv_decode_combine")[1] == 2
    finally:
        gpu.profile_enable(False)
        gpu.decode_tuning()
    assert_attn_close(three_kernels, want, "three kernels")
    assert_attn_close(own_merge, want, "own merge")
    assert_attn_close(own_queries, want, "own queries")
    assert_attn_close(one_kernel, want, "one kernel")
    assert_attn_close(one_kernel_p, want_p, "one kernel, prefix lengths")
    np.testing.assert_allclose(one_kernel, three_kernels, rtol=2e-5, atol=2e-6)
    assert np.all(one_kernel_p[S // 2] == 0.0)
    # a second call gives the same bits (the order of every sum is fixed)
    assert np.array_equal(again, one_kernel)
    cache.close()


@pytest.mark.parametrize("d,Hkv,Hq,S,L,waves", [(128, 2, 8, 4, 4096, 64), (128, 2, 8, 2, 4096, 64), (64, 2, 4, 2, 3072, 48)])
def test_runs_that_take_turns(gpu, oracle, d, Hkv, Hq, S, L, waves):
    """In batches of equal sequences the wavefronts of neighbouring runs take the blocks of their common piece in turns
    (each keeps its number of blocks); with one contiguous piece per wavefront instead, the call adds the same blocks
    in another grouping: both agree with the checker, and they differ in the last bits (so the turns were taken)."""
    rng = np.random.default_rng(59)
    wl = workloads.Workload("turns", S, Hq, Hkv, d, [L] * S, 3, 4, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, False)
    try:
        gpu.decode_tuning(waves)
        turns = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
        gpu.decode_tuning(waves, contiguous_runs=True)
        pieces = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
    finally:
        gpu.decode_tuning()
    assert_attn_close(turns, want, "turns")
    assert_attn_close(pieces, want, "contiguous pieces")
    np.testing.assert_allclose(turns, pieces, rtol=2e-5, atol=2e-6)
    assert not np.array_equal(turns, pieces)
    cache.close()


@pytest.mark.parametrize("cap_blocks,top,step,S,Hkv,d", [(24, 23 * 64 - 20, 0, 32, 8, 128), (23, 23 * 64 - 20, 0, 32, 8, 128),
                                                         (24, 24 * 64 - 10, 30, 32, 8, 128), (128, 125 * 64 - 7, 0, 2, 2, 128),
                                                         (64, 61 * 64 - 1, 70, 3, 4, 128), (128, 8000, 2500, 3, 2, 128),
                                                         (23, 23 * 64 - 20, 0, 32, 8, 256), (24, 24 * 64 - 10, 30, 32, 8, 96)])
def test_block_counts_that_no_run_length_divides(gpu, oracle, cap_blocks, top, step, S, Hkv, d):
    """Sequences of 23 blocks on a full device: no run length divides them into whole regions per workgroup.
    The partition counts 24 blocks per region, the last one without tokens, and the call stays one kernel with whole
    regions per workgroup -- also with a capacity of 23 blocks, where the 24th block of the last region would lie
    behind the cache's memory and is never read.  The third case mixes sequences of 23 and 24
    blocks, which are counted alike.  Three cases are small batches, where a region is several workgroups' shares
    and the count is rounded to a whole number of those; in the last of them the sequences hold 8000, 5500 and 3000
    tokens and are all counted as 128 blocks, so whole workgroups find no tokens in their share.  Head_dims 256
    and 96 merge whole regions like 128 (at 96 a workgroup of twelve wavefronts is eight rows of 96 threads, at 256
    one of eight wavefronts is two rows).  All must
    agree with the checker, with the three-kernel way, under prefix lengths (zero among them), and after a step's
    one-token append."""
    import torch
    Hq = 2 * Hkv
    lens = [top - step * (s % 3) for s in range(S)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    rng = np.random.default_rng(78)
    wl = workloads.Workload("rounded", S, Hq, Hkv, d, lens, 3, 4, 0, 0, 0)
    Rk, Rv = rotations(oracle, d, 9)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, cap_blocks * 64, 3, 4, 0, 0)
    cache.set_rotations(dev(Rk), dev(Rv))
    K = torch.randn((S, Hkv, top + 1, d), generator=gen, device="cuda")
    V = torch.randn((S, Hkv, top + 1, d), generator=gen, device="cuda")
    for s in range(S):
        cache.encode_append(K[s:s + 1, :, :lens[s]], V[s:s + 1, :, :lens[s]], seq_begin=s, rotate=1)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    want = checker_output(oracle, gpu, cache, wl, q, False, Rk=Rk, Rv=Rv)
    prefix = [max(0, lens[s] - 1 - 45 * s) for s in range(S)]
    prefix[S // 2] = 0
    wl_p = workloads.Workload("rounded", S, Hq, Hkv, d, prefix, 3, 4, 0, 0, 0)
    want_p = checker_output(oracle, gpu, cache, wl_p, q, False, Rk=Rk, Rv=Rv)
    lens_dev = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    try:
        gpu.profile_reset()
        gpu.profile_enable(True)
        got = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        again = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        qd = dev(q)
        out = torch.zeros_like(qd)
        cache.decode_attn_prefix(lens_dev, qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
        gpu.sync()
        got_p = out.cpu().numpy()
        assert gpu.profile_read("kv_decode_attn")[1] == 3
        assert gpu.profile_read("kv_decode_combine")[1] == 0
        gpu.decode_tuning(separate_merge=True, separate_query=True)
        three_kernels = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
    finally:
        gpu.profile_enable(False)
        gpu.decode_tuning()
    assert_attn_close(got, want, "one kernel")
    assert_attn_close(three_kernels, want, "three kernels")
    assert_attn_close(got_p, want_p, "prefix lengths")
    assert np.all(got_p[S // 2] == 0.0)
    assert np.array_equal(again, got)
    # the next step of a decode loop: one more token everywhere (the block counts stay), attended again
    cache.encode_append(torch.stack([K[s, :, lens[s]:lens[s] + 1] for s in range(S)]),
                        torch.stack([V[s, :, lens[s]:lens[s] + 1] for s in range(S)]), rotate=1)
    wl1 = workloads.Workload("rounded", S, Hq, Hkv, d, [n + 1 for n in lens], 3, 4, 0, 0, 0)
    want1 = checker_output(oracle, gpu, cache, wl1, q, False, Rk=Rk, Rv=Rv)
    assert_attn_close(run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags), want1, "after one more token")
    cache.close()


@pytest.mark.parametrize("lloyd,d,Hkv,Hq,lens,kb,vb,waves", [
    (True, 128, 2, 8, [700, 64, 3000, 129, 1, 2049], 3, 4, 0),      # ragged, runs straddle regions
    (True, 128, 2, 4, [700, 64, 3000, 129, 1, 2049], 3, 4, 40),     # few, long runs: up to six regions (twelve rows) per workgroup
    (True, 128, 8, 8, [2048, 517, 8192, 1030, 4100], 3, 3, 400),    # groups of one, three wavefronts per SIMD
    (False, 64, 2, 16, [1000, 333, 90, 2500], 4, 4, 0),             # uniform coder, head_dim 64, groups of 8
    (True, 128, 2, 8, [1500] * 5, 3, 4, 0),                         # equal sequences that do not line up
    (True, 128, 1, 4, [640] * 40, 3, 4, 0),                         # many short equal sequences per workgroup
    (True, 128, 1, 16, [3000, 700, 1300], 3, 4, 0),                 # groups of 16, ragged
    # head_dims 96 and 32: the third variant of their instances
    (True, 96, 2, 8, [700, 64, 3000, 129, 1, 2049], 3, 4, 0),       # head_dim 96, ragged
    (True, 80, 2, 16, [1000, 333, 90, 2500], 3, 4, 0),              # head_dim 80, groups of 8
    (True, 96, 8, 8, [2048, 517, 4096, 1030], 3, 3, 0),             # head_dim 96, groups of one
    (True, 32, 2, 8, [700, 64, 3000, 129, 1, 2049], 3, 4, 0),       # head_dim 32, ragged
    (False, 24, 1, 4, [1500] * 5, 4, 4, 0),                         # head_dim 24, uniform coder, equal sequences that do not line up
])
def test_any_batch_as_one_kernel(gpu, oracle, lloyd, d, Hkv, Hq, lens, kb, vb, waves):
    """Batches whose regions do not line up with the workgroups (ragged, or equal but unaligned): the wavefronts'
    partials go through memory, the workgroup that arrives last at a region merges it, and the call is still one
    kernel.  Against the checker and the three-kernel way, with prefix lengths, twice in a row."""
    import torch
    rng = np.random.default_rng(59)
    S, L = len(lens), max(lens)
    wl = workloads.Workload("any", S, Hq, Hkv, d, lens, kb, vb, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, 11)
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    cache = build_cache(gpu, wl, mode, K, V, rotations=(Rk, Rv), scales=None if lloyd else (1.0, 1.0), rotate=1)
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    want = checker_output(oracle, gpu, cache, wl, q, False, Rk=Rk, Rv=Rv)
    prefix = [max(0, n - 1 - 13 * s) for s, n in enumerate(lens)]
    prefix[S // 2] = 0
    wl_p = workloads.Workload("any", S, Hq, Hkv, d, prefix, kb, vb, 0, 0, 0)
    want_p = checker_output(oracle, gpu, cache, wl_p, q, False, Rk=Rk, Rv=Rv)
    lens_dev = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    try:
        gpu.profile_reset()
        gpu.profile_enable(True)
        gpu.decode_tuning(waves)
        one_kernel = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        again = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        qd = dev(q)
        out = torch.zeros_like(qd)
        cache.decode_attn_prefix(lens_dev, qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
        gpu.sync()
        one_kernel_p = out.cpu().numpy()
        assert gpu.profile_read("kv_decode_attn")[1] == 3 and gpu.profile_read("kv_decode_combine")[1] == 0
        gpu.decode_tuning(waves, separate_query=True)
        own_merge = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        gpu.decode_tuning(waves, separate_merge=True, separate_query=True)
        three_kernels = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, flags)
        assert gpu.profile_read("kv_decode_combine")[1] == 1
    finally:
        gpu.profile_enable(False)
        gpu.decode_tuning()
    assert_attn_close(three_kernels, want, "three kernels")
    assert_attn_close(own_merge, want, "own merge")
    assert_attn_close(one_kernel, want, "one kernel")
    assert_attn_close(one_kernel_p, want_p, "one kernel, prefix lengths")
    np.testing.assert_allclose(one_kernel, three_kernels, rtol=2e-5, atol=2e-6)
    assert np.all(one_kernel_p[S // 2] == 0.0)
    assert np.array_equal(again, one_kernel)
    cache.close()


@pytest.mark.parametrize("which", ["cfg4_reduced", "equal_24", "small_4"])
def test_merges_through_memory_repeat_bit_for_bit(gpu, oracle, which):
    """The merges that go through memory and an arrival counter per region -- ragged batches (configuration 4 at a
    sixteenth of its lengths), equal sequences whose regions do not line up with the workgroups (24 sequences), and a
    small batch whose regions are several workgroups' shares (4 sequences) -- run 300 times back to back through the
    one-kernel path: every output must equal the first one bit for bit (the order of the additions is fixed, so any
    difference would be a partial read before its writer's store was visible), and the first must match the
    checker.  The counters' release / acquire pair is what this leans on."""
    import torch
    rng = np.random.default_rng(7)
    if which == "cfg4_reduced":
        wl = workloads.config(4, scale=1.0 / 16)
        Hq = 32
    else:
        n = 24 if which == "equal_24" else 4
        wl = workloads.Workload(which, n, 32, 8, 128, [1984 if n == 24 else 8192] * n, 3, 4, 0, 0, 0)
        Hq = 32
    S, Hkv, d, L = wl.n_seq, wl.n_kv_heads, wl.head_dim, wl.max_len
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, L, wl.k_bits, wl.v_bits, wl.k_sign, wl.v_sign)
    for s0, n_tok in enumerate(wl.lens):
        Ks = torch.randn((1, Hkv, n_tok, d), device="cuda")
        Vs = torch.randn((1, Hkv, n_tok, d), device="cuda")
        cache.encode_append(Ks, Vs, seq_begin=s0)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    qd = dev(q)
    outs = [torch.zeros_like(qd) for _ in range(4)]
    try:
        gpu.profile_reset()
        gpu.profile_enable(True)
        cache.decode_attn(qd, outs[0], gpu.GQA_BLOCKED, 0)
        gpu.sync()
        assert gpu.profile_read("kv_decode_attn")[1] == 1 and gpu.profile_read("kv_decode_combine")[1] == 0
    finally:
        gpu.profile_enable(False)
    first = outs[0].clone()
    wl_q = workloads.Workload(which, S, Hq, Hkv, d, wl.lens, wl.k_bits, wl.v_bits, wl.k_sign, wl.v_sign, 0)
    if which != "small_4":  # (the scalar checker takes seconds per thousand tokens and head)
        assert_attn_close(first.cpu().numpy(), checker_output(oracle, gpu, cache, wl_q, q, False), which)
    # launches back to back, three outputs in flight between comparisons so that the device never idles between them
    for rep in range(100):
        for o in outs[1:]:
            cache.decode_attn(qd, o, gpu.GQA_BLOCKED, 0)
        gpu.sync()
        for i, o in enumerate(outs[1:]):
            assert torch.equal(o, first), "%s: repeat %d differs from the first result" % (which, 3 * rep + i + 1)
    cache.close()


def test_random_batches_planned_against_plain(gpu):
    """Sixty seeded random batches -- equal, nearly equal, mildly and widely different lengths, up to 128 sequences,
    caches with and without room behind the longest sequence, both coders, head_dims with and without instances that
    merge their own partials: what the default plan gives (block counts rounded up, sequences counted alike, one kernel
    where it can) against the plain plan (real block counts, region search, three kernels), which the other tests
    check against the CPU checker.  The bar is this file's."""
    import torch
    rng = np.random.default_rng(4242)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)

    def randn(*shape):
        return torch.randn(shape, generator=gen, device="cuda")

    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    try:
        for case in range(60):
            d = int(rng.choice([32, 96, 160, 256, 128, 64]))
            Hkv = int(rng.choice([1, 2, 4, 8]))
            G = int(rng.choice([1, 2, 4, 8]))
            S = int(rng.choice([1, 2, 3, 5, 8, 16, 31, 40, 64, 70, 128]))
            top = max(1, int(rng.integers(1, 50)) * 64 + int(rng.integers(-63, 1)))
            kind = int(rng.integers(0, 4))
            if kind == 0:
                lens = [top] * S
            elif kind == 1:
                lens = [max(1, top - int(rng.integers(0, 130))) for _ in range(S)]
            elif kind == 2:
                lens = [max(1, int(top * rng.uniform(0.5, 1.0))) for _ in range(S)]
            else:
                lens = [max(1, int(top * rng.uniform(0.02, 1.0))) for _ in range(S)]
            cap = max(lens) + int(rng.choice([0, 1, 64, 200, 1000]))
            lloyd = bool(rng.integers(2))
            if lloyd:
                kb, vb = int(rng.choice([2, 3, 4])), int(rng.choice([2, 3, 4]))
                ks, vs = int(rng.integers(2)), int(rng.integers(2))
            else:
                kb = vb = int(rng.choice([2, 3, 4, 5, 6, 8]))
                ks = vs = 0
            cache = gpu.KVCache(gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM, S, Hkv, d, cap, kb, vb, ks, vs)
            if not lloyd:
                cache.set_scales(1.1, 0.9)
            rk, rv = torch.zeros(d * d, device="cuda"), torch.zeros(d * d, device="cuda")
            gpu.make_rotation(5, d, rk)
            gpu.make_rotation(6, d, rv)
            cache.set_rotations(rk, rv)
            for s, n in enumerate(lens):
                cache.encode_append(randn(1, Hkv, n, d), randn(1, Hkv, n, d), seq_begin=s, rotate=1)
            q = randn(S, Hkv * G, d)
            planned, plain = torch.zeros_like(q), torch.zeros_like(q)
            gpu.decode_tuning()
            cache.decode_attn(q, planned, gpu.GQA_BLOCKED, flags)
            gpu.decode_tuning(always_search=True, separate_merge=True, separate_query=True)
            cache.decode_attn(q, plain, gpu.GQA_BLOCKED, flags)
            gpu.sync()
            what = "case %d: d %d, K %d+%d V %d+%d bits, lloyd %d, %d x %d heads, capacity %d, lengths %s" % (
                case, d, kb, ks, vb, vs, lloyd, Hkv, G, cap, lens)
            assert not torch.isnan(planned).any(), what
            excess = ((planned - plain).abs() - (1e-4 + 1e-3 * plain.abs())).max().item()
            assert excess <= 0, what
            cache.close()
    finally:
        gpu.decode_tuning()


def test_edge_lengths(gpu, oracle):
    """Empty sequences give zeros; lengths 1, 63, 64, 65 around the 64-token block; an appended token changes the
    result exactly as the checker says."""
    import torch
    rng = np.random.default_rng(31)
    d, Hkv, Hq = 128, 2, 8
    lens = [0, 1, 63, 64, 65, 257]
    S = len(lens)
    wl = workloads.Workload("edges", S, Hq, Hkv, d, lens, 3, 4, 1, 0, 0)
    K = rng.standard_normal((S, Hkv, max(lens) + 1, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens) + 1, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, S, Hkv, d, max(lens) + 1, 3, 4, 1, 0)
    Kd, Vd = dev(K), dev(V)
    for s, L in enumerate(lens):
        if L:
            cache.encode_append(Kd[s:s + 1, :, :L], Vd[s:s + 1, :, :L], seq_begin=s)
    want = checker_output(oracle, gpu, cache, wl, q, False)
    got = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
    assert not got[0].any()
    assert_attn_close(got, want, "edge lengths")
    # decode step: append one token to every sequence and attend again
    cache.encode_append(torch.stack([Kd[s, :, L:L + 1] for s, L in enumerate(lens)]),
                        torch.stack([Vd[s, :, L:L + 1] for s, L in enumerate(lens)]))
    wl2 = workloads.Workload("edges+1", S, Hq, Hkv, d, [L + 1 for L in lens], 3, 4, 1, 0, 0)
    want2 = checker_output(oracle, gpu, cache, wl2, q, False)
    got2 = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
    assert_attn_close(got2, want2, "edge lengths + 1")
    assert np.abs(got2[1] - got[1]).max() > 1e-3
    cache.close()


def test_head_dims_and_wide_groups(gpu, oracle):
    """head_dim 32 and 256, and 16 query heads per kv head (two passes of the 8-head inner loop)."""
    rng = np.random.default_rng(41)
    for d, Hkv, Hq, L in ((32, 2, 2, 300), (256, 1, 4, 200), (64, 1, 16, 333)):
        wl = workloads.Workload("dims", 2, Hq, Hkv, d, [L, L // 2], 4, 2, 0, 1, 0)
        K = rng.standard_normal((2, Hkv, L, d), dtype=np.float32)
        V = rng.standard_normal((2, Hkv, L, d), dtype=np.float32)
        q = rng.standard_normal((2, Hq, d), dtype=np.float32)
        cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
        for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
            want = checker_output(oracle, gpu, cache, wl, q, weed)
            got = run_decode(gpu, cache, q, gqa, 0)
            assert_attn_close(got, want, "d=%d Hq=%d" % (d, Hq))
        cache.close()


@pytest.mark.parametrize("d", [8, 48, 80, 100, 250])
@pytest.mark.parametrize("lloyd", [False, True])
def test_any_head_dim(gpu, oracle, d, lloyd):
    """QuantizedKVCache::allocate takes any d (multihead_attention.cpp:31-41; the reference's transformer example
    runs head_dim 8): rows are stored with head_dim rounded up to a multiple of 32 and zeros in the extra coordinates.
    The whole chain on the device (rotation in the reference's rounding order, coder, fused attention, un-rotation)
    against the checker fed the raw inputs, the codes bit for bit, Weed's words included."""
    import torch
    rng = np.random.default_rng(7 * d + lloyd)
    Hkv, Hq, lens = 2, 4, [150, 64, 1]
    S, L = len(lens), max(lens)
    bits = 4 if d <= 128 else 3
    wl = workloads.Workload("any_d", S, Hq, Hkv, d, lens, bits, bits, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, L, d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, 500 + d)
    Kr = oracle.apply_rotation(K.reshape(-1, d), Rk).reshape(K.shape)
    Vr = oracle.apply_rotation(V.reshape(-1, d), Rv).reshape(V.shape)
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    scales = None if lloyd else (oracle.block_scale(Kr), oracle.block_scale(Vr))
    cache = build_cache(gpu, wl, mode, K, V, rotations=(Rk, Rv), scales=scales, rotate=2)
    kspec, vspec = coder_specs(oracle, cache)
    for which, xr, spec in ((0, Kr, kspec), (1, Vr, vspec)):
        for sq, n in enumerate(lens):
            want_f, want_a = oracle.encode_rows(spec, xr[sq, :, :n].reshape(-1, d))
            got_f, got_a = export(cache, which, n, seq_begin=sq, seq_count=1)
            np.testing.assert_array_equal(got_f.reshape(-1, d), want_f)
            if lloyd:
                np.testing.assert_array_equal(got_a.reshape(-1), want_a)
            else:
                wpr = oracle.words_per_row(d, bits)
                words = torch.zeros((1, Hkv, n, wpr), dtype=torch.int32, device="cuda")
                cache.export_weed_words(which, words, seq_begin=sq)
                want_w = oracle.uniform_write_rows(xr[sq, :, :n].reshape(-1, d), bits, spec.block_scale)
                np.testing.assert_array_equal(words.cpu().numpy().reshape(-1, wpr), want_w)
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
        want = checker_output(oracle, gpu, cache, wl, q, weed, Rk=Rk, Rv=Rv)
        assert_attn_close(run_decode(gpu, cache, q, gqa, flags), want, "head_dim %d" % d)
    cache.close()


@pytest.mark.parametrize("d", [32, 64, 96, 128])
@pytest.mark.parametrize("wk", [2, 3, 4, 5])
@pytest.mark.parametrize("wv", [2, 3, 4, 5])
def test_every_pair_of_field_widths(gpu, oracle, d, wk, wv):
    """Lloyd-Max fields of 2 to 5 bits on either side (a width is code bits plus the optional sign bit; both ways of
    making 3 and 4 occur): every pair has its own instance of the matrix-core kernel, the 5-bit ones with single-value
    tables.  Ragged lengths across block edges, groups of 4 and of 16 heads per KV head, both GQA mappings."""
    rng = np.random.default_rng(100 * wk + 10 * wv + d)
    with_sign = (wk + wv) % 2 == 0
    split = {2: (2, 0), 3: (2, 1) if with_sign else (3, 0), 4: (3, 1) if with_sign else (4, 0), 5: (4, 1)}
    (kb, ks), (vb, vs) = split[wk], split[wv]
    Hkv, lens = 2, [200, 65, 64]
    S = len(lens)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32) * rng.uniform(0.3, 3.0, size=(S, Hkv, max(lens), 1)).astype(np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    wl = workloads.Workload("widths", S, 4 * Hkv, Hkv, d, lens, kb, vb, ks, vs, 0)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    assert cache.row_bytes() == (d * wk // 8 + 4, d * wv // 8 + 4)
    for Hq, gqa, weed in ((4 * Hkv, gpu.GQA_BLOCKED, False), (16 * Hkv, gpu.GQA_WEED, True)):
        q = rng.standard_normal((S, Hq, d), dtype=np.float32)
        wl_q = workloads.Workload("widths", S, Hq, Hkv, d, lens, kb, vb, ks, vs, 0)
        want = checker_output(oracle, gpu, cache, wl_q, q, weed)
        assert_attn_close(run_decode(gpu, cache, q, gqa, 0), want, "K %d+%d V %d+%d, %d heads" % (kb, ks, vb, vs, Hq))
    cache.close()


@pytest.mark.parametrize("d,Hkv,G", [(128, 1, 32), (64, 2, 24), (128, 2, 40), (256, 1, 12), (64, 1, 71), (96, 1, 32),
                                     (32, 2, 20)])
def test_groups_larger_than_a_tile(gpu, oracle, d, Hkv, G):
    """Multi-query shapes (one or two KV heads for dozens of query heads): the group goes through the cache in several
    passes of the matrix-core kernel, 16 heads (8 at head_dim 256) at most per pass, one merge for all of them; both
    GQA mappings, ragged lengths, group sizes that do not split evenly."""
    rng = np.random.default_rng(d + Hkv + G)
    lens = [190, 64, 3]
    S, Hq = len(lens), Hkv * G
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    wl = workloads.Workload("mqa", S, Hq, Hkv, d, lens, 3, 4, 1, 0, 0)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
        want = checker_output(oracle, gpu, cache, wl, q, weed)
        assert_attn_close(run_decode(gpu, cache, q, gqa, 0), want, "group of %d" % G)
    cache.close()


def test_passes_of_a_large_group_share_one_launch(gpu, oracle):
    """40 query heads per KV head are three passes of the matrix-core kernel, and they are ONE launch whose workgroups
    find their pass from their index (those of a pass are rounded up to a multiple of eight, the extra ones leave at
    once): enough sequences for several octets of workgroups per pass, ragged lengths, one sequence without tokens;
    against the checker."""
    rng = np.random.default_rng(40)
    d, Hkv, G = 128, 2, 40
    lens = [int(x) for x in rng.integers(1, 700, size=24)]
    lens[5] = 0
    S, Hq = len(lens), Hkv * G
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    wl = workloads.Workload("mqa", S, Hq, Hkv, d, lens, 3, 4, 1, 0, 0)
    cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX, K, V)
    want = checker_output(oracle, gpu, cache, wl, q, False)
    got = run_decode(gpu, cache, q, gpu.GQA_BLOCKED, 0)
    assert_attn_close(got, want, "three passes in one launch")
    assert np.all(got[5] == 0.0)
    cache.close()


@pytest.mark.parametrize("d", [160, 192, 224, 256])
@pytest.mark.parametrize("wk,wv,Hq", [(2, 2, 2), (3, 4, 8), (4, 4, 16), (4, 3, 4), (4, 2, 32)])
def test_head_dims_above_128(gpu, oracle, d, wk, wv, Hq):
    """head_dim 160 to 256 on the matrix cores (fields of 2 to 4 bits, up to 8 heads per KV head and pass; 16 heads
    per KV head take two passes): ragged lengths, both coders, rotations, a chunk of two positions."""
    import torch
    rng = np.random.default_rng(wk * 10 + wv + Hq + d)
    Hkv, lens = 2, [130, 64, 257]
    S = len(lens)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, wk)
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    for lloyd in (True, False):
        (kb, ks), (vb, vs) = ((wk - 1, 1), (wv, 0)) if lloyd else ((wk, 0), (wv, 0))
        wl = workloads.Workload("wide_heads", S, Hq, Hkv, d, lens, kb, vb, ks, vs, 0)
        cache = build_cache(gpu, wl, gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM, K, V, (Rk, Rv),
                            None if lloyd else (1.0, 1.1), rotate=2)
        for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
            want = checker_output(oracle, gpu, cache, wl, q, weed, Rk, Rv)
            assert_attn_close(run_decode(gpu, cache, q, gqa, flags), want, "d %d, %d + %d bits" % (d, wk, wv))
        if Hq // Hkv <= 4:
            T = 2
            qc = rng.standard_normal((S, T, Hq, d), dtype=np.float32)
            out = torch.zeros((S, T, Hq, d), device="cuda")
            cache.decode_attn_chunk(dev(qc), out, gqa_mapping=gpu.GQA_WEED, flags=flags)
            for t in range(T):
                wl_t = workloads.Workload("wide_heads", S, Hq, Hkv, d, [n - (T - 1 - t) for n in lens], kb, vb, ks, vs, 0)
                want = checker_output(oracle, gpu, cache, wl_t, np.ascontiguousarray(qc[:, t]), True, Rk, Rv)
                assert_attn_close(out[:, t].cpu().numpy(), want, "chunk position %d" % t)
        cache.close()


@pytest.mark.parametrize("kb,vb,d", [(8, 8, 128), (8, 8, 64), (8, 8, 96), (8, 8, 32), (7, 7, 128), (7, 7, 32),
                                     (6, 6, 64), (6, 6, 96), (1, 1, 128), (1, 1, 32), (1, 1, 256), (5, 5, 128),
                                     (5, 4, 64), (5, 6, 64), (8, 4, 128), (1, 7, 32)])
def test_uniform_widths_beyond_four_bits(gpu, oracle, kb, vb, d):
    """Weed's uniform coder at any width the reference's `kv_quant_bits` may take: attention equals the checker on the
    same codes, with rotations and both GQA mappings.  Equal widths of 6 to 8 bits (8 is the common request) run on the
    matrix cores, their codes turned into fp16 arithmetically, also for a chunk of query positions and for 16 heads
    per KV head; 5-bit codes use the single-value tables, 1-bit codes four-entry pair tables; unequal widths beyond
    five bits go through the generic kernel."""
    import torch
    rng = np.random.default_rng(kb * 16 + vb + d)
    Hkv, Hq, lens = 2, 8, [300, 77, 64]
    S = len(lens)
    wl = workloads.Workload("wide", S, Hq, Hkv, d, lens, kb, vb, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, kb)
    cache = build_cache(gpu, wl, gpu.KV_UNIFORM, K, V, (Rk, Rv), (1.1, 0.9), rotate=2)
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    for gqa, weed in ((gpu.GQA_WEED, True), (gpu.GQA_BLOCKED, False)):
        want = checker_output(oracle, gpu, cache, wl, q, weed, Rk, Rv)
        got = run_decode(gpu, cache, q, gqa, flags)
        assert_attn_close(got, want, "K %d-bit V %d-bit" % (kb, vb))
    # the codes really use the whole range
    kf, _ = export(cache, 0, 64)
    assert kf.max() == (1 << kb) - 1 and kf.min() == 0
    if kb == vb and kb >= 6:
        T = 2
        qc = rng.standard_normal((S, T, Hq, d), dtype=np.float32)
        out = torch.zeros((S, T, Hq, d), device="cuda")
        cache.decode_attn_chunk(dev(qc), out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
        for t in range(T):
            wl_t = workloads.Workload("wide", S, Hq, Hkv, d, [n - (T - 1 - t) for n in lens], kb, vb, 0, 0, 0)
            want = checker_output(oracle, gpu, cache, wl_t, np.ascontiguousarray(qc[:, t]), False, Rk, Rv)
            assert_attn_close(out[:, t].cpu().numpy(), want, "chunk position %d" % t)
        # sixteen heads per KV head (the 16-column instance)
        q16 = rng.standard_normal((S, 16 * Hkv, d), dtype=np.float32)
        wl16 = workloads.Workload("wide", S, 16 * Hkv, Hkv, d, lens, kb, vb, 0, 0, 0)
        want = checker_output(oracle, gpu, cache, wl16, q16, True, Rk, Rv)
        assert_attn_close(run_decode(gpu, cache, q16, gpu.GQA_WEED, flags), want, "16 heads per KV head")
    cache.close()


def test_prefix_lengths_override(gpu, oracle):
    """Attention over the first n tokens of each cached sequence (the per-position form of a causal mask) equals the
    checker run with those lengths; the cache's own lengths are untouched."""
    import torch
    rng = np.random.default_rng(41)
    d, Hkv, Hq = 64, 2, 4
    lens = [300, 129, 64]
    S = len(lens)
    wl = workloads.Workload("prefix", S, Hq, Hkv, d, lens, 4, 4, 0, 0, 0)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, Hq, d), dtype=np.float32)
    cache = build_cache(gpu, wl, gpu.KV_UNIFORM, K, V, scales=(1.0, 1.0))
    for prefix in ([300, 129, 64], [1, 128, 63], [257, 0, 17]):
        wl_p = workloads.Workload("prefix", S, Hq, Hkv, d, prefix, 4, 4, 0, 0, 0)
        want = checker_output(oracle, gpu, cache, wl_p, q, True)
        qd = dev(q)
        out = torch.zeros_like(qd)
        cache.decode_attn_prefix(torch.tensor(prefix, dtype=torch.int32, device="cuda"), qd, out)
        gpu.sync()
        assert_attn_close(out.cpu().numpy(), want, "prefix %s" % prefix)
    assert list(cache.seq_lens()) == lens
    cache.close()


@pytest.mark.parametrize("lloyd,d,Hkv,Hq,T,gqa_weed", [(False, 64, 2, 4, 3, True), (True, 128, 2, 8, 2, False),
                                                       (True, 128, 1, 4, 4, True), (False, 128, 2, 2, 5, False),
                                                       (True, 64, 2, 16, 2, True), (True, 128, 2, 8, 4, False),
                                                       (True, 96, 2, 8, 3, True), (False, 32, 1, 4, 4, False),
                                                       (True, 128, 2, 8, 7, False), (False, 64, 1, 4, 11, True),
                                                       (True, 256, 1, 4, 5, True)])
def test_chunk_of_query_positions(gpu, oracle, lloyd, d, Hkv, Hq, T, gqa_weed):
    """Several query positions per sequence in one call (one pass over the cache per tile of (position, head) pairs;
    the larger cases need two or three): position t must equal the checker run over all but the last T - 1 - t tokens.  The lengths put the chunk across a block boundary (a block whose tokens are
    all hidden from the early positions), inside one block, and far from any edge; both GQA mappings; column-major
    operands; rotations on; and the same with the attended lengths given explicitly."""
    import torch
    rng = np.random.default_rng(1000 * T + Hq + d)
    lens = [64 + 1, 300, 129, 64 + T, 5 * 64]
    S = len(lens)
    kb, vb, ks = (3, 4, 1) if lloyd else (4, 3, 0)
    vs = 0
    if lloyd and d == 64:
        kb, vb, ks, vs = 4, 4, 1, 1  # 5-bit fields on both sides
    mode = gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM
    wl = workloads.Workload("chunk", S, Hq, Hkv, d, lens, kb, vb, ks, vs, 0)
    K = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    V = rng.standard_normal((S, Hkv, max(lens), d), dtype=np.float32)
    q = rng.standard_normal((S, T, Hq, d), dtype=np.float32)
    Rk, Rv = rotations(oracle, d, 5)
    cache = build_cache(gpu, wl, mode, K, V, (Rk, Rv), None if lloyd else (1.0, 1.0))
    gqa = gpu.GQA_WEED if gqa_weed else gpu.GQA_BLOCKED
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT

    def check(seen, lens_dev, what):
        for mk in (dev, col_major):
            qd = mk(q)
            out = torch.zeros_like(qd)
            cache.decode_attn_chunk(qd, out, lens=lens_dev, gqa_mapping=gqa, flags=flags)
            gpu.sync()
            got = out.cpu().numpy()
            for t in range(T):
                wl_t = workloads.Workload("chunk", S, Hq, Hkv, d, [n - (T - 1 - t) for n in seen], kb, vb, ks, vs, 0)
                want = checker_output(oracle, gpu, cache, wl_t, np.ascontiguousarray(q[:, t]), gqa_weed, Rk, Rv)
                assert_attn_close(got[:, t], want, "%s position %d" % (what, t))

    check(lens, None, "cached lengths")
    shorter = [max(T, n - 37) for n in lens]
    check(shorter, torch.tensor(shorter, dtype=torch.int32, device="cuda"), "explicit lengths")
    # a chunk of one position is the single-query call
    q1 = dev(np.ascontiguousarray(q[:, :1]))
    out1 = torch.zeros_like(q1)
    cache.decode_attn_chunk(q1, out1, gqa_mapping=gqa, flags=flags)
    ref1 = torch.zeros_like(q1[:, 0])
    cache.decode_attn(q1[:, 0], ref1, gqa_mapping=gqa, flags=flags)
    assert torch.equal(out1[:, 0], ref1)
    # more positions than the entry point takes
    too_many = dev(np.zeros((S, 65, Hq, d), dtype=np.float32))
    with pytest.raises(gpu.WeedHipError):
        cache.decode_attn_chunk(too_many, torch.zeros_like(too_many), gqa_mapping=gqa)
    cache.close()


def test_random_shapes_chunk_equals_single_positions(gpu):
    """Sixty seeded random shapes -- head_dim, coder, field widths, group size (also beyond a tile), chunk length,
    ragged lengths, GQA mapping: a chunk call must give what the single-position calls give (which the other tests
    check against the CPU checker), so every instance family is exercised with every way the work is cut."""
    import torch
    rng = np.random.default_rng(2024)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)

    def randn(*shape):
        return torch.randn(shape, generator=gen, device="cuda")

    for case in range(60):
        d = int(rng.choice([32, 64, 96, 128, 160, 192, 224, 256]))
        lloyd = bool(rng.integers(2))
        if d > 128:
            wk, wv = int(rng.integers(2, 5)), int(rng.integers(2, 5))
        elif rng.random() < 0.25:
            wk = wv = int(rng.choice([1, 6, 7, 8]))
            lloyd = lloyd and wk == 1
        else:
            wk, wv = int(rng.integers(2, 6)), int(rng.integers(2, 6))

        def split(w):
            if not lloyd:
                return w, 0
            if w == 5:
                return 4, 1
            if w == 1:
                return 1, 0
            return (w - 1, 1) if rng.random() < 0.5 else (w, 0)

        (kb, ks), (vb, vs) = split(wk), split(wv)
        Hkv = int(rng.integers(1, 4))
        G = int(rng.choice([1, 2, 3, 4, 7, 8, 12, 16, 20]))
        T, S = int(rng.integers(1, 10)), int(rng.integers(1, 5))
        lens = [int(rng.integers(T, 400)) for _ in range(S)]
        cache = gpu.KVCache(gpu.KV_LLOYDMAX if lloyd else gpu.KV_UNIFORM, S, Hkv, d, max(lens) + 8, kb, vb, ks, vs)
        if not lloyd:
            cache.set_scales(1.0, 0.9)
        for s, L in enumerate(lens):
            cache.encode_append(randn(1, Hkv, L, d), randn(1, Hkv, L, d), seq_begin=s)
        q = randn(S, T, Hkv * G, d)
        out, ref = torch.zeros_like(q), torch.zeros_like(q)
        mapping = gpu.GQA_BLOCKED if rng.integers(2) else gpu.GQA_WEED
        cache.decode_attn_chunk(q, out, gqa_mapping=mapping)
        for t in range(T):
            lt = torch.tensor([L - (T - 1 - t) for L in lens], dtype=torch.int32, device="cuda")
            cache.decode_attn_prefix(lt, q[:, t], ref[:, t], gqa_mapping=mapping)
        gpu.sync()
        what = "case %d: d %d, K %d+%d V %d+%d bits, %d x %d heads, %d positions, lengths %s" % (
            case, d, kb, ks, vb, vs, Hkv, G, T, lens)
        assert not torch.isnan(out).any(), what
        assert (out - ref).abs().max().item() < 5e-5, what
        cache.close()
