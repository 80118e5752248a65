"""The decode entry point that allocates nothing (weed_hip_kv_decode_attn_noalloc) against weed_hip_kv_decode_attn.

Both run the same kernels with the same work partition, so their outputs must be identical bit for bit; the first is
also held to the attention tolerance against the CPU checker.  Two calls in a row share the library's static workspace,
the second with a smaller input, so stale contents of the first would show.
"""
import numpy as np
import pytest

from gpu_helpers import assert_attn_close, coder_specs, dev, export
from weed_amd import workloads

pytestmark = pytest.mark.gpu


def _cache(gpu, oracle, wl, seed):
    K, V, q = wl.tensors()
    rng = np.random.default_rng(seed)
    d = wl.head_dim
    Rk = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    Rv = oracle.orthonormalize_columns(rng.normal(size=d * d).astype(np.float32))
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, wl.n_seq, wl.n_kv_heads, d, wl.max_len, wl.k_bits, wl.v_bits, wl.k_sign,
                        wl.v_sign)
    cache.set_rotations(dev(Rk), dev(Rv))
    Kd, Vd = dev(K), dev(V)
    for s, L in enumerate(wl.lens):
        cache.encode_append(Kd[s:s + 1, :, :L], Vd[s:s + 1, :, :L], seq_begin=s, rotate=1)
    return cache, q, Rk, Rv


def _both(gpu, cache, q, flags):
    import torch
    qd = dev(q)
    ref = torch.zeros_like(qd)
    out = torch.full_like(qd, float("nan"))
    cache.decode_attn(qd, ref, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
    cache.decode_attn_noalloc(qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
    gpu.sync()
    return ref.cpu().numpy(), out.cpu().numpy()


def test_noalloc_matches_decode_attn_on_two_calls_in_a_row(gpu, oracle):
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    # first call: 6 ragged sequences, long enough for several context splits per region
    big = workloads.Workload("noalloc_a", 6, 16, 4, 128, [1500, 700, 2048, 64, 1, 999], 3, 4, 0, 0, 21)
    cache_a, q_a, Rk, Rv = _cache(gpu, oracle, big, 5)
    ref_a, out_a = _both(gpu, cache_a, q_a, flags)
    assert np.array_equal(ref_a, out_a), "first call differs from weed_hip_kv_decode_attn"
    kspec, vspec = coder_specs(oracle, cache_a)
    kf, ka = export(cache_a, 0, big.max_len)
    vf, va = export(cache_a, 1, big.max_len)
    want = oracle.decode_attn(kspec, vspec, kf, ka, vf, va, q_a, big.lens, gqa_weed=False, Rk=Rk, Rv=Rv)
    assert_attn_close(out_a, want, "noalloc first call vs checker")
    # second call, smaller in every dimension: it reuses the workspace the first one left behind
    small = workloads.Workload("noalloc_b", 2, 4, 2, 64, [130, 37], 2, 3, 1, 0, 22)
    cache_b, q_b, Rk2, Rv2 = _cache(gpu, oracle, small, 6)
    ref_b, out_b = _both(gpu, cache_b, q_b, flags)
    assert np.array_equal(ref_b, out_b), "second (smaller) call differs from weed_hip_kv_decode_attn"
    kspec, vspec = coder_specs(oracle, cache_b)
    kf, ka = export(cache_b, 0, small.max_len)
    vf, va = export(cache_b, 1, small.max_len)
    want = oracle.decode_attn(kspec, vspec, kf, ka, vf, va, q_b, small.lens, gqa_weed=False, Rk=Rk2, Rv=Rv2)
    assert_attn_close(out_b, want, "noalloc second call vs checker")
    # and the first shape again after the small one
    ref_c, out_c = _both(gpu, cache_a, q_a, flags)
    assert np.array_equal(ref_c, out_c) and np.array_equal(out_c, out_a)
    cache_a.close()
    cache_b.close()


def test_noalloc_head_dim_256_whole_regions_per_workgroup(gpu, oracle):
    """A batch of equal sequences at head_dim 256, which is one kernel (the workgroups rotate their queries and merge
    their partials themselves): the same bits from both entry points, and the checker's values."""
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    wl = workloads.Workload("noalloc_256", 4, 8, 2, 256, [1024] * 4, 3, 4, 0, 0, 23)
    cache, q, Rk, Rv = _cache(gpu, oracle, wl, 7)
    try:
        gpu.decode_tuning(32)
        ref, out = _both(gpu, cache, q, flags)
    finally:
        gpu.decode_tuning()
    assert np.array_equal(ref, out)
    kspec, vspec = coder_specs(oracle, cache)
    kf, ka = export(cache, 0, wl.max_len)
    vf, va = export(cache, 1, wl.max_len)
    want = oracle.decode_attn(kspec, vspec, kf, ka, vf, va, q, wl.lens, gqa_weed=False, Rk=Rk, Rv=Rv)
    assert_attn_close(out, want, "noalloc at head_dim 256 vs checker")
    cache.close()


def test_noalloc_refuses_shapes_beyond_its_workspace(gpu):
    import torch
    # 1024 sequences x 64 heads x 128: the rotated queries alone are 32 MiB, the size of the static workspace
    cache = gpu.KVCache(gpu.KV_LLOYDMAX, 1024, 4, 128, 64, 3, 4)
    K = torch.randn((1024, 4, 64, 128), device="cuda")
    cache.encode_append(K, K)
    q = torch.randn((1024, 64, 128), device="cuda")
    out = torch.zeros_like(q)
    with pytest.raises(gpu.WeedHipError) as err:
        cache.decode_attn_noalloc(q, out, gqa_mapping=gpu.GQA_BLOCKED, flags=0)
    assert err.value.code == gpu.EINVAL and "static scratch" in str(err.value)
    cache.decode_attn(q, out, gqa_mapping=gpu.GQA_BLOCKED, flags=0)  # the allocating entry point takes it
    gpu.sync()
    assert bool(torch.isfinite(out).all())
    cache.close()


@pytest.mark.parametrize("n_seq,ctx", [(1, 2048), (8, 1024), (3, 1000)])
def test_noalloc_call_replayed_from_a_graph(gpu, oracle, n_seq, ctx):
    """The allocation-free entry point under graph capture: the captured call is one kernel whose workgroups count
    their arrivals per region and leave the counters at zero, so every replay must give the bits of the eager call,
    also with eager calls of another shape in between."""
    import torch
    flags = gpu.ATTN_ROTATE_Q | gpu.ATTN_UNROTATE_OUT
    wl = workloads.Workload("graph", n_seq, 8, 2, 128, [ctx] * n_seq, 3, 4, 0, 0, 31)
    cache, q, _, _ = _cache(gpu, oracle, wl, 9)
    other = workloads.Workload("graph_b", 2, 4, 2, 64, [130, 37], 2, 3, 1, 0, 32)
    cache_b, q_b, _, _ = _cache(gpu, oracle, other, 10)
    qd, qb = dev(q), dev(q_b)
    eager = torch.zeros_like(qd)
    cache.decode_attn_noalloc(qd, eager, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
    gpu.sync()
    out = torch.full_like(qd, float("nan"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.current_stream()):
        cache.decode_attn_noalloc(qd, out, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
    for _ in range(4):
        out.fill_(float("nan"))
        graph.replay()
        gpu.sync()
        assert np.array_equal(out.cpu().numpy(), eager.cpu().numpy())
        ob = torch.zeros_like(qb)
        cache_b.decode_attn_noalloc(qb, ob, gqa_mapping=gpu.GQA_BLOCKED, flags=flags)
        gpu.sync()
    cache.close()
    cache_b.close()
