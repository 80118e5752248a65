#!/usr/bin/env python3
"""Benchmark of fused quantized-KV decode attention on one MI355X.

One "step" = one decode step (one new token per sequence) of the Qwen-style GQA configuration -- 32 query heads,
8 kv heads, head_dim 128, ctx 8192, keys 3-bit, values 4-bit Lloyd-Max codes with an fp32 row scale -- over
`--seqs` independent sequence caches held side by side (default 64 = 0.5 GB of packed cache, more than the 256 MB
Infinity Cache, so the timed reads come from HBM).  Inputs are synthetic and already resident in HBM.

Prints ONE JSON line: tokens/s (whole job), the HBM roofline of the dominant kernel measured with HIP events on the
launch stream, and the CPU checker (a scalar restatement of the reference's path) timed on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def build_cache(capi, torch, wl, seed):
    """Encode `wl.n_seq` sequences of synthetic K/V (N(0,1), 1 % of channels x10) generated on the device."""
    d = wl.head_dim
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    rk = torch.zeros(d * d, device="cuda")
    rv = torch.zeros(d * d, device="cuda")
    capi.make_rotation(seed + 1, d, rk)
    capi.make_rotation(seed + 2, d, rv)
    cache = capi.KVCache(capi.KV_LLOYDMAX, wl.n_seq, wl.n_kv_heads, d, wl.max_len, wl.k_bits, wl.v_bits, wl.k_sign,
                         wl.v_sign)
    cache.set_rotations(rk, rv)
    n_out = max(1, d // 100)
    ch = torch.randperm(d, generator=gen, device="cuda")[:n_out]
    for s, L in enumerate(wl.lens):
        K = torch.randn((1, wl.n_kv_heads, L, d), generator=gen, device="cuda")
        V = torch.randn((1, wl.n_kv_heads, L, d), generator=gen, device="cuda")
        K[..., ch] *= 10.0
        V[..., ch] *= 10.0
        cache.encode_append(K, V, seq_begin=s, rotate=1)
    q = torch.randn((wl.n_seq, wl.n_q_heads, d), generator=gen, device="cuda")
    return cache, q, rk, rv


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def host_threads():
    """Threads for the all-cores legs: the cores this process may run on, at most 16 (a GPU box's CPU share)."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return max(1, min(16, n))


def run_threads(n, fn):
    """fn(thread index) on n host threads (the checker's C functions release the interpreter lock); wall seconds."""
    import threading
    threads = [threading.Thread(target=fn, args=(i,)) for i in range(n)]
    t0 = time.perf_counter()
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    return time.perf_counter() - t0


def cpu_other_legs(np, n_threads):
    """CPU legs of configurations 5a and 5b on bounded samples (a few seconds each)."""
    from oracle import oracle as orc
    out = {}
    rng = np.random.default_rng(5)
    d = 128
    # 5a: rotation (naive product, multihead_attention.cpp:206-207 -> matmul.cpp:34-47) and the row coder
    # (write_row loop, multihead_attention.cpp:244-257) over a sample of the 2 x 32768 rows, one core
    rows = 2048
    X = rng.standard_normal((rows, d), dtype=np.float32)
    R = orc.orthonormalize_columns(rng.standard_normal(d * d).astype(np.float32))
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 3.0:
        Y = orc.apply_rotation(X, R)
        orc.uniform_write_rows(Y, 3, 1.0)
        reps += 1
    secs = time.perf_counter() - t0
    # one token = 8 kv heads x (K row + V row) = 16 rows
    out["cfg5a_encode"] = {
        "value": reps * rows / 16.0 / secs, "unit": "tokens/s", "cores": 1, "kind": "port",
        "sample": "%d x %d rows of 128 (of the 65536 rows of K and V of 4096 tokens x 8 heads): naive rotation "
                  "product + write_row at 3 bits, %.1f s" % (reps, rows, secs)}
    # 5b: naive fp32 product with sequential-k accumulation (matmul.cpp:34-47), column-major operands; the reference
    # splits the 2^24 outputs over min(cores, 64) workers, so: a slab of rows per host thread
    M, K, N = 4096, 1024, 4096
    m_per = 32
    A = rng.standard_normal(M * K).astype(np.float32)   # column-major [M, K]: element (i, k) at i + M*k
    B = rng.standard_normal(K * N).astype(np.float32)   # column-major [K, N]
    C = np.zeros(M * N, dtype=np.float32)

    def slab(i):
        orc.matmul(m_per, N, K, A, (i * m_per, 1, M), B, (0, 1, K), C, (i * m_per, 1, M))

    secs = run_threads(n_threads, slab)
    flops = 2.0 * n_threads * m_per * N * K
    out["cfg5b_matmul"] = {
        "value": flops / secs / 1e9, "unit": "GFLOP/s", "cores": n_threads, "kind": "port",
        "sample": "%d of the 4096 output rows (%d per host thread), naive product with k ascending, %.1f s"
                  % (n_threads * m_per, m_per, secs)}
    return out


def cpu_baseline(capi, torch, cache, wl, q, rk, rv, budget_s=10.0, n_threads=1):
    """Time the CPU checker (reference cost structure) on one sequence of the same workload: one core (the
    reference's own policy at this shape: workers = min(cores, items / 2^18) = 1, parallel_for.cpp:91-106), then one
    sequence per host thread on all cores."""
    from oracle import oracle as orc
    d = wl.head_dim
    L = wl.lens[0]
    fields, scales = [], []
    for which in (0, 1):
        f = torch.empty((1, wl.n_kv_heads, L, d), dtype=torch.uint8, device="cuda")
        a = torch.zeros((1, wl.n_kv_heads, L), device="cuda")
        cache.export_fields(which, f, a)
        fields.append(f.cpu().numpy())
        scales.append(a.cpu().numpy())
    specs = []
    for which in (0, 1):
        bounds, levels, recon = cache.get_tables(which)
        specs.append(orc.CoderSpec(1, d, wl.v_bits if which else wl.k_bits, sign=wl.v_sign if which else wl.k_sign,
                                   bounds=bounds, levels=levels, recon=recon))
    qh = q[0:1].cpu().numpy()
    rkh, rvh = rk.cpu().numpy(), rv.cpu().numpy()
    steps, t0 = 0, time.perf_counter()
    out = None
    while True:
        out = orc.decode_attn(specs[0], specs[1], fields[0], scales[0], fields[1], scales[1], qh, [L], gqa_weed=False,
                              Rk=rkh, Rv=rvh)
        steps += 1
        elapsed = time.perf_counter() - t0
        if elapsed >= budget_s or steps >= 200:
            break
    # all cores: every host thread decodes the same sequence `per_thread` times (independent sequences in effect)
    per_thread = max(1, int(round(0.5 * budget_s * steps / elapsed)))

    def many(_):
        for _i in range(per_thread):
            orc.decode_attn(specs[0], specs[1], fields[0], scales[0], fields[1], scales[1], qh, [L], gqa_weed=False,
                            Rk=rkh, Rv=rvh)

    all_secs = run_threads(n_threads, many) if n_threads > 1 else elapsed * per_thread / steps
    all_cores = {"value": n_threads * per_thread / all_secs, "unit": "tokens/s", "cores": n_threads,
                 "sample": "%d decode steps of one sequence on each of %d host threads in %.1f s"
                           % (per_thread, n_threads, all_secs)}
    return steps / elapsed, steps, elapsed, out, all_cores


def time_calls(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_region(torch, fn, steps, warmup):
    """Seconds per call on the device: two events on the launch stream around `steps` back-to-back calls."""
    for _ in range(warmup):
        fn()
    stream = torch.cuda.current_stream()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record(stream)
    for _ in range(steps):
        fn()
    ev1.record(stream)
    ev1.synchronize()
    return 1e-3 * ev0.elapsed_time(ev1) / steps


def time_one_kernel_op(capi, torch, fn, name, steps, warmup):
    """(seconds per call, seconds per launch, how the latter was taken) for an op that is one kernel per call: the
    launch duration is the device time of a run of back-to-back calls divided by their number, as for the headline
    (an event pair around every single launch adds the events' own 2-3 us to a kernel of a few dozen); an op that
    turns out to take several launches per call keeps the event pairs."""
    secs, pair_s = time_kernel(capi, torch, fn, name, steps, warmup)
    launches = capi.profile_read(name)[1]
    note = {"kernel_ms_event_pair_per_launch": 1e3 * pair_s}
    if launches == steps:
        note["kernel_ms_source"] = "device time of %d back-to-back calls (one kernel each) between two events, divided by their number" % steps
        return secs, time_region(torch, fn, steps, warmup), note
    note["kernel_ms_source"] = "event pairs around the launches"
    return secs, pair_s, note


def time_kernel(capi, torch, fn, name, steps, warmup):
    """(seconds per call, seconds per launch of the kernel recorded under `name`): one untimed call first, so that
    one-off work of a shape's first launch (workspace growth, kernel attributes) stays out of both figures."""
    fn()
    torch.cuda.synchronize()
    secs = time_calls(torch, fn, steps, warmup)  # (without the event pairs around the kernels)
    capi.profile_reset()
    capi.profile_enable(True)
    time_calls(torch, fn, steps, 0)
    k_ms, k_n = capi.profile_read(name)
    capi.profile_enable(False)
    return secs, 1e-3 * k_ms / max(1, k_n)


def decode_entry(capi, torch, fn, n_seq, nbytes, steps, warmup):
    """One decode-attention configuration: step and kernel time, the kernel's roofline, and -- when the call is one
    kernel (it rotated its queries and merged its partials itself) -- the same call as three kernels beside it."""
    secs, kernel_s = time_kernel(capi, torch, fn, "kv_decode_attn", steps, warmup)
    one_kernel = capi.profile_read("kv_decode_combine")[1] == 0
    pair_s = kernel_s
    if one_kernel:
        # the call is that kernel: its launch duration is the device time of a run of calls divided by their number,
        # as for the headline
        kernel_s = time_region(torch, fn, steps, warmup)
    entry = {"tokens_per_s": n_seq / secs, "ms_per_step": 1e3 * secs, "packed_cache_bytes": nbytes,
             "kernel_ms": 1e3 * kernel_s, "kernel_ms_event_pair_per_launch": 1e3 * pair_s,
             "kernels_per_step": 1 if one_kernel else 3,
             "step_frac": nbytes / secs / 1e9 / HBM_PEAK_GBS,
             "roofline": {"bound": "hbm", "achieved": nbytes / kernel_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": nbytes / kernel_s / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes_per_launch": nbytes}}
    if one_kernel:
        capi.decode_tuning(separate_merge=True, separate_query=True)
        try:
            secs3, kernel3_s = time_kernel(capi, torch, fn, "kv_decode_attn", steps, warmup)
        finally:
            capi.decode_tuning()
        entry["same_step_as_three_kernels"] = {"ms_per_step": 1e3 * secs3, "attention_kernel_ms": 1e3 * kernel3_s,
                                               "attention_kernel_frac": nbytes / kernel3_s / 1e9 / HBM_PEAK_GBS}
    return entry


def extras(capi, torch, workloads, steps, warmup):
    """The other configurations, measured the same way (reported beside the headline, not as `value`)."""
    out = {}
    # configuration 5b: [4096 x 1024] . [1024 x 4096] fp32, column-major operands as Weed passes them
    A = torch.randn((1024, 4096), device="cuda").t()           # logical [4096, 1024], column-major
    W = (torch.randn((4096, 1024), device="cuda") * 0.02).t()  # logical [1024, 4096], column-major
    C = torch.empty((4096, 4096), device="cuda").t()
    secs, kernel_s, how = time_one_kernel_op(capi, torch, lambda: capi.matmul(A, W, C), "matmul", steps, warmup)
    flops = 2.0 * 4096 * 1024 * 4096
    out["cfg5b_matmul_f32_4096x1024x4096"] = {
        "tflops": flops / secs / 1e12, "kernel_ms": 1e3 * kernel_s, "kernel_tflops": flops / kernel_s / 1e12,
        "roofline": {"bound": "mfma", "achieved": flops / kernel_s / 1e12, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": flops / kernel_s / 1e12 / 157.3}}
    out["cfg5b_matmul_f32_4096x1024x4096"].update(how)
    del A, W, C
    # decode-time projection y = x.W: 8 rows against a [4096 x 4096] column-major weight (64 MiB streamed per call)
    X = torch.randn((4096, 8), device="cuda").t()               # logical [8, 4096], column-major
    Wp = (torch.randn((4096, 4096), device="cuda") * 0.02).t()  # logical [4096, 4096], column-major
    Y = torch.empty((4096, 8), device="cuda").t()
    secs, kernel_s, how = time_one_kernel_op(capi, torch, lambda: capi.matmul(X, Wp, Y), "matmul", steps, warmup)
    wbytes = 4096 * 4096 * 4
    out["projection_8x4096x4096"] = {
        "ms": 1e3 * secs, "kernel_ms": 1e3 * kernel_s,
        "roofline": {"bound": "hbm", "achieved": wbytes / kernel_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": wbytes / kernel_s / 1e9 / HBM_PEAK_GBS}}
    out["projection_8x4096x4096"].update(how)
    del X, Wp, Y
    # standalone softmax and sum over an [8192 x 8192] column-major matrix (256 MiB), along the contiguous axis and
    # along the strided one: 8 B per element (softmax) and 4 B per element (sum) of algorithmic traffic
    S = torch.randn((8192, 8192), device="cuda").t()
    So = torch.empty((8192, 8192), device="cuda").t()
    Sr = torch.empty(8192, device="cuda")
    dense = {}
    for axis, name in ((0, "contiguous_axis"), (1, "strided_axis")):
        for op, fn, bytes_per in (("softmax", lambda: capi.softmax(S, So, axis), 8),
                                  ("reduce", lambda: capi.reduce(capi.REDUCE_SUM, S, Sr, axis), 4)):
            _, kernel_s, how = time_one_kernel_op(capi, torch, fn, op, steps, warmup)
            gbs = S.numel() * bytes_per / kernel_s / 1e9
            dense["%s_%s" % (op, name)] = {"kernel_ms": 1e3 * kernel_s,
                                           "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS,
                                                        "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}}
            dense["%s_%s" % (op, name)].update(how)
    out["softmax_sum_f32_8192x8192"] = dense
    del S, So, Sr
    # configuration 5a: encode-and-append 4096 tokens x 8 kv heads x 128, 3-bit codes (rotate, quantise, pack)
    wl = workloads.config(5)
    d = wl.head_dim
    cache = capi.KVCache(capi.KV_LLOYDMAX, 1, wl.n_kv_heads, d, 4096, 3, 3)
    rk = torch.zeros(d * d, device="cuda")
    rv = torch.zeros(d * d, device="cuda")
    capi.make_rotation(5, d, rk)
    capi.make_rotation(6, d, rv)
    cache.set_rotations(rk, rv)
    K = torch.randn((1, wl.n_kv_heads, 4096, d), device="cuda")
    V = torch.randn((1, wl.n_kv_heads, 4096, d), device="cuda")

    def enc():
        cache.reset()
        cache.encode_append(K, V, rotate=1)

    secs, kernel_s = time_kernel(capi, torch, enc, "kv_encode", steps, warmup)
    in_bytes = 2 * K.numel() * 4
    rot_flops = 2 * 2.0 * K.numel() * d  # K and V: rows x 2 d^2
    out["cfg5a_encode_4096x8x128_3bit"] = {
        "tokens_per_s": 4096 / secs, "ms": 1e3 * secs, "input_gbs": in_bytes / secs / 1e9,
        "rotation_tflops": rot_flops / secs / 1e12, "kernel_ms": 1e3 * kernel_s,
        "roofline": {"bound": "mfma", "achieved": rot_flops / kernel_s / 1e12, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": rot_flops / kernel_s / 1e12 / 157.3, "kernel": "encode_rows_pair_kernel (K and V)",
                     "flops_per_launch": rot_flops},
        "kernel_ms_source": "event pairs around the launches (the call also resets the cache and moves the lengths, so "
                            "a run of calls does not time the kernel alone; the events' own 2-3 us are in the figure)"}
    cache.close()
    # the append of a decode step: one new token for each of 64 sequences (one launch: the encoder writes the items
    # and moves the lengths itself)
    n_app = 1 + 2 * warmup + 3 * steps
    cache1 = capi.KVCache(capi.KV_LLOYDMAX, 64, wl.n_kv_heads, d, n_app, 3, 3, 1, 0)
    cache1.set_rotations(rk, rv)
    k1 = torch.randn((64, wl.n_kv_heads, 1, d), device="cuda")
    v1 = torch.randn((64, wl.n_kv_heads, 1, d), device="cuda")
    secs, kernel_s, how = time_one_kernel_op(capi, torch, lambda: cache1.encode_append(k1, v1, rotate=1), "kv_encode",
                                             steps, warmup)
    out["append_one_token_64_sequences"] = {"ms": 1e3 * secs, "kernel_ms": 1e3 * kernel_s, "kernels_per_append": 1,
                                            "rows": 2 * 64 * wl.n_kv_heads}
    out["append_one_token_64_sequences"].update(how)
    cache1.close()
    # configuration 4: 16 ragged sequences in [2048, 32768], K 2-bit + sign, V 3-bit, split-context merge
    wl4 = workloads.config(4)
    cache4 = capi.KVCache(capi.KV_LLOYDMAX, wl4.n_seq, wl4.n_kv_heads, d, wl4.max_len, wl4.k_bits, wl4.v_bits,
                          wl4.k_sign, wl4.v_sign)
    for s, L in enumerate(wl4.lens):
        Ks = torch.randn((1, wl4.n_kv_heads, L, d), device="cuda")
        Vs = torch.randn((1, wl4.n_kv_heads, L, d), device="cuda")
        cache4.encode_append(Ks, Vs, seq_begin=s)
    for hq in (8, 32):
        q = torch.randn((wl4.n_seq, hq, d), device="cuda")
        o = torch.zeros_like(q)
        out["cfg4_ragged16_hq%d" % hq] = decode_entry(
            capi, torch, lambda: cache4.decode_attn(q, o, capi.GQA_BLOCKED, 0), wl4.n_seq, wl4.bytes_per_step(True),
            steps, warmup)
    cache4.close()
    # Weed's own uniform coder at kv_quant_bits = 8 on the headline shape (64 x 8192 tokens x 8 heads, 256 B per token
    # and head): the matrix-core kernel with arithmetic de-quantisation instead of tables
    wl8 = workloads.config(3, n_seq=64)
    cache8 = capi.KVCache(capi.KV_UNIFORM, wl8.n_seq, wl8.n_kv_heads, d, wl8.max_len, 8, 8)
    cache8.set_scales(1.0, 1.0)
    for s0 in range(0, wl8.n_seq, 8):
        Ks = torch.randn((8, wl8.n_kv_heads, wl8.max_len, d), device="cuda")
        Vs = torch.randn((8, wl8.n_kv_heads, wl8.max_len, d), device="cuda")
        cache8.encode_append(Ks, Vs, seq_begin=s0)
    del Ks, Vs
    q8 = torch.randn((wl8.n_seq, wl8.n_q_heads, d), device="cuda")
    o8 = torch.zeros_like(q8)
    out["uniform_8bit_64_sequences"] = decode_entry(
        capi, torch, lambda: cache8.decode_attn(q8, o8, capi.GQA_BLOCKED, 0), wl8.n_seq,
        sum(wl8.lens) * wl8.n_kv_heads * 2 * d, steps, warmup)
    cache8.close()
    del q8, o8
    # a decode loop as a server runs it on the headline shape: one new token for each of the 64 sequences, then the
    # attention over everything cached (two launches per step), the contexts growing towards 8192 through every
    # residue of the 64-token blocks
    wlL = workloads.config(3, n_seq=64)
    n_loop = warmup + steps
    cacheL = capi.KVCache(capi.KV_LLOYDMAX, wlL.n_seq, wlL.n_kv_heads, d, wlL.max_len, wlL.k_bits, wlL.v_bits,
                          wlL.k_sign, wlL.v_sign)
    cacheL.set_rotations(rk, rv)
    for s0 in range(0, wlL.n_seq, 8):
        Ks = torch.randn((8, wlL.n_kv_heads, wlL.max_len - n_loop, d), device="cuda")
        Vs = torch.randn((8, wlL.n_kv_heads, wlL.max_len - n_loop, d), device="cuda")
        cacheL.encode_append(Ks, Vs, seq_begin=s0, rotate=1)
    del Ks, Vs
    qL = torch.randn((wlL.n_seq, wlL.n_q_heads, d), device="cuda")
    oL = torch.zeros_like(qL)
    kL = torch.randn((wlL.n_seq, wlL.n_kv_heads, 1, d), device="cuda")
    vL = torch.randn((wlL.n_seq, wlL.n_kv_heads, 1, d), device="cuda")
    flagsL = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT

    def loop_step():
        cacheL.encode_append(kL, vL, rotate=1)
        cacheL.decode_attn(qL, oL, capi.GQA_BLOCKED, flagsL)

    secs = time_calls(torch, loop_step, steps, warmup)
    out["decode_loop_64_sequences_towards_ctx8192"] = {"ms_per_step": 1e3 * secs, "tokens_per_s": wlL.n_seq / secs,
                                                       "launches_per_step": 2,
                                                       "ctx_from": wlL.max_len - steps, "ctx_to": wlL.max_len}
    cacheL.close()
    del qL, oL, kL, vL
    # the headline shape with 64 sequences of different lengths, drawn uniformly from [4096, 8192] (seeded): what a
    # serving batch looks like; the partition counts every sequence as the longest one
    import random
    rnd = random.Random(4096)
    lens_r = [rnd.randint(4096, 8192) for _ in range(64)]
    wlR = workloads.Workload("cfg3_ragged", 64, wlL.n_q_heads, wlL.n_kv_heads, d, lens_r, wlL.k_bits, wlL.v_bits,
                             wlL.k_sign, wlL.v_sign, 0)
    cacheR = capi.KVCache(capi.KV_LLOYDMAX, 64, wlR.n_kv_heads, d, 8192, wlR.k_bits, wlR.v_bits, wlR.k_sign, wlR.v_sign)
    cacheR.set_rotations(rk, rv)
    for s0, n in enumerate(lens_r):
        Ks = torch.randn((1, wlR.n_kv_heads, n, d), device="cuda")
        Vs = torch.randn((1, wlR.n_kv_heads, n, d), device="cuda")
        cacheR.encode_append(Ks, Vs, seq_begin=s0, rotate=1)
    del Ks, Vs
    qR = torch.randn((64, wlR.n_q_heads, d), device="cuda")
    oR = torch.zeros_like(qR)
    out["cfg3_64_sequences_of_4096_to_8192_tokens"] = decode_entry(
        capi, torch, lambda: cacheR.decode_attn(qR, oR, capi.GQA_BLOCKED, flagsL), 64, wlR.bytes_per_step(lloydmax=True),
        steps, warmup)
    cacheR.close()
    del qR, oR
    # configuration 3 again with 256 sequence caches per launch (2 GB of packed rows): what the per-launch fixed cost
    # (launch, table build, first-block latency, uneven finish) amortises to with four times the bytes
    wl3 = workloads.config(3, n_seq=256)
    cache3, q3, _, _ = build_cache(capi, torch, wl3, seed=77)
    o3 = torch.zeros_like(q3)
    flags = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT
    out["cfg3_256_sequences"] = decode_entry(
        capi, torch, lambda: cache3.decode_attn(q3, o3, capi.GQA_BLOCKED, flags), wl3.n_seq,
        wl3.bytes_per_step(lloydmax=True), steps, warmup)
    cache3.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (a burst of a few dozen launches falls into the clock transient that follows the start of sustained load; a
    # thousand steps are a tenth of a second and show the steady state)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--seqs", type=int, default=64, help="independent ctx-8192 sequence caches per launch")
    ap.add_argument("--ctx", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations (4, 5a, 5b)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="only launch the library's plain copy kernel on MIB mebibytes (5 launches): the known-size "
                         "reference against which rocprofv3's FETCH_SIZE / WRITE_SIZE readings are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path is sharded by (sequence, kv head) with no "
              "exchange between GPUs); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from weed_amd import capi, workloads

    lib = capi.load()  # raises if the HIP library is missing: there is no fallback path
    capi.check(lib.weed_hip_init(0))
    stream = torch.cuda.Stream()
    capi.use_torch_stream(stream)
    if args.calibrate_copy:
        with torch.cuda.stream(stream):
            n = args.calibrate_copy * (1 << 20) // 4
            src = torch.ones(n, device="cuda")
            dst = torch.empty(n, device="cuda")
            for _ in range(5):
                capi.copy(src, dst)
            torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": 4 * n, "calibrate_copy_bytes_written": 4 * n, "launches": 5}))
        return
    with torch.cuda.stream(stream):
        wl = workloads.config(3, n_seq=args.seqs, scale=args.ctx / 8192.0)
        cache, q, rk, rv = build_cache(capi, torch, wl, seed=1234)
        out = torch.zeros_like(q)
        flags = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT

        def step():
            cache.decode_attn(q, out, capi.GQA_BLOCKED, flags)

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        # (two HIP events on the launch stream around the timed region, beside the host clock)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record(stream)
        for _ in range(args.steps):
            step()
        ev1.record(stream)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        ms_per_step = 1e3 * elapsed / args.steps
        tokens_per_s = wl.n_seq * args.steps / elapsed
        region_ms_per_step = ev0.elapsed_time(ev1) / args.steps

        # dominant kernel alone: HIP events recorded by the library around its launch, on the launch stream
        capi.profile_reset()
        capi.profile_enable(True)
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        k_ms, k_n = capi.profile_read("kv_decode_attn")
        c_ms, c_n = capi.profile_read("kv_decode_combine")
        capi.profile_enable(False)
        pair_ms = k_ms / max(1, k_n)
        one_kernel = c_n == 0  # the matrix-core kernel rotated the queries and merged its partials itself
        # When the step is that one kernel, its average launch duration is what the two events around the timed region
        # give per step (launch gaps included); an event pair around every launch adds its own 1-2 us to each.
        kernel_ms = region_ms_per_step if one_kernel else pair_ms
        bytes_per_launch = wl.bytes_per_step(lloydmax=True)
        achieved = bytes_per_launch / (kernel_ms * 1e-3) / 1e9

        # the same step as three kernels (query rotation, attention, merge), for comparison
        separate = None
        if one_kernel:
            capi.decode_tuning(separate_merge=True, separate_query=True)
            try:
                for _ in range(args.warmup):
                    step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    step()
                torch.cuda.synchronize()
                sep_ms = 1e3 * (time.perf_counter() - t0) / args.steps
                capi.profile_reset()
                capi.profile_enable(True)
                for _ in range(args.steps):
                    step()
                torch.cuda.synchronize()
                sk_ms, sk_n = capi.profile_read("kv_decode_attn")
                sc_ms, sc_n = capi.profile_read("kv_decode_combine")
                capi.profile_enable(False)
            finally:
                capi.decode_tuning()
            separate = {"ms_per_step": sep_ms, "attention_kernel_ms": sk_ms / max(1, sk_n),
                        "attention_kernel_frac": bytes_per_launch / (sk_ms / max(1, sk_n) * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "merge_kernel_ms": sc_ms / max(1, sc_n)}

        # batch = 1 latency of the same shape (one sequence per launch: launch-latency bound); part of the extras, so
        # that a --no-extras run launches the main kernel at the headline shape only
        wl1 = workloads.config(3, n_seq=1, scale=args.ctx / 8192.0)
        single_ms = None
        if not args.no_extras:
            cache1, q1, _, _ = build_cache(capi, torch, wl1, seed=99)
            out1 = torch.zeros_like(q1)
            for _ in range(args.warmup):
                cache1.decode_attn(q1, out1, capi.GQA_BLOCKED, flags)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                cache1.decode_attn(q1, out1, capi.GQA_BLOCKED, flags)
            torch.cuda.synchronize()
            single_ms = 1e3 * (time.perf_counter() - t0) / args.steps
            cache1.close()

        # HBM bytes per launch measured with rocprofv3 counters (scaled by a copy kernel of known size); the committed
        # summary applies to one workload shape only
        traffic = None
        traffic_file = os.path.join(ROOT, "profiles", "kv_decode_attn_cfg3x64_hbm_traffic.txt")
        if os.path.exists(traffic_file):
            t = {}
            with open(traffic_file) as f:
                for line in f:
                    key, sep, val = line.partition(":")
                    if sep and val.strip().isdigit():
                        t[key.strip()] = int(val)
            if t.get("seqs") == args.seqs and t.get("ctx") == args.ctx:
                traffic = t.get("hbm_bytes_per_launch")
        traffic_source = ("replayed from profiles/%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, "
                          "scaled by a copy kernel of known size); not measured in this run"
                          % os.path.basename(traffic_file)) if traffic is not None else None

        result = {
            "metric": "quantized-KV decode attn tokens/sec + HBM GB/s (% roofline) at ctx 8192",
            "value": tokens_per_s,
            "unit": "tokens/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": ms_per_step,
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "f32",
            "data": "synthetic",
            "config": {
                "workload": "cfg3 Qwen-style GQA decode: 32 q / 8 kv heads, head_dim 128, ctx %d, K 3-bit + V 4-bit "
                            "Lloyd-Max codes + fp32 row scale, %d independent sequence caches per launch "
                            "(1 new token each), split-context" % (args.ctx, wl.n_seq),
                "n_seq": wl.n_seq, "ctx": args.ctx, "n_q_heads": wl.n_q_heads, "n_kv_heads": wl.n_kv_heads,
                "head_dim": wl.head_dim, "k_bits": wl.k_bits, "v_bits": wl.v_bits,
                "packed_cache_bytes": bytes_per_launch,
            },
            "roofline": {
                "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                "kernel": ("decode attention kernel; the only kernel of the step: it rotates the queries and merges "
                           "its partials itself") if one_kernel else "decode attention main kernel",
                "kernels_per_step": 1 if one_kernel else 3,
                "kernel_ms": kernel_ms,
                "kernel_ms_source": ("HIP events on the launch stream around the %d back-to-back launches of the timed "
                                     "region, divided by their number" % args.steps) if one_kernel else
                                    "HIP event pairs recorded by the library around each launch",
                "kernel_ms_event_pair_per_launch": pair_ms,
                "algorithmic_bytes_per_launch": bytes_per_launch,
                "combine_kernel_ms": c_ms / max(1, c_n),
                "same_step_as_three_kernels": separate,
            },
            "whole_step_gbs": bytes_per_launch / (ms_per_step * 1e-3) / 1e9,
        }
        if not args.no_extras:
            # a chunk of 4 query positions per sequence in one pass over the same caches (speculative decoding)
            S_, Hq_, d_ = q.shape
            qc = torch.randn((S_, 4, Hq_, d_), device="cuda")
            oc = torch.zeros_like(qc)
            chunk_s = time_calls(torch, lambda: cache.decode_attn_chunk(qc, oc, None, capi.GQA_BLOCKED, flags),
                                 min(args.steps, 20), min(args.warmup, 3))
            result["chunk_of_4_positions"] = {"ms_per_call": 1e3 * chunk_s, "positions_per_s": 4 * wl.n_seq / chunk_s,
                                              "vs_4_single_position_calls": 4 * ms_per_step * 1e-3 / chunk_s}
            del qc, oc
        if single_ms is not None:
            result["single_sequence"] = {"ms_per_step": single_ms, "tokens_per_s": 1e3 / single_ms,
                                         "gbs": wl1.bytes_per_step(True) / (single_ms * 1e-3) / 1e9}
        if not args.no_cpu_baseline:
            n_threads = host_threads()
            tps, n, secs, cpu_out, all_cores = cpu_baseline(capi, torch, cache, wl, q, rk, rv, n_threads=n_threads)
            got = out[0:1].cpu().numpy()
            err = float(np.abs(got - cpu_out).max())
            all_cores["gbs"] = wl1.bytes_per_step(True) * all_cores["value"] / 1e9
            result["cpu_baseline"] = {
                "value": tps, "unit": "tokens/s", "cores": 1, "kind": "port",
                "cpu_model": cpu_model(), "host_threads_available": n_threads,
                "threading": "one core is the reference's own policy at this shape: workers = min(cores, items / 2^18)",
                "all_cores": all_cores,
                "other_configs": cpu_other_legs(np, n_threads),
                "sample": "%d decode steps of ONE of the %d sequences (same shape, ctx %d) in %.1f s; scalar C "
                          "restatement of the reference's path: full dequantise, GQA replicate, K^T copy, naive dots, "
                          "divide, 3-pass softmax" % (n, wl.n_seq, args.ctx, secs),
                "gbs": wl1.bytes_per_step(True) * tps / 1e9,
                "max_abs_diff_vs_gpu": err,
            }
        cache.close()
        if not args.no_extras:
            # (short kernels need their own warm-up: after an idle stretch the first dozens of launches run at a lower
            # clock, 5 us slower on a 50 us kernel)
            result["other_configs"] = extras(capi, torch, workloads, min(args.steps, 200), max(args.warmup, 50))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
