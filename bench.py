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
# Launches that run ahead of every timed region whatever --warmup says: the first dozens of launches after an idle
# stretch sit in a clock transient (a burst of 25 launches of the headline kernel reads 3-4 % slower than a thousand).
WARMUP_FLOOR_HEADLINE = 150
WARMUP_FLOOR_EXTRA = 50


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


def streaming_read(capi, torch, nbytes, steps, warmup):
    """What merely reading `nbytes` costs on this part: a buffer of that size swept by the library's read-only kernel,
    in the decode kernel's launch shape (one contiguous run per wavefront) and as a plain sweep; ms per launch from two
    events around `steps` back-to-back launches."""
    buf = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device="cuda")
    buf.fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    runs_s = time_region(torch, lambda: capi.read_sweep(buf, nbytes, 1, sink), steps, warmup)
    sweep_s = time_region(torch, lambda: capi.read_sweep(buf, nbytes, 0, sink), steps, warmup)
    del buf
    return {"bytes": nbytes, "per_wavefront_runs_ms": 1e3 * runs_s, "per_wavefront_runs_gbs": nbytes / runs_s / 1e9,
            "plain_sweep_ms": 1e3 * sweep_s, "plain_sweep_gbs": nbytes / sweep_s / 1e9, "launches": steps,
            "kernel": "weed_hip_read_sweep: 16-byte loads, nothing written; 256 workgroups x 8 wavefronts with one "
                      "contiguous run each (the decode kernel's shape), and the same wavefronts taking the 8 KB units in turns"}


def layer_decode_step(capi, torch, np, n_calls, n_seq=64, ctx=8192, d_model=4096, n_heads=32, n_kv=8, d_ff=14336,
                      side_by_side=False, n_tokens=1):
    """One decode step of one Qwen-style decoder layer (include/modules/qwen_decoder_layer.hpp:104-115) through the C
    ABI, launch for launch what the host mirror's QwenDecoderLayer::forward issues for a (B, 1, d_model) input:
    RMSNorm, the Q / K / V projections (with bias), RoPE on Q and K at position ctx, append, fused attention over the
    packed cache, the output projection, residual, RMSNorm, gate / up projections, SiLU gate, down projection,
    residual.  Activations are column-major (batch index fastest) as Weed lays them out; weights are random.  The
    cache starts n_calls tokens short of ctx and every call of the returned step appends one token per sequence.
    side_by_side: the weights of Q, K, V lie side by side in one buffer, and so do gate and up, as after the host
    mirror's fuse_projections(); the projections that share their input are then one product each (13 launches).
    n_tokens > 1: a prefill chunk instead, (B, n_tokens, d_model): the same launches over B * n_tokens rows, every call
    appends n_tokens per sequence and attends with the chunk's causal mask over the packed cache."""
    B, D, H, Hkv, hd = n_seq, d_model, n_heads, n_kv, d_model // n_heads
    T, R = n_tokens, n_seq * n_tokens  # rows of an activation: r = b + B * t (column-major (B, T, features))
    dev = "cuda"
    g = torch.Generator(device=dev)
    g.manual_seed(31)

    def cm(rows, cols, scale=1.0):  # logical [rows, cols], column-major
        return (torch.randn((cols, rows), generator=g, device=dev) * scale).t()

    x = cm(R, D)
    nq, nkv = H * hd, Hkv * hd
    if side_by_side:
        w_qkv, b_qkv, w_gu = cm(D, nq + 2 * nkv, 0.02), torch.zeros(nq + 2 * nkv, device=dev), cm(D, 2 * d_ff, 0.02)
        w_q, w_k, w_v = w_qkv[:, :nq], w_qkv[:, nq:nq + nkv], w_qkv[:, nq + nkv:]
        b_q, b_k, b_v = b_qkv[:nq], b_qkv[nq:nq + nkv], b_qkv[nq + nkv:]
        w_gate, w_up = w_gu[:, :d_ff], w_gu[:, d_ff:]
        w_o, b_o, w_down = cm(nq, D, 0.02), torch.zeros(D, device=dev), cm(d_ff, D, 0.02)
    else:
        w_q, w_k, w_v, w_o = cm(D, nq, 0.02), cm(D, nkv, 0.02), cm(D, nkv, 0.02), cm(nq, D, 0.02)
        b_q, b_k, b_v, b_o = (torch.zeros(n, device=dev) for n in (nq, nkv, nkv, D))
        w_gate, w_up, w_down = cm(D, d_ff, 0.02), cm(D, d_ff, 0.02), cm(d_ff, D, 0.02)
    ln1, ln2 = torch.ones(D, device=dev), torch.ones(D, device=dev)
    # RoPE tables, column-major [rows, head_dim] (src/modules/rope.cpp:18-51); only row `ctx - 1` is used
    rows = ctx + 1
    i = np.arange(hd // 2, dtype=np.float32)
    theta = np.power(np.float32(10000.0), -2.0 * i / np.float32(hd)).astype(np.float32)
    ang = np.arange(rows, dtype=np.float32)[:, None] * np.repeat(theta, 2)[None, :]
    cos_t = torch.from_numpy(np.ascontiguousarray(np.cos(ang).T.astype(np.float32))).to(dev).reshape(-1)
    sin_t = torch.from_numpy(np.ascontiguousarray(np.sin(ang).T.astype(np.float32))).to(dev).reshape(-1)
    cache = capi.KVCache(capi.KV_LLOYDMAX, B, Hkv, hd, ctx, 3, 4)
    rk, rv = torch.zeros(hd * hd, device=dev), torch.zeros(hd * hd, device=dev)
    capi.make_rotation(41, hd, rk)
    capi.make_rotation(42, hd, rv)
    cache.set_rotations(rk, rv)
    for s0 in range(0, B, 8):
        Ks = torch.randn((8, Hkv, ctx - n_calls * T, hd), generator=g, device=dev)
        Vs = torch.randn((8, Hkv, ctx - n_calls * T, hd), generator=g, device=dev)
        cache.encode_append(Ks, Vs, seq_begin=s0, rotate=1)
    del Ks, Vs

    def buf(cols):
        return torch.empty((cols, R), device=dev).t()  # logical [B * T, cols], column-major

    h1, qr, kr, att, o, res1, h2, act, down, out = (
        buf(D), buf(nq), buf(nkv), buf(nq), buf(D), buf(D), buf(D), buf(d_ff), buf(D), buf(D))
    if side_by_side:
        qkv, gu = buf(nq + 2 * nkv), buf(2 * d_ff)
        q, k, v, gate, up = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:], gu[:, :d_ff], gu[:, d_ff:]
    else:
        q, k, v, gate, up = buf(nq), buf(nkv), buf(nkv), buf(d_ff), buf(d_ff)
    eps = float(np.float32(np.finfo(np.float32).eps / 4))

    def heads(t, n):  # the (B, heads, T, head_dim) view of a (B, T, heads * head_dim) activation: feature = h + n * j
        return torch.as_strided(t, (B, n, T, hd), (1, R, B, R * n))

    flags = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT

    def step():
        capi.rms_norm(x, ln1, eps, h1)
        if side_by_side:
            capi.linear(h1, w_qkv, b_qkv, qkv)
        else:
            capi.linear(h1, w_q, b_q, q)
            capi.linear(h1, w_k, b_k, k)
            capi.linear(h1, w_v, b_v, v)
        capi.rope(heads(q, H), cos_t, sin_t, rows, heads(qr, H), pos0=ctx - T)
        capi.rope(heads(k, Hkv), cos_t, sin_t, rows, heads(kr, Hkv), pos0=ctx - T)
        cache.encode_append(heads(kr, Hkv), heads(v, Hkv), rotate=1)
        if T == 1:
            cache.decode_attn(heads(qr, H)[:, :, 0], heads(att, H)[:, :, 0], capi.GQA_BLOCKED, flags)
        else:
            cache.decode_attn_chunk(heads(qr, H).permute(0, 2, 1, 3), heads(att, H).permute(0, 2, 1, 3), None,
                                    capi.GQA_BLOCKED, flags)
        capi.linear(att, w_o, b_o, o)
        capi.elementwise(capi.EW_ADD, o, x, res1)
        capi.rms_norm(res1, ln2, eps, h2)
        if side_by_side:
            capi.linear(h2, w_gu, None, gu)
        else:
            capi.linear(h2, w_gate, None, gate)
            capi.linear(h2, w_up, None, up)
        capi.elementwise(capi.EW_SILU_MUL, gate, up, act)
        capi.linear(act, w_down, None, down)
        capi.elementwise(capi.EW_ADD, down, res1, out)

    return cache, step


def plan_scan(capi, torch, steps=100, warmup=WARMUP_FLOOR_EXTRA, d=128):
    """The decode planner's default plan against the plain three-kernel plan (query kernel, attention, merge) over a
    grid of batch sizes, context lengths, group sizes and ragged batches: microseconds per call by two events around
    `steps` back-to-back calls (the better of two such measurements per plan).  A record to check changes of the planner's thresholds against: `behind` lists the
    shapes where the default is more than 3 us slower than three kernels, `differ` those where the two plans' results
    are further apart than the GPU tests allow (2e-5 relative + 2e-6)."""
    import random
    flags = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT
    rk, rv = torch.zeros(d * d, device="cuda"), torch.zeros(d * d, device="cuda")
    capi.make_rotation(5, d, rk)
    capi.make_rotation(6, d, rv)
    shapes = []
    for Hkv, Hq in ((8, 32), (2, 16)):
        for S in (3, 12, 24, 50, 96, 200, 512):
            for ctx in (100, 300, 1000, 2100, 5000):
                shapes.append(("equal", Hkv, Hq, [ctx] * S))
    for S in (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128):
        shapes.append(("equal", 8, 32, [8192] * S))
    for S, ctx in ((1, 1000), (1, 8192), (16, 8192), (64, 2100)):
        shapes.append(("equal, groups of 32", 2, 64, [ctx] * S))  # (two passes of sixteen heads)
    for ctx in (7744, 8000, 8129):
        shapes.append(("equal", 8, 32, [ctx] * 64))
    rnd = random.Random(17)
    for S in (4, 16, 48, 64, 128):
        shapes.append(("ragged 4096..8192", 8, 32, [rnd.randint(4096, 8192) for _ in range(S)]))
        shapes.append(("ragged 512..8192", 8, 32, [rnd.randint(512, 8192) for _ in range(S)]))
        shapes.append(("half 8192 half 1024", 8, 32, [8192 if i % 2 == 0 else 1024 for i in range(S)]))
    rows, behind, differ = [], [], []
    for kind, Hkv, Hq, lens in shapes:
        S = len(lens)
        cache = capi.KVCache(capi.KV_LLOYDMAX, S, Hkv, d, max(lens), 3, 4, 0, 0)
        cache.set_rotations(rk, rv)
        if len(set(lens)) == 1:
            K = torch.randn((min(S, 64), Hkv, lens[0], d), device="cuda")
            for s0 in range(0, S, 64):
                n = min(64, S - s0)
                cache.encode_append(K[:n], K[:n], seq_begin=s0, rotate=1)
        else:
            K = torch.randn((1, Hkv, max(lens), d), device="cuda")
            for s0, n in enumerate(lens):
                cache.encode_append(K[:, :, :n], K[:, :, :n], seq_begin=s0, rotate=1)
        del K
        q = torch.randn((S, Hq, d), device="cuda")
        out = torch.zeros_like(q)
        us = [float("inf"), float("inf")]
        kernels = None
        # (each plan twice, in turns, the better of the two: whichever plan is timed first after the cache was filled
        # reads a few percent slow)
        for i, kw in enumerate(({}, dict(separate_merge=True, separate_query=True)) * 2):
            capi.decode_tuning(**kw)
            try:
                if i == 0:
                    capi.profile_reset()
                    capi.profile_enable(True)
                    cache.decode_attn(q, out, capi.GQA_BLOCKED, flags)
                    torch.cuda.synchronize()
                    kernels = 1 if capi.profile_read("kv_decode_combine")[1] == 0 else 3
                    capi.profile_enable(False)
                t = 1e6 * time_region(torch, lambda: cache.decode_attn(q, out, capi.GQA_BLOCKED, flags), steps, warmup)
                us[i % 2] = min(us[i % 2], t)
            finally:
                capi.decode_tuning()
        # the two plans' results, element by element (they add the same partial results in different places)
        results = []
        for kw in ({}, dict(separate_merge=True, separate_query=True)):
            capi.decode_tuning(**kw)
            try:
                out.zero_()
                cache.decode_attn(q, out, capi.GQA_BLOCKED, flags)
                torch.cuda.synchronize()
                results.append(out.clone())
            finally:
                capi.decode_tuning()
        diff = (results[0] - results[1]).abs()
        row = {"kind": kind, "n_seq": S, "kv_heads": Hkv, "q_heads": Hq,
               "ctx": lens[0] if len(set(lens)) == 1 else [min(lens), max(lens)], "default_us": round(us[0], 2),
               "default_kernels": kernels, "three_kernels_us": round(us[1], 2),
               "max_abs_difference": float(diff.max())}
        rows.append(row)
        if us[0] > us[1] + 3.0:
            behind.append(row)
        if bool((diff > 2e-5 * results[1].abs() + 2e-6).any()) or not bool(torch.isfinite(results[0]).all()):
            differ.append(row)
        del results, diff
        cache.close()
    return {"plan_scan": rows, "behind_three_kernels_by_more_than_3us": behind,
            "results_differ_by_more_than_2e-5_relative_plus_2e-6": differ, "steps": steps, "warmup": warmup,
            "head_dim": d}


def extras(capi, torch, workloads, steps, warmup):
    """The other configurations, measured the same way (reported beside the headline, not as `value`)."""
    out = {}
    # configuration 5b: [4096 x 1024] . [1024 x 4096] fp32, column-major operands as Weed passes them
    A = torch.randn((1024, 4096), device="cuda").t()           # logical [4096, 1024], column-major
    W = (torch.randn((4096, 1024), device="cuda") * 0.02).t()  # logical [1024, 4096], column-major
    C = torch.empty((4096, 4096), device="cuda").t()
    secs, kernel_s, how = time_one_kernel_op(capi, torch, lambda: capi.matmul(A, W, C), "matmul", steps, warmup)
    flops = 2.0 * 4096 * 1024 * 4096
    # The product runs on the bfloat16 matrix instruction with both operands split exactly into three parts and six
    # products of parts per fp32 product, so its matrix-core bound is the bfloat16 peak over six; the same product on
    # the fp32 instruction (weed_hip_matmul_tuning) is measured beside it against that instruction's own peak.
    split_peak = 2500.0 / 6.0
    out["cfg5b_matmul_f32_4096x1024x4096"] = {
        "tflops": flops / secs / 1e12, "kernel_ms": 1e3 * kernel_s, "kernel_tflops": flops / kernel_s / 1e12,
        "roofline": {"bound": "mfma", "achieved": flops / kernel_s / 1e12, "peak": split_peak, "unit": "TFLOP/s",
                     "frac": flops / kernel_s / 1e12 / split_peak,
                     "peak_is": "bf16 dense 2500 TFLOP/s / 6 products of bfloat16 parts per fp32 product",
                     "frac_of_fp32_instruction_peak_157.3": flops / kernel_s / 1e12 / 157.3}}
    out["cfg5b_matmul_f32_4096x1024x4096"].update(how)
    capi.matmul_tuning(True)
    try:
        _, k32, _ = time_one_kernel_op(capi, torch, lambda: capi.matmul(A, W, C), "matmul", steps, warmup)
    finally:
        capi.matmul_tuning(False)
    out["cfg5b_matmul_f32_4096x1024x4096"]["on_the_fp32_instruction"] = {
        "kernel_ms": 1e3 * k32,
        "roofline": {"bound": "mfma", "achieved": flops / k32 / 1e12, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": flops / k32 / 1e12 / 157.3}}
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
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    read_s = time_region(torch, lambda: capi.read_sweep(Wp, wbytes, 0, sink), steps, warmup)
    out["projection_8x4096x4096"]["roofline"]["streaming_read_ms"] = 1e3 * read_s
    out["projection_8x4096x4096"]["roofline"]["streaming_read_what"] = (
        "the library's read-only sweep over the same 64 MiB weight: what a launch that only reads the bytes takes")
    # The same product over six weights in turn (384 MiB, more than the 256 MB Infinity Cache holds): back-to-back
    # calls on ONE 64 MiB weight are served in part by that cache; a model's step reads every weight once.
    Wr = [Wp] + [(torch.randn((4096, 4096), device="cuda") * 0.02).t() for _ in range(5)]
    turn = [0]

    def in_turn():
        capi.matmul(X, Wr[turn[0] % 6], Y)
        turn[0] += 1
    rot_s = time_region(torch, in_turn, steps, warmup)
    out["projection_8x4096x4096"]["six_weights_in_turn"] = {
        "kernel_ms": 1e3 * rot_s, "gbs": wbytes / rot_s / 1e9, "frac": wbytes / rot_s / 1e9 / HBM_PEAK_GBS,
        "what": "the same call over six different weights in turn, so that every call reads its weight from HBM"}
    del X, Wr, Wp, Y, sink
    # 64 rows (a decode step of 64 sequences) against [4096 x 14336] weights (235 MB each), four in turn: the
    # matrix-core kernel for 17 to 64 rows (bfloat16 products of exactly split operands) and the kernel that adds its
    # k ranges, two launches per call
    X = torch.randn((4096, 64), device="cuda").t()               # logical [64, 4096], column-major
    Wg = [(torch.randn((14336, 4096), device="cuda") * 0.02).t() for _ in range(4)]  # logical [4096, 14336], column-major
    Y = torch.empty((14336, 64), device="cuda").t()
    turn[0] = 0

    def wide_in_turn():
        capi.matmul(X, Wg[turn[0] % 4], Y)
        turn[0] += 1
    wide_s = time_region(torch, wide_in_turn, steps, warmup)
    wide_bytes = 4096 * 14336 * 4
    out["projection_64x4096x14336"] = {
        "ms": 1e3 * wide_s, "launches_per_call": 2,
        "roofline": {"bound": "hbm", "achieved": wide_bytes / wide_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": wide_bytes / wide_s / 1e9 / HBM_PEAK_GBS},
        "what": "64 rows, four weights in turn (0.94 GB); the time is the whole call: the product's kernel and the sum "
                "over its k ranges"}
    del X, Wg, Y
    # standalone softmax and sum over an [8192 x 16384] column-major matrix (512 MiB, twice the Infinity Cache, so
    # that back-to-back launches read from HBM), along the contiguous axis and along the strided one: 8 B per element
    # (softmax) and 4 B per element (sum) of algorithmic traffic.  Along the strided axis a column block of 32 rows
    # x 16384 does not fit a compute unit, so that softmax reads the data twice: 12 B per element actually moved
    # (`bytes_model`); its fraction by the 8 B the metric counts is the one in `roofline.frac`.
    S = torch.randn((16384, 8192), device="cuda").t()
    So = torch.empty((16384, 8192), device="cuda").t()
    dense = {}
    for axis, name in ((0, "contiguous_axis"), (1, "strided_axis")):
        Sr = torch.empty(S.shape[1 - axis], device="cuda")
        for op, fn, bytes_per in (("softmax", lambda: capi.softmax(S, So, axis), 8),
                                  ("reduce", lambda: capi.reduce(capi.REDUCE_SUM, S, Sr, axis), 4)):
            _, kernel_s, how = time_one_kernel_op(capi, torch, fn, op, steps, warmup)
            gbs = S.numel() * bytes_per / kernel_s / 1e9
            e = {"kernel_ms": 1e3 * kernel_s, "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS,
                                                           "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}}
            if op == "softmax" and axis == 1:
                moved = S.numel() * 12 / kernel_s / 1e9
                e["roofline"]["bytes_model"] = {"bytes_per_element_moved": 12, "gbs_moved": moved,
                                                "frac_moved": moved / HBM_PEAK_GBS,
                                                "why": "a 32-row column block of this length exceeds a compute unit's "
                                                       "registers and LDS: one pass for (max, sum), one to normalise"}
            e.update(how)
            dense["%s_%s" % (op, name)] = e
        del Sr
    out["softmax_sum_f32_8192x16384"] = dense
    del S, So
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

    secs, pair_s = time_kernel(capi, torch, enc, "kv_encode", steps, warmup)
    # the kernel alone: a run of back-to-back appends of 4096 tokens into a cache that holds them all, no reset in
    # between (every append after the first is the same launch: whole half blocks behind whole half blocks, followed by
    # the small kernel that moves the lengths), two events around the run
    n_run = min(steps, 40)
    n_warm = WARMUP_FLOOR_EXTRA
    big = capi.KVCache(capi.KV_LLOYDMAX, 1, wl.n_kv_heads, d, 4096 * (n_run + n_warm), 3, 3)
    big.set_rotations(rk, rv)
    kernel_s = time_region(torch, lambda: big.encode_append(K, V, rotate=1), n_run, n_warm)
    big.close()
    in_bytes = 2 * K.numel() * 4
    rot_flops = 2 * 2.0 * K.numel() * d  # K and V: rows x 2 d^2
    out["cfg5a_encode_4096x8x128_3bit"] = {
        "tokens_per_s": 4096 / secs, "ms": 1e3 * secs, "input_gbs": in_bytes / secs / 1e9,
        "rotation_tflops": rot_flops / secs / 1e12, "kernel_ms": 1e3 * kernel_s,
        "kernel_ms_event_pair_per_launch": 1e3 * pair_s,
        "roofline": {"bound": "mfma", "achieved": rot_flops / kernel_s / 1e12, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": rot_flops / kernel_s / 1e12 / 157.3, "kernel": "encode_rows_pair_kernel (K and V)",
                     "flops_per_launch": rot_flops},
        "kernel_ms_source": "device time of %d back-to-back appends of 4096 tokens (encoder kernel + the kernel that "
                            "moves the lengths, no cache reset) between two events, divided by their number; `ms` is "
                            "the call with the reset that a benchmark loop needs" % n_run}
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
    del q3, o3
    # one decode step of one Qwen-style decoder layer on the headline shape (64 sequences near ctx 8192)
    import numpy as np
    n_l = min(steps, 50)
    cacheQ, layer_step = layer_decode_step(capi, torch, np, n_calls=WARMUP_FLOOR_EXTRA + 3 * n_l + 1)
    layer_step()
    torch.cuda.synchronize()
    host_s = time_calls(torch, layer_step, n_l, WARMUP_FLOOR_EXTRA)
    dev_s = time_region(torch, layer_step, n_l, 0)
    capi.profile_reset()
    capi.profile_enable(True)
    time_calls(torch, layer_step, n_l, 0)
    parts = {}
    for name in ("kv_decode_attn", "kv_encode", "matmul", "rms_norm", "elementwise", "rope"):
        ms, n = capi.profile_read(name)
        parts[name] = {"ms_per_step": ms / n_l, "launches_per_step": n / n_l}
    capi.profile_enable(False)
    out["qwen_layer_decode_step_64_sequences_ctx8192"] = {
        "ms_per_step": 1e3 * host_s, "device_ms_per_step": 1e3 * dev_s, "tokens_per_s": 64 / host_s,
        "launches_per_step": sum(p["launches_per_step"] for p in parts.values()),
        "attention_share": parts["kv_decode_attn"]["ms_per_step"] / (1e3 * dev_s),
        "by_kernel_family_event_pairs": parts,
        "shape": "d_model 4096, 32 / 8 heads of 128, d_ff 14336, fp32 weights (0.97 GB per layer), K 3-bit + V 4-bit "
                 "cache; RMSNorm, Q/K/V projections, RoPE x2, append, attention, output projection, residual, RMSNorm, "
                 "gate/up projections, SiLU gate, down projection, residual",
        "weight_bytes": 4 * (2 * 4096 * 4096 + 2 * 4096 * 1024 + 3 * 4096 * 14336)}
    cacheQ.close()
    del cacheQ, layer_step
    # the same step with the weights of the projections that share their input side by side (the host mirror's
    # fuse_projections()): Q, K, V are one product, gate and up another
    cacheF, fused_step = layer_decode_step(capi, torch, np, n_calls=WARMUP_FLOOR_EXTRA + 2 * n_l + 1, side_by_side=True)
    fused_step()
    torch.cuda.synchronize()
    fused_host_s = time_calls(torch, fused_step, n_l, WARMUP_FLOOR_EXTRA)
    fused_dev_s = time_region(torch, fused_step, n_l, 0)
    out["qwen_layer_decode_step_64_sequences_ctx8192"]["projections_side_by_side"] = {
        "ms_per_step": 1e3 * fused_host_s, "device_ms_per_step": 1e3 * fused_dev_s, "launches_per_step": 13,
        "what": "the weights of Q, K, V in one buffer and those of gate and up in another, as after "
                "fuse_projections() of the host mirror's layer: one product for each group"}
    cacheF.close()
    del cacheF, fused_step
    # a prefill chunk through the same layer: 64 tokens for each of the 64 sequences (4096 rows per product), appended
    # behind ctx ~ 7700 and attended with the chunk's causal mask over the packed cache
    n_c = 4
    cacheP, chunk_step = layer_decode_step(capi, torch, np, n_calls=2 * n_c + 3, n_tokens=64)
    chunk_step()
    torch.cuda.synchronize()
    chunk_host_s = time_calls(torch, chunk_step, n_c, 2)
    capi.profile_reset()
    capi.profile_enable(True)
    time_calls(torch, chunk_step, n_c, 0)
    partsP = {}
    for name in ("kv_decode_attn", "kv_encode", "matmul", "rms_norm", "elementwise", "rope"):
        ms, n = capi.profile_read(name)
        partsP[name] = {"ms_per_step": ms / n_c, "launches_per_step": n / n_c}
    capi.profile_enable(False)
    chunk_flops = 2.0 * 4096 * 4096 * (2 * 4096 + 2 * 1024 + 3 * 14336)
    out["qwen_layer_prefill_chunk_64_tokens_64_sequences"] = {
        "ms_per_step": 1e3 * chunk_host_s, "tokens_per_s": 4096 / chunk_host_s,
        "by_kernel_family_event_pairs": partsP,
        "projection_tflops": chunk_flops / (1e-3 * partsP["matmul"]["ms_per_step"]) / 1e12,
        "shape": "the layer of qwen_layer_decode_step on (64, 64, 4096) activations: seven products of 4096 rows "
                 "(1.79 TFLOP), append of 64 tokens per sequence, attention of the 64 positions over ~7700 cached tokens"}
    cacheP.close()
    del cacheP, chunk_step
    # the same chunk with every product on the fp32 matrix instruction (weed_hip_matmul_tuning)
    capi.matmul_tuning(True)
    try:
        cache32, chunk32 = layer_decode_step(capi, torch, np, n_calls=n_c + 3, n_tokens=64)
        chunk32()
        torch.cuda.synchronize()
        out["qwen_layer_prefill_chunk_64_tokens_64_sequences"]["on_the_fp32_instruction_ms_per_step"] = \
            1e3 * time_calls(torch, chunk32, n_c, 2)
        cache32.close()
    finally:
        capi.matmul_tuning(False)
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
    ap.add_argument("--calibrate-read", action="store_true",
                    help="only launch the library's read-only sweeps over as many bytes as the headline step reads "
                         "(the practical ceiling of a read stream on this part), for a rocprofv3 kernel trace")
    ap.add_argument("--plan-scan", action="store_true",
                    help="only scan the decode planner: its default plan against three kernels over a grid of batch "
                         "sizes, contexts, group sizes and ragged batches (about a minute)")
    ap.add_argument("--head-dim", type=int, default=128, help="head_dim of --plan-scan")
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
    if args.plan_scan:
        with torch.cuda.stream(stream):
            print(json.dumps(plan_scan(capi, torch, d=args.head_dim)))
        return
    if args.calibrate_read:
        with torch.cuda.stream(stream):
            wl = workloads.config(3, n_seq=args.seqs, scale=args.ctx / 8192.0)
            r = streaming_read(capi, torch, wl.bytes_per_step(lloydmax=True), max(args.steps, 200), WARMUP_FLOOR_HEADLINE)
        print(json.dumps({"streaming_read": r}))
        return
    with torch.cuda.stream(stream):
        wl = workloads.config(3, n_seq=args.seqs, scale=args.ctx / 8192.0)
        cache, q, rk, rv = build_cache(capi, torch, wl, seed=1234)
        out = torch.zeros_like(q)
        flags = capi.ATTN_ROTATE_Q | capi.ATTN_UNROTATE_OUT

        def step():
            cache.decode_attn(q, out, capi.GQA_BLOCKED, flags)

        warm = max(args.warmup, WARMUP_FLOOR_HEADLINE)
        for _ in range(warm):
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
                for _ in range(max(args.warmup, WARMUP_FLOOR_EXTRA)):
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

        # The same step for a module whose projections have the rotations folded in (no RoPE between W_q and the cache:
        # R_k goes into W_q offline; R_v^T into W_o with or without RoPE): flags = 0, nothing rotated in the kernel
        def step_folded():
            cache.decode_attn(q, out, capi.GQA_BLOCKED, 0)

        folded_s = time_region(torch, step_folded, args.steps, max(args.warmup, WARMUP_FLOOR_EXTRA))
        for _ in range(WARMUP_FLOOR_EXTRA):
            step()  # (leaves `out` as the full call computes it, for the CPU cross-check below)
        # what merely reading the step's bytes costs
        read_ceiling = streaming_read(capi, torch, bytes_per_launch, min(max(args.steps, 50), 200), WARMUP_FLOOR_EXTRA)

        # batch = 1 latency of the same shape (one sequence per launch: launch-latency bound); part of the extras, so
        # that a --no-extras run launches the main kernel at the headline shape only
        wl1 = workloads.config(3, n_seq=1, scale=args.ctx / 8192.0)
        single_ms = None
        if not args.no_extras:
            cache1, q1, _, _ = build_cache(capi, torch, wl1, seed=99)
            out1 = torch.zeros_like(q1)
            for _ in range(max(args.warmup, WARMUP_FLOOR_EXTRA)):
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
            "warmup_floor_launches": WARMUP_FLOOR_HEADLINE,
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
                "streaming_read_ms": read_ceiling["per_wavefront_runs_ms"],
                "streaming_read": read_ceiling,
                "frac_of_streaming_read": read_ceiling["per_wavefront_runs_ms"] / kernel_ms,
                "rotations_folded_into_projections": {
                    "kernel_ms": 1e3 * folded_s, "frac": bytes_per_launch / folded_s / 1e9 / HBM_PEAK_GBS,
                    "what": "the same call with flags = 0: queries arrive in the K basis and the result stays in the V "
                            "basis, as for a module that folds R_k into W_q (no RoPE) and R_v^T into W_o offline"},
            },
            "whole_step_gbs": bytes_per_launch / (ms_per_step * 1e-3) / 1e9,
        }
        if not args.no_extras:
            # a chunk of 4 query positions per sequence in one pass over the same caches (speculative decoding)
            S_, Hq_, d_ = q.shape
            qc = torch.randn((S_, 4, Hq_, d_), device="cuda")
            oc = torch.zeros_like(qc)
            chunk_s = time_calls(torch, lambda: cache.decode_attn_chunk(qc, oc, None, capi.GQA_BLOCKED, flags),
                                 min(args.steps, 200), max(args.warmup, WARMUP_FLOOR_EXTRA))
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
            result["other_configs"] = extras(capi, torch, workloads, min(args.steps, 200), max(args.warmup, WARMUP_FLOOR_EXTRA))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
