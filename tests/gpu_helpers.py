"""Shared plumbing of the GPU parity tests: device tensors via torch, the CPU checker via oracle/."""
import numpy as np


def dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def col_major(x):
    """Device tensor with the logical shape of `x` and Weed's column-major strides (dimension 0 fastest)."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(np.transpose(x))).cuda()  # reversed dims, row-major
    return t.permute(*reversed(range(x.ndim)))


def coder_specs(oracle, cache):
    """CPU-checker coder descriptions that mirror a device cache (tables are read back through the C ABI)."""
    cfg = cache.cfg
    specs = []
    for which in (0, 1):
        bits = cfg.v_bits if which else cfg.k_bits
        sign = cfg.v_sign if which else cfg.k_sign
        if cfg.mode == 0:
            import ctypes
            ks, vs = ctypes.c_float(), ctypes.c_float()
            cache.lib.weed_hip_kv_cache_get_scales(cache.handle, ctypes.byref(ks), ctypes.byref(vs))
            specs.append(oracle.CoderSpec(0, cfg.head_dim, bits, block_scale=(vs if which else ks).value))
        else:
            bounds, levels, recon = cache.get_tables(which)
            specs.append(oracle.CoderSpec(1, cfg.head_dim, bits, sign=sign, bounds=bounds, levels=levels, recon=recon))
    return specs


def export(cache, which, T, seq_begin=0, seq_count=None, tok_begin=0):
    """(fields uint8 [S, Hkv, T, d], scales float32 [S, Hkv, T]) read back from the device cache."""
    import torch
    cfg = cache.cfg
    S = seq_count if seq_count is not None else cfg.n_seq
    fields = torch.empty((S, cfg.n_kv_heads, T, cfg.head_dim), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((S, cfg.n_kv_heads, T), dtype=torch.float32, device="cuda")
    cache.export_fields(which, fields, scales, seq_begin=seq_begin, tok_begin=tok_begin)
    return fields.cpu().numpy(), scales.cpu().numpy()


def assert_attn_close(got, want, what=""):
    """The north-star tolerance for attention outputs: max-abs 1e-4 / rel 1e-3 in fp32."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    bound = np.maximum(1e-4, 1e-3 * np.abs(want))  # either bound, not their sum
    assert np.all(err <= bound), "%s: max abs err %.3e (allowed max(1e-4, 1e-3*|ref|)), worst ref %.3e" % (
        what, err.max(), np.abs(want).flat[np.argmax(err - bound)])
