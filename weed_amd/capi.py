"""ctypes binding of the C ABI in include/weed_hip.h.

Used by tests and bench.py.  Device memory comes from PyTorch (plumbing only): tensors are passed as raw
`data_ptr()` values plus Weed-style geometry (offset and strides in elements).  Import torch before loading the
library so that both share one HIP runtime.
"""
import ctypes
import os
from ctypes import (POINTER, byref, c_char_p, c_double, c_float, c_int, c_int32, c_size_t, c_uint8, c_uint32, c_uint64,
                    c_void_p)

from .build import library_path

OK, EINVAL, ENOMEM, EDEVICE, ECAPACITY = 0, 1, 2, 3, 4
KV_UNIFORM, KV_LLOYDMAX = 0, 1
GQA_WEED, GQA_BLOCKED = 0, 1
ATTN_ROTATE_Q, ATTN_UNROTATE_OUT = 1, 2
REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2
EW_COPY, EW_ADD, EW_SUB, EW_MUL, EW_DIV, EW_SILU_MUL, EW_RELU, EW_SIGMOID, EW_TANH, EW_GELU = range(10)


class KVConfig(ctypes.Structure):
    _fields_ = [(n, c_int32) for n in ("mode", "n_seq", "n_kv_heads", "head_dim", "max_tokens", "k_bits", "v_bits",
                                       "k_sign", "v_sign")]


class WeedHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("weed_hip error %d: %s" % (code, message))
        self.code = code


U32P = POINTER(c_uint32)

# name -> (restype, argtypes); every symbol include/weed_hip.h declares
SIGNATURES = {
    "weed_hip_init": (c_int, [c_int]),
    "weed_hip_device_count": (c_int, [POINTER(c_int)]),
    "weed_hip_device_name": (c_int, [c_char_p, c_size_t]),
    "weed_hip_set_stream": (c_int, [c_void_p]),
    "weed_hip_stream": (c_void_p, []),
    "weed_hip_sync": (c_int, []),
    "weed_hip_last_error": (c_char_p, []),
    "weed_hip_version": (c_char_p, []),
    "weed_hip_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "weed_hip_free": (c_int, [c_void_p]),
    "weed_hip_release_cached": (c_int, []),
    "weed_hip_memset": (c_int, [c_void_p, c_int, c_size_t]),
    "weed_hip_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_size_t]),
    "weed_hip_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_size_t]),
    "weed_hip_memcpy_d2d": (c_int, [c_void_p, c_void_p, c_size_t]),
    "weed_hip_profile_enable": (c_int, [c_int]),
    "weed_hip_profile_reset": (c_int, []),
    "weed_hip_profile_read": (c_int, [c_char_p, POINTER(c_double), POINTER(c_uint64)]),
    "weed_hip_matmul_f32": (c_int, [c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_void_p,
                                    c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32]),
    "weed_hip_matmul_batched_f32": (c_int, [U32P, c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32,
                                            U32P, c_void_p, c_uint32, c_uint32, c_uint32, U32P, c_void_p, c_uint32,
                                            c_uint32, c_uint32, U32P]),
    "weed_hip_linear_f32": (c_int, [c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32, c_void_p,
                                    c_uint32, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32,
                                    c_uint32, c_uint32]),
    "weed_hip_copy_f32": (c_int, [c_uint64, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32]),
    "weed_hip_read_sweep": (c_int, [c_void_p, c_uint64, c_int, c_void_p]),
    "weed_hip_elementwise_f32": (c_int, [c_int, c_uint32, U32P, c_void_p, c_uint32, U32P, c_void_p, c_uint32, U32P,
                                         c_void_p, c_uint32, U32P]),
    "weed_hip_triu_fill_f32": (c_int, [c_uint32, c_uint32, c_float, c_uint32, c_void_p, c_uint32, c_uint32, c_uint32]),
    "weed_hip_rope_f32": (c_int, [U32P, c_void_p, c_uint32, U32P, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p,
                                  c_uint32, U32P]),
    "weed_hip_rms_norm_f32": (c_int, [c_uint32, U32P, c_uint32, c_void_p, c_uint32, U32P, c_void_p, c_uint32, c_uint32,
                                      c_float, c_void_p, c_uint32, U32P]),
    "weed_hip_layer_norm_f32": (c_int, [c_uint32, U32P, c_uint32, c_void_p, c_uint32, U32P, c_void_p, c_uint32, c_uint32,
                                        c_void_p, c_uint32, c_uint32, c_float, c_void_p, c_uint32, U32P]),
    "weed_hip_softmax_f32": (c_int, [c_uint32, U32P, c_uint32, c_void_p, c_uint32, U32P, c_void_p, c_uint32, U32P]),
    "weed_hip_reduce_f32": (c_int, [c_int, c_uint32, U32P, c_uint32, c_void_p, c_uint32, U32P, c_void_p, c_uint32,
                                    U32P]),
    "weed_hip_make_rotation": (c_int, [c_uint32, c_uint32, c_void_p]),
    "weed_hip_orthonormalize_columns": (c_int, [c_uint32, c_void_p]),
    "weed_hip_apply_rotation_f32": (c_int, [c_uint32, c_void_p, c_uint32, U32P, c_void_p, c_uint32, U32P, c_void_p,
                                            c_uint32, U32P]),
    "weed_hip_kv_cache_create": (c_int, [POINTER(c_void_p), POINTER(KVConfig)]),
    "weed_hip_kv_cache_destroy": (c_int, [c_void_p]),
    "weed_hip_kv_cache_reset": (c_int, [c_void_p, c_int]),
    "weed_hip_kv_cache_row_bytes": (c_int, [c_void_p, U32P, U32P]),
    "weed_hip_kv_cache_seq_lens": (c_int, [c_void_p, POINTER(c_int32)]),
    "weed_hip_kv_cache_set_rotations": (c_int, [c_void_p, c_void_p, c_void_p]),
    "weed_hip_kv_cache_set_scales": (c_int, [c_void_p, c_float, c_float]),
    "weed_hip_kv_cache_get_scales": (c_int, [c_void_p, POINTER(c_float), POINTER(c_float)]),
    "weed_hip_kv_cache_set_tables": (c_int, [c_void_p, c_int, POINTER(c_float), POINTER(c_float), POINTER(c_float),
                                             POINTER(c_float)]),
    "weed_hip_kv_cache_get_tables": (c_int, [c_void_p, c_int, POINTER(c_float), POINTER(c_float), POINTER(c_float)]),
    "weed_hip_block_scale_f32": (c_int, [c_void_p, c_uint32, U32P, U32P, c_int, POINTER(c_float)]),
    "weed_hip_kv_encode_append": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_void_p, c_uint32, U32P, c_void_p,
                                          c_uint32, U32P, c_int]),
    "weed_hip_kv_dequant": (c_int, [c_void_p, c_int, c_int32, c_int32, c_int32, c_int32, c_void_p, c_uint32, U32P]),
    "weed_hip_kv_export_fields": (c_int, [c_void_p, c_int, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "weed_hip_kv_export_weed_words": (c_int, [c_void_p, c_int, c_int32, c_int32, c_int32, c_int32, c_void_p]),
    "weed_hip_kv_append_weed_words": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "weed_hip_kv_decode_attn": (c_int, [c_void_p, c_int32, c_int32, c_void_p, c_uint32, U32P, c_void_p, c_uint32, U32P,
                                        c_uint32]),
    "weed_hip_kv_decode_tuning": (c_int, [c_int32, c_int32, c_int32]),
    "weed_hip_matmul_tuning": (c_int, [c_int32]),
    "weed_hip_shutdown": (c_int, []),
    "weed_hip_kv_decode_attn_noalloc": (c_int, [c_void_p, c_int32, c_int32, c_void_p, c_uint32, U32P, c_void_p, c_uint32,
                                                U32P, c_uint32]),
    "weed_hip_kv_decode_attn_prefix": (c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_uint32, U32P, c_void_p,
                                               c_uint32, U32P, c_uint32]),
    "weed_hip_kv_decode_attn_chunk": (c_int, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_void_p, c_uint32, U32P,
                                              c_void_p, c_uint32, U32P, c_uint32]),
}

_lib = None


def load(path=None):
    """Load libweed_hip.so and declare every entry point.  Raises when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = path or library_path()
    if not os.path.exists(path):
        raise RuntimeError("%s not found: build it with __graft_entry__.build() or `make -C weed_amd/csrc`" % path)
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status):
    if status != OK:
        raise WeedHipError(status, load().weed_hip_last_error().decode())


def u32(values):
    return (c_uint32 * len(values))(*[int(v) for v in values])


def _geom(t):
    """(data_ptr, offset, strides) of a torch tensor view in Weed's terms (elements)."""
    return c_void_p(t.data_ptr()), 0, u32(t.stride())


class KVCache:
    """RAII wrapper around weed_hip_kv_cache."""

    def __init__(self, mode, n_seq, n_kv_heads, head_dim, max_tokens, k_bits, v_bits, k_sign=0, v_sign=0):
        self.lib = load()
        self.cfg = KVConfig(mode, n_seq, n_kv_heads, head_dim, max_tokens, k_bits, v_bits, k_sign, v_sign)
        self.handle = c_void_p()
        check(self.lib.weed_hip_kv_cache_create(byref(self.handle), byref(self.cfg)))

    def close(self):
        if self.handle:
            self.lib.weed_hip_kv_cache_destroy(self.handle)
            self.handle = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- configuration -------------------------------------------------------------------------
    def set_rotations(self, rk, rv):
        check(self.lib.weed_hip_kv_cache_set_rotations(self.handle, c_void_p(rk.data_ptr()), c_void_p(rv.data_ptr())))

    def set_scales(self, k_scale, v_scale):
        check(self.lib.weed_hip_kv_cache_set_scales(self.handle, c_float(k_scale), c_float(v_scale)))

    def get_tables(self, which):
        bits = self.cfg.v_bits if which else self.cfg.k_bits
        sign = self.cfg.v_sign if which else self.cfg.k_sign
        n = 1 << bits
        bounds = (c_float * (n - 1))()
        levels = (c_float * n)()
        recon = (c_float * (n << sign))()
        check(self.lib.weed_hip_kv_cache_get_tables(self.handle, which, bounds, levels, recon))
        return list(bounds), list(levels), list(recon)

    def set_tables(self, which, bounds, levels, recon):
        out = (c_float * len(recon))()
        check(self.lib.weed_hip_kv_cache_set_tables(self.handle, which, (c_float * len(bounds))(*bounds),
                                                    (c_float * len(levels))(*levels), (c_float * len(recon))(*recon),
                                                    out))
        return list(out)

    def reset(self, drop_rotations=False):
        check(self.lib.weed_hip_kv_cache_reset(self.handle, int(drop_rotations)))

    def seq_lens(self):
        lens = (c_int32 * self.cfg.n_seq)()
        check(self.lib.weed_hip_kv_cache_seq_lens(self.handle, lens))
        return list(lens)

    def row_bytes(self):
        k, v = c_uint32(), c_uint32()
        check(self.lib.weed_hip_kv_cache_row_bytes(self.handle, byref(k), byref(v)))
        return k.value, v.value

    # -- data path -----------------------------------------------------------------------------
    def encode_append(self, k, v, seq_begin=0, rotate=0):
        """k, v: torch views of logical shape [seq_count, n_kv_heads, T_new, d] (any strides)."""
        assert k.dim() == 4 and k.shape == v.shape
        kp, ko, ks = _geom(k)
        vp, vo, vs = _geom(v)
        check(self.lib.weed_hip_kv_encode_append(self.handle, seq_begin, k.shape[0], k.shape[2], kp, ko, ks, vp, vo, vs,
                                                 rotate))

    def dequant(self, which, out, seq_begin=0, tok_begin=0):
        op, oo, os_ = _geom(out)
        check(self.lib.weed_hip_kv_dequant(self.handle, which, seq_begin, out.shape[0], tok_begin, out.shape[2], op, oo,
                                           os_))

    def export_fields(self, which, fields, scales=None, seq_begin=0, tok_begin=0):
        assert fields.is_contiguous() and (scales is None or scales.is_contiguous())
        check(self.lib.weed_hip_kv_export_fields(self.handle, which, seq_begin, fields.shape[0], tok_begin,
                                                 fields.shape[2], c_void_p(fields.data_ptr()),
                                                 c_void_p(scales.data_ptr()) if scales is not None else None))

    def export_weed_words(self, which, words, seq_begin=0, tok_begin=0):
        assert words.is_contiguous()
        check(self.lib.weed_hip_kv_export_weed_words(self.handle, which, seq_begin, words.shape[0], tok_begin,
                                                     words.shape[2], c_void_p(words.data_ptr())))

    def append_weed_words(self, k_words, v_words, seq_begin=0):
        """k_words, v_words: contiguous int32 torch tensors [seq_count, n_kv_heads, T_new, words per row]."""
        assert k_words.is_contiguous() and v_words.is_contiguous() and k_words.shape[:3] == v_words.shape[:3]
        check(self.lib.weed_hip_kv_append_weed_words(self.handle, seq_begin, k_words.shape[0], k_words.shape[2],
                                                     c_void_p(k_words.data_ptr()), c_void_p(v_words.data_ptr())))

    def decode_attn(self, q, out, gqa_mapping=GQA_WEED, flags=0):
        """q, out: torch views of logical shape [n_seq, n_q_heads, d]."""
        assert q.dim() == 3 and q.shape == out.shape
        qp, qo, qs = _geom(q)
        op, oo, os_ = _geom(out)
        check(self.lib.weed_hip_kv_decode_attn(self.handle, q.shape[1], gqa_mapping, qp, qo, qs, op, oo, os_, flags))

    def decode_attn_noalloc(self, q, out, gqa_mapping=GQA_WEED, flags=0):
        """decode_attn on the library's static workspace: allocates nothing, refuses shapes beyond 32 MiB of it."""
        assert q.dim() == 3 and q.shape == out.shape
        qp, qo, qs = _geom(q)
        op, oo, os_ = _geom(out)
        check(self.lib.weed_hip_kv_decode_attn_noalloc(self.handle, q.shape[1], gqa_mapping, qp, qo, qs, op, oo, os_,
                                                       flags))

    def decode_attn_prefix(self, lens, q, out, gqa_mapping=GQA_WEED, flags=0):
        """As decode_attn, over the first lens[s] cached tokens only (lens: int32 torch tensor on the device)."""
        assert q.dim() == 3 and q.shape == out.shape
        assert lens.element_size() == 4 and lens.is_cuda and lens.is_contiguous() and lens.numel() == q.shape[0]
        qp, qo, qs = _geom(q)
        op, oo, os_ = _geom(out)
        check(self.lib.weed_hip_kv_decode_attn_prefix(self.handle, c_void_p(lens.data_ptr()), q.shape[1], gqa_mapping,
                                                      qp, qo, qs, op, oo, os_, flags))


    def decode_attn_chunk(self, q, out, lens=None, gqa_mapping=GQA_WEED, flags=0):
        """q, out: torch views of logical shape [n_seq, n_tokens, n_q_heads, d]; the last n_tokens of the attended
        tokens (lens, or the cached lengths) are the chunk's own and are masked causally."""
        assert q.dim() == 4 and q.shape == out.shape
        qp, qo, qs = _geom(q)
        op, oo, os_ = _geom(out)
        lp = None
        if lens is not None:
            assert lens.element_size() == 4 and lens.is_cuda and lens.is_contiguous() and lens.numel() == q.shape[0]
            lp = c_void_p(lens.data_ptr())
        check(self.lib.weed_hip_kv_decode_attn_chunk(self.handle, lp, q.shape[1], q.shape[2], gqa_mapping, qp, qo, qs,
                                                     op, oo, os_, flags))


def use_torch_stream(stream):
    """Route every launch to a torch.cuda.Stream (so that torch events and allocations order with them)."""
    check(load().weed_hip_set_stream(c_void_p(stream.cuda_stream)))


def sync():
    check(load().weed_hip_sync())


def matmul(a, b, out):
    """2-D torch views (any strides): out = a @ b."""
    M, K = a.shape
    K2, N = b.shape
    assert K == K2 and tuple(out.shape) == (M, N)
    check(load().weed_hip_matmul_f32(M, N, K, c_void_p(a.data_ptr()), 0, a.stride(0), a.stride(1),
                                     c_void_p(b.data_ptr()), 0, b.stride(0), b.stride(1), c_void_p(out.data_ptr()), 0,
                                     out.stride(0), out.stride(1)))


def matmul_tuning(fp32_instruction=False):
    """Large products on the fp32 matrix instruction (True) or as six bfloat16 products of split operands (default)."""
    check(load().weed_hip_matmul_tuning(1 if fp32_instruction else 0))


def matmul_batched(a, b, out):
    """4-D torch views [B0, B1, ., .] (any strides): out[i, j] = a[i, j] @ b[i, j], one launch."""
    B0, B1, M, K = a.shape
    N = b.shape[3]
    assert tuple(b.shape) == (B0, B1, K, N) and tuple(out.shape) == (B0, B1, M, N)
    check(load().weed_hip_matmul_batched_f32(
        u32([B0, B1]), M, N, K, c_void_p(a.data_ptr()), 0, a.stride(2), a.stride(3), u32([a.stride(0), a.stride(1)]),
        c_void_p(b.data_ptr()), 0, b.stride(2), b.stride(3), u32([b.stride(0), b.stride(1)]),
        c_void_p(out.data_ptr()), 0, out.stride(2), out.stride(3), u32([out.stride(0), out.stride(1)])))


def linear(a, w, bias, out):
    """2-D torch views: out = a @ w + bias (bias: 1-D view of length N, or None), one launch."""
    M, K = a.shape
    K2, N = w.shape
    assert K == K2 and tuple(out.shape) == (M, N) and (bias is None or tuple(bias.shape) == (N,))
    check(load().weed_hip_linear_f32(M, N, K, c_void_p(a.data_ptr()), 0, a.stride(0), a.stride(1),
                                     c_void_p(w.data_ptr()), 0, w.stride(0), w.stride(1),
                                     c_void_p(bias.data_ptr()) if bias is not None else None, 0,
                                     bias.stride(0) if bias is not None else 0, c_void_p(out.data_ptr()), 0,
                                     out.stride(0), out.stride(1)))


def copy(a, out):
    """1-D torch views (any stride): out[i] = a[i]."""
    assert a.dim() == 1 and a.shape == out.shape
    check(load().weed_hip_copy_f32(a.numel(), c_void_p(a.data_ptr()), 0, a.stride(0), c_void_p(out.data_ptr()), 0,
                                   out.stride(0)))


EW_COPY, EW_ADD, EW_SUB, EW_MUL, EW_DIV = range(5)


def read_sweep(buf, nbytes, per_wavefront_runs, sink):
    """Read the first nbytes of the torch tensor `buf` once (calibration); sink: a one-element int32 device tensor."""
    check(load().weed_hip_read_sweep(c_void_p(buf.data_ptr()), nbytes, int(per_wavefront_runs), c_void_p(sink.data_ptr())))


def elementwise(op, a, b, out):
    """out = a (op) b on torch views; a and b are expanded (stride 0) to out's shape."""
    a = a.expand(out.shape)
    bp, bs = None, u32(out.stride())
    if b is not None:
        b = b.expand(out.shape)
        bp, bs = c_void_p(b.data_ptr()), u32(b.stride())
    check(load().weed_hip_elementwise_f32(op, out.dim(), u32(out.shape), c_void_p(a.data_ptr()), 0, u32(a.stride()),
                                          bp, 0, bs, c_void_p(out.data_ptr()), 0, u32(out.stride())))


def rms_norm(x, w, eps, out, axis=-1):
    """out = x / sqrt(mean(x^2 over axis) + eps) * w on torch views; w is a 1-D view along the axis."""
    axis %= x.dim()
    check(load().weed_hip_rms_norm_f32(x.dim(), u32(x.shape), axis, c_void_p(x.data_ptr()), 0, u32(x.stride()),
                                       c_void_p(w.data_ptr()), 0, w.stride(0), eps, c_void_p(out.data_ptr()), 0,
                                       u32(out.stride())))


def layer_norm(x, gamma, beta, eps, out, axis=-1):
    axis %= x.dim()
    check(load().weed_hip_layer_norm_f32(x.dim(), u32(x.shape), axis, c_void_p(x.data_ptr()), 0, u32(x.stride()),
                                         c_void_p(gamma.data_ptr()), 0, gamma.stride(0), c_void_p(beta.data_ptr()), 0,
                                         beta.stride(0), eps, c_void_p(out.data_ptr()), 0, u32(out.stride())))


def triu_fill(a, val, diagonal=1):
    rows, cols = a.shape
    check(load().weed_hip_triu_fill_f32(rows, cols, val, diagonal, c_void_p(a.data_ptr()), 0, a.stride(0),
                                        a.stride(1)))


def rope(x, cos_t, sin_t, table_rows, out, pos0=0):
    """x, out: torch views [B, H, T, head_dim]; cos_t / sin_t: flat column-major [table_rows, head_dim] tables."""
    check(load().weed_hip_rope_f32(u32(x.shape), c_void_p(x.data_ptr()), 0, u32(x.stride()), c_void_p(cos_t.data_ptr()),
                                   c_void_p(sin_t.data_ptr()), table_rows, pos0, c_void_p(out.data_ptr()), 0,
                                   u32(out.stride())))


def softmax(a, out, axis):
    assert a.shape == out.shape
    check(load().weed_hip_softmax_f32(a.dim(), u32(a.shape), axis, c_void_p(a.data_ptr()), 0, u32(a.stride()),
                                      c_void_p(out.data_ptr()), 0, u32(out.stride())))


def reduce(op, a, out, axis):
    """out has a's shape with `axis` removed."""
    o_stride = list(out.stride())
    o_stride.insert(axis, 0)
    check(load().weed_hip_reduce_f32(op, a.dim(), u32(a.shape), axis, c_void_p(a.data_ptr()), 0, u32(a.stride()),
                                     c_void_p(out.data_ptr()), 0, u32(o_stride)))


def make_rotation(seed, d, out):
    check(load().weed_hip_make_rotation(seed, d, c_void_p(out.data_ptr())))


def apply_rotation(x, r, out):
    """out = x . r over the last dimension of torch views x / out (same shape); r is d x d column-major."""
    d = x.shape[-1]
    check(load().weed_hip_apply_rotation_f32(d, c_void_p(r.data_ptr()), x.dim(), u32(x.shape), c_void_p(x.data_ptr()),
                                             0, u32(x.stride()), c_void_p(out.data_ptr()), 0, u32(out.stride())))


def orthonormalize_columns(d, r):
    check(load().weed_hip_orthonormalize_columns(d, c_void_p(r.data_ptr())))


def block_scale(x, sequential=False):
    """x: 4-D torch view.  Returns sqrt(sum(x^2)/n + 1e-8)."""
    out = c_float()
    check(load().weed_hip_block_scale_f32(c_void_p(x.data_ptr()), 0, u32(x.shape), u32(x.stride()), int(sequential),
                                          byref(out)))
    return out.value


def malloc(nbytes):
    """Device block from the library's stream-ordered cache; returns the address."""
    ptr = c_void_p()
    check(load().weed_hip_malloc(byref(ptr), ctypes.c_size_t(nbytes)))
    return ptr.value


def free(ptr):
    check(load().weed_hip_free(c_void_p(ptr)))


def shutdown():
    """Drain the stream and free what the library itself holds on the device; the next call starts it again."""
    check(load().weed_hip_shutdown())


def decode_tuning(wavefronts=0, skew_percent=-1, always_search=False, separate_merge=False, separate_query=False,
                  contiguous_runs=False):
    """Work partition of the decode kernels (defaults: 0, -1, False); results do not depend on it beyond the
    rounding of the last bits.  separate_merge / separate_query: never let the matrix-core kernel merge its partials /
    rotate its queries itself."""
    flags = (int(bool(always_search)) | 2 * int(bool(separate_merge)) | 4 * int(bool(separate_query)) |
             8 * int(bool(contiguous_runs)))
    check(load().weed_hip_kv_decode_tuning(int(wavefronts), int(skew_percent), flags))


def profile_enable(on):
    check(load().weed_hip_profile_enable(int(on)))


def profile_reset():
    check(load().weed_hip_profile_reset())


def profile_read(name):
    ms, n = c_double(), c_uint64()
    check(load().weed_hip_profile_read(name.encode(), byref(ms), byref(n)))
    return ms.value, n.value
