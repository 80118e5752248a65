"""numpy front end of the CPU oracle (oracle/weed_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by
weed_amd/.  `build()` compiles the C file with the recipe in oracle/Makefile.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int, c_int32, c_size_t, c_uint8, c_uint32, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libweed_oracle.so")
_lib = None


def build(force=False):
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


class Coder(ctypes.Structure):
    _fields_ = [("mode", c_int), ("d", c_int), ("bits", c_int), ("sign", c_int), ("block_scale", c_float),
                ("bounds", POINTER(c_float)), ("levels", POINTER(c_float)), ("recon", POINTER(c_float))]


class AttnGeom(ctypes.Structure):
    _fields_ = [("n_seq", c_int), ("n_q_heads", c_int), ("n_kv_heads", c_int), ("d", c_int), ("max_tokens", c_int),
                ("seq_lens", POINTER(c_int32)), ("gqa_weed_mapping", c_int), ("rotate_q", c_int),
                ("unrotate_out", c_int)]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.wo_block_scale.restype = c_float
        _lib.wo_block_scale.argtypes = [c_void_p, c_size_t]
        _lib.wo_words_per_row.restype = c_int
        _lib.wo_values_per_word.restype = c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(c_void_p)


# ---- Weed's uniform coder ------------------------------------------------------------------------

def words_per_row(d, bits):
    return lib().wo_words_per_row(int(d), int(bits))


def uniform_write_rows(x, bits, block_scale):
    """x: [rows, d] -> int32 [rows, wpr] in Weed's word packing (write_row on a zeroed cache)."""
    x = _f32(x)
    rows, d = x.shape
    wpr = words_per_row(d, bits)
    packed = np.zeros((rows, wpr), dtype=np.int32)
    fn = lib().wo_uniform_write_rows
    fn.argtypes = [c_void_p, c_void_p, c_size_t, c_int, c_int, c_float]
    fn(_p(packed), _p(x), rows, d, bits, c_float(block_scale))
    return packed


def uniform_read_rows(packed, d, bits, block_scale):
    packed = np.ascontiguousarray(packed, dtype=np.int32)
    rows = packed.shape[0]
    out = np.empty((rows, d), dtype=np.float32)
    fn = lib().wo_uniform_read_rows
    fn.argtypes = [c_void_p, c_void_p, c_size_t, c_int, c_int, c_float]
    fn(_p(packed), _p(out), rows, d, bits, c_float(block_scale))
    return out


def block_scale(x):
    x = _f32(x).reshape(-1)
    return float(lib().wo_block_scale(_p(x), x.size))


# ---- rotation ------------------------------------------------------------------------------------

def orthonormalize_columns(gauss):
    """gauss: flat column-major d*d (or [d, d] whose .ravel() is the column-major buffer).  Returns the flat buffer."""
    R = _f32(gauss).reshape(-1).copy()
    d = int(round(np.sqrt(R.size)))
    fn = lib().wo_orthonormalize_columns
    fn.argtypes = [c_void_p, c_int]
    fn(_p(R), d)
    return R


def apply_rotation(x, R):
    """x: [rows, d]; R: flat column-major d*d.  y = x . R, i ascending."""
    x = _f32(x)
    R = _f32(R).reshape(-1)
    rows, d = x.shape
    y = np.empty_like(x)
    fn = lib().wo_apply_rotation
    fn.argtypes = [c_void_p, c_size_t, c_int, c_void_p, c_void_p]
    fn(_p(x), rows, d, _p(R), _p(y))
    return y


# ---- table-driven coder --------------------------------------------------------------------------

class CoderSpec:
    """Keeps the numpy tables alive next to the ctypes struct."""

    def __init__(self, mode, d, bits, sign=0, block_scale=1.0, bounds=None, levels=None, recon=None):
        self.mode, self.d, self.bits, self.sign, self.block_scale = mode, d, bits, sign, float(block_scale)
        self.bounds = _f32(bounds if bounds is not None else np.zeros(1))
        self.levels = _f32(levels if levels is not None else np.zeros(1))
        self.recon = _f32(recon if recon is not None else np.zeros(1))
        self.c = Coder(mode, d, bits, sign, self.block_scale, self.bounds.ctypes.data_as(POINTER(c_float)),
                       self.levels.ctypes.data_as(POINTER(c_float)), self.recon.ctypes.data_as(POINTER(c_float)))


def encode_rows(spec, y):
    """y: [rows, d] (already rotated) -> (fields uint8 [rows, d], alpha float32 [rows])."""
    y = _f32(y)
    rows, d = y.shape
    fields = np.empty((rows, d), dtype=np.uint8)
    alpha = np.zeros(rows, dtype=np.float32)
    fn = lib().wo_encode_rows
    fn.argtypes = [POINTER(Coder), c_void_p, c_size_t, c_void_p, c_void_p]
    fn(ctypes.byref(spec.c), _p(y), rows, _p(fields), _p(alpha))
    return fields, alpha


def decode_rows(spec, fields, alpha):
    fields = np.ascontiguousarray(fields, dtype=np.uint8)
    alpha = _f32(alpha)
    rows, d = fields.shape
    out = np.empty((rows, d), dtype=np.float32)
    fn = lib().wo_decode_rows
    fn.argtypes = [POINTER(Coder), c_void_p, c_void_p, c_size_t, c_void_p]
    fn(ctypes.byref(spec.c), _p(fields), _p(alpha), rows, _p(out))
    return out


# ---- dense ops -----------------------------------------------------------------------------------

def matmul(M, N, K, A, a_geom, B, b_geom, C, c_geom):
    """Strided GEMM on flat float32 buffers; geom = (offset, stride0, stride1).  Writes into C in place."""
    fn = lib().wo_matmul
    fn.argtypes = [c_uint32] * 3 + [c_void_p, c_uint32, c_uint32, c_uint32] * 3
    fn(M, N, K, _p(A), *a_geom, _p(B), *b_geom, _p(C), *c_geom)
    return C


def _u32(v):
    return (c_uint32 * len(v))(*[int(x) for x in v])


def softmax(shape, axis, a, a_off, a_stride, out, o_off, o_stride):
    fn = lib().wo_softmax
    fn.argtypes = [c_int, POINTER(c_uint32), c_int, c_void_p, c_uint32, POINTER(c_uint32), c_void_p, c_uint32,
                   POINTER(c_uint32)]
    fn(len(shape), _u32(shape), axis, _p(a), a_off, _u32(a_stride), _p(out), o_off, _u32(o_stride))
    return out


def reduce(op, shape, axis, a, a_off, a_stride, out, o_off, o_stride):
    fn = lib().wo_reduce
    fn.argtypes = [c_int, c_int, POINTER(c_uint32), c_int, c_void_p, c_uint32, POINTER(c_uint32), c_void_p, c_uint32,
                   POINTER(c_uint32)]
    fn(op, len(shape), _u32(shape), axis, _p(a), a_off, _u32(a_stride), _p(out), o_off, _u32(o_stride))
    return out


def triu_fill(a, off, rows, cols, s0, s1, val, diagonal):
    fn = lib().wo_triu_fill
    fn.argtypes = [c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_uint32]
    fn(_p(a), off, rows, cols, s0, s1, c_float(val), diagonal)
    return a


def rope_tables(head_dim, max_seq_len, base=10000.0):
    """(cos, sin) float32 [max_seq_len, head_dim] (logical view of the column-major tables)."""
    cos_t = np.empty(max_seq_len * head_dim, dtype=np.float32)
    sin_t = np.empty_like(cos_t)
    fn = lib().wo_rope_tables
    fn.argtypes = [c_uint32, c_uint32, c_float, c_void_p, c_void_p]
    fn(head_dim, max_seq_len, c_float(base), _p(cos_t), _p(sin_t))
    return cos_t, sin_t


def rope_forward(x, cos_t, sin_t, max_seq_len, pos0=0):
    """x: [B, H, T, head_dim]; cos_t / sin_t: flat column-major tables from rope_tables."""
    x = _f32(x)
    B, H, T, d = x.shape
    out = np.empty_like(x)
    fn = lib().wo_rope_forward
    fn.argtypes = [c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]
    fn(_p(x), B, H, T, d, _p(cos_t), _p(sin_t), max_seq_len, pos0, _p(out))
    return out


# ---- activations and norms -----------------------------------------------------------------------

RELU, SIGMOID, TANH, GELU = 0, 1, 2, 3


def unary(op, x):
    x = _f32(x)
    out = np.empty_like(x)
    fn = lib().wo_unary
    fn.argtypes = [c_int, c_void_p, c_size_t, c_void_p]
    fn(op, _p(x), x.size, _p(out))
    return out


def silu_mul(gate, up):
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    fn = lib().wo_silu_mul
    fn.argtypes = [c_void_p, c_void_p, c_size_t, c_void_p]
    fn(_p(gate), _p(up), gate.size, _p(out))
    return out


def norm_epsilon():
    fn = lib().wo_norm_epsilon
    fn.restype = c_float
    return float(fn())


def rms_norm(x, w, eps=None):
    """x: [rows, n] (normalised along the last axis), w: [n]."""
    x, w = _f32(x), _f32(w)
    rows, n = x.shape
    out = np.empty_like(x)
    fn = lib().wo_rms_norm
    fn.argtypes = [c_void_p, c_size_t, c_size_t, c_void_p, c_float, c_void_p]
    fn(_p(x), rows, n, _p(w), c_float(norm_epsilon() if eps is None else eps), _p(out))
    return out


def layer_norm(x, gamma, beta, eps=None):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    rows, n = x.shape
    out = np.empty_like(x)
    fn = lib().wo_layer_norm
    fn.argtypes = [c_void_p, c_size_t, c_size_t, c_void_p, c_void_p, c_float, c_void_p]
    fn(_p(x), rows, n, _p(gamma), _p(beta), c_float(norm_epsilon() if eps is None else eps), _p(out))
    return out


# ---- decode attention ----------------------------------------------------------------------------

def decode_attn(kspec, vspec, kf, ka, vf, va, q, seq_lens, gqa_weed=True, Rk=None, Rv=None, want_scores=False):
    """kf, vf: uint8 [n_seq, Hkv, max_tokens, d]; ka, va: float32 [n_seq, Hkv, max_tokens] or None;
    q: [n_seq, Hq, d].  Returns out [n_seq, Hq, d] (and the scaled scores when asked)."""
    kf = np.ascontiguousarray(kf, dtype=np.uint8)
    vf = np.ascontiguousarray(vf, dtype=np.uint8)
    q = _f32(q)
    n_seq, Hkv, max_tokens, d = kf.shape
    Hq = q.shape[1]
    lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    g = AttnGeom(n_seq, Hq, Hkv, d, max_tokens, lens.ctypes.data_as(POINTER(c_int32)), int(gqa_weed),
                 int(Rk is not None), int(Rv is not None))
    ka_ = _f32(ka) if ka is not None else None
    va_ = _f32(va) if va is not None else None
    Rk_ = _f32(Rk).reshape(-1) if Rk is not None else None
    Rv_ = _f32(Rv).reshape(-1) if Rv is not None else None
    out = np.zeros((n_seq, Hq, d), dtype=np.float32)
    scores = np.zeros((n_seq, Hq, max_tokens), dtype=np.float32) if want_scores else None
    fn = lib().wo_decode_attn
    fn.argtypes = [POINTER(AttnGeom), POINTER(Coder), POINTER(Coder)] + [c_void_p] * 9
    fn(ctypes.byref(g), ctypes.byref(kspec.c), ctypes.byref(vspec.c), _p(kf), _p(ka_) if ka_ is not None else None,
       _p(vf), _p(va_) if va_ is not None else None, _p(q), _p(Rk_) if Rk_ is not None else None,
       _p(Rv_) if Rv_ is not None else None, _p(out), _p(scores) if scores is not None else None)
    return (out, scores) if want_scores else out
