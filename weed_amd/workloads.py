"""Seeded synthetic inputs for the five benchmark configurations (numpy, host side).

Shapes follow Weed's attention module: K, V are logical [n_seq, n_kv_heads, ctx, head_dim], q is
[n_seq, n_q_heads, head_dim] (src/modules/multihead_attention.cpp:155-161).  Used by tests, bench.py and the smoke
run so that all three see identical data for a given seed.
"""
import numpy as np


class Workload:
    def __init__(self, name, n_seq, n_q_heads, n_kv_heads, head_dim, lens, k_bits, v_bits, k_sign, v_sign, seed):
        self.name = name
        self.n_seq, self.n_q_heads, self.n_kv_heads, self.head_dim = n_seq, n_q_heads, n_kv_heads, head_dim
        self.lens = [int(x) for x in lens]
        self.k_bits, self.v_bits, self.k_sign, self.v_sign = k_bits, v_bits, k_sign, v_sign
        self.seed = seed

    @property
    def max_len(self):
        return max(self.lens)

    def row_bytes(self, lloydmax=True):
        """(K row bytes, V row bytes) of the packed cache: fields plus the fp32 row scale."""
        extra = 4 if lloydmax else 0
        return (self.head_dim * (self.k_bits + self.k_sign) // 8 + extra,
                self.head_dim * (self.v_bits + self.v_sign) // 8 + extra)

    def bytes_per_step(self, lloydmax=True):
        """Algorithmic bytes one decode step reads: every cached row once, whatever the GQA group size."""
        kb, vb = self.row_bytes(lloydmax)
        return sum(self.lens) * self.n_kv_heads * (kb + vb)

    def tensors(self, dtype=np.float32):
        """K, V: [n_seq, n_kv_heads, max_len, d] (rows beyond a sequence's length are unused), q: [n_seq, Hq, d]."""
        rng = np.random.default_rng(self.seed)
        shape = (self.n_seq, self.n_kv_heads, self.max_len, self.head_dim)
        K = rng.standard_normal(shape, dtype=np.float32)
        V = rng.standard_normal(shape, dtype=np.float32)
        q = rng.standard_normal((self.n_seq, self.n_q_heads, self.head_dim), dtype=np.float32)
        if self.name == "cfg2":
            # per-head scale drawn from U(0.5, 2)
            K *= rng.uniform(0.5, 2.0, size=(1, self.n_kv_heads, 1, 1)).astype(np.float32)
            V *= rng.uniform(0.5, 2.0, size=(1, self.n_kv_heads, 1, 1)).astype(np.float32)
        if self.name == "cfg3":
            # 1 % of the channels (at least one) scaled 10x: a fixed channel set from the seed
            n_out = max(1, self.head_dim // 100)
            ch = rng.choice(self.head_dim, size=n_out, replace=False)
            K[..., ch] *= 10.0
            V[..., ch] *= 10.0
        return K.astype(dtype, copy=False), V.astype(dtype, copy=False), q.astype(dtype, copy=False)


def config(index, seed=1234, scale=1.0, n_seq=None):
    """The five benchmark configurations, 1..5 (index 5 returns the encode half; see matmul_config for the dense half).

    `scale` < 1 shrinks context lengths (for tests that run the scalar CPU checker), `n_seq` overrides the number of
    side-by-side sequences for configurations 1-3 (the bench times many distinct caches per launch)."""
    def ctx(n):
        return max(1, int(round(n * scale)))

    if index == 1:
        return Workload("cfg1", n_seq or 1, 1, 1, 64, [ctx(512)] * (n_seq or 1), 4, 4, 1, 1, seed)
    if index == 2:
        return Workload("cfg2", n_seq or 1, 12, 12, 64, [ctx(1024)] * (n_seq or 1), 3, 4, 1, 0, seed)
    if index == 3:
        return Workload("cfg3", n_seq or 1, 32, 8, 128, [ctx(8192)] * (n_seq or 1), 3, 4, 0, 0, seed)
    if index == 4:
        rng = np.random.default_rng(seed + 4)
        lens = rng.integers(ctx(2048), ctx(32768) + 1, size=16)
        return Workload("cfg4", 16, 8, 8, 128, lens, 2, 3, 1, 0, seed)
    if index == 5:
        return Workload("cfg5", 1, 8, 8, 128, [ctx(4096)], 3, 3, 0, 0, seed)
    raise ValueError("configuration index must be 1..5")


def matmul_config(seed=1234, scale=1.0):
    """Configuration 5b: [4096 x 1024] . [1024 x 4096], A ~ N(0,1), W ~ N(0, 0.02), column-major operands."""
    rng = np.random.default_rng(seed + 5)
    M, K, N = (max(1, int(round(v * scale))) for v in (4096, 1024, 4096))
    A = rng.standard_normal((M, K), dtype=np.float32)
    W = (rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    return A, W
