// Quantized KV cache: allocation, encode-and-append, dequantise, export.
//
// Device twin of Weed::QuantizedKVCache (src/modules/multihead_attention.cpp:31-79) and of the encode half of
// MultiHeadAttention::forward (cpp:206-257).  Compiled with -ffp-contract=off: every multiply-add that must round
// twice (as the reference's x86-64 build does) is written as separate operations, every fused one as fmaf().
#include "kv_cache.h"
#include "kv_decode_mfma.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <new>

#include "lloyd_tables.inc"

using namespace weedhip;
using namespace weedkv;

namespace {

struct Geom4 {
    uint32_t off;
    uint32_t s[4];
};

struct BuiltinTable {
    const float *levels, *bounds, *refined;
};

BuiltinTable builtin_table(int bits)
{
    switch (bits) {
    case 1:
        return { WEED_LM_LEVELS_1, WEED_LM_BOUNDS_1, WEED_LM_REFINED_1 };
    case 2:
        return { WEED_LM_LEVELS_2, WEED_LM_BOUNDS_2, WEED_LM_REFINED_2 };
    case 3:
        return { WEED_LM_LEVELS_3, WEED_LM_BOUNDS_3, WEED_LM_REFINED_3 };
    default:
        return { WEED_LM_LEVELS_4, WEED_LM_BOUNDS_4, WEED_LM_REFINED_4 };
    }
}

// Round to the nearest IEEE binary16 value (ties to even), saturating at the largest finite one.
float round_to_half(float x)
{
    if (!std::isfinite(x)) {
        return x;
    }
    const float max_half = 65504.0f;
    if (std::fabs(x) >= max_half) {
        return std::copysign(max_half, x);
    }
    int e;
    (void)std::frexp(x, &e); // x = m * 2^e, 0.5 <= |m| < 1
    // binary16 keeps 11 significant bits for normal numbers (e >= -13), fewer below.
    int quantum_exp = e - 11;
    if (quantum_exp < -24) {
        quantum_exp = -24;
    }
    const float q = std::ldexp(1.0f, quantum_exp);
    return std::nearbyint(x / q) * q;
}

void load_builtin(Side &s)
{
    if (s.bits > 4) {
        return; // uniform coder only: its cells are arithmetic, no table
    }
    const BuiltinTable t = builtin_table(s.bits);
    const int n = 1 << s.bits;
    std::memcpy(s.levels, t.levels, sizeof(float) * n);
    std::memcpy(s.bounds, t.bounds, sizeof(float) * (n - 1));
    if (s.sign) {
        std::memcpy(s.recon, t.refined, sizeof(float) * 2 * n);
    } else {
        std::memcpy(s.recon, t.levels, sizeof(float) * n);
    }
}

// ------------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------------

__global__ void transpose_square_kernel(const float *__restrict__ r, float *__restrict__ rt, uint32_t d)
{
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= d * d) {
        return;
    }
    const uint32_t i = idx % d, j = idx / d;
    rt[j + d * i] = r[i + d * j];
}

// dst (column-major n x n) = src (column-major m x m, m <= n) in the leading block, identity in the rest.
__global__ void embed_square_kernel(const float *__restrict__ src, uint32_t m, float *__restrict__ dst, uint32_t n)
{
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * n) {
        return;
    }
    const uint32_t i = idx % n, j = idx / n;
    dst[idx] = (i < m && j < m) ? src[i + m * j] : (i == j ? 1.0f : 0.0f);
}

__global__ void bump_lens_kernel(int32_t *lens, int32_t seq_begin, int32_t seq_count, int32_t add)
{
    const int32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < seq_count) {
        lens[seq_begin + i] += add;
    }
}

// The last step of a small append, done by whichever workgroup of its last kernel finishes last: every workgroup of that
// kernel reads the lengths as they were before the append, so they may only move once all of them are through.
// `done` counts the workgroups that are (zero between appends: the last one puts it back).  Only for kernels of at
// most kBumpWorkgroups workgroups: the additions to one counter come in one after the other, and two thousand of
// them doubled the time of a prefill's encoder.  Larger appends end with bump_lens_kernel.
constexpr uint32_t kBumpWorkgroups = 128;
struct LensBump {
    uint32_t *done; // null: a later kernel of this append moves the lengths
    int32_t *lens;
    int32_t seq_begin, seq_count, add;
    uint32_t workgroups;
};
__device__ __forceinline__ void bump_lens_when_last(const LensBump &b)
{
    if (!b.done) {
        return;
    }
    __shared__ uint32_t arrived;
    __syncthreads(); // the loads of lens by this workgroup have returned: their values were used above
    if (threadIdx.x == 0) {
        arrived = __hip_atomic_fetch_add(b.done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (arrived + 1 != b.workgroups) {
        return;
    }
    for (int32_t i = (int32_t)threadIdx.x; i < b.seq_count; i += (int32_t)blockDim.x) {
        b.lens[b.seq_begin + i] += b.add;
    }
    if (threadIdx.x == 0) {
        __hip_atomic_store(b.done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

__global__ void fill_i32_kernel(int32_t *p, int32_t v, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// A load of a float through a buffer descriptor: the lane's 32-bit byte offset and one that is the same in every
// lane, so that a batch of loads needs no address arithmetic per load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const float *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buffer_f32(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, (int)uniform_off, 0));
}

struct CoderParams {
    int mode;
    int bits;
    int sign;
    float block_scale;
    float bounds[15];
    float levels[16];
};

// The bucket arithmetic of QuantizedKVCache::write_row (multihead_attention.cpp:49-58), operation for operation.
__device__ __forceinline__ uint32_t uniform_bucket(float v, float lo, float hi, float step, int levels)
{
    int bucket = 0;
    if (step > 1e-8f) {
        const float hs = hi - step;
        const float m = (v < hs) ? v : hs;
        const float clamped = (lo < m) ? m : lo;
        bucket = (int)((clamped - lo) / step);
        bucket = bucket > levels - 1 ? levels - 1 : bucket;
        bucket = bucket < 0 ? 0 : bucket;
    }
    return (uint32_t)bucket;
}

constexpr int kEncRows = 32;     // rows per workgroup
constexpr int kEncThreads = 256;

// Rotate (optional) and quantise kEncRows rows of a strided [S, Hkv, T, d] tensor into one field per byte.
//   rotate 0: y = x            1: y = x.R on the matrix cores (fp32)        2: y = x.R with the reference's
//   rounding (multiply, then add, i ascending: src/ops/matmul.cpp:40-44).
// PARTS = number of row slices the 256 threads are split into (each thread owns one output column of its slice).
// `block` = index of the workgroup among those that work on this tensor.
// Where an append whose rows fill whole 32-token half blocks, or one that adds one token per sequence, goes directly
// (see encode_rows_body): the cache side's own arrays.  `out` null: the rows go to the scratch arrays and a second
// kernel packs them.
struct DirectOut {
    uint8_t *out;        // packed fields of the side
    uint64_t region_bytes;
    float *alpha;        // [region][padded] row scales, null for the uniform coder
    uint32_t *alpha_max; // [region][kScaleMaxSlots] largest row scale (V side), or null
    const int32_t *lens; // cached lengths BEFORE this append
    int32_t seq_begin;
    uint32_t padded, w;
    int is_v;
};

// The kEncRows = 32 staged rows are tokens [n0, n0 + 32) of one (sequence, head), n0 a multiple of 32: one half of a
// 64-token block.  Every K item (8 coordinates of a token) and every V item (8 tokens of a coordinate, all inside
// this half) is assembled from LDS and written to its place; nothing already cached shares an item with them.
__device__ __forceinline__ void write_half_block(const uint8_t *staged, const DirectOut &o, uint32_t Hkv, uint32_t T,
                                                 uint32_t d, uint32_t row0)
{
    const uint32_t h = (row0 / T) % Hkv, sq = row0 / (T * Hkv);
    const uint64_t region = (uint64_t)(o.seq_begin + (int32_t)sq) * Hkv + h;
    const uint32_t n0 = (uint32_t)o.lens[o.seq_begin + (int32_t)sq] + row0 % T;
    const uint32_t w = o.w;
    // the half's block; items of w bytes are stored whole where w is a power of two, else byte by byte
    uint8_t *base = o.out + region * o.region_bytes + (uint64_t)(n0 >> 6) * block_bytes(d, w);
    auto store_item = [&](uint8_t *dst, uint32_t lo, uint32_t hi) { // fields 0..3 in lo, 4..7 in hi, 4 w bits each
        const uint64_t bits = (uint64_t)lo | ((uint64_t)hi << (4 * w));
        if (w == 4) {
            *reinterpret_cast<uint32_t *>(dst) = (uint32_t)bits;
        } else if (w == 8) {
            *reinterpret_cast<uint2 *>(dst) = uint2{ lo, hi };
        } else if (w == 2) {
            *reinterpret_cast<uint16_t *>(dst) = (uint16_t)bits;
        } else {
            for (uint32_t b = 0; b < w; ++b) {
                dst[b] = (uint8_t)(bits >> (8 * b));
            }
        }
    };
    // (small quotients by multiplication with the rounded reciprocal: (x + 0.5) / n is never closer than 0.5 / n to an
    // integer, and x stays below 1024)
    if (!o.is_v) {
        // item `it` of row r: coordinates 8 it .. 8 it + 7, which are item it % (d / 32) of lane group it / (d / 32)
        const uint32_t ipl = d / 32, items = 4 * ipl;
        const float inv_items = 1.0f / (float)items, inv_ipl = 1.0f / (float)ipl;
        for (uint32_t idx = threadIdx.x; idx < kEncRows * items; idx += kEncThreads) {
            const uint32_t r = (uint32_t)(((float)idx + 0.5f) * inv_items), it = idx - r * items;
            const uint32_t gq = (uint32_t)(((float)it + 0.5f) * inv_ipl), ks = it - gq * ipl;
            const uint2 f = *reinterpret_cast<const uint2 *>(staged + (uint64_t)r * d + it * 8); // 8-byte aligned
            const uint32_t lo = (f.x & 0xffu) | (((f.x >> 8) & 0xffu) << w) | (((f.x >> 16) & 0xffu) << (2 * w)) |
                                ((f.x >> 24) << (3 * w));
            const uint32_t hi = (f.y & 0xffu) | (((f.y >> 8) & 0xffu) << w) | (((f.y >> 16) & 0xffu) << (2 * w)) |
                                ((f.y >> 24) << (3 * w));
            const uint32_t n = n0 + r, t = (n >> 4) & 3, r16 = n & 15;
            store_item(base + (((gq * 16 + r16) * 4 + t) * ipl + ks) * w, lo, hi);
        }
        return;
    }
    // item of coordinate j and lane group gq: the tokens 4 gq .. 4 gq + 3 of the half's two 16-token tiles
    const uint32_t u = (n0 >> 5) & 1U;
    const float inv_d = 1.0f / (float)d;
    for (uint32_t idx = threadIdx.x; idx < 4 * d; idx += kEncThreads) {
        const uint32_t gq = (uint32_t)(((float)idx + 0.5f) * inv_d), j = idx - gq * d;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e) {
            // token of field e inside this half: rows 4g .. 4g+3 of its first tile, then of its second
            lo |= (uint32_t)staged[(uint64_t)(4 * gq + e) * d + j] << (e * w);
            hi |= (uint32_t)staged[(uint64_t)(16 + 4 * gq + e) * d + j] << (e * w);
        }
        store_item(base + (((gq * 16 + (j & 15)) * 2 + u) * (d / 16) + (j >> 4)) * w, lo, hi);
    }
}

// What a thread of a V-side workgroup knows of the items its fields will join, asked for as soon as the lengths are
// there (the rotation runs while these loads are under way): where each run of items starts, the bit its field
// starts at, and the byte of every item that the field starts in.  A task is a row and a coordinate mod 16: the
// items of its d / 16 coordinates follow each other in memory, w bytes each.
struct ScatterV {
    static constexpr uint32_t kPasses = kEncRows * 16 / kEncThreads; // tasks per thread
    static_assert(kEncRows * 16 % kEncThreads == 0, "whole passes over (row, coordinate mod 16)");
    uint8_t *dst[kPasses]; // null: no such row
    uint32_t bit[kPasses];
    uint32_t old[kPasses][16]; // head_dim <= 256: at most 16 items per run
};
__device__ __forceinline__ void request_scattered_v(ScatterV &pre, const uint32_t *tok_s, const DirectOut &o,
                                                    uint32_t Hkv, uint32_t d, uint32_t row0, uint32_t rows)
{
    const uint32_t w = o.w, per = d / 16;
    const uint64_t region0 = (uint64_t)o.seq_begin * Hkv + row0; // T = 1: one row per region, in region order
#pragma unroll
    for (uint32_t pass = 0; pass < ScatterV::kPasses; ++pass) {
        const uint32_t idx = threadIdx.x + pass * kEncThreads;
        const uint32_t r = idx >> 4, c = idx & 15;
        pre.dst[pass] = nullptr;
        if (row0 + r < rows) {
            const FieldPos p = v_field_pos(tok_s[r], c, d, w);
            pre.dst[pass] = o.out + (region0 + r) * o.region_bytes + p.byte;
            pre.bit[pass] = p.bit;
#pragma unroll
            for (uint32_t jb = 0; jb < 16; ++jb) {
                pre.old[pass][jb] = ((p.bit & 7) && jb < per) ? pre.dst[pass][jb * w + (p.bit >> 3)] : 0u;
            }
        }
    }
}

// One new token per sequence (T = 1): staged row r is token tok_s[r] (the sequence's length so far) of region
// row0 + r.  Its K items are whole (8 coordinates of the token).  Each of its V fields joins the item of its
// coordinate: the bytes below the field stay as they are (the tokens already cached sit below it in the item), the
// byte the field starts in keeps its low bits, and what lies above becomes the field and zeros.  No two rows share
// an item.
__device__ __forceinline__ void write_scattered(const uint8_t *staged, const uint32_t *tok_s, const ScatterV &pre,
                                                const DirectOut &o, uint32_t Hkv, uint32_t d, uint32_t row0,
                                                uint32_t rows)
{
    const uint32_t w = o.w;
    const uint64_t region0 = (uint64_t)o.seq_begin * Hkv + row0; // T = 1: one row per region, in region order
    if (!o.is_v) {
        const uint32_t items = d / 8;
        for (uint32_t idx = threadIdx.x; idx < kEncRows * items; idx += kEncThreads) {
            const uint32_t r = idx / items, it = idx - r * items;
            if (row0 + r >= rows) {
                break;
            }
            uint8_t bytes[8];
            item_build(staged + (uint64_t)r * d + it * 8, w, bytes);
            uint8_t *dst = o.out + (region0 + r) * o.region_bytes + k_field_pos(tok_s[r], it * 8, d, w).byte;
            for (uint32_t b = 0; b < w; ++b) {
                dst[b] = bytes[b];
            }
        }
        return;
    }
    const uint32_t per = d / 16;
#pragma unroll
    for (uint32_t pass = 0; pass < ScatterV::kPasses; ++pass) {
        if (!pre.dst[pass]) {
            break;
        }
        const uint32_t idx = threadIdx.x + pass * kEncThreads;
        const uint32_t r = idx >> 4, c = idx & 15;
        const uint32_t b0 = pre.bit[pass] >> 3, low = pre.bit[pass] & 7;
#pragma unroll
        for (uint32_t jb = 0; jb < 16; ++jb) {
            if (jb < per) {
                const uint32_t f = staged[(uint64_t)r * d + 16 * jb + c];
                uint32_t bits = (pre.old[pass][jb] & ((1u << low) - 1u)) | (f << low); // w <= 8: at most 15 bits
                for (uint32_t b = b0; b < w; ++b) {
                    pre.dst[pass][jb * w + b] = (uint8_t)bits;
                    bits >>= 8;
                }
            }
        }
    }
}

// Lloyd-Max fields of the staged rows: code = number of thresholds at or below the scaled coordinate (they ascend, so
// the level of that code is the one behind the last threshold passed), then the sign bit against that level.  Four
// consecutive coordinates per thread, stored as one 32-bit word (d is a multiple of 32, the destination is 4-byte
// aligned and its rows are d bytes long).
template <int BITS>
__device__ __forceinline__ void lloyd_fields(const float *ys, uint32_t pitch, const float *inv_s, const CoderParams &cp,
                                             uint8_t *fdst, uint32_t d, uint32_t row0, uint32_t rows)
{
    constexpr int NB = (1 << BITS) - 1;
    float bound[NB], level[NB + 1];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
        bound[k] = cp.bounds[k];
    }
#pragma unroll
    for (int k = 0; k <= NB; ++k) {
        level[k] = cp.levels[k];
    }
    const uint32_t tid = threadIdx.x, jl = tid & 31;
    if (!cp.sign) {
        for (uint32_t r = tid >> 5; r < kEncRows && row0 + r < rows; r += kEncThreads / 32) {
            const float inv = inv_s[r];
            for (uint32_t j = 4 * jl; j < d; j += 128) {
                uint32_t word = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float u = ys[r * pitch + j + i] * inv;
                    uint32_t code = 0;
#pragma unroll
                    for (int k = 0; k < NB; ++k) {
                        code += (u >= bound[k]) ? 1u : 0u;
                    }
                    word |= code << (8 * i);
                }
                *reinterpret_cast<uint32_t *>(fdst + (uint64_t)r * d + j) = word;
            }
        }
        return;
    }
    for (uint32_t r = tid >> 5; r < kEncRows && row0 + r < rows; r += kEncThreads / 32) {
        const float inv = inv_s[r];
        for (uint32_t j = 4 * jl; j < d; j += 128) {
            uint32_t word = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float u = ys[r * pitch + j + i] * inv;
                uint32_t code = 0;
                float lvl = level[0];
#pragma unroll
                for (int k = 0; k < NB; ++k) {
                    const bool ge = u >= bound[k];
                    code += ge ? 1u : 0u;
                    lvl = ge ? level[k + 1] : lvl;
                }
                word |= ((code << 1) | ((u >= lvl) ? 1u : 0u)) << (8 * i);
            }
            *reinterpret_cast<uint32_t *>(fdst + (uint64_t)r * d + j) = word;
        }
    }
}

// ONE: an append of one token per sequence, which this kernel finishes itself (write_scattered).
template <int PARTS, bool ONE>
__device__ __forceinline__ void encode_rows_body(const float *__restrict__ x, const Geom4 &g, uint32_t Hkv, uint32_t T,
                                                 uint32_t d, uint32_t d_real, uint32_t rows,
                                                 const float *__restrict__ rot_t, int rotate, const CoderParams &cp,
                                                 uint8_t *__restrict__ fields, float *__restrict__ alpha_out,
                                                 const DirectOut &direct, uint32_t block)
{
    // d: head_dim as stored (a multiple of 32); d_real <= d: coordinates the caller's rows have, the rest are zeros
    extern __shared__ float smem[];
    const uint32_t pitch = d + 1;
    float *xs = smem;                   // [kEncRows][pitch]
    float *ys = smem + kEncRows * pitch; // [kEncRows][pitch]
    float *inv_s = ys + kEncRows * pitch; // [kEncRows]
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = block * kEncRows;

    // gather the rows (logical row = (s*Hkv + h)*T + t): the first 32 threads work out where their row starts, then
    // thread (tid / 32, tid % 32) walks rows tid / 32, +8, ... and columns tid % 32, +32, ... (no divisions per element)
    unsigned long long *row_base = reinterpret_cast<unsigned long long *>(inv_s + kEncRows); // [kEncRows], 8-byte aligned
    uint32_t *tok_s = reinterpret_cast<uint32_t *>(row_base + kEncRows); // [kEncRows] tokens cached so far (T = 1 appends)
    // the first 128 steps of the rotation's columns for this wavefront's first tile, in flight during the gather
    float bpre[64];
    const bool prefetched = ONE && rotate == 1 && d >= 128 && (tid >> 6) < d / 32;
    if (prefetched) {
        const __amdgpu_buffer_rsrc_t rot = buffer_of(rot_t, 4 * d * d);
        const uint32_t at = 4 * (32 * (tid >> 6) + (tid & 31) + d * ((tid & 63) >> 5));
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            bpre[u] = buffer_f32(rot, at, 8 * d * u);
        }
    }
    uint32_t cached = 0;
    if (tid < kEncRows) {
        const uint32_t row = row0 + tid;
        unsigned long long base = ~0ull;
        if (row < rows) {
            const uint32_t t = row % T;
            const uint32_t h = (row / T) % Hkv;
            const uint32_t s = row / (T * Hkv);
            base = (uint64_t)g.off + (uint64_t)s * g.s[0] + (uint64_t)h * g.s[1] + (uint64_t)t * g.s[2];
        }
        row_base[tid] = base;
        if (ONE && row < rows) {
            cached = (uint32_t)direct.lens[direct.seq_begin + (int32_t)(row / Hkv)]; // in flight during the gather
        }
    }
    __syncthreads();
    {
        float *dst = rotate ? xs : ys;
        const uint32_t jl = tid & 31;
        // rows that are contiguous and 16-byte aligned (the usual case) come in four coordinates per load
        const bool wide = g.s[3] == 1 && d_real % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                          ((g.off | g.s[0] | g.s[1] | g.s[2]) & 3) == 0;
        if (wide) {
            float4 v[kEncRows / (kEncThreads / 32)];
            for (uint32_t j = 4 * jl; j < d; j += 128) {
#pragma unroll
                for (uint32_t i = 0; i < kEncRows / (kEncThreads / 32); ++i) {
                    const unsigned long long base = row_base[(tid >> 5) + i * (kEncThreads / 32)];
                    v[i] = (base != ~0ull && j < d_real) ? *reinterpret_cast<const float4 *>(x + base + j)
                                                         : float4{ 0.0f, 0.0f, 0.0f, 0.0f };
                }
#pragma unroll
                for (uint32_t i = 0; i < kEncRows / (kEncThreads / 32); ++i) {
                    float *at = dst + ((tid >> 5) + i * (kEncThreads / 32)) * pitch + j;
                    at[0] = v[i].x;
                    at[1] = v[i].y;
                    at[2] = v[i].z;
                    at[3] = v[i].w;
                }
            }
        } else {
            for (uint32_t r = tid >> 5; r < kEncRows; r += kEncThreads / 32) {
                const unsigned long long base = row_base[r];
                for (uint32_t j = jl; j < d; j += 32) {
                    dst[r * pitch + j] = (base != ~0ull && j < d_real) ? x[base + (uint64_t)j * g.s[3]] : 0.0f;
                }
            }
        }
    }
    if (ONE && tid < kEncRows) {
        tok_s[tid] = cached;
    }
    __syncthreads();
    [[maybe_unused]] ScatterV pre;
    if constexpr (ONE) {
        if (direct.is_v) {
            request_scattered_v(pre, tok_s, direct, Hkv, d, row0, rows);
        }
    }

    if (rotate == 1) {
        // y = x . R on the matrix cores: each wavefront owns 32-column tiles of the 32 x d result and walks the
        // contraction two coordinates at a time (v_mfma_f32_32x32x2f32: lane l feeds row/column l % 32 of step
        // k = l / 32).  Sums are in a different order than the scalar loop below, as rotate = 1 allows.
        typedef float float16v __attribute__((ext_vector_type(16)));
        static_assert(kEncRows == 32, "one 32-row matrix tile per workgroup");
        const uint32_t lane = tid & 63, wave = tid >> 6;
        const uint32_t l32 = lane & 31, khalf = lane >> 5;
        for (uint32_t tile = wave; tile < d / 32; tile += kEncThreads / 64) {
            float16v acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc[i] = 0.0f;
            }
            // R[k][32*tile + l32] = rot_t[col + d*k]: the lane's part of the address is its column and its half of
            // the step, the step itself is the same in every lane
            const __amdgpu_buffer_rsrc_t rot = buffer_of(rot_t, 4 * d * d);
            const uint32_t at = 4 * (32 * tile + l32 + d * khalf);
            // d is a multiple of 32: sixty-four steps at a time where d allows (the loads of the rotation come from
            // L2 and are the long pole: as many as possible are issued together), else sixteen
            uint32_t k0 = 0;
            for (; k0 + 128 <= d; k0 += 128) {
                float b[64];
                if (prefetched && tile == wave && k0 == 0) {
#pragma unroll
                    for (int u = 0; u < 64; ++u) {
                        b[u] = bpre[u];
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < 64; ++u) {
                        b[u] = buffer_f32(rot, at, 4 * d * (k0 + 2 * u));
                    }
                }
#pragma unroll
                for (int u = 0; u < 64; ++u) {
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[l32 * pitch + k0 + 2 * u + khalf], b[u], acc, 0, 0, 0);
                }
            }
            for (; k0 < d; k0 += 32) {
                float a[16], b[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    a[u] = xs[l32 * pitch + k0 + 2 * u + khalf];
                    b[u] = buffer_f32(rot, at, 4 * d * (k0 + 2 * u));
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t r = 8 * (i / 4) + 4 * khalf + (i % 4);
                ys[r * pitch + 32 * tile + l32] = acc[i];
            }
        }
        __syncthreads();
    } else if (rotate) {
        constexpr int RPP = kEncRows / PARTS; // rows per part
        const uint32_t j = tid % d;
        const uint32_t part = tid / d;
        if (part < PARTS) {
            float acc[RPP];
#pragma unroll
            for (int r = 0; r < RPP; ++r) {
                acc[r] = 0.0f;
            }
            const float *xrow = xs + part * RPP * pitch;
            // the reference's order and rounding: multiply, then add, i ascending
            for (uint32_t i = 0; i < d; ++i) {
                const float rv = rot_t[j + d * i];
#pragma unroll
                for (int r = 0; r < RPP; ++r) {
                    acc[r] = acc[r] + xrow[r * pitch + i] * rv;
                }
            }
#pragma unroll
            for (int r = 0; r < RPP; ++r) {
                ys[(part * RPP + r) * pitch + j] = acc[r];
            }
        }
        __syncthreads();
    }

    // one field per byte: into the scratch array, or (direct append) into LDS where xs was, [kEncRows][d]
    uint8_t *staged = reinterpret_cast<uint8_t *>(xs);
    uint8_t *fdst = direct.out ? staged : fields + (uint64_t)row0 * d;

    if (cp.mode == WEED_HIP_KV_UNIFORM) {
        const int levels = 1 << cp.bits;
        const float lo = -3.0f * cp.block_scale;
        const float hi = 3.0f * cp.block_scale;
        const float step = (hi - lo) / (float)levels;
        const uint32_t jl = tid & 31;
        for (uint32_t r = tid >> 5; r < kEncRows && row0 + r < rows; r += kEncThreads / 32) {
            for (uint32_t j = jl; j < d; j += 32) {
                fdst[(uint64_t)r * d + j] = (uint8_t)uniform_bucket(ys[r * pitch + j], lo, hi, step, levels);
            }
        }
        if (direct.out) {
            __syncthreads();
            if constexpr (ONE) {
                write_scattered(staged, tok_s, pre, direct, Hkv, d, row0, rows);
            } else {
                write_half_block(staged, direct, Hkv, T, d, row0);
            }
        }
        return;
    }

    // LLOYDMAX: row scale from an fma-accumulated sum of squares, j ascending
    if (tid < kEncRows) {
        float n2 = 0.0f;
        for (uint32_t j0 = 0; j0 < d; j0 += 16) { // d is a multiple of 32
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                v[u] = ys[tid * pitch + j0 + u];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                n2 = fmaf(v[u], v[u], n2);
            }
        }
        const float norm = sqrtf(n2);
        const float sqrt_d = sqrtf((float)d_real);
        float inv = 0.0f, a = 0.0f;
        if (norm > 1e-30f) {
            inv = sqrt_d / norm;
            a = norm / sqrt_d;
        }
        inv_s[tid] = inv;
        if (ONE) {
            // one row per (sequence, head): scale to its token slot, and into the region's largest scale
            if (row0 + tid < rows) {
                const uint32_t region = (uint32_t)direct.seq_begin * Hkv + row0 + tid;
                direct.alpha[(uint64_t)region * direct.padded + tok_s[tid]] = a;
                if (direct.alpha_max) {
                    atomicMax(direct.alpha_max + (uint64_t)region * kScaleMaxSlots, __float_as_uint(fabsf(a)));
                }
            }
        } else if (direct.out) {
            // all kEncRows rows belong to one (sequence, head): scale to its token slot, largest scale to the region
            const uint32_t h = (row0 / T) % Hkv, sq = row0 / (T * Hkv);
            const uint32_t region = (uint32_t)(direct.seq_begin + (int32_t)sq) * Hkv + h;
            const uint32_t n = (uint32_t)direct.lens[direct.seq_begin + (int32_t)sq] + row0 % T + tid;
            direct.alpha[(uint64_t)region * direct.padded + n] = a;
            if (direct.alpha_max) {
                uint32_t bits = __float_as_uint(fabsf(a));
                for (int o = 16; o > 0; o >>= 1) {
                    bits = max(bits, (uint32_t)__shfl_xor((int)bits, o));
                }
                if (tid == 0) {
                    // (the half blocks of a region take the words in turn)
                    atomicMax(direct.alpha_max + (uint64_t)region * kScaleMaxSlots + (n >> 5) % kScaleMaxSlots, bits);
                }
            }
        } else if (row0 + tid < rows) {
            alpha_out[row0 + tid] = a;
        }
    }
    __syncthreads();
    // one instance per code width: its thresholds (and, with a sign bit, its levels) sit in registers and nothing is
    // compared against a threshold that the width does not have
    switch (cp.bits) {
    case 1:
        lloyd_fields<1>(ys, pitch, inv_s, cp, fdst, d, row0, rows);
        break;
    case 2:
        lloyd_fields<2>(ys, pitch, inv_s, cp, fdst, d, row0, rows);
        break;
    case 3:
        lloyd_fields<3>(ys, pitch, inv_s, cp, fdst, d, row0, rows);
        break;
    default:
        lloyd_fields<4>(ys, pitch, inv_s, cp, fdst, d, row0, rows);
        break;
    }
    if (direct.out) {
        __syncthreads();
        if constexpr (ONE) {
            write_scattered(staged, tok_s, pre, direct, Hkv, d, row0, rows);
        } else {
            write_half_block(staged, direct, Hkv, T, d, row0);
        }
    }
}

// K and V of an append in ONE launch (the first `blocks_per_side` workgroups take K, the rest V): the appends of a
// decode step are a chain of small kernels whose launches cost more than their work.
struct EncSide {
    const float *x;
    Geom4 g;
    const float *rot_t;
    CoderParams cp;
    uint8_t *fields;
    float *alpha_out;
    DirectOut direct;
};
template <int PARTS, bool ONE>
__global__ void __launch_bounds__(kEncThreads)
    encode_rows_pair_kernel(EncSide k, EncSide v, uint32_t blocks_per_side, uint32_t Hkv, uint32_t T, uint32_t d,
                            uint32_t d_real, uint32_t rows, int rotate, LensBump bump)
{
    if (blockIdx.x < blocks_per_side) {
        encode_rows_body<PARTS, ONE>(k.x, k.g, Hkv, T, d, d_real, rows, k.rot_t, rotate, k.cp, k.fields, k.alpha_out,
                                     k.direct, blockIdx.x);
    } else {
        encode_rows_body<PARTS, ONE>(v.x, v.g, Hkv, T, d, d_real, rows, v.rot_t, rotate, v.cp, v.fields, v.alpha_out,
                                     v.direct, blockIdx.x - blocks_per_side);
    }
    bump_lens_when_last(bump);
}

// One thread per (new row, item of 8 coordinates): 8 bytes in, w bytes out.
__device__ __forceinline__ void pack_k_body(const uint8_t *__restrict__ fields, const float *__restrict__ alpha_in,
                                            uint32_t rows, uint32_t Hkv, uint32_t T, uint32_t d, uint32_t w,
                                            int32_t seq_begin, const int32_t *__restrict__ lens,
                                            uint8_t *__restrict__ out, uint64_t region_bytes,
                                            float *__restrict__ alpha_out, uint32_t padded, uint32_t block)
{
    const uint32_t items = d / 8;
    const uint32_t idx = block * blockDim.x + threadIdx.x;
    if (idx >= rows * items) {
        return;
    }
    const uint32_t it = idx % items, row = idx / items;
    const uint32_t t = row % T, h = (row / T) % Hkv, s = row / (T * Hkv);
    const uint32_t n = (uint32_t)lens[seq_begin + s] + t;
    uint8_t bytes[8];
    item_build(fields + (uint64_t)row * d + it * 8, w, bytes);
    const uint64_t region = (uint64_t)(seq_begin + s) * Hkv + h;
    uint8_t *dst = out + region * region_bytes + k_field_pos(n, it * 8, d, w).byte;
    for (uint32_t b = 0; b < w; ++b) {
        dst[b] = bytes[b];
    }
    if (alpha_out && it == 0) {
        alpha_out[region * padded + n] = alpha_in[row];
    }
}

// Row scales of the new V rows: one thread per new row copies the scale to its token slot and the region's largest
// scale is kept up to date (one atomic per wavefront and region, not one per row).
__device__ __forceinline__ void scatter_v_scales_body(const float *__restrict__ alpha_in, uint32_t rows, uint32_t Hkv,
                                                      uint32_t T, int32_t seq_begin, const int32_t *__restrict__ lens,
                                                      float *__restrict__ alpha_out, uint32_t *__restrict__ alpha_max,
                                                      uint32_t padded, uint32_t block)
{
    const uint32_t row = block * blockDim.x + threadIdx.x;
    const bool valid = row < rows;
    uint32_t region = 0xffffffffu, bits = 0;
    if (valid) {
        const uint32_t t = row % T, h = (row / T) % Hkv, s = row / (T * Hkv);
        const float a = alpha_in[row];
        region = (uint32_t)(seq_begin + s) * Hkv + h;
        alpha_out[(uint64_t)region * padded + (uint32_t)lens[seq_begin + s] + t] = a;
        bits = __float_as_uint(fabsf(a));
    }
    // lanes of a wavefront that share the first valid lane's region fold their maximum into one atomic
    const uint32_t lead = __builtin_amdgcn_readfirstlane(region);
    uint32_t mine = (valid && region == lead) ? bits : 0u;
    for (int o = 32; o > 0; o >>= 1) {
        mine = max(mine, (uint32_t)__shfl_xor((int)mine, o));
    }
    if (valid) {
        // (the wavefronts take the region's words in turn)
        const uint32_t slot = (row >> 6) % kScaleMaxSlots;
        if (region != lead) {
            atomicMax(alpha_max + (uint64_t)region * kScaleMaxSlots + slot, bits);
        } else if ((threadIdx.x & 63) == (uint32_t)__builtin_ctzll(__ballot(valid && region == lead))) {
            atomicMax(alpha_max + (uint64_t)region * kScaleMaxSlots + slot, mine);
        }
    }
}

// One thread per (sequence, kv head, 32-token half block, lane group, coordinate): rebuilds one item of 8 tokens,
// keeping the fields of tokens that were already cached and zeroing those not yet written.
__device__ __forceinline__ void pack_v_body(const uint8_t *__restrict__ fields, uint32_t S, uint32_t Hkv, uint32_t T,
                                            uint32_t d, uint32_t w, int32_t seq_begin, const int32_t *__restrict__ lens,
                                            uint32_t halves, uint8_t *__restrict__ out, uint64_t region_bytes,
                                            uint32_t wg)
{
    const uint64_t idx = (uint64_t)wg * blockDim.x + threadIdx.x;
    const uint64_t total = (uint64_t)S * Hkv * halves * 4 * d;
    if (idx >= total) {
        return;
    }
    const uint32_t j = (uint32_t)(idx % d);
    const uint32_t g = (uint32_t)((idx / d) % 4);
    const uint32_t hf = (uint32_t)((idx / (4ull * d)) % halves);
    const uint32_t h = (uint32_t)((idx / (4ull * d * halves)) % Hkv);
    const uint32_t s = (uint32_t)(idx / (4ull * d * halves * Hkv));
    const uint32_t old_len = (uint32_t)lens[seq_begin + s];
    const uint32_t new_len = old_len + T;
    const uint32_t half = old_len / 32 + hf; // halves are 32 consecutive tokens
    const uint32_t block = half >> 1, u = half & 1;
    const uint32_t tok0 = block * 64;
    if (tok0 + 32 * u >= new_len) {
        return;
    }
    const uint64_t region = (uint64_t)(seq_begin + s) * Hkv + h;
    // all 8 tokens of the item share block, u, g and the coordinate, hence the item address
    const FieldPos p0 = v_field_pos(tok0 + v_item_token(u, g, 0), j, d, w);
    uint8_t *dst = out + region * region_bytes + p0.byte;
    uint8_t f8[8];
    bool touched = false;
    for (uint32_t e = 0; e < 8; ++e) {
        const uint32_t n = tok0 + v_item_token(u, g, e);
        if (n < old_len) {
            f8[e] = (uint8_t)item_get(dst, e * w, w);
        } else if (n < new_len) {
            const uint32_t row = (s * Hkv + h) * T + (n - old_len);
            f8[e] = fields[(uint64_t)row * d + j];
            touched = true;
        } else {
            f8[e] = 0;
        }
    }
    if (!touched) {
        return;
    }
    uint8_t bytes[8];
    item_build(f8, w, bytes);
    for (uint32_t b = 0; b < w; ++b) {
        dst[b] = bytes[b];
    }
}

// The three packing steps of an append in ONE launch: workgroups [0, bk) pack the K items, [bk, bk + bv) rebuild the
// V items, the rest store the V row scales.  All of them read the sequence lengths as they were before the append.
struct PackArgs {
    const uint8_t *k_fields, *v_fields; // one field per byte, as the encoder left them
    const float *k_alpha_in, *v_alpha_in;
    uint32_t rows, S, Hkv, T, d, wk, wv, halves, padded;
    int32_t seq_begin;
    const int32_t *lens;
    uint8_t *k_out, *v_out;
    uint64_t k_region_bytes, v_region_bytes;
    float *k_alpha_out, *v_alpha_out; // null: the coder has no row scales
    uint32_t *v_alpha_max;
    uint32_t blocks_k, blocks_v;
    LensBump bump;
};
__global__ void __launch_bounds__(256) pack_all_kernel(PackArgs a)
{
    if (blockIdx.x < a.blocks_k) {
        pack_k_body(a.k_fields, a.k_alpha_in, a.rows, a.Hkv, a.T, a.d, a.wk, a.seq_begin, a.lens, a.k_out,
                    a.k_region_bytes, a.k_alpha_out, a.padded, blockIdx.x);
    } else if (blockIdx.x < a.blocks_k + a.blocks_v) {
        pack_v_body(a.v_fields, a.S, a.Hkv, a.T, a.d, a.wv, a.seq_begin, a.lens, a.halves, a.v_out, a.v_region_bytes,
                    blockIdx.x - a.blocks_k);
    } else {
        scatter_v_scales_body(a.v_alpha_in, a.rows, a.Hkv, a.T, a.seq_begin, a.lens, a.v_alpha_out, a.v_alpha_max,
                              a.padded, blockIdx.x - a.blocks_k - a.blocks_v);
    }
    bump_lens_when_last(a.bump);
}

__device__ __forceinline__ uint32_t load_field(const SideParams &sp, int which, uint64_t region, uint32_t n, uint32_t j,
                                               uint32_t d)
{
    const uint8_t *base = sp.fields + region * sp.region_bytes;
    const FieldPos p = which ? v_field_pos(n, j, d, sp.w) : k_field_pos(n, j, d, sp.w);
    return item_get(base + p.byte, p.bit, sp.w);
}

// mode 0: dense fp32 (read_row, multihead_attention.cpp:64-79: lo + (code + 0.5) * step, two roundings);
// mode 1: one field per byte (+ row scales).
__global__ void unpack_kernel(SideParams sp, int which, int kv_mode, uint32_t Hkv, uint32_t d, uint32_t d_stored,
                              uint32_t padded, int32_t seq_begin, uint32_t S, uint32_t tok_begin, uint32_t T, int out_mode,
                              float *__restrict__ out_f, Geom4 og, uint8_t *__restrict__ out_b,
                              float *__restrict__ out_scale)
{
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t total = (uint64_t)S * Hkv * T * d;
    if (idx >= total) {
        return;
    }
    const uint32_t j = (uint32_t)(idx % d);
    const uint32_t t = (uint32_t)((idx / d) % T);
    const uint32_t h = (uint32_t)((idx / ((uint64_t)d * T)) % Hkv);
    const uint32_t s = (uint32_t)(idx / ((uint64_t)d * T * Hkv));
    const uint64_t region = (uint64_t)(seq_begin + s) * Hkv + h;
    const uint32_t n = tok_begin + t;
    const uint32_t f = load_field(sp, which, region, n, j, d_stored);
    const float a = sp.alpha ? sp.alpha[region * padded + n] : 0.0f;
    if (out_mode == 1) {
        out_b[idx] = (uint8_t)f;
        if (out_scale && j == 0) {
            out_scale[(uint64_t)(s * Hkv + h) * T + t] = a;
        }
        return;
    }
    float val;
    if (kv_mode == WEED_HIP_KV_UNIFORM) {
        // sp.beta = lo, sp.alpha_const = step
        val = sp.beta + ((float)f + 0.5f) * sp.alpha_const;
    } else {
        val = a * sp.table[f];
    }
    const uint64_t o = (uint64_t)og.off + (uint64_t)s * og.s[0] + (uint64_t)h * og.s[1] + (uint64_t)t * og.s[2] +
                       (uint64_t)j * og.s[3];
    out_f[o] = val;
}

// Rows in Weed's word packing: floor(32/bits) codes per int32 (multihead_attention.cpp:43-62).
__global__ void weed_words_kernel(SideParams sp, int which, uint32_t Hkv, uint32_t d, uint32_t d_stored,
                                  int32_t seq_begin, uint32_t S, uint32_t tok_begin, uint32_t T, uint32_t bits,
                                  int32_t *__restrict__ words)
{
    const uint32_t vpw = 32 / bits;
    const uint32_t wpr = (d + vpw - 1) / vpw;
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t total = (uint64_t)S * Hkv * T * wpr;
    if (idx >= total) {
        return;
    }
    const uint32_t wi = (uint32_t)(idx % wpr);
    const uint32_t t = (uint32_t)((idx / wpr) % T);
    const uint32_t h = (uint32_t)((idx / ((uint64_t)wpr * T)) % Hkv);
    const uint32_t s = (uint32_t)(idx / ((uint64_t)wpr * T * Hkv));
    const uint64_t region = (uint64_t)(seq_begin + s) * Hkv + h;
    uint32_t word = 0;
    for (uint32_t k = 0; k < vpw; ++k) {
        const uint32_t j = wi * vpw + k;
        if (j < d) {
            word |= load_field(sp, which, region, tok_begin + t, j, d_stored) << (k * bits);
        }
    }
    words[idx] = (int32_t)word;
}

// The reverse: rows in Weed's word packing become one code per byte, rows in (sequence, head, token) order.
__global__ void fields_from_words_kernel(const int32_t *__restrict__ words, uint64_t rows, uint32_t d,
                                         uint32_t d_stored, uint32_t bits, uint8_t *__restrict__ fields)
{
    // rows of d codes in words; rows of d_stored >= d bytes out (zero codes in the coordinates beyond d)
    const uint32_t vpw = 32 / bits;
    const uint32_t wpr = (d + vpw - 1) / vpw;
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * d_stored) {
        return;
    }
    const uint64_t row = idx / d_stored;
    const uint32_t j = (uint32_t)(idx - row * d_stored);
    uint32_t code = 0;
    if (j < d) {
        const uint32_t word = (uint32_t)words[row * wpr + j / vpw];
        code = (word >> ((j % vpw) * bits)) & ((1u << bits) - 1u);
    }
    fields[idx] = (uint8_t)code;
}

// sum of squares: tree reduction (one partial per block, finished on the host in double)
__global__ void sumsq_kernel(const float *__restrict__ x, Geom4 g, uint32_t n1, uint32_t n2, uint32_t n3, uint64_t total,
                             double *__restrict__ partials)
{
    __shared__ double red[256];
    double acc = 0.0;
    for (uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t i3 = (uint32_t)(idx % n3);
        const uint32_t i2 = (uint32_t)((idx / n3) % n2);
        const uint32_t i1 = (uint32_t)((idx / ((uint64_t)n3 * n2)) % n1);
        const uint32_t i0 = (uint32_t)(idx / ((uint64_t)n3 * n2 * n1));
        const float v = x[(uint64_t)g.off + (uint64_t)i0 * g.s[0] + (uint64_t)i1 * g.s[1] + (uint64_t)i2 * g.s[2] +
                          (uint64_t)i3 * g.s[3]];
        acc += (double)v * (double)v;
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (uint32_t s = blockDim.x / 2; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            red[threadIdx.x] += red[threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partials[blockIdx.x] = red[0];
    }
}

// The reference's order: one fp32 accumulator over the flat column-major index of the [B, heads, T, d] tensor
// (multihead_attention.cpp:229-240 walks the contiguous reshape of it): the first dimension runs fastest, the last
// slowest, whatever the strides of the view handed in are.
__global__ void sumsq_sequential_kernel(const float *__restrict__ x, Geom4 g, uint32_t n0, uint32_t n1, uint32_t n2,
                                        uint32_t n3, float *__restrict__ out)
{
    if (blockIdx.x || threadIdx.x) {
        return;
    }
    float sum = 0.0f;
    for (uint32_t i3 = 0; i3 < n3; ++i3) {
        for (uint32_t i2 = 0; i2 < n2; ++i2) {
            for (uint32_t i1 = 0; i1 < n1; ++i1) {
                const uint64_t base =
                    (uint64_t)g.off + (uint64_t)i1 * g.s[1] + (uint64_t)i2 * g.s[2] + (uint64_t)i3 * g.s[3];
                for (uint32_t i0 = 0; i0 < n0; ++i0) {
                    const float v = x[base + (uint64_t)i0 * g.s[0]];
                    sum = sum + v * v;
                }
            }
        }
    }
    out[0] = sum;
}

int check_cache(const weed_hip_kv_cache *c, const char *fn)
{
    if (!c) {
        return fail(WEED_HIP_EINVAL, "%s: null cache", fn);
    }
    return WEED_HIP_OK;
}

int check_range(const weed_hip_kv_cache *c, const char *fn, int32_t seq_begin, int32_t seq_count)
{
    if (seq_begin < 0 || seq_count < 0 || seq_begin + seq_count > c->cfg.n_seq) {
        return fail(WEED_HIP_EINVAL, "%s: sequences [%d, %d) outside [0, %d)", fn, seq_begin, seq_begin + seq_count,
                    c->cfg.n_seq);
    }
    return WEED_HIP_OK;
}

void free_side(Side &s)
{
    (void)hipFree(s.fields);
    (void)hipFree(s.alpha);
    (void)hipFree(s.alpha_max);
    (void)hipFree(s.rot);
    (void)hipFree(s.rot_t);
    s.fields = nullptr;
    s.alpha = nullptr;
    s.alpha_max = nullptr;
    s.rot = nullptr;
    s.rot_t = nullptr;
}

EncSide enc_side_args(const weed_hip_kv_cache *c, const Side &side, const float *x, uint32_t off,
                      const uint32_t stride[4], uint8_t *fields, float *alpha)
{
    EncSide e;
    e.x = x;
    e.g.off = off;
    for (int i = 0; i < 4; ++i) {
        e.g.s[i] = stride[i];
    }
    e.rot_t = side.rot_t;
    e.cp.mode = c->cfg.mode;
    e.cp.bits = side.bits;
    e.cp.sign = side.sign;
    e.cp.block_scale = side.block_scale;
    std::memcpy(e.cp.bounds, side.bounds, sizeof(e.cp.bounds));
    std::memcpy(e.cp.levels, side.levels, sizeof(e.cp.levels));
    e.fields = fields;
    e.alpha_out = alpha;
    e.direct = DirectOut{ nullptr, 0, nullptr, nullptr, nullptr, 0, 0, 0, 0 };
    return e;
}

// Rotate, quantise and pack the new K and V rows, and move the lengths on.  One launch where the encoder can write
// the items itself (whole half blocks, or one token per sequence), else one for the two encoders and one for the
// three packing steps; a grid of more than kBumpWorkgroups is followed by one that moves the lengths.  The scratch
// holds the K rows first, then the V rows.
int pack_rows(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new);

LensBump lens_bump(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new, uint32_t workgroups)
{
    return LensBump{ workgroups <= kBumpWorkgroups ? c->append_done : nullptr, c->lens_dev, seq_begin, seq_count, T_new,
                     workgroups };
}

// After the last kernel of an append that was too large to move the lengths itself.
int bump_lens(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new)
{
    bump_lens_kernel<<<((uint32_t)seq_count + 255) / 256, 256, 0, stream()>>>(c->lens_dev, seq_begin, seq_count, T_new);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int encode_both(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new, const float *k_dev,
                uint32_t k_off, const uint32_t k_stride[4], const float *v_dev, uint32_t v_off,
                const uint32_t v_stride[4], int rotate)
{
    const uint32_t d = c->dp, d_real = (uint32_t)c->cfg.head_dim;
    const uint32_t Hkv = (uint32_t)c->cfg.n_kv_heads;
    const uint32_t rows = (uint32_t)seq_count * Hkv * (uint32_t)T_new;
    uint8_t *k_fields = c->enc_fields, *v_fields = c->enc_fields + (size_t)rows * d;
    float *k_alpha = c->enc_alpha, *v_alpha = c->enc_alpha + rows;
    EncSide ek = enc_side_args(c, c->k, k_dev, k_off, k_stride, k_fields, k_alpha);
    EncSide ev = enc_side_args(c, c->v, v_dev, v_off, v_stride, v_fields, v_alpha);
    // An append that adds whole 32-token half blocks behind whole half blocks (a prefill, in chunks or not) needs no
    // packing pass: every workgroup of the encoder holds one half block of one (sequence, head) and writes its items
    // itself.
    bool direct = T_new % 32 == 0;
    for (int32_t sq = 0; direct && sq < seq_count; ++sq) {
        direct = c->lens[(size_t)(seq_begin + sq)] % 32 == 0;
    }
    // A decode step's append (one token per sequence) is finished by the encoder too: a workgroup's 32 rows are the
    // new tokens of 32 (sequence, head) pairs, and nothing else touches the items they go to.
    const int scattered = !direct && T_new == 1;
    direct = direct || scattered;
    if (direct) {
        const bool scales = c->cfg.mode == WEED_HIP_KV_LLOYDMAX;
        ek.direct = DirectOut{ c->k.fields, c->k.region_bytes, scales ? c->k.alpha : nullptr, nullptr, c->lens_dev,
                               seq_begin, c->padded_tokens, c->k.w, 0 };
        ev.direct = DirectOut{ c->v.fields, c->v.region_bytes, scales ? c->v.alpha : nullptr,
                               scales ? c->v.alpha_max : nullptr, c->lens_dev, seq_begin, c->padded_tokens, c->v.w, 1 };
    }
    const size_t smem = sizeof(float) * (2 * kEncRows * (d + 1) + kEncRows) + sizeof(unsigned long long) * kEncRows +
                        sizeof(uint32_t) * kEncRows;
    const uint32_t blocks = (rows + kEncRows - 1) / kEncRows;
    int parts = 1;
    while (parts * 2 * d <= (uint32_t)kEncThreads && parts < 8) {
        parts *= 2;
    }
    typedef void (*EncKernel)(EncSide, EncSide, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int, LensBump);
    static const EncKernel kernels[2][4] = {
        { encode_rows_pair_kernel<1, false>, encode_rows_pair_kernel<2, false>, encode_rows_pair_kernel<4, false>,
          encode_rows_pair_kernel<8, false> },
        { encode_rows_pair_kernel<1, true>, encode_rows_pair_kernel<2, true>, encode_rows_pair_kernel<4, true>,
          encode_rows_pair_kernel<8, true> },
    };
    const EncKernel kernel = kernels[scattered][parts == 8 ? 3 : parts == 4 ? 2 : parts == 2 ? 1 : 0];
    if (smem > 48 * 1024) {
        // more than the default dynamic LDS limit (head_dim 256): opt in per kernel instance
        WEED_HIP_CHECK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    }
    {
        ProfileScope prof("kv_encode");
        LensBump bump = lens_bump(c, seq_begin, seq_count, T_new, 2 * blocks);
        if (!direct) {
            bump.done = nullptr; // the packing kernel reads the old lengths too
        }
        kernel<<<2 * blocks, kEncThreads, smem, stream()>>>(ek, ev, blocks, Hkv, (uint32_t)T_new, d, d_real, rows, rotate,
                                                           bump);
        WEED_HIP_LAUNCH_CHECK();
        if (direct && !bump.done) {
            WEED_HIP_TRY(bump_lens(c, seq_begin, seq_count, T_new));
        }
    }
    return direct ? WEED_HIP_OK : pack_rows(c, seq_begin, seq_count, T_new);
}

// Second stage of an append: the one-field-per-byte rows in the scratch buffers (K rows, then V rows, each in
// (sequence, head, token) order) go into the block layout behind the tokens already cached.
int pack_rows(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new)
{
    const uint32_t d = c->dp;
    const uint32_t Hkv = (uint32_t)c->cfg.n_kv_heads;
    const uint32_t rows = (uint32_t)seq_count * Hkv * (uint32_t)T_new;
    uint8_t *k_fields = c->enc_fields, *v_fields = c->enc_fields + (size_t)rows * d;
    float *k_alpha = c->enc_alpha, *v_alpha = c->enc_alpha + rows;
    ProfileScope prof("kv_pack");
    const bool scales = c->cfg.mode == WEED_HIP_KV_LLOYDMAX;
    PackArgs a;
    a.k_fields = k_fields;
    a.v_fields = v_fields;
    a.k_alpha_in = k_alpha;
    a.v_alpha_in = v_alpha;
    a.rows = rows;
    a.S = (uint32_t)seq_count;
    a.Hkv = Hkv;
    a.T = (uint32_t)T_new;
    a.d = d;
    a.wk = c->k.w;
    a.wv = c->v.w;
    // a run of T_new tokens starting anywhere touches at most (T_new + 30) / 32 + 1 half blocks
    a.halves = ((uint32_t)T_new + 30) / 32 + 1;
    a.padded = c->padded_tokens;
    a.seq_begin = seq_begin;
    a.lens = c->lens_dev;
    a.k_out = c->k.fields;
    a.v_out = c->v.fields;
    a.k_region_bytes = c->k.region_bytes;
    a.v_region_bytes = c->v.region_bytes;
    a.k_alpha_out = scales ? c->k.alpha : nullptr;
    a.v_alpha_out = scales ? c->v.alpha : nullptr;
    a.v_alpha_max = c->v.alpha_max;
    const uint64_t nk = (uint64_t)rows * (d / 8);
    const uint64_t nv = (uint64_t)seq_count * Hkv * a.halves * 4 * d;
    a.blocks_k = (uint32_t)((nk + 255) / 256);
    a.blocks_v = (uint32_t)((nv + 255) / 256);
    const uint32_t blocks_s = scales ? (rows + 255) / 256 : 0;
    a.bump = lens_bump(c, seq_begin, seq_count, T_new, a.blocks_k + a.blocks_v + blocks_s);
    pack_all_kernel<<<a.blocks_k + a.blocks_v + blocks_s, 256, 0, stream()>>>(a);
    WEED_HIP_LAUNCH_CHECK();
    return a.bump.done ? WEED_HIP_OK : bump_lens(c, seq_begin, seq_count, T_new);
}

// Scratch for the rows of one append (K rows, then V rows): grows as needed.
int reserve_append_scratch(weed_hip_kv_cache *c, const char *fn, int32_t seq_count, int32_t T_new)
{
    const uint64_t rows64 = (uint64_t)seq_count * c->cfg.n_kv_heads * T_new;
    WEED_HIP_REQUIRE(rows64 * c->dp < (1ull << 32), "%s: more than 2^32 elements in one call", fn);
    const size_t rows = (size_t)rows64;
    if (rows > c->enc_rows_cap) {
        WEED_HIP_CHECK(hipStreamSynchronize(stream()));
        (void)hipFree(c->enc_fields);
        (void)hipFree(c->enc_alpha);
        c->enc_fields = nullptr;
        c->enc_alpha = nullptr;
        c->enc_rows_cap = 0;
        if (hipMalloc((void **)&c->enc_fields, 2 * rows * c->dp) != hipSuccess ||
            hipMalloc((void **)&c->enc_alpha, 2 * rows * sizeof(float)) != hipSuccess) {
            return fail(WEED_HIP_ENOMEM, "%s: scratch allocation failed", fn);
        }
        c->enc_rows_cap = rows;
    }
    return WEED_HIP_OK;
}

// The host copy of the lengths follows the device's, which the last kernel of the append has moved.
int finish_append(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new)
{
    for (int32_t s = 0; s < seq_count; ++s) {
        c->lens[(size_t)(seq_begin + s)] += T_new;
    }
    return WEED_HIP_OK;
}

int launch_unpack(const weed_hip_kv_cache *c, int which, int32_t seq_begin, int32_t seq_count, int32_t tok_begin,
                  int32_t T, int out_mode, float *out_f, uint32_t o_off, const uint32_t *o_stride, uint8_t *out_b,
                  float *out_scale, const char *fn)
{
    WEED_HIP_TRY(check_cache(c, fn));
    WEED_HIP_TRY(check_range(c, fn, seq_begin, seq_count));
    WEED_HIP_REQUIRE(which == 0 || which == 1, "%s: which must be 0 (keys) or 1 (values)", fn);
    WEED_HIP_REQUIRE(tok_begin >= 0 && T >= 0 && (uint32_t)(tok_begin + T) <= c->padded_tokens,
                     "%s: tokens [%d, %d) outside the cache (capacity %d)", fn, tok_begin, tok_begin + T,
                     c->cfg.max_tokens);
    const uint64_t total = (uint64_t)seq_count * c->cfg.n_kv_heads * T * c->cfg.head_dim;
    if (!total) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(total < (1ull << 40), "%s: request too large", fn);
    Geom4 og = { 0, { 0, 0, 0, 0 } };
    if (out_mode == 0) {
        WEED_HIP_REQUIRE(out_f && o_stride, "%s: null output", fn);
        og.off = o_off;
        for (int i = 0; i < 4; ++i) {
            og.s[i] = o_stride[i];
        }
    } else {
        WEED_HIP_REQUIRE(out_b, "%s: null output", fn);
    }
    const SideParams sp = side_params(c, which);
    unpack_kernel<<<(uint32_t)((total + 255) / 256), 256, 0, stream()>>>(
        sp, which, c->cfg.mode, (uint32_t)c->cfg.n_kv_heads, (uint32_t)c->cfg.head_dim, c->dp, c->padded_tokens,
        seq_begin, (uint32_t)seq_count, (uint32_t)tok_begin, (uint32_t)T, out_mode, out_f, og, out_b, out_scale);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // namespace

namespace weedhip {

SideParams side_params(const weed_hip_kv_cache *c, int which)
{
    const Side &s = which ? c->v : c->k;
    SideParams sp;
    sp.fields = s.fields;
    sp.alpha = (c->cfg.mode == WEED_HIP_KV_LLOYDMAX) ? s.alpha : nullptr;
    sp.alpha_max = (c->cfg.mode == WEED_HIP_KV_LLOYDMAX) ? s.alpha_max : nullptr;
    sp.region_bytes = s.region_bytes;
    sp.w = s.w;
    if (c->cfg.mode == WEED_HIP_KV_UNIFORM) {
        // read_row (multihead_attention.cpp:71-78): lo = -3s, hi = 3s, step = (hi - lo) / levels
        const float lo = -3.0f * s.block_scale;
        const float hi = 3.0f * s.block_scale;
        sp.alpha_const = (hi - lo) / (float)(1 << s.bits);
        sp.beta = lo;
        for (int i = 0; i < 32; ++i) {
            sp.table[i] = (float)i + 0.5f;
        }
    } else {
        sp.alpha_const = 0.0f;
        sp.beta = 0.0f;
        std::memcpy(sp.table, s.recon, sizeof(sp.table));
    }
    return sp;
}

int upload_table_image(weed_hip_kv_cache *c)
{
    const SideParams k = side_params(c, 0), v = side_params(c, 1);
    uint16_t kl[32], vl[32];
    for (int i = 0; i < 32; ++i) {
        // the levels are exactly representable in binary16 (set_tables rounds them; the uniform coder's are code + 0.5)
        kl[i] = __builtin_bit_cast(uint16_t, (_Float16)k.table[i]);
        vl[i] = __builtin_bit_cast(uint16_t, (_Float16)v.table[i]);
    }
    const uint32_t words = mfma_table_rows(k.w, v.w) * (kMfmaTableRowBytes / 4);
    if (!words) {
        return WEED_HIP_OK;
    }
    // what the kernel reads: one word per 32 equal words of the LDS image (an entry's replicas over the banks)
    std::vector<uint32_t> img(words / 32);
    for (uint32_t i = 0; i < words / 32; ++i) {
        img[i] = mfma_table_word(32 * i, k.w, v.w, kl, vl);
    }
    // kernels already enqueued may still read the old image
    WEED_HIP_CHECK(hipStreamSynchronize(stream()));
    WEED_HIP_CHECK(hipMemcpy(c->table_image, img.data(), sizeof(uint32_t) * img.size(), hipMemcpyHostToDevice));
    return WEED_HIP_OK;
}

} // namespace weedhip

extern "C" {

int weed_hip_kv_cache_create(weed_hip_kv_cache **cache, const weed_hip_kv_config *cfg)
{
    WEED_HIP_REQUIRE(cache && cfg, "weed_hip_kv_cache_create: null pointer");
    *cache = nullptr;
    WEED_HIP_TRY(ensure_init());
    WEED_HIP_REQUIRE(cfg->mode == WEED_HIP_KV_UNIFORM || cfg->mode == WEED_HIP_KV_LLOYDMAX,
                     "weed_hip_kv_cache_create: unknown mode %d", cfg->mode);
    WEED_HIP_REQUIRE(cfg->n_seq > 0 && cfg->n_kv_heads > 0 && cfg->max_tokens > 0,
                     "weed_hip_kv_cache_create: n_seq, n_kv_heads and max_tokens must be positive");
    WEED_HIP_REQUIRE(cfg->head_dim >= 1 && cfg->head_dim <= 256,
                     "weed_hip_kv_cache_create: head_dim %d outside [1, 256]", cfg->head_dim);
    // Weed's uniform coder takes any width that divides into its 32-bit words sensibly; the Lloyd-Max tables exist
    // for 1..4 bits
    const int max_bits = cfg->mode == WEED_HIP_KV_UNIFORM ? 8 : 4;
    WEED_HIP_REQUIRE(cfg->k_bits >= 1 && cfg->k_bits <= max_bits && cfg->v_bits >= 1 && cfg->v_bits <= max_bits,
                     "weed_hip_kv_cache_create: code widths must be 1..%d bits in this mode (got K %d, V %d)", max_bits,
                     cfg->k_bits, cfg->v_bits);
    WEED_HIP_REQUIRE((cfg->k_sign == 0 || cfg->k_sign == 1) && (cfg->v_sign == 0 || cfg->v_sign == 1),
                     "weed_hip_kv_cache_create: sign flags must be 0 or 1");
    WEED_HIP_REQUIRE(cfg->mode == WEED_HIP_KV_LLOYDMAX || (!cfg->k_sign && !cfg->v_sign),
                     "weed_hip_kv_cache_create: the uniform coder keeps no residual sign bit");
    weed_hip_kv_cache *c = new (std::nothrow) weed_hip_kv_cache();
    if (!c) {
        return fail(WEED_HIP_ENOMEM, "weed_hip_kv_cache_create: host allocation failed");
    }
    c->cfg = *cfg;
    c->dp = ((uint32_t)cfg->head_dim + 31u) / 32u * 32u;
    c->padded_tokens = padded_tokens((uint32_t)cfg->max_tokens);
    c->lens.assign((size_t)cfg->n_seq, 0);
    const uint64_t regions = (uint64_t)cfg->n_seq * cfg->n_kv_heads;
    Side *sides[2] = { &c->k, &c->v };
    for (int which = 0; which < 2; ++which) {
        Side &s = *sides[which];
        s.bits = which ? cfg->v_bits : cfg->k_bits;
        s.sign = which ? cfg->v_sign : cfg->k_sign;
        s.w = (uint32_t)(s.bits + s.sign);
        s.region_bytes = region_bytes((uint32_t)cfg->max_tokens, c->dp, s.w);
        load_builtin(s);
        const size_t fbytes = (size_t)(regions * s.region_bytes);
        hipError_t e = hipMalloc((void **)&s.fields, fbytes);
        if (e == hipSuccess) {
            e = hipMemsetAsync(s.fields, 0, fbytes, stream());
        }
        if (e == hipSuccess && cfg->mode == WEED_HIP_KV_LLOYDMAX) {
            const size_t abytes = (size_t)(regions * c->padded_tokens * sizeof(float));
            e = hipMalloc((void **)&s.alpha, abytes);
            if (e == hipSuccess) {
                e = hipMemsetAsync(s.alpha, 0, abytes, stream());
            }
            if (e == hipSuccess) {
                e = hipMalloc((void **)&s.alpha_max, regions * kScaleMaxSlots * sizeof(uint32_t));
            }
            if (e == hipSuccess) {
                e = hipMemsetAsync(s.alpha_max, 0, regions * kScaleMaxSlots * sizeof(uint32_t), stream());
            }
        }
        if (e != hipSuccess) {
            weed_hip_kv_cache_destroy(c);
            return fail(WEED_HIP_ENOMEM, "weed_hip_kv_cache_create: device allocation failed: %s",
                        hipGetErrorString(e));
        }
    }
    // the lengths, and behind them the count of workgroups that are through with the append under way
    hipError_t e = hipMalloc((void **)&c->lens_dev, sizeof(int32_t) * ((size_t)cfg->n_seq + 1));
    if (e == hipSuccess) {
        e = hipMemsetAsync(c->lens_dev, 0, sizeof(int32_t) * ((size_t)cfg->n_seq + 1), stream());
        c->append_done = reinterpret_cast<uint32_t *>(c->lens_dev + cfg->n_seq);
    }
    if (e != hipSuccess) {
        weed_hip_kv_cache_destroy(c);
        return fail(WEED_HIP_ENOMEM, "weed_hip_kv_cache_create: device allocation failed: %s", hipGetErrorString(e));
    }
    if (hipMalloc((void **)&c->table_image, kMfmaTableImageBytes) != hipSuccess) {
        weed_hip_kv_cache_destroy(c);
        return fail(WEED_HIP_ENOMEM, "weed_hip_kv_cache_create: device allocation failed");
    }
    const int st = upload_table_image(c);
    if (st != WEED_HIP_OK) {
        weed_hip_kv_cache_destroy(c);
        return st;
    }
    *cache = c;
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_destroy(weed_hip_kv_cache *c)
{
    if (!c) {
        return WEED_HIP_OK;
    }
    (void)hipStreamSynchronize(stream());
    free_side(c->k);
    free_side(c->v);
    (void)hipFree(c->lens_dev);
    (void)hipFree(c->enc_fields);
    (void)hipFree(c->enc_alpha);
    (void)hipFree(c->dec_ws);
    (void)hipFree(c->table_image);
    delete c;
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_reset(weed_hip_kv_cache *c, int drop_rotations)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_reset"));
    std::fill(c->lens.begin(), c->lens.end(), 0);
    const uint32_t n = (uint32_t)c->cfg.n_seq;
    fill_i32_kernel<<<(n + 256) / 256, 256, 0, stream()>>>(c->lens_dev, 0, n + 1); // and the append's counter
    WEED_HIP_LAUNCH_CHECK();
    if (c->v.alpha_max) {
        const uint32_t words = n * (uint32_t)c->cfg.n_kv_heads * kScaleMaxSlots;
        fill_i32_kernel<<<(words + 255) / 256, 256, 0, stream()>>>((int32_t *)c->k.alpha_max, 0, words);
        fill_i32_kernel<<<(words + 255) / 256, 256, 0, stream()>>>((int32_t *)c->v.alpha_max, 0, words);
        WEED_HIP_LAUNCH_CHECK();
    }
    if (c->dec_ws) {
        // the arrival counters at the start of the decode workspace (zero between launches; cleared here too, so that
        // a reset also recovers from a launch that the device aborted midway)
        const uint32_t counters = std::min<size_t>(kMfmaMergeCounters, c->dec_ws_bytes / sizeof(int32_t));
        fill_i32_kernel<<<(counters + 255) / 256, 256, 0, stream()>>>((int32_t *)c->dec_ws, 0, counters);
        WEED_HIP_LAUNCH_CHECK();
    }
    // ... and those at the start of the device's static scratch (weed_hip_kv_decode_attn_noalloc), which no cache owns
    WEED_HIP_TRY(decode_scratch_clear_counters());
    if (drop_rotations) {
        c->has_rotations = false;
    }
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_row_bytes(const weed_hip_kv_cache *c, uint32_t *k_row_bytes, uint32_t *v_row_bytes)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_row_bytes"));
    const uint32_t extra = (c->cfg.mode == WEED_HIP_KV_LLOYDMAX) ? 4u : 0u;
    if (k_row_bytes) {
        *k_row_bytes = c->dp * c->k.w / 8 + extra;
    }
    if (v_row_bytes) {
        *v_row_bytes = c->dp * c->v.w / 8 + extra;
    }
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_seq_lens(const weed_hip_kv_cache *c, int32_t *lens)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_seq_lens"));
    WEED_HIP_REQUIRE(lens, "weed_hip_kv_cache_seq_lens: null pointer");
    std::memcpy(lens, c->lens.data(), sizeof(int32_t) * c->lens.size());
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_set_rotations(weed_hip_kv_cache *c, const float *rk_dev, const float *rv_dev)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_set_rotations"));
    WEED_HIP_REQUIRE(rk_dev && rv_dev, "weed_hip_kv_cache_set_rotations: null pointer");
    // kept as dp x dp: the caller's matrix in the leading block, an identity block for the coordinates beyond head_dim
    const uint32_t d = c->dp, d_real = (uint32_t)c->cfg.head_dim;
    const size_t bytes = sizeof(float) * d * d;
    Side *sides[2] = { &c->k, &c->v };
    const float *src[2] = { rk_dev, rv_dev };
    for (int which = 0; which < 2; ++which) {
        Side &s = *sides[which];
        if (!s.rot) {
            if (hipMalloc((void **)&s.rot, bytes) != hipSuccess || hipMalloc((void **)&s.rot_t, bytes) != hipSuccess) {
                return fail(WEED_HIP_ENOMEM, "weed_hip_kv_cache_set_rotations: device allocation failed");
            }
        }
        embed_square_kernel<<<(d * d + 255) / 256, 256, 0, stream()>>>(src[which], d_real, s.rot, d);
        WEED_HIP_LAUNCH_CHECK();
        transpose_square_kernel<<<(d * d + 255) / 256, 256, 0, stream()>>>(s.rot, s.rot_t, d);
        WEED_HIP_LAUNCH_CHECK();
    }
    c->has_rotations = true;
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_set_scales(weed_hip_kv_cache *c, float k_scale, float v_scale)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_set_scales"));
    WEED_HIP_REQUIRE(c->cfg.mode == WEED_HIP_KV_UNIFORM, "weed_hip_kv_cache_set_scales: only the uniform coder has a block scale");
    c->k.block_scale = k_scale;
    c->v.block_scale = v_scale;
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_get_scales(const weed_hip_kv_cache *c, float *k_scale, float *v_scale)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_get_scales"));
    if (k_scale) {
        *k_scale = c->k.block_scale;
    }
    if (v_scale) {
        *v_scale = c->v.block_scale;
    }
    return WEED_HIP_OK;
}

int weed_hip_kv_cache_set_tables(weed_hip_kv_cache *c, int which, const float *bounds, const float *levels,
                                 const float *recon, float *recon_rounded)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_set_tables"));
    WEED_HIP_REQUIRE(which == 0 || which == 1, "weed_hip_kv_cache_set_tables: which must be 0 or 1");
    WEED_HIP_REQUIRE(c->cfg.mode == WEED_HIP_KV_LLOYDMAX, "weed_hip_kv_cache_set_tables: only the Lloyd-Max coder uses tables");
    WEED_HIP_REQUIRE(bounds && levels && recon, "weed_hip_kv_cache_set_tables: null pointer");
    Side &s = which ? c->v : c->k;
    const int n = 1 << s.bits;
    for (int i = 0; i + 1 < n - 1; ++i) {
        WEED_HIP_REQUIRE(bounds[i] <= bounds[i + 1], "weed_hip_kv_cache_set_tables: thresholds must ascend");
    }
    std::memcpy(s.bounds, bounds, sizeof(float) * (n - 1));
    std::memcpy(s.levels, levels, sizeof(float) * n);
    const int nr = n << s.sign;
    for (int i = 0; i < nr; ++i) {
        s.recon[i] = round_to_half(recon[i]);
        if (recon_rounded) {
            recon_rounded[i] = s.recon[i];
        }
    }
    return upload_table_image(c);
}

int weed_hip_kv_cache_get_tables(const weed_hip_kv_cache *c, int which, float *bounds, float *levels, float *recon)
{
    WEED_HIP_TRY(check_cache(c, "weed_hip_kv_cache_get_tables"));
    WEED_HIP_REQUIRE(which == 0 || which == 1, "weed_hip_kv_cache_get_tables: which must be 0 or 1");
    const Side &s = which ? c->v : c->k;
    WEED_HIP_REQUIRE(s.bits <= 4, "weed_hip_kv_cache_get_tables: there are no tables for %d-bit codes", s.bits);
    const int n = 1 << s.bits;
    if (bounds) {
        std::memcpy(bounds, s.bounds, sizeof(float) * (n - 1));
    }
    if (levels) {
        std::memcpy(levels, s.levels, sizeof(float) * n);
    }
    if (recon) {
        std::memcpy(recon, s.recon, sizeof(float) * (n << s.sign));
    }
    return WEED_HIP_OK;
}

int weed_hip_block_scale_f32(const float *x_dev, uint32_t off, const uint32_t shape[4], const uint32_t stride[4],
                             int sequential, float *scale_out)
{
    WEED_HIP_REQUIRE(x_dev && shape && stride && scale_out, "weed_hip_block_scale_f32: null pointer");
    WEED_HIP_TRY(ensure_init());
    const uint64_t total = (uint64_t)shape[0] * shape[1] * shape[2] * shape[3];
    WEED_HIP_REQUIRE(total > 0, "weed_hip_block_scale_f32: empty tensor");
    if (sequential) {
        float *sum_dev = nullptr;
        if (hipMalloc((void **)&sum_dev, sizeof(float)) != hipSuccess) {
            return fail(WEED_HIP_ENOMEM, "weed_hip_block_scale_f32: device allocation failed");
        }
        Geom4 gs;
        gs.off = off;
        for (int i = 0; i < 4; ++i) {
            gs.s[i] = stride[i];
        }
        sumsq_sequential_kernel<<<1, 64, 0, stream()>>>(x_dev, gs, shape[0], shape[1], shape[2], shape[3], sum_dev);
        float sum = 0.0f;
        hipError_t e = hipMemcpyAsync(&sum, sum_dev, sizeof(float), hipMemcpyDeviceToHost, stream());
        if (e == hipSuccess) {
            e = hipStreamSynchronize(stream());
        }
        (void)hipFree(sum_dev);
        WEED_HIP_CHECK(e);
        // multihead_attention.cpp:240: sqrt(sum / n + 1e-8) in fp32
        *scale_out = std::sqrt(sum / (float)(uint32_t)total + 1e-8f);
        return WEED_HIP_OK;
    }
    const uint32_t blocks = 1024;
    double *partials_dev = nullptr;
    if (hipMalloc((void **)&partials_dev, sizeof(double) * blocks) != hipSuccess) {
        return fail(WEED_HIP_ENOMEM, "weed_hip_block_scale_f32: device allocation failed");
    }
    Geom4 g;
    g.off = off;
    for (int i = 0; i < 4; ++i) {
        g.s[i] = stride[i];
    }
    sumsq_kernel<<<blocks, 256, 0, stream()>>>(x_dev, g, shape[1], shape[2], shape[3], total, partials_dev);
    std::vector<double> partials(blocks);
    hipError_t e = hipMemcpyAsync(partials.data(), partials_dev, sizeof(double) * blocks, hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess) {
        e = hipStreamSynchronize(stream());
    }
    (void)hipFree(partials_dev);
    WEED_HIP_CHECK(e);
    double sum = 0.0;
    for (double p : partials) {
        sum += p;
    }
    *scale_out = (float)std::sqrt(sum / (double)total + 1e-8);
    return WEED_HIP_OK;
}

int weed_hip_kv_encode_append(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new,
                              const float *k_dev, uint32_t k_off, const uint32_t k_stride[4], const float *v_dev,
                              uint32_t v_off, const uint32_t v_stride[4], int rotate)
{
    const char *fn = "weed_hip_kv_encode_append";
    WEED_HIP_TRY(check_cache(c, fn));
    WEED_HIP_TRY(check_range(c, fn, seq_begin, seq_count));
    WEED_HIP_REQUIRE(T_new >= 0, "%s: negative token count", fn);
    WEED_HIP_REQUIRE(rotate >= 0 && rotate <= 2, "%s: rotate must be 0, 1 or 2", fn);
    if (!seq_count || !T_new) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(k_dev && v_dev && k_stride && v_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(!rotate || c->has_rotations, "%s: rotation requested but no rotations are set", fn);
    for (int32_t s = 0; s < seq_count; ++s) {
        if (c->lens[(size_t)(seq_begin + s)] + T_new > c->cfg.max_tokens) {
            return fail(WEED_HIP_ECAPACITY, "%s: sequence %d would hold %d tokens, capacity is %d", fn, seq_begin + s,
                        c->lens[(size_t)(seq_begin + s)] + T_new, c->cfg.max_tokens);
        }
    }
    WEED_HIP_TRY(reserve_append_scratch(c, fn, seq_count, T_new));
    WEED_HIP_TRY(encode_both(c, seq_begin, seq_count, T_new, k_dev, k_off, k_stride, v_dev, v_off, v_stride, rotate));
    return finish_append(c, seq_begin, seq_count, T_new);
}

int weed_hip_kv_append_weed_words(weed_hip_kv_cache *c, int32_t seq_begin, int32_t seq_count, int32_t T_new,
                                  const int32_t *k_words_dev, const int32_t *v_words_dev)
{
    const char *fn = "weed_hip_kv_append_weed_words";
    WEED_HIP_TRY(check_cache(c, fn));
    WEED_HIP_TRY(check_range(c, fn, seq_begin, seq_count));
    WEED_HIP_REQUIRE(c->cfg.mode == WEED_HIP_KV_UNIFORM, "%s: Weed's word packing exists for the uniform coder only", fn);
    WEED_HIP_REQUIRE(T_new >= 0, "%s: negative token count", fn);
    if (!seq_count || !T_new) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(k_words_dev && v_words_dev, "%s: null pointer", fn);
    for (int32_t s = 0; s < seq_count; ++s) {
        if (c->lens[(size_t)(seq_begin + s)] + T_new > c->cfg.max_tokens) {
            return fail(WEED_HIP_ECAPACITY, "%s: sequence %d would hold %d tokens, capacity is %d", fn, seq_begin + s,
                        c->lens[(size_t)(seq_begin + s)] + T_new, c->cfg.max_tokens);
        }
    }
    WEED_HIP_TRY(reserve_append_scratch(c, fn, seq_count, T_new));
    const uint32_t d = (uint32_t)c->cfg.head_dim, dp = c->dp;
    const uint64_t rows = (uint64_t)seq_count * c->cfg.n_kv_heads * T_new;
    const uint32_t blocks = (uint32_t)((rows * dp + 255) / 256);
    fields_from_words_kernel<<<blocks, 256, 0, stream()>>>(k_words_dev, rows, d, dp, (uint32_t)c->k.bits, c->enc_fields);
    WEED_HIP_LAUNCH_CHECK();
    fields_from_words_kernel<<<blocks, 256, 0, stream()>>>(v_words_dev, rows, d, dp, (uint32_t)c->v.bits,
                                                           c->enc_fields + rows * dp);
    WEED_HIP_LAUNCH_CHECK();
    WEED_HIP_TRY(pack_rows(c, seq_begin, seq_count, T_new));
    return finish_append(c, seq_begin, seq_count, T_new);
}

int weed_hip_kv_dequant(const weed_hip_kv_cache *c, int which, int32_t seq_begin, int32_t seq_count, int32_t tok_begin,
                        int32_t T, float *out_dev, uint32_t o_off, const uint32_t o_stride[4])
{
    return launch_unpack(c, which, seq_begin, seq_count, tok_begin, T, 0, out_dev, o_off, o_stride, nullptr, nullptr,
                         "weed_hip_kv_dequant");
}

int weed_hip_kv_export_fields(const weed_hip_kv_cache *c, int which, int32_t seq_begin, int32_t seq_count,
                              int32_t tok_begin, int32_t T, uint8_t *fields_dev, float *scales_dev)
{
    return launch_unpack(c, which, seq_begin, seq_count, tok_begin, T, 1, nullptr, 0, nullptr, fields_dev, scales_dev,
                         "weed_hip_kv_export_fields");
}

int weed_hip_kv_export_weed_words(const weed_hip_kv_cache *c, int which, int32_t seq_begin, int32_t seq_count,
                                  int32_t tok_begin, int32_t T, int32_t *words_dev)
{
    const char *fn = "weed_hip_kv_export_weed_words";
    WEED_HIP_TRY(check_cache(c, fn));
    WEED_HIP_TRY(check_range(c, fn, seq_begin, seq_count));
    WEED_HIP_REQUIRE(which == 0 || which == 1, "%s: which must be 0 (keys) or 1 (values)", fn);
    WEED_HIP_REQUIRE(c->cfg.mode == WEED_HIP_KV_UNIFORM, "%s: Weed's word packing exists for the uniform coder only", fn);
    WEED_HIP_REQUIRE(tok_begin >= 0 && T >= 0 && (uint32_t)(tok_begin + T) <= c->padded_tokens,
                     "%s: tokens [%d, %d) outside the cache", fn, tok_begin, tok_begin + T);
    WEED_HIP_REQUIRE(words_dev, "%s: null output", fn);
    const Side &s = which ? c->v : c->k;
    const uint32_t vpw = 32 / (uint32_t)s.bits;
    const uint32_t wpr = ((uint32_t)c->cfg.head_dim + vpw - 1) / vpw;
    const uint64_t total = (uint64_t)seq_count * c->cfg.n_kv_heads * T * wpr;
    if (!total) {
        return WEED_HIP_OK;
    }
    const SideParams sp = side_params(c, which);
    weed_words_kernel<<<(uint32_t)((total + 255) / 256), 256, 0, stream()>>>(
        sp, which, (uint32_t)c->cfg.n_kv_heads, (uint32_t)c->cfg.head_dim, c->dp, seq_begin, (uint32_t)seq_count,
        (uint32_t)tok_begin, (uint32_t)T, (uint32_t)s.bits, words_dev);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // extern "C"
