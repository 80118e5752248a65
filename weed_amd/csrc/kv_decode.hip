// Fused single-query decode attention over the packed cache.
//
// One call does what MultiHeadAttention::forward does between the cache rebuild and the output projection when
// T = 1 (src/modules/multihead_attention.cpp:259-348): un-pack K and V, rotate q, Q.K^T, divide by sqrt(d), softmax
// over each sequence's own length, P.V, un-rotate -- without ever materialising the dense K, V, K^T, the replicated
// GQA copies or the score matrix the reference builds.
//
// Launches: (1) rotate the queries; (2) one workgroup per (context split, kv head, sequence) produces an
// un-normalised partial (running max m, running sum l, o[d]) per query head; (3) merge the partials of all splits,
// normalise and un-rotate.
#include "kv_cache.h"
#include "kv_decode_mfma.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>

using namespace weedhip;
using namespace weedkv;

namespace {

constexpr int kGMax = 8;        // query heads of one kv head handled per pass
constexpr int kThreads = 256;
constexpr int kChunk = 256;     // tokens per inner iteration of the generic kernel

struct Geom3 {
    uint32_t off;
    uint32_t s[3];
};

struct DecodeParams {
    SideParams k, v;
    const int32_t *lens;
    uint32_t padded;
    uint32_t d;
    uint32_t Hq, Hkv, G;
    int blocked; // 1: kv = h / G, 0: kv = h % Hkv (Weed)
    const float *q_rot; // [n_seq][Hq][d]
    float *partials;    // [n_seq][Hq][n_splits][d + 2]
    uint32_t n_splits, split_tokens;
};

__device__ __forceinline__ uint32_t q_head_of(const DecodeParams &p, uint32_t kvh, uint32_t g)
{
    return p.blocked ? (kvh * p.G + g) : (g * p.Hkv + kvh);
}

// q_rot[s][h][:] = q[s][h][:] . Rk  (multihead_attention.cpp:276), or a plain gather when rotate == 0.
// For the matrix-core kernel the rotated query is also scaled by log2(e)/sqrt(d), divided by a power of two that
// brings it into [-1, 1], and split into fp16 hi + lo halves.
__global__ void __launch_bounds__(256) prep_q_kernel(const float *__restrict__ q, Geom3 g, uint32_t Hq, uint32_t d,
                                                     const float *__restrict__ rot_t, int rotate,
                                                     float *__restrict__ q_rot, uint16_t *__restrict__ q_hi,
                                                     uint16_t *__restrict__ q_lo, float *__restrict__ q_scale,
                                                     float *__restrict__ q_sum)
{
    __shared__ float qs[256];
    __shared__ float red_max[256];
    __shared__ float red_sum[256];
    const uint32_t h = blockIdx.x, s = blockIdx.y;
    const uint32_t tid = threadIdx.x;
    if (tid < d) {
        qs[tid] = q[(uint64_t)g.off + (uint64_t)s * g.s[0] + (uint64_t)h * g.s[1] + (uint64_t)tid * g.s[2]];
    }
    __syncthreads();
    float acc = 0.0f;
    if (tid < d) {
        if (rotate) {
            for (uint32_t i = 0; i < d; ++i) {
                acc = fmaf(qs[i], rot_t[tid + d * i], acc);
            }
        } else {
            acc = qs[tid];
        }
        q_rot[((uint64_t)s * Hq + h) * d + tid] = acc;
    }
    const float qc = acc * (1.4426950408889634f / sqrtf((float)d));
    red_max[tid] = fabsf(qc);
    red_sum[tid] = qc;
    __syncthreads();
    for (uint32_t k = 128; k > 0; k >>= 1) {
        if (tid < k) {
            red_max[tid] = fmaxf(red_max[tid], red_max[tid + k]);
            red_sum[tid] += red_sum[tid + k];
        }
        __syncthreads();
    }
    int e = 0;
    (void)frexpf(red_max[0], &e); // max = f * 2^e with f in [0.5, 1), so 2^e exceeds every |qc|
    e = e < -100 ? -100 : (e > 100 ? 100 : e);
    const float inv = ldexpf(1.0f, -e);
    if (tid < d) {
        const float qn = qc * inv;
        const _Float16 hi = (_Float16)qn;
        const _Float16 lo = (_Float16)(qn - (float)hi);
        q_hi[((uint64_t)s * Hq + h) * d + tid] = __builtin_bit_cast(uint16_t, hi);
        q_lo[((uint64_t)s * Hq + h) * d + tid] = __builtin_bit_cast(uint16_t, lo);
    }
    if (tid == 0) {
        q_scale[(uint64_t)s * Hq + h] = ldexpf(1.0f, e);
        q_sum[(uint64_t)s * Hq + h] = red_sum[0];
    }
}

__device__ __forceinline__ float wave_max(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v = fmaxf(v, __shfl_xor(v, o));
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_xor(v, o);
    }
    return v;
}

// Generic kernel: any head_dim that is a multiple of 32, any field width, any group size.
__global__ void __launch_bounds__(kThreads) decode_generic_kernel(DecodeParams p)
{
    __shared__ float q_s[kGMax * 256];
    __shared__ float qsum_s[kGMax];
    __shared__ float sc[kGMax * kChunk];
    __shared__ float m_s[kGMax], l_s[kGMax], scale_s[kGMax];
    __shared__ float o_s[kGMax * 256];
    __shared__ float ktab[32], vtab[32];

    const uint32_t split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t d = p.d;
    const uint32_t L = (uint32_t)p.lens[seq];
    const uint32_t n0 = split * p.split_tokens;
    const uint32_t n1 = min(L, n0 + p.split_tokens);
    const uint64_t region = (uint64_t)seq * p.Hkv + kvh;
    const float sqrt_d = sqrtf((float)d);
    const uint32_t parts = kThreads / d ? kThreads / d : 1;
    const uint32_t part = tid / d, jj = tid % d;
    const bool pv_active = part < parts;

    if (tid < 32) {
        ktab[tid] = p.k.table[tid];
        vtab[tid] = p.v.table[tid];
    }

    for (uint32_t hc = 0; hc < p.G; hc += kGMax) {
        const uint32_t gh = min((uint32_t)kGMax, p.G - hc);
        __syncthreads();
        for (uint32_t e = tid; e < gh * d; e += kThreads) {
            const uint32_t h = e / d, j = e % d;
            q_s[h * 256 + j] = p.q_rot[((uint64_t)seq * p.Hq + q_head_of(p, kvh, hc + h)) * d + j];
        }
        if (tid < kGMax) {
            m_s[tid] = -INFINITY;
            l_s[tid] = 0.0f;
        }
        __syncthreads();
        if (tid < gh) {
            float s = 0.0f;
            for (uint32_t j = 0; j < d; ++j) {
                s += q_s[tid * 256 + j];
            }
            qsum_s[tid] = s;
        }
        float o[kGMax];
#pragma unroll
        for (int h = 0; h < kGMax; ++h) {
            o[h] = 0.0f;
        }
        __syncthreads();

        for (uint32_t c0 = n0; c0 < n1; c0 += kChunk) {
            // ---- scores for token c0 + tid ----
            const uint32_t n = c0 + tid;
            float acc[kGMax];
#pragma unroll
            for (int h = 0; h < kGMax; ++h) {
                acc[h] = 0.0f;
            }
            if (n < n1) {
                const uint8_t *kbase = p.k.fields + region * p.k.region_bytes;
                for (uint32_t j0 = 0; j0 < d; j0 += 8) {
                    const uint8_t *item = kbase + k_field_pos(n, j0, d, p.k.w).byte;
                    for (uint32_t e = 0; e < 8; ++e) {
                        const float kv = ktab[item_get(item, e * p.k.w, p.k.w)];
#pragma unroll
                        for (int h = 0; h < kGMax; ++h) {
                            acc[h] = fmaf(q_s[h * 256 + j0 + e], kv, acc[h]);
                        }
                    }
                }
                const float a = p.k.alpha ? p.k.alpha[region * p.padded + n] : p.k.alpha_const;
#pragma unroll
                for (int h = 0; h < kGMax; ++h) {
                    if ((uint32_t)h < gh) {
                        sc[h * kChunk + tid] = (a * acc[h] + p.k.beta * qsum_s[h]) / sqrt_d;
                    }
                }
            } else {
#pragma unroll
                for (int h = 0; h < kGMax; ++h) {
                    sc[h * kChunk + tid] = -INFINITY;
                }
            }
            __syncthreads();
            // ---- running softmax statistics, one wave per head ----
            for (uint32_t h = wave; h < gh; h += kThreads / 64) {
                float v[kChunk / 64];
                float mx = -INFINITY;
#pragma unroll
                for (int k = 0; k < kChunk / 64; ++k) {
                    v[k] = sc[h * kChunk + lane + 64 * k];
                    mx = fmaxf(mx, v[k]);
                }
                mx = wave_max(mx);
                const float m_old = m_s[h];
                const float m_new = fmaxf(m_old, mx);
                float sum = 0.0f;
#pragma unroll
                for (int k = 0; k < kChunk / 64; ++k) {
                    const float e = (v[k] == -INFINITY) ? 0.0f : expf(v[k] - m_new);
                    sc[h * kChunk + lane + 64 * k] = e;
                    sum += e;
                }
                sum = wave_sum(sum);
                if (lane == 0) {
                    const float scale = (m_old == -INFINITY) ? 0.0f : expf(m_old - m_new);
                    scale_s[h] = scale;
                    l_s[h] = l_s[h] * scale + sum;
                    m_s[h] = m_new;
                }
            }
            __syncthreads();
            // ---- o += p . V, thread = (token slice, coordinate) ----
            if (pv_active) {
#pragma unroll
                for (int h = 0; h < kGMax; ++h) {
                    if ((uint32_t)h < gh) {
                        o[h] *= scale_s[h];
                    }
                }
                const uint32_t cnt = min((uint32_t)kChunk, n1 - c0);
                const uint8_t *vbase = p.v.fields + region * p.v.region_bytes;
                for (uint32_t nl = part; nl < cnt; nl += parts) {
                    const uint32_t nn = c0 + nl;
                    const FieldPos vp = v_field_pos(nn, jj, d, p.v.w);
                    const float a = p.v.alpha ? p.v.alpha[region * p.padded + nn] : p.v.alpha_const;
                    const float vv = fmaf(a, vtab[item_get(vbase + vp.byte, vp.bit, p.v.w)], p.v.beta);
#pragma unroll
                    for (int h = 0; h < kGMax; ++h) {
                        if ((uint32_t)h < gh) {
                            o[h] = fmaf(sc[h * kChunk + nl], vv, o[h]);
                        }
                    }
                }
            }
            __syncthreads();
        }

        // ---- fold the token slices together and emit the partial ----
        for (uint32_t r = 0; r < parts; ++r) {
            if (pv_active && part == r) {
#pragma unroll
                for (int h = 0; h < kGMax; ++h) {
                    if ((uint32_t)h < gh) {
                        o_s[h * 256 + jj] = (r ? o_s[h * 256 + jj] : 0.0f) + o[h];
                    }
                }
            }
            __syncthreads();
        }
        for (uint32_t e = tid; e < gh * d; e += kThreads) {
            const uint32_t h = e / d, j = e % d;
            const uint32_t qh = q_head_of(p, kvh, hc + h);
            float *dst = p.partials + (((uint64_t)seq * p.Hq + qh) * p.n_splits + split) * (d + 2);
            dst[2 + j] = o_s[h * 256 + j];
            if (j == 0) {
                dst[0] = m_s[h];
                dst[1] = l_s[h];
            }
        }
    }
}

// Merge the partials of all splits: out = sum_s e^(m_s - M) o_s / sum_s e^(m_s - M) l_s, then multiply by
// v_rotation^T (multihead_attention.cpp:343-348): out_i = sum_j O_j Rv[i + d*j].
__global__ void combine_kernel(const float *__restrict__ partials, uint32_t Hq, uint32_t d, uint32_t n_splits,
                               const float *__restrict__ rv, int unrotate, int log2_domain, float *__restrict__ out,
                               Geom3 og)
{
    __shared__ float w_s[1024];
    __shared__ float o_sh[256];
    __shared__ float red[2];
    const uint32_t h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
    const float *base = partials + ((uint64_t)s * Hq + h) * n_splits * (d + 2);
    // n_splits <= 1024 is enforced by the host
    if (tid < 64) {
        float mx = -INFINITY;
        for (uint32_t k = tid; k < n_splits; k += 64) {
            mx = fmaxf(mx, base[(uint64_t)k * (d + 2)]);
        }
        mx = wave_max(mx);
        float sum = 0.0f;
        for (uint32_t k = tid; k < n_splits; k += 64) {
            const float m = base[(uint64_t)k * (d + 2)];
            const float w = (m == -INFINITY) ? 0.0f : (log2_domain ? exp2f(m - mx) : expf(m - mx));
            w_s[k] = w;
            sum = fmaf(w, base[(uint64_t)k * (d + 2) + 1], sum);
        }
        sum = wave_sum(sum);
        if (tid == 0) {
            red[0] = sum;
        }
    }
    __syncthreads();
    const float denom = red[0];
    if (tid < d) {
        float acc = 0.0f;
        for (uint32_t k = 0; k < n_splits; ++k) {
            const float w = w_s[k];
            if (w != 0.0f) {
                acc = fmaf(w, base[(uint64_t)k * (d + 2) + 2 + tid], acc);
            }
        }
        o_sh[tid] = (denom > 0.0f) ? acc / denom : 0.0f;
    }
    __syncthreads();
    if (tid >= d) {
        return;
    }
    float r;
    if (unrotate) {
        r = 0.0f;
        for (uint32_t j = 0; j < d; ++j) {
            r = fmaf(o_sh[j], rv[tid + d * j], r);
        }
    } else {
        r = o_sh[tid];
    }
    out[(uint64_t)og.off + (uint64_t)s * og.s[0] + (uint64_t)h * og.s[1] + (uint64_t)tid * og.s[2]] = r;
}

// `lens_dev` (optional): attend over these per-sequence lengths instead of the cached ones.
int decode_impl(const char *fn, weed_hip_kv_cache *c, int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev,
                uint32_t q_off, const uint32_t q_stride[3], float *out_dev, uint32_t o_off, const uint32_t o_stride[3],
                uint32_t flags, const int32_t *lens_dev)
{
    WEED_HIP_REQUIRE(c, "%s: null cache", fn);
    WEED_HIP_REQUIRE(q_dev && out_dev && q_stride && o_stride, "%s: null pointer", fn);
    const uint32_t Hkv = (uint32_t)c->cfg.n_kv_heads, d = (uint32_t)c->cfg.head_dim, S = (uint32_t)c->cfg.n_seq;
    WEED_HIP_REQUIRE(n_q_heads > 0 && (uint32_t)n_q_heads % Hkv == 0,
                     "%s: n_q_heads %d must be a positive multiple of n_kv_heads %u", fn, n_q_heads, Hkv);
    WEED_HIP_REQUIRE(gqa_mapping == WEED_HIP_GQA_WEED || gqa_mapping == WEED_HIP_GQA_BLOCKED,
                     "%s: unknown GQA mapping %d", fn, gqa_mapping);
    const bool rot_q = flags & WEED_HIP_ATTN_ROTATE_Q, unrot = flags & WEED_HIP_ATTN_UNROTATE_OUT;
    WEED_HIP_REQUIRE(!(rot_q || unrot) || c->has_rotations, "%s: rotation requested but no rotations are set", fn);
    const uint32_t Hq = (uint32_t)n_q_heads;

    uint32_t max_len = 0;
    for (int32_t l : c->lens) {
        max_len = std::max(max_len, (uint32_t)l);
    }
    const uint32_t G = Hq / Hkv;
    const bool use_mfma = mfma_decode_supported(d, c->k.w, c->v.w, G);
    uint32_t n_splits, split_tokens = 0, blocks_per_split = 0;
    if (use_mfma) {
        // a workgroup's four wavefronts interleave over its 64-token blocks; aim for ~6 workgroups per compute unit
        const uint32_t nblk = std::max(1u, (max_len + 63) / 64);
        uint32_t target_wgs = 1024u;
        if (const char *env = std::getenv("WEED_HIP_DECODE_WGS")) {
            target_wgs = (uint32_t)std::max(1, std::atoi(env)); // tuning knob
        }
        const uint32_t want = std::max(1u, (target_wgs + S * Hkv - 1) / (S * Hkv));
        blocks_per_split = std::max(4u, (nblk + want - 1) / want);
        blocks_per_split = (blocks_per_split + 3) / 4 * 4;
        n_splits = (nblk + blocks_per_split - 1) / blocks_per_split;
    } else {
        // split the context so that the launch has a few workgroups per compute unit
        const uint32_t target_wgs = 2048;
        uint32_t want = std::max(1u, target_wgs / (S * Hkv));
        n_splits = std::max(1u, std::min((max_len + kChunk - 1) / kChunk, want));
        split_tokens = (max_len + n_splits - 1) / n_splits;
        split_tokens = std::max((uint32_t)kChunk, (split_tokens + kChunk - 1) / kChunk * kChunk);
        n_splits = std::max(1u, (max_len + split_tokens - 1) / split_tokens);
    }
    WEED_HIP_REQUIRE(n_splits <= 1024, "%s: internal split count %u too large", fn, n_splits);

    // workspace: rotated q (fp32), its fp16 hi / lo halves, per-head scale and sum, split partials
    const size_t n_q = (size_t)S * Hq * d;
    const size_t q_bytes = sizeof(float) * n_q;
    const size_t h_bytes = (sizeof(uint16_t) * n_q + 15) / 16 * 16;
    const size_t s_bytes = (sizeof(float) * (size_t)S * Hq + 15) / 16 * 16;
    const size_t part_bytes = sizeof(float) * (size_t)S * Hq * n_splits * (d + 2);
    const size_t need = q_bytes + 2 * h_bytes + 2 * s_bytes + part_bytes;
    if (need > c->dec_ws_bytes) {
        WEED_HIP_CHECK(hipStreamSynchronize(stream()));
        (void)hipFree(c->dec_ws);
        c->dec_ws = nullptr;
        c->dec_ws_bytes = 0;
        if (hipMalloc((void **)&c->dec_ws, need) != hipSuccess) {
            return fail(WEED_HIP_ENOMEM, "%s: workspace allocation of %zu bytes failed", fn, need);
        }
        c->dec_ws_bytes = need;
    }
    uint8_t *wsp = reinterpret_cast<uint8_t *>(c->dec_ws);
    float *q_rot = reinterpret_cast<float *>(wsp);
    uint16_t *q_hi = reinterpret_cast<uint16_t *>(wsp + q_bytes);
    uint16_t *q_lo = reinterpret_cast<uint16_t *>(wsp + q_bytes + h_bytes);
    float *q_scale = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes);
    float *q_sum = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes + s_bytes);
    float *partials = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes + 2 * s_bytes);

    Geom3 qg = { q_off, { q_stride[0], q_stride[1], q_stride[2] } };
    Geom3 og = { o_off, { o_stride[0], o_stride[1], o_stride[2] } };
    prep_q_kernel<<<dim3(Hq, S), 256, 0, stream()>>>(q_dev, qg, Hq, d, c->k.rot_t, rot_q ? 1 : 0, q_rot, q_hi, q_lo,
                                                     q_scale, q_sum);
    WEED_HIP_LAUNCH_CHECK();

    if (use_mfma) {
        MfmaParams mp;
        mp.k = side_params(c, 0);
        mp.v = side_params(c, 1);
        mp.lens = lens_dev ? lens_dev : c->lens_dev;
        mp.padded = c->padded_tokens;
        mp.Hq = Hq;
        mp.Hkv = Hkv;
        mp.G = G;
        mp.blocked = gqa_mapping == WEED_HIP_GQA_BLOCKED;
        mp.q_hi = q_hi;
        mp.q_lo = q_lo;
        mp.q_scale = q_scale;
        mp.q_sum = q_sum;
        mp.partials = partials;
        mp.n_splits = n_splits;
        mp.blocks_per_split = blocks_per_split;
        ProfileScope prof("kv_decode_attn");
        WEED_HIP_TRY(launch_mfma_decode(mp, d, S, stream()));
    } else {
        DecodeParams p;
        p.k = side_params(c, 0);
        p.v = side_params(c, 1);
        p.lens = lens_dev ? lens_dev : c->lens_dev;
        p.padded = c->padded_tokens;
        p.d = d;
        p.Hq = Hq;
        p.Hkv = Hkv;
        p.G = G;
        p.blocked = gqa_mapping == WEED_HIP_GQA_BLOCKED;
        p.q_rot = q_rot;
        p.partials = partials;
        p.n_splits = n_splits;
        p.split_tokens = split_tokens;
        ProfileScope prof("kv_decode_attn");
        decode_generic_kernel<<<dim3(n_splits, Hkv, S), kThreads, 0, stream()>>>(p);
        WEED_HIP_LAUNCH_CHECK();
    }
    {
        ProfileScope prof("kv_decode_combine");
        combine_kernel<<<dim3(Hq, S), 256, 0, stream()>>>(partials, Hq, d, n_splits, c->v.rot, unrot ? 1 : 0,
                                                          use_mfma ? 1 : 0, out_dev, og);
        WEED_HIP_LAUNCH_CHECK();
    }
    return WEED_HIP_OK;
}

} // namespace

extern "C" int weed_hip_kv_decode_attn(weed_hip_kv_cache *c, int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev,
                                       uint32_t q_off, const uint32_t q_stride[3], float *out_dev, uint32_t o_off,
                                       const uint32_t o_stride[3], uint32_t flags)
{
    return decode_impl("weed_hip_kv_decode_attn", c, n_q_heads, gqa_mapping, q_dev, q_off, q_stride, out_dev, o_off,
                       o_stride, flags, nullptr);
}

extern "C" int weed_hip_kv_decode_attn_prefix(weed_hip_kv_cache *c, const int32_t *lens_dev, int32_t n_q_heads,
                                              int32_t gqa_mapping, const float *q_dev, uint32_t q_off,
                                              const uint32_t q_stride[3], float *out_dev, uint32_t o_off,
                                              const uint32_t o_stride[3], uint32_t flags)
{
    const char *fn = "weed_hip_kv_decode_attn_prefix";
    WEED_HIP_REQUIRE(lens_dev, "%s: null length array", fn);
    return decode_impl(fn, c, n_q_heads, gqa_mapping, q_dev, q_off, q_stride, out_dev, o_off, o_stride, flags, lens_dev);
}
