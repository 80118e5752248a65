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

// Workspace of weed_hip_kv_decode_attn_noalloc: rotated queries, their fp16 halves, block offsets and the split
// partials of one call.  Every device the library runs on holds its own copy until the process ends; in host code the
// array's name is only a handle for hipGetSymbolAddress, the kernels get the address kept in g_scratch_dev.
constexpr size_t kStaticScratchBytes = 32u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_dev[kMaxDevices] = {};
__global__ void __launch_bounds__(256) clear_words_kernel(uint32_t *p, uint32_t n)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        p[i] = 0u;
    }
}
} // namespace

namespace weedhip {
// Called by weed_hip_init with `device_id` current: looks the device's copy of `scratch` up once.
int decode_scratch_setup(int device_id)
{
    if (device_id < 0 || device_id >= kMaxDevices) {
        return fail(WEED_HIP_EINVAL, "decode_scratch_setup: device %d outside [0, %d)", device_id, kMaxDevices);
    }
    if (!g_scratch_dev[device_id]) {
        void *ptr = nullptr;
        WEED_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        g_scratch_dev[device_id] = ptr;
    }
    return WEED_HIP_OK;
}
int decode_scratch_clear_counters()
{
    const int dev = current_device();
    if (dev < 0 || dev >= kMaxDevices || !g_scratch_dev[dev]) {
        return WEED_HIP_OK; // the library has not been started on this device: nothing to clear
    }
    clear_words_kernel<<<(kMfmaMergeCounters + 255) / 256, 256, 0, stream()>>>(static_cast<uint32_t *>(g_scratch_dev[dev]),
                                                                              kMfmaMergeCounters);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}
} // namespace weedhip

namespace {

constexpr int kGMax = 8;        // query heads of one kv head handled per pass
constexpr int kThreads = 256;
constexpr int kChunk = 256;     // tokens per inner iteration of the generic kernel

struct DecodeParams {
    SideParams k, v;
    const int32_t *lens;
    uint32_t padded;
    uint32_t d;      // head_dim as stored (a multiple of 32)
    uint32_t d_real; // the caller's head_dim (the scores are divided by its square root)
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

// blk_off[i] = number of 64-token blocks of the sequences before i, blk_off[n_seq] = all of them.  One workgroup of
// 256 threads: every thread sums a chunk, the chunk sums are scanned in LDS.
__device__ void block_offsets(const int32_t *__restrict__ lens, uint32_t n_seq, uint32_t *__restrict__ blk_off)
{
    __shared__ uint32_t chunk_sum[256];
    const uint32_t tid = threadIdx.x;
    const uint32_t per = (n_seq + 255) / 256;
    const uint32_t i0 = min(tid * per, n_seq), i1 = min(i0 + per, n_seq);
    uint32_t mine = 0;
    for (uint32_t i = i0; i < i1; ++i) {
        mine += ((uint32_t)lens[i] + 63u) >> 6;
    }
    chunk_sum[tid] = mine;
    __syncthreads();
    for (uint32_t k = 1; k < 256; k <<= 1) {
        const uint32_t add = tid >= k ? chunk_sum[tid - k] : 0;
        __syncthreads();
        chunk_sum[tid] += add;
        __syncthreads();
    }
    uint32_t run = chunk_sum[tid] - mine; // exclusive prefix of this thread's chunk
    for (uint32_t i = i0; i < i1; ++i) {
        blk_off[i] = run;
        run += ((uint32_t)lens[i] + 63u) >> 6;
    }
    if (tid == 255) {
        blk_off[n_seq] = chunk_sum[255];
    }
    __syncthreads();
}

// q_rot[s][h][:] = q[s][h][:] . Rk  (multihead_attention.cpp:276), or a plain gather when rotate == 0.
// For the matrix-core kernel the rotated query is also scaled by log2(e)/sqrt(d), divided by a power of two that
// brings it into [-1, 1], and split into fp16 hi + lo halves.
// `d`: head_dim as stored (a multiple of 32); `d_real` <= d: coordinates the caller's query has (zeros beyond them).
__global__ void __launch_bounds__(256) prep_q_kernel(const float *__restrict__ q, Geom3 g, uint32_t Hq, uint32_t d,
                                                     uint32_t d_real, const float *__restrict__ rot_t, int rotate,
                                                     float *__restrict__ q_rot, uint16_t *__restrict__ q_hi,
                                                     uint16_t *__restrict__ q_lo, float *__restrict__ q_scale,
                                                     float *__restrict__ q_sum, const int32_t *__restrict__ lens,
                                                     uint32_t n_seq, uint32_t *__restrict__ blk_off)
{
    __shared__ float qs[256];
    __shared__ float red_max[256];
    __shared__ float red_sum[256];
    const uint32_t h = blockIdx.x, s = blockIdx.y;
    const uint32_t tid = threadIdx.x;
    if (s == n_seq) {
        // the extra grid row: one of its workgroups builds the block offsets while the others rotate queries (as part
        // of a query's workgroup the scan would be the kernel's longest chain)
        if (blk_off && h == 0) {
            block_offsets(lens, n_seq, blk_off);
        }
        return;
    }
    if (tid < d) {
        qs[tid] = tid < d_real
                      ? q[(uint64_t)g.off + (uint64_t)s * g.s[0] + head_offset(g, h) + (uint64_t)tid * g.s[2]]
                      : 0.0f;
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
    const float qc = acc * (1.4426950408889634f / sqrtf((float)d_real));
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

constexpr int kRowsPerWg = 4;

// The same as prep_q_kernel for kRowsPerWg (sequence, head) rows per workgroup: thread j owns output coordinate j of
// every row, so each element of the rotation is read once per workgroup instead of once per row.  Used when there
// are many rows (batched decode); results are identical (same order of fused multiply-adds).
__global__ void __launch_bounds__(256) prep_q_rows_kernel(const float *__restrict__ q, Geom3 g, uint32_t Hq, uint32_t d,
                                                          uint32_t d_real, uint32_t n_rows,
                                                          const float *__restrict__ rot_t, int rotate,
                                                          float *__restrict__ q_rot, uint16_t *__restrict__ q_hi,
                                                          uint16_t *__restrict__ q_lo, float *__restrict__ q_scale,
                                                          float *__restrict__ q_sum, const int32_t *__restrict__ lens,
                                                          uint32_t n_seq, uint32_t *__restrict__ blk_off)
{
    __shared__ float qs[kRowsPerWg][256];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t row0 = blockIdx.x * kRowsPerWg;
    // The rotation does not depend on the query: its first 64 elements per thread are requested before anything else,
    // so that they travel together with the query rows (one round trip to memory instead of two).  d is a multiple of
    // 64 here (the host checks).
    const bool rot_thread = rotate && tid < d;
    float x0[64];
    auto request = [&](float (&x)[64], uint32_t i0) {
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            x[u] = rot_t[tid + d * (i0 + u)];
        }
    };
    if (blockIdx.x * kRowsPerWg >= n_rows) {
        // the extra workgroup behind the last rows: it builds the block offsets while the others rotate queries (as
        // part of a query's workgroup the scan would be the kernel's longest chain)
        if (blk_off) {
            block_offsets(lens, n_seq, blk_off);
        }
        return;
    }
    if (rot_thread) {
        request(x0, 0);
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWg; ++r) {
        const uint32_t row = row0 + r;
        float v = 0.0f;
        if (row < n_rows && tid < d_real) {
            const uint32_t s = row / Hq, h = row % Hq;
            v = q[(uint64_t)g.off + (uint64_t)s * g.s[0] + head_offset(g, h) + (uint64_t)tid * g.s[2]];
        }
        qs[r][tid] = v;
    }
    __syncthreads();
    float acc[kRowsPerWg];
#pragma unroll
    for (int r = 0; r < kRowsPerWg; ++r) {
        acc[r] = rotate ? 0.0f : qs[r][tid];
    }
    if (rot_thread) {
        // sixty-four elements at a time (same order of fused multiply-adds as the single-row kernel)
        for (uint32_t i0 = 0; i0 < d; i0 += 64) {
            if (i0) {
                request(x0, i0);
            }
#pragma unroll
            for (int u = 0; u < 64; ++u) {
#pragma unroll
                for (int r = 0; r < kRowsPerWg; ++r) {
                    acc[r] = fmaf(qs[r][i0 + u], x0[u], acc[r]);
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kRowsPerWg; ++r) {
        qs[r][tid] = tid < d ? acc[r] : 0.0f;
    }
    __syncthreads();
    // one wavefront per row from here on
    for (uint32_t r = wave; r < (uint32_t)kRowsPerWg; r += 4) {
        const uint32_t row = row0 + r;
        if (row >= n_rows) {
            break;
        }
        const float k = 1.4426950408889634f / sqrtf((float)d_real);
        float mx = 0.0f, sum = 0.0f;
        for (uint32_t j = lane; j < d; j += 64) {
            const float qc = qs[r][j] * k;
            mx = fmaxf(mx, fabsf(qc));
            sum += qc;
        }
        mx = wave_max(mx);
        // the single-row kernel adds the coordinates pairwise over 256 slots; keep its summation tree: fold 64 lanes
        sum = wave_sum(sum);
        int e = 0;
        (void)frexpf(mx, &e);
        e = e < -100 ? -100 : (e > 100 ? 100 : e);
        const float inv = ldexpf(1.0f, -e);
        for (uint32_t j = lane; j < d; j += 64) {
            const float a = qs[r][j];
            const float qn = a * k * inv;
            const _Float16 hi = (_Float16)qn;
            const _Float16 lo = (_Float16)(qn - (float)hi);
            q_rot[(uint64_t)row * d + j] = a;
            q_hi[(uint64_t)row * d + j] = __builtin_bit_cast(uint16_t, hi);
            q_lo[(uint64_t)row * d + j] = __builtin_bit_cast(uint16_t, lo);
        }
        if (lane == 0) {
            q_scale[row] = ldexpf(1.0f, e);
            q_sum[row] = sum;
        }
    }
}

// Generic kernel: any head_dim that is a multiple of 32, any field width, any group size.
__global__ void __launch_bounds__(kThreads) decode_generic_kernel(DecodeParams p)
{
    __shared__ float q_s[kGMax * 256];
    __shared__ float qsum_s[kGMax];
    __shared__ float sc[kGMax * kChunk];
    __shared__ float m_s[kGMax], l_s[kGMax], scale_s[kGMax];
    __shared__ float o_s[kGMax * 256];
    __shared__ float ktab[256], vtab[256];

    const uint32_t split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t d = p.d;
    const uint32_t L = (uint32_t)p.lens[seq];
    const uint32_t n0 = split * p.split_tokens;
    const uint32_t n1 = min(L, n0 + p.split_tokens);
    const uint64_t region = (uint64_t)seq * p.Hkv + kvh;
    const float sqrt_d = sqrtf((float)p.d_real);
    const uint32_t parts = kThreads / d ? kThreads / d : 1;
    const uint32_t part = tid / d, jj = tid % d;
    const bool pv_active = part < parts;

    // fields wider than 5 bits exist in the uniform coder only, whose table is code + 0.5
    static_assert(kThreads == 256, "one table entry per thread");
    ktab[tid] = p.k.w > 5U ? (float)tid + 0.5f : p.k.table[tid & 31U];
    vtab[tid] = p.v.w > 5U ? (float)tid + 0.5f : p.v.table[tid & 31U];

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
constexpr uint32_t kMaxSlots = 1024; // partials per (sequence, head) that combine_kernel can weigh in one pass

// Run-length skew between the wavefront age classes of a workgroup, in percent of the mean run (see RunGeom): with
// two wavefronts per SIMD the older one gets 16 % more than the mean; with three the spread between oldest and
// youngest is wider (measured on the ragged batch: 16 % -> 47.8 us, 24-40 % -> 46.7-46.9 us, 48 % -> 48.2 us).
constexpr uint32_t kRunSkewPercent = 16, kRunSkewPercent3 = 28;
// Most regions that the blocks of one workgroup may lie in for the workgroups to merge their regions themselves in the
// general case (see decode_impl).
constexpr uint32_t kMostRegionsMergedByWorkgroup = 6;
// ... and most rows (region, head) of them: two passes of the merge (96 sequences of 2100 or 5000 tokens with four heads
// per kv head, five regions = 20 rows per workgroup: 59.2 and 116.8 us, against 51.2 and 111.9 with the merge kernel)
constexpr uint32_t kMostRowsMergedByWorkgroup = 16;

// Tuning knobs of the work partition.  The defaults come from the environment, read ONCE per process (at the first
// decode call or the first weed_hip_kv_decode_tuning): WEED_HIP_DECODE_WAVES (wavefronts the block list is cut for),
// WEED_HIP_DECODE_SKEW (percent), WEED_HIP_DECODE_SEARCH=1 (always find a wavefront's first region by search, even in
// a batch of equal contexts).
// Shortest and longest mean run for which neighbouring runs take their blocks in turns (see RunGeom::group_cycles).
constexpr uint32_t kFewestBlocksOfRunsInTurns = 4, kMostBlocksOfRunsInTurns = 32;
struct DecodeTuning {
    int wavefronts = 0;    // 0: as many as the device holds at once
    int skew_percent = -1; // < 0: kRunSkewPercent
    bool always_search = false;
    bool separate_merge = false; // always merge the partials with the second kernel
    bool separate_query = false; // always rotate the queries with the kernel ahead
    bool contiguous_runs = false; // never let neighbouring runs take turns (RunGeom::group_cycles)
    bool print_plan = false;      // WEED_HIP_DECODE_PLAN=1: every call writes its partition to stderr
};
DecodeTuning &decode_tuning()
{
    static DecodeTuning t = [] {
        DecodeTuning v;
        if (const char *env = std::getenv("WEED_HIP_DECODE_WAVES")) {
            v.wavefronts = std::max(0, std::atoi(env));
        }
        if (const char *env = std::getenv("WEED_HIP_DECODE_SKEW")) {
            v.skew_percent = std::atoi(env);
        }
        if (const char *env = std::getenv("WEED_HIP_DECODE_SEARCH")) {
            v.always_search = (std::atoi(env) & 1) != 0;
            v.separate_merge = (std::atoi(env) & 2) != 0;
            v.separate_query = (std::atoi(env) & 4) != 0;
            v.contiguous_runs = (std::atoi(env) & 8) != 0;
        }
        if (const char *env = std::getenv("WEED_HIP_DECODE_PLAN")) {
            v.print_plan = std::atoi(env) != 0;
        }
        return v;
    }();
    return t;
}

struct SlotGeom {
    const uint32_t *blk_off; // null: every (sequence, head) has `max_slots` valid partials
    uint32_t Hkv, G;
    RunGeom runs; // matrix-core kernel: how the block list was cut into per-wavefront runs
    int blocked;
    uint32_t uniform_blocks; // blocks per sequence when all sequences span the same number (blk_off is then not read:
                             // nothing may have computed it), else 0
};

// Partial slots of head h of sequence s: the wavefronts whose runs intersect the head's region, in order.
__device__ __forceinline__ uint32_t slots_of_row(const SlotGeom &sg, uint32_t s, uint32_t h)
{
    const uint32_t first_blk = sg.uniform_blocks ? s * sg.uniform_blocks : sg.blk_off[s];
    const uint32_t nb = sg.uniform_blocks ? sg.uniform_blocks : sg.blk_off[s + 1] - first_blk;
    if (nb == 0) {
        return 0;
    }
    const uint32_t kvh = sg.blocked ? h / sg.G : h % sg.Hkv;
    const uint32_t begin = first_blk * sg.Hkv + kvh * nb;
    return run_of_block(sg.runs, begin + nb - 1) - run_of_block(sg.runs, begin) + 1;
}

__global__ void combine_kernel(const float *__restrict__ partials, uint32_t Hq, uint32_t d, uint32_t d_real,
                               uint32_t max_slots, SlotGeom sg, const float *__restrict__ rv, int unrotate,
                               int log2_domain, float *__restrict__ out, Geom3 og)
{
    __shared__ float w_s[1024];
    __shared__ float o_sh[256];
    __shared__ float o_part[1024];
    __shared__ float red[2];
    const uint32_t h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
    const float *base = partials + ((uint64_t)s * Hq + h) * max_slots * (d + 2);
    uint32_t n_splits = max_slots;
    if (sg.blk_off) {
        n_splits = slots_of_row(sg, s, h);
    }
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
    {
        // thread groups of d2 (power of two >= d) threads take the partials in turn, then the groups are added up
        uint32_t d2 = 32;
        while (d2 < d) {
            d2 <<= 1;
        }
        const uint32_t grp = tid / d2, ngrp = blockDim.x / d2, j = tid % d2;
        float acc = 0.0f;
        if (j < d) {
            // eight partials at a time, so that their loads are in flight together
            for (uint32_t k0 = grp; k0 < n_splits; k0 += 8 * ngrp) {
                float y[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const uint32_t k = k0 + u * ngrp;
                    y[u] = (k < n_splits && w_s[k] != 0.0f) ? base[(uint64_t)k * (d + 2) + 2 + j] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const uint32_t k = k0 + u * ngrp;
                    if (k < n_splits && w_s[k] != 0.0f) {
                        acc = fmaf(w_s[k], y[u], acc);
                    }
                }
            }
        }
        o_part[tid] = acc;
        __syncthreads();
        if (tid < d) {
            float tot = 0.0f;
            for (uint32_t gI = 0; gI < ngrp; ++gI) {
                tot += o_part[gI * d2 + tid];
            }
            o_sh[tid] = (denom > 0.0f) ? tot / denom : 0.0f;
        }
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
    if (tid < d_real) {
        out[(uint64_t)og.off + (uint64_t)s * og.s[0] + head_offset(og, h) + (uint64_t)tid * og.s[2]] = r;
    }
}

// The same as combine_kernel for kRowsPerWg (sequence, head) rows per workgroup and at most 64 partials per row:
// thread j owns coordinate j of every row, so the rotation is read once per workgroup.
__global__ void __launch_bounds__(256) combine_rows_kernel(const float *__restrict__ partials, uint32_t Hq, uint32_t d,
                                                           uint32_t d_real, uint32_t max_slots, uint32_t n_rows,
                                                           SlotGeom sg,
                                                           const float *__restrict__ rv, int unrotate, int log2_domain,
                                                           float *__restrict__ out, Geom3 og)
{
    __shared__ float w_s[kRowsPerWg][64];
    __shared__ float denom_s[kRowsPerWg];
    __shared__ uint32_t n_s[kRowsPerWg];
    __shared__ float o_sh[kRowsPerWg][256];
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = blockIdx.x * kRowsPerWg;
    const uint32_t PS = d + 2;
    // The rotation does not depend on the partials: its first elements are requested before anything else, so that they
    // travel together with the partials.  d is a multiple of 64 here (the host checks).
    const bool rot_thread = unrotate && tid < d;
    float x0[64];
    auto request = [&](float (&x)[64], uint32_t j0) {
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            x[u] = rv[tid + d * (j0 + u)];
        }
    };
    if (rot_thread) {
        request(x0, 0);
    }
    // Thread groups of d2 (power of two >= d) threads take the partials in turn.  The first four partials of every
    // group and row are requested here, before their weights are known (slots that turn out to be unused are read
    // and dropped), so that they travel together with the partials' headers.
    uint32_t d2 = 32;
    while (d2 < d) {
        d2 <<= 1;
    }
    const uint32_t grp = tid / d2, ngrp = 256 / d2, j = tid % d2;
    const bool col_ok = j < d;
    float x[kRowsPerWg][4];
#pragma unroll
    for (int r = 0; r < kRowsPerWg; ++r) {
        const float *base = partials + (uint64_t)(row0 + r) * max_slots * PS + 2 + j;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t k = grp + u * ngrp;
            x[r][u] = (col_ok && row0 + r < n_rows && k < max_slots) ? base[(uint64_t)k * PS] : 0.0f;
        }
    }
    {
        // one wavefront per row, one lane per partial: weights of the row's partials
        static_assert(kRowsPerWg == 4, "one 64-lane wavefront per row");
        const uint32_t r = tid >> 6, l = tid & 63;
        const uint32_t row = row0 + r;
        uint32_t n = 0;
        if (row < n_rows) {
            n = max_slots;
            if (sg.blk_off) {
                n = slots_of_row(sg, row / Hq, row % Hq);
            }
        }
        const float *base = partials + (uint64_t)row * max_slots * PS;
        float m0 = -INFINITY, l0 = 0.0f;
        if (l < n) {
            m0 = base[(uint64_t)l * PS];
            l0 = base[(uint64_t)l * PS + 1];
        }
        const float mx = wave_max(m0);
        const float w0 = (m0 == -INFINITY) ? 0.0f : (log2_domain ? exp2f(m0 - mx) : expf(m0 - mx));
        const float sum = wave_sum(w0 * l0);
        w_s[r][l] = w0;
        if (l == 0) {
            denom_s[r] = sum;
            n_s[r] = n;
        }
    }
    __syncthreads();
    {
        float acc[kRowsPerWg];
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            const float *base = partials + (uint64_t)(row0 + r) * max_slots * PS + 2 + j;
            const uint32_t n = n_s[r];
            float a = 0.0f;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t k = grp + u * ngrp;
                // (an unused slot may hold anything, so it is skipped rather than weighted with zero)
                a = k < n ? fmaf(w_s[r][k], x[r][u], a) : a;
            }
            if (col_ok) {
                // further partials eight at a time, so that their loads are in flight together (ragged batches and
                // long contexts leave dozens of partials per row)
                for (uint32_t k0 = grp + 4 * ngrp; k0 < n; k0 += 8 * ngrp) {
                    float y[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const uint32_t k = k0 + u * ngrp;
                        y[u] = k < n ? base[(uint64_t)k * PS] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const uint32_t k = k0 + u * ngrp;
                        a = k < n ? fmaf(w_s[r][k], y[u], a) : a;
                    }
                }
            }
            acc[r] = a;
        }
        // add the groups up through LDS (o_sh doubles as the staging area: [row][group * d2 + j])
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            o_sh[r][tid] = acc[r];
        }
        __syncthreads();
        float tot[kRowsPerWg];
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            float t = 0.0f;
            if (tid < d) {
                for (uint32_t gI = 0; gI < ngrp; ++gI) {
                    t += o_sh[r][gI * d2 + tid];
                }
                const float den = denom_s[r];
                t = den > 0.0f ? t / den : 0.0f;
            }
            tot[r] = t;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            o_sh[r][tid] = tot[r];
        }
    }
    __syncthreads();
    if (tid >= d) {
        return;
    }
    float res[kRowsPerWg];
    if (unrotate) {
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            res[r] = 0.0f;
        }
        for (uint32_t j0 = 0; j0 < d; j0 += 64) {
            if (j0) {
                request(x0, j0);
            }
#pragma unroll
            for (int u = 0; u < 64; ++u) {
#pragma unroll
                for (int r = 0; r < kRowsPerWg; ++r) {
                    res[r] = fmaf(o_sh[r][j0 + u], x0[u], res[r]);
                }
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < kRowsPerWg; ++r) {
            res[r] = o_sh[r][tid];
        }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWg; ++r) {
        const uint32_t row = row0 + r;
        if (row < n_rows && tid < d_real) {
            const uint32_t s = row / Hq, h = row % Hq;
            out[(uint64_t)og.off + (uint64_t)s * og.s[0] + head_offset(og, h) + (uint64_t)tid * og.s[2]] = res[r];
        }
    }
}

// `lens_dev` (optional): attend over these per-sequence lengths instead of the cached ones.
// `n_tokens` > 1: a chunk of query positions per sequence, the last `n_tokens` of the attended tokens being the
// chunk's own (position t sees all but the last n_tokens - 1 - t); q_tstride / o_tstride step between positions.
int decode_impl(const char *fn, weed_hip_kv_cache *c, int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev,
                uint32_t q_off, const uint32_t q_stride[3], float *out_dev, uint32_t o_off, const uint32_t o_stride[3],
                uint32_t flags, const int32_t *lens_dev, uint32_t n_tokens = 1, uint32_t q_tstride = 0,
                uint32_t o_tstride = 0, uint8_t *fixed_ws = nullptr, size_t fixed_ws_bytes = 0)
{
    WEED_HIP_REQUIRE(c, "%s: null cache", fn);
    WEED_HIP_REQUIRE(q_dev && out_dev && q_stride && o_stride, "%s: null pointer", fn);
    // d: head_dim as stored (a multiple of 32, see weed_hip_kv_cache::dp); d_real: the caller's
    const uint32_t Hkv = (uint32_t)c->cfg.n_kv_heads, d = c->dp, S = (uint32_t)c->cfg.n_seq;
    const uint32_t d_real = (uint32_t)c->cfg.head_dim;
    WEED_HIP_REQUIRE(n_q_heads > 0 && (uint32_t)n_q_heads % Hkv == 0,
                     "%s: n_q_heads %d must be a positive multiple of n_kv_heads %u", fn, n_q_heads, Hkv);
    WEED_HIP_REQUIRE(gqa_mapping == WEED_HIP_GQA_WEED || gqa_mapping == WEED_HIP_GQA_BLOCKED,
                     "%s: unknown GQA mapping %d", fn, gqa_mapping);
    const bool rot_q = flags & WEED_HIP_ATTN_ROTATE_Q, unrot = flags & WEED_HIP_ATTN_UNROTATE_OUT;
    WEED_HIP_REQUIRE(!(rot_q || unrot) || c->has_rotations, "%s: rotation requested but no rotations are set", fn);
    // the kernels see (position, head) pairs as heads
    const uint32_t real_heads = (uint32_t)n_q_heads;
    const uint32_t Hq = real_heads * n_tokens;

    uint32_t max_len = 0;
    for (int32_t l : c->lens) {
        max_len = std::max(max_len, (uint32_t)l);
    }
    const uint32_t G = Hq / Hkv;
    // groups (or chunks: positions x heads) beyond a tile's rows take several passes of the matrix-core kernel
    const uint32_t tile_rows = mfma_decode_tile_rows(d);
    const uint32_t passes = (G + tile_rows - 1) / tile_rows;
    const uint32_t pass_heads = (G + passes - 1) / passes;
    const bool use_mfma = mfma_decode_supported(d, c->k.w, c->v.w, pass_heads);
    WEED_HIP_REQUIRE(n_tokens == 1 || use_mfma,
                     "%s: head_dim %u with fields of %u and %u bits is not served by the matrix-core kernel, which a "
                     "chunk of positions needs", fn, d, c->k.w, c->v.w);
    // ONE copy of the process-wide tuning for the whole plan: weed_hip_kv_decode_tuning may change it from another host
    // thread at any time, and a plan must not pair a block count chosen under one setting with a search mode of another.
    const DecodeTuning tune = decode_tuning();
    uint32_t n_splits, split_tokens = 0;
    uint32_t total_blocks = 0;
    RunGeom runs = { 1, 0, 8, 0 };
    // Blocks per sequence as the partition counts them when that is more than the sequences have (see below), else 0.
    uint32_t virtual_blocks = 0;
    auto partition_blocks = [&](int32_t l) { return virtual_blocks ? virtual_blocks : ((uint32_t)l + 63u) >> 6; };
    if (use_mfma) {
        // every wavefront takes an equal run of 64-token blocks from the list of all regions' blocks; as many
        // wavefronts as the device holds at once
        runs.waves = mfma_decode_workgroup_waves(pass_heads, d, c->k.w, c->v.w);
        // Equal sequences of nb blocks: prefer a run length with which every workgroup holds whole regions (the
        // kernel then does the whole call by itself, see below): nb / (classes * q) blocks with q = 1, 2 or 4, that
        // is 4 / q regions per workgroup, provided the workgroups fill the compute units in at most two rounds.
        // A block count that no such run length divides is rounded up to the next one that one does (see below):
        // the partition then counts blocks at the end of every region that hold no tokens, which the kernel skips
        // as it skips those beyond a prefix length, and the wavefront they fall to has that much less to do -- far
        // cheaper than runs that straddle regions.
        uint32_t preferred_unit = 0;
        // Sequences with different block counts are counted alike, as the longest of them, within the same bounds.
        uint32_t most = 0, fewest = ~0u;
        uint64_t real_blocks = 0;
        for (int32_t l : c->lens) {
            most = std::max(most, ((uint32_t)l + 63u) >> 6);
            fewest = std::min(fewest, ((uint32_t)l + 63u) >> 6);
            real_blocks += ((uint32_t)l + 63u) >> 6;
        }
        // (The blocks without tokens may come to three quarters of those with, over the whole batch: a wavefront
        // whose run holds few tokens or none is done early and leaves the memory system to the others, so the call
        // takes about as long as its tokens' bytes take -- down to the time that the longest sequence's own
        // wavefronts need, which is what bounds the ratio.  Measured on 64 sequences with lengths drawn from
        // [4096, 8192]: 104.6 us with runs that straddle regions, 84.4 us counted alike; from [512, 8192], where the
        // partition would count 1.78 blocks per block with tokens: 76.3 against 73.9 us, a tie.)
        // Calls of less than a few dozen microseconds are all fixed cost, of which runs that straddle regions have
        // more: there the ratio may be four (16 sequences from [512, 8192]: 42 us against 33 us).  What bounds such
        // calls is the blocks as counted, which is what a wavefront of the longest sequence works through: 32
        // sequences with up to 8192 tokens each gain 8 to 17 us counted alike, 48 such sequences lose 5 to 44 us.
        const uint64_t counted_alike = (uint64_t)most * S * Hkv;
        const uint64_t most_counted = counted_alike > 32768 ? real_blocks * 7 / 4
            : counted_alike > 16384                         ? real_blocks * 5 / 2
                                                            : real_blocks * 4;
        // (counts beyond what a region's memory holds are fine: the kernel reads nothing behind a region's last block)
        // (and no further than 4096 blocks past the longest: the counts that qualify below recur every few hundred
        // blocks at most, so a search that has found none by then finds none, and the host's time stays bounded)
        const uint32_t reach = (uint32_t)std::min<uint64_t>(std::max<uint64_t>(most_counted / S, fewest + 1),
                                                            std::min<uint64_t>((uint64_t)most + 4096, 1u << 24));
        // (instances that cannot merge their partials themselves gain from runs that stay inside regions as well)
        // (not for groups that take several passes: they do not merge in their workgroups, and every pass would walk
        // the blocks that the rounding adds -- 64 sequences of 2100 tokens, 64 heads on 2 kv heads of 224: 198 us with
        // the rounding, 160 without)
        const bool may_round =
            fewest != 0 && tune.wavefronts == 0 && !tune.separate_merge && !tune.always_search && passes == 1;
        {
            const uint32_t nb = most;
            // Fewer blocks than wavefronts and regions of no more blocks than a workgroup has wavefronts: the call is
            // all fixed cost, of which the rows that a workgroup rotates and merges one pass after the other are the
            // largest part, so as few regions per workgroup as one round of workgroups allows, however few of the
            // compute units they fill (3 to 96 sequences of 100 tokens with groups of eight: 27 us with four regions
            // per workgroup, 14 us with one).
            const bool tiny = real_blocks * Hkv <= (uint64_t)runs.waves * 256u && nb <= runs.waves;
            if (may_round && tiny) {
                const uint32_t classes = run_classes(runs), regions = S * Hkv;
                for (uint32_t q = 4; q >= 1 && !preferred_unit; q /= 2) {
                    if ((regions * q + 3) / 4 > 256) {
                        continue;
                    }
                    for (uint32_t cand = nb; cand <= reach; ++cand) {
                        if (cand % (classes * q) == 0) {
                            preferred_unit = cand / (classes * q);
                            virtual_blocks = cand == fewest ? 0 : cand;
                            break;
                        }
                    }
                }
            }
            if (may_round && !preferred_unit) {
                const uint32_t classes = run_classes(runs), regions = S * Hkv;
                for (uint32_t cand = nb; cand <= reach && !preferred_unit; ++cand) {
                    // (one or two rounds of workgroups; above head_dim 128, where a workgroup's queries and merges
                    // take longer and a compute unit holds one workgroup, one round only)
                    uint32_t best_rounds = d > 128 ? 2 : 3;
                    for (uint32_t q = 1; q <= 4; q *= 2) {
                        if (cand % (classes * q) != 0) {
                            continue;
                        }
                        const uint32_t wgs = (regions * q + 3) / 4, rounds = (wgs + 255) / 256;
                        if (rounds < best_rounds && wgs * 100 >= rounds * 256 * 95) {
                            best_rounds = rounds;
                            preferred_unit = cand / (classes * q);
                            virtual_blocks = cand == fewest ? 0 : cand;
                        }
                    }
                }
            }
        }
        uint64_t blocks = 0;
        for (int32_t l : c->lens) {
            blocks += partition_blocks(l);
        }
        blocks *= Hkv;
        WEED_HIP_REQUIRE(blocks < (1ull << 32), "%s: too many cached tokens for one launch", fn);
        total_blocks = (uint32_t)blocks;
        // one workgroup per compute unit
        const uint32_t target_units = tune.wavefronts > 0 ? (uint32_t)tune.wavefronts : runs.waves * 256u;
        runs.unit_blocks = preferred_unit ? preferred_unit : std::max(1u, (total_blocks + target_units - 1) / target_units);
        // Small batches of long sequences, where a region is several workgroups' shares: the same rounding, to a
        // whole number of those shares.
        if (!preferred_unit && may_round) {
            for (uint32_t cand = most; cand <= reach; ++cand) {
                // (the run length that this count would get)
                const uint64_t all = (uint64_t)cand * S * Hkv;
                const uint32_t unit = (uint32_t)std::max<uint64_t>(1, (all + target_units - 1) / target_units);
                const uint32_t wg_blocks = runs.waves * unit;
                if (cand % wg_blocks == 0 && cand / wg_blocks <= 64 && all < (1ull << 32)) {
                    if (cand != fewest) {
                        virtual_blocks = cand;
                        total_blocks = (uint32_t)all;
                    }
                    runs.unit_blocks = unit;
                    break;
                }
            }
        }
        const uint32_t skew_pct = tune.skew_percent >= 0 ? (uint32_t)std::min(90, tune.skew_percent)
                                                         : (runs.waves == 12 ? kRunSkewPercent3 : kRunSkewPercent);
        const uint32_t nblk = virtual_blocks ? virtual_blocks : (max_len + 63) / 64;
        for (;;) {
            runs.skew = std::min(runs.unit_blocks - 1, (runs.unit_blocks * skew_pct + 50) / 100);
            const uint32_t shortest = runs.unit_blocks - runs.skew;
            n_splits = (nblk + shortest - 1) / shortest + 1; // partial slots per (sequence, head)
            if (n_splits <= kMaxSlots) {
                break;
            }
            // one very long region and few of them: longer runs (fewer wavefronts) keep the merge within its limit
            runs.unit_blocks += std::max(1u, runs.unit_blocks / 8);
        }
    } else {
        // split the context so that the launch has a few workgroups per compute unit
        const uint32_t target_wgs = 2048;
        const uint32_t want = std::min((uint32_t)kMaxSlots, std::max(1u, target_wgs / (S * Hkv)));
        n_splits = std::max(1u, std::min((max_len + kChunk - 1) / kChunk, want));
        split_tokens = (max_len + n_splits - 1) / n_splits;
        split_tokens = std::max((uint32_t)kChunk, (split_tokens + kChunk - 1) / kChunk * kChunk);
        n_splits = std::max(1u, (max_len + split_tokens - 1) / split_tokens);
    }
    WEED_HIP_REQUIRE(n_splits <= kMaxSlots, "%s: internal split count %u too large", fn, n_splits);

    // workspace: rotated q (fp32), its fp16 hi / lo halves, per-head scale and sum, split partials
    const size_t n_q = (size_t)S * Hq * d;
    const size_t q_bytes = sizeof(float) * n_q;
    const size_t h_bytes = (sizeof(uint16_t) * n_q + 15) / 16 * 16;
    const size_t s_bytes = (sizeof(float) * (size_t)S * Hq + 15) / 16 * 16;
    const size_t part_bytes = sizeof(float) * (size_t)S * Hq * n_splits * (d + 2);
    const size_t off_bytes = (sizeof(uint32_t) * ((size_t)S + 1) + 15) / 16 * 16;
    // (the arrival counters of the kernel's own merge come first, at the same place whatever the shape, because they
    // have to be zero when a launch starts: they are cleared when the workspace is allocated and every launch leaves
    // them at zero; the static scratch starts as zeros)
    const size_t arrive_bytes = sizeof(uint32_t) * kMfmaMergeCounters;
    const size_t need = arrive_bytes + q_bytes + 2 * h_bytes + 2 * s_bytes + off_bytes + part_bytes;
    if (fixed_ws) {
        // the caller's workspace (the static scratch): nothing is allocated, larger shapes are refused
        WEED_HIP_REQUIRE(need <= fixed_ws_bytes,
                         "%s: this shape needs %zu bytes of workspace, the static scratch holds %zu (use "
                         "weed_hip_kv_decode_attn)", fn, need, fixed_ws_bytes);
    } else if (need > c->dec_ws_bytes) {
        WEED_HIP_CHECK(hipStreamSynchronize(stream()));
        (void)hipFree(c->dec_ws);
        c->dec_ws = nullptr;
        c->dec_ws_bytes = 0;
        if (hipMalloc((void **)&c->dec_ws, need) != hipSuccess) {
            return fail(WEED_HIP_ENOMEM, "%s: workspace allocation of %zu bytes failed", fn, need);
        }
        c->dec_ws_bytes = need;
        WEED_HIP_CHECK(hipMemsetAsync(c->dec_ws, 0, arrive_bytes, stream()));
    }
    uint8_t *ws0 = fixed_ws ? fixed_ws : reinterpret_cast<uint8_t *>(c->dec_ws);
    uint32_t *arrive = reinterpret_cast<uint32_t *>(ws0);
    uint8_t *wsp = ws0 + arrive_bytes;
    const bool timed = !fixed_ws; // the timing scopes create events, which the allocation-free entry point must not
    float *q_rot = reinterpret_cast<float *>(wsp);
    uint16_t *q_hi = reinterpret_cast<uint16_t *>(wsp + q_bytes);
    uint16_t *q_lo = reinterpret_cast<uint16_t *>(wsp + q_bytes + h_bytes);
    float *q_scale = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes);
    float *q_sum = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes + s_bytes);
    uint32_t *blk_off = reinterpret_cast<uint32_t *>(wsp + q_bytes + 2 * h_bytes + 2 * s_bytes);
    float *partials = reinterpret_cast<float *>(wsp + q_bytes + 2 * h_bytes + 2 * s_bytes + off_bytes);

    const int blocked = gqa_mapping == WEED_HIP_GQA_BLOCKED ? 1 : 0;
    Geom3 qg = { q_off, { q_stride[0], q_stride[1], q_stride[2] }, n_tokens, real_heads, q_tstride, blocked };
    Geom3 og = { o_off, { o_stride[0], o_stride[1], o_stride[2] }, n_tokens, real_heads, o_tstride, blocked };
    const uint32_t n_rows = S * Hq;
    // the multi-row kernels pay off with many (sequence, head) rows; their rotation loops step by 64
    const bool many_rows = n_rows >= 512 && d % 64 == 0;

    // Blocks per sequence when all sequences span the same number, else 0.
    uint32_t uniform_blocks = 0;
    // The workgroups of the matrix-core kernel merge their regions themselves (wg_regions regions each, else 0) when
    // every workgroup's share of the block list is a whole number of regions and no run straddles a region boundary:
    // equal sequences of nb blocks each, nb a multiple of one cycle of the age classes' runs, and a workgroup's blocks
    // a multiple of nb.  They then also rotate their regions' queries themselves, and the call is ONE kernel.
    uint32_t wg_regions = 0, region_wgs = 0;
    bool general_merge = false;
    bool fused_query = false;
    if (use_mfma && total_blocks) {
        uniform_blocks = partition_blocks(c->lens[0]);
        for (int32_t l : c->lens) {
            if (partition_blocks(l) != uniform_blocks || tune.always_search) {
                uniform_blocks = 0;
                break;
            }
        }
        const uint32_t gp = pass_heads <= 4 ? 4u : (pass_heads <= 8 ? 8u : 16u);
        const uint32_t nb = uniform_blocks, cycle = run_classes(runs) * runs.unit_blocks;
        const uint32_t wg_blocks = runs.waves * runs.unit_blocks;
        // (Groups that take several passes of the kernel -- more than sixteen heads per kv head, more than eight at
        // head_dims above 128 -- go the three-kernel way: every pass would rotate its queries and merge at the end of
        // its workgroups, where one kernel ahead and one behind serve all passes.  Measured, 64 heads on 2 kv heads
        // of 128: 16 sequences of 8192 tokens 63.4 against 59.5 us, one sequence 57.7 against 37.2, two of 30000
        // tokens 105 against 58; 96 heads on 2: 91 against 61.)
        const bool may_merge = mfma_decode_merges_whole_regions(gp, d, runs.waves) && passes == 1;
        // (above head_dim 128 in one round of workgroups only: 64 sequences of 300 or 2100 tokens on 32 kv heads of
        // 256 in two rounds took 69 and 224 us against 61 and 216 with three kernels, where one round is 13 us ahead)
        if (may_merge && nb != 0 && nb % cycle == 0 && wg_blocks % nb == 0 && !tune.separate_merge &&
            (d <= 128 || (total_blocks + wg_blocks - 1) / wg_blocks <= 256)) {
            wg_regions = wg_blocks / nb;
        } else if (may_merge && nb != 0 && nb % wg_blocks == 0 && nb / wg_blocks >= 2 &&
                   nb / wg_blocks <= std::min(n_splits, 64u) && (size_t)S * Hkv <= kMfmaMergeCounters &&
                   !tune.separate_merge) {
            // small batches of long sequences: every region is a whole number of workgroups' shares
            region_wgs = nb / wg_blocks;
        }
        // Most regions that the blocks of one workgroup lie in (exact: the host knows the cached lengths).
        uint32_t wg_most_regions = wg_regions;
        bool every_sequence_has_tokens = true;
        if (wg_regions == 0) {
            // (a buffer of the cache object, so that a decode call allocates nothing on the host either)
            std::vector<uint64_t> &region_end = c->plan_region_end; // blocks up to and including region r
            region_end.clear();
            region_end.reserve((size_t)S * Hkv);
            uint64_t run = 0;
            for (int32_t l : c->lens) {
                const uint32_t b = partition_blocks(l);
                every_sequence_has_tokens = every_sequence_has_tokens && b != 0;
                for (uint32_t h = 0; h < Hkv; ++h) {
                    run += b;
                    region_end.push_back(run);
                }
            }
            size_t r = 0;
            for (uint64_t first = 0; first < total_blocks; first += wg_blocks) {
                const uint64_t last = std::min<uint64_t>(first + wg_blocks, total_blocks) - 1;
                while (region_end[r] <= first) {
                    ++r;
                }
                size_t r1 = r;
                while (region_end[r1] <= last) {
                    ++r1;
                }
                wg_most_regions = std::max(wg_most_regions, (uint32_t)(r1 - r + 1));
            }
        }
        // Anything else that the instance can merge: one slot per (run, region) in memory, an arrival counter per
        // region (ragged batches: up to 63 sequences, whose block offsets a wavefront keeps in one register).
        // A workgroup merges the regions that it completes one after the other, at its end, about 2 us each, where
        // the separate kernel merges all regions at once for 10 to 12 us: measured on batches that are half long and
        // half short sequences, the workgroups win up to 6 regions per workgroup, tie at 7 and lose from 8 on (5 to
        // 30 us at 8 to 17).  Nor do they where they could not rotate their queries as well (a kernel ahead and the
        // merges at the end: 3 to 200 sequences of 100 tokens with groups of eight, 27 us against 22 to 25).
        if (wg_regions == 0 && region_wgs == 0 && passes == 1 && mfma_decode_merges_in_general(gp, d, runs.waves) && every_sequence_has_tokens &&
            (nb != 0 || (S <= 63 && !tune.always_search)) && n_splits <= (d % 64 == 0 ? 64u : 24u) &&
            wg_most_regions <= kMostRegionsMergedByWorkgroup &&
            wg_most_regions * pass_heads <= std::min(kMostRowsMergedByWorkgroup, mfma_query_rows(d)) &&
            (size_t)S * Hkv <= kMfmaMergeCounters && !tune.separate_merge) {
            general_merge = true;
        }
        // A workgroup rotates the queries of the regions its blocks lie in itself when they are few enough for its
        // LDS (equal sequences, or the ragged batches above); nothing then runs ahead of the matrix-core kernel.
        fused_query = passes == 1 && (wg_regions != 0 || region_wgs != 0 || mfma_decode_merges_in_general(gp, d, runs.waves)) &&
                      (nb != 0 || general_merge) &&
                      wg_most_regions * pass_heads <= mfma_query_rows(d) && !tune.separate_query;
    }
    // Workgroups that merge whole regions or whole shares of a region: neighbouring runs take their blocks in turns
    // (see RunGeom), as many cycles' runs together as divide both a workgroup's share and a region, so that no group
    // crosses a region boundary.  (Measured on 1 to 256 sequences of 1024 to 16384 tokens: 1 to 6 % faster with runs
    // of 4 to 32 blocks, nothing with shorter ones, 1 to 1.5 % slower with runs of 64.  Not at head_dim 256, where
    // a block is twice the bytes: 64 sequences of 8192 tokens took 267 us with turns and 232 us without.)
    if ((wg_regions != 0 || region_wgs != 0) && runs.unit_blocks >= kFewestBlocksOfRunsInTurns &&
        runs.unit_blocks <= kMostBlocksOfRunsInTurns && !tune.contiguous_runs && d <= 128) {
        const uint32_t cycle = run_classes(runs) * runs.unit_blocks;
        uint32_t cycles = runs.waves / run_classes(runs);
        while (uniform_blocks % (cycles * cycle) != 0) {
            cycles /= 2; // (4, 2, 1: a region is whole cycles)
        }
        runs.group_cycles = cycles;
    }
    const bool fused_merge = wg_regions != 0 || region_wgs != 0 || general_merge;
    if (tune.print_plan) {
        std::fprintf(stderr,
                     "%s: S %u Hkv %u G %u d %u bits %u/%u  matrix cores %d  passes %u  blocks %u  run %u (skew %u, in turns %u) "
                     "x %u wavefronts  whole regions per workgroup %u  workgroups per region %u  general merge %d  "
                     "queries in the kernel %d  slots %u\n",
                     fn, S, Hkv, G, d, c->k.w, c->v.w, (int)use_mfma, passes, total_blocks, runs.unit_blocks, runs.skew,
                     runs.group_cycles, runs.waves, wg_regions, region_wgs, (int)general_merge, (int)fused_query, n_splits);
    }
    // (the kernels that take one (sequence, head) row per workgroup have the sequence on a 16-bit grid dimension)
    // (prep_q_kernel puts one more row on that dimension when it also builds the block offsets)
    WEED_HIP_REQUIRE(S + ((use_mfma && !fused_query && !many_rows) ? 1u : 0u) <= 65535u || (use_mfma && many_rows && n_splits <= 64),
                     "%s: %u sequences in one call are served only for head_dims that are multiples of 64 with "
                     "matrix-core instances; split the batch", fn, S);
    if (fused_query) {
        // (nothing runs ahead of the matrix-core kernel)
    } else if (many_rows) {
        prep_q_rows_kernel<<<(n_rows + kRowsPerWg - 1) / kRowsPerWg + (use_mfma ? 1 : 0), 256, 0, stream()>>>(
            q_dev, qg, Hq, d, d_real, n_rows, c->k.rot_t, rot_q ? 1 : 0, q_rot, q_hi, q_lo, q_scale, q_sum, c->lens_dev, S,
            use_mfma ? blk_off : nullptr);
    } else {
        prep_q_kernel<<<dim3(Hq, S + (use_mfma ? 1 : 0)), 256, 0, stream()>>>(q_dev, qg, Hq, d, d_real, c->k.rot_t, rot_q ? 1 : 0, q_rot, q_hi, q_lo,
                                                         q_scale, q_sum, c->lens_dev, S, use_mfma ? blk_off : nullptr);
    }
    WEED_HIP_LAUNCH_CHECK();

    if (use_mfma) {
        MfmaParams mp;
        const SideParams ks = side_params(c, 0), vs = side_params(c, 1);
        mp.k = MfmaSide{ ks.fields, ks.alpha, ks.region_bytes, ks.alpha_max, ks.alpha_const, ks.beta, ks.w };
        mp.v = MfmaSide{ vs.fields, vs.alpha, vs.region_bytes, vs.alpha_max, vs.alpha_const, vs.beta, vs.w };
        mp.table_image = c->table_image;
        mp.lens = lens_dev ? lens_dev : c->lens_dev;
        mp.padded = c->padded_tokens;
        mp.Hq = Hq;
        mp.Hkv = Hkv;
        mp.G = G;
        mp.blocked = gqa_mapping == WEED_HIP_GQA_BLOCKED;
        mp.q_tokens = n_tokens;
        mp.real_group = real_heads / Hkv;
        mp.q_hi = q_hi;
        mp.q_lo = q_lo;
        mp.q_scale = q_scale;
        mp.q_sum = q_sum;
        mp.partials = partials;
        mp.blk_off = blk_off;
        mp.n_seq = S;
        mp.total_blocks = total_blocks;
        mp.uniform_blocks = uniform_blocks;
        mp.merge = MfmaMerge{ wg_regions, region_wgs, general_merge ? 1u : 0u, arrive, d_real, out_dev, og, c->v.rot,
                              unrot ? 1 : 0 };
        mp.cached_lens = c->lens_dev;
        mp.query = MfmaQuery{ fused_query ? q_dev : nullptr, qg, c->k.rot_t, rot_q ? 1 : 0 };
        mp.runs = runs;
        mp.max_slots = n_splits;
        mp.group_total = G;
        mp.tile_rows = pass_heads;
        ProfileScope prof("kv_decode_attn", timed);
        mp.grid_passes = 0;
        if (passes > 1 && total_blocks && !fused_merge && !fused_query) {
            // every pass in ONE launch: the passes' workgroups that read the same blocks run next to each other on one
            // XCD, so the cache is fetched from memory once instead of once per pass
            mp.grid_passes = passes;
            mp.head_first = 0;
            mp.G = pass_heads;
            WEED_HIP_TRY(launch_mfma_decode(mp, d, stream()));
        } else {
            for (uint32_t first = 0; total_blocks && first < G; first += pass_heads) {
                mp.head_first = first;
                mp.G = std::min(pass_heads, G - first);
                WEED_HIP_TRY(launch_mfma_decode(mp, d, stream()));
            }
        }
    } else {
        DecodeParams p;
        p.k = side_params(c, 0);
        p.v = side_params(c, 1);
        p.lens = lens_dev ? lens_dev : c->lens_dev;
        p.padded = c->padded_tokens;
        p.d = d;
        p.d_real = d_real;
        p.Hq = Hq;
        p.Hkv = Hkv;
        p.G = G;
        p.blocked = gqa_mapping == WEED_HIP_GQA_BLOCKED;
        p.q_rot = q_rot;
        p.partials = partials;
        p.n_splits = n_splits;
        p.split_tokens = split_tokens;
        ProfileScope prof("kv_decode_attn", timed);
        decode_generic_kernel<<<dim3(n_splits, Hkv, S), kThreads, 0, stream()>>>(p);
        WEED_HIP_LAUNCH_CHECK();
    }
    if (!fused_merge) {
        ProfileScope prof("kv_decode_combine", timed);
        const SlotGeom sg = { use_mfma ? blk_off : nullptr, Hkv, G, runs,
                              gqa_mapping == WEED_HIP_GQA_BLOCKED ? 1 : 0, uniform_blocks };
        if (many_rows && n_splits <= 64) {
            combine_rows_kernel<<<(n_rows + kRowsPerWg - 1) / kRowsPerWg, 256, 0, stream()>>>(
                partials, Hq, d, d_real, n_splits, n_rows, sg, c->v.rot, unrot ? 1 : 0, use_mfma ? 1 : 0, out_dev, og);
        } else {
            combine_kernel<<<dim3(Hq, S), n_splits > 16 ? 1024 : 256, 0, stream()>>>(
                partials, Hq, d, d_real, n_splits, sg, c->v.rot, unrot ? 1 : 0, use_mfma ? 1 : 0, out_dev, og);
        }
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

extern "C" int weed_hip_kv_decode_tuning(int32_t wavefronts, int32_t skew_percent, int32_t always_search)
{
    DecodeTuning &t = decode_tuning();
    t.wavefronts = std::max(0, wavefronts);
    t.skew_percent = skew_percent;
    t.always_search = (always_search & 1) != 0;
    t.separate_merge = (always_search & 2) != 0;
    t.separate_query = (always_search & 4) != 0;
    t.contiguous_runs = (always_search & 8) != 0;
    return WEED_HIP_OK;
}

extern "C" int weed_hip_kv_decode_attn_noalloc(weed_hip_kv_cache *c, int32_t n_q_heads, int32_t gqa_mapping,
                                               const float *q_dev, uint32_t q_off, const uint32_t q_stride[3],
                                               float *out_dev, uint32_t o_off, const uint32_t o_stride[3],
                                               uint32_t flags)
{
    const char *fn = "weed_hip_kv_decode_attn_noalloc";
    const int dev = current_device();
    WEED_HIP_REQUIRE(dev >= 0 && dev < kMaxDevices && g_scratch_dev[dev],
                     "%s: weed_hip_init has not run on the current device", fn);
    return decode_impl(fn, c, n_q_heads, gqa_mapping, q_dev, q_off, q_stride, out_dev, o_off, o_stride, flags, nullptr,
                       1, 0, 0, static_cast<uint8_t *>(g_scratch_dev[dev]), kStaticScratchBytes);
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

extern "C" int weed_hip_kv_decode_attn_chunk(weed_hip_kv_cache *c, const int32_t *lens_dev, int32_t n_tokens,
                                             int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev, uint32_t q_off,
                                             const uint32_t q_stride[4], float *out_dev, uint32_t o_off,
                                             const uint32_t o_stride[4], uint32_t flags)
{
    const char *fn = "weed_hip_kv_decode_attn_chunk";
    WEED_HIP_REQUIRE(q_stride && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(n_tokens >= 1 && n_tokens <= 64, "%s: %d positions outside [1, 64]", fn, n_tokens);
    if (c && !lens_dev) {
        for (int32_t l : c->lens) {
            WEED_HIP_REQUIRE(l >= n_tokens, "%s: a sequence holds %d tokens, fewer than the chunk's %d", fn, l, n_tokens);
        }
    }
    const uint32_t qs3[3] = { q_stride[0], q_stride[2], q_stride[3] }, os3[3] = { o_stride[0], o_stride[2], o_stride[3] };
    return decode_impl(fn, c, n_q_heads, gqa_mapping, q_dev, q_off, qs3, out_dev, o_off, os3, flags, lens_dev,
                       (uint32_t)n_tokens, q_stride[1], o_stride[1]);
}
