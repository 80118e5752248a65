// Strided fp32 softmax and axis reductions (the standalone ops that feed attention in the reference:
// src/ops/softmax.cpp:276-287, src/ops/reduce.cpp:342-386).
//
// Rows (all index combinations of the non-reduced dimensions) are enumerated with dimension 0 fastest, which is the
// contiguous direction of Weed's column-major tensors; a workgroup takes RT neighbouring rows and spreads the
// remaining threads along the reduced axis, so that loads are coalesced whether the axis is the contiguous
// dimension (RT = 1, float4 accesses where alignment allows) or a strided one (RT = 32 or 16).  Softmax keeps a
// running (max, sum) per thread, so the data is read twice, or once when a contiguous row fits the registers.
#include "common.h"

#include <algorithm>
#include <cmath>

using namespace weedhip;

namespace {

constexpr int kMaxRank = 8;

struct AxisGeom {
    uint32_t rank;
    uint32_t axis;
    uint32_t shape[kMaxRank];
    uint32_t a_stride[kMaxRank];
    uint32_t o_stride[kMaxRank];
    uint32_t a_off, o_off;
    uint32_t rows;
    uint32_t axis_len;
};

__device__ __forceinline__ void row_bases(const AxisGeom &g, uint32_t row, uint64_t &a_base, uint64_t &o_base)
{
    a_base = g.a_off;
    o_base = g.o_off;
    uint32_t tmp = row;
    for (uint32_t dd = 0; dd < g.rank; ++dd) {
        if (dd == g.axis) {
            continue;
        }
        const uint32_t dim = g.shape[dd];
        const uint32_t i = tmp % dim;
        tmp /= dim;
        a_base += (uint64_t)i * g.a_stride[dd];
        o_base += (uint64_t)i * g.o_stride[dd];
    }
}

// op: 0 sum, 1 max, 2 min
template <int OP> __device__ __forceinline__ float combine(float a, float b)
{
    if (OP == 0) {
        return a + b;
    }
    if (OP == 1) {
        return b > a ? b : a;
    }
    return b < a ? b : a;
}

template <int OP> __device__ __forceinline__ float identity()
{
    if (OP == 0) {
        return 0.0f;
    }
    return OP == 1 ? -INFINITY : INFINITY;
}

// Reduce `v` over the NY threads that share threadIdx.x % RT; the result is valid in every thread.
template <int OP, int RT, int THREADS> __device__ __forceinline__ float block_reduce(float v, float *red)
{
    constexpr int NY = THREADS / RT;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    red[ty * RT + tx] = v;
    __syncthreads();
    for (int s = NY / 2; s > 0; s >>= 1) {
        if ((int)ty < s) {
            red[ty * RT + tx] = combine<OP>(red[ty * RT + tx], red[(ty + s) * RT + tx]);
        }
        __syncthreads();
    }
    const float r = red[tx];
    __syncthreads();
    return r;
}

// Running (max, sum of exp(x - max)) of a softmax row: one exponential per element, one pass over the data.
// -inf elements (masked positions) add nothing, also while the running maximum is still -inf.
__device__ __forceinline__ void softmax_accumulate(float &m, float &s, float x)
{
    if (x > m) {
        s = s * expf(m - x) + 1.0f;
        m = x;
    } else if (x > -INFINITY) {
        s += expf(x - m);
    }
}

// The same for N elements at once: their maximum first, then one exponential per element (and one more where the
// running maximum rises), instead of a branch with an exponential on either side per element.
template <int N> __device__ __forceinline__ void softmax_accumulate(float &m, float &s, const float (&x)[N])
{
    float top = x[0];
#pragma unroll
    for (int u = 1; u < N; ++u) {
        top = fmaxf(top, x[u]);
    }
    if (top > m) {
        s *= expf(m - top); // (m = -inf: s is 0 and stays 0)
        m = top;
    }
    if (m > -INFINITY) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            s += expf(x[u] - m);
        }
    }
}

// Merge the per-thread (m, s) pairs of the threads that share a row; returns the row's (max, sum) in every thread.
template <int RT, int THREADS> __device__ __forceinline__ void softmax_merge(float &m, float &s, float *red)
{
    const float row_max = block_reduce<1, RT, THREADS>(m, red);
    const float scaled = (m > -INFINITY) ? s * expf(m - row_max) : 0.0f;
    s = block_reduce<0, RT, THREADS>(scaled, red);
    m = row_max;
}

constexpr int kAxisUnroll = 8; // independent loads in flight per thread

// Softmax along any axis.  First pass: running (max, sum) with kAxisUnroll loads in flight per thread; second pass:
// exp(x - max) / sum.  Two reads and one write per element.
template <int RT, int THREADS> __global__ void __launch_bounds__(THREADS) softmax_kernel(const float *__restrict__ a,
                                                                                        float *__restrict__ out,
                                                                                        AxisGeom g)
{
    __shared__ float red[THREADS];
    constexpr int NY = THREADS / RT;
    constexpr int U = kAxisUnroll;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t a_base = 0, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis], os = g.o_stride[g.axis];
    const uint32_t len = valid ? g.axis_len : 0U;
    const float *ap = a + a_base;
    float *op = out + o_base;
    float m = -INFINITY, s = 0.0f;
    for (uint32_t j0 = ty; j0 < len; j0 += NY * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * NY;
            x[u] = j < len ? ap[(uint64_t)j * as] : -INFINITY;
        }
        softmax_accumulate(m, s, x);
    }
    softmax_merge<RT, THREADS>(m, s, red);
    const float inv = 1.0f / s; // (s >= 1 wherever the row has a finite element)
    for (uint32_t j0 = ty; j0 < len; j0 += NY * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * NY;
            x[u] = j < len ? ap[(uint64_t)j * as] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * NY;
            if (j < len) {
                op[(uint64_t)j * os] = expf(x[u] - m) * inv;
            }
        }
    }
}

// Softmax along a strided axis of at most kStridedCached * (THREADS / RT) elements: RT neighbouring rows per
// workgroup, every thread keeps its share of a row in registers (all loads in flight at once), so the data is read
// once and each element costs one exponential.
constexpr int kStridedCached = 64;
constexpr int kStridedThreads = 512;
constexpr int kStridedThreadsLong = 1024; // (few rows of up to 8192 or 16384 elements: 8 or 4 rows per workgroup)

// (SPREAD, for tiles narrower than a 128-byte line: the grid is eight equal shares and workgroup b takes tile b / 8 of
// share b % 8, so that the workgroups which complete each other's lines run at the same time behind the same L2.)
template <int RT, int THREADS = 512, bool SPREAD = false, int CACHED = kStridedCached>
__global__ void __launch_bounds__(THREADS) softmax_strided_cached_kernel(const float *__restrict__ a,
                                                                      float *__restrict__ out, AxisGeom g)
{
    __shared__ float red[THREADS];
    constexpr int NY = THREADS / RT;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t tile = SPREAD ? (blockIdx.x % 8U) * (gridDim.x / 8U) + blockIdx.x / 8U : blockIdx.x;
    const uint32_t row = tile * RT + tx;
    const bool valid = row < g.rows;
    uint64_t a_base = 0, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis], os = g.o_stride[g.axis];
    const uint32_t len = valid ? g.axis_len : 0U;
    // rows past the end read row 0's first element (any readable address) and are discarded
    const float *ap = a + (valid ? a_base : (uint64_t)g.a_off);
    float *op = out + o_base;
    float x[CACHED];
    // unconditional loads of clamped positions (the host checks that the row's span fits 32 bits), then the select
    const uint32_t last = len ? len - 1U : 0U;
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const uint32_t j = ty + c * NY;
        x[c] = ap[min(j, last) * as];
    }
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const uint32_t j = ty + c * NY;
        x[c] = j < len ? x[c] : -INFINITY;
    }
    float m = -INFINITY, s = 0.0f;
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        m = fmaxf(m, x[c]);
    }
    m = block_reduce<1, RT, THREADS>(m, red);
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        x[c] = expf(x[c] - m);
        s += x[c];
    }
    s = block_reduce<0, RT, THREADS>(s, red);
    const float inv = 1.0f / s;
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const uint32_t j = ty + c * NY;
        if (j < len) {
            op[(uint64_t)j * os] = x[c] * inv;
        }
    }
}

// ---- Few rows, long strided axis (the scores of a decode step as the reference lays them out: [B * heads] rows whose
//      elements are B * heads apart): 64 rows per workgroup would be a handful of workgroups, so the axis is cut into
//      bands.  Workgroup (row group x, band y) = 64 rows x 4 lanes of the band's positions; three small launches:
//      every band's (max, sum) per row, their merge per row, exp(x - max) / sum per band.  The partial results live
//      in a static array (the library serves one stream per device: calls do not overlap).
constexpr uint32_t kBandRows = 4096, kMostBands = 128, kBandPartials = 65536; // (about 512 workgroups: bands x rows <= 32768 + a row group)
__device__ float2 g_band_part[kBandPartials]; // [band][pitch]
__device__ float2 g_band_final[kBandRows];

struct BandGeom {
    uint32_t bands, band_len, pitch; // pitch: the rows, rounded up to whole row groups
};

template <int OP> // 0 sum, 1 max, 2 min, 3 softmax's (max, sum)
__global__ void __launch_bounds__(256) band_partial_kernel(const float *__restrict__ a, AxisGeom g, BandGeom bg)
{
    __shared__ float2 red[256];
    constexpr int U = kAxisUnroll;
    const uint32_t rr = threadIdx.x % 64U, jj = threadIdx.x / 64U;
    const uint32_t row = blockIdx.x * 64U + rr;
    const bool valid = row < g.rows;
    uint64_t a_base = g.a_off, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis];
    const uint32_t j0 = blockIdx.y * bg.band_len, j1 = valid ? min(j0 + bg.band_len, g.axis_len) : 0U;
    const float *ap = a + a_base;
    float m = OP == 3 ? -INFINITY : identity<OP == 3 ? 1 : OP>(), s = 0.0f;
    for (uint32_t j = j0 + jj; j < j1; j += 4U * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t k = j + 4U * u;
            x[u] = k < j1 ? ap[(uint64_t)k * as] : (OP == 3 ? -INFINITY : identity<OP == 3 ? 1 : OP>());
        }
        if constexpr (OP == 3) {
            softmax_accumulate(m, s, x);
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                m = combine<OP == 3 ? 1 : OP>(m, x[u]);
            }
        }
    }
    red[threadIdx.x] = make_float2(m, s);
    __syncthreads();
    if (jj == 0U && valid) {
#pragma unroll
        for (uint32_t k = 1; k < 4U; ++k) {
            const float2 o = red[64U * k + rr];
            if constexpr (OP == 3) {
                const float top = fmaxf(m, o.x);
                s = (m > -INFINITY ? s * expf(m - top) : 0.0f) + (o.x > -INFINITY ? o.y * expf(o.x - top) : 0.0f);
                m = top;
            } else {
                m = combine<OP == 3 ? 1 : OP>(m, o.x);
            }
        }
        g_band_part[blockIdx.y * bg.pitch + row] = make_float2(m, s);
    }
}

// 64 rows per workgroup, four lanes per row that take every fourth band (all of a lane's partial results are requested
// before the first is used: one thread per row walking 128 bands one after the other took 35 us), then the four lanes'
// results in lane order
template <int OP>
__global__ void __launch_bounds__(256) band_merge_kernel(float *__restrict__ out, AxisGeom g, BandGeom bg)
{
    __shared__ float2 red[256];
    const uint32_t rr = threadIdx.x % 64U, jj = threadIdx.x / 64U;
    const uint32_t row = blockIdx.x * 64U + rr;
    const bool valid = row < g.rows;
    auto merge = [](float2 &acc, const float2 o) {
        if constexpr (OP == 3) {
            const float top = fmaxf(acc.x, o.x);
            acc.y = (acc.x > -INFINITY ? acc.y * expf(acc.x - top) : 0.0f) + (o.x > -INFINITY ? o.y * expf(o.x - top) : 0.0f);
            acc.x = top;
        } else {
            acc.x = combine<OP == 3 ? 1 : OP>(acc.x, o.x);
        }
    };
    float2 acc = make_float2(OP == 3 ? -INFINITY : identity<OP == 3 ? 1 : OP>(), 0.0f);
    constexpr uint32_t kMine = kMostBands / 4U; // bands jj, jj + 4, ...
    float2 mine[kMine];
#pragma unroll
    for (uint32_t k = 0; k < kMine; ++k) {
        const uint32_t b = jj + 4U * k;
        mine[k] = (valid && b < bg.bands) ? g_band_part[b * bg.pitch + row] : acc;
    }
#pragma unroll
    for (uint32_t k = 0; k < kMine; ++k) {
        if (jj + 4U * k < bg.bands) {
            merge(acc, mine[k]);
        }
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    if (jj != 0U || !valid) {
        return;
    }
#pragma unroll
    for (uint32_t k = 1; k < 4U; ++k) {
        merge(acc, red[64U * k + rr]);
    }
    if constexpr (OP == 3) {
        g_band_final[row] = make_float2(acc.x, 1.0f / acc.y);
    } else {
        uint64_t a_base, o_base;
        row_bases(g, row, a_base, o_base);
        out[o_base] = acc.x;
    }
}

__global__ void __launch_bounds__(256) band_softmax_finish_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                                  AxisGeom g, BandGeom bg)
{
    constexpr int U = kAxisUnroll;
    const uint32_t rr = threadIdx.x % 64U, jj = threadIdx.x / 64U;
    const uint32_t row = blockIdx.x * 64U + rr;
    if (row >= g.rows) {
        return;
    }
    uint64_t a_base, o_base;
    row_bases(g, row, a_base, o_base);
    const uint32_t as = g.a_stride[g.axis], os = g.o_stride[g.axis];
    const uint32_t j0 = blockIdx.y * bg.band_len, j1 = min(j0 + bg.band_len, g.axis_len);
    const float2 ms = g_band_final[row];
    const float *ap = a + a_base;
    float *op = out + o_base;
    for (uint32_t j = j0 + jj; j < j1; j += 4U * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t k = j + 4U * u;
            x[u] = k < j1 ? ap[(uint64_t)k * as] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t k = j + 4U * u;
            if (k < j1) {
                op[(uint64_t)k * os] = expf(x[u] - ms.x) * ms.y;
            }
        }
    }
}

// Softmax along a contiguous, 16-byte aligned axis: one workgroup per row, float4 accesses, and the first
// CACHED * 4 * THREADS elements of the row stay in registers between the passes.  Rows up to that length (FITS) are
// read once and cost one exponential per element; longer rows keep a running (max, sum) and are read twice.
template <int CACHED, int THREADS, bool FITS>
__global__ void __launch_bounds__(THREADS) softmax_contiguous_kernel(const float *__restrict__ a,
                                                                    float *__restrict__ out, AxisGeom g)
{
    __shared__ float red[THREADS];
    uint64_t a_base, o_base;
    row_bases(g, blockIdx.x, a_base, o_base);
    const float4 *ap = reinterpret_cast<const float4 *>(a + a_base);
    float4 *op = reinterpret_cast<float4 *>(out + o_base);
    const uint32_t n4 = g.axis_len / 4U;
    float4 cache[CACHED];
    float m = -INFINITY, s = 0.0f;
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const uint32_t idx = threadIdx.x + c * THREADS;
        cache[c] = idx < n4 ? ap[idx] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    if (FITS) {
        // the whole row is in registers: maximum, then ONE exponential per element (kept), then the division -- the
        // reference's three passes (src/ops/softmax.cpp:276-287) without touching memory again
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            m = fmaxf(fmaxf(m, fmaxf(cache[c].x, cache[c].y)), fmaxf(cache[c].z, cache[c].w));
        }
        m = block_reduce<1, 1, THREADS>(m, red);
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            cache[c] = make_float4(expf(cache[c].x - m), expf(cache[c].y - m), expf(cache[c].z - m), expf(cache[c].w - m));
            s += (cache[c].x + cache[c].y) + (cache[c].z + cache[c].w);
        }
        s = block_reduce<0, 1, THREADS>(s, red);
        const float inv = 1.0f / s;
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t idx = threadIdx.x + c * THREADS;
            if (idx < n4) {
                op[idx] = make_float4(cache[c].x * inv, cache[c].y * inv, cache[c].z * inv, cache[c].w * inv);
            }
        }
        return;
    }
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const float v4[4] = { cache[c].x, cache[c].y, cache[c].z, cache[c].w };
        softmax_accumulate(m, s, v4);
    }
    for (uint32_t idx = threadIdx.x + CACHED * THREADS; idx < n4; idx += THREADS) {
        const float4 v = ap[idx];
        const float v4[4] = { v.x, v.y, v.z, v.w };
        softmax_accumulate(m, s, v4);
    }
    softmax_merge<1, THREADS>(m, s, red);
    const float inv = 1.0f / s;
#pragma unroll
    for (int c = 0; c < CACHED; ++c) {
        const uint32_t idx = threadIdx.x + c * THREADS;
        if (idx < n4) {
            const float4 v = cache[c];
            op[idx] = make_float4(expf(v.x - m) * inv, expf(v.y - m) * inv, expf(v.z - m) * inv, expf(v.w - m) * inv);
        }
    }
    for (uint32_t idx = threadIdx.x + CACHED * THREADS; idx < n4; idx += THREADS) {
        const float4 v = ap[idx];
        op[idx] = make_float4(expf(v.x - m) * inv, expf(v.y - m) * inv, expf(v.z - m) * inv, expf(v.w - m) * inv);
    }
}

template <int OP> __device__ __forceinline__ float wave_reduce(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v = combine<OP>(v, __shfl_xor(v, off, 64));
    }
    return v;
}

// Short contiguous rows (a causal prefill's scores: [B * heads * T] rows of at most a few thousand key positions):
// one WAVEFRONT per row, four rows per workgroup, so no lane idles on a 64..2048-element row and nothing goes
// through LDS.  V = 4: float4 accesses (every row 16-byte aligned, length a multiple of 4), V = 1: scalar.  The first
// CACHED * 64 * V elements of a row stay in registers between the two passes.
template <int V, int CACHED, bool FITS>
__global__ void __launch_bounds__(256) softmax_wave_rows_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                                AxisGeom g)
{
    const uint32_t lane = threadIdx.x & 63U;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nvec = g.axis_len / V;
    for (uint32_t row = blockIdx.x * 4U + wave; row < g.rows; row += gridDim.x * 4U) {
        uint64_t a_base, o_base;
        row_bases(g, row, a_base, o_base);
        const float *ap = a + a_base;
        float *op = out + o_base;
        float cache[CACHED][V];
        float m = -INFINITY, s = 0.0f;
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t idx = lane + 64U * c;
            if (V == 4) {
                const float4 v = idx < nvec ? reinterpret_cast<const float4 *>(ap)[idx]
                                            : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
                cache[c][0] = v.x;
                cache[c][V > 1 ? 1 : 0] = v.y;
                cache[c][V > 2 ? 2 : 0] = v.z;
                cache[c][V > 3 ? 3 : 0] = v.w;
            } else {
                cache[c][0] = idx < nvec ? ap[idx] : -INFINITY;
            }
        }
        if (FITS) {
            // the row is in registers: maximum, one exponential per element (kept), division
#pragma unroll
            for (int c = 0; c < CACHED; ++c) {
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    m = fmaxf(m, cache[c][e]);
                }
            }
            m = wave_reduce<1>(m);
#pragma unroll
            for (int c = 0; c < CACHED; ++c) {
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    cache[c][e] = expf(cache[c][e] - m);
                    s += cache[c][e];
                }
            }
            s = wave_reduce<0>(s);
            const float inv = 1.0f / s;
#pragma unroll
            for (int c = 0; c < CACHED; ++c) {
                const uint32_t idx = lane + 64U * c;
                if (idx < nvec) {
                    if (V == 4) {
                        reinterpret_cast<float4 *>(op)[idx] = make_float4(cache[c][0] * inv, cache[c][V > 1 ? 1 : 0] * inv,
                                                                          cache[c][V > 2 ? 2 : 0] * inv,
                                                                          cache[c][V > 3 ? 3 : 0] * inv);
                    } else {
                        op[idx] = cache[c][0] * inv;
                    }
                }
            }
            continue;
        }
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            softmax_accumulate(m, s, cache[c]);
        }
        for (uint32_t idx = lane + 64U * CACHED; idx < nvec; idx += 64U) {
            float v[V];
#pragma unroll
            for (int e = 0; e < V; ++e) {
                v[e] = ap[(uint64_t)idx * V + e];
            }
            softmax_accumulate(m, s, v);
        }
        const float row_max = wave_reduce<1>(m);
        const float total = wave_reduce<0>((m > -INFINITY) ? s * expf(m - row_max) : 0.0f);
        const float inv = 1.0f / total;
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t idx = lane + 64U * c;
            if (idx < nvec) {
                if (V == 4) {
                    reinterpret_cast<float4 *>(op)[idx] =
                        make_float4(expf(cache[c][0] - row_max) * inv, expf(cache[c][V > 1 ? 1 : 0] - row_max) * inv,
                                    expf(cache[c][V > 2 ? 2 : 0] - row_max) * inv,
                                    expf(cache[c][V > 3 ? 3 : 0] - row_max) * inv);
                } else {
                    op[idx] = expf(cache[c][0] - row_max) * inv;
                }
            }
        }
        for (uint32_t idx = lane + 64U * CACHED; idx < nvec; idx += 64U) {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                op[(uint64_t)idx * V + e] = expf(ap[(uint64_t)idx * V + e] - row_max) * inv;
            }
        }
    }
}

// Rows of up to CACHED * LPR * V elements, LPR lanes per row (a power of two below 64): 64 / LPR rows per wavefront, so
// that a wavefront's loads are whole contiguous stretches of memory also where a row is a few dozen elements (a
// wavefront per row would leave most lanes idle there: 262144 rows of 16 took 209 us, 65536 rows of 128 54 us).
template <int V, int CACHED, int LPR>
__global__ void __launch_bounds__(256) softmax_short_rows_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                                 AxisGeom g)
{
    constexpr uint32_t RPW = 64U / LPR; // rows per wavefront
    const uint32_t lane = threadIdx.x & 63U, sub = lane % LPR;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t nvec = g.axis_len / V;
    // (every lane of a wavefront makes the same number of trips, so that the exchanges between lanes are whole)
    for (uint32_t row0 = (blockIdx.x * 4U + wave) * RPW; row0 < g.rows; row0 += gridDim.x * 4U * RPW) {
        const uint32_t row = row0 + lane / LPR;
        const bool valid = row < g.rows;
        uint64_t a_base = g.a_off, o_base = g.o_off;
        if (valid) {
            row_bases(g, row, a_base, o_base);
        }
        const float *ap = a + a_base;
        float *op = out + o_base;
        float cache[CACHED][V];
        float m = -INFINITY, s = 0.0f;
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t idx = sub + LPR * c;
            const bool ok = valid && idx < nvec;
            if (V == 4) {
                const float4 v = ok ? reinterpret_cast<const float4 *>(ap)[idx]
                                    : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
                cache[c][0] = v.x;
                cache[c][V > 1 ? 1 : 0] = v.y;
                cache[c][V > 2 ? 2 : 0] = v.z;
                cache[c][V > 3 ? 3 : 0] = v.w;
            } else {
                cache[c][0] = ok ? ap[idx] : -INFINITY;
            }
#pragma unroll
            for (int e = 0; e < V; ++e) {
                m = fmaxf(m, cache[c][e]);
            }
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) {
            m = fmaxf(m, __shfl_xor(m, off, 64));
        }
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                cache[c][e] = expf(cache[c][e] - m);
                s += cache[c][e];
            }
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) {
            s += __shfl_xor(s, off, 64);
        }
        const float inv = 1.0f / s;
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t idx = sub + LPR * c;
            if (valid && idx < nvec) {
                if (V == 4) {
                    reinterpret_cast<float4 *>(op)[idx] = make_float4(cache[c][0] * inv, cache[c][V > 1 ? 1 : 0] * inv,
                                                                      cache[c][V > 2 ? 2 : 0] * inv,
                                                                      cache[c][V > 3 ? 3 : 0] * inv);
                } else {
                    op[idx] = cache[c][0] * inv;
                }
            }
        }
    }
}

template <int OP, int V>
__global__ void __launch_bounds__(256) reduce_wave_rows_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                               AxisGeom g)
{
    const uint32_t lane = threadIdx.x & 63U;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nvec = g.axis_len / V;
    for (uint32_t row = blockIdx.x * 4U + wave; row < g.rows; row += gridDim.x * 4U) {
        uint64_t a_base, o_base;
        row_bases(g, row, a_base, o_base);
        const float *ap = a + a_base;
        float v = identity<OP>();
        for (uint32_t idx = lane; idx < nvec; idx += 64U) {
            if (V == 4) {
                const float4 x = reinterpret_cast<const float4 *>(ap)[idx];
                v = combine<OP>(v, combine<OP>(combine<OP>(x.x, x.y), combine<OP>(x.z, x.w)));
            } else {
                v = combine<OP>(v, ap[idx]);
            }
        }
        v = wave_reduce<OP>(v);
        if (lane == 0U) {
            out[o_base] = v;
        }
    }
}

// Short contiguous rows, LPR lanes per row (see softmax_short_rows_kernel): 64 / LPR rows per wavefront.
template <int OP, int V, int LPR>
__global__ void __launch_bounds__(256) reduce_short_rows_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                                AxisGeom g)
{
    constexpr uint32_t RPW = 64U / LPR;
    const uint32_t lane = threadIdx.x & 63U, sub = lane % LPR;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t nvec = g.axis_len / V;
    for (uint32_t row0 = (blockIdx.x * 4U + wave) * RPW; row0 < g.rows; row0 += gridDim.x * 4U * RPW) {
        const uint32_t row = row0 + lane / LPR;
        const bool valid = row < g.rows;
        uint64_t a_base = g.a_off, o_base = g.o_off;
        if (valid) {
            row_bases(g, row, a_base, o_base);
        }
        const float *ap = a + a_base;
        float v = identity<OP>();
        for (uint32_t idx = sub; valid && idx < nvec; idx += LPR) {
            if (V == 4) {
                const float4 x = reinterpret_cast<const float4 *>(ap)[idx];
                v = combine<OP>(v, combine<OP>(combine<OP>(x.x, x.y), combine<OP>(x.z, x.w)));
            } else {
                v = combine<OP>(v, ap[idx]);
            }
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) {
            v = combine<OP>(v, __shfl_xor(v, off, 64));
        }
        if (valid && sub == 0U) {
            out[o_base] = v;
        }
    }
}

template <int OP, int RT, int THREADS>
__global__ void __launch_bounds__(THREADS) reduce_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                         AxisGeom g)
{
    __shared__ float red[THREADS];
    constexpr int NY = THREADS / RT;
    constexpr int U = kAxisUnroll;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t a_base = 0, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis];
    const uint32_t len = valid ? g.axis_len : 0U;
    const float *ap = a + a_base;
    float v = identity<OP>();
    for (uint32_t j0 = ty; j0 < len; j0 += NY * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t j = j0 + u * NY;
            x[u] = j < len ? ap[(uint64_t)j * as] : identity<OP>();
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v = combine<OP>(v, x[u]);
        }
    }
    v = block_reduce<OP, RT, THREADS>(v, red);
    if (valid && ty == 0) {
        out[o_base] = v;
    }
}

// Reduction along a contiguous, 16-byte aligned axis: one workgroup per row, four float4 loads in flight per thread.
template <int OP, int THREADS>
__global__ void __launch_bounds__(THREADS) reduce_contiguous_kernel(const float *__restrict__ a,
                                                                   float *__restrict__ out, AxisGeom g)
{
    __shared__ float red[THREADS];
    constexpr int U = 4;
    uint64_t a_base, o_base;
    row_bases(g, blockIdx.x, a_base, o_base);
    const float4 *ap = reinterpret_cast<const float4 *>(a + a_base);
    const uint32_t n4 = g.axis_len / 4U;
    float v = identity<OP>();
    for (uint32_t i0 = threadIdx.x; i0 < n4; i0 += THREADS * U) {
        float4 x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t idx = i0 + u * THREADS;
            x[u] = idx < n4 ? ap[idx] : make_float4(identity<OP>(), identity<OP>(), identity<OP>(), identity<OP>());
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v = combine<OP>(v, combine<OP>(combine<OP>(x[u].x, x[u].y), combine<OP>(x[u].z, x[u].w)));
        }
    }
    v = block_reduce<OP, 1, THREADS>(v, red);
    if (threadIdx.x == 0) {
        out[o_base] = v;
    }
}

// out[o_off + i*o_stride] = a[a_off + i*a_stride] (the reference's copy_real, src/common/qengine.cl:979)
__global__ void __launch_bounds__(256) copy_kernel(const float *__restrict__ a, float *__restrict__ out, uint64_t n,
                                                   uint32_t a_off, uint32_t a_stride, uint32_t o_off, uint32_t o_stride)
{
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) {
        out[(uint64_t)o_off + i * o_stride] = a[(uint64_t)a_off + i * a_stride];
    }
}

// Read-only sweeps of a buffer, for calibration: what the part delivers when bytes are only read.  Every lane reads
// 16 bytes per load; the xor of everything read is stored only if it equals a value it cannot be expected to have, so
// the reads cannot be optimised away and nothing is written.
typedef uint32_t sweep_u4 __attribute__((ext_vector_type(4)));
// The decode kernel's launch shape: one workgroup of 8 wavefronts per compute unit; a wavefront reads units of 8 KB
// (eight 16-byte loads per lane), the next unit requested before the current one is consumed.  RUNS: every wavefront
// walks ONE contiguous run of the buffer, as the decode kernel's wavefronts do; otherwise the wavefronts of the device
// take the units in turns (unit u goes to wavefront u mod 2048), so that at any moment the device reads one
// contiguous stretch of the buffer -- the fastest order found for this part.
constexpr uint32_t kRunUnitVecs = 512; // 16-byte vectors per unit
template <bool RUNS>
__global__ void __launch_bounds__(512) read_runs_kernel(const sweep_u4 *__restrict__ src, uint64_t n_units,
                                                        uint32_t units_per_run, uint32_t *sink)
{
    const uint32_t lane = threadIdx.x & 63, run = blockIdx.x * 8 + (threadIdx.x >> 6);
    const uint64_t stride = RUNS ? 1u : gridDim.x * 8u;
    const uint64_t u0 = RUNS ? (uint64_t)run * units_per_run : run;
    const uint64_t u1 = RUNS ? (u0 + units_per_run < n_units ? u0 + units_per_run : n_units) : n_units;
    sweep_u4 acc = { 0, 0, 0, 0 };
    if (u0 < u1) {
        sweep_u4 cur[8], nxt[8];
        const sweep_u4 *p = src + u0 * kRunUnitVecs + lane;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            cur[k] = p[64 * k];
        }
        for (uint64_t u = u0; u < u1; u += stride) {
            const sweep_u4 *q = src + (u + stride < u1 ? u + stride : u) * kRunUnitVecs + lane;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                nxt[k] = q[64 * k];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                acc ^= cur[k];
                cur[k] = nxt[k];
            }
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) {
        sink[0] = acc.x;
    }
}

struct PointGeom {
    uint32_t rank;
    uint32_t shape[kMaxRank];
    uint32_t a_stride[kMaxRank];
    uint32_t b_stride[kMaxRank];
    uint32_t o_stride[kMaxRank];
    uint32_t a_off, b_off, o_off;
    uint64_t n;
};

// The operation of an elementwise op on one pair of operands (unary ops ignore y).
template <int OP> __device__ __forceinline__ float elementwise_apply(float x, float y)
{
    if (OP == 0) {
        return x;
    } else if (OP == 5) {
        // SwiGLU's gate (include/modules/swiglu.hpp:71-77): gate * sigmoid(gate) * up, left to right
        const float sg = 1.0f / (1.0f + expf(-x));
        return (x * sg) * y;
    } else if (OP <= 4) {
        return OP == 1 ? x + y : OP == 2 ? x - y : OP == 3 ? x * y : x / y;
    } else if (OP == 6) {
        return fmaxf(x, 0.0f); // src/ops/real_unary.cpp:80
    } else if (OP == 7) {
        return 1.0f / (1.0f + expf(-x)); // src/ops/real_unary.cpp:135
    } else if (OP == 8) {
        return tanhf(x); // src/ops/real_unary.cpp:191
    }
    // Tensor::gelu (src/tensors/tensor.cpp:841-851), one rounded operation after the other as the reference's
    // chain of elementwise ops: x3 = x * x * x; inner = k2 * (x + k1 * x3); k0 * x * (1 + tanh(inner))
    const float x3 = (x * x) * x;
    const float inner = 0.7978845608028654f * (x + 0.044715f * x3);
    return (0.5f * x) * (1.0f + tanhf(inner));
}

// All operands dense in the same order of dimensions, 16-byte aligned, a multiple of four elements: 16-byte accesses,
// four of them in flight per thread and operand, no index arithmetic per element.
typedef float ew_f4 __attribute__((ext_vector_type(4)));
template <int OP> __global__ void __launch_bounds__(256) elementwise_flat_kernel(const ew_f4 *__restrict__ a,
                                                                                 const ew_f4 *__restrict__ b, ew_f4 *out,
                                                                                 uint64_t n4)
{
    constexpr bool kBinary = OP >= 1 && OP <= 5;
    auto one = [](const ew_f4 &x, const ew_f4 &y) {
        return ew_f4{ elementwise_apply<OP>(x[0], y[0]), elementwise_apply<OP>(x[1], y[1]),
                      elementwise_apply<OP>(x[2], y[2]), elementwise_apply<OP>(x[3], y[3]) };
    };
    // a workgroup takes whole pieces of 16 KB (its 256 threads x four 16-byte accesses, consecutive in memory), piece
    // number blockIdx.x + k * gridDim.x: the workgroups that run at one time work through one contiguous stretch of
    // every operand
    const uint64_t pieces = n4 / 1024U;
    for (uint64_t pc = blockIdx.x; pc < pieces; pc += gridDim.x) {
        const uint64_t i = pc * 1024U + threadIdx.x;
        ew_f4 x[4], y[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            x[u] = a[i + 256 * u];
            y[u] = kBinary ? b[i + 256 * u] : x[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            out[i + 256 * u] = one(x[u], y[u]);
        }
    }
    // what is left behind the last whole piece
    for (uint64_t i = pieces * 1024U + (uint64_t)blockIdx.x * 256U + threadIdx.x; i < n4; i += (uint64_t)gridDim.x * 256U) {
        const ew_f4 x = a[i];
        out[i] = one(x, kBinary ? b[i] : x);
    }
}

// One thread per logical element, dimension 0 fastest (the host orders the dimensions so that this is the direction
// in which the output is most contiguous).
template <int OP> __global__ void __launch_bounds__(256) elementwise_kernel(const float *__restrict__ a,
                                                                            const float *__restrict__ b, float *out,
                                                                            PointGeom g)
{
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < g.n; i += step) {
        uint64_t ai = g.a_off, bi = g.b_off, oi = g.o_off;
        if (g.n <= 0xffffffffull) {
            // the usual case: 32-bit index arithmetic (a 64-bit division costs several times as much)
            uint32_t tmp = (uint32_t)i;
            for (uint32_t dd = 0; dd < g.rank; ++dd) {
                const uint32_t dim = g.shape[dd];
                const uint32_t q = tmp / dim;
                const uint32_t c = tmp - q * dim;
                tmp = q;
                ai += (uint64_t)c * g.a_stride[dd];
                bi += (uint64_t)c * g.b_stride[dd];
                oi += (uint64_t)c * g.o_stride[dd];
            }
        } else {
            uint64_t tmp = i;
            for (uint32_t dd = 0; dd < g.rank; ++dd) {
                const uint32_t dim = g.shape[dd];
                const uint32_t c = (uint32_t)(tmp % dim);
                tmp /= dim;
                ai += (uint64_t)c * g.a_stride[dd];
                bi += (uint64_t)c * g.b_stride[dd];
                oi += (uint64_t)c * g.o_stride[dd];
            }
        }
        const float x = a[ai];
        out[oi] = elementwise_apply<OP>(x, (OP >= 1 && OP <= 5) ? b[bi] : x);
    }
}

// Copy between layouts whose contiguous dimensions differ (a transposed view made contiguous): 64 x 64 tiles of
// dimensions (0, k) go through LDS, read along k, where `a` is contiguous, and written along dimension 0, where `out`
// is.  One workgroup per tile; the other dimensions are enumerated by the workgroup index, dimension order kept.
__global__ void __launch_bounds__(256) transpose_copy_kernel(const float *__restrict__ a, float *__restrict__ out,
                                                             PointGeom g, uint32_t k, uint32_t tiles0, uint32_t tilesk)
{
    __shared__ float tile[64][65];
    uint32_t b = blockIdx.x;
    const uint32_t t0 = b % tiles0;
    b /= tiles0;
    const uint32_t tk = b % tilesk;
    uint32_t rest = b / tilesk;
    uint64_t ai = g.a_off, oi = g.o_off;
    for (uint32_t dd = 1; dd < g.rank; ++dd) {
        if (dd == k) {
            continue;
        }
        const uint32_t c = rest % g.shape[dd];
        rest /= g.shape[dd];
        ai += (uint64_t)c * g.a_stride[dd];
        oi += (uint64_t)c * g.o_stride[dd];
    }
    const uint32_t lx = threadIdx.x % 64U, ly = threadIdx.x / 64U;
    const uint32_t n0 = g.shape[0], nk = g.shape[k];
    {
        const uint32_t ik = tk * 64U + lx;
#pragma unroll 4
        for (uint32_t r = ly; r < 64U; r += 4U) {
            const uint32_t i0 = t0 * 64U + r;
            if (i0 < n0 && ik < nk) {
                tile[r][lx] = a[ai + (uint64_t)i0 * g.a_stride[0] + (uint64_t)ik * g.a_stride[k]];
            }
        }
    }
    __syncthreads();
    {
        const uint32_t i0 = t0 * 64U + lx;
#pragma unroll 4
        for (uint32_t r = ly; r < 64U; r += 4U) {
            const uint32_t ik = tk * 64U + r;
            if (i0 < n0 && ik < nk) {
                out[oi + (uint64_t)i0 * g.o_stride[0] + (uint64_t)ik * g.o_stride[k]] = tile[lx][r];
            }
        }
    }
}

__global__ void __launch_bounds__(256) triu_fill_kernel(float *a, uint32_t rows, uint32_t cols, float val,
                                                        uint32_t diagonal, uint32_t a_off, uint32_t s0, uint32_t s1)
{
    const uint64_t n = (uint64_t)rows * cols;
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += step) {
        const uint32_t i = (uint32_t)(idx % rows), j = (uint32_t)(idx / rows);
        if ((uint64_t)i + diagonal <= j) {
            a[(uint64_t)a_off + (uint64_t)i * s0 + (uint64_t)j * s1] = val;
        }
    }
}

struct RopeGeom {
    uint32_t shape[4]; // B, H, T, head_dim
    uint32_t x_stride[4], o_stride[4];
    uint32_t x_off, o_off;
    uint32_t table_rows, pos0;
    uint64_t n;
};

// out = x * cos + rotate_half(x) * sin (src/modules/rope.cpp:53-98): two rounded products, then the add.
// One thread per element, dimension 0 fastest.
__global__ void __launch_bounds__(256) rope_kernel(const float *__restrict__ x, const float *__restrict__ cos_t,
                                                   const float *__restrict__ sin_t, float *__restrict__ out, RopeGeom g)
{
    const uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    const uint32_t half = g.shape[3] >> 1;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < g.n; i += step) {
        uint64_t tmp = i;
        uint32_t c[4];
        uint64_t xi = g.x_off, oi = g.o_off;
        for (int dd = 0; dd < 4; ++dd) {
            c[dd] = (uint32_t)(tmp % g.shape[dd]);
            tmp /= g.shape[dd];
            oi += (uint64_t)c[dd] * g.o_stride[dd];
            if (dd < 3) {
                xi += (uint64_t)c[dd] * g.x_stride[dd];
            }
        }
        const uint32_t j = c[3];
        const float xv = x[xi + (uint64_t)j * g.x_stride[3]];
        const float partner = (j < half) ? -x[xi + (uint64_t)(j + half) * g.x_stride[3]]
                                         : x[xi + (uint64_t)(j - half) * g.x_stride[3]];
        const uint64_t ti = (uint64_t)(g.pos0 + c[2]) + (uint64_t)j * g.table_rows;
        const float a = xv * cos_t[ti];
        const float b = partner * sin_t[ti];
        out[oi] = a + b;
    }
}

int make_geom(const char *fn, uint32_t rank, const uint32_t *shape, uint32_t axis, uint32_t a_off,
              const uint32_t *a_stride, uint32_t o_off, const uint32_t *o_stride, bool out_keeps_axis, AxisGeom &g)
{
    WEED_HIP_REQUIRE(shape && a_stride && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(rank >= 1 && rank <= (uint32_t)kMaxRank, "%s: rank %u outside [1, %d]", fn, rank, kMaxRank);
    WEED_HIP_REQUIRE(axis < rank, "%s: axis %u out of range for rank %u", fn, axis, rank);
    g.rank = rank;
    g.axis = axis;
    g.a_off = a_off;
    g.o_off = o_off;
    uint64_t rows = 1;
    for (uint32_t i = 0; i < rank; ++i) {
        WEED_HIP_REQUIRE(shape[i] > 0, "%s: dimension %u is empty", fn, i);
        g.shape[i] = shape[i];
        g.a_stride[i] = a_stride[i];
        g.o_stride[i] = (i == axis && !out_keeps_axis) ? 0 : o_stride[i];
        if (i != axis) {
            rows *= shape[i];
        }
    }
    WEED_HIP_REQUIRE(rows < (1ull << 31), "%s: too many rows", fn);
    g.rows = (uint32_t)rows;
    g.axis_len = shape[axis];
    return WEED_HIP_OK;
}

enum AxisLaunch { AXIS_CONTIGUOUS, AXIS_ROW, AXIS_WAVE_VEC, AXIS_WAVE, AXIS_ROWS32, AXIS_ROWS32_WIDE, AXIS_ROWS16 };
constexpr uint32_t kWaveRowMax = 2048; // longest contiguous row that one wavefront takes

// How a softmax or reduction spreads its threads.  A contiguous axis gets one workgroup per row, or one wavefront
// per row when there are many rows of at most kWaveRowMax elements (float4 accesses where every row starts on a
// 16-byte boundary); a strided axis gets 32 neighbouring rows per workgroup (128-byte
// segments; 256 threads when that still makes a thousand workgroups, else 1024), and 16 rows with 1024 threads when
// rows are few and long (decode-time scores, [B * heads] rows of the context's length), so that enough loads stay
// in flight.
AxisLaunch choose_axis_launch(const AxisGeom &g, const float *a_dev, const float *out_dev, bool out_keeps_axis)
{
    const uint32_t as = g.a_stride[g.axis];
    if (as <= 1U || g.rows < 16U) {
        bool vec = as == 1U && g.axis_len % 4U == 0U && g.a_off % 4U == 0U &&
            reinterpret_cast<uintptr_t>(a_dev) % 16U == 0U;
        if (out_keeps_axis) {
            vec = vec && g.o_stride[g.axis] == 1U && g.o_off % 4U == 0U && reinterpret_cast<uintptr_t>(out_dev) % 16U == 0U;
        }
        for (uint32_t i = 0; vec && i < g.rank; ++i) {
            if (i != g.axis && g.shape[i] > 1U) {
                vec = g.a_stride[i] % 4U == 0U && (!out_keeps_axis || g.o_stride[i] % 4U == 0U);
            }
        }
        const bool unit_strides = as == 1U && (!out_keeps_axis || g.o_stride[g.axis] == 1U);
        if (unit_strides && g.axis_len <= kWaveRowMax && g.rows >= 1024U) {
            return vec ? AXIS_WAVE_VEC : AXIS_WAVE;
        }
        return (vec && g.axis_len >= 256U) ? AXIS_CONTIGUOUS : AXIS_ROW;
    }
    return g.rows >= 32U * 1024U ? AXIS_ROWS32 : g.rows >= 32U * 128U ? AXIS_ROWS32_WIDE : AXIS_ROWS16;
}

// Few rows and a long strided axis: bands of the axis (see band_partial_kernel); bands == 0: not this way.
// (Fewer than 16 rows fill an eighth of a band workgroup's lanes or less, and the launches have a floor of their own:
// they only go this way from `few_rows_least` elements on -- 15 strided rows of 100000: softmax 155 -> 54 us, sum 53 -> 15;
// 8 rows of 32768: 43 -> 38 and 17 -> 10; 8 rows of 8192 stay with one workgroup per row, 15 and 6 us against 18 and 8.)
BandGeom choose_bands(const AxisGeom &g, uint32_t most_rows, uint64_t few_rows_least)
{
    BandGeom bg = { 0U, 0U, 0U };
    if (g.rows < 16U && (uint64_t)g.rows * g.axis_len < few_rows_least) {
        return bg;
    }
    if (g.a_stride[g.axis] <= 1U || g.rows > std::min(most_rows, kBandRows) || g.axis_len < 4096U ||
        (uint64_t)g.axis_len * g.a_stride[g.axis] >= (1ull << 32)) {
        return bg;
    }
    const uint32_t row_groups = (g.rows + 63U) / 64U;
    const uint32_t want = std::max(1U, std::min(kMostBands, 512U / row_groups));
    bg.band_len = std::max(32U, (g.axis_len + want - 1U) / want);
    bg.band_len = (bg.band_len + 31U) / 32U * 32U;
    bg.bands = (g.axis_len + bg.band_len - 1U) / bg.band_len;
    bg.pitch = row_groups * 64U;
    if ((uint64_t)bg.bands * bg.pitch > kBandPartials) {
        bg.bands = 0U;
    }
    return bg;
}

// Four rows per workgroup; beyond 16 workgroups per compute unit the wavefronts loop over rows.
uint32_t wave_row_blocks(uint32_t rows) { return std::min<uint32_t>((rows + 3U) / 4U, 256U * 16U); }
// ... with 64 / lanes_per_row rows per wavefront
uint32_t short_row_blocks(uint32_t rows, uint32_t lanes_per_row)
{
    const uint32_t per_wg = 4U * (64U / lanes_per_row);
    return std::min<uint32_t>((rows + per_wg - 1U) / per_wg, 256U * 16U);
}

} // namespace

extern "C" {

int weed_hip_copy_f32(uint64_t n, const float *a_dev, uint32_t a_off, uint32_t a_stride, float *out_dev,
                      uint32_t o_off, uint32_t o_stride)
{
    WEED_HIP_REQUIRE(a_dev && out_dev, "weed_hip_copy_f32: null pointer");
    WEED_HIP_TRY(ensure_init());
    if (!n) {
        return WEED_HIP_OK;
    }
    ProfileScope prof("copy");
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + 255) / 256, 256u * 64u);
    copy_kernel<<<blocks, 256, 0, stream()>>>(a_dev, out_dev, n, a_off, a_stride, o_off, o_stride);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_read_sweep(const void *src_dev, uint64_t bytes, int per_wavefront_runs, uint32_t *sink_dev)
{
    const char *fn = "weed_hip_read_sweep";
    WEED_HIP_REQUIRE(src_dev && sink_dev, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(reinterpret_cast<uintptr_t>(src_dev) % 16U == 0U, "%s: the buffer must be 16-byte aligned", fn);
    WEED_HIP_TRY(ensure_init());
    ProfileScope prof("read_sweep");
    const uint64_t n_units = bytes / (16ull * kRunUnitVecs); // (a tail below one unit is not read)
    const uint32_t runs = 256u * 8u;
    const uint64_t per = (n_units + runs - 1) / runs;
    WEED_HIP_REQUIRE(per < (1ull << 32), "%s: buffer too large", fn);
    if (n_units && per_wavefront_runs) {
        read_runs_kernel<true><<<256, 512, 0, stream()>>>(static_cast<const sweep_u4 *>(src_dev), n_units, (uint32_t)per,
                                                          sink_dev);
    } else if (n_units) {
        read_runs_kernel<false><<<256, 512, 0, stream()>>>(static_cast<const sweep_u4 *>(src_dev), n_units, (uint32_t)per,
                                                           sink_dev);
    }
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_elementwise_f32(int op, uint32_t rank, const uint32_t *shape, const float *a_dev, uint32_t a_off,
                             const uint32_t *a_stride, const float *b_dev, uint32_t b_off, const uint32_t *b_stride,
                             float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_elementwise_f32";
    WEED_HIP_REQUIRE(op >= WEED_HIP_EW_COPY && op <= WEED_HIP_EW_GELU, "%s: unknown op %d", fn, op);
    WEED_HIP_REQUIRE(a_dev && out_dev && shape && a_stride && o_stride, "%s: null pointer", fn);
    const bool unary = op == WEED_HIP_EW_COPY || op >= WEED_HIP_EW_RELU;
    WEED_HIP_REQUIRE(unary || (b_dev && b_stride), "%s: null second operand", fn);
    WEED_HIP_REQUIRE(rank >= 1 && rank <= (uint32_t)kMaxRank, "%s: rank %u outside [1, %d]", fn, rank, kMaxRank);
    WEED_HIP_TRY(ensure_init());
    PointGeom g;
    g.rank = rank;
    g.a_off = a_off;
    g.b_off = b_off;
    g.o_off = o_off;
    g.n = 1;
    for (uint32_t i = 0; i < rank; ++i) {
        WEED_HIP_REQUIRE(shape[i] > 0, "%s: dimension %u is empty", fn, i);
        g.shape[i] = shape[i];
        g.a_stride[i] = a_stride[i];
        g.b_stride[i] = unary ? 0 : b_stride[i];
        g.o_stride[i] = o_stride[i];
        g.n *= shape[i];
    }
    WEED_HIP_REQUIRE(g.n < (1ull << 32), "%s: more than 2^32 elements", fn);
    // The order in which the dimensions are enumerated does not change an elementwise result, so they are walked in
    // rising order of the output's strides (size-1 dimensions last): neighbouring threads then write neighbouring
    // addresses whatever the layout (column-major, row-major views, permuted outputs).
    for (uint32_t i = 1; i < rank; ++i) {
        for (uint32_t j = i; j > 0; --j) {
            const bool prev_last = g.shape[j - 1] == 1U, cur_last = g.shape[j] == 1U;
            const bool swap = prev_last != cur_last ? prev_last : (!cur_last && g.o_stride[j] < g.o_stride[j - 1]);
            if (!swap) {
                break;
            }
            std::swap(g.shape[j], g.shape[j - 1]);
            std::swap(g.a_stride[j], g.a_stride[j - 1]);
            std::swap(g.b_stride[j], g.b_stride[j - 1]);
            std::swap(g.o_stride[j], g.o_stride[j - 1]);
        }
    }
    ProfileScope prof("elementwise");
    if (op == WEED_HIP_EW_COPY && g.rank >= 2 && g.o_stride[0] == 1U && g.a_stride[0] > 1U && g.shape[0] >= 16U) {
        // a transposed view: find the dimension along which `a` is contiguous
        uint32_t k = 0;
        for (uint32_t dd = 1; dd < g.rank && !k; ++dd) {
            if (g.a_stride[dd] == 1U && g.shape[dd] >= 16U) {
                k = dd;
            }
        }
        const uint32_t tiles0 = (g.shape[0] + 63U) / 64U, tilesk = k ? (g.shape[k] + 63U) / 64U : 0U;
        uint64_t tiles = (uint64_t)tiles0 * tilesk;
        for (uint32_t dd = 1; dd < g.rank; ++dd) {
            if (dd != k) {
                tiles *= g.shape[dd];
            }
        }
        if (k && tiles < (1ull << 31)) {
            transpose_copy_kernel<<<(uint32_t)tiles, 256, 0, stream()>>>(a_dev, out_dev, g, k, tiles0, tilesk);
            WEED_HIP_LAUNCH_CHECK();
            return WEED_HIP_OK;
        }
    }
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((g.n + 255) / 256, 256u * 64u);
    const float *b = unary ? a_dev : b_dev;
    // every operand dense in the same order of dimensions, aligned, whole 16-byte pieces: the flat kernel
    bool flat = g.n % 4U == 0U && g.n >= 4096U;
    uint64_t dense = 1;
    for (uint32_t dd = 0; dd < g.rank && flat; ++dd) {
        if (g.shape[dd] == 1U) {
            continue;
        }
        flat = g.o_stride[dd] == dense && g.a_stride[dd] == dense && (unary || g.b_stride[dd] == dense);
        dense *= g.shape[dd];
    }
    auto aligned = [](const float *p, uint32_t off) { return ((reinterpret_cast<uintptr_t>(p) + 4ull * off) & 15U) == 0U; };
    flat = flat && aligned(a_dev, a_off) && aligned(out_dev, o_off) && (unary || aligned(b_dev, b_off));
    if (flat) {
        const uint64_t n4 = g.n / 4U;
        const uint32_t fb = (uint32_t)std::min<uint64_t>((n4 + 1023) / 1024, 256u * 16u);
        const ew_f4 *a4 = reinterpret_cast<const ew_f4 *>(a_dev + a_off);
        const ew_f4 *b4 = reinterpret_cast<const ew_f4 *>(unary ? a_dev + a_off : b_dev + b_off);
        ew_f4 *o4 = reinterpret_cast<ew_f4 *>(out_dev + o_off);
        switch (op) {
        case WEED_HIP_EW_COPY: elementwise_flat_kernel<0><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_ADD: elementwise_flat_kernel<1><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_SUB: elementwise_flat_kernel<2><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_MUL: elementwise_flat_kernel<3><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_DIV: elementwise_flat_kernel<4><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_SILU_MUL: elementwise_flat_kernel<5><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_RELU: elementwise_flat_kernel<6><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_SIGMOID: elementwise_flat_kernel<7><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        case WEED_HIP_EW_TANH: elementwise_flat_kernel<8><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        default: elementwise_flat_kernel<9><<<fb, 256, 0, stream()>>>(a4, b4, o4, n4); break;
        }
        WEED_HIP_LAUNCH_CHECK();
        return WEED_HIP_OK;
    }
    switch (op) {
    case WEED_HIP_EW_SILU_MUL:
        elementwise_kernel<5><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_RELU:
        elementwise_kernel<6><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_SIGMOID:
        elementwise_kernel<7><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_TANH:
        elementwise_kernel<8><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_GELU:
        elementwise_kernel<9><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_COPY:
        elementwise_kernel<0><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_ADD:
        elementwise_kernel<1><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_SUB:
        elementwise_kernel<2><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    case WEED_HIP_EW_MUL:
        elementwise_kernel<3><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    default:
        elementwise_kernel<4><<<blocks, 256, 0, stream()>>>(a_dev, b, out_dev, g);
        break;
    }
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_triu_fill_f32(uint32_t rows, uint32_t cols, float val, uint32_t diagonal, float *a_dev, uint32_t a_off,
                           uint32_t a_s0, uint32_t a_s1)
{
    WEED_HIP_REQUIRE(a_dev, "weed_hip_triu_fill_f32: null pointer");
    WEED_HIP_TRY(ensure_init());
    const uint64_t n = (uint64_t)rows * cols;
    if (!n) {
        return WEED_HIP_OK;
    }
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + 255) / 256, 256u * 64u);
    triu_fill_kernel<<<blocks, 256, 0, stream()>>>(a_dev, rows, cols, val, diagonal, a_off, a_s0, a_s1);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_rope_f32(const uint32_t shape[4], const float *x_dev, uint32_t x_off, const uint32_t x_stride[4],
                      const float *cos_dev, const float *sin_dev, uint32_t table_rows, uint32_t pos0, float *out_dev,
                      uint32_t o_off, const uint32_t o_stride[4])
{
    const char *fn = "weed_hip_rope_f32";
    WEED_HIP_REQUIRE(shape && x_dev && x_stride && cos_dev && sin_dev && out_dev && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(x_dev != out_dev, "%s: cannot run in place", fn);
    WEED_HIP_TRY(ensure_init());
    RopeGeom g;
    g.n = 1;
    for (int i = 0; i < 4; ++i) {
        WEED_HIP_REQUIRE(shape[i] > 0, "%s: dimension %d is empty", fn, i);
        g.shape[i] = shape[i];
        g.x_stride[i] = x_stride[i];
        g.o_stride[i] = o_stride[i];
        g.n *= shape[i];
    }
    WEED_HIP_REQUIRE(shape[3] % 2 == 0, "%s: head_dim %u must be even", fn, shape[3]);
    WEED_HIP_REQUIRE((uint64_t)pos0 + shape[2] <= table_rows, "%s: positions [%u, %u) exceed the table's %u rows", fn,
                     pos0, pos0 + shape[2], table_rows);
    WEED_HIP_REQUIRE(g.n < (1ull << 32), "%s: more than 2^32 elements", fn);
    g.x_off = x_off;
    g.o_off = o_off;
    g.table_rows = table_rows;
    g.pos0 = pos0;
    ProfileScope prof("rope");
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((g.n + 255) / 256, 256u * 64u);
    rope_kernel<<<blocks, 256, 0, stream()>>>(x_dev, cos_dev, sin_dev, out_dev, g);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

// Up to this many contiguous rows beyond 8192 elements get sixteen wavefronts each instead of four (one workgroup per
// row either way; with more rows the compute units are full of four-wavefront workgroups anyway).
constexpr uint32_t kFewLongRows = 512U;

int weed_hip_softmax_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *a_dev, uint32_t a_off,
                         const uint32_t *a_stride, float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_softmax_f32";
    WEED_HIP_REQUIRE(a_dev && out_dev, "%s: null pointer", fn);
    WEED_HIP_TRY(ensure_init());
    AxisGeom g;
    WEED_HIP_TRY(make_geom(fn, rank, shape, axis, a_off, a_stride, o_off, o_stride, true, g));
    ProfileScope prof("softmax");
    const AxisLaunch how = choose_axis_launch(g, a_dev, out_dev, true);
    if (how == AXIS_CONTIGUOUS) {
        if (g.axis_len <= 8U * 4U * 256U) {
            softmax_contiguous_kernel<8, 256, true><<<g.rows, 256, 0, stream()>>>(a_dev, out_dev, g);
        } else if (g.rows <= kFewLongRows && g.axis_len <= 8U * 4U * 1024U) {
            // few rows, each a workgroup's: sixteen wavefronts keep up to 32768 elements in registers and read once
            softmax_contiguous_kernel<8, 1024, true><<<g.rows, 1024, 0, stream()>>>(a_dev, out_dev, g);
        } else if (g.rows <= kFewLongRows) {
            softmax_contiguous_kernel<8, 1024, false><<<g.rows, 1024, 0, stream()>>>(a_dev, out_dev, g);
        } else {
            softmax_contiguous_kernel<8, 256, false><<<g.rows, 256, 0, stream()>>>(a_dev, out_dev, g);
        }
    } else if (how == AXIS_WAVE_VEC && g.axis_len <= 512U) {
        // short rows: as few lanes per row as keep a lane's share at one or two 16-byte pieces
        const uint32_t n4 = g.axis_len / 4U;
#define WEED_SHORT_ROWS(V, C, LPR)                                                                                     \
    softmax_short_rows_kernel<V, C, LPR><<<short_row_blocks(g.rows, LPR), 256, 0, stream()>>>(a_dev, out_dev, g)
        if (n4 <= 4U) {
            WEED_SHORT_ROWS(4, 1, 4);
        } else if (n4 <= 8U) {
            WEED_SHORT_ROWS(4, 2, 4);
        } else if (n4 <= 16U) {
            WEED_SHORT_ROWS(4, 1, 16);
        } else if (n4 <= 32U) {
            WEED_SHORT_ROWS(4, 2, 16);
        } else if (n4 <= 64U) {
            WEED_SHORT_ROWS(4, 4, 16);
        } else {
            WEED_SHORT_ROWS(4, 4, 32);
        }
    } else if (how == AXIS_WAVE_VEC) {
        // (kWaveRowMax = 8 * 4 * 64: such a row always fits a wavefront's registers)
        softmax_wave_rows_kernel<4, 8, true><<<wave_row_blocks(g.rows), 256, 0, stream()>>>(a_dev, out_dev, g);
    } else if (how == AXIS_WAVE && g.axis_len <= 128U) {
        if (g.axis_len <= 8U) {
            WEED_SHORT_ROWS(1, 2, 4);
        } else if (g.axis_len <= 32U) {
            WEED_SHORT_ROWS(1, 2, 16);
        } else {
            WEED_SHORT_ROWS(1, 4, 32);
        }
#undef WEED_SHORT_ROWS
    } else if (how == AXIS_WAVE) {
        if (g.axis_len <= 16U * 64U) {
            softmax_wave_rows_kernel<1, 16, true><<<wave_row_blocks(g.rows), 256, 0, stream()>>>(a_dev, out_dev, g);
        } else {
            softmax_wave_rows_kernel<1, 16, false><<<wave_row_blocks(g.rows), 256, 0, stream()>>>(a_dev, out_dev, g);
        }
    } else if (how == AXIS_ROW && choose_bands(g, 4096U, 3U << 16).bands == 0U) { // (fewer than 16 long strided rows go by bands)
        softmax_kernel<1, 256><<<g.rows, 256, 0, stream()>>>(a_dev, out_dev, g);
    } else if ((uint64_t)g.axis_len * g.a_stride[axis] >= (1ull << 32)) {
        softmax_kernel<16, 1024><<<(g.rows + 15) / 16, 1024, 0, stream()>>>(a_dev, out_dev, g);
    } else if (g.axis_len <= 16U * kStridedThreads / 32 && g.rows >= 32U * 256U) {
        // (short axes keep fewer registers per thread, so that more workgroups share a compute unit and their
        // loads, sums and stores overlap: 2^18 rows of 512 at 4.2 TB/s of algorithmic bytes with 32 registers,
        // 2.9 with 64; 2^19 rows of 256 at 4.1 with 16)
        softmax_strided_cached_kernel<32, kStridedThreads, false, 16>
            <<<(g.rows + 31) / 32, kStridedThreads, 0, stream()>>>(a_dev, out_dev, g);
    } else if (g.axis_len <= 32U * kStridedThreads / 32 && g.rows >= 32U * 256U) {
        softmax_strided_cached_kernel<32, kStridedThreads, false, 32>
            <<<(g.rows + 31) / 32, kStridedThreads, 0, stream()>>>(a_dev, out_dev, g);
    } else if (g.axis_len <= (uint32_t)(kStridedCached * kStridedThreads / 32) && g.rows >= 32U * 256U) {
        softmax_strided_cached_kernel<32><<<(g.rows + 31) / 32, kStridedThreads, 0, stream()>>>(a_dev, out_dev, g);
    } else if (g.axis_len <= (uint32_t)(kStridedCached * kStridedThreads / 16) && g.rows < 12288U) {
        // (with more rows the two passes over 32 rows per workgroup are faster: 16-row tiles are half lines.
        // 4096 rows of 2048: 22 us against 35; 16384 rows: 83 against 72; 65536 rows: 427 against 369)
        softmax_strided_cached_kernel<16><<<(g.rows + 15) / 16, kStridedThreads, 0, stream()>>>(a_dev, out_dev, g);
    } else if (const BandGeom bg = choose_bands(g, 4096U, 3U << 16); bg.bands != 0U) {
        // (up to 4096 rows of at least 4096 strided elements -- with 8192 rows and more the walks over 32 rows per
        // workgroup are as fast or faster: 8192 x 8192 174 against 187 us; 4096 x 32768 372 us here against 525 --: 64 rows of 32768 25 us, where 16 rows per workgroup took
        // 166; 256 rows of 8192 16 us against 25 with the narrow tiles below; 2048 rows of 16384 83 against 127)
        const dim3 grid((g.rows + 63U) / 64U, bg.bands);
        band_partial_kernel<3><<<grid, 256, 0, stream()>>>(a_dev, g, bg);
        band_merge_kernel<3><<<(g.rows + 63U) / 64U, 256, 0, stream()>>>(out_dev, g, bg);
        band_softmax_finish_kernel<<<grid, 256, 0, stream()>>>(a_dev, out_dev, g, bg);
    } else if (g.rows < 2048U && g.axis_len <= (uint32_t)(kStridedCached * kStridedThreadsLong / 4)) {
        // few rows of 2049 to 4095 elements: narrow tiles, so that there are workgroups enough, and one pass
        softmax_strided_cached_kernel<4, kStridedThreadsLong, true>
            <<<8 * ((g.rows + 31) / 32), kStridedThreadsLong, 0, stream()>>>(a_dev, out_dev, g);
    } else if (g.rows < 3072U && g.axis_len <= (uint32_t)(kStridedCached * kStridedThreadsLong / 8)) {
        // (2049 to 3071 rows; from 3072 rows on the two passes over 16 or 32 rows are as fast or faster)
        softmax_strided_cached_kernel<8, kStridedThreadsLong, true>
            <<<8 * ((g.rows + 63) / 64), kStridedThreadsLong, 0, stream()>>>(a_dev, out_dev, g);
    } else if (how == AXIS_ROWS32) {
        softmax_kernel<32, 256><<<(g.rows + 31) / 32, 256, 0, stream()>>>(a_dev, out_dev, g);
    } else if (how == AXIS_ROWS32_WIDE) {
        softmax_kernel<32, 1024><<<(g.rows + 31) / 32, 1024, 0, stream()>>>(a_dev, out_dev, g);
    } else {
        softmax_kernel<16, 1024><<<(g.rows + 15) / 16, 1024, 0, stream()>>>(a_dev, out_dev, g);
    }
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_reduce_f32(int op, uint32_t rank, const uint32_t *shape, uint32_t axis, const float *a_dev, uint32_t a_off,
                        const uint32_t *a_stride, float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_reduce_f32";
    WEED_HIP_REQUIRE(a_dev && out_dev, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(op >= 0 && op <= 2, "%s: unknown op %d", fn, op);
    WEED_HIP_TRY(ensure_init());
    AxisGeom g;
    WEED_HIP_TRY(make_geom(fn, rank, shape, axis, a_off, a_stride, o_off, o_stride, false, g));
    ProfileScope prof("reduce");
    const AxisLaunch how = choose_axis_launch(g, a_dev, out_dev, false);
    const BandGeom bands = choose_bands(g, g.axis_len >= 16384U ? 4096U : 3072U, 1U << 18); // (4096 rows of 4096 to 8192: 13 and 23 us without bands, 16 and 26 with)
#define WEED_LAUNCH_REDUCE(OP)                                                                                         \
    if (bands.bands != 0U && how != AXIS_CONTIGUOUS && how != AXIS_WAVE && how != AXIS_WAVE_VEC) {                     \
        band_partial_kernel<OP><<<dim3((g.rows + 63U) / 64U, bands.bands), 256, 0, stream()>>>(a_dev, g, bands);       \
        band_merge_kernel<OP><<<(g.rows + 63U) / 64U, 256, 0, stream()>>>(out_dev, g, bands);                         \
    } else if (how == AXIS_CONTIGUOUS) {                                                                               \
        reduce_contiguous_kernel<OP, 256><<<g.rows, 256, 0, stream()>>>(a_dev, out_dev, g);                            \
    } else if (how == AXIS_WAVE_VEC && g.axis_len <= 64U) {                                                            \
        reduce_short_rows_kernel<OP, 4, 4><<<short_row_blocks(g.rows, 4), 256, 0, stream()>>>(a_dev, out_dev, g);      \
    } else if (how == AXIS_WAVE_VEC && g.axis_len <= 256U) {                                                           \
        reduce_short_rows_kernel<OP, 4, 16><<<short_row_blocks(g.rows, 16), 256, 0, stream()>>>(a_dev, out_dev, g);    \
    } else if (how == AXIS_WAVE_VEC) {                                                                                 \
        reduce_wave_rows_kernel<OP, 4><<<wave_row_blocks(g.rows), 256, 0, stream()>>>(a_dev, out_dev, g);              \
    } else if (how == AXIS_WAVE && g.axis_len <= 64U) {                                                                \
        reduce_short_rows_kernel<OP, 1, 16><<<short_row_blocks(g.rows, 16), 256, 0, stream()>>>(a_dev, out_dev, g);    \
    } else if (how == AXIS_WAVE) {                                                                                     \
        reduce_wave_rows_kernel<OP, 1><<<wave_row_blocks(g.rows), 256, 0, stream()>>>(a_dev, out_dev, g);              \
    } else if (how == AXIS_ROW) {                                                                                      \
        reduce_kernel<OP, 1, 256><<<g.rows, 256, 0, stream()>>>(a_dev, out_dev, g);                                    \
    } else if (how == AXIS_ROWS32) {                                                                                   \
        reduce_kernel<OP, 32, 256><<<(g.rows + 31) / 32, 256, 0, stream()>>>(a_dev, out_dev, g);                       \
    } else if (how == AXIS_ROWS32_WIDE) {                                                                              \
        reduce_kernel<OP, 32, 1024><<<(g.rows + 31) / 32, 1024, 0, stream()>>>(a_dev, out_dev, g);                     \
    } else {                                                                                                           \
        reduce_kernel<OP, 16, 1024><<<(g.rows + 15) / 16, 1024, 0, stream()>>>(a_dev, out_dev, g);                     \
    }
    if (op == WEED_HIP_REDUCE_SUM) {
        WEED_LAUNCH_REDUCE(0)
    } else if (op == WEED_HIP_REDUCE_MAX) {
        WEED_LAUNCH_REDUCE(1)
    } else {
        WEED_LAUNCH_REDUCE(2)
    }
#undef WEED_LAUNCH_REDUCE
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // extern "C"
