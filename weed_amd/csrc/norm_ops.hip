// RMSNorm and LayerNorm over one axis of a strided fp32 tensor, each as ONE kernel (the reference composes them from
// elementwise ops and an axis mean: include/modules/rms_norm.hpp:34-38, src/modules/layernorm.cpp:29-42).
//
// Rows (all index combinations of the other dimensions) are enumerated with dimension 0 fastest, the contiguous
// direction of Weed's column-major tensors.  A workgroup takes RT neighbouring rows and spreads its other threads along
// the normalised axis: RT = 1 when the axis itself is contiguous, RT = 16 or 32 when it is strided (a decode step's
// [B, 1, d_model] activations have the batch index fastest), so that loads and stores are coalesced either way.  A row
// whose share per thread fits CACHED registers is read once; longer rows are read again for every pass.
//
// Per element the arithmetic is the reference's, operation for operation: x / r * w with r = sqrt(mean(x^2) + eps)
// (RMSNorm), and (x - mu) / r * gamma + beta with r = sqrt(mean((x - mu)^2) + eps) (LayerNorm); only the sums are
// added as trees instead of one after the other.
#include "common.h"

#include <algorithm>

using namespace weedhip;

namespace {

constexpr int kMaxRank = 8;

struct NormGeom {
    uint32_t rank;
    uint32_t axis;
    uint32_t shape[kMaxRank];
    uint32_t x_stride[kMaxRank];
    uint32_t o_stride[kMaxRank];
    uint32_t x_off, o_off;
    uint32_t rows;
    uint32_t axis_len;
    uint32_t w_off, w_stride; // weight / gamma along the axis
    uint32_t b_off, b_stride; // beta along the axis (LayerNorm)
    float eps;
};

__device__ __forceinline__ void row_bases(const NormGeom &g, uint32_t row, uint64_t &x_base, uint64_t &o_base)
{
    x_base = g.x_off;
    o_base = g.o_off;
    uint32_t tmp = row;
    for (uint32_t dd = 0; dd < g.rank; ++dd) {
        if (dd == g.axis) {
            continue;
        }
        const uint32_t dim = g.shape[dd];
        const uint32_t i = tmp % dim;
        tmp /= dim;
        x_base += (uint64_t)i * g.x_stride[dd];
        o_base += (uint64_t)i * g.o_stride[dd];
    }
}

// Sum of `v` over the NY threads that share threadIdx.x % RT; valid in every thread.  RT divides 64: the threads of a
// row inside one wavefront are combined by shuffles first, the wavefronts through LDS.
template <int RT, int THREADS> __device__ __forceinline__ float row_sum(float v, float *red)
{
    constexpr int WAVES = THREADS / 64;
#pragma unroll
    for (int o = 32; o >= RT; o >>= 1) {
        v += __shfl_xor(v, o);
    }
    if constexpr (WAVES == 1) {
        return v;
    }
    const uint32_t tx = threadIdx.x % RT, wave = threadIdx.x / 64;
    if ((threadIdx.x & 63) < RT) {
        red[wave * RT + tx] = v;
    }
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        s += red[w * RT + tx];
    }
    __syncthreads();
    return s;
}

// LAYER false: RMSNorm, true: LayerNorm.  CACHED: elements of a row that a thread keeps in registers (0: none, every
// pass reads memory again).
template <bool LAYER, int RT, int THREADS, int CACHED>
__global__ void __launch_bounds__(THREADS) norm_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                       const float *__restrict__ beta, float *__restrict__ out,
                                                       NormGeom g)
{
    __shared__ float red[(THREADS / 64) * RT];
    constexpr int NY = THREADS / RT;
    constexpr int NC = CACHED ? CACHED : 1;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t x_base = g.x_off, o_base = g.o_off;
    if (valid) {
        row_bases(g, row, x_base, o_base);
    }
    const uint32_t xs = g.x_stride[g.axis], os = g.o_stride[g.axis];
    const uint32_t len = valid ? g.axis_len : 0U;
    const float *xp = x + x_base;
    float *op = out + o_base;
    const float n = (float)g.axis_len;
    float v[NC];
    if constexpr (CACHED != 0) {
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t j = ty + c * NY;
            v[c] = j < len ? xp[(uint64_t)j * xs] : 0.0f;
        }
    }
    auto element = [&](int c, uint32_t j) -> float { return CACHED != 0 ? v[c] : xp[(uint64_t)j * xs]; };
    float mu = 0.0f;
    if constexpr (LAYER) {
        float s = 0.0f;
        if constexpr (CACHED != 0) {
#pragma unroll
            for (int c = 0; c < CACHED; ++c) {
                s += v[c]; // (positions beyond the row hold zeros)
            }
        } else {
            for (uint32_t j = ty; j < len; j += NY) {
                s += xp[(uint64_t)j * xs];
            }
        }
        mu = row_sum<RT, THREADS>(s, red) / n;
    }
    float sq = 0.0f;
    if constexpr (CACHED != 0) {
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t j = ty + c * NY;
            const float xc = v[c] - mu;
            const float p = xc * xc;
            sq += j < len ? p : 0.0f;
        }
    } else {
        for (uint32_t j = ty; j < len; j += NY) {
            const float xc = xp[(uint64_t)j * xs] - mu;
            sq += xc * xc;
        }
    }
    const float mean_sq = row_sum<RT, THREADS>(sq, red) / n;
    const float r = sqrtf(mean_sq + g.eps);
    auto finish = [&](int c, uint32_t j) {
        const float xc = element(c, j) - mu; // (mu is 0 for RMSNorm: x - 0 is x exactly)
        float y = (xc / r) * w[(uint64_t)g.w_off + (uint64_t)j * g.w_stride];
        if constexpr (LAYER) {
            y = y + beta[(uint64_t)g.b_off + (uint64_t)j * g.b_stride];
        }
        op[(uint64_t)j * os] = y;
    };
    if constexpr (CACHED != 0) {
#pragma unroll
        for (int c = 0; c < CACHED; ++c) {
            const uint32_t j = ty + c * NY;
            if (j < len) {
                finish(c, j);
            }
        }
    } else {
        for (uint32_t j = ty; j < len; j += NY) {
            finish(0, j);
        }
    }
}

// Few rows along a strided axis (a decode step's (B, 1, d_model) activations: the batch index is the contiguous one):
// a workgroup takes 16 neighbouring rows and adds up the WHOLE axis for them, but finishes only its own slice of the
// axis (gridDim.y slices).  The sums are computed once per slice -- redundant reads of a tensor that sits in L2 -- so
// that the per-element work (a correctly rounded division among it) spreads over enough compute units.
template <bool LAYER> __global__ void __launch_bounds__(1024) norm_sliced_kernel(const float *__restrict__ x,
                                                                               const float *__restrict__ w,
                                                                               const float *__restrict__ beta,
                                                                               float *__restrict__ out, NormGeom g)
{
    constexpr int RT = 16, THREADS = 1024, NY = THREADS / RT, U = 8;
    __shared__ float red[(THREADS / 64) * RT];
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t x_base = g.x_off, o_base = g.o_off;
    if (valid) {
        row_bases(g, row, x_base, o_base);
    }
    const uint32_t xs = g.x_stride[g.axis], os = g.o_stride[g.axis];
    const uint32_t len = valid ? g.axis_len : 0U;
    const float *xp = x + x_base;
    float *op = out + o_base;
    const float n = (float)g.axis_len;
    // sum of f(element) over the thread's share of the row, U loads in flight
    auto share = [&](auto f) {
        float s = 0.0f;
        for (uint32_t j0 = ty; j0 < len; j0 += NY * U) {
            float v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t j = j0 + u * NY;
                v[u] = j < len ? xp[(uint64_t)j * xs] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                s += (j0 + u * NY < len) ? f(v[u]) : 0.0f;
            }
        }
        return s;
    };
    float mu = 0.0f;
    if constexpr (LAYER) {
        mu = row_sum<RT, THREADS>(share([](float v) { return v; }), red) / n;
    }
    const float mean_sq = row_sum<RT, THREADS>(share([mu](float v) { return (v - mu) * (v - mu); }), red) / n;
    const float r = sqrtf(mean_sq + g.eps);
    const uint32_t per = (g.axis_len + gridDim.y - 1) / gridDim.y;
    const uint32_t j_end = min(len, (blockIdx.y + 1) * per);
    for (uint32_t j = blockIdx.y * per + ty; j < j_end; j += NY) {
        const float xc = xp[(uint64_t)j * xs] - mu;
        float y = (xc / r) * w[(uint64_t)g.w_off + (uint64_t)j * g.w_stride];
        if constexpr (LAYER) {
            y = y + beta[(uint64_t)g.b_off + (uint64_t)j * g.b_stride];
        }
        op[(uint64_t)j * os] = y;
    }
}

template <bool LAYER, int RT, int THREADS>
void launch_cached(const float *x, const float *w, const float *b, float *out, const NormGeom &g, hipStream_t s)
{
    constexpr uint32_t NY = THREADS / RT;
    const uint32_t blocks = (g.rows + RT - 1) / RT;
    const uint32_t per_thread = (g.axis_len + NY - 1) / NY;
    if (per_thread <= 4) {
        norm_kernel<LAYER, RT, THREADS, 4><<<blocks, THREADS, 0, s>>>(x, w, b, out, g);
    } else if (per_thread <= 16) {
        norm_kernel<LAYER, RT, THREADS, 16><<<blocks, THREADS, 0, s>>>(x, w, b, out, g);
    } else if (per_thread <= 64) {
        norm_kernel<LAYER, RT, THREADS, 64><<<blocks, THREADS, 0, s>>>(x, w, b, out, g);
    } else {
        norm_kernel<LAYER, RT, THREADS, 0><<<blocks, THREADS, 0, s>>>(x, w, b, out, g);
    }
}

template <bool LAYER>
int norm_impl(const char *fn, uint32_t rank, const uint32_t *shape, uint32_t axis, const float *x_dev, uint32_t x_off,
              const uint32_t *x_stride, const float *w_dev, uint32_t w_off, uint32_t w_stride, const float *b_dev,
              uint32_t b_off, uint32_t b_stride, float eps, float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    WEED_HIP_REQUIRE(x_dev && w_dev && out_dev && shape && x_stride && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(!LAYER || b_dev, "%s: null beta", fn);
    WEED_HIP_REQUIRE(rank >= 1 && rank <= (uint32_t)kMaxRank, "%s: rank %u outside [1, %d]", fn, rank, kMaxRank);
    WEED_HIP_REQUIRE(axis < rank, "%s: axis %u out of range for rank %u", fn, axis, rank);
    WEED_HIP_TRY(ensure_init());
    NormGeom g;
    g.rank = rank;
    g.axis = axis;
    g.x_off = x_off;
    g.o_off = o_off;
    uint64_t rows = 1;
    for (uint32_t i = 0; i < rank; ++i) {
        WEED_HIP_REQUIRE(shape[i] > 0, "%s: dimension %u is empty", fn, i);
        g.shape[i] = shape[i];
        g.x_stride[i] = x_stride[i];
        g.o_stride[i] = o_stride[i];
        if (i != axis) {
            rows *= shape[i];
        }
    }
    WEED_HIP_REQUIRE(rows < (1ull << 31), "%s: too many rows", fn);
    g.rows = (uint32_t)rows;
    g.axis_len = shape[axis];
    g.w_off = w_off;
    g.w_stride = w_stride;
    g.b_off = b_off;
    g.b_stride = b_stride;
    g.eps = eps;
    ProfileScope prof(LAYER ? "layer_norm" : "rms_norm");
    hipStream_t s = stream();
    const uint32_t xs = x_stride[axis];
    if (xs <= 1U || g.rows < 16U) {
        // the axis is the contiguous direction (or there are too few rows to share a workgroup): one workgroup per row
        launch_cached<LAYER, 1, 256>(x_dev, w_dev, b_dev, out_dev, g, s);
    } else if (g.rows >= 32U * 512U) {
        launch_cached<LAYER, 32, 256>(x_dev, w_dev, b_dev, out_dev, g, s);
    } else if (x_dev == out_dev) {
        // in place: the whole row must be summed before any of it is overwritten, so one workgroup does both
        launch_cached<LAYER, 16, 1024>(x_dev, w_dev, b_dev, out_dev, g, s);
    } else {
        // few rows, strided axis (a decode step's activations): see norm_sliced_kernel
        const uint32_t row_tiles = (g.rows + 15U) / 16U;
        const uint32_t slices = std::max(1U, std::min((128U + row_tiles - 1U) / row_tiles, (g.axis_len + 63U) / 64U));
        norm_sliced_kernel<LAYER><<<dim3(row_tiles, slices), 1024, 0, s>>>(x_dev, w_dev, b_dev, out_dev, g);
    }
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // namespace

extern "C" {

int weed_hip_rms_norm_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *x_dev, uint32_t x_off,
                          const uint32_t *x_stride, const float *w_dev, uint32_t w_off, uint32_t w_stride, float eps,
                          float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    return norm_impl<false>("weed_hip_rms_norm_f32", rank, shape, axis, x_dev, x_off, x_stride, w_dev, w_off, w_stride,
                            nullptr, 0U, 0U, eps, out_dev, o_off, o_stride);
}

int weed_hip_layer_norm_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *x_dev, uint32_t x_off,
                            const uint32_t *x_stride, const float *gamma_dev, uint32_t gamma_off, uint32_t gamma_stride,
                            const float *beta_dev, uint32_t beta_off, uint32_t beta_stride, float eps, float *out_dev,
                            uint32_t o_off, const uint32_t *o_stride)
{
    return norm_impl<true>("weed_hip_layer_norm_f32", rank, shape, axis, x_dev, x_off, x_stride, gamma_dev, gamma_off,
                           gamma_stride, beta_dev, beta_off, beta_stride, eps, out_dev, o_off, o_stride);
}

} // extern "C"
