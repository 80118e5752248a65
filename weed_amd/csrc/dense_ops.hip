// Strided fp32 softmax and axis reductions (the standalone ops that feed attention in the reference:
// src/ops/softmax.cpp:276-287, src/ops/reduce.cpp:342-386).
//
// Rows (all index combinations of the non-reduced dimensions) are enumerated with dimension 0 fastest, which is the
// contiguous direction of Weed's column-major tensors; a workgroup takes RT neighbouring rows and spreads the
// remaining threads along the reduced axis, so that loads are coalesced whether the axis is the contiguous
// dimension (RT = 1) or a strided one (RT = 16).
#include "common.h"

#include <algorithm>
#include <cmath>

using namespace weedhip;

namespace {

constexpr int kMaxRank = 8;
constexpr int kThreads = 256;

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
template <int OP, int RT> __device__ __forceinline__ float block_reduce(float v, float *red)
{
    constexpr int NY = kThreads / RT;
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

template <int RT> __global__ void __launch_bounds__(kThreads) softmax_kernel(const float *__restrict__ a,
                                                                            float *__restrict__ out, AxisGeom g)
{
    __shared__ float red[kThreads];
    constexpr int NY = kThreads / RT;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t a_base = 0, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis], os = g.o_stride[g.axis];
    float mx = -INFINITY;
    if (valid) {
        for (uint32_t j = ty; j < g.axis_len; j += NY) {
            mx = fmaxf(mx, a[a_base + (uint64_t)j * as]);
        }
    }
    mx = block_reduce<1, RT>(mx, red);
    float s = 0.0f;
    if (valid) {
        for (uint32_t j = ty; j < g.axis_len; j += NY) {
            s += expf(a[a_base + (uint64_t)j * as] - mx);
        }
    }
    s = block_reduce<0, RT>(s, red);
    if (valid) {
        for (uint32_t j = ty; j < g.axis_len; j += NY) {
            out[o_base + (uint64_t)j * os] = expf(a[a_base + (uint64_t)j * as] - mx) / s;
        }
    }
}

template <int OP, int RT> __global__ void __launch_bounds__(kThreads) reduce_kernel(const float *__restrict__ a,
                                                                                   float *__restrict__ out, AxisGeom g)
{
    __shared__ float red[kThreads];
    constexpr int NY = kThreads / RT;
    const uint32_t tx = threadIdx.x % RT, ty = threadIdx.x / RT;
    const uint32_t row = blockIdx.x * RT + tx;
    const bool valid = row < g.rows;
    uint64_t a_base = 0, o_base = 0;
    if (valid) {
        row_bases(g, row, a_base, o_base);
    }
    const uint32_t as = g.a_stride[g.axis];
    float v = identity<OP>();
    if (valid) {
        for (uint32_t j = ty; j < g.axis_len; j += NY) {
            v = combine<OP>(v, a[a_base + (uint64_t)j * as]);
        }
    }
    v = block_reduce<OP, RT>(v, red);
    if (valid && ty == 0) {
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

struct PointGeom {
    uint32_t rank;
    uint32_t shape[kMaxRank];
    uint32_t a_stride[kMaxRank];
    uint32_t b_stride[kMaxRank];
    uint32_t o_stride[kMaxRank];
    uint32_t a_off, b_off, o_off;
    uint64_t n;
};

// One thread per logical element, dimension 0 fastest (the contiguous direction of column-major tensors).
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
        float r;
        if (OP == 0) {
            r = x;
        } else {
            const float y = b[bi];
            r = OP == 1 ? x + y : OP == 2 ? x - y : OP == 3 ? x * y : x / y;
        }
        out[oi] = r;
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

int weed_hip_elementwise_f32(int op, uint32_t rank, const uint32_t *shape, const float *a_dev, uint32_t a_off,
                             const uint32_t *a_stride, const float *b_dev, uint32_t b_off, const uint32_t *b_stride,
                             float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_elementwise_f32";
    WEED_HIP_REQUIRE(op >= WEED_HIP_EW_COPY && op <= WEED_HIP_EW_DIV, "%s: unknown op %d", fn, op);
    WEED_HIP_REQUIRE(a_dev && out_dev && shape && a_stride && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(op == WEED_HIP_EW_COPY || (b_dev && b_stride), "%s: null second operand", fn);
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
        g.b_stride[i] = op == WEED_HIP_EW_COPY ? 0 : b_stride[i];
        g.o_stride[i] = o_stride[i];
        g.n *= shape[i];
    }
    WEED_HIP_REQUIRE(g.n < (1ull << 32), "%s: more than 2^32 elements", fn);
    ProfileScope prof("elementwise");
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((g.n + 255) / 256, 256u * 64u);
    const float *b = op == WEED_HIP_EW_COPY ? a_dev : b_dev;
    switch (op) {
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

int weed_hip_softmax_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *a_dev, uint32_t a_off,
                         const uint32_t *a_stride, float *out_dev, uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_softmax_f32";
    WEED_HIP_REQUIRE(a_dev && out_dev, "%s: null pointer", fn);
    WEED_HIP_TRY(ensure_init());
    AxisGeom g;
    WEED_HIP_TRY(make_geom(fn, rank, shape, axis, a_off, a_stride, o_off, o_stride, true, g));
    ProfileScope prof("softmax");
    if (g.a_stride[axis] <= 1 || g.rows < 16) {
        softmax_kernel<1><<<g.rows, kThreads, 0, stream()>>>(a_dev, out_dev, g);
    } else {
        softmax_kernel<16><<<(g.rows + 15) / 16, kThreads, 0, stream()>>>(a_dev, out_dev, g);
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
    const bool narrow = g.a_stride[axis] <= 1 || g.rows < 16;
    const uint32_t blocks = narrow ? g.rows : (g.rows + 15) / 16;
#define WEED_LAUNCH_REDUCE(OP)                                                                                         \
    if (narrow) {                                                                                                      \
        reduce_kernel<OP, 1><<<blocks, kThreads, 0, stream()>>>(a_dev, out_dev, g);                                    \
    } else {                                                                                                           \
        reduce_kernel<OP, 16><<<blocks, kThreads, 0, stream()>>>(a_dev, out_dev, g);                                   \
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
