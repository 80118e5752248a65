// Random orthogonal rotation: seeded stand-in for make_random_rotation
// (src/modules/multihead_attention.cpp:84-121).
#include "common.h"

#include <random>
#include <vector>

using namespace weedhip;

namespace {

__device__ __forceinline__ float wave_sum(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_xor(v, o);
    }
    return v;
}

// One workgroup; the matrix stays in device memory (L2).  Column j starts at r[j*d].
// Order of operations as in the reference (cpp:94-118): normalise column j (norm floored at 1e-8), then subtract
// its projection from every later column.  Dot products are tree sums, so results agree to rounding only.
__global__ void __launch_bounds__(256) gram_schmidt_kernel(float *r, uint32_t d)
{
    __shared__ float red[4];
    __shared__ float norm_s;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (uint32_t j = 0; j < d; ++j) {
        float *cj = r + (uint64_t)j * d;
        float part = 0.0f;
        for (uint32_t i = tid; i < d; i += 256) {
            part = fmaf(cj[i], cj[i], part);
        }
        part = wave_sum(part);
        if (lane == 0) {
            red[wave] = part;
        }
        __syncthreads();
        if (tid == 0) {
            float n = sqrtf(red[0] + red[1] + red[2] + red[3]);
            norm_s = n < 1e-8f ? 1e-8f : n;
        }
        __syncthreads();
        const float norm = norm_s;
        for (uint32_t i = tid; i < d; i += 256) {
            cj[i] = cj[i] / norm;
        }
        __threadfence_block();
        __syncthreads();
        for (uint32_t k = j + 1 + wave; k < d; k += 4) {
            float *ck = r + (uint64_t)k * d;
            float dot = 0.0f;
            for (uint32_t i = lane; i < d; i += 64) {
                dot = fmaf(cj[i], ck[i], dot);
            }
            dot = wave_sum(dot);
            for (uint32_t i = lane; i < d; i += 64) {
                ck[i] = ck[i] - dot * cj[i];
            }
        }
        __threadfence_block();
        __syncthreads();
    }
}

constexpr int kRotMaxRank = 8;
struct RotGeom {
    uint32_t rank; // the last dimension is the rotated one
    uint32_t shape[kRotMaxRank];
    uint32_t x_stride[kRotMaxRank];
    uint32_t o_stride[kRotMaxRank];
    uint32_t x_off, o_off;
    uint32_t rows, d;
};

constexpr int kRotOutputs = 16; // outputs per thread: one pass over a row of x serves this many columns of R
constexpr int kRotBatch = 4; // contraction steps per batch of loads

// y[row, j] = sum_i x[row, i] * R[i + d*j], products added in ascending i with separate multiply and add, the order
// of the reference's naive matmul (src/ops/matmul.cpp:40-44).  Neighbouring threads take neighbouring rows (the
// contiguous direction of a column-major tensor) and share kRotOutputs columns of R, so x loads coalesce, R loads
// are wave-uniform and x is read d / kRotOutputs times instead of d times.
__global__ void __launch_bounds__(256) apply_rotation_kernel(const float *__restrict__ x, const float *__restrict__ rot,
                                                             float *__restrict__ out, RotGeom g)
{
    const uint32_t row = blockIdx.x * 256 + threadIdx.x;
    const uint32_t j0 = blockIdx.y * kRotOutputs;
    if (row >= g.rows) {
        return;
    }
    uint64_t xb = g.x_off, ob = g.o_off;
    uint32_t tmp = row;
    for (uint32_t dd = 0; dd + 1 < g.rank; ++dd) {
        const uint32_t c = tmp % g.shape[dd];
        tmp /= g.shape[dd];
        xb += (uint64_t)c * g.x_stride[dd];
        ob += (uint64_t)c * g.o_stride[dd];
    }
    const uint32_t d = g.d;
    const uint32_t xs = g.x_stride[g.rank - 1];
    const float *xp = x + xb;
    // every accumulator adds its products in the order i = 0, 1, ..., d - 1 with separately rounded products; the
    // columns of R are addressed by workgroup-wide values, so they travel through the scalar data path
    float acc[kRotOutputs];
#pragma unroll
    for (int jj = 0; jj < kRotOutputs; ++jj) {
        acc[jj] = 0.0f;
    }
    uint32_t i = 0;
    for (; i + kRotBatch <= d; i += kRotBatch) {
        float xv[kRotBatch];
#pragma unroll
        for (int u = 0; u < kRotBatch; ++u) {
            xv[u] = xp[(uint64_t)(i + u) * xs];
        }
#pragma unroll
        for (int jj = 0; jj < kRotOutputs; ++jj) {
            const uint32_t j = min(j0 + (uint32_t)jj, d - 1U);
            const float *col = rot + (uint64_t)j * d + i;
#pragma unroll
            for (int u = 0; u < kRotBatch; ++u) {
                acc[jj] = acc[jj] + xv[u] * col[u];
            }
        }
    }
    for (; i < d; ++i) {
        const float xv = xp[(uint64_t)i * xs];
#pragma unroll
        for (int jj = 0; jj < kRotOutputs; ++jj) {
            const uint32_t j = min(j0 + (uint32_t)jj, d - 1U);
            acc[jj] = acc[jj] + xv * rot[(uint64_t)j * d + i];
        }
    }
    const uint32_t os = g.o_stride[g.rank - 1];
#pragma unroll
    for (int jj = 0; jj < kRotOutputs; ++jj) {
        if (j0 + jj < d) {
            out[ob + (uint64_t)(j0 + jj) * os] = acc[jj];
        }
    }
}

// The same sums for head-sized d (d <= kRotTiledMaxD) with every global access coalesced whatever the two layouts:
// a workgroup stages 64 rows of x in LDS (walking x along whichever of its directions is contiguous), wavefront w
// computes the column chunks w, w + 4, ... for all 64 rows (x from LDS, R through the scalar path, every sum in
// ascending i with separately rounded products, as above) and writes them along the contiguous direction of `out`
// (through a per-wavefront LDS patch when that is the rotated dimension itself).
constexpr int kRotTileRows = 64;
constexpr int kRotTiledMaxD = 128;
constexpr int kRotPitch = kRotTileRows + 1;

__global__ void __launch_bounds__(256) apply_rotation_tiled_kernel(const float *__restrict__ x,
                                                                   const float *__restrict__ rot,
                                                                   float *__restrict__ out, RotGeom g)
{
    __shared__ float tile[kRotTiledMaxD * kRotPitch];
    __shared__ float patch[4][kRotOutputs * kRotPitch];
    __shared__ uint64_t xbase[kRotTileRows], obase[kRotTileRows];
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = blockIdx.x * kRotTileRows;
    const uint32_t nrows = min((uint32_t)kRotTileRows, g.rows - row0);
    if (tid < nrows) {
        uint64_t xb = g.x_off, ob = g.o_off;
        uint32_t tmp = row0 + tid;
        for (uint32_t dd = 0; dd + 1 < g.rank; ++dd) {
            const uint32_t c = tmp % g.shape[dd];
            tmp /= g.shape[dd];
            xb += (uint64_t)c * g.x_stride[dd];
            ob += (uint64_t)c * g.o_stride[dd];
        }
        xbase[tid] = xb;
        obase[tid] = ob;
    }
    __syncthreads();
    const uint32_t d = g.d;
    const uint32_t xs = g.x_stride[g.rank - 1], os = g.o_stride[g.rank - 1];
    if (xs == 1U) {
        // rows of x are contiguous: neighbouring threads take neighbouring i
#pragma unroll 4
        for (uint32_t e = tid; e < kRotTileRows * d; e += 256) {
            const uint32_t r = e / d, i = e - r * d;
            if (r < nrows) {
                tile[i * kRotPitch + r] = x[xbase[r] + i];
            }
        }
    } else {
#pragma unroll 4
        for (uint32_t e = tid; e < kRotTileRows * d; e += 256) {
            const uint32_t r = e % kRotTileRows, i = e / kRotTileRows;
            if (r < nrows) {
                tile[i * kRotPitch + r] = x[xbase[r] + (uint64_t)i * xs];
            }
        }
    }
    __syncthreads();
    const uint32_t r = tid % kRotTileRows;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kRotTileRows);
    for (uint32_t j0 = wave * kRotOutputs; j0 < d; j0 += 4 * kRotOutputs) {
        float acc[kRotOutputs];
#pragma unroll
        for (int jj = 0; jj < kRotOutputs; ++jj) {
            acc[jj] = 0.0f;
        }
        uint32_t i = 0;
        for (; i + kRotBatch <= d; i += kRotBatch) {
            float xv[kRotBatch];
#pragma unroll
            for (int u = 0; u < kRotBatch; ++u) {
                xv[u] = tile[(i + u) * kRotPitch + r];
            }
#pragma unroll
            for (int jj = 0; jj < kRotOutputs; ++jj) {
                const uint32_t j = min(j0 + (uint32_t)jj, d - 1U);
                const float *col = rot + (uint64_t)j * d + i;
#pragma unroll
                for (int u = 0; u < kRotBatch; ++u) {
                    acc[jj] = acc[jj] + xv[u] * col[u];
                }
            }
        }
        for (; i < d; ++i) {
            const float xv = tile[i * kRotPitch + r];
#pragma unroll
            for (int jj = 0; jj < kRotOutputs; ++jj) {
                const uint32_t j = min(j0 + (uint32_t)jj, d - 1U);
                acc[jj] = acc[jj] + xv * rot[(uint64_t)j * d + i];
            }
        }
        if (os == 1U) {
            // rows of out are contiguous: turn the 64 x 16 patch so that neighbouring lanes write neighbouring j
            float *mine = patch[wave];
#pragma unroll
            for (int jj = 0; jj < kRotOutputs; ++jj) {
                mine[jj * kRotPitch + r] = acc[jj];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll 4
            for (uint32_t e = r; e < kRotTileRows * kRotOutputs; e += kRotTileRows) {
                const uint32_t jj = e % kRotOutputs, rr = e / kRotOutputs;
                if (rr < nrows && j0 + jj < d) {
                    out[obase[rr] + j0 + jj] = mine[jj * kRotPitch + rr];
                }
            }
            __builtin_amdgcn_wave_barrier();
        } else if (r < nrows) {
#pragma unroll
            for (int jj = 0; jj < kRotOutputs; ++jj) {
                if (j0 + jj < d) {
                    out[obase[r] + (uint64_t)(j0 + jj) * os] = acc[jj];
                }
            }
        }
    }
}

} // namespace

extern "C" {

int weed_hip_orthonormalize_columns(uint32_t d, float *r_dev)
{
    WEED_HIP_REQUIRE(r_dev, "weed_hip_orthonormalize_columns: null pointer");
    WEED_HIP_REQUIRE(d >= 1 && d <= 4096, "weed_hip_orthonormalize_columns: d = %u outside [1, 4096]", d);
    WEED_HIP_TRY(ensure_init());
    gram_schmidt_kernel<<<1, 256, 0, stream()>>>(r_dev, d);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

int weed_hip_make_rotation(uint32_t seed, uint32_t d, float *r_dev)
{
    WEED_HIP_REQUIRE(r_dev, "weed_hip_make_rotation: null pointer");
    WEED_HIP_REQUIRE(d >= 1 && d <= 4096, "weed_hip_make_rotation: d = %u outside [1, 4096]", d);
    WEED_HIP_TRY(ensure_init());
    // cpp:85-92: std::mt19937 + std::normal_distribution<real1>(0, 1), filled in storage (column-major) order;
    // the reference seeds from std::random_device, here the caller supplies the seed.
    std::mt19937 rng(seed);
    std::normal_distribution<float> normal(0.0f, 1.0f);
    std::vector<float> host((size_t)d * d);
    for (float &v : host) {
        v = normal(rng);
    }
    WEED_HIP_CHECK(hipMemcpyAsync(r_dev, host.data(), sizeof(float) * host.size(), hipMemcpyHostToDevice, stream()));
    WEED_HIP_CHECK(hipStreamSynchronize(stream()));
    return weed_hip_orthonormalize_columns(d, r_dev);
}

int weed_hip_apply_rotation_f32(uint32_t d, const float *r_dev, uint32_t rank, const uint32_t *shape,
                                const float *x_dev, uint32_t x_off, const uint32_t *x_stride, float *out_dev,
                                uint32_t o_off, const uint32_t *o_stride)
{
    const char *fn = "weed_hip_apply_rotation_f32";
    WEED_HIP_REQUIRE(r_dev && x_dev && out_dev && shape && x_stride && o_stride, "%s: null pointer", fn);
    WEED_HIP_REQUIRE(x_dev != out_dev, "%s: cannot rotate in place", fn);
    WEED_HIP_REQUIRE(rank >= 1 && rank <= (uint32_t)kRotMaxRank, "%s: rank %u outside [1, %d]", fn, rank, kRotMaxRank);
    WEED_HIP_REQUIRE(d >= 1 && d <= 65535 && shape[rank - 1] == d, "%s: the last dimension must be d = %u", fn, d);
    WEED_HIP_TRY(ensure_init());
    RotGeom g;
    g.rank = rank;
    g.d = d;
    g.x_off = x_off;
    g.o_off = o_off;
    uint64_t rows = 1;
    for (uint32_t i = 0; i < rank; ++i) {
        WEED_HIP_REQUIRE(shape[i] > 0, "%s: dimension %u is empty", fn, i);
        g.shape[i] = shape[i];
        g.x_stride[i] = x_stride[i];
        g.o_stride[i] = o_stride[i];
        if (i + 1 < rank) {
            rows *= shape[i];
        }
    }
    WEED_HIP_REQUIRE(rows * d < (1ull << 32), "%s: more than 2^32 elements", fn);
    g.rows = (uint32_t)rows;
    // the LDS-tiled kernel pays off when the rotated dimension is the contiguous one on either side; with both sides
    // contiguous along the rows (Weed's column-major tensors) the register-only kernel is already coalesced and faster
    const bool rows_contiguous = g.x_stride[rank - 1] != 1U && g.o_stride[rank - 1] != 1U;
    if (d <= (uint32_t)kRotTiledMaxD && !rows_contiguous) {
        apply_rotation_tiled_kernel<<<(g.rows + kRotTileRows - 1) / kRotTileRows, 256, 0, stream()>>>(x_dev, r_dev, out_dev,
                                                                                                     g);
        WEED_HIP_LAUNCH_CHECK();
        return WEED_HIP_OK;
    }
    apply_rotation_kernel<<<dim3((g.rows + 255) / 256, (d + kRotOutputs - 1) / kRotOutputs), 256, 0, stream()>>>(x_dev, r_dev, out_dev, g);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // extern "C"
