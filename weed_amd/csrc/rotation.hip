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

} // extern "C"
