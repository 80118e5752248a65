// Strided fp32 GEMM: out[M,N] = a[M,K] . b[K,N] with Weed's geometry (offset + two element strides per operand,
// src/ops/matmul.cpp:95-122).  Replaces the OpenCL kernel matmul_real (src/common/qengine.cl:598-640).
#include "common.h"

using namespace weedhip;

namespace {

struct MatGeom {
    uint32_t M, N, K;
    uint32_t a_off, a_s0, a_s1;
    uint32_t b_off, b_s0, b_s1;
    uint32_t o_off, o_s0, o_s1;
};

constexpr int BM = 64, BN = 64, BK = 16;

// Generic tiled kernel on the vector ALU: any shape, any strides.
__global__ void __launch_bounds__(256) matmul_tiled_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          float *__restrict__ out, MatGeom g)
{
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    const uint32_t tid = threadIdx.x;
    const uint32_t tx = tid % 16, ty = tid / 16;
    const uint32_t m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
    float acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < g.K; k0 += BK) {
        for (uint32_t e = tid; e < BM * BK; e += 256) {
            const uint32_t i = e % BM, k = e / BM;
            float v = 0.0f;
            if (m0 + i < g.M && k0 + k < g.K) {
                v = a[(uint64_t)g.a_off + (uint64_t)(m0 + i) * g.a_s0 + (uint64_t)(k0 + k) * g.a_s1];
            }
            As[k][i] = v;
        }
        for (uint32_t e = tid; e < BN * BK; e += 256) {
            const uint32_t k = e % BK, j = e / BK;
            float v = 0.0f;
            if (n0 + j < g.N && k0 + k < g.K) {
                v = b[(uint64_t)g.b_off + (uint64_t)(k0 + k) * g.b_s0 + (uint64_t)(n0 + j) * g.b_s1];
            }
            Bs[k][j] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                av[r] = As[kk][ty * 4 + r];
                bv[r] = Bs[kk][tx * 4 + r];
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[r][c] = fmaf(av[r], bv[c], acc[r][c]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t i = m0 + ty * 4 + r, j = n0 + tx * 4 + c;
            if (i < g.M && j < g.N) {
                out[(uint64_t)g.o_off + (uint64_t)i * g.o_s0 + (uint64_t)j * g.o_s1] = acc[r][c];
            }
        }
    }
}

} // namespace

extern "C" int weed_hip_matmul_f32(uint32_t M, uint32_t N, uint32_t K, const float *a_dev, uint32_t a_off,
                                   uint32_t a_s0, uint32_t a_s1, const float *b_dev, uint32_t b_off, uint32_t b_s0,
                                   uint32_t b_s1, float *out_dev, uint32_t o_off, uint32_t o_s0, uint32_t o_s1)
{
    const char *fn = "weed_hip_matmul_f32";
    WEED_HIP_REQUIRE(a_dev && b_dev && out_dev, "%s: null pointer", fn);
    WEED_HIP_TRY(ensure_init());
    if (!M || !N) {
        return WEED_HIP_OK;
    }
    MatGeom g = { M, N, K, a_off, a_s0, a_s1, b_off, b_s0, b_s1, o_off, o_s0, o_s1 };
    const dim3 grid((M + BM - 1) / BM, (N + BN - 1) / BN);
    WEED_HIP_REQUIRE(grid.y <= 65535u, "%s: N = %u too large", fn, N);
    ProfileScope prof("matmul");
    matmul_tiled_kernel<<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}
