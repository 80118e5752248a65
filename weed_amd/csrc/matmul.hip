// Strided fp32 GEMM: out[M,N] = a[M,K] . b[K,N] with Weed's geometry (offset + two element strides per operand,
// src/ops/matmul.cpp:95-122).  Replaces the OpenCL kernel matmul_real (src/common/qengine.cl:598-640).
#include "common.h"

#include <atomic>
#include <cstdlib>
#include <cmath>
#include <algorithm>
#include <type_traits>

using namespace weedhip;

namespace {

struct MatGeom {
    uint32_t M, N, K;
    uint32_t a_off, a_s0, a_s1;
    uint32_t b_off, b_s0, b_s1;
    uint32_t o_off, o_s0, o_s1;
    // batched products: grid.z = nb0 * nb1 independent products, product (c0, c1) starts at off + c0*bs[0] + c1*bs[1]
    uint32_t nb0;
    uint32_t a_bs[2], b_bs[2], o_bs[2];
    // optional row vector added to every row of the product after the sum is rounded (null: none), so the result
    // equals a product followed by a broadcast add, bit for bit
    const float *bias;
    uint32_t bias_off, bias_s;
};

__device__ __forceinline__ float with_bias(const MatGeom &g, float v, uint32_t col)
{
    return g.bias ? v + g.bias[(uint64_t)g.bias_off + (uint64_t)col * g.bias_s] : v;
}

// The geometry of the product this workgroup belongs to (blockIdx.z selects it).
__device__ __forceinline__ MatGeom batch_geom(MatGeom g)
{
    const uint32_t c0 = blockIdx.z % g.nb0, c1 = blockIdx.z / g.nb0;
    g.a_off += c0 * g.a_bs[0] + c1 * g.a_bs[1];
    g.b_off += c0 * g.b_bs[0] + c1 * g.b_bs[1];
    g.o_off += c0 * g.o_bs[0] + c1 * g.o_bs[1];
    return g;
}

constexpr int BM = 64, BN = 64, BK = 16;

// Generic tiled kernel on the vector ALU: any shape, any strides.
__global__ void __launch_bounds__(256) matmul_tiled_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          float *__restrict__ out, MatGeom g_launch)
{
    const MatGeom g = batch_geom(g_launch);
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
                out[(uint64_t)g.o_off + (uint64_t)i * g.o_s0 + (uint64_t)j * g.o_s1] = with_bias(g, acc[r][c], j);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Matrix-core kernel: v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate; products are exact to fp32 rounding).
//   workgroup = 4 wavefronts, output tile 128 x 128, each wavefront a 64 x 64 quadrant = 2 x 2 instructions tiles;
//   K is walked in slices of 16 staged through double-buffered LDS ([k][i] and [k][j], so a half-wavefront reads 32
//   consecutive floats); the next slice is fetched from HBM into registers while the current one is multiplied.
// Each operand must be contiguous along one of its two dimensions (Weed's column-major tensors and their transposes
// are); the four combinations are template instances.  Shapes that are not multiples of the tile, operands strided
// in both dimensions and unaligned views use the EDGE instances: the same tiles and instructions, with element-wise
// guarded loads (zeros beyond the edges) and guarded stores; there the two flags only choose which way the threads
// walk an operand.  Sizes that are not multiples of the tile in the unguarded kernel's layout (contiguous dimensions
// of a multiple of 4 elements, 16-byte aligned) use the QUAD instances: the unguarded kernel's 16-byte loads, each
// checked as a whole.  Products with fewer than 17 rows or columns use the generic kernel above.
// ------------------------------------------------------------------------------------------------
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int TM = 128, TN = 128, TK = 16, PITCH = 132;

template <bool A_ICONTIG, bool B_KCONTIG, int GUARD = 0, bool SPLIT = GUARD == 1>
__global__ void __launch_bounds__(256) matmul_mfma_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          float *__restrict__ out, MatGeom g_launch,
                                                          uint32_t k_per_split = 0)
{
    // GUARD: 0 whole tiles, nothing checked; 1 (EDGE) any shape and strides, element by element; 2 (QUAD) the layout of
    // 0 -- one contiguous dimension per operand, 16-byte aligned, its extent a multiple of 4 -- with sizes that are not
    // multiples of the tile: 16-byte loads, each checked as a whole.
    constexpr bool EDGE = GUARD == 1, QUAD = GUARD == 2;
    // EDGE and SPLIT instances may split k over blockIdx.z (unbatched products only, so batch_geom adds nothing then):
    // k_per_split != 0 means `out` is the dense scratch part[split][row][column] and a second kernel adds the splits
    MatGeom g = batch_geom(g_launch);
    const uint32_t k_first = (SPLIT && k_per_split) ? blockIdx.z * k_per_split : 0U;
    if (SPLIT && k_per_split) {
        g.K = min(g.K, k_first + k_per_split);
    }
    // Row pitch of a staged slice.  An operand that arrives contiguous along its own index is stored with 16-byte
    // writes (pitch 132: a multiple of 4).  One that arrives contiguous along k is stored transposed, element by
    // element: thread (k4, j) writes rows 4 k4 .. 4 k4 + 3 of column j, and with pitch 130 the four k4 of 32
    // neighbouring threads start 8 banks apart, so their writes hit 32 different banks (with 132 they pair up).
    constexpr int PITCH_A = A_ICONTIG ? PITCH : PITCH - 2, PITCH_B = B_KCONTIG ? PITCH - 2 : PITCH;
    __shared__ __attribute__((aligned(16))) float As[2][TK][PITCH_A];
    __shared__ __attribute__((aligned(16))) float Bs[2][TK][PITCH_B];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wi = wave >> 1, wj = wave & 1;
    const uint32_t m0 = blockIdx.x * TM, n0 = blockIdx.y * TN;
    const uint32_t l32 = lane & 31, lk = lane >> 5;

    float16v acc[2][2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
#pragma unroll
        for (int y = 0; y < 2; ++y) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[x][y][r] = 0.0f;
            }
        }
    }

    // two float4 per operand per thread and K slice
    // (Guarded loads sit in branches of their own.  Issuing every load from an address clamped into the operand
    // instead was measured twice and was slower both times: zeroed right behind the load, 1000 x 4099 x 4096 took 1076
    // us against 488; with a bit per load kept and the zeroing left to the staging, a slice later, 543.)
    float4v ra[2], rb[2];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t idx = tid + 256 * q;
            if (EDGE) {
                // any shape, any strides: element-wise loads, zeros beyond the edges (they add nothing to the sums)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t ai = A_ICONTIG ? m0 + 4 * (idx & 31) + e : m0 + (idx >> 2);
                    const uint32_t ak = A_ICONTIG ? k0 + (idx >> 5) : k0 + 4 * (idx & 3) + e;
                    ra[q][e] = (ai < g.M && ak < g.K)
                        ? a[(uint64_t)g.a_off + (uint64_t)ai * g.a_s0 + (uint64_t)ak * g.a_s1]
                        : 0.0f;
                    const uint32_t bj = B_KCONTIG ? n0 + (idx >> 2) : n0 + 4 * (idx & 31) + e;
                    const uint32_t bk = B_KCONTIG ? k0 + 4 * (idx & 3) + e : k0 + (idx >> 5);
                    rb[q][e] = (bj < g.N && bk < g.K)
                        ? b[(uint64_t)g.b_off + (uint64_t)bk * g.b_s0 + (uint64_t)bj * g.b_s1]
                        : 0.0f;
                }
                continue;
            }
            const float4v zero4 = { 0.0f, 0.0f, 0.0f, 0.0f }; // (QUAD: each 16-byte load checked as a whole)
            if (A_ICONTIG) {
                const uint32_t i4 = idx & 31, k = idx >> 5;
                const bool in = !QUAD || (m0 + 4 * i4 < g.M && k0 + k < g.K);
                ra[q] = in ? *reinterpret_cast<const float4v *>(a + (uint64_t)g.a_off + (m0 + 4 * i4) +
                                                                (uint64_t)(k0 + k) * g.a_s1)
                           : zero4;
            } else {
                const uint32_t k4 = idx & 3, i = idx >> 2;
                const bool in = !QUAD || (m0 + i < g.M && k0 + 4 * k4 < g.K);
                ra[q] = in ? *reinterpret_cast<const float4v *>(a + (uint64_t)g.a_off + (uint64_t)(m0 + i) * g.a_s0 +
                                                                (k0 + 4 * k4))
                           : zero4;
            }
            if (B_KCONTIG) {
                const uint32_t k4 = idx & 3, j = idx >> 2;
                const bool in = !QUAD || (n0 + j < g.N && k0 + 4 * k4 < g.K);
                rb[q] = in ? *reinterpret_cast<const float4v *>(b + (uint64_t)g.b_off + (k0 + 4 * k4) +
                                                                (uint64_t)(n0 + j) * g.b_s1)
                           : zero4;
            } else {
                const uint32_t j4 = idx & 31, k = idx >> 5;
                const bool in = !QUAD || (n0 + 4 * j4 < g.N && k0 + k < g.K);
                rb[q] = in ? *reinterpret_cast<const float4v *>(b + (uint64_t)g.b_off + (uint64_t)(k0 + k) * g.b_s0 +
                                                                (n0 + 4 * j4))
                           : zero4;
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t idx = tid + 256 * q;
            if (A_ICONTIG) {
                const uint32_t i4 = idx & 31, k = idx >> 5;
                *reinterpret_cast<float4v *>(&As[buf][k][4 * i4]) = ra[q];
            } else {
                const uint32_t k4 = idx & 3, i = idx >> 2;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    As[buf][4 * k4 + x][i] = ra[q][x];
                }
            }
            if (B_KCONTIG) {
                const uint32_t k4 = idx & 3, j = idx >> 2;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    Bs[buf][4 * k4 + x][j] = rb[q][x];
                }
            } else {
                const uint32_t j4 = idx & 31, k = idx >> 5;
                *reinterpret_cast<float4v *>(&Bs[buf][k][4 * j4]) = rb[q];
            }
        }
    };

    const uint32_t n_slices = (g.K - k_first + TK - 1) / TK;
    fetch(k_first);
    stage(0);
    __syncthreads();
    for (uint32_t kt = 0; kt < n_slices; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < n_slices) {
            fetch(k_first + (kt + 1) * TK);
        }
#pragma unroll
        for (int kk = 0; kk < TK; kk += 2) {
            const float a0 = As[buf][kk + lk][64 * wi + l32];
            const float a1 = As[buf][kk + lk][64 * wi + 32 + l32];
            const float b0 = Bs[buf][kk + lk][64 * wj + l32];
            const float b1 = Bs[buf][kk + lk][64 * wj + 32 + l32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        if (kt + 1 < n_slices) {
            stage(buf ^ 1);
        }
        __syncthreads();
    }

    // register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32 x 32 tile
#pragma unroll
    for (int x = 0; x < 2; ++x) {
#pragma unroll
        for (int y = 0; y < 2; ++y) {
            const uint32_t col = n0 + 64 * wj + 32 * y + l32;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const uint32_t row = m0 + 64 * wi + 32 * x + 8 * r4 + 4 * lk;
                float *dst = out + (uint64_t)g.o_off + (uint64_t)row * g.o_s0 + (uint64_t)col * g.o_s1;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = (GUARD == 0 || col < g.N) ? with_bias(g, acc[x][y][4 * r4 + e], col) : 0.0f;
                }
                if (SPLIT && k_per_split) {
                    float *part = out + ((uint64_t)blockIdx.z * g.M + row) * g.N + col;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (row + e < g.M && col < g.N) {
                            part[(uint64_t)e * g.N] = acc[x][y][4 * r4 + e];
                        }
                    }
                } else if (EDGE || (QUAD && (g.o_s0 != 1 || row + 3 >= g.M))) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (row + e < g.M && col < g.N) {
                            dst[(uint64_t)e * g.o_s0] = v[e];
                        }
                    }
                } else if (QUAD) {
                    if (col < g.N) {
                        *reinterpret_cast<float4v *>(dst) = float4v{ v[0], v[1], v[2], v[3] };
                    }
                } else if (g.o_s0 == 1) {
                    *reinterpret_cast<float4v *>(dst) = float4v{ v[0], v[1], v[2], v[3] };
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dst[(uint64_t)e * g.o_s0] = v[e];
                    }
                }
            }
        }
    }
}


// ---- "Skinny" products: few rows (M <= 64) against a tall weight matrix whose columns are contiguous along k -- the
//      decode-time projections y = x.W of the attention module (src/modules/linear.cpp:86-100 with x = [B, d_model]).
//      The time is the time to stream W once from HBM, so W is read with 16-byte loads along k, every element once.
//
//      A workgroup of 8 wavefronts owns 16 output columns; wavefront w takes the k range [w*k_per_wave, (w+1)*...).
//      The products run on v_mfma_f32_16x16x4f32 (16 rows x 16 columns x 4 k per instruction).  The contraction
//      index of an instruction may be any four k as long as both operands agree, so lane (column c = l % 16,
//      group g = l / 16) keeps the k  kb + 16 q + 4 g .. + 3  (q = 0..3) of its column -- four 16-byte loads, each of
//      which reads 64 consecutive bytes per column across the four groups -- and instruction j = 4 q + i of an
//      iteration contracts over  { kb + 16 q + 4 g + i : g = 0..3 }.  The few rows of `a`
//      come from L2 (every workgroup reads all of them).  The eight partial tiles of a workgroup are added in LDS.
constexpr int kSkinnyWaves = 8;

template <int I, int N, typename F> __device__ __forceinline__ void static_for_sets(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_sets<I + 1, N>(f);
    }
}

template <int MT> // 16-row tiles of a: M <= 16 * MT
__global__ void __launch_bounds__(64 * kSkinnyWaves)
    matmul_skinny_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out,
                         MatGeom g_launch, uint32_t k_per_wave)
{
    const MatGeom g = batch_geom(g_launch);
    typedef float float4v __attribute__((ext_vector_type(4)));
    __shared__ float red[kSkinnyWaves][MT][256];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 15, grp = lane >> 4;
    const uint32_t n = blockIdx.x * 16 + c;
    const bool n_ok = n < g.N;
    const float *wcol = b + (uint64_t)g.b_off + (uint64_t)(n_ok ? n : 0) * g.b_s1; // b_s0 == 1: k contiguous
    const uint32_t kb0 = wave * k_per_wave;
    const uint32_t kb1 = min(kb0 + k_per_wave, g.K);
    float4v acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        acc[mt] = float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
    }
    // sixteen consecutive k of this lane's column, zero beyond the range (K is a multiple of 4: whole 16-byte loads)
    auto load_w = [&](uint32_t kb, float4v (&w)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t k = kb + 16 * q + 4 * grp; // the four lanes of a column read 64 consecutive bytes
            w[q] = (n_ok && k < kb1) ? *reinterpret_cast<const float4v *>(wcol + k) : float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
        }
    };
    // the rows of a that go with them, for row tiles mt0 and mt0 + 1 (or mt0 alone): a[16 mt + c][kb + 16 grp + j]
    constexpr int TA = MT >= 2 ? 2 : 1; // row tiles fetched and multiplied together
    auto load_a = [&](uint32_t kb, int mt0, float (&av)[TA][16]) {
#pragma unroll
        for (int t = 0; t < TA; ++t) {
            const uint32_t m = 16 * (mt0 + t) + c;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const uint32_t k = kb + 16 * (j / 4) + 4 * grp + (j % 4); // as the lane's element j of b
                av[t][j] = (m < g.M && k < kb1)
                    ? a[(uint64_t)g.a_off + (uint64_t)m * g.a_s0 + (uint64_t)k * g.a_s1] : 0.0f;
            }
        }
    };
    // Register sets in a ring: the operands of the next kAhead iterations travel while this one is multiplied.  With
    // one or two row tiles both operands are fetched ahead; with four only the columns of b are, and the rows of a
    // (which come from L2) are fetched pair by pair when needed.
    constexpr bool kPrefetchA = MT <= 2;
    constexpr int kAhead = 1; // more sets did not pay: a wavefront only runs a handful of iterations
    constexpr int kSets = kAhead + 1;
    float4v w[kSets][4];
    float av[kPrefetchA ? kSets : 1][TA][16];
    auto iterate = [&](auto pc, uint32_t kb) {
        constexpr int P = decltype(pc)::value;
        constexpr int Q = (P + kAhead) % kSets; // the set that was used last iteration is free again
        load_w(kb + 64 * kAhead, w[Q]);
        if constexpr (kPrefetchA) {
            load_a(kb + 64 * kAhead, 0, av[Q]);
#pragma unroll
            for (int j = 0; j < 16; ++j) {
#pragma unroll
                for (int t = 0; t < TA; ++t) {
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[P][t][j], w[P][j / 4][j % 4], acc[t], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int mt0 = 0; mt0 < MT; mt0 += TA) {
                load_a(kb, mt0, av[0]);
#pragma unroll
                for (int j = 0; j < 16; ++j) {
#pragma unroll
                    for (int t = 0; t < TA; ++t) {
                        acc[mt0 + t] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][t][j], w[P][j / 4][j % 4], acc[mt0 + t], 0, 0, 0);
                    }
                }
            }
        }
    };
    if (kb0 < kb1) {
        static_for_sets<0, kAhead>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            load_w(kb0 + 64 * i, w[i]);
            if constexpr (kPrefetchA) {
                load_a(kb0 + 64 * i, 0, av[i]);
            }
        });
        uint32_t kb = kb0;
        while (kb < kb1) {
            // kSets iterations per round so that the set indices are compile-time constants
            static_for_sets<0, kSets>([&](auto ic) {
                if (kb < kb1) {
                    iterate(ic, kb);
                    kb += 64;
                }
            });
        }
    }
    // lane (c, grp), register v of a tile: row 4 * grp + v, column c
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            red[wave][mt][(4 * grp + v) * 16 + c] = acc[mt][v];
        }
    }
    __syncthreads();
    for (uint32_t e = tid; e < (uint32_t)MT * 256; e += 64 * kSkinnyWaves) {
        const uint32_t mt = e >> 8, r = (e >> 4) & 15, cc = e & 15;
        float sum = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kSkinnyWaves; ++wv) {
            sum += red[wv][mt][r * 16 + cc];
        }
        const uint32_t m = 16 * mt + r, nn = blockIdx.x * 16 + cc;
        if (m < g.M && nn < g.N) {
            out[(uint64_t)g.o_off + (uint64_t)m * g.o_s0 + (uint64_t)nn * g.o_s1] = with_bias(g, sum, nn);
        }
    }
}


// ---- Seventeen to 64 rows: the same streaming of b, but at this many rows the fp32 matrix instruction would bound
//      the product (128 flop per byte of b against the part's 20), and the rows of a no longer come cheaply from L2 if
//      every 16-column workgroup reads all of them.  So the products run on the bfloat16 matrix instruction
//      v_mfma_f32_16x16x32_bf16 (sixteen times the fp32 rate) with BOTH operands split exactly into three bfloat16
//      parts: a float's 24-bit significand is three 8-bit pieces, x = x1 + x2 + x3 with every part a bfloat16, so
//      x.w is the sum of nine exact products of which the six with i + j <= 4 carry everything above 2^-24 of the
//      result; they accumulate in fp32 inside the instruction.  The outcome has the quality of an fp32 product
//      (measured: error below 1.2e-7 of the sum of the terms' magnitudes), not the bits of a sequential fp32 sum.
//      A workgroup owns 128 columns (16 per wavefront); all its wavefronts walk the same k range and share the rows
//      of `a`, which the workgroup splits step by step into LDS ([part][row][k], rows padded to 144 bytes so that
//      sixteen rows' 16-byte reads cover all banks once; two buffers, one barrier per 64-k step); the k ranges are
//      split over gridDim.y workgroups whose partial results a small kernel behind adds up in a fixed order.
//      64 rows, back to back on one weight (which the 256 MB memory-side cache then holds in part): 4096 x 4096
//      weights 39 -> 33 us per product, 4096 x 14336 125 -> 76 us, 14336 x 4096 105 -> 72 us.  Over four 4096 x 14336
//      weights in turn, so that every product reads HBM: 94 us, then 82 with the two changes noted at load_w and
//      in iterate() below (whole cache lines per load instruction; the rows requested ahead of the columns).
//      Counters: matrix pipe 27 % busy, vector issue 41 % (the splits), LDS 34 %, wavefronts waiting for memory 35 %
//      of their time: nothing is saturated, the phases of a step follow each other in every wavefront.
//      Measured and dropped: the rows split once by a kernel ahead and copied into LDS as an image (more L2 traffic
//      than the fp32 rows: 84 us), two column tiles per wavefront (72 us), sixteen wavefronts per workgroup (78 us),
//      four wavefronts per workgroup (73 us), three or four register sets of b instead of two (86 and 101 us against
//      82), 224 to 896 workgroups instead of about 448 (87 to 94 us), the sum over the k ranges by the last
//      workgroup of a column tile instead of a kernel behind (32 workgroups then read 458 KB each at the very end:
//      a layer's seven products 416 -> 731 us).
constexpr int kWideWaves = 8;
constexpr int kWidePitchH = 72; // halves per staged row: 64 k + 8 of padding

typedef uint32_t uint4w __attribute__((ext_vector_type(4)));
typedef uint32_t uint2w __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// w = p1 + p2 + p3 exactly, every part a bfloat16 (the upper halves of the returned words): w rounded to 8 significant
// bits, what is left rounded to 8 bits, and the rest (at most 8 bits).  Rounding to nearest (ties away from zero: half a
// unit added to the bits before they are cut) keeps the second part below 2^-8 and the third below 2^-16 of w, so the
// three products of parts that the kernels leave out stay below 2^-23 of a term; cutting the bits instead would let
// them reach 2^-21, and all with the term's sign.  (|w| within 2^-9 of the largest float rounds up to infinity.)
__device__ __forceinline__ void split_bf16x3(float w, uint32_t &p1, uint32_t &p2, uint32_t &p3)
{
    p1 = (__float_as_uint(w) + 0x8000u) & 0xffff0000u;
    const float r1 = w - __uint_as_float(p1);
    p2 = (__float_as_uint(r1) + 0x8000u) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(p2);
    p3 = __float_as_uint(r2);
}
// the upper halves of (lo, hi) as one word, `lo` in the low half
__device__ __forceinline__ uint32_t pack_upper_halves(uint32_t lo, uint32_t hi)
{
    return __builtin_amdgcn_perm(hi, lo, 0x07060302u);
}
// eight consecutive values -> three operands of the matrix instruction (one per part)
__device__ __forceinline__ void split_eight(const float (&v)[8], uint4w (&part)[3])
{
    uint32_t p[3][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        split_bf16x3(v[e], p[0][e], p[1][e], p[2][e]);
    }
#pragma unroll
    for (int pl = 0; pl < 3; ++pl) {
        part[pl] = uint4w{ pack_upper_halves(p[pl][0], p[pl][1]), pack_upper_halves(p[pl][2], p[pl][3]),
                           pack_upper_halves(p[pl][4], p[pl][5]), pack_upper_halves(p[pl][6], p[pl][7]) };
    }
}

template <int MT, bool AK = false> // AK: the rows of a are contiguous along k (a_s1 == 1), 16-byte aligned
__global__ void __launch_bounds__(64 * kWideWaves)
    matmul_skinny_wide_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ part,
                              MatGeom g, uint32_t k_per_split)
{
    typedef float float4v __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint16_t xs[2][3][16 * MT][kWidePitchH];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 15, grp = lane >> 4;
    const uint32_t n = blockIdx.x * (16 * kWideWaves) + wave * 16 + c;
    const bool n_ok = n < g.N;
    const float *wcol = b + (uint64_t)g.b_off + (uint64_t)(n_ok ? n : 0) * g.b_s1;
    const uint32_t kb0 = blockIdx.y * k_per_split;
    const uint32_t kb1 = min(kb0 + k_per_split, g.K);
    float4v acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        acc[mt] = float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
    }
    // Sixteen k of this lane's column per 64-k step, zero beyond the range (K is a multiple of 4): load q takes
    // kb + 16 q + 4 grp .. + 3, so that the four lanes of a column read 64 consecutive bytes per instruction and every
    // cache line a load touches is used up by that load (with the lane's sixteen k consecutive, each of the four
    // loads touched every line of the step, and the lines had to survive in the first-level cache between them).
    auto load_w = [&](uint32_t kb, float4v (&w)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t k = kb + 16 * q + 4 * grp;
            w[q] = (n_ok && k < kb1) ? *reinterpret_cast<const float4v *>(wcol + k) : float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
        }
    };
    // the rows of a for one 64-k step: thread (row = tid % (16 MT), octet = tid / (16 MT)) fetches a[row][kb + 8 octet
    // .. + 7], splits the eight values and stores two 8-byte pieces per part.  A row lies in LDS in the order in which
    // the matrix instructions contract: instruction j of a step contracts, in lane group grp, over the k
    // 32 j + 4 grp .. + 3 and 32 j + 16 + 4 grp .. + 3 (what the lane's loads 2 j and 2 j + 1 of b hold), so k =
    // 32 j + 16 h + 4 grp + e sits at position 32 j + 8 grp + 4 h + e and a lane's eight values are one 16-byte read.
    // (With rows that are contiguous along k the eight lanes of a row's octets are neighbours and fetch 256 consecutive
    // bytes with two 16-byte loads each; else the lanes of an octet are 64 neighbouring rows, eight 4-byte loads each.)
    constexpr uint32_t kRows = 16 * MT;
    const uint32_t srow = AK ? tid / 8 : tid % kRows, soct = AK ? tid % 8 : tid / kRows;
    const bool stager = AK ? srow < kRows : soct < 8;
    const float *arow = a + (uint64_t)g.a_off + (uint64_t)(srow < g.M ? srow : 0) * g.a_s0;
    auto fetch_rows = [&](uint32_t kb, float (&v)[8]) {
        if constexpr (AK) {
            const uint32_t k = kb + 8 * soct;
            const bool ok = stager && srow < g.M && k < kb1; // (K is a multiple of 4; a range ends on a multiple of 64 or at K)
            const float4v lo = ok ? *reinterpret_cast<const float4v *>(arow + k) : float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
            const float4v hi = (ok && k + 4 < kb1) ? *reinterpret_cast<const float4v *>(arow + k + 4)
                                                    : float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
            v[0] = lo[0], v[1] = lo[1], v[2] = lo[2], v[3] = lo[3];
            v[4] = hi[0], v[5] = hi[1], v[6] = hi[2], v[7] = hi[3];
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t k = kb + 8 * soct + e;
                v[e] = (stager && srow < g.M && k < kb1) ? arow[(uint64_t)k * g.a_s1] : 0.0f;
            }
        }
    };
    auto store_rows = [&](int buf, const float (&v)[8]) {
        if (stager) {
            uint4w part3[3];
            split_eight(v, part3);
            // the thread's k = 8 soct + e': j = soct / 4, h = (soct % 4) / 2, grp = 2 (soct % 2) + e' / 4
            const uint32_t at = 32 * (soct / 4) + 16 * (soct % 2) + 4 * ((soct % 4) / 2);
#pragma unroll
            for (int pl = 0; pl < 3; ++pl) {
                *reinterpret_cast<uint2w *>(&xs[buf][pl][srow][at]) = uint2w{ part3[pl][0], part3[pl][1] };
                *reinterpret_cast<uint2w *>(&xs[buf][pl][srow][at + 8]) = uint2w{ part3[pl][2], part3[pl][3] };
            }
        }
    };
    constexpr int kDepth = 2; // register sets of b: the columns of the next step travel while one is multiplied (more sets: slower)
    float4v w[kDepth][4];
    float stage[8];
    if (kb0 < kb1) {
#pragma unroll
        for (int i = 0; i < kDepth - 1; ++i) {
            load_w(kb0 + 64 * i, w[i]);
        }
        fetch_rows(kb0, stage);
        store_rows(0, stage);
    }
    __syncthreads();
    auto iterate = [&](auto pc, auto xc, uint32_t kb) {
        constexpr int P = decltype(pc)::value; // register set of this step
        constexpr int X = decltype(xc)::value; // LDS buffer of this step
        // (the rows first: loads return in order, so waiting for the rows at the end of the step must not mean waiting
        // for the columns requested behind them, which are not needed before a later step)
        fetch_rows(kb + 64, stage); // lands in registers while this step is multiplied
        load_w(kb + 64 * (kDepth - 1), w[(P + kDepth - 1) % kDepth]);
        // the two halves of this lane's sixteen k: instruction j contracts over what the loads 2 j and 2 j + 1 hold
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float v[8] = { w[P][2 * j][0], w[P][2 * j][1], w[P][2 * j][2], w[P][2 * j][3],
                                 w[P][2 * j + 1][0], w[P][2 * j + 1][1], w[P][2 * j + 1][2], w[P][2 * j + 1][3] };
            uint4w bw[3];
            split_eight(v, bw);
            const bf16x8 B0 = __builtin_bit_cast(bf16x8, bw[0]), B1 = __builtin_bit_cast(bf16x8, bw[1]),
                         B2 = __builtin_bit_cast(bf16x8, bw[2]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                bf16x8 A[3];
#pragma unroll
                for (int pl = 0; pl < 3; ++pl) {
                    A[pl] = __builtin_bit_cast(
                        bf16x8, *reinterpret_cast<const uint4w *>(&xs[X][pl][16 * mt + c][32 * j + 8 * grp]));
                }
                // the small terms first
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[2], B0, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[1], B1, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[0], B2, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[1], B0, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[0], B1, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[0], B0, acc[mt], 0, 0, 0);
            }
        }
        store_rows(1 - X, stage);
        __syncthreads(); // the other buffer is complete, and nobody reads this one any more
    };
    // rounds of 2 kDepth steps so that register set and LDS buffer are compile-time constants
    uint32_t kb = kb0;
    while (kb < kb1) {
        static_for_sets<0, 2 * kDepth>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if (kb < kb1) {
                iterate(std::integral_constant<int, i % kDepth>{}, std::integral_constant<int, i % 2>{}, kb);
                kb += 64;
            }
        });
    }
    // partial result of this k range: part[split][row][column] (dense, row-major in columns)
    float *dst = part + (uint64_t)blockIdx.y * g.M * g.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t m = 16 * mt + 4 * grp + v;
            if (m < g.M && n_ok) {
                dst[(uint64_t)m * g.N + n] = acc[mt][v];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Whole tiles on the bfloat16 matrix instruction without giving up fp32 results: both operands are split exactly into
// three bfloat16 parts (split_bf16x3 above) and six of the nine products of parts -- all but the three smallest, which
// lie below 2^-24 of the terms -- are accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  Six instructions of 32 cycles
// do the work of eight fp32 instructions of 64, so the matrix pipe has 3/8 of the cycles to spend.  The error against
// the exact product is that of a chain of fp32 additions (about 1.2e-7 of the sum of |a.b|).  An operand that is not
// finite gives NaN where a plain fp32 product would give an infinity (inf - inf in the split).
//   workgroup = 4 wavefronts, tile 128 x 128, each wavefront a 64 x 64 quadrant = 2 x 2 instruction tiles;
//   k in slices of 32: the slice is fetched as fp32 (16 values per thread and operand) while the previous one is
//   multiplied, split by the thread that fetched it and staged in LDS as [part][row][k] bfloat16 (80 bytes per row, so
//   the 16-byte operand reads of 16 neighbouring rows fall on different banks); one LDS buffer, two barriers per slice,
//   two workgroups per compute unit to overlap them.
// ------------------------------------------------------------------------------------------------
constexpr int SK = 32;     // k per slice
constexpr int SPITCH = 40; // bfloat16 per staged row: 32 k + 8 of padding

// Which (row, k) of the 128 x 32 slice a thread fetches and stages.
//  ALONG_ROWS (the operand is contiguous along its row index): thread = (k quad kq = lane % 8, row quad i4 = 8 wave +
//    lane / 8): four 16-byte loads, rows 4 i4 .. + 3 at k = 4 kq + e; a wavefront reads eight k, 128 contiguous bytes
//    each.  It stores 8 bytes (four k) per row and part: 32 neighbouring lanes hit 32 different pairs of banks.
//  else (contiguous along k): two units u = tid + 256 q of (row, k octet kg = u % 4): two 16-byte loads each, four
//    lanes read a row's 128 bytes; rows are permuted inside groups of 16 so that the 16-byte stores of 16 neighbouring
//    lanes hit different banks.
// GUARD: sizes that are not multiples of the tile (the contiguous dimension's extent a multiple of 4): every 16-byte
// load is checked as a whole against the operand's `rows` and `k_end`, zeros beyond.
template <bool ALONG_ROWS, bool GUARD>
__device__ __forceinline__ void split_fetch(const float *__restrict__ p, uint64_t off, uint32_t s_row, uint32_t s_k,
                                            uint32_t row0, uint32_t k0, uint32_t rows, uint32_t k_end, float4v (&r)[4])
{
    const uint32_t tid = threadIdx.x;
    const float4v zero4 = { 0.0f, 0.0f, 0.0f, 0.0f };
    if constexpr (ALONG_ROWS) {
        const uint32_t kq = tid & 7, i4 = tid >> 3;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool in = !GUARD || (row0 + 4 * i4 < rows && k0 + 4 * kq + e < k_end);
            r[e] = in ? *reinterpret_cast<const float4v *>(p + off + (row0 + 4 * i4) + (uint64_t)(k0 + 4 * kq + e) * s_k)
                      : zero4;
        }
    } else {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t u = tid + 256 * q, kg = u & 3;
            const uint32_t row = (u >> 6) * 16 + 4 * ((u >> 2) & 3) + ((u >> 4) & 3);
            const float *src = p + off + (uint64_t)(row0 + row) * s_row + (k0 + 8 * kg);
            const bool in0 = !GUARD || (row0 + row < rows && k0 + 8 * kg < k_end);
            const bool in1 = !GUARD || (row0 + row < rows && k0 + 8 * kg + 4 < k_end);
            r[2 * q] = in0 ? *reinterpret_cast<const float4v *>(src) : zero4;
            r[2 * q + 1] = in1 ? *reinterpret_cast<const float4v *>(src + 4) : zero4;
        }
    }
}

template <bool ALONG_ROWS>
__device__ __forceinline__ void split_stage(uint16_t (*S)[TM][SPITCH], const float4v (&r)[4])
{
    const uint32_t tid = threadIdx.x;
    if constexpr (ALONG_ROWS) {
        const uint32_t kq = tid & 7, i4 = tid >> 3;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            uint32_t part[3][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                split_bf16x3(r[e][x], part[0][e], part[1][e], part[2][e]);
            }
#pragma unroll
            for (int pl = 0; pl < 3; ++pl) {
                *reinterpret_cast<uint2w *>(&S[pl][4 * i4 + x][4 * kq]) =
                    uint2w{ pack_upper_halves(part[pl][0], part[pl][1]), pack_upper_halves(part[pl][2], part[pl][3]) };
            }
        }
    } else {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t u = tid + 256 * q, kg = u & 3;
            const uint32_t row = (u >> 6) * 16 + 4 * ((u >> 2) & 3) + ((u >> 4) & 3);
            const float v[8] = { r[2 * q][0],     r[2 * q][1],     r[2 * q][2],     r[2 * q][3],
                                 r[2 * q + 1][0], r[2 * q + 1][1], r[2 * q + 1][2], r[2 * q + 1][3] };
            uint4w part[3];
            split_eight(v, part);
#pragma unroll
            for (int pl = 0; pl < 3; ++pl) {
                *reinterpret_cast<uint4w *>(&S[pl][row][8 * kg]) = part[pl];
            }
        }
    }
}

// k_per_split != 0 (unbatched products): blockIdx.z takes the k range [z k_per_split, ...) and `out` is the dense
// scratch part[split][row][column], which a second kernel adds up.
template <bool A_ICONTIG, bool B_KCONTIG, bool GUARD>
__global__ void __launch_bounds__(256) matmul_split_mfma_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                float *__restrict__ out, MatGeom g_launch,
                                                                uint32_t k_per_split)
{
    const MatGeom g = batch_geom(g_launch);
    const uint32_t k_first = k_per_split ? blockIdx.z * k_per_split : 0U;
    const uint32_t k_end = k_per_split ? min(g.K, k_first + k_per_split) : g.K;
    __shared__ __attribute__((aligned(16))) uint16_t As[3][TM][SPITCH];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[3][TN][SPITCH];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wi = wave >> 1, wj = wave & 1;
    const uint32_t m0 = blockIdx.x * TM, n0 = blockIdx.y * TN;
    const uint32_t l32 = lane & 31, lk = lane >> 5;

    float16v acc[2][2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
#pragma unroll
        for (int y = 0; y < 2; ++y) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[x][y][r] = 0.0f;
            }
        }
    }

    float4v ra[4], rb[4];
    auto fetch = [&](uint32_t k0) {
        // a: rows are the row index i (stride a_s0), k has stride a_s1; b: "rows" are the columns j (stride b_s1)
        split_fetch<A_ICONTIG, GUARD>(a, g.a_off, g.a_s0, g.a_s1, m0, k0, g.M, k_end, ra);
        split_fetch<!B_KCONTIG, GUARD>(b, g.b_off, g.b_s1, g.b_s0, n0, k0, g.N, k_end, rb);
    };
    auto stage = [&]() {
        split_stage<A_ICONTIG>(As, ra);
        split_stage<!B_KCONTIG>(Bs, rb);
    };

    const uint32_t n_slices = (k_end - k_first + SK - 1) / SK;
    fetch(k_first);
    stage();
    __syncthreads();
    for (uint32_t kt = 0; kt < n_slices; ++kt) {
        if (kt + 1 < n_slices) {
            fetch(k_first + (kt + 1) * SK);
        }
        // (a wavefront that multiplies goes ahead of one that splits and stages: the two workgroups of a compute unit
        // start together and would otherwise stay in step, all multiplying, then all splitting; 4096^3: 187 -> 194
        // TFLOP/s, 2048 x 4096 x 4096: 190 -> 200; the kernel on the fp32 instruction, with three workgroups per compute
        // unit, does not gain from it: 122 against 126)
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int ks = 0; ks < SK / 16; ++ks) {
            // lane (row or column l32, k octet lk) of an instruction tile
            bf16x8 A[2][3], B[2][3];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int pl = 0; pl < 3; ++pl) {
                    A[t][pl] = __builtin_bit_cast(
                        bf16x8, *reinterpret_cast<const uint4w *>(&As[pl][64 * wi + 32 * t + l32][16 * ks + 8 * lk]));
                    B[t][pl] = __builtin_bit_cast(
                        bf16x8, *reinterpret_cast<const uint4w *>(&Bs[pl][64 * wj + 32 * t + l32][16 * ks + 8 * lk]));
                }
            }
            // the small products first
#pragma unroll
            for (int x = 0; x < 2; ++x) {
#pragma unroll
                for (int y = 0; y < 2; ++y) {
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][2], B[y][0], acc[x][y], 0, 0, 0);
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][1], B[y][1], acc[x][y], 0, 0, 0);
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][0], B[y][2], acc[x][y], 0, 0, 0);
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][1], B[y][0], acc[x][y], 0, 0, 0);
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][0], B[y][1], acc[x][y], 0, 0, 0);
                    acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A[x][0], B[y][0], acc[x][y], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
        __syncthreads(); // everybody has read the slice
        if (kt + 1 < n_slices) {
            stage();
        }
        __syncthreads();
    }

    // register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32 x 32 tile
#pragma unroll
    for (int x = 0; x < 2; ++x) {
#pragma unroll
        for (int y = 0; y < 2; ++y) {
            const uint32_t col = n0 + 64 * wj + 32 * y + l32;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const uint32_t row = m0 + 64 * wi + 32 * x + 8 * r4 + 4 * lk;
                float *dst = out + (uint64_t)g.o_off + (uint64_t)row * g.o_s0 + (uint64_t)col * g.o_s1;
                if (k_per_split) {
                    float *part = out + ((uint64_t)blockIdx.z * g.M + row) * g.N + col;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (!GUARD || (row + e < g.M && col < g.N)) {
                            part[(uint64_t)e * g.N] = acc[x][y][4 * r4 + e];
                        }
                    }
                    continue;
                }
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = (!GUARD || col < g.N) ? with_bias(g, acc[x][y][4 * r4 + e], col) : 0.0f;
                }
                if (GUARD && (g.o_s0 != 1 || row + 3 >= g.M)) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (row + e < g.M && col < g.N) {
                            dst[(uint64_t)e * g.o_s0] = v[e];
                        }
                    }
                } else if (g.o_s0 == 1) {
                    if (!GUARD || col < g.N) {
                        *reinterpret_cast<float4v *>(dst) = float4v{ v[0], v[1], v[2], v[3] };
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dst[(uint64_t)e * g.o_s0] = v[e];
                    }
                }
            }
        }
    }
}

// Launches the instance for the operands' layouts (a contiguous along i or k, b along k or j).
template <bool GUARD>
void launch_split_mfma(dim3 grid, const float *a_dev, const float *b_dev, float *dst, const MatGeom &g, uint32_t k_per_split)
{
    const bool a_i = g.a_s0 == 1, b_k = g.b_s0 == 1;
    if (a_i && b_k) {
        matmul_split_mfma_kernel<true, true, GUARD><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
    } else if (a_i) {
        matmul_split_mfma_kernel<true, false, GUARD><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
    } else if (b_k) {
        matmul_split_mfma_kernel<false, true, GUARD><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
    } else {
        matmul_split_mfma_kernel<false, false, GUARD><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
    }
}

// out = sum over the k splits, in rising split order.
__global__ void __launch_bounds__(256) matmul_split_sum_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                              MatGeom g_launch, uint32_t splits)
{
    const MatGeom g = batch_geom(g_launch);
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= g.M * g.N) {
        return;
    }
    const uint32_t m = idx / g.N, n = idx - m * g.N;
    const float *src = part + (uint64_t)blockIdx.z * splits * g.M * g.N + idx;
    // (eight loads on their way at a time, added in rising order: one round trip per eight splits, not per split)
    const uint64_t plane = (uint64_t)g.M * g.N;
    float sum = 0.0f;
    for (uint32_t s0 = 0; s0 < splits; s0 += 8) {
        float v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            v[u] = src[(uint64_t)min(s0 + u, splits - 1) * plane];
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            if (s0 + u < splits) {
                sum += v[u];
            }
        }
    }
    out[(uint64_t)g.o_off + (uint64_t)m * g.o_s0 + (uint64_t)n * g.o_s1] = with_bias(g, sum, n);
}

// Scratch for the partial results of split products: grows as needed, kept for the life of the process.
float *g_split_ws = nullptr;
size_t g_split_ws_bytes = 0;

} // namespace
namespace weedhip {
// weed_hip_shutdown: the stream has been drained
void release_split_scratch()
{
    (void)hipFree(g_split_ws);
    g_split_ws = nullptr;
    g_split_ws_bytes = 0;
}
} // namespace weedhip
namespace {
int grow_split_scratch(const char *fn, size_t need)
{
    if (need > g_split_ws_bytes) {
        WEED_HIP_CHECK(hipStreamSynchronize(stream()));
        (void)hipFree(g_split_ws);
        g_split_ws = nullptr;
        g_split_ws_bytes = 0;
        if (hipMalloc((void **)&g_split_ws, need) != hipSuccess) {
            return fail(WEED_HIP_ENOMEM, "%s: scratch allocation of %zu bytes failed", fn, need);
        }
        g_split_ws_bytes = need;
    }
    return WEED_HIP_OK;
}

// Few rows, columns of b contiguous along k and 16-byte aligned, enough k to be worth streaming.
bool skinny_eligible(const MatGeom &g, const float *b)
{
    return g.M <= 64 && g.K >= 256 && g.K % 4 == 0 && g.b_s0 == 1 && (g.b_s1 & 3) == 0 &&
        ((g.b_bs[0] | g.b_bs[1]) & 3) == 0 && (((uintptr_t)b + 4 * (uint64_t)g.b_off) & 15) == 0;
}

bool aligned16(const float *p, uint64_t elem_off) { return (((uintptr_t)p + 4 * elem_off) & 15) == 0; }

// The matrix-core kernel needs full tiles, one contiguous dimension per operand and 16-byte aligned vector accesses.
bool mfma_eligible(const MatGeom &g, const float *a, const float *b, const float *out, bool whole_tiles = true)
{
    if (whole_tiles && (g.M % TM || g.N % TN || g.K % TK)) {
        return false;
    }
    if (!g.K) {
        return false;
    }
    if (!whole_tiles) {
        // 16-byte loads checked as a whole: the contiguous dimension's extent is a multiple of 4
        if ((g.a_s0 == 1 ? g.M : g.K) % 4 || (g.b_s0 == 1 ? g.K : g.N) % 4) {
            return false;
        }
    }
    const bool a_i = g.a_s0 == 1, a_k = g.a_s1 == 1;
    const bool b_k = g.b_s0 == 1, b_j = g.b_s1 == 1;
    if (!(a_i || a_k) || !(b_k || b_j)) {
        return false;
    }
    // vector loads step along the contiguous dimension in units of 4 floats; the other stride must keep alignment
    if (!aligned16(a, g.a_off) || ((a_i ? g.a_s1 : g.a_s0) & 3)) {
        return false;
    }
    if (!aligned16(b, g.b_off) || ((b_k ? g.b_s1 : g.b_s0) & 3)) {
        return false;
    }
    if (g.o_s0 == 1 && (!aligned16(out, g.o_off) || (g.o_s1 & 3))) {
        return false;
    }
    // every product of a batch keeps the alignment
    return !((g.a_bs[0] | g.a_bs[1] | g.b_bs[0] | g.b_bs[1] | g.o_bs[0] | g.o_bs[1]) & 3);
}

// Into how many ranges to split k over workgroups (1: not at all).  The tiles run in rounds of two per compute unit,
// each of k / splits slices plus a fixed part per workgroup (prologue, write-out: about 128 slices' worth), and a second
// kernel adds the ranges.  So 128 tiles gain from four ranges (512 x 4096 x 4096: 308 us whole on the fp32
// instruction, 184 in two ranges; with split operands 143 in two and 108 in four), 256 tiles from two (1024 x 4096 x
// 4096: 235 -> 204 us), and 512 tiles from none.
uint32_t choose_k_splits(uint64_t out_tiles, uint32_t K)
{
    if (out_tiles > 512) {
        return 1;
    }
    const auto cost = [&](uint32_t s) {
        // (two workgroups share a compute unit and fill each other's barrier waits: together they take 1.5 times
        // what one alone takes -- 1024 x 4096 x 4096, 256 tiles: 235 us whole, 204 in two ranges)
        const double wgs = (double)(out_tiles * s);
        const double rounds = std::ceil(wgs / 512.0), crowd = wgs <= 256.0 ? 1.0 : 1.5;
        return rounds * crowd * ((double)K / s + 128.0) + (s > 1 ? 40.0 + 0.3 * (double)(s * out_tiles) : 0.0);
    };
    uint32_t best = 1;
    double best_cost = cost(1) * 0.92; // (a split has to gain something beyond what two measurements differ by)
    for (uint32_t s = 2; s <= std::min(64U, K / 256U); ++s) {
        if (cost(s) < best_cost) {
            best_cost = cost(s);
            best = s;
        }
    }
    return best;
}

} // namespace

namespace {

int launch_matmul_body(const char *fn, const MatGeom &g, uint32_t batch, const float *a_dev, const float *b_dev, float *out_dev);

// weed_hip_matmul_tuning: the fp32 matrix instruction for every product (false: six bfloat16 products of split operands
// where the layout allows)
// (the process-wide default comes from the environment variable WEED_HIP_MATMUL_FP32, read once: 1 = the fp32 instruction)
std::atomic<bool> g_fp32_instruction{ [] {
    const char *e = std::getenv("WEED_HIP_MATMUL_FP32");
    return e != nullptr && e[0] == '1';
}() };

int launch_matmul(const char *fn, const MatGeom &g, uint32_t batch, const float *a_dev, const float *b_dev, float *out_dev)
{
    WEED_HIP_REQUIRE(a_dev && b_dev && out_dev, "%s: null pointer", fn);
    WEED_HIP_TRY(ensure_init());
    if (!g.M || !g.N || !batch) {
        return WEED_HIP_OK;
    }
    ProfileScope prof("matmul");
    return launch_matmul_body(fn, g, batch, a_dev, b_dev, out_dev);
}

int launch_matmul_body(const char *fn, const MatGeom &g, uint32_t batch, const float *a_dev, const float *b_dev, float *out_dev)
{
    WEED_HIP_REQUIRE(batch <= 65535u, "%s: %u products in one call (at most 65535)", fn, batch);
    if (batch > 1) {
        // the kernels add a product's batch offsets to the operand offsets in 32 bits: refuse what would wrap
        const uint64_t c0 = g.nb0 - 1, c1 = batch / g.nb0 - 1, lim = 0xffffffffull;
        WEED_HIP_REQUIRE((uint64_t)g.a_off + c0 * g.a_bs[0] + c1 * g.a_bs[1] <= lim &&
                             (uint64_t)g.b_off + c0 * g.b_bs[0] + c1 * g.b_bs[1] <= lim &&
                             (uint64_t)g.o_off + c0 * g.o_bs[0] + c1 * g.o_bs[1] <= lim,
                         "%s: a batch offset exceeds 32 bits", fn);
    }
    const uint32_t M = g.M, N = g.N, K = g.K;
    const bool split_parts = !g_fp32_instruction.load(std::memory_order_relaxed);
    // few output tiles and a long k: the tiles' k ranges are split over more workgroups (guarded instances below)
    const uint64_t out_tiles = (uint64_t)((M + TM - 1) / TM) * ((N + TN - 1) / TN) * batch;
    const uint32_t want_splits = (batch == 1 && M > 16 && N > 16 && K >= 1024) ? choose_k_splits(out_tiles, K) : 1U;
    const bool split_k = want_splits >= 2;
    if (split_k && mfma_eligible(g, a_dev, b_dev, out_dev) && !skinny_eligible(g, b_dev)) {
        // few whole tiles and a long k: the unguarded kernel over k ranges, a second kernel adds them
        uint32_t splits = want_splits;
        const uint32_t k_unit = (split_parts && K % SK == 0) ? SK : TK; // (whole slices of the kernel that takes the ranges)
        const uint32_t k_per_split = ((K + splits - 1) / splits + k_unit - 1) / k_unit * k_unit;
        splits = (K + k_per_split - 1) / k_per_split;
        if (splits >= 2) {
            WEED_HIP_TRY(grow_split_scratch(fn, sizeof(float) * (size_t)splits * M * N));
            const dim3 grid(M / TM, N / TN, splits);
            WEED_HIP_REQUIRE(grid.y <= 65535u, "%s: N = %u too large", fn, N);
            const bool a_i = g.a_s0 == 1, b_k = g.b_s0 == 1;
            if (split_parts && k_per_split % SK == 0) {
                launch_split_mfma<false>(grid, a_dev, b_dev, g_split_ws, g, k_per_split);
            } else if (a_i && b_k) {
                matmul_mfma_kernel<true, true, 0, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            } else if (a_i) {
                matmul_mfma_kernel<true, false, 0, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            } else if (b_k) {
                matmul_mfma_kernel<false, true, 0, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            } else {
                matmul_mfma_kernel<false, false, 0, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            }
            WEED_HIP_LAUNCH_CHECK();
            matmul_split_sum_kernel<<<dim3((M * N + 255) / 256, 1, 1), 256, 0, stream()>>>(g_split_ws, out_dev, g, splits);
            WEED_HIP_LAUNCH_CHECK();
            return WEED_HIP_OK;
        }
    }
    if (!split_k && mfma_eligible(g, a_dev, b_dev, out_dev)) {
        const dim3 grid(M / TM, N / TN, batch);
        WEED_HIP_REQUIRE(grid.y <= 65535u, "%s: N = %u too large", fn, N);
        const bool a_i = g.a_s0 == 1, b_k = g.b_s0 == 1;
        if (split_parts && K % SK == 0) {
            // six bfloat16 products of exactly split operands in place of the fp32 instruction
            launch_split_mfma<false>(grid, a_dev, b_dev, out_dev, g, 0);
            WEED_HIP_LAUNCH_CHECK();
            return WEED_HIP_OK;
        }
        if (a_i && b_k) {
            matmul_mfma_kernel<true, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
        } else if (a_i) {
            matmul_mfma_kernel<true, false><<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
        } else if (b_k) {
            matmul_mfma_kernel<false, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
        } else {
            matmul_mfma_kernel<false, false><<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
        }
        WEED_HIP_LAUNCH_CHECK();
        return WEED_HIP_OK;
    }
    if (skinny_eligible(g, b_dev)) { // (few rows: this streaming kernel splits k by itself)
        // every wavefront of a workgroup takes a whole number of 64-k iterations
        const uint32_t k_per_wave = ((K + kSkinnyWaves - 1) / kSkinnyWaves + 63) / 64 * 64;
        const dim3 wgs((N + 15) / 16, 1, batch);
        if (M > 16 && N >= 512 && batch == 1 && split_parts) {
            // shared rows, k split over workgroups (about 450 workgroups in all), a second pass adds the splits
            const uint32_t col_wgs = (N + 16 * kWideWaves - 1) / (16 * kWideWaves);
            uint32_t splits = std::max(1u, std::min((448u + col_wgs / 2) / col_wgs, K / 256u));
            const uint32_t k_per_split = ((K + splits - 1) / splits + 63) / 64 * 64;
            splits = (K + k_per_split - 1) / k_per_split;
            WEED_HIP_TRY(grow_split_scratch(fn, sizeof(float) * (size_t)splits * M * N));
            const dim3 wide(col_wgs, splits, 1);
            const bool a_k = g.a_s1 == 1 && (g.a_s0 & 3) == 0 && aligned16(a_dev, g.a_off);
            if (M <= 32) {
                if (a_k) {
                    matmul_skinny_wide_kernel<2, true><<<wide, 64 * kWideWaves, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
                } else {
                    matmul_skinny_wide_kernel<2><<<wide, 64 * kWideWaves, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
                }
            } else if (a_k) {
                matmul_skinny_wide_kernel<4, true><<<wide, 64 * kWideWaves, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            } else {
                matmul_skinny_wide_kernel<4><<<wide, 64 * kWideWaves, 0, stream()>>>(a_dev, b_dev, g_split_ws, g, k_per_split);
            }
            WEED_HIP_LAUNCH_CHECK();
            matmul_split_sum_kernel<<<dim3((M * N + 255) / 256, 1, 1), 256, 0, stream()>>>(g_split_ws, out_dev, g, splits);
            WEED_HIP_LAUNCH_CHECK();
            return WEED_HIP_OK;
        }
        if (M <= 16) {
            matmul_skinny_kernel<1><<<wgs, 64 * kSkinnyWaves, 0, stream()>>>(a_dev, b_dev, out_dev, g, k_per_wave);
        } else if (M <= 32) {
            matmul_skinny_kernel<2><<<wgs, 64 * kSkinnyWaves, 0, stream()>>>(a_dev, b_dev, out_dev, g, k_per_wave);
        } else {
            matmul_skinny_kernel<4><<<wgs, 64 * kSkinnyWaves, 0, stream()>>>(a_dev, b_dev, out_dev, g, k_per_wave);
        }
        WEED_HIP_LAUNCH_CHECK();
        return WEED_HIP_OK;
    }
    // Ragged sizes around an interior of whole 128 x 128 tiles (a prefill of 1000 tokens): one launch takes the interior,
    // the strips behind it go the way their own shapes call for.  Two things can pay for the extra launches (never below
    // 2^32 multiply-adds).  Where the whole product would need the element-wise guards (a row count that is not a
    // multiple of 4, an unaligned view), the interior does not: 1000 x 4096 x 4096 took 379 us so, 469 with every tile
    // guarded element by element.  And where the loads are checked 16 bytes at a time anyway, the tiles run in rounds of
    // one per compute unit, so a few tiles beyond a whole number of rounds cost a whole round: 1000 x 4096 x 4100 is
    // 8 x 33 = 264 tiles, 582 us in one launch against 365 for N = 4096, and 407 us as an interior of 7 x 31 tiles with
    // its two strips; 1000 x 4096 x 4096 itself is 256 tiles and stays one launch (365 us either way).  (Guarded
    // instances that read the tiles inside the matrix with the unguarded loads, one launch for everything, were
    // measured too: 579 us for that product -- the instance's registers and address arithmetic slow every tile.)
    if (batch == 1 && M >= TM && N >= 2 * TN && (M % TM || N % TN) && (uint64_t)M * N * K >= (1ull << 32)) {
        MatGeom in = g;
        in.M = M / TM * TM;
        in.N = N / TN * TN;
        if (N % TN && N % TN <= 16) in.N -= TN; // a strip of under 17 columns has no matrix-core kernel: one more tile goes with it
                                                // (a strip of under 17 rows is the skinny kernels' own shape)
        bool strips_pay = true;
        if (mfma_eligible(g, a_dev, b_dev, out_dev, false)) {
            // in rounds of 256 tiles; a strip's few tiles split k and fill the part, plus what its launch costs
            const auto tiles = [](uint32_t m, uint32_t n) { return (double)((m + TM - 1) / TM) * ((n + TN - 1) / TN); };
            const double whole = std::ceil(tiles(M, N) / 256.0);
            double split = std::ceil(tiles(in.M, in.N) / 256.0);
            if (in.M < M) split += tiles(M - in.M, N) / 256.0 + 0.15;
            if (in.N < N) split += tiles(in.M, N - in.N) / 256.0 + 0.15;
            strips_pay = split < whole;
        }
        const uint64_t lim = 0xffffffffull;
        const bool fits = (uint64_t)g.a_off + (uint64_t)in.M * g.a_s0 <= lim && (uint64_t)g.o_off + (uint64_t)in.M * g.o_s0 <= lim &&
            (uint64_t)g.b_off + (uint64_t)in.N * g.b_s1 <= lim && (uint64_t)g.o_off + (uint64_t)in.N * g.o_s1 <= lim &&
            (uint64_t)g.bias_off + (uint64_t)in.N * g.bias_s <= lim;
        if (strips_pay && fits && mfma_eligible(in, a_dev, b_dev, out_dev, false)) { // (k not a multiple of 16: the interior is checked per load)
            WEED_HIP_TRY(launch_matmul_body(fn, in, 1, a_dev, b_dev, out_dev));
            if (in.M < M) { // the rows behind, all columns
                MatGeom e = g;
                e.M = M - in.M;
                e.a_off += in.M * g.a_s0;
                e.o_off += in.M * g.o_s0;
                WEED_HIP_TRY(launch_matmul_body(fn, e, 1, a_dev, b_dev, out_dev));
            }
            if (in.N < N) { // the columns behind, the interior's rows
                MatGeom e = g;
                e.M = in.M;
                e.N = N - in.N;
                e.b_off += in.N * g.b_s1;
                e.o_off += in.N * g.o_s1;
                e.bias_off += in.N * g.bias_s;
                WEED_HIP_TRY(launch_matmul_body(fn, e, 1, a_dev, b_dev, out_dev));
            }
            return WEED_HIP_OK;
        }
    }
    if (M > 16 && N > 16 && K >= 8) {
        // ragged, unaligned or doubly strided: matrix-core tiles with guarded loads and stores
        uint32_t splits = 1, k_per_split = 0;
        if (split_k) {
            splits = want_splits;
            k_per_split = ((K + splits - 1) / splits + TK - 1) / TK * TK;
            splits = (K + k_per_split - 1) / k_per_split;
            if (splits < 2) {
                k_per_split = 0;
            }
        }
        float *dst = out_dev;
        if (k_per_split) {
            WEED_HIP_TRY(grow_split_scratch(fn, sizeof(float) * (size_t)splits * M * N));
            dst = g_split_ws;
        }
        const dim3 grid((M + TM - 1) / TM, (N + TN - 1) / TN, k_per_split ? splits : batch);
        WEED_HIP_REQUIRE(grid.y <= 65535u, "%s: N = %u too large", fn, N);
        if (mfma_eligible(g, a_dev, b_dev, out_dev, false)) {
            // the unguarded kernels' layout, sizes that are not multiples of the tile: 16-byte loads checked as a whole
            const bool a_i = g.a_s0 == 1, b_k = g.b_s0 == 1;
            if (split_parts) {
                launch_split_mfma<true>(grid, a_dev, b_dev, dst, g, k_per_split);
            } else if (a_i && b_k) {
                matmul_mfma_kernel<true, true, 2, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
            } else if (a_i) {
                matmul_mfma_kernel<true, false, 2, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
            } else if (b_k) {
                matmul_mfma_kernel<false, true, 2, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
            } else {
                matmul_mfma_kernel<false, false, 2, true><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
            }
            WEED_HIP_LAUNCH_CHECK();
            if (k_per_split) {
                matmul_split_sum_kernel<<<dim3((M * N + 255) / 256, 1, 1), 256, 0, stream()>>>(g_split_ws, out_dev, g, splits);
                WEED_HIP_LAUNCH_CHECK();
            }
            return WEED_HIP_OK;
        }
        const bool a_i = g.a_s0 <= g.a_s1, b_k = g.b_s0 <= g.b_s1;
        if (a_i && b_k) {
            matmul_mfma_kernel<true, true, 1><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
        } else if (a_i) {
            matmul_mfma_kernel<true, false, 1><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
        } else if (b_k) {
            matmul_mfma_kernel<false, true, 1><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
        } else {
            matmul_mfma_kernel<false, false, 1><<<grid, 256, 0, stream()>>>(a_dev, b_dev, dst, g, k_per_split);
        }
        WEED_HIP_LAUNCH_CHECK();
        if (k_per_split) {
            matmul_split_sum_kernel<<<dim3((M * N + 255) / 256, 1, 1), 256, 0, stream()>>>(g_split_ws, out_dev, g, splits);
            WEED_HIP_LAUNCH_CHECK();
        }
        return WEED_HIP_OK;
    }
    const dim3 grid((M + BM - 1) / BM, (N + BN - 1) / BN, batch);
    WEED_HIP_REQUIRE(grid.y <= 65535u, "%s: N = %u too large", fn, N);
    matmul_tiled_kernel<<<grid, 256, 0, stream()>>>(a_dev, b_dev, out_dev, g);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

} // namespace

extern "C" int weed_hip_matmul_tuning(int32_t fp32_instruction)
{
    g_fp32_instruction.store(fp32_instruction != 0, std::memory_order_relaxed);
    return WEED_HIP_OK;
}

extern "C" int weed_hip_matmul_f32(uint32_t M, uint32_t N, uint32_t K, const float *a_dev, uint32_t a_off,
                                   uint32_t a_s0, uint32_t a_s1, const float *b_dev, uint32_t b_off, uint32_t b_s0,
                                   uint32_t b_s1, float *out_dev, uint32_t o_off, uint32_t o_s0, uint32_t o_s1)
{
    const MatGeom g = { M, N, K, a_off, a_s0, a_s1, b_off, b_s0, b_s1, o_off, o_s0, o_s1, 1, { 0, 0 }, { 0, 0 }, { 0, 0 },
                        nullptr, 0, 0 };
    return launch_matmul("weed_hip_matmul_f32", g, 1, a_dev, b_dev, out_dev);
}

extern "C" int weed_hip_linear_f32(uint32_t M, uint32_t N, uint32_t K, const float *a_dev, uint32_t a_off, uint32_t a_s0,
                                   uint32_t a_s1, const float *w_dev, uint32_t w_off, uint32_t w_s0, uint32_t w_s1,
                                   const float *bias_dev, uint32_t bias_off, uint32_t bias_stride, float *out_dev,
                                   uint32_t o_off, uint32_t o_s0, uint32_t o_s1)
{
    const MatGeom g = { M, N, K, a_off, a_s0, a_s1, w_off, w_s0, w_s1, o_off, o_s0, o_s1, 1, { 0, 0 }, { 0, 0 }, { 0, 0 },
                        bias_dev, bias_off, bias_stride };
    return launch_matmul("weed_hip_linear_f32", g, 1, a_dev, w_dev, out_dev);
}

extern "C" int weed_hip_matmul_batched_f32(const uint32_t batch[2], uint32_t M, uint32_t N, uint32_t K,
                                           const float *a_dev, uint32_t a_off, uint32_t a_s0, uint32_t a_s1,
                                           const uint32_t a_bs[2], const float *b_dev, uint32_t b_off, uint32_t b_s0,
                                           uint32_t b_s1, const uint32_t b_bs[2], float *out_dev, uint32_t o_off,
                                           uint32_t o_s0, uint32_t o_s1, const uint32_t o_bs[2])
{
    const char *fn = "weed_hip_matmul_batched_f32";
    WEED_HIP_REQUIRE(batch && a_bs && b_bs && o_bs, "%s: null pointer", fn);
    const uint64_t n = (uint64_t)batch[0] * batch[1];
    WEED_HIP_REQUIRE(n <= 65535u, "%s: %llu products in one call (at most 65535)", fn, (unsigned long long)n);
    const MatGeom g = { M, N, K, a_off, a_s0, a_s1, b_off, b_s0, b_s1, o_off, o_s0, o_s1, batch[0] ? batch[0] : 1u,
                        { a_bs[0], a_bs[1] }, { b_bs[0], b_bs[1] }, { o_bs[0], o_bs[1] }, nullptr, 0, 0 };
    return launch_matmul(fn, g, (uint32_t)n, a_dev, b_dev, out_dev);
}
