// Matrix-core decode attention over the packed cache (gfx950).
//
// One wavefront owns 64-token blocks of one (sequence, kv head).  Per block it
//   1. streams its lane-major run of packed K items (coalesced 128-bit loads, every byte of the block read once),
//   2. turns every pair of fields into two fp16 values with one conflict-free LDS lookup (the pair table is replicated
//      over the 32 banks) and feeds them as the A operand of v_mfma_f32_16x16x32_f16 against the query, which sits in
//      registers as fp16 hi + lo halves (products of fp16 values are exact in fp32, so the split keeps ~22 bits),
//   3. runs an online softmax on the 16 tokens x 16 heads score tiles in registers (base-2 exponentials; 1/sqrt(d) and
//      log2(e) are folded into the query),
//   4. splits the probabilities (times the V row scales) into fp16 hi + lo, which are already in A-operand order,
//      and multiplies them with the looked-up V items: out[head][coordinate] accumulates in 4*(d/16) registers.
// The four wavefronts of a workgroup share the lookup tables, split the workgroup's blocks between them and merge
// their partial results in LDS; one un-normalised partial (m, l, o[d]) per query head leaves the workgroup.
//
// Table values are exactly representable in fp16 (the Lloyd-Max tables are generated that way; the uniform coder's
// table is code + 0.5), so de-quantisation itself is exact; the only roundings are those of the fp32 accumulators.
#include "kv_decode_mfma.h"

using namespace weedhip;
using namespace weedkv;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

constexpr int kWaves = 4;

__device__ __forceinline__ uint32_t pack_half2(float a, float b)
{
    const _Float16 ha = (_Float16)a, hb = (_Float16)b;
    return (uint32_t)__builtin_bit_cast(uint16_t, ha) | ((uint32_t)__builtin_bit_cast(uint16_t, hb) << 16);
}

// N dwords from a pointer aligned to 16 bytes when N % 4 == 0, else to 8 bytes (N is even for every supported shape).
template <int N> __device__ __forceinline__ void load_dwords(const uint8_t *p, uint32_t (&x)[N])
{
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const uint4v v = *reinterpret_cast<const uint4v *>(p + 16 * i);
            x[4 * i] = v.x;
            x[4 * i + 1] = v.y;
            x[4 * i + 2] = v.z;
            x[4 * i + 3] = v.w;
        }
    } else {
        static_assert(N % 2 == 0, "lane runs are multiples of 8 bytes");
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const uint2v v = *reinterpret_cast<const uint2v *>(p + 8 * i);
            x[2 * i] = v.x;
            x[2 * i + 1] = v.y;
        }
    }
}

// Pair `P` (2*W bits at bit 2*W*P of the lane's run) -> dword index of its table entry for this lane.
template <int W, int N> __device__ __forceinline__ uint32_t pair_index(const uint32_t (&x)[N], int P)
{
    const int bit = 2 * W * P;
    const int dw = bit >> 5, sh = bit & 31;
    constexpr uint32_t mask = (1u << (2 * W)) - 1u;
    uint32_t v;
    if (sh + 2 * W <= 32) {
        v = __builtin_amdgcn_ubfe(x[dw], sh, 2 * W);
    } else {
        v = __builtin_amdgcn_alignbit(x[dw + 1 < N ? dw + 1 : dw], x[dw], sh) & mask;
    }
    return v << 5;
}

// Item k (8 fields) of the lane's run -> 8 fp16 values in matrix-operand order.
template <int W, int N> __device__ __forceinline__ half8 dequant_item(const uint32_t (&x)[N], int k, const uint32_t *tab_lane)
{
    uint4v r;
    r.x = tab_lane[pair_index<W, N>(x, 4 * k)];
    r.y = tab_lane[pair_index<W, N>(x, 4 * k + 1)];
    r.z = tab_lane[pair_index<W, N>(x, 4 * k + 2)];
    r.w = tab_lane[pair_index<W, N>(x, 4 * k + 3)];
    return __builtin_bit_cast(half8, r);
}

__device__ __forceinline__ float4v mfma16(half8 a, half8 b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float xor16_32_max(float v)
{
    v = fmaxf(v, __shfl_xor(v, 16));
    return fmaxf(v, __shfl_xor(v, 32));
}

__device__ __forceinline__ float xor16_32_sum(float v)
{
    v += __shfl_xor(v, 16);
    return v + __shfl_xor(v, 32);
}

template <int D, int WK, int WV>
__global__ void __launch_bounds__(64 * kWaves) decode_mfma_kernel(MfmaParams p)
{
    constexpr int KS = D / 32;       // Q.K^T k-steps (32 coordinates each); also K items per tile per lane
    constexpr int JB = D / 16;       // 16-coordinate column blocks of the output
    constexpr int NK = KS * WK;      // dwords of packed K per lane per block
    constexpr int NV = D * WV / 32;  // dwords of packed V per lane per block
    constexpr uint32_t KT = (1u << (2 * WK)) * 32u; // dwords of the replicated K pair table
    constexpr uint32_t VT = (1u << (2 * WV)) * 32u;

    extern __shared__ uint32_t lds[];
    uint32_t *ktab = lds;
    uint32_t *vtab = lds + KT;

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 15, g = lane >> 4;
    const uint32_t split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const uint32_t L = (uint32_t)p.lens[seq];
    const uint32_t nblk = (L + 63) >> 6;
    const uint32_t b0 = split * p.blocks_per_split;
    const uint32_t b1 = min(nblk, b0 + p.blocks_per_split);
    const uint64_t region = (uint64_t)seq * p.Hkv + kvh;
    const bool lloyd = p.k.alpha != nullptr;

    // ---- pair tables: entry e, replica i at dword e*32 + i; a lane always reads replica lane%32 ----
    for (uint32_t i = tid; i < KT; i += 64 * kWaves) {
        const uint32_t e = i >> 5;
        ktab[i] = pack_half2(p.k.table[e & ((1u << WK) - 1u)], p.k.table[e >> WK]);
    }
    for (uint32_t i = tid; i < VT; i += 64 * kWaves) {
        const uint32_t e = i >> 5;
        vtab[i] = pack_half2(p.v.table[e & ((1u << WV) - 1u)], p.v.table[e >> WV]);
    }
    __syncthreads();
    const uint32_t *ktab_lane = ktab + (lane & 31);
    const uint32_t *vtab_lane = vtab + (lane & 31);

    // ---- query operand: column c of B is query head c of this kv head, rows are the lane group's coordinates ----
    const bool head_ok = c < p.G;
    const uint32_t qh = head_ok ? (p.blocked ? kvh * p.G + c : c * p.Hkv + kvh) : 0;
    half8 qhi[KS], qlo[KS];
    {
        const uint64_t qbase = ((uint64_t)seq * p.Hq + qh) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4v hi = { 0, 0, 0, 0 }, lo = { 0, 0, 0, 0 };
            if (head_ok) {
                hi = *reinterpret_cast<const uint4v *>(p.q_hi + qbase + 8 * ks);
                lo = *reinterpret_cast<const uint4v *>(p.q_lo + qbase + 8 * ks);
            }
            qhi[ks] = __builtin_bit_cast(half8, hi);
            qlo[ks] = __builtin_bit_cast(half8, lo);
        }
    }
    const float qscale = head_ok ? p.q_scale[(uint64_t)seq * p.Hq + qh] : 0.0f;
    const float betaq = head_ok ? p.k.beta * p.q_sum[(uint64_t)seq * p.Hq + qh] : 0.0f;

    // ---- exponent that keeps probability * V-row-scale inside fp16's normal range ----
    int ep = 10;
    if (lloyd) {
        const uint32_t bits = p.v.alpha_max[region];
        ep = bits ? 136 - (int)((bits >> 23) & 0xff) : 0;
        ep = ep > 100 ? 100 : (ep < -100 ? -100 : ep);
    }
    const float unscale = __uint_as_float((uint32_t)(127 - ep) << 23); // 2^-ep

    float m_run = -INFINITY; // running maximum of this lane's head (same value in the 4 lanes that share a head)
    float l_run = 0.0f;      // this lane's share of the running denominator, scaled by 2^ep
    float4v O[JB];
#pragma unroll
    for (int jb = 0; jb < JB; ++jb) {
        O[jb] = float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
    }

    const uint8_t *kreg = p.k.fields + region * p.k.region_bytes + (uint64_t)lane * (4 * NK);
    const uint8_t *vreg = p.v.fields + region * p.v.region_bytes + (uint64_t)lane * (4 * NV);
    const float *ka = lloyd ? p.k.alpha + region * p.padded + 4 * g : nullptr;
    const float *va = lloyd ? p.v.alpha + region * p.padded + 4 * g : nullptr;

    for (uint32_t blk = b0 + wave; blk < b1; blk += kWaves) {
        // The lane's run holds its 4 tiles back to back: tile t occupies items t*KS .. t*KS + KS - 1.
        uint32_t kraw[NK];
        uint32_t vraw[NV];
        load_dwords<NK>(kreg + (uint64_t)blk * (8u * D * WK), kraw);
        load_dwords<NV>(vreg + (uint64_t)blk * (8u * D * WV), vraw);
        float4v ak[4], av[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (lloyd) {
                ak[t] = *reinterpret_cast<const float4v *>(ka + blk * 64 + 16 * t);
                av[t] = *reinterpret_cast<const float4v *>(va + blk * 64 + 16 * t);
            } else {
                ak[t] = float4v{ p.k.alpha_const, p.k.alpha_const, p.k.alpha_const, p.k.alpha_const };
                av[t] = float4v{ 1.0f, 1.0f, 1.0f, 1.0f };
            }
        }

        // ---- S[t] = K_tile . q: rows = tokens 16t + (lane%16), contraction over the lane groups' coordinates ----
        float4v S[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            S[t] = float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const half8 a = dequant_item<WK, NK>(kraw, t * KS + ks, ktab_lane);
                S[t] = mfma16(a, qhi[ks], S[t]);
                S[t] = mfma16(a, qlo[ks], S[t]);
            }
        }

        // ---- scores in log2 units: lane (c, g) register r of tile t = token blk*64 + 16t + 4g + r, head c ----
        float mloc = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                S[t][r] = fmaf(S[t][r], ak[t][r] * qscale, betaq);
            }
        }
        if (blk * 64 + 64 > L) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (blk * 64 + 16 * t + 4 * g + r >= L) {
                        S[t][r] = -INFINITY;
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                mloc = fmaxf(mloc, S[t][r]);
            }
        }
        mloc = xor16_32_max(mloc);
        const float m_new = fmaxf(m_run, mloc);
        if (__any(m_new > m_run)) {
            const float scale = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= scale;
            // output row 4g + r belongs to head 4g + r, whose scale lives in lane 4g + r
            float sr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sr[r] = __shfl(scale, (int)(4 * g + r));
            }
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    O[jb][r] *= sr[r];
                }
            }
            m_run = m_new;
        }
        const float mm = m_run - (float)ep;
        uint32_t Ahi[2][4], Alo[2][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            float pv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(S[t][r] - mm); // exp2(-inf) = 0 masks the tail
                l_run += e;
                pv[r] = e * av[t][r];
            }
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                // hi = top 11 significant bits (exact in fp16), lo = the rest
                const float a0 = pv[2 * h2], a1 = pv[2 * h2 + 1];
                const float h0 = __uint_as_float(__float_as_uint(a0) & 0xffffe000u);
                const float h1 = __uint_as_float(__float_as_uint(a1) & 0xffffe000u);
                const int slot = 2 * (t & 1) + h2; // k-slots 0..3 come from tile 2u, 4..7 from tile 2u + 1
                Ahi[t >> 1][slot] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(h0, h1));
                Alo[t >> 1][slot] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a0 - h0, a1 - h1));
            }
        }

        // ---- O[head][coordinate] += P . V over the block's two 32-token halves ----
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const half8 phi = __builtin_bit_cast(half8, uint4v{ Ahi[u][0], Ahi[u][1], Ahi[u][2], Ahi[u][3] });
            const half8 plo = __builtin_bit_cast(half8, uint4v{ Alo[u][0], Alo[u][1], Alo[u][2], Alo[u][3] });
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) {
                const half8 b = dequant_item<WV, NV>(vraw, u * JB + jb, vtab_lane);
                O[jb] = mfma16(phi, b, O[jb]);
                O[jb] = mfma16(plo, b, O[jb]);
            }
        }
    }

    // ---- per-wave results -> LDS (the tables are no longer needed), then one merged partial per head ----
    const float l_head = xor16_32_sum(l_run) * unscale; // all four lanes of a head now hold its denominator
    float lrow[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        lrow[r] = __shfl(l_head, (int)(4 * g + r));
    }
    __syncthreads();
    float *ws = reinterpret_cast<float *>(lds); // [wave][head slot 0..15][D + 2]
    constexpr int PS = D + 2;
    const float o_mul = unscale * (lloyd ? 1.0f : p.v.alpha_const);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t hs = 4 * g + r;
        if (hs < p.G) {
            float *dst = ws + ((size_t)wave * 16 + hs) * PS;
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) {
                // uniform coder: value = step * (code + 0.5) + lo, so add lo * sum(p)
                dst[2 + 16 * jb + c] = fmaf(O[jb][r], o_mul, p.v.beta * lrow[r]);
            }
        }
    }
    if (g == 0 && head_ok) {
        float *dst = ws + ((size_t)wave * 16 + c) * PS;
        dst[0] = m_run;
        dst[1] = l_head;
    }
    __syncthreads();
    for (uint32_t idx = tid; idx < p.G * (uint32_t)PS; idx += 64 * kWaves) {
        const uint32_t hs = idx / PS, j = idx % PS;
        float mw[kWaves], mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            mw[w] = ws[((size_t)w * 16 + hs) * PS];
            mx = fmaxf(mx, mw[w]);
        }
        float val;
        if (j == 0) {
            val = mx;
        } else {
            val = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const float f = (mw[w] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(mw[w] - mx);
                val = fmaf(f, ws[((size_t)w * 16 + hs) * PS + j], val);
            }
        }
        const uint32_t head = p.blocked ? kvh * p.G + hs : hs * p.Hkv + kvh;
        p.partials[(((uint64_t)seq * p.Hq + head) * p.n_splits + split) * PS + j] = val;
    }
}

template <int D, int WK, int WV> int launch_one(const MfmaParams &p, dim3 grid, hipStream_t s)
{
    constexpr size_t tab_bytes = (((size_t)1 << (2 * WK)) + ((size_t)1 << (2 * WV))) * 32 * sizeof(uint32_t);
    constexpr size_t merge_bytes = (size_t)kWaves * 16 * (D + 2) * sizeof(float);
    constexpr size_t smem = tab_bytes > merge_bytes ? tab_bytes : merge_bytes;
    static bool configured = false;
    if (!configured) {
        WEED_HIP_CHECK(hipFuncSetAttribute((const void *)decode_mfma_kernel<D, WK, WV>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        configured = true;
    }
    decode_mfma_kernel<D, WK, WV><<<grid, 64 * kWaves, smem, s>>>(p);
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

template <int D> int launch_d(const MfmaParams &p, dim3 grid, hipStream_t s)
{
    const uint32_t wk = p.k.w, wv = p.v.w;
#define WEED_CASE(K, V)                                                                                                \
    if (wk == K && wv == V) {                                                                                          \
        return launch_one<D, K, V>(p, grid, s);                                                                        \
    }
    WEED_CASE(2, 2)
    WEED_CASE(2, 3)
    WEED_CASE(2, 4)
    WEED_CASE(3, 2)
    WEED_CASE(3, 3)
    WEED_CASE(3, 4)
    WEED_CASE(4, 2)
    WEED_CASE(4, 3)
    WEED_CASE(4, 4)
#undef WEED_CASE
    return fail(WEED_HIP_EINVAL, "decode_mfma: unsupported field widths %u / %u", wk, wv);
}

} // namespace

namespace weedhip {

bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G)
{
    return (d == 64 || d == 128) && wk >= 2 && wk <= 4 && wv >= 2 && wv <= 4 && G >= 1 && G <= 16;
}

int launch_mfma_decode(const MfmaParams &p, uint32_t d, uint32_t n_seq, hipStream_t s)
{
    const dim3 grid(p.n_splits, p.Hkv, n_seq);
    if (d == 64) {
        return launch_d<64>(p, grid, s);
    }
    return launch_d<128>(p, grid, s);
}

} // namespace weedhip
