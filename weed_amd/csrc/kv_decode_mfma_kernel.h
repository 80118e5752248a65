#pragma once
// Matrix-core decode attention over the packed cache (gfx950).
//
// One wavefront owns a run of 64-token blocks of the launch's block list (region after region).  Per block it
//   1. streams its lane-major run of packed K items (coalesced 128-bit loads, every byte of the block read once),
//   2. turns every pair of fields into two fp16 values with one conflict-free LDS lookup (each pair-table entry is
//      replicated over the 32 banks) and feeds them as the A operand of v_mfma_f32_16x16x32_f16 against the query,
//      which sits in registers as fp16 hi + lo halves (products of fp16 values are exact in fp32, so the split keeps
//      ~22 bits),
//   3. runs an online softmax on the 16 tokens x 16 heads score tiles in registers (base-2 exponentials; 1/sqrt(d) and
//      log2(e) are folded into the query),
//   4. splits the probabilities (times the V row scales) into fp16 hi + lo, which are already in A-operand order,
//      and multiplies them with the looked-up V items: out[head][coordinate] accumulates in 4*(d/16) registers.
// The wavefronts of a workgroup share the lookup tables; every wavefront leaves one un-normalised partial (m, l, o[d])
// per query head and region segment.  Where the instance allows it (groups of up to 8 heads at head_dim 64 or 128) the
// kernel is the whole decode call: the workgroup rotates, scales and splits the queries of its regions before its first
// block arrives (MfmaQuery), and the partials are merged, un-rotated and stored by the workgroup itself -- through LDS
// when it holds whole regions, through memory and an arrival counter per region otherwise (MfmaMerge).  Else a kernel
// ahead prepares the queries and one behind merges the partials.
//
// Table values are exactly representable in fp16 (the Lloyd-Max tables are generated that way; the uniform coder's
// table is code + 0.5), so de-quantisation itself is exact; the only roundings are those of the fp32 accumulators.
#include "kv_decode_mfma.h"

#include <mutex>
#include <type_traits>

using namespace weedhip;
using namespace weedkv;

namespace weedhip_mfma {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// N dwords from a pointer aligned to 16 bytes when N % 4 == 0, to 8 bytes when N is even, else to 4.
// `base` is the same in every lane and `lane_off` a 32-bit byte offset, so the loads take the scalar-base form (one
// offset register per lane instead of a 64-bit address).
template <int N> __device__ __forceinline__ void load_dwords(const uint8_t *base, uint32_t lane_off, uint32_t (&x)[N])
{
    const uint8_t *p = base + lane_off;
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const uint4v v = *reinterpret_cast<const uint4v *>(p + 16 * i);
            x[4 * i] = v.x;
            x[4 * i + 1] = v.y;
            x[4 * i + 2] = v.z;
            x[4 * i + 3] = v.w;
        }
    } else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const uint2v v = *reinterpret_cast<const uint2v *>(p + 8 * i);
            x[2 * i] = v.x;
            x[2 * i + 1] = v.y;
        }
    } else {
        // odd runs (head_dim 96 with an odd field width): dword by dword
#pragma unroll
        for (int i = 0; i < N; ++i) {
            x[i] = *reinterpret_cast<const uint32_t *>(p + 4 * i);
        }
    }
}

// ---- pair tables in LDS.  Entry e of a table is a row of 256 bytes starting at LDS byte e * 256; the V table uses
//      the first 128 bytes of its rows (32 replicas of the entry, one per bank), the K table the second 128 bytes of
//      rows [0, 2^(2 WK)).  The tables start at LDS address 0 (the kernel has no other LDS), so the byte address of
//      a lookup is  (entry << 8) | lane byte,  lane byte = (lane % 32) * 4 (+ 128 for K): the entry index lands in
//      byte 1 of the address.  When a pair is a whole byte of the packed run (4-bit fields), ONE byte-permute builds
//      the address from the run's dword and the lane byte; otherwise a bit-field extract and a shift-add do. ----
constexpr uint32_t kTableRowBytes = kMfmaTableRowBytes;
template <int WK, int WV> constexpr uint32_t table_rows() { return mfma_table_rows(WK, WV); }

template <int W, int N, int P> __device__ __forceinline__ uint32_t pair_addr(const uint32_t (&x)[N], uint32_t lane_byte)
{
    constexpr int bit = 2 * W * P;
    constexpr int dw = bit >> 5, sh = bit & 31;
    if constexpr (W == 4) {
        // result bytes (3..0) = (0, 0, byte sh/8 of the run's dword, lane byte); selector values 4..7 name the bytes of
        // the first source, 0..3 those of the second, 0x0c a zero byte
        constexpr uint32_t sel = 0x0c0c0000u | ((4u + sh / 8) << 8);
        return __builtin_amdgcn_perm(x[dw], lane_byte, sel);
    } else {
        // (builtins rather than inline assembly: the compiler then knows that no wait state is needed between the two
        // instructions and may interleave the pairs)
        uint32_t t;
        if constexpr (sh + 2 * W <= 32) {
            t = __builtin_amdgcn_ubfe(x[dw], sh, 2 * W);
        } else {
            // the pair straddles two dwords: funnel-shift it down first
            t = __builtin_amdgcn_ubfe(__builtin_amdgcn_alignbit(x[dw + 1 < N ? dw + 1 : dw], x[dw], sh), 0, 2 * W);
        }
        return (t << 8) + lane_byte;
    }
}

// LDS byte address of the single-value entry of field F (5-bit fields): (field << 8) | lane byte.
template <int W, int N, int F> __device__ __forceinline__ uint32_t field_addr(const uint32_t (&x)[N], uint32_t lane_byte)
{
    constexpr int bit = W * F;
    constexpr int dw = bit >> 5, sh = bit & 31;
    uint32_t t, a;
    if constexpr (sh + W <= 32) {
        asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(t) : "v"(x[dw]), "n"(sh), "n"(W));
    } else {
        uint32_t f;
        asm("v_alignbit_b32 %0, %1, %2, %3" : "=v"(f) : "v"(x[dw + 1 < N ? dw + 1 : dw]), "v"(x[dw]), "n"(sh));
        asm("v_bfe_u32 %0, %1, 0, %2" : "=v"(t) : "v"(f), "n"(W));
    }
    asm("v_lshl_add_u32 %0, %1, 8, %2" : "=v"(a) : "v"(t), "v"(lane_byte));
    return a;
}

typedef const uint32_t __attribute__((address_space(3))) *lds_u32_ptr;

__device__ __forceinline__ uint32_t lds_read(uint32_t byte_addr)
{
    return *reinterpret_cast<lds_u32_ptr>((uintptr_t)byte_addr);
}

template <int I, int N, typename F> __device__ __forceinline__ void static_for_fields(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_fields<I + 1, N>(f);
    }
}

// 8-bit fields (uniform coder only, value = code + 0.5): pair P of the run is two bytes of one dword.  A byte-permute
// puts each code under the byte 0x64 -- the fp16 number 1024 + code, exactly -- and one packed fp16 add of -1023.5
// leaves code + 0.5, also exact.
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
template <int N, int P> __device__ __forceinline__ uint32_t pair_from_bytes(const uint32_t (&x)[N])
{
    constexpr int dw = P >> 1, hi = P & 1;
    // result bytes (3..0) = (0x64, code 2P + 1, 0x64, code 2P): selector values 4..7 name the bytes of the first
    // source, 0..3 those of the second
    constexpr uint32_t sel = hi ? 0x00070006u : 0x00050004u;
    uint32_t a;
    asm("v_perm_b32 %0, %1, %2, %3" : "=v"(a) : "v"(x[dw]), "v"(0x64646464u), "s"(sel));
    const half2v h = __builtin_bit_cast(half2v, a) + half2v{ (_Float16)-1023.5f, (_Float16)-1023.5f };
    return __builtin_bit_cast(uint32_t, h);
}

// 6- and 7-bit fields (uniform coder only): the same arithmetic, with the two codes of a pair cut out of the run by
// bit-field extracts (a funnel shift first where a code straddles two dwords).
template <int W, int N, int F> __device__ __forceinline__ uint32_t field_bits(const uint32_t (&x)[N])
{
    constexpr int bit = W * F;
    constexpr int dw = bit >> 5, sh = bit & 31;
    uint32_t t;
    if constexpr (sh + W <= 32) {
        asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(t) : "v"(x[dw]), "n"(sh), "n"(W));
    } else {
        uint32_t f;
        asm("v_alignbit_b32 %0, %1, %2, %3" : "=v"(f) : "v"(x[dw + 1 < N ? dw + 1 : dw]), "v"(x[dw]), "n"(sh));
        asm("v_bfe_u32 %0, %1, 0, %2" : "=v"(t) : "v"(f), "n"(W));
    }
    return t;
}
template <int W, int N, int P> __device__ __forceinline__ uint32_t pair_from_fields(const uint32_t (&x)[N])
{
    const uint32_t lo = field_bits<W, N, 2 * P>(x), hi = field_bits<W, N, 2 * P + 1>(x);
    const uint32_t a = (lo | (hi << 16)) | 0x64006400u; // fp16 (1024 + code) twice
    const half2v h = __builtin_bit_cast(half2v, a) + half2v{ (_Float16)-1023.5f, (_Float16)-1023.5f };
    return __builtin_bit_cast(uint32_t, h);
}

// Item K (8 fields) of the lane's run -> 8 fp16 values in matrix-operand order.
template <int W, int N, int K>
__device__ __forceinline__ half8 dequant_item(const uint32_t (&x)[N], uint32_t lane_byte)
{
    uint4v r;
    if constexpr (W == 6 || W == 7) {
        r.x = pair_from_fields<W, N, 4 * K>(x);
        r.y = pair_from_fields<W, N, 4 * K + 1>(x);
        r.z = pair_from_fields<W, N, 4 * K + 2>(x);
        r.w = pair_from_fields<W, N, 4 * K + 3>(x);
        return __builtin_bit_cast(half8, r);
    }
    if constexpr (W == 8) {
        r.x = pair_from_bytes<N, 4 * K>(x);
        r.y = pair_from_bytes<N, 4 * K + 1>(x);
        r.z = pair_from_bytes<N, 4 * K + 2>(x);
        r.w = pair_from_bytes<N, 4 * K + 3>(x);
        return __builtin_bit_cast(half8, r);
    }
    if constexpr (W == 5) {
        // every entry holds its value in both halves: low half from the even field, high half from the odd one
        uint32_t v[8];
        static_for_fields<0, 8>([&](auto fc) {
            constexpr int f = decltype(fc)::value;
            v[f] = lds_read(field_addr<W, N, 8 * K + f>(x, lane_byte));
        });
        r.x = (v[0] & 0xffffu) | (v[1] & 0xffff0000u);
        r.y = (v[2] & 0xffffu) | (v[3] & 0xffff0000u);
        r.z = (v[4] & 0xffffu) | (v[5] & 0xffff0000u);
        r.w = (v[6] & 0xffffu) | (v[7] & 0xffff0000u);
        return __builtin_bit_cast(half8, r);
    }
    r.x = lds_read(pair_addr<W, N, 4 * K>(x, lane_byte));
    r.y = lds_read(pair_addr<W, N, 4 * K + 1>(x, lane_byte));
    r.z = lds_read(pair_addr<W, N, 4 * K + 2>(x, lane_byte));
    r.w = lds_read(pair_addr<W, N, 4 * K + 3>(x, lane_byte));
    return __builtin_bit_cast(half8, r);
}

// Compile-time loop: f(std::integral_constant<int, I>) for I = 0..N-1.
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ float4v mfma16(half8 a, half8 b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// ---- cross-lane helpers.  A wavefront is 4 rows of 16 lanes; DPP moves data inside a row. ----
template <int CTRL, int BANK_MASK> __device__ __forceinline__ uint32_t dpp_u32(uint32_t old, uint32_t src)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, 0xf, BANK_MASK, false);
}
template <int CTRL, int BANK_MASK> __device__ __forceinline__ float dpp_f32(float old, float src)
{
    return __uint_as_float(dpp_u32<CTRL, BANK_MASK>(__float_as_uint(old), __float_as_uint(src)));
}
constexpr int kRowShl = 0x100, kRowShr = 0x110, kRowRor = 0x120;

// Combine over the lanes that hold the same head: c % GP equal inside a row, then the 4 rows.
template <int GP> __device__ __forceinline__ float head_max(float v)
{
    if constexpr (GP <= 4) {
        v = fmaxf(v, dpp_f32<kRowRor + 4, 0xf>(v, v));
    }
    if constexpr (GP <= 8) {
        v = fmaxf(v, dpp_f32<kRowRor + 8, 0xf>(v, v));
    }
    v = fmaxf(v, __shfl_xor(v, 16));
    return fmaxf(v, __shfl_xor(v, 32));
}
template <int GP> __device__ __forceinline__ float head_sum(float v)
{
    if constexpr (GP <= 4) {
        v += dpp_f32<kRowRor + 4, 0xf>(v, v);
    }
    if constexpr (GP <= 8) {
        v += dpp_f32<kRowRor + 8, 0xf>(v, v);
    }
    v += __shfl_xor(v, 16);
    return v + __shfl_xor(v, 32);
}

// Query head that row `x` of this launch's tile stands for under KV head `kvh`: the launch covers the rows
// [head_first, head_first + G) of the group_total heads that share the KV head.
__device__ __forceinline__ uint32_t q_head_of(const MfmaParams &p, uint32_t kvh, uint32_t x)
{
    return p.blocked ? kvh * p.group_total + p.head_first + x : (p.head_first + x) * p.Hkv + kvh;
}

__device__ __forceinline__ float wave_max64(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v = fmaxf(v, __shfl_xor(v, o));
    }
    return v;
}
__device__ __forceinline__ float wave_sum64(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_xor(v, o);
    }
    return v;
}

// A load through a buffer descriptor: one descriptor, the lane's 32-bit byte offset and an offset that is the same in
// every lane, so that a batch of loads needs no address register pair per load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const float *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, (int)bytes, 0x00020000);
}
// COHERENT: the load is served at device scope (it does not hit a line that this XCD's L2 holds from before another
// XCD wrote it), as a relaxed atomic load of device scope is.
template <bool COHERENT = false>
__device__ __forceinline__ float buffer_f32(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off)
{
    constexpr int kDeviceScope = 16; // the sc1 bit of the cache policy
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, (int)uniform_off,
                                                                          COHERENT ? kDeviceScope : 0));
}
__device__ __forceinline__ float lane_value(float v, uint32_t l)
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), (int)l));
}

// Bank mask (4-lane banks of a row) of the lanes [GP*i, GP*i + GP).
template <int GP, int I> constexpr int bank_mask_of() { return ((1 << (GP / 4)) - 1) << (I * GP / 4); }

// GP = number of query-head columns kept per score tile (the group size rounded up to 4, 8 or 16).  The Q.K^T
// instruction always produces 16 columns; with GP < 16 the useful columns of 16/GP tiles are merged into one register
// set before the softmax, so the exponentials and the fp16 splitting run on full registers.
// MODE 1 (WGM): the workgroups merge their regions themselves (see MfmaMerge); every wavefront then has at most one
// segment.  MODE 0: any partition; it merges in the general case (ragged batches) and rotates its queries where
// mfma_decode_merges(GP, D) says so.  MODE 2: as MODE 0 with both of these, for the head_dims whose MODE 0 leaves them
// out because they cost it registers that every other launch would pay for (mfma_decode_general_variant).
template <int D, int WK, int WV, int GP, bool LLOYD, int MODE>
__global__ void __launch_bounds__(64 * mfma_decode_waves_per_wg(GP, D, WK, WV)) decode_mfma_kernel(MfmaParams launch)
{
    constexpr bool WGM = MODE == 1;
    constexpr int kWaves = (int)mfma_decode_waves_per_wg(GP, D, WK, WV);
    MfmaParams p = launch;
    uint32_t wg_index = blockIdx.x; // this workgroup's place among those of its pass
    if constexpr (MODE == 0) {
        if (launch.grid_passes > 1) {
            const uint32_t octet = blockIdx.x >> 3, pass = octet % launch.grid_passes;
            wg_index = (octet / launch.grid_passes) * 8 + (blockIdx.x & 7);
            const uint32_t wg_blocks = kWaves * launch.runs.unit_blocks;
            if (wg_index >= (launch.total_blocks + wg_blocks - 1) / wg_blocks) {
                return; // (the workgroups of a pass were rounded up to a multiple of eight)
            }
            p.head_first = pass * launch.tile_rows;
            p.G = min(launch.tile_rows, launch.group_total - p.head_first);
        }
    }
    constexpr int KS = D / 32;       // Q.K^T k-steps (32 coordinates each); also K items per tile per lane
    constexpr int JB = D / 16;       // 16-coordinate column blocks of the output
    constexpr int NK = KS * WK;      // dwords of packed K per lane per block
    constexpr int NV = D * WV / 32;  // dwords of packed V per lane per block
    constexpr int TPS = 16 / GP;     // score tiles merged into one register set
    constexpr int NSETS = 4 / TPS;   // register sets per 64-token block
    constexpr uint32_t ROWS = table_rows<WK, WV>();

    extern __shared__ uint32_t lds[]; // the lookup tables

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 15, g = lane >> 4;
    constexpr bool lloyd = LLOYD;

    // ---- the lookup tables.  Their words were put together when the cache's tables were set; the workgroup spreads
    //      them over the LDS banks, 16 bytes per thread and step.  The words are requested first thing and stored after
    //      the wavefront has requested its first block and query, so that those loads travel meanwhile.  Every wavefront of the
    //      workgroup calls build_tables exactly once (it contains a barrier). ----
    // The arguments span six 64-byte lines of kernel-argument memory, each a miss of its own when first touched.
    // Naming one value of every line here makes the compiler fetch all of them at once instead of one after the other
    // as the prologue gets to them.
    asm volatile("" ::"s"(p.total_blocks), "s"(p.v.fields), "s"(p.table_image), "s"(p.q_hi), "s"(p.merge.out),
                 "s"(p.query.q));
    constexpr uint32_t kThreads = 64 * kWaves;
    constexpr uint32_t kImgVecs = ROWS * (kTableRowBytes / 16);
    constexpr uint32_t kImgLoads = (kImgVecs + kThreads - 1) / kThreads;
    uint4v timg[kImgLoads ? kImgLoads : 1];
    if constexpr (ROWS != 0) {
        // (the image in memory holds every entry once; its 32 replicas over the banks are made here: 16-byte piece i
        // of the LDS image is four times word i / 8)
#pragma unroll
        for (uint32_t u = 0; u < kImgLoads; ++u) {
            const uint32_t w = p.table_image[min(tid + u * kThreads, kImgVecs - 1) / 8];
            timg[u] = uint4v{ w, w, w, w };
        }
    }
    auto build_tables = [&]() {
        if constexpr (ROWS == 0) {
            return; // no tables, hence no barrier either
        }
        uint4v *dst = reinterpret_cast<uint4v *>(lds);
#pragma unroll
        for (uint32_t u = 0; u < kImgLoads; ++u) {
            const uint32_t i = tid + u * kThreads;
            if (i < kImgVecs) {
                dst[i] = timg[u];
            }
        }
        __syncthreads();
    };
    bool tables_ready = false;
    const uint32_t vbase = (lane & 31) * 4; // lane byte of a V lookup
    const uint32_t kbase = vbase + 128;     // lane byte of a K lookup

    // ---- this wavefront's share of the launch: a contiguous run (see RunGeom) of 64-token blocks of the global block
    //      list (all blocks of (sequence 0, kv head 0), then (0, 1), ...).  A run is cut into segments at region
    //      boundaries; every segment leaves one partial in the slot `unit - first unit of the region`. ----
    // `unit`: position index of this wavefront's run (runs are numbered along the block list)
    const uint32_t unit =
        __builtin_amdgcn_readfirstlane(wg_index * kWaves + run_position_of_wave(p.runs, wave));
    // Runs that take turns (RunGeom::group_cycles; instances whose workgroups merge only): g0 .. g1 are then the blocks
    // of the run's whole group, of which this wavefront takes its `turn_count` blocks -- one segment, since no group
    // crosses a region boundary.  In turn i the runs that are still short of their length take one block each, ordered
    // by (class, cycle); the youngest class drops out after u0 turns, the middle one (three classes) after u1.  Block
    // number i of a run, counted from the group's first block, is therefore
    // turn_at + turn_cycles * (i + min(i, u0) + min(i, u1))   (u1 = 0 with two classes).
    constexpr uint32_t kClasses = kWaves / 4;
    const uint32_t turn_cycles = WGM ? p.runs.group_cycles : 0u; // 0, 1, 2 or 4
    const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave); // (the same in all lanes: block indices stay scalar)
    const uint32_t age_class = wave_s >> 2, cycle_in_group = (wave_s & 3) & (turn_cycles - 1u);
    const uint32_t turn_at = age_class * turn_cycles + cycle_in_group;
    const uint32_t turn_count =
        (uint32_t)((int)p.runs.unit_blocks + (int)p.runs.skew * ((int)kClasses - 1 - 2 * (int)age_class) / ((int)kClasses - 1));
    const uint32_t turn_u0 = p.runs.unit_blocks - p.runs.skew, turn_u1 = kClasses == 3 ? p.runs.unit_blocks : 0u;
    uint32_t g0 = __builtin_amdgcn_readfirstlane(
        turn_cycles ? (unit - (cycle_in_group * kClasses + age_class)) * p.runs.unit_blocks : run_begin(p.runs, unit));
    const uint32_t g1 = min(g0 + (turn_cycles ? turn_cycles * kClasses * p.runs.unit_blocks
                                              : run_len(p.runs, (unit % kWaves) % run_classes(p.runs))),
                            p.total_blocks);
    // ---- merge inside the kernel (see MfmaMerge): LDS behind the tables, and this thread's share of the rotation ----
    static_assert(!WGM || mfma_decode_merges_whole_regions(GP, D, kWaves), "this instance cannot merge");
    static_assert(MODE != 2 || mfma_decode_general_variant(GP, D, kWaves), "there is no such variant of this instance");
    constexpr bool kCanMerge = MODE != 0 ? mfma_decode_merges_whole_regions(GP, D, kWaves) : mfma_decode_merges(GP, D);
    constexpr bool kQuery = kCanMerge;   // this instance can rotate its queries itself (MfmaQuery)
    // (head_dim 96: a wavefront's 64 threads are not all in one row; what is a scalar elsewhere is per thread there)
    constexpr bool kRowPerWave = D % 64 == 0;
    float *const part_s = reinterpret_cast<float *>(lds) + ROWS * (kTableRowBytes / 4); // [position][GP][D + 2]
    // The two small rotations (queries ahead of the loop, merged rows behind it) run on the fp32 matrix instruction
    // v_mfma_f32_16x16x4f32: tile w < D / 16 is the output columns [16 w, 16 w + 16) of up to 16 rows.  Step s of
    // D / 4 contracts over the coordinates 4 s + g (g = lane / 16): lane (c, g) supplies row c's coordinate 4 s + g
    // from LDS and the rotation's element [4 s + g][16 w + c], which it holds in a register.  The rows lie in LDS as
    // [row][g][s] with a pitch of D + 4 floats, so that a lane's D / 4 values are contiguous (16-byte reads) and the
    // sixteen rows' reads fall into different banks.
    constexpr uint32_t SG = D / 4;       // steps = coordinates per lane
    constexpr uint32_t NT = (D / 16 + kWaves - 1) / kWaves; // tiles per wavefront: tile wave + t * kWaves, t < NT
    constexpr uint32_t kQRows = mfma_query_rows(D);
    constexpr uint32_t RPITCH = D + 4;   // floats per staged row
    auto staged_at = [](uint32_t row, uint32_t j) { return row * RPITCH + (j % 4) * SG + j / 4; };
    // element s of the lane's share of a rotation matrix m (row-major [D][D], out[t] = sum_j in[j] * m[j][t])
    // (Where a wavefront has two tiles, at head_dim 256, it holds one at a time: both together are half of its
    // registers, and the loop's state lies in the others.)
    auto request_matrix = [&](const float *m, float (&x)[kCanMerge ? SG : 1], uint32_t t) {
        if constexpr (kCanMerge) {
            const uint32_t tile = wave + t * kWaves;
            if (tile < D / 16) {
                const __amdgpu_buffer_rsrc_t rot = buffer_of(m, 4 * D * D);
#pragma unroll
                for (uint32_t s_ = 0; s_ < SG; ++s_) {
                    x[s_] = buffer_f32(rot, 4 * (g * D + 16 * tile + c), 16 * D * s_);
                }
            }
        }
    };
    // rows r0 .. r0 + 15 of `staged` (staged_at layout) times the matrix whose elements the lane holds in x: lane
    // (c, g), register v of the result = row r0 + 4 g + v, column 16 * tile + c
    auto rotate_staged = [&](const float *staged, uint32_t r0, const float (&x)[kCanMerge ? SG : 1]) -> float4v {
        float4v acc = { 0.0f, 0.0f, 0.0f, 0.0f };
        if constexpr (kCanMerge) {
            const float4v *mine = reinterpret_cast<const float4v *>(staged + (r0 + c) * RPITCH + g * SG);
            float4v in[SG / 4];
#pragma unroll
            for (uint32_t u = 0; u < SG / 4; ++u) {
                in[u] = mine[u];
            }
#pragma unroll
            for (uint32_t s_ = 0; s_ < SG; ++s_) {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(in[s_ / 4][s_ % 4], x[s_], acc, 0, 0, 0);
            }
        }
        return acc;
    };
    float xrot[kCanMerge ? SG : 1];
    auto request_rotation = [&]() {
        if constexpr (kCanMerge) {
            if (p.merge.unrotate) {
                request_matrix(p.merge.rv, xrot, 0);
            }
        }
    };
    // (The un-rotation's elements are requested when the wavefront is through with its blocks.  Requesting them at the
    // start, where two wavefronts per SIMD have the registers for them, adds 16 MB of L2 traffic to the start of the
    // launch and made the kernel 0.4 us slower.)
    // ---- query rotation inside the kernel (see MfmaQuery).  Row (region ri of the workgroup, head slot hs) has index
    //      ri * G + hs.  Requested here: this thread's share of the K rotation and of the raw queries. ----
    // Where a thread is a column of a row (the raw queries, the merged rows), the workgroup's first kRowsAtOnce * D
    // threads are kRowsAtOnce whole rows; at head_dims that do not divide the threads (160, 192, 224) the rest idle.
    // (Known at compile time where the threads are whole rows, and the same in all lanes of a wavefront where D is a
    // multiple of 64: what depends on it stays scalar, as the rows' address arithmetic must.)
    constexpr uint32_t kRowsAtOnce = kThreads / D;
    const bool row_thread = kRowsAtOnce * D == kThreads ||
        (D % 64 == 0 ? (uint32_t)__builtin_amdgcn_readfirstlane((int)tid) : tid) < kRowsAtOnce * D;
    constexpr uint32_t QPT = kQuery ? (kQRows + kRowsAtOnce - 1) / kRowsAtOnce : 1; // raw query elements per thread
    constexpr uint32_t PW = mfma_merge_partials_words(kWaves, GP, D);
    float *const qraw_s = part_s;                                       // [rows (+ 8 that a tile of 16 reaches into)] staged
    constexpr uint32_t kRotatedRows = mfma_rotated_query_rows(D);
    float *const qrot_s = part_s + (kQRows + 8) * RPITCH;       // [kRotatedRows][D] rotated rows of a pass
    uint16_t *const qh_s = reinterpret_cast<uint16_t *>(part_s + PW); // [rows][D] fp16 high halves
    uint16_t *const ql_s = qh_s + kQRows * D;                 // [rows][D] low halves
    float *const qscale_s = part_s + PW + kQRows * D;         // [rows]
    float *const qsum_s = qscale_s + kQRows;                  // [rows]
    const bool fused_q = kQuery && p.query.q != nullptr;
    // ---- general merge (see MfmaMerge): in a ragged batch every wavefront keeps the prefix sums of the sequences'
    //      block counts in a register, lane i the blocks ahead of sequence i (lanes from n_seq on: all blocks) ----
    const bool general = kQuery && !WGM && p.merge.general != 0;
    const bool own_offsets = general && p.uniform_blocks == 0;
    uint32_t off_lane = 0;
    if constexpr (kQuery && !WGM) {
        if (own_offsets) {
            const uint32_t nbl = lane < p.n_seq ? ((uint32_t)p.cached_lens[lane] + 63u) >> 6 : 0u;
            uint32_t incl = nbl;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t t = __shfl_up(incl, o);
                incl += lane >= (uint32_t)o ? t : 0u;
            }
            off_lane = incl - nbl;
        }
    }
    // blocks ahead of sequence i (i the same in all lanes)
    auto blk_off_at = [&](uint32_t i) -> uint32_t {
        if (p.uniform_blocks) {
            return i * p.uniform_blocks;
        }
        if (own_offsets) {
            return (uint32_t)__builtin_amdgcn_readlane((int)off_lane, (int)i);
        }
        return p.blk_off[i];
    };
    // sequence that holds block b of the list (b the same in all lanes): the largest s with blk_off[s] * Hkv <= b
    // (sequences without tokens share their offset with the next one)
    auto seq_of_block = [&](uint32_t b) -> uint32_t {
        if (p.uniform_blocks) {
            return b / (p.uniform_blocks * p.Hkv);
        }
        if (own_offsets) {
            const bool le = lane < p.n_seq && off_lane * p.Hkv <= b; // true for a prefix of the lanes, lane 0 included
            return (uint32_t)__builtin_popcountll(__ballot(le)) - 1u;
        }
        // a 64-way search, one probe per lane and step
        uint32_t lo = 0, hi = p.n_seq;
        while (hi - lo > 1) {
            const uint32_t stride = (hi - lo + 63) >> 6;
            const uint32_t idx = lo + lane * stride;
            const bool le = idx < hi && p.blk_off[idx] * p.Hkv <= b; // true for a prefix of the lanes, lane 0 included
            const uint32_t n_le = (uint32_t)__builtin_popcountll(__ballot(le));
            lo += (n_le - 1) * stride;
            hi = min(lo + stride, hi);
        }
        return __builtin_amdgcn_readfirstlane(lo);
    };
    // region (sequence * Hkv + kv head) that holds block b
    auto region_of_block = [&](uint32_t b) -> uint32_t {
        const uint32_t s_ = seq_of_block(b), first = blk_off_at(s_), nb_ = blk_off_at(s_ + 1) - first;
        return s_ * p.Hkv + (b - first * p.Hkv) / nb_;
    };
    // the regions this workgroup's blocks lie in
    uint32_t wg_region0 = 0, wg_rows = 0;
    if (WGM && p.merge.wg_regions != 0) {
        wg_region0 = blockIdx.x * p.merge.wg_regions;
        wg_rows = p.merge.wg_regions * p.G;
    } else if (WGM) {
        wg_region0 = (blockIdx.x * kWaves * p.runs.unit_blocks) / p.uniform_blocks; // a share of one region
        wg_rows = p.G;
    } else if (fused_q || general) {
        const uint32_t wg_blocks = kWaves * p.runs.unit_blocks;
        const uint32_t first = blockIdx.x * wg_blocks, last = min(first + wg_blocks, p.total_blocks) - 1;
        wg_region0 = region_of_block(first);
        wg_rows = (region_of_block(last) - wg_region0 + 1) * p.G;
    }
    float xq[kQuery ? SG : 1], qr[QPT];
    auto request_queries = [&]() {
      if constexpr (kQuery) {
        if (fused_q) {
            if (p.query.rotate) {
                request_matrix(p.query.rot_t, xq, 0);
            }
            const uint32_t n_regions = p.n_seq * p.Hkv;
            // thread (row tid / D + i * kRowsAtOnce, column tid % D): where D is a multiple of 64 the row is the same in
            // all lanes of a wavefront, so the row's address arithmetic is scalar
            static_assert(kRowsAtOnce >= 1, "the workgroup's threads are at least one row");
            const uint32_t row_of_wave = kRowPerWave ? __builtin_amdgcn_readfirstlane(tid / D) : tid / D, j = tid % D;
#pragma unroll
            for (uint32_t i = 0; i < QPT; ++i) {
                const uint32_t row = row_of_wave + i * kRowsAtOnce;
                const uint32_t ri = row / p.G, hs = row - ri * p.G, region = wg_region0 + ri;
                float v = 0.0f;
                if (row_thread && row < wg_rows && region < n_regions) {
                    const uint32_t s_ = region / p.Hkv, kv_ = region - s_ * p.Hkv;
                    const float *qrow = p.query.q + (uint64_t)p.query.qg.off + (uint64_t)s_ * p.query.qg.s[0] +
                                        head_offset(p.query.qg, q_head_of(p, kv_, hs));
                    if (j < p.merge.d_real) {
                        v = qrow[(uint64_t)j * p.query.qg.s[2]];
                    }
                }
                qr[i] = v;
            }
        }
      }
    };
    // (Asking for the first block of packed data before these requests gets that block on its way 2 us earlier and the
    // loop going 0.7 us earlier, and the kernel 0.6 us slower: measured, not kept.)
    request_queries();
    // The workgroup's queries: rotated on the matrix instruction (see rotate_staged), then one wavefront per row scales,
    // normalises and splits the row as the stand-alone kernel does.  Contains the tables' barrier; every wavefront calls it once.
    auto rotate_queries = [&]() {
        if constexpr (kQuery) {
#pragma unroll
            for (uint32_t i = 0; i < QPT; ++i) {
                const uint32_t row = tid / D + i * kRowsAtOnce;
                if (row_thread && row < kQRows) {
                    qraw_s[staged_at(row, tid % D)] = qr[i];
                }
            }
            build_tables(); // (its barrier also makes the raw queries visible)
            if constexpr (ROWS == 0) {
                __syncthreads(); // (no tables, no barrier of theirs)
            }
            for (uint32_t r0 = 0; r0 < wg_rows; r0 += kMfmaMergeRows) {
                if (p.query.rotate) {
                    // (with two tiles per wavefront: all sixteen rows in the first pass, tile after tile)
                    if (NT == 1 || r0 == 0) {
#pragma unroll
                        for (uint32_t t = 0; t < NT; ++t) {
                            const uint32_t tile = wave + t * kWaves;
                            if (t > 0) {
                                request_matrix(p.query.rot_t, xq, t);
                            }
                            if (tile < D / 16) {
                                const float4v rot = rotate_staged(qraw_s, r0, xq);
                                if (g < kRotatedRows / 4) {
#pragma unroll
                                    for (uint32_t v = 0; v < 4; ++v) {
                                        qrot_s[(4 * g + v) * D + 16 * tile + c] = rot[v];
                                    }
                                }
                            }
                        }
                    }
                    __syncthreads();
                }
                if (wave < kMfmaMergeRows && r0 + wave < wg_rows) {
                    const uint32_t row = r0 + wave;
                    constexpr uint32_t CPL = (D + 63) / 64;
                    float a[CPL];
                    const float k = 1.4426950408889634f / sqrtf((float)p.merge.d_real);
                    float mx = 0.0f, sum = 0.0f;
#pragma unroll
                    for (uint32_t cc = 0; cc < CPL; ++cc) {
                        const uint32_t j = lane + 64 * cc;
                        float v = 0.0f;
                        if (D % 64 == 0 || j < D) {
                            v = p.query.rotate ? qrot_s[(NT == 1 ? wave : row) * D + j] : qraw_s[staged_at(row, j)];
                        }
                        a[cc] = v;
                        const float qc = v * k;
                        mx = fmaxf(mx, fabsf(qc));
                        sum += qc;
                    }
                    mx = wave_max64(mx);
                    sum = wave_sum64(sum);
                    int e = 0;
                    (void)frexpf(mx, &e);
                    e = e < -100 ? -100 : (e > 100 ? 100 : e);
                    const float inv = ldexpf(1.0f, -e);
#pragma unroll
                    for (uint32_t cc = 0; cc < CPL; ++cc) {
                        const uint32_t j = lane + 64 * cc;
                        const float qn = a[cc] * k * inv;
                        const _Float16 hi = (_Float16)qn;
                        const _Float16 lo = (_Float16)(qn - (float)hi);
                        if (D % 64 == 0 || j < D) {
                            qh_s[row * D + j] = __builtin_bit_cast(uint16_t, hi);
                            ql_s[row * D + j] = __builtin_bit_cast(uint16_t, lo);
                        }
                    }
                    if (lane == 0) {
                        qscale_s[row] = ldexpf(1.0f, e);
                        qsum_s[row] = sum;
                    }
                }
                __syncthreads(); // the rows are there; the partial sums may be overwritten
            }
        }
    };
    const bool has_blocks = g0 < g1;
    if (g0 >= g1 && !tables_ready) {
        // a wavefront without blocks
        if (fused_q) {
            rotate_queries();
        } else {
            build_tables();
        }
        tables_ready = true;
    }
    uint32_t seq = 0;
    const uint32_t uniform_nb = p.uniform_blocks;
    if (g0 >= g1) {
        // (nothing to find)
    } else {
        seq = seq_of_block(g0);
    }
    if constexpr (kQuery && !WGM) {
        // (ahead of the loop over the segments, which must not carry the requested elements around)
        if (fused_q && !tables_ready) {
            rotate_queries();
            tables_ready = true;
        }
    }
    while (g0 < g1) {
    const uint32_t seq_first = blk_off_at(seq);
    // blocks the cached length of this sequence spans
    const uint32_t nb_cap = uniform_nb ? uniform_nb : blk_off_at(seq + 1) - seq_first;
    if constexpr (!WGM) {
        if (nb_cap == 0) {
            ++seq;
            continue;
        }
    }
    const uint32_t rel = g0 - seq_first * p.Hkv;
    const uint32_t kvh = rel / nb_cap;
    const uint32_t b0 = rel - kvh * nb_cap;
    const uint32_t seg = min(nb_cap - b0, g1 - g0);
    const uint32_t slot = unit - run_of_block(p.runs, seq_first * p.Hkv + kvh * nb_cap);
    const uint32_t L = (uint32_t)p.lens[seq]; // may be shorter than the cached length (prefix attention)
    const uint32_t b1 = min(b0 + seg, (L + 63) >> 6);
    const uint64_t region = (uint64_t)seq * p.Hkv + kvh;
    g0 += seg;
    // after merging, this lane works on head c % GP of tile (set * TPS + c / GP)
    const uint32_t hc = c % GP;
    const uint32_t tile_in_set = c / GP;

    // region bases are the same in every lane; the lane's share is a 32-bit offset
    const uint8_t *kreg = p.k.fields + region * p.k.region_bytes;
    const uint8_t *vreg = p.v.fields + region * p.v.region_bytes;
    const uint32_t klane = lane * (4 * NK), vlane = lane * (4 * NV);
    const float *ka = lloyd ? p.k.alpha + region * p.padded : nullptr;
    const float *va = lloyd ? p.v.alpha + region * p.padded : nullptr;
    const uint32_t alane = 16 * tile_in_set + 4 * g;

    // Register buffers for the packed block: one (refilled as soon as its last reader is done: K right after the
    // Q.K^T phase, V right after the P.V phase), or two when the shape is double-buffered (the whole next block is
    // requested before the current one is touched).
    constexpr int NB = mfma_decode_double_buffered(GP, D, WK, WV) ? 2 : 1;
    uint32_t kraw_[NB][NK], vraw_[NB][NV];
    float4v ak_[NB][NSETS], av_[NB][NSETS];

    auto load_k = [&](auto pc, uint32_t blk) {
        constexpr int P = decltype(pc)::value;
        load_dwords<NK>(kreg + (uint64_t)blk * (8u * D * WK), klane, kraw_[P]);
#pragma unroll
        for (int s = 0; s < NSETS; ++s) {
            if constexpr (lloyd) {
                ak_[P][s] = *reinterpret_cast<const float4v *>(ka + blk * 64 + 16 * TPS * s + alane);
            } else {
                ak_[P][s] = float4v{ p.k.alpha_const, p.k.alpha_const, p.k.alpha_const, p.k.alpha_const };
            }
        }
    };
    auto load_v = [&](auto pc, uint32_t blk) {
        constexpr int P = decltype(pc)::value;
        load_dwords<NV>(vreg + (uint64_t)blk * (8u * D * WV), vlane, vraw_[P]);
#pragma unroll
        for (int s = 0; s < NSETS; ++s) {
            if constexpr (lloyd) {
                av_[P][s] = *reinterpret_cast<const float4v *>(va + blk * 64 + 16 * TPS * s + alane);
            } else {
                av_[P][s] = float4v{ 1.0f, 1.0f, 1.0f, 1.0f };
            }
        }
    };

    // The first block of the segment is requested before anything else of the segment is read (the sequence's
    // attended length, the query): it exists whatever that length is, and its latency is the longest of the prologue.
    // (A partition that counts more blocks per region than the cache holds may put b0 behind the region's memory:
    // such a segment has no tokens and what is read for it is not used, but it is read from inside the region.)
    constexpr std::integral_constant<int, 0> p0{};
    // block number i of this wavefront in the segment (an index into the region); ~0 behind its last one
    auto nth_block = [&](uint32_t i) -> uint32_t {
        return i < turn_count ? b0 + turn_at + turn_cycles * (i + min(i, turn_u0) + min(i, turn_u1)) : ~0u;
    };
    const uint32_t first_read = min(turn_cycles ? b0 + turn_at : b0, (p.padded >> 6) - 1u);
    load_k(p0, first_read);
    load_v(p0, first_read);

    // ---- query operand.  The score instruction has 16 columns.  With GP <= 8 the fp16 high halves of the GP heads sit
    //      in columns [0, GP) and the low halves in [GP, 2GP), so ONE instruction per item yields both partial scores
    //      (they are added with a lane shift afterwards); with GP = 16 the halves take two instructions. ----
    constexpr bool PACKED = GP <= 8;
    constexpr int NQ = PACKED ? 1 : 2;
    half8 qop[NQ][KS];
    if (fused_q) {
        if constexpr (kQuery) {
            if constexpr (WGM) {
                // (the only segment: the first block is on its way meanwhile)
                rotate_queries();
                tables_ready = true;
            }
            const uint32_t col_head = PACKED ? c % GP : c;
            const uint32_t col_part = PACKED ? c / GP : 0; // 0: high half, 1: low half, above: unused column
            const bool col_ok = col_head < p.G && col_part < 2;
            const uint32_t at = (((uint32_t)region - wg_region0) * p.G + (col_ok ? col_head : 0)) * D + g * (D / 4);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                uint4v hi = { 0, 0, 0, 0 }, lo = { 0, 0, 0, 0 };
                if (col_ok) {
                    if (!PACKED || col_part == 0) {
                        hi = *reinterpret_cast<const uint4v *>(qh_s + at + 8 * ks);
                    }
                    if (!PACKED || col_part == 1) {
                        lo = *reinterpret_cast<const uint4v *>(ql_s + at + 8 * ks);
                    }
                }
                if constexpr (PACKED) {
                    qop[0][ks] = __builtin_bit_cast(half8, col_part ? lo : hi);
                } else {
                    qop[0][ks] = __builtin_bit_cast(half8, hi);
                    qop[NQ - 1][ks] = __builtin_bit_cast(half8, lo);
                }
            }
        }
    } else {
        const uint32_t col_head = PACKED ? c % GP : c;
        const uint32_t col_part = PACKED ? c / GP : 0; // 0: high half, 1: low half, above: unused column
        const bool col_ok = col_head < p.G && col_part < 2;
        const uint32_t qh = col_ok ? q_head_of(p, kvh, col_head) : 0;
        const uint64_t qbase = ((uint64_t)seq * p.Hq + qh) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4v hi = { 0, 0, 0, 0 }, lo = { 0, 0, 0, 0 };
            if (col_ok) {
                hi = *reinterpret_cast<const uint4v *>(p.q_hi + qbase + 8 * ks);
                lo = *reinterpret_cast<const uint4v *>(p.q_lo + qbase + 8 * ks);
            }
            if constexpr (PACKED) {
                qop[0][ks] = __builtin_bit_cast(half8, col_part ? lo : hi);
            } else {
                qop[0][ks] = __builtin_bit_cast(half8, hi);
                qop[NQ - 1][ks] = __builtin_bit_cast(half8, lo);
            }
        }
    }
    const bool head_ok = hc < p.G;
    // tokens at the end of the region that this lane's (position, head) pair does not see (0 unless the call is a
    // multi-token chunk), and the largest such count over the pairs
    const uint32_t hidden_max = p.q_tokens - 1U;
    const uint32_t pair = p.head_first + hc; // index of the (position, head) pair among those of the KV head
    const uint32_t hidden = (hidden_max && head_ok) ? hidden_max - (p.blocked ? pair % p.q_tokens : pair / p.real_group) : 0U;
    const uint32_t qh_c = head_ok ? q_head_of(p, kvh, hc) : 0;
    float qscale = 0.0f, betaq = 0.0f;
    if (fused_q) {
        const uint32_t row = ((uint32_t)region - wg_region0) * p.G + hc;
        if (head_ok) {
            qscale = qscale_s[row];
            betaq = p.k.beta * qsum_s[row];
        }
    } else if (head_ok) {
        qscale = p.q_scale[(uint64_t)seq * p.Hq + qh_c];
        betaq = p.k.beta * p.q_sum[(uint64_t)seq * p.Hq + qh_c];
    }

    // ---- The running maximum is only raised when a block exceeds it by more than 2^kSlack, so most blocks skip the
    //      rescaling of the output accumulators; probabilities may therefore reach 2^kSlack.  `ep` is the exponent
    //      that keeps probability * V-row-scale * 2^ep below 2^15, inside fp16's range. ----
    constexpr float kSlack = 8.0f;
    int ep = 7;
    if (lloyd) {
        uint32_t bits = 0; // (non-negative floats order like their bit patterns)
#pragma unroll
        for (uint32_t i = 0; i < kScaleMaxSlots; ++i) {
            bits = max(bits, p.v.alpha_max[region * kScaleMaxSlots + i]);
        }
        ep = bits ? 133 - (int)((bits >> 23) & 0xff) : 0;
        ep = ep > 100 ? 100 : (ep < -100 ? -100 : ep);
    }
    const float unscale = __uint_as_float((uint32_t)(127 - ep) << 23); // 2^-ep

    if (!tables_ready) {
        build_tables(); // while the first block and the query are on their way, and before the accumulators exist
        tables_ready = true;
    }

    float m_run = -INFINITY; // running maximum of this lane's head (same value in every lane that shares the head)
    float l_run = 0.0f;      // this lane's share of the running denominator, scaled by 2^ep
    float4v O[JB];           // lane (c, g), register r: head slot 4g + r, coordinate 16*jb + c
#pragma unroll
    for (int jb = 0; jb < JB; ++jb) {
        O[jb] = float4v{ 0.0f, 0.0f, 0.0f, 0.0f };
    }

    auto process_block = [&](auto pc, uint32_t blk, uint32_t next_blk) {
        constexpr int P = decltype(pc)::value;
        constexpr std::integral_constant<int, (NB == 2 ? 1 - P : 0)> other{};
        auto &kraw = kraw_[P];
        auto &vraw = vraw_[P];
        auto &ak = ak_[P];
        auto &av = av_[P];
        if constexpr (NB == 2) {
            // double buffering: the whole next block is requested before this one is touched
            load_k(other, next_blk);
            load_v(other, next_blk);
        }
        // ---- S[t] = K_tile . q: rows = tokens 16t + (lane%16), contraction over the lane groups' coordinates.
        //      Items are taken in memory order (tile after tile); lookups run two items ahead of the matrix
        //      instructions that consume them. ----
        float4v S[4];
        {
            constexpr int NI = 4 * KS;
            half8 a0 = dequant_item<WK, NK, 0>(kraw, kbase);
            half8 a1 = dequant_item<WK, NK, 1>(kraw, kbase);
            static_for<0, NI>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int t = i / KS, ks = i % KS;
                half8 a2 = a1;
                if constexpr (i + 2 < NI) {
                    a2 = dequant_item<WK, NK, i + 2>(kraw, kbase);
                }
                // keep the look-ahead lookups ahead of this item's matrix instruction
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (ks == 0) {
                    S[t] = mfma16(a0, qop[0][0], float4v{ 0.0f, 0.0f, 0.0f, 0.0f });
                } else {
                    S[t] = mfma16(a0, qop[0][ks], S[t]);
                }
                if constexpr (!PACKED) {
                    S[t] = mfma16(a0, qop[NQ - 1][ks], S[t]);
                }
                a0 = a1;
                a1 = a2;
            });
        }

        // ---- merge the useful columns: C[s][r] of lane (c, g) = token 16*(s*TPS + c/GP) + 4g + r, head c % GP ----
        float C[NSETS][4];
#pragma unroll
        for (int s = 0; s < NSETS; ++s) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // columns [0, GP) += columns [GP, 2GP): high-half score + low-half score
                float part[TPS];
#pragma unroll
                for (int i = 0; i < TPS; ++i) {
                    part[i] = S[s * TPS + i][r];
                    if constexpr (PACKED) {
                        part[i] += dpp_f32<kRowShl + (PACKED ? GP : 1), 0xf>(part[i], part[i]);
                    }
                }
                float v = part[0];
                if constexpr (TPS >= 2) {
                    v = dpp_f32<kRowShr + GP, bank_mask_of<GP, 1>()>(v, part[TPS >= 2 ? 1 : 0]);
                }
                if constexpr (TPS >= 4) {
                    v = dpp_f32<kRowShr + 2 * GP, bank_mask_of<GP, 2>()>(v, part[TPS >= 4 ? 2 : 0]);
                    v = dpp_f32<kRowShr + 3 * GP, bank_mask_of<GP, 3>()>(v, part[TPS >= 4 ? 3 : 0]);
                }
                // scores in log2 units
                C[s][r] = fmaf(v, ak[s][r] * qscale, betaq);
            }
        }
        if constexpr (NB == 1) {
            load_k(other, next_blk); // the K buffer is free again
        }
        if (blk * 64 + 64 + hidden_max > L) {
#pragma unroll
            for (int s = 0; s < NSETS; ++s) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (blk * 64 + 16 * (s * TPS + tile_in_set) + 4 * g + r + hidden >= L) {
                        C[s][r] = -INFINITY;
                    }
                }
            }
        }
        float mloc = -INFINITY;
#pragma unroll
        for (int s = 0; s < NSETS; ++s) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                mloc = fmaxf(mloc, C[s][r]);
            }
        }
        mloc = head_max<GP>(mloc);
        const float m_new = fmaxf(m_run, mloc);
        if (__any(mloc > m_run + kSlack)) {
            const float scale = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= scale;
            // output row 4g + r belongs to head (4g + r) % GP (rows [GP, 2GP) hold the low-half products), whose scale
            // lives in lane (4g + r) % GP of row 0
            float sr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sr[r] = __shfl(scale, (int)((4 * g + r) % GP));
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
        // (a chunk's early positions can have a whole block hidden before anything was seen: m_run is still -inf)
        const float mm = (m_run == -INFINITY ? 0.0f : m_run) - (float)ep;

        // ---- probabilities (times V row scale, times 2^ep), split into fp16 hi + lo pairs ----
        uint32_t Phi[NSETS][2], Plo[NSETS][2];
#pragma unroll
        for (int s = 0; s < NSETS; ++s) {
            float pv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(C[s][r] - mm); // exp2(-inf) = 0 masks the tail
                l_run += e;
                pv[r] = e * av[s][r];
            }
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                // hi = top 11 significant bits (exact in fp16), lo = the rest
                const float a0 = pv[2 * h2], a1 = pv[2 * h2 + 1];
                const float h0 = __uint_as_float(__float_as_uint(a0) & 0xffffe000u);
                const float h1 = __uint_as_float(__float_as_uint(a1) & 0xffffe000u);
                Phi[s][h2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(h0, h1));
                Plo[s][h2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a0 - h0, a1 - h1));
            }
        }

        // ---- O[head][coordinate] += P . V over the block's two 32-token halves.  The A operand of half u wants,
        //      in lane (head, g), the tokens 4g..4g+3 of tile 2u (k-slots 0..3) and of tile 2u+1 (k-slots 4..7):
        //      move each tile's pairs back from the lanes they were merged into. ----
        // A operand of half u, lane (row, g): rows [0, GP) carry the high halves of the probabilities of head `row`,
        // rows [GP, 2GP) the low halves (GP <= 8); the tokens are 4g..4g+3 of tile 2u (k-slots 0..3) and of tile
        // 2u+1 (k-slots 4..7).  Each tile's pairs are moved back from the lanes they were merged into.
        half8 pa[2][NQ];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            uint32_t ah[4], al[4];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int t = 2 * u + half;
                const int s = t / TPS;
                constexpr int kQuadId = 0xe4; // quad_perm [0,1,2,3]: no movement, used for bank-masked copies
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    uint32_t xh = Phi[s][h2], xl = Plo[s][h2];
                    const int i = t % TPS; // the tile sits in lanes [GP*i, GP*i + GP)
                    if constexpr (PACKED) {
                        // high halves -> lanes [0, GP), low halves -> lanes [GP, 2GP)
                        uint32_t x = xh;
                        if (i == 1) {
                            x = dpp_u32<kRowShl + GP, bank_mask_of<GP, 0>()>(xh, xh);
                        } else if (i == 2) {
                            x = dpp_u32<kRowShl + (TPS >= 4 ? 2 * GP : 1), bank_mask_of<GP, 0>()>(xh, xh);
                        } else if (i == 3) {
                            x = dpp_u32<kRowShl + (TPS >= 4 ? 3 * GP : 1), bank_mask_of<GP, 0>()>(xh, xh);
                        }
                        if (i == 0) {
                            x = dpp_u32<kRowShr + GP, bank_mask_of<GP, 1>()>(x, xl);
                        } else if (i == 1) {
                            x = dpp_u32<kQuadId, bank_mask_of<GP, 1>()>(x, xl);
                        } else if (i == 2) {
                            x = dpp_u32<kRowShl + GP, bank_mask_of<GP, 1>()>(x, xl);
                        } else {
                            x = dpp_u32<kRowShl + (TPS >= 4 ? 2 * GP : 1), bank_mask_of<GP, 1>()>(x, xl);
                        }
                        ah[2 * half + h2] = x;
                    } else {
                        ah[2 * half + h2] = xh;
                        al[2 * half + h2] = xl;
                    }
                }
            }
            pa[u][0] = __builtin_bit_cast(half8, uint4v{ ah[0], ah[1], ah[2], ah[3] });
            if constexpr (!PACKED) {
                pa[u][NQ - 1] = __builtin_bit_cast(half8, uint4v{ al[0], al[1], al[2], al[3] });
            }
        }
        {
            constexpr int NI = 2 * JB;
            half8 b0v = dequant_item<WV, NV, 0>(vraw, vbase);
            half8 b1v = dequant_item<WV, NV, 1>(vraw, vbase);
            static_for<0, NI>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int u = i / JB, jb = i % JB;
                half8 b2v = b1v;
                if constexpr (i + 2 < NI) {
                    b2v = dequant_item<WV, NV, i + 2>(vraw, vbase);
                }
                __builtin_amdgcn_sched_barrier(0);
                O[jb] = mfma16(pa[u][0], b0v, O[jb]);
                if constexpr (!PACKED) {
                    O[jb] = mfma16(pa[u][NQ - 1], b0v, O[jb]);
                }
                b0v = b1v;
                b1v = b2v;
            });
        }
        if constexpr (NB == 1) {
            load_v(other, next_blk); // the V buffer is free again
        }
    };

    // ---- main loop.  The refills are unconditional (the next block index is clamped to the last block of the
    //      segment) so that the loop body has no branch around loads and outstanding loads can be counted exactly. ----
    if (!WGM || turn_cycles == 0) {
        // contiguous runs
        uint32_t blk = b0;
        if (blk < b1) {
            const uint32_t last = b1 - 1;
            if constexpr (NB == 2) {
                constexpr std::integral_constant<int, 1> p1{};
                for (; blk + 1 < b1; blk += 2) {
                    process_block(p0, blk, blk + 1);
                    process_block(p1, blk + 1, min(blk + 2, last));
                }
                if (blk < b1) {
                    process_block(p0, blk, last);
                }
            } else {
                for (; blk < b1; ++blk) {
                    process_block(p0, blk, min(blk + 1, last));
                }
            }
        }
    } else {
        // runs that take turns (the wavefront's blocks ascend, so the first one at or behind b1 ends the segment)
        uint32_t i = 0, blk = nth_block(0);
        const uint32_t last = b1 - 1; // (only used while blk < b1, so b1 >= 1)
        if constexpr (NB == 2) {
            constexpr std::integral_constant<int, 1> p1{};
            while (blk < b1) {
                const uint32_t second = nth_block(i + 1);
                process_block(p0, blk, min(second, last));
                if (second >= b1) {
                    break;
                }
                const uint32_t third = nth_block(i + 2);
                process_block(p1, second, min(third, last));
                blk = third;
                i += 2;
            }
        } else {
            while (blk < b1) {
                const uint32_t next = nth_block(++i);
                process_block(p0, blk, min(next, last));
                blk = next;
            }
        }
    }

    // ---- this segment's un-normalised partial (m, l, o[d]) per query head: to LDS when the workgroup merges (every
    //      wavefront then has one segment, and its position in the workgroup is its slot), else straight to global
    //      memory ----
    constexpr int PS = D + 2;
    auto leave_partial = [&](auto to_lds) {
        constexpr bool TO_LDS = decltype(to_lds)::value;
        const float l_head = head_sum<GP>(l_run) * unscale; // every lane of a head now holds its denominator
        float lrow[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            lrow[r] = __shfl(l_head, (int)(4 * g + r));
        }
        const float o_mul = unscale * (lloyd ? 1.0f : p.v.alpha_const);
        if constexpr (PACKED) {
            // rows [GP, 2GP) hold the low-half products of heads [0, GP): they sit GP/4 lane rows further up
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    O[jb][r] += __shfl_down(O[jb][r], 4 * GP);
                }
            }
        }
        float *const mine = part_s + run_position_of_wave(p.runs, wave) * (GP * PS);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t hs = 4 * g + r;
            if (hs < p.G) {
                float *dst = TO_LDS ? mine + hs * PS
                                    : p.partials + (((uint64_t)seq * p.Hq + q_head_of(p, kvh, hs)) * p.max_slots + slot) * PS;
#pragma unroll
                for (int jb = 0; jb < JB; ++jb) {
                    // uniform coder: value = step * (code + 0.5) + lo, so add lo * sum(p)
                    const float v = fmaf(O[jb][r], o_mul, p.v.beta * lrow[r]);
                    dst[2 + 16 * jb + c] = v;
                }
            }
        }
        if (g == 0 && c < p.G) {
            // lane c of row 0 holds head c (c < GP)
            float *dst = TO_LDS ? mine + c * PS
                                : p.partials + (((uint64_t)seq * p.Hq + q_head_of(p, kvh, c)) * p.max_slots + slot) * PS;
            dst[0] = m_run;
            dst[1] = l_head;
        }
    };
    if constexpr (WGM) {
        request_rotation(); // on its way while the partial is put together
        leave_partial(std::true_type{});
        break; // (the only segment: for the compiler this is no loop, so nothing is carried around it)
    } else {
        leave_partial(std::false_type{});
    }
    if (kvh + 1 == p.Hkv && b0 + seg == nb_cap) {
        ++seq;
    }
    } // segments

    // ---- the workgroup's merge: rows (region, head) in passes of kMfmaMergeRows ----
    if constexpr (kQuery) {
        if constexpr (WGM) {
            if (!has_blocks) {
                request_rotation(); // (the others did so before they left their partial)
            }
        } else {
            if (!general) {
                return; // a second kernel merges
            }
            request_rotation();
        }
        constexpr int PS = D + 2;
        constexpr uint32_t RP = kMfmaMergeRows;
        float *const o_s = part_s + PW;               // [RP (+ 8 that a tile of 16 reaches into)] merged, normalised rows, staged
        uint32_t *const count_s = reinterpret_cast<uint32_t *>(o_s + mfma_merge_rows_words(D) - 64); // (the area's end)
        // where the pass's rows go: element offset of row rr's first coordinate in the output (~0: no such row), found
        // once per row while the rows are merged
        unsigned long long *const rowbase_s = reinterpret_cast<unsigned long long *>(o_s + 16 * RPITCH);
        const uint32_t n_regions = p.n_seq * p.Hkv;
        // (the row of an element is the same in all lanes of a wavefront where D is a multiple of 64; threads that are
        // not part of a whole row start behind the pass's rows)
        const uint32_t rr_of_wave = !row_thread ? RP : kRowPerWave ? __builtin_amdgcn_readfirstlane(tid / D) : tid / D;
        const uint32_t col = tid % D;
        // rows r0 .. r0 + RP - 1 of the workgroup (row = region index in the workgroup * G + head slot): o_s = the
        // merge of the row's `slots` partials, which partial(ri, hs, k) finds; normalised, or with NORMALISE false
        // left as the partial (m, l, o) that leave(rr, m, l, o) puts somewhere
        auto merge_rows = [&](uint32_t r0, uint32_t rows, uint32_t slots, auto partial, auto normalise, auto leave) {
            constexpr bool NORMALISE = decltype(normalise)::value;
            constexpr uint32_t KS = kWaves; // most partials of a row (one per wavefront)
            for (uint32_t rr = rr_of_wave; rr < RP; rr += kRowsAtOnce) {
                const uint32_t row = r0 + rr;
                float v = 0.0f;
                if (row < rows) {
                    const uint32_t ri = row / p.G, hs = row - ri * p.G;
                    // all reads first (slots that do not exist read the last one again), so that they travel together
                    float m[KS], l[KS], o[KS];
#pragma unroll
                    for (uint32_t k = 0; k < KS; ++k) {
                        const uint32_t kk = min(k, slots - 1);
                        m[k] = partial(ri, hs, kk, 0u);
                        l[k] = partial(ri, hs, kk, 1u);
                        o[k] = partial(ri, hs, kk, 2u + col);
                    }
                    float mx = -INFINITY;
#pragma unroll
                    for (uint32_t k = 0; k < KS; ++k) {
                        mx = k < slots ? fmaxf(mx, m[k]) : mx;
                    }
                    float den = 0.0f, acc = 0.0f;
#pragma unroll
                    for (uint32_t k = 0; k < KS; ++k) {
                        // (the bare instruction, as in the main loop: arguments are <= 0, and a weight below 2^-126 is none)
                        const float w = (k >= slots || m[k] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m[k] - mx);
                        den = fmaf(w, l[k], den);
                        acc = fmaf(w, o[k], acc);
                    }
                    if constexpr (NORMALISE) {
                        v = den > 0.0f ? acc * __builtin_amdgcn_rcpf(den) : 0.0f;
                    } else {
                        leave(ri, hs, mx, den, acc);
                    }
                }
                if constexpr (NORMALISE) {
                    o_s[staged_at(rr, col)] = v;
                }
            }
        };
        // un-rotation of the rows in o_s and the output rows of the regions region_of(ri); `more`: another pass follows
        auto finish_rows = [&](uint32_t r0, uint32_t rows, auto region_of, bool more) {
            if (tid < RP) {
                const uint32_t row = r0 + tid;
                const uint32_t ri = row / p.G, hs = row - ri * p.G;
                unsigned long long base = ~0ull;
                if (row < rows && region_of(ri) < n_regions) {
                    const uint32_t region = region_of(ri);
                    const uint32_t s_ = region / p.Hkv, kv_ = region - s_ * p.Hkv;
                    base = (uint64_t)p.merge.og.off + (uint64_t)s_ * p.merge.og.s[0] +
                           head_offset(p.merge.og, q_head_of(p, kv_, hs));
                }
                rowbase_s[tid] = base;
            }
            __syncthreads(); // the merged rows are complete
            auto store_row = [&](uint32_t rr, uint32_t column, float v) {
                const unsigned long long base = rowbase_s[rr];
                if (base != ~0ull && column < p.merge.d_real) {
                    p.merge.out[base + (uint64_t)column * p.merge.og.s[2]] = v;
                }
            };
            if (p.merge.unrotate) {
#pragma unroll
                for (uint32_t t = 0; t < NT; ++t) {
                    const uint32_t tile = wave + t * kWaves;
                    if (NT > 1 && (t > 0 || r0 > 0)) {
                        request_matrix(p.merge.rv, xrot, t); // (the first pass's first tile is there, see request_rotation)
                    }
                    if (tile < D / 16) {
                        const float4v out = rotate_staged(o_s, 0, xrot);
                        if (g < RP / 4) {
#pragma unroll
                            for (uint32_t v = 0; v < 4; ++v) {
                                store_row(4 * g + v, 16 * tile + c, out[v]);
                            }
                        }
                    }
                }
            } else {
                for (uint32_t rr = rr_of_wave; rr < RP; rr += kRowsAtOnce) {
                    store_row(rr, col, o_s[staged_at(rr, col)]);
                }
            }
            if (more) {
                __syncthreads(); // before the next pass overwrites the rows
            }
        };
        // `count` regions, region_of(i) with slots_of(i) partials each (at most 64, the host sees to that), from memory,
        // in passes of RP rows.  Lane k of every wavefront reads the header of its row's partial k, the wavefront's 64
        // columns of the partials come eight partials at a time; all of these loads are independent of each other (and
        // of device scope), so a pass costs two trips to memory, not one per partial.  Then the rows are finished.
        auto finish_regions_from_memory = [&](uint32_t count, auto region_of, auto slots_of) {
            const uint32_t rows = count * p.G;
            // row rr of the pass (the same in all lanes of the wavefront), this lane's column of it (col_ok: it has one)
            auto one_row = [&](uint32_t r0, uint32_t rr, uint32_t column, bool col_ok) {
                const uint32_t row = r0 + rr;
                float v = 0.0f;
                if (row < rows) {
                    const uint32_t ri = row / p.G, hs = row - ri * p.G;
                    const uint32_t region = region_of(ri), slots = slots_of(ri);
                    const uint32_t s_ = region / p.Hkv, kv_ = region - s_ * p.Hkv;
                    const float *first = p.partials + ((uint64_t)s_ * p.Hq + q_head_of(p, kv_, hs)) * p.max_slots * PS;
                    const __amdgpu_buffer_rsrc_t src = buffer_of(first, slots * (4 * PS));
                    const uint32_t cb = 4 * (col_ok ? column : 0u);
                    float m0 = buffer_f32<true>(src, lane * (4 * PS), 0), l0 = buffer_f32<true>(src, lane * (4 * PS), 4);
                    float y[8];
#pragma unroll
                    for (uint32_t u = 0; u < 8; ++u) {
                        y[u] = buffer_f32<true>(src, cb, 4 * (min(u, slots - 1) * PS + 2));
                    }
                    if (lane >= slots) {
                        m0 = -INFINITY;
                        l0 = 0.0f;
                    }
                    const float mx = wave_max64(m0);
                    const float w0 = (m0 == -INFINITY) ? 0.0f : exp2f(m0 - mx);
                    const float den = wave_sum64(w0 * l0);
                    float acc = 0.0f;
                    for (uint32_t k0 = 0; k0 < slots; k0 += 8) {
                        float z[8];
                        if (k0 + 8 < slots) {
#pragma unroll
                            for (uint32_t u = 0; u < 8; ++u) {
                                z[u] = buffer_f32<true>(src, cb, 4 * (min(k0 + 8 + u, slots - 1) * PS + 2));
                            }
                        }
#pragma unroll
                        for (uint32_t u = 0; u < 8; ++u) {
                            if (k0 + u < slots) {
                                acc = fmaf(lane_value(w0, k0 + u), y[u], acc);
                            }
                        }
#pragma unroll
                        for (uint32_t u = 0; u < 8; ++u) {
                            y[u] = z[u];
                        }
                    }
                    v = den > 0.0f ? acc / den : 0.0f;
                }
                if (col_ok) {
                    o_s[staged_at(rr, column)] = v;
                }
            };
            for (uint32_t r0 = 0; r0 < rows; r0 += RP) {
                if constexpr (kRowPerWave) {
                    for (uint32_t rr = rr_of_wave; rr < RP; rr += kRowsAtOnce) {
                        one_row(r0, rr, col, true);
                    }
                } else {
                    // (a wavefront's threads are not all in one row: wavefront w takes row w, 64 columns at a time)
                    if (wave < RP) {
#pragma unroll
                        for (uint32_t cc = 0; cc < (D + 63) / 64; ++cc) {
                            one_row(r0, wave, lane + 64 * cc, lane + 64 * cc < D);
                        }
                    }
                }
                finish_rows(r0, rows, region_of, r0 + RP < rows);
            }
        };
        if constexpr (!WGM) {
            // General case: this wavefront's partials are stored; when every wavefront's are, the workgroup counts
            // itself in every region it has blocks of (thread t: region wg_region0 + t), and merges those whose count
            // it completes.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            const uint32_t wg_regions_here = wg_rows / p.G, wg_blocks = kWaves * p.runs.unit_blocks;
            if (wave == 0) {
                // The partials were ordinary stores (stores of device scope between a wavefront's segments would hold
                // up the loads of its next segment, which wait on the same counter): they sit in this XCD's L2.  The
                // arrival below is a RELEASE of device scope -- one L2 write-back per workgroup, ordered after every
                // wavefront's stores by the barrier above -- and the workgroup that completes a count takes an ACQUIRE
                // fence of device scope before it reads the region's partials: release / acquire on the counter is what
                // makes the other workgroups' partials visible, not the timing of the caches.
                // (all lanes compute: the offsets travel between lanes)
                const uint32_t region = min(wg_region0 + lane, n_regions - 1);
                const uint32_t s_ = region / p.Hkv, kv_ = region - s_ * p.Hkv;
                uint32_t first, nb_;
                if (p.uniform_blocks) {
                    first = s_ * p.uniform_blocks;
                    nb_ = p.uniform_blocks;
                } else {
                    first = __shfl(off_lane, (int)s_);
                    nb_ = __shfl(off_lane, (int)(s_ + 1)) - first;
                }
                const uint32_t begin = first * p.Hkv + kv_ * nb_, end = begin + nb_ - 1; // (the host refuses empty ones)
                const uint32_t wgs = end / wg_blocks - begin / wg_blocks + 1;
                const uint32_t slots = run_of_block(p.runs, end) - run_of_block(p.runs, begin) + 1;
                uint32_t before_plus_one = 0;
                if (lane < wg_regions_here) {
                    uint32_t before = 0;
                    if (wgs > 1) {
                        before = __hip_atomic_fetch_add(p.merge.arrive + region, 1u, __ATOMIC_RELEASE,
                                                        __HIP_MEMORY_SCOPE_AGENT);
                        if (before + 1 == wgs) {
                            __hip_atomic_store(p.merge.arrive + region, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                    before_plus_one = before + 1;
                }
                // the regions to merge, packed: count_s[1 + 2 i] = region, count_s[2 + 2 i] = its slots, count_s[0] = how many
                // (at most 31, the host sees to that)
                const bool mine = lane < wg_regions_here && before_plus_one == wgs;
                const uint64_t mask = __ballot(mine);
                if (mask) {
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                }
                if (mine) {
                    const uint32_t at = (uint32_t)__builtin_popcountll(mask & ((1ull << lane) - 1ull));
                    count_s[1 + 2 * at] = region;
                    count_s[2 + 2 * at] = slots;
                }
                if (lane == 0) {
                    count_s[0] = (uint32_t)__builtin_popcountll(mask);
                }
            }
            __syncthreads();
            finish_regions_from_memory(
                count_s[0], [&](uint32_t i) { return count_s[1 + 2 * i]; }, [&](uint32_t i) { return count_s[2 + 2 * i]; });
        } else {
        __syncthreads(); // every wavefront's partial is in LDS (and nobody reads the tables any more)
        if (p.merge.wg_regions != 0) {
            // whole regions: slots = wavefronts per region
            const uint32_t slots = kWaves / p.merge.wg_regions, rows = p.merge.wg_regions * p.G;
            auto in_lds = [&](uint32_t ri, uint32_t hs, uint32_t k, uint32_t word) {
                return part_s[((ri * slots + k) * GP + hs) * PS + word];
            };
            for (uint32_t r0 = 0; r0 < rows; r0 += RP) {
                merge_rows(r0, rows, slots, in_lds, std::true_type{}, [](uint32_t, uint32_t, float, float, float) {});
                finish_rows(r0, rows, [&](uint32_t ri) { return blockIdx.x * p.merge.wg_regions + ri; }, r0 + RP < rows);
            }
        } else {
            // A share of ONE region: the wavefronts' partials become one partial of the region in
            // memory; behind a barrier ONE thread counts the workgroup with a RELEASE of device scope, and the
            // workgroup that completes the region's count takes an ACQUIRE fence of device scope, then reads all of
            // the region's partials and finishes the rows.  (One write-back per workgroup and one invalidation per
            // region: every wavefront issuing them costs more than the whole merge.)
            const uint32_t wg_blocks = kWaves * p.runs.unit_blocks;
            const uint32_t region = (blockIdx.x * wg_blocks) / p.uniform_blocks;
            const uint32_t my_slot = blockIdx.x - (region * p.uniform_blocks) / wg_blocks;
            const uint32_t s_ = region / p.Hkv, kv_ = region - s_ * p.Hkv;
            auto in_lds = [&](uint32_t, uint32_t hs, uint32_t k, uint32_t word) {
                return part_s[(k * GP + hs) * PS + word];
            };
            auto slot_of = [&](uint32_t hs, uint32_t k) {
                return p.partials + (((uint64_t)s_ * p.Hq + q_head_of(p, kv_, hs)) * p.max_slots + k) * PS;
            };
            for (uint32_t r0 = 0; r0 < p.G; r0 += RP)
            merge_rows(r0, p.G, kWaves, in_lds, std::false_type{},
                       [&](uint32_t, uint32_t hs, float m, float l, float o) {
                           float *dst = slot_of(hs, my_slot);
                           __hip_atomic_store(dst + 2 + col, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                           if (col == 0) {
                               __hip_atomic_store(dst, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                               __hip_atomic_store(dst + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                           }
                       });
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const uint32_t before = __hip_atomic_fetch_add(p.merge.arrive + region, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                if (before + 1 == p.merge.region_wgs) {
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                }
                *count_s = before;
            }
            __syncthreads();
            if (*count_s + 1 != p.merge.region_wgs) {
                return;
            }
            if (tid == 0) {
                __hip_atomic_store(p.merge.arrive + region, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            finish_regions_from_memory(
                1, [&](uint32_t) { return region; }, [&](uint32_t) { return p.merge.region_wgs; });
        }
        }
    }
}

template <int D, int WK, int WV, int GP, bool LLOYD> int launch_gp(const MfmaParams &p, hipStream_t s)
{
    constexpr uint32_t waves = mfma_decode_waves_per_wg(GP, D, WK, WV);
    constexpr size_t smem = (size_t)table_rows<WK, WV>() * kTableRowBytes;
    constexpr size_t smem_merging =
        smem + (mfma_decode_merges_whole_regions(GP, D, waves) ? mfma_merge_lds_bytes(waves, GP, D) : 0u);
    static_assert(smem_merging <= 160u * 1024u, "tables and merge area exceed a compute unit's LDS");
    // once per instance and process, whichever host thread gets here first (the others wait for it)
    static std::once_flag configured;
    static hipError_t config_status = hipSuccess;
    constexpr bool kMerges = mfma_decode_merges_whole_regions(GP, D, waves);
    constexpr bool kGeneralVariant = mfma_decode_general_variant(GP, D, waves);
    std::call_once(configured, [] {
        config_status = hipFuncSetAttribute((const void *)decode_mfma_kernel<D, WK, WV, GP, LLOYD, 0>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_merging);
        if constexpr (kMerges) {
            if (config_status == hipSuccess) {
                config_status = hipFuncSetAttribute((const void *)decode_mfma_kernel<D, WK, WV, GP, LLOYD, 1>,
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_merging);
            }
        }
        if constexpr (kGeneralVariant) {
            if (config_status == hipSuccess) {
                config_status = hipFuncSetAttribute((const void *)decode_mfma_kernel<D, WK, WV, GP, LLOYD, 2>,
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_merging);
            }
        }
    });
    WEED_HIP_CHECK(config_status);
    if (p.runs.waves != waves) {
        return fail(WEED_HIP_EDEVICE, "decode_mfma: runs were cut for %u wavefronts per workgroup, the kernel has %u",
                    p.runs.waves, waves);
    }
    const uint32_t wg_blocks = waves * p.runs.unit_blocks;
    uint32_t grid = (p.total_blocks + wg_blocks - 1) / wg_blocks;
    if (p.grid_passes > 1) {
        if (p.merge.wg_regions != 0 || p.merge.region_wgs != 0 || p.merge.general || p.query.q) {
            return fail(WEED_HIP_EDEVICE, "decode_mfma: several passes in one launch neither merge nor rotate queries");
        }
        grid = (grid + 7) / 8 * 8 * p.grid_passes;
    }
    if (p.merge.wg_regions != 0 || p.merge.region_wgs != 0) {
        if constexpr (kMerges) {
            decode_mfma_kernel<D, WK, WV, GP, LLOYD, 1><<<grid, 64 * waves, smem_merging, s>>>(p);
        } else {
            return fail(WEED_HIP_EDEVICE, "decode_mfma: this kernel instance cannot merge its partials itself");
        }
    } else {
        // (the area behind the tables is where a workgroup rotates its queries, when it does)
        if constexpr (kGeneralVariant) {
            if (p.query.q || p.merge.general) {
                decode_mfma_kernel<D, WK, WV, GP, LLOYD, 2><<<grid, 64 * waves, smem_merging, s>>>(p);
                WEED_HIP_LAUNCH_CHECK();
                return WEED_HIP_OK;
            }
        }
        decode_mfma_kernel<D, WK, WV, GP, LLOYD, 0>
            <<<grid, 64 * waves, (p.query.q || p.merge.general) ? smem_merging : smem, s>>>(p);
    }
    WEED_HIP_LAUNCH_CHECK();
    return WEED_HIP_OK;
}

template <int D, int WK, int WV, bool LLOYD> int launch_one(const MfmaParams &p, hipStream_t s)
{
    // (all launches of a call use the instance of the call's largest pass, for which the runs were cut)
    const uint32_t rows = p.tile_rows ? p.tile_rows : p.G;
    if (rows <= 4) {
        return launch_gp<D, WK, WV, 4, LLOYD>(p, s);
    }
    if (rows <= 8) {
        return launch_gp<D, WK, WV, 8, LLOYD>(p, s);
    }
    if constexpr (D <= 128) {
        return launch_gp<D, WK, WV, 16, LLOYD>(p, s);
    } else {
        // (64 output registers per lane at head_dim 256 leave no room for the 16-column variant)
        return fail(WEED_HIP_EINVAL, "decode_mfma: groups above 8 are not served at head_dim %d", D);
    }
}

template <int D, bool LLOYD> int launch_d(const MfmaParams &p, hipStream_t s)
{
    const uint32_t wk = p.k.w, wv = p.v.w;
#define WEED_CASE(K, V)                                                                                                \
    if (wk == K && wv == V) {                                                                                          \
        return launch_one<D, K, V, LLOYD>(p, s);                                                                       \
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
    if constexpr (D <= 128) {
    // 5-bit fields: 4-bit codes with the residual sign (or 5-bit uniform codes)
    WEED_CASE(5, 2)
    WEED_CASE(5, 3)
    WEED_CASE(5, 4)
    WEED_CASE(5, 5)
    WEED_CASE(2, 5)
    WEED_CASE(3, 5)
    WEED_CASE(4, 5)
    if constexpr (!LLOYD) {
        // kv_quant_bits = 6, 7, 8 of the reference's uniform coder
        WEED_CASE(6, 6)
        WEED_CASE(7, 7)
        WEED_CASE(8, 8)
    }
    }
    WEED_CASE(1, 1) // one-bit codes (pair tables of four entries)
#undef WEED_CASE
    return fail(WEED_HIP_EINVAL, "decode_mfma: unsupported field widths %u / %u", wk, wv);
}

} // namespace weedhip_mfma
