// Interface between the decode-attention entry point and the matrix-core kernel.
#pragma once

#include "kv_cache.h"

namespace weedhip {

// How the launch's list of 64-token blocks is cut into one run per wavefront.  Workgroup j owns blocks
// [j * waves * unit_blocks, (j + 1) * waves * unit_blocks); inside it the runs follow each other by POSITION
// 0 .. waves-1.  The hardware serves the wavefronts of a SIMD by age (the first four wavefronts of a workgroup are the
// oldest of their SIMDs, the next four the second oldest, ...), so the age classes get runs of different length: the
// oldest `skew` blocks more than the mean, the youngest `skew` fewer, and all classes finish at about the same time.
// Positions cycle through the classes (position p belongs to class p % classes, and is worked on by wavefront
// (p % classes) * 4 + p / classes), so every group of `classes` consecutive runs spans classes * unit_blocks blocks:
// regions whose boundaries fall on multiples of that (equal sequences, the common case) are never straddled by a run.
// `group_cycles` > 0 (1, 2 or 4): the runs of that many consecutive cycles share their blocks in turns instead of
// taking one contiguous piece each: the group's blocks go round the runs one by one (the runs of the oldest class
// first) until the youngest class has its share, then round the remaining classes, and so on.  Each run keeps its
// length, so the partition into regions, slots and workgroups is the same; what changes is that neighbouring
// wavefronts read neighbouring blocks at about the same time.  Only for launches whose workgroups merge and in which
// no group crosses a region boundary (equal sequences whose block count is a multiple of the group's).
struct RunGeom {
    uint32_t unit_blocks;  // mean run length
    uint32_t skew;         // < unit_blocks
    uint32_t waves;        // wavefronts per workgroup: 8 or 12
    uint32_t group_cycles; // 0: every run is one contiguous piece
};
__host__ __device__ inline uint32_t run_classes(const RunGeom &rg) { return rg.waves / 4; } // 2 or 3
__host__ __device__ inline uint32_t run_len(const RunGeom &rg, uint32_t age_class)
{
    const int classes = (int)run_classes(rg);
    return (uint32_t)((int)rg.unit_blocks + (int)rg.skew * (classes - 1 - 2 * (int)age_class) / (classes - 1));
}
// Position in the workgroup of its wavefront w, and back.
__host__ __device__ inline uint32_t run_position_of_wave(const RunGeom &rg, uint32_t w)
{
    return (w & 3) * run_classes(rg) + (w >> 2);
}
// First block of the run at position index P (= workgroup * waves + position in workgroup).
__host__ __device__ inline uint32_t run_begin(const RunGeom &rg, uint32_t P)
{
    const uint32_t classes = run_classes(rg);
    const uint32_t wg = P / rg.waves, pos = P % rg.waves;
    uint32_t b = wg * rg.waves * rg.unit_blocks + (pos / classes) * classes * rg.unit_blocks;
    for (uint32_t t = 0; t < pos % classes; ++t) {
        b += run_len(rg, t);
    }
    return b;
}
// Position index of the run that holds block b (contiguous runs; with runs that take turns: the same for the first
// block of a group).
__host__ __device__ inline uint32_t run_of_block(const RunGeom &rg, uint32_t b)
{
    const uint32_t classes = run_classes(rg);
    const uint32_t wg_blocks = rg.waves * rg.unit_blocks, cycle = classes * rg.unit_blocks;
    const uint32_t wg = b / wg_blocks;
    uint32_t r = b - wg * wg_blocks;
    const uint32_t group = r / cycle;
    r -= group * cycle;
    uint32_t t = 0;
    for (; t + 1 < classes; ++t) {
        const uint32_t len = run_len(rg, t);
        if (r < len) {
            break;
        }
        r -= len;
    }
    return wg * rg.waves + group * classes + t;
}

// What the matrix-core kernel needs of one tensor of the cache (the reconstruction levels travel in the table image).
struct MfmaSide {
    const uint8_t *fields;     // packed items, one region per (sequence, kv head)
    const float *alpha;        // [n_seq][n_kv_heads][padded_tokens] row scales, LLOYDMAX only
    uint64_t region_bytes;
    const uint32_t *alpha_max; // [n_seq][n_kv_heads][kScaleMaxSlots]: the largest of them is the bit pattern of the largest row scale seen, LLOYDMAX only
    float alpha_const;         // UNIFORM: step
    float beta;                // UNIFORM: lo
    uint32_t w;                // field width
};

// Rows of one side's lookup table in LDS (256 bytes each): pair tables (2^(2w) entries) for fields of up to 4 bits;
// a table of the 32 single values for 5-bit fields; none for 6 to 8 bits, which are turned into numbers arithmetically.
constexpr uint32_t mfma_side_rows(uint32_t w) { return w >= 6 ? 0u : (w == 5 ? 32u : 1u << (2 * w)); }
constexpr uint32_t mfma_table_rows(uint32_t wk, uint32_t wv)
{
    return mfma_side_rows(wk) > mfma_side_rows(wv) ? mfma_side_rows(wk) : mfma_side_rows(wv);
}
constexpr uint32_t kMfmaTableRowBytes = 256;
constexpr uint32_t kMfmaTableImageBytes = 256 * kMfmaTableRowBytes; // the largest image (4-bit pair tables)
// Word i of the image a workgroup builds in LDS before its first block (32 equal words in a row, held once in memory): entry e = i / 64 of the V table in the
// first 32 words of row e (one replica per bank), of the K table in the last 32.  `k_levels` / `v_levels`: the fp16 bit
// patterns of the 2^w reconstruction levels of each side.
inline uint32_t mfma_table_word(uint32_t i, uint32_t wk, uint32_t wv, const uint16_t *k_levels, const uint16_t *v_levels)
{
    const uint32_t e = i >> 6, k_half = (i >> 5) & 1;
    const uint32_t w = k_half ? wk : wv;
    const uint16_t *lv = k_half ? k_levels : v_levels;
    if (w >= 6) {
        return 0;
    }
    if (w == 5) {
        // the 32 single values, in both halves of the word
        return e < 32u ? ((uint32_t)lv[e] | ((uint32_t)lv[e] << 16)) : 0u;
    }
    const uint32_t mask = (1u << w) - 1u;
    return e < (1u << (2 * w)) ? ((uint32_t)lv[e & mask] | ((uint32_t)lv[(e >> w) & mask] << 16)) : 0u;
}

// Strides of a (sequence, head, coordinate) tensor.  With `tokens` > 1 the "heads" the kernels see are (query
// position, head) pairs of a multi-token chunk: virtual head hv stands for head hv / tokens at position hv % tokens
// (blocked GQA: the pairs of one KV head stay together) or for head hv % heads at position hv / heads (Weed's
// kv = h % Hkv, which the pairs then follow without change); `ts` is the stride between query positions.
struct Geom3 {
    uint32_t off;
    uint32_t s[3];
    uint32_t tokens, heads, ts;
    int blocked;
};

__device__ __forceinline__ uint64_t head_offset(const Geom3 &g, uint32_t hv)
{
    if (g.tokens <= 1U) {
        return (uint64_t)hv * g.s[1];
    }
    const uint32_t h = g.blocked ? hv / g.tokens : hv % g.heads;
    const uint32_t t = g.blocked ? hv % g.tokens : hv / g.heads;
    return (uint64_t)h * g.s[1] + (uint64_t)t * g.ts;
}

// Merge inside the matrix-core kernel.  When every workgroup's share of the block list is a whole number of regions
// and no run straddles a region boundary (`wg_regions` regions per workgroup, each worked on by
// waves / wg_regions wavefronts), the wavefronts leave their partials in LDS, and the workgroup merges them,
// un-rotates the result and writes the output rows itself: no partials in memory, no second kernel.
// `wg_regions` 0: the kernel writes the partials to memory and a second kernel merges them.
// `region_wgs` >= 2 instead (wg_regions 0): every region is a whole number of workgroups' shares (small batches of long
// sequences).  A workgroup then merges its wavefronts' partials into ONE partial of the region in memory and counts
// itself in `arrive[region]`; the workgroup that completes the count merges the region's partials, un-rotates and
// writes the output rows, and puts the counter back to zero (so the counters are zero between launches; whoever
// allocates them clears them once).
// `general` (wg_regions and region_wgs 0): anything else -- ragged batches (up to 63 sequences: a wavefront then
// keeps the prefix sums of the sequences' block counts in a register), equal sequences that do not line up.  The
// wavefronts store their partials through to device scope as one slot per (run, region); a workgroup that is done
// counts itself in `arrive` of every region it has blocks of, and the workgroup that completes a region's count merges
// that region's slots from memory.
struct MfmaMerge {
    uint32_t wg_regions;
    uint32_t region_wgs;
    uint32_t general;
    uint32_t *arrive;  // [n_seq * Hkv] arrival counters, zero when the launch starts
    uint32_t d_real;   // coordinates the caller's rows have (<= the stored head_dim)
    float *out;        // attention output
    Geom3 og;          // its strides
    const float *rv;   // V rotation, row-major [d][d]: out[t] = sum_j o[j] * rv[t + d * j]
    int unrotate;
};
// Query rotation inside the matrix-core kernel, for launches whose workgroups merge (MfmaMerge): a workgroup rotates,
// scales and splits the queries of its own regions' heads (at most kMfmaQueryRows rows) before its first block arrives,
// so that no kernel runs ahead of this one.  `q` null: the kernel reads q_hi / q_lo / q_scale / q_sum from memory.
struct MfmaQuery {
    const float *q;      // the caller's queries
    Geom3 qg;            // their strides
    const float *rot_t;  // K rotation, transposed: q_rot[j] = sum_i q[i] * rot_t[j + d * i]
    int rotate;          // 0: the queries are rotated already
};
constexpr uint32_t kMfmaQueryRows = 32;
// ... of which head_dims above 128 use 16 (their rows are twice as long, and the area is shared with the partials)
constexpr uint32_t mfma_query_rows(uint32_t d) { return d > 128u ? 16u : kMfmaQueryRows; }
// Query rows that the kernel rotates in one go: a pass's eight, or (head_dims above 128) all sixteen
constexpr uint32_t mfma_rotated_query_rows(uint32_t d) { return d > 128u ? 16u : 8u; }

// Instances that can merge: head_dim 64 or 128.
constexpr bool mfma_decode_merges(uint32_t gp, uint32_t d) { return gp <= 16 && (d == 64u || d == 128u); }
// Instances whose workgroups can merge whole regions, or whole shares of one region, and rotate their queries
// (MfmaMerge::wg_regions and region_wgs; not the general case, which is compiled into the other variant of an
// instance): the above, head_dim 96 where a workgroup has twelve wavefronts, so that its 768 threads are eight
// rows of 96, head_dim 32 (two rows per wavefront), and head_dims 160 to 256 with groups of up to eight (a wavefront
// then takes two of the ten to sixteen 16-column tiles of the small rotations; at 160, 192 and 224 the threads
// behind the last whole row idle where a thread is a column).  (`waves`: mfma_decode_waves_per_wg.)
constexpr bool mfma_decode_merges_whole_regions(uint32_t gp, uint32_t d, uint32_t waves)
{
    return mfma_decode_merges(gp, d) || (gp <= 16 && ((d == 96u && waves == 12u) || d == 32u)) ||
        (gp <= 8 && d > 128u && d <= 256u && waves == 8u);
}
// Head_dims whose instances have a third variant that merges in the general case and rotates its queries (ragged
// batches; see decode_mfma_kernel's MODE): 96 and 32, where the workgroups merge whole regions.  Above 128 the
// instances have no registers for it.
constexpr bool mfma_decode_general_variant(uint32_t gp, uint32_t d, uint32_t waves)
{
    return !mfma_decode_merges(gp, d) && (d == 96u || d == 32u) && mfma_decode_merges_whole_regions(gp, d, waves);
}
// ... so the general case is served by these instances:
constexpr bool mfma_decode_merges_in_general(uint32_t gp, uint32_t d, uint32_t waves)
{
    return mfma_decode_merges(gp, d) || mfma_decode_general_variant(gp, d, waves);
}
// Rows (region, head) that one pass of the merge or of the query rotation takes (the matrix instruction behind both
// has 16 rows, so a pass reads 8 rows beyond its own), and the LDS of both behind the lookup tables, in words.
// Rows are staged for the matrix instruction with a pitch of d + 4 words.
//   Area A: the wavefronts' partials [waves][gp][d + 2] at the end of the kernel; at its start the staged raw queries
//           [kMfmaQueryRows + 8][d + 4] and the rotated rows of a pass [kMfmaMergeRows][d].
//   Area B: at the end the staged merged rows of a pass [kMfmaMergeRows + 8][d + 4], the pass's output row addresses
//           (2 words each) and 64 words of arrival counts; at the start the queries' fp16 halves
//           [kMfmaQueryRows][d] each (d words per row together), a scale and a sum per row.
constexpr uint32_t kMfmaMergeRows = 8;
constexpr uint32_t mfma_merge_partials_words(uint32_t waves, uint32_t gp, uint32_t d)
{
    const uint32_t partials = waves * gp * (d + 2u);
    const uint32_t query = (mfma_query_rows(d) + 8u) * (d + 4u) + mfma_rotated_query_rows(d) * d;
    return partials > query ? partials : query;
}
constexpr uint32_t mfma_merge_rows_words(uint32_t d)
{
    const uint32_t merged = (kMfmaMergeRows + 8u) * (d + 4u) + 2u * kMfmaMergeRows;
    const uint32_t query = mfma_query_rows(d) * d + 2u * mfma_query_rows(d);
    return (merged > query ? merged : query) + 64u;
}
constexpr uint32_t mfma_merge_lds_bytes(uint32_t waves, uint32_t gp, uint32_t d)
{
    return 4u * (mfma_merge_partials_words(waves, gp, d) + mfma_merge_rows_words(d));
}
// Arrival counters that a workspace reserves.
constexpr uint32_t kMfmaMergeCounters = 16384;

// Kernel arguments.  What a wavefront needs before it can request its first block comes first, so that it arrives
// with the first kernel-argument fetches.
struct MfmaParams {
    // Work partition: the 64-token blocks of all (sequence, kv head) regions form one list, region after region
    // (sequence-major), cut into one run per wavefront (`runs`).
    RunGeom runs;
    uint32_t total_blocks;   // blk_off[n_seq] * Hkv
    // Blocks per sequence when every sequence spans the same number (the common batch of equal contexts), else 0:
    // a wavefront then finds its region by division instead of searching blk_off, and requests its first block
    // without waiting for any other load.
    uint32_t uniform_blocks;
    uint32_t Hkv, n_seq;
    uint32_t padded;
    MfmaSide k, v;
    const uint32_t *table_image; // mfma_table_rows(k.w, v.w) * 2 words: word j = word 32 j of the LDS image (mfma_table_word)
    const uint32_t *blk_off; // [n_seq + 1] prefix sums of the sequences' block counts (cached lengths)
    const int32_t *lens;
    const int32_t *cached_lens; // the lengths the block list was made from (lens may be shorter: prefix attention)
    uint32_t Hq, G;
    int blocked;            // 1: kv = h / G, 0: kv = h % Hkv (Weed)
    // multi-token chunks: the G "heads" of a KV head are (position, head) pairs, q_tokens positions x real_group
    // heads; pair hc stands for position hc % q_tokens (blocked) or hc / real_group (Weed mapping), and position t
    // does not see the last q_tokens - 1 - t tokens
    uint32_t q_tokens, real_group;
    // groups larger than a tile has rows go through the cache in several launches: this one serves the heads
    // [head_first, head_first + G) of the group_total that share a KV head; tile_rows (0: G) picks the kernel instance
    uint32_t head_first, group_total, tile_rows;
    // grid_passes > 1 (instances that do not merge): ONE launch holds that many such passes, tile_rows heads each, and
    // a workgroup finds its pass and its place in it from its index: launch index = ((w / 8) * grid_passes + pass) * 8
    // + w % 8, so that the workgroups that read the same blocks for different heads are dispatched next to each other
    // and onto the same XCD (launch index % 8), whose L2 then serves all but the first of them
    uint32_t grid_passes;
    uint32_t max_slots;      // partial slots per (sequence, head): most wavefronts that can touch one region
    const uint16_t *q_hi;   // [n_seq][Hq][d] fp16 bits: high half of the scaled, normalised query
    const uint16_t *q_lo;   // [n_seq][Hq][d] fp16 bits: what the high half misses
    const float *q_scale;   // [n_seq][Hq] power of two the query was divided by
    const float *q_sum;     // [n_seq][Hq] sum of the scaled query (for the uniform coder's offset term)
    float *partials;        // [n_seq][Hq][max_slots][d + 2]: m (log2 units), l, o[d]
    MfmaMerge merge;
    MfmaQuery query;
};

bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G);
// Heads of a group that one launch can take (rows of its tile): 16, or 8 at head_dim 256.
uint32_t mfma_decode_tile_rows(uint32_t d);
// Shapes whose 64-token block is large (7 KB or more of packed K + V per wavefront) run with two register buffers
// per wavefront and two wavefronts per SIMD: the deeper prefetch is worth more than the third wavefront there.  Smaller
// blocks run single-buffered with three wavefronts per SIMD.  The 16-column variant (groups above 8) and head_dim 256
// need too many registers for either and run single-buffered with two.
constexpr bool mfma_decode_double_buffered(uint32_t gp, uint32_t d, uint32_t wk, uint32_t wv)
{
    return gp <= 8 && wk < 6 && d <= 128u && d * (wk + wv) >= 128u * 7u;
}
// Wavefronts per workgroup; one workgroup fills a compute unit, so one copy of the lookup tables serves it.
constexpr uint32_t mfma_decode_waves_per_wg(uint32_t gp, uint32_t d, uint32_t wk, uint32_t wv)
{
    // (6- to 8-bit fields: up to 64 registers of packed data per block and wavefront, so one buffer and two wavefronts
    // per SIMD)
    return (gp > 8 || wk >= 6 || d > 128u || mfma_decode_double_buffered(gp, d, wk, wv)) ? 8u : 12u;
}
// Wavefronts per workgroup of the kernel instance that serves this shape (one workgroup fills a compute unit).
uint32_t mfma_decode_workgroup_waves(uint32_t G, uint32_t d, uint32_t wk, uint32_t wv);
int launch_mfma_decode(const MfmaParams &p, uint32_t d, hipStream_t s);

} // namespace weedhip
