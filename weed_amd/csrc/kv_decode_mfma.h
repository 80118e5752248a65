// Interface between the decode-attention entry point and the matrix-core kernel.
#pragma once

#include "kv_cache.h"

namespace weedhip {

struct MfmaParams {
    SideParams k, v;
    const int32_t *lens;
    uint32_t padded;
    uint32_t Hq, Hkv, G;
    int blocked;            // 1: kv = h / G, 0: kv = h % Hkv (Weed)
    const uint16_t *q_hi;   // [n_seq][Hq][d] fp16 bits: high half of the scaled, normalised query
    const uint16_t *q_lo;   // [n_seq][Hq][d] fp16 bits: what the high half misses
    const float *q_scale;   // [n_seq][Hq] power of two the query was divided by
    const float *q_sum;     // [n_seq][Hq] sum of the scaled query (for the uniform coder's offset term)
    float *partials;        // [n_seq][Hq][max_slots][d + 2]: m (log2 units), l, o[d]
    // Work partition: the 64-token blocks of all (sequence, kv head) regions form one list, region after region
    // (sequence-major); wavefront u of the launch takes blocks [u * unit_blocks, (u + 1) * unit_blocks).
    const uint32_t *blk_off; // [n_seq + 1] prefix sums of the sequences' block counts (cached lengths)
    uint32_t n_seq;
    uint32_t total_blocks;   // blk_off[n_seq] * Hkv
    uint32_t unit_blocks;
    uint32_t max_slots;      // partial slots per (sequence, head): most wavefronts that can touch one region
};

bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G);
// Shapes whose 64-token block is large (7 KB or more of packed K + V per wavefront) run with two register buffers
// per wavefront and two wavefronts per SIMD: the deeper prefetch is worth more than the third wavefront there.  Smaller
// blocks run single-buffered with three wavefronts per SIMD.  The 16-column variant (groups above 8) needs too many
// registers for either and runs single-buffered with two.
constexpr bool mfma_decode_double_buffered(uint32_t gp, uint32_t d, uint32_t wk, uint32_t wv)
{
    return gp <= 8 && d * (wk + wv) >= 128u * 7u;
}
// Wavefronts per workgroup; one workgroup fills a compute unit, so one copy of the lookup tables serves it.
constexpr uint32_t mfma_decode_waves_per_wg(uint32_t gp, uint32_t d, uint32_t wk, uint32_t wv)
{
    return (gp > 8 || mfma_decode_double_buffered(gp, d, wk, wv)) ? 8u : 12u;
}
// Wavefronts that fill the device: the launch is cut into that many block runs.
uint32_t mfma_decode_wavefronts(uint32_t G, uint32_t d, uint32_t wk, uint32_t wv);
int launch_mfma_decode(const MfmaParams &p, uint32_t d, hipStream_t s);

} // namespace weedhip
