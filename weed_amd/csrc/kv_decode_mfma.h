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
    float *partials;        // [n_seq][Hq][n_splits][d + 2]: m (log2 units), l, o[d]
    uint32_t n_splits, blocks_per_split;
};

bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G);
int launch_mfma_decode(const MfmaParams &p, uint32_t d, uint32_t n_seq, hipStream_t s);

} // namespace weedhip
