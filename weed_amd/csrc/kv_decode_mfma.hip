// Dispatch of the matrix-core decode kernel (instantiated per head_dim and coder in kv_decode_mfma_d*.hip).
#include "kv_decode_mfma.h"

namespace weedhip {

int launch_mfma_decode_d32_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d32_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d96_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d96_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d64_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d64_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d128_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d128_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d160_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d160_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d192_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d192_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d224_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d224_lloyd(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d256_uniform(const MfmaParams &p, hipStream_t s);
int launch_mfma_decode_d256_lloyd(const MfmaParams &p, hipStream_t s);

uint32_t mfma_decode_tile_rows(uint32_t d) { return d > 128 ? 8u : 16u; }

// `G` heads per KV head in ONE launch; larger groups are split by the caller.
bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G)
{
    if (G < 1 || G > mfma_decode_tile_rows(d)) {
        return false;
    }
    const bool one_bit = wk == 1 && wv == 1;
    if (d == 160 || d == 192 || d == 224 || d == 256) {
        // up to 64 output registers per lane: fields of up to 4 bits only
        return (wk >= 2 && wk <= 4 && wv >= 2 && wv <= 4) || one_bit;
    }
    // fields of 2..5 bits through lookup tables (any pair of widths), or equal widths of 1 or 6..8 bits (the latter
    // exist in the uniform coder only)
    const bool widths = (wk >= 2 && wk <= 5 && wv >= 2 && wv <= 5) || one_bit || (wk == wv && wk >= 6 && wk <= 8);
    return (d == 32 || d == 64 || d == 96 || d == 128) && widths;
}

uint32_t mfma_decode_workgroup_waves(uint32_t G, uint32_t d, uint32_t wk, uint32_t wv)
{
    const uint32_t gp = G <= 4 ? 4u : (G <= 8 ? 8u : 16u);
    return mfma_decode_waves_per_wg(gp, d, wk, wv);
}

int launch_mfma_decode(const MfmaParams &p, uint32_t d, hipStream_t s)
{
    const bool lloyd = p.k.alpha != nullptr;
    if (d == 32) {
        return lloyd ? launch_mfma_decode_d32_lloyd(p, s) : launch_mfma_decode_d32_uniform(p, s);
    }
    if (d == 64) {
        return lloyd ? launch_mfma_decode_d64_lloyd(p, s) : launch_mfma_decode_d64_uniform(p, s);
    }
    if (d == 96) {
        return lloyd ? launch_mfma_decode_d96_lloyd(p, s) : launch_mfma_decode_d96_uniform(p, s);
    }
    if (d == 160) {
        return lloyd ? launch_mfma_decode_d160_lloyd(p, s) : launch_mfma_decode_d160_uniform(p, s);
    }
    if (d == 192) {
        return lloyd ? launch_mfma_decode_d192_lloyd(p, s) : launch_mfma_decode_d192_uniform(p, s);
    }
    if (d == 224) {
        return lloyd ? launch_mfma_decode_d224_lloyd(p, s) : launch_mfma_decode_d224_uniform(p, s);
    }
    if (d == 256) {
        return lloyd ? launch_mfma_decode_d256_lloyd(p, s) : launch_mfma_decode_d256_uniform(p, s);
    }
    return lloyd ? launch_mfma_decode_d128_lloyd(p, s) : launch_mfma_decode_d128_uniform(p, s);
}

} // namespace weedhip
