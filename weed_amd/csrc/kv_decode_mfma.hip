// Dispatch of the matrix-core decode kernel (instantiated per head_dim and coder in kv_decode_mfma_d*.hip).
#include "kv_decode_mfma.h"

namespace weedhip {

int launch_mfma_decode_d64_uniform(const MfmaParams &p, dim3 grid, hipStream_t s);
int launch_mfma_decode_d64_lloyd(const MfmaParams &p, dim3 grid, hipStream_t s);
int launch_mfma_decode_d128_uniform(const MfmaParams &p, dim3 grid, hipStream_t s);
int launch_mfma_decode_d128_lloyd(const MfmaParams &p, dim3 grid, hipStream_t s);

bool mfma_decode_supported(uint32_t d, uint32_t wk, uint32_t wv, uint32_t G)
{
    return (d == 64 || d == 128) && wk >= 2 && wk <= 4 && wv >= 2 && wv <= 4 && G >= 1 && G <= 16;
}

int launch_mfma_decode(const MfmaParams &p, uint32_t d, hipStream_t s)
{
    const uint32_t units = (p.total_blocks + p.unit_blocks - 1) / p.unit_blocks;
    const dim3 grid((units + kMfmaDecodeWaves - 1) / kMfmaDecodeWaves);
    const bool lloyd = p.k.alpha != nullptr;
    if (d == 64) {
        return lloyd ? launch_mfma_decode_d64_lloyd(p, grid, s) : launch_mfma_decode_d64_uniform(p, grid, s);
    }
    return lloyd ? launch_mfma_decode_d128_lloyd(p, grid, s) : launch_mfma_decode_d128_uniform(p, grid, s);
}

} // namespace weedhip
