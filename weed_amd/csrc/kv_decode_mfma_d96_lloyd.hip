// Instantiates the matrix-core decode kernel for head_dim 96, Lloyd-Max coder.
#include "kv_decode_mfma_kernel.h"

namespace weedhip {
int launch_mfma_decode_d96_lloyd(const MfmaParams &p, hipStream_t s)
{
    return weedhip_mfma::launch_d<96, true>(p, s);
}
} // namespace weedhip
