// Instantiates the matrix-core decode kernel for head_dim 32, uniform coder.
#include "kv_decode_mfma_kernel.h"

namespace weedhip {
int launch_mfma_decode_d32_uniform(const MfmaParams &p, hipStream_t s)
{
    return weedhip_mfma::launch_d<32, false>(p, s);
}
} // namespace weedhip
