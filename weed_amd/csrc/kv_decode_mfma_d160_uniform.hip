// Instantiates the matrix-core decode kernel for head_dim 160, uniform coder (fields of 2..4 bits, groups up to 8).
#include "kv_decode_mfma_kernel.h"

namespace weedhip {
int launch_mfma_decode_d160_uniform(const MfmaParams &p, hipStream_t s)
{
    return weedhip_mfma::launch_d<160, false>(p, s);
}
} // namespace weedhip
