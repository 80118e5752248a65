// Instantiates the matrix-core decode kernel for head_dim 224, Lloyd-Max coder (fields of 2..4 bits, groups up to 8).
#include "kv_decode_mfma_kernel.h"

namespace weedhip {
int launch_mfma_decode_d224_lloyd(const MfmaParams &p, hipStream_t s)
{
    return weedhip_mfma::launch_d<224, true>(p, s);
}
} // namespace weedhip
