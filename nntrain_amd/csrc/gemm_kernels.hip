// Prefill mat-mul (bf16 MFMA) - placeholder until the tiled kernel lands.
#include "nnhip_internal.h"

namespace nnhip {

hipError_t launch_matmul_bf16(Lane*, uint32_t, const uint16_t*, const void*, const float*, float*, int, int, int)
{
    return hipErrorNotSupported;
}

}  // namespace nnhip
