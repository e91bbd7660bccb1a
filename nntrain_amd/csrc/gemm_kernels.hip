// Prefill mat-mul (bf16 MFMA) - placeholder until the tiled kernel lands.
#include "nnhip_internal.h"

namespace nnhip {

hipError_t launch_matmul_bf16(Lane*, uint32_t, const uint16_t*, const void*, const float*, float*, int, int, int)
{
    return hipErrorNotSupported;
}

hipError_t launch_matvec_batch(Lane* lane, const nnhip_matvec_desc* descs, int count)
{
    for (int i = 0; i < count; ++i) {
        const nnhip_matvec_desc& d = descs[i];
        hipError_t e = launch_matvec(lane, d.ggml_type, d.x, d.w, d.bias, d.y, d.rows, d.in_w, d.out_w);
        if (e != hipSuccess) return e;
        lane->counters.kernel_launches += 1;
    }
    return hipSuccess;
}

}  // namespace nnhip
