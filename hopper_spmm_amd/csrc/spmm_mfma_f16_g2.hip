// Instantiations of the MFMA kernel: element type f16, 2 window(s) per unit.
#include <hip/hip_runtime.h>
#include "spmm_mfma_kernel.hpp"

namespace hspmm {

hipError_t launch_mfma_f16_g2(int layout, const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group,
                             hipStream_t s, hipEvent_t mid)
{
    constexpr int G = 2;
    (void)layout;
    return layout == kLayoutDW ? launch_v<Fp16DW, G>(ka, V, prefetch, narrow, waves_per_group, s, mid)
                               : launch_v<Fp16X4, G>(ka, V, prefetch, narrow, waves_per_group, s, mid);
}

}  // namespace hspmm
