// Instantiations of the MFMA kernel: element type f32, 1 window(s) per unit.
#include <hip/hip_runtime.h>
#include "spmm_mfma_kernel.hpp"

namespace hspmm {

hipError_t launch_mfma_f32_g1(int layout, const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group,
                             hipStream_t s, hipEvent_t mid)
{
    constexpr int G = 1;
    (void)layout;
    return launch_v<Fp32Tile, G>(ka, V, prefetch, narrow, waves_per_group, s, mid);
}

}  // namespace hspmm
