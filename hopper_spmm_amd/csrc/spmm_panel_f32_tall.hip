// Instantiations of the LDS-panel kernel: fp32 storage in bf16 hi / lo parts, two units per consumer wave.
#include <hip/hip_runtime.h>
#include "spmm_panel_kernel.hpp"

namespace hspmm {

hipError_t launch_panel_f32_tall(int G, bool packed, const PanelArgs &pa, const KernelArgs &ka, hipStream_t s, hipEvent_t mid)
{
    if (G != 1 && G != 2) return hipErrorInvalidValue;
    return G == 2 ? launch_panel_tall<Fp32Split<2>>(pa, ka, packed, s, mid)
                  : launch_panel_tall<Fp32Split<1>>(pa, ka, packed, s, mid);
}

}  // namespace hspmm
