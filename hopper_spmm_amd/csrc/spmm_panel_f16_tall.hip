// Instantiations of the LDS-panel kernel: element type f16, two units per consumer wave.
#include <hip/hip_runtime.h>
#include "spmm_panel_kernel.hpp"

namespace hspmm {

template <int G> using PanelTile = Fp16Tr<G, false>;

hipError_t launch_panel_f16_tall(int G, bool packed, const PanelArgs &pa, const KernelArgs &ka, hipStream_t s, hipEvent_t mid)
{
    if (G != 1 && G != 2) return hipErrorInvalidValue;
    return G == 2 ? launch_panel_tall<PanelTile<2>>(pa, ka, packed, s, mid)
                  : launch_panel_tall<PanelTile<1>>(pa, ka, packed, s, mid);
}

}  // namespace hspmm
