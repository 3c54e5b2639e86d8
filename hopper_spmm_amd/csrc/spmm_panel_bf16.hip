// Instantiations of the LDS-panel kernel: element type bf16.
#include <hip/hip_runtime.h>
#include "spmm_panel_kernel.hpp"

namespace hspmm {

template <int G> using PanelTile = Fp16Tr<G, true>;

hipError_t launch_panel_bf16_tall(int G, bool packed, const PanelArgs &pa, const KernelArgs &ka, hipStream_t s, hipEvent_t mid);

hipError_t launch_panel_bf16(int G, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka, int waves, hipStream_t s,
                           hipEvent_t mid)
{
#ifdef HSPMM_EXPERIMENTAL
    if (tall) return launch_panel_bf16_tall(G, packed, pa, ka, s, mid);
#else
    if (tall || packed) return hipErrorInvalidValue;
#endif
    if (G == 4) return launch_panel_nw<PanelTile<4>>(pa, ka, waves, s, mid);
    return G == 2 ? launch_panel_nw<PanelTile<2>>(pa, ka, waves, s, mid)
                  : launch_panel_nw<PanelTile<1>>(pa, ka, waves, s, mid);
}

}  // namespace hspmm
