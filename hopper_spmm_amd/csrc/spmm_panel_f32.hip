// Instantiations of the LDS-panel kernel: element type f32.
#include <hip/hip_runtime.h>
#include "spmm_panel_kernel.hpp"

namespace hspmm {

template <int G> using PanelTile = Fp32Tile<4, G>;

// G = 0: single windows through the 4x4x1 instruction (the plan's ids are in that tile's format);
// G = 1, 2, 4 with split: the bf16 hi / lo form (the plan's ids and tiles are in that form).
hipError_t launch_panel_f32_tall(int G, bool packed, const PanelArgs &pa, const KernelArgs &ka, hipStream_t s, hipEvent_t mid);

hipError_t launch_panel_f32(int G, bool split, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka, int waves,
                            hipStream_t s, hipEvent_t mid)
{
#ifdef HSPMM_EXPERIMENTAL
    if (tall) return split ? launch_panel_f32_tall(G, packed, pa, ka, s, mid) : hipErrorInvalidValue;
    if (split && G == 4) return launch_panel_nw<Fp32Split<4>>(pa, ka, waves, s, mid);
#else
    if (tall || packed || (split && G == 4)) return hipErrorInvalidValue;
#endif
    if (split)
        return G == 2 ? launch_panel_nw<Fp32Split<2>>(pa, ka, waves, s, mid)
                      : launch_panel_nw<Fp32Split<1>>(pa, ka, waves, s, mid);
    if (G == 0) return launch_panel_nw<Fp32Quad>(pa, ka, waves, s, mid);
#ifdef HSPMM_EXPERIMENTAL
    if (G == 1) return launch_panel_nw<PanelTile<1>>(pa, ka, waves, s, mid);
#endif
    return G == 2 ? launch_panel_nw<PanelTile<2>>(pa, ka, waves, s, mid) : hipErrorInvalidValue;
}

}  // namespace hspmm
