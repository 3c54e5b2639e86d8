// Instantiations of the MFMA kernel: element type f32, single windows, tiles as bitmap + stored elements.
#include <hip/hip_runtime.h>
#include "spmm_mfma_kernel.hpp"

namespace hspmm {

hipError_t launch_mfma_f32_bm(const KernelArgs &ka, int V, int prefetch, bool narrow, int waves_per_group, hipStream_t s,
                              hipEvent_t mid)
{
    if (V == 4) return launch_tt<Fp32TileB<4>>(ka, prefetch, narrow, waves_per_group, s, mid);
    if (V == 2) return launch_tt<Fp32TileB<2>>(ka, prefetch, narrow, waves_per_group, s, mid);
    return launch_tt<Fp32TileB<1>>(ka, prefetch, narrow, waves_per_group, s, mid);
}

}  // namespace hspmm
