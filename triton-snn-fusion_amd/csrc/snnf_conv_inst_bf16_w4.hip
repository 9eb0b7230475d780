// bf16 activations: the matrix kernel with 4-wave workgroups (two per CU), fast variant, one input frame per tile.
#include "snnf_conv_mm_kernel.h"

namespace snnf {
// Only layers whose T timesteps share one input frame (a single matrix stage, tt == 1) run this way.
int launch_conv_mm_w4_bf16(const ConvLaunch& L, int tt, int load_mode) {
    if (tt != 1) return fail(SNNF_ERR_LAUNCH, "snnf_conv_lif: 4-wave workgroups take one timestep per stage, got %d", tt);
    return launch_conv_mm_tt<bf16_t, 1, 4>(L, load_mode, true);
}
}  // namespace snnf
