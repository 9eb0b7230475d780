// Instantiates the blocked-layout conv+LIF kernel for a dense input frame shared by all timesteps, f16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16_frame(const SpkLaunch& L, bool pooled) { return launch_conv_spk_frame<f16_t>(L, pooled); }
}  // namespace snnf
