// Instantiates the blocked-layout conv+LIF kernel with a projection shortcut in the accumulators, f16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16_shortcut(const SpkLaunch& L) { return launch_conv_spk_shortcut<f16_t>(L); }
}  // namespace snnf
