// Instantiates the blocked-layout conv+LIF kernel with a projection shortcut in the accumulators, bf16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_bf16_shortcut(const SpkLaunch& L) { return launch_conv_spk_shortcut<bf16_t>(L); }
}  // namespace snnf
