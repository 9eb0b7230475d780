// Instantiates the blocked-layout conv+LIF kernel for f16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16(const SpkLaunch& L, int tt) { return launch_conv_spk_tt<f16_t>(L, tt); }
}  // namespace snnf
