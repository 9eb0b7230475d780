// Instantiates the blocked-layout conv+LIF kernel for f16_t activations and inputs in the BITS layout.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16_bits(const SpkLaunch& L, int tt) { return launch_conv_spk_tt<f16_t, SNNF_LAYOUT_BITS>(L, tt); }
}  // namespace snnf
