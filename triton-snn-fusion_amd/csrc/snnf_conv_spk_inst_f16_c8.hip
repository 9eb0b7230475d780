// Instantiates the blocked-layout conv+LIF kernel for f16_t activations and inputs in the C8 layout.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16_c8(const SpkLaunch& L, int tt) { return launch_conv_spk_tt<f16_t, SNNF_LAYOUT_C8>(L, tt); }
}  // namespace snnf
