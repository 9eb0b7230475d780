// Instantiates the blocked-layout conv+LIF kernel for bf16_t activations and inputs in the BITS layout.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_bf16_bits(const SpkLaunch& L, int tt) { return launch_conv_spk_tt<bf16_t, SNNF_LAYOUT_BITS>(L, tt); }
}  // namespace snnf
