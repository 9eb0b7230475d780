// Instantiates the blocked-layout conv+LIF kernel for bf16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_bf16(const SpkLaunch& L, int tt) { return launch_conv_spk_tt<bf16_t>(L, tt); }
}  // namespace snnf
