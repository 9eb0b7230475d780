// Instantiates the implicit-GEMM conv+LIF kernel for bf16_t activations.
#include "snnf_conv_kernel.h"

namespace snnf {
int launch_conv_bf16(const ConvLaunch& L, int tt, int load_mode) { return launch_conv_tt<bf16_t>(L, tt, load_mode); }
}  // namespace snnf
