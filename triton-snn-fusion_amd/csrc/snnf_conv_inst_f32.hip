// Instantiates the implicit-GEMM conv+LIF kernel for float activations.
#include "snnf_conv_kernel.h"

namespace snnf {
int launch_conv_f32(const ConvLaunch& L, int tt, int load_mode) { return launch_conv_tt<float>(L, tt, load_mode); }
}  // namespace snnf
