// Instantiates the implicit-GEMM conv+LIF kernels for f16_t activations.
#include "snnf_conv_mm_kernel.h"
#include "snnf_conv_pw_kernel.h"
#include "snnf_conv_tout_kernel.h"

namespace snnf {
// tt < 0 selects the pointwise kernel (-2: its fast variant), tt == 0 the time-outer kernel, tt in {1, 2, 4} the kernel that accumulates tt timesteps side by side.
int launch_conv_f16(const ConvLaunch& L, int tt, int load_mode) {
    if (tt < 0) return launch_conv_pw<f16_t>(L, load_mode, tt == -2);
    if (tt >= 30) return launch_conv_mm_w4_f16(L, tt - 30, load_mode);
    if (tt >= 20) return launch_conv_mm<f16_t>(L, tt - 20, load_mode, true);
    if (tt >= 10) return launch_conv_mm<f16_t>(L, tt - 10, load_mode, false);
    if (tt == 0) return launch_conv_tout<f16_t>(L, load_mode);
    return launch_conv_tt<f16_t>(L, tt, load_mode);
}
}  // namespace snnf
