// Instantiates the implicit-GEMM conv+LIF kernels for bf16_t activations.
#include "snnf_conv_mm_kernel.h"
#include "snnf_conv_pw_kernel.h"
#include "snnf_conv_tout_kernel.h"

namespace snnf {
// tt < 0 selects the pointwise kernel (-2: its fast variant), tt == 0 the time-outer kernel, tt in {1, 2, 4} the kernel that accumulates tt timesteps side by side.
int launch_conv_bf16(const ConvLaunch& L, int tt, int load_mode) {
    if (tt < 0) return launch_conv_pw<bf16_t>(L, load_mode, tt == -2);
    if (tt >= 30) return launch_conv_mm_w4_bf16(L, tt - 30, load_mode);
    if (tt >= 20) return launch_conv_mm<bf16_t>(L, tt - 20, load_mode, true);
    if (tt >= 10) return launch_conv_mm<bf16_t>(L, tt - 10, load_mode, false);
    if (tt == 0) return launch_conv_tout<bf16_t>(L, load_mode);
    return launch_conv_tt<bf16_t>(L, tt, load_mode);
}
}  // namespace snnf
