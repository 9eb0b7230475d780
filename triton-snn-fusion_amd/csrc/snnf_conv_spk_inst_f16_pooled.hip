// Instantiates the blocked-layout conv+LIF kernel whose spikes leave as 2x2 average pools, f16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_f16_pooled(const SpkLaunch& L, int tt) {
    return L.g.in_layout == SNNF_LAYOUT_BITS ? launch_conv_spk_pooled<f16_t, SNNF_LAYOUT_BITS>(L, tt) : launch_conv_spk_pooled<f16_t, SNNF_LAYOUT_C8>(L, tt);
}
}  // namespace snnf
