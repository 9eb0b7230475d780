// Instantiates the blocked-layout conv+LIF kernel whose spikes leave as 2x2 average pools, bf16_t activations.
#include "snnf_conv_spk_kernel.h"

namespace snnf {
int launch_conv_spk_bf16_pooled(const SpkLaunch& L, int tt) {
    return L.g.in_layout == SNNF_LAYOUT_BITS ? launch_conv_spk_pooled<bf16_t, SNNF_LAYOUT_BITS>(L, tt) : launch_conv_spk_pooled<bf16_t, SNNF_LAYOUT_C8>(L, tt);
}
}  // namespace snnf
