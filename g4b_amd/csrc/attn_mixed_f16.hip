// Mixed prefill + decode launch, fp16 caches (attn_mixed.hpp).
#include "attn_mixed.hpp"

namespace g4b {
hipError_t launch_attn_mixed_f16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, int D, hipStream_t stream) {
    return launch_mixed_dtype<F16>(pp, pd, mp, D, stream);
}
}  // namespace g4b
