// Mixed prefill + decode launch, bf16 caches (attn_mixed.hpp).
#include "attn_mixed.hpp"

namespace g4b {
hipError_t launch_attn_mixed_bf16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, int D, hipStream_t stream) {
    return launch_mixed_dtype<BF16>(pp, pd, mp, D, stream);
}
}  // namespace g4b
