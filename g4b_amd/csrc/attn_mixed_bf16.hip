// Mixed prefill + decode launch, bf16 caches, head dimension 256 (attn_mixed.hpp).
#include "attn_mixed.hpp"

namespace g4b {
hipError_t launch_attn_mixed_bf16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream) {
    return launch_mixed_dtype<256, BF16>(pp, pd, mp, stream);
}
}  // namespace g4b
