// Launchers of the prefill attention kernel for head dimension 512 (attn_prefill_wide.hpp).
#include "attn_prefill_wide.hpp"
#include "launch.hpp"

namespace g4b {

template <class T, bool QS>
static hipError_t launch_prefill_wide_t(const AttnParams& p, hipStream_t stream) {
    const int slots = p.part_o ? p.split_slots : 1;
    const int blocks = prefill_grid(p, QS ? PW_BM / 2 : PW_BM, false);
    static uint64_t attr_done = 0;
    hipError_t e = allow_dynamic_smem(reinterpret_cast<const void*>(&attn_prefill_wide_kernel<T, QS>), PW_SMEM, attr_done);
    if (e != hipSuccess) return e;
    if (p.kernel_mask & 1) G4B_LAUNCH_DOMINANT((attn_prefill_wide_kernel<T, QS>), dim3(blocks), dim3(256), PW_SMEM, stream, p);
    if (slots > 1 && (p.kernel_mask & 2))
        launch_prefill_combine<PW_D, T>(p, slots, stream);
    return hipGetLastError();
}

hipError_t launch_attn_prefill_wide(const AttnParams& p, int kv_dt, hipStream_t stream) {
    if (p.q_split) return kv_dt == DT_F16 ? launch_prefill_wide_t<F16, true>(p, stream) : launch_prefill_wide_t<BF16, true>(p, stream);
    return kv_dt == DT_F16 ? launch_prefill_wide_t<F16, false>(p, stream) : launch_prefill_wide_t<BF16, false>(p, stream);
}

}  // namespace g4b
