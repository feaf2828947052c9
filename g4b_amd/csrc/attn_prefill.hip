// Launchers of the prefill attention kernel for head dimensions 128 and 256 (attn_prefill.hpp).
#include "attn_prefill.hpp"
#include "launch.hpp"

namespace g4b {

template <int D, class T, bool QS, bool PS>
static hipError_t launch_prefill_ps(const AttnParams& p, hipStream_t stream) {
    const int TOKB = PF_BM / p.R;
    const int slots = p.part_o ? p.split_slots : 1;
    const int blocks = prefill_grid(p);
    dim3 grid(blocks);
    const int smem = 4 * PfSmem<D>::TILE;
    static uint64_t attr_done = 0;
    hipError_t e = allow_dynamic_smem(reinterpret_cast<const void*>(&attn_prefill_kernel<D, T, QS, PS>), smem, attr_done);
    if (e != hipSuccess) return e;
    if (p.kernel_mask & 1) G4B_LAUNCH_DOMINANT((attn_prefill_kernel<D, T, QS, PS>), grid, dim3(256), smem, stream, p);
    if (slots > 1 && (p.kernel_mask & 2))
        launch_prefill_combine<D, T>(p, slots, stream);
    return hipGetLastError();
}

template <int D, class T, bool QS>
static hipError_t launch_prefill_t(const AttnParams& p, hipStream_t stream) {
    return p.pair_split ? launch_prefill_ps<D, T, QS, true>(p, stream) : launch_prefill_ps<D, T, QS, false>(p, stream);
}

hipError_t launch_attn_prefill(const AttnParams& p, int D, int kv_dt, hipStream_t stream) {
    if (p.q_split) {
        if (kv_dt == DT_F16) {
            if (D == 256) return launch_prefill_t<256, F16, true>(p, stream);
            if (D == 128) return launch_prefill_t<128, F16, true>(p, stream);
        } else {
            if (D == 256) return launch_prefill_t<256, BF16, true>(p, stream);
            if (D == 128) return launch_prefill_t<128, BF16, true>(p, stream);
        }
    } else if (kv_dt == DT_F16) {
        if (D == 256) return launch_prefill_t<256, F16, false>(p, stream);
        if (D == 128) return launch_prefill_t<128, F16, false>(p, stream);
    } else {
        if (D == 256) return launch_prefill_t<256, BF16, false>(p, stream);
        if (D == 128) return launch_prefill_t<128, BF16, false>(p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace g4b
