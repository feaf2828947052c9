// Launchers of the decode attention kernels (attn_decode.hpp).
#include "attn_decode.hpp"
#include "launch.hpp"

namespace g4b {

template <int D, int CL, class T, bool QS>
static hipError_t launch_decode_t(const AttnParams& p, hipStream_t stream) {
    if constexpr (D <= 256) {
        if (decode_pair_path(p, D)) {
            static uint64_t attr_done = 0;
            hipError_t e = allow_dynamic_smem(reinterpret_cast<const void*>(&attn_decode_pair<D, CL, T, QS>), dec_pair_smem<D>(), attr_done);
            if (e != hipSuccess) return e;
            if (p.kernel_mask & 1)
                G4B_LAUNCH_DOMINANT((attn_decode_pair<D, CL, T, QS>), dim3(p.B * p.G), dim3(64 * DEC_PAIR_WAVES), dec_pair_smem<D>(),
                                    stream, p);
            return hipGetLastError();
        }
    }
    constexpr int DH = D > 256 ? D / 256 : 1;  // waves per worker: each owns at most 256 columns
    if (p.kernel_mask & 1) {
        G4B_LAUNCH_DOMINANT((attn_decode_worker<D, CL, T, DH, QS>), dim3(p.NW > 0 ? p.NW : p.B * p.G), dim3(64 * DH), 0, stream,
                            p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    // without a workspace every pair belongs to one wave, which also writes the zeros of an empty slot: nothing to merge
    if ((p.kernel_mask & 2) && p.NW > 0) hipLaunchKernelGGL((attn_decode_combine<D>), dim3(p.B * p.G, p.R * p.Tq), dim3(256), 0, stream, p);
    return hipGetLastError();
}

template <int D, class T>
static hipError_t launch_decode_cl(const AttnParams& p, hipStream_t stream) {
    const int rows = p.R * p.Tq;
    if (p.q_split) {
        if (rows <= 4) return launch_decode_t<D, 4, T, true>(p, stream);
        if (rows <= 8) return launch_decode_t<D, 2, T, true>(p, stream);
        return launch_decode_t<D, 1, T, true>(p, stream);
    }
    if (rows <= 4) return launch_decode_t<D, 4, T, false>(p, stream);
    if (rows <= 8) return launch_decode_t<D, 2, T, false>(p, stream);
    return launch_decode_t<D, 1, T, false>(p, stream);
}

hipError_t launch_attn_decode(const AttnParams& p, int D, int kv_dt, hipStream_t stream) {
    if (kv_dt == DT_F16) {
        if (D == 512) return launch_decode_cl<512, F16>(p, stream);
        if (D == 256) return launch_decode_cl<256, F16>(p, stream);
        if (D == 128) return launch_decode_cl<128, F16>(p, stream);
    } else {
        if (D == 512) return launch_decode_cl<512, BF16>(p, stream);
        if (D == 256) return launch_decode_cl<256, BF16>(p, stream);
        if (D == 128) return launch_decode_cl<128, BF16>(p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace g4b
