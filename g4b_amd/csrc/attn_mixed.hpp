// One launch for a mixed step: the prefill-phase slots (a chunk of query tokens each) and the decode-phase slots
// (one query token each) of the same batch, over the same caches.
//
// The two halves want different things from the chip.  The chunk is bound by the matrix pipes and scales with the
// number of compute units it gets; the decode stream is bound by HBM and reaches its full rate with a wave on about
// a third of the SIMDs (384 single-wave workers read as fast as 1024).  Launched one after the other, each half
// leaves the other's resource idle.  Here one grid carries both: workgroup ids are dealt so that every XCD gets the
// same mix, the decode workgroups first and `npx` prefill workgroups per XCD after them; a prefill workgroup runs the
// body of the prefill kernel, a decode workgroup is four single-wave workers of the streaming kernel (or one
// (slot, kv head) pair of the short-window variant).  Both kinds occupy a compute unit alone (registers, LDS), so
// the hardware places prefill and decode workgroups side by side on different units and the chunk's matrix work runs
// under the stream's memory time.  A second launch merges the split partials of both halves.
//
// Head dimension 512: the prefill workgroups run the body of the 512 kernel, and a decode workgroup is ONE worker
// whose four waves own 128 columns each (the streaming kernel's column split, which adds the waves' partial dot
// products through LDS once per tile).
#pragma once
#include "attn_decode.hpp"
#include "attn_prefill.hpp"
#include "attn_prefill_wide.hpp"
#include "launch.hpp"

namespace g4b {

// Key tiles that a decode worker of a head-dimension-512 mixed launch keeps in flight: its four waves own 128 columns
// each and so half the bytes per tile of a streaming worker elsewhere (the 35-layer step with 512-wide global layers
// 5.44 -> 5.30 ms; at head dimension 256, where a worker is one wave with a whole tile, two measured the same as one).
constexpr int MIXED_DECODE_PF = 2;

template <int D, int CL, class T, bool QS>
__global__ __launch_bounds__(256) void attn_mixed_kernel(const AttnParams pp, const AttnParams pd, const MixedPlan mp) {
    extern __shared__ __align__(16) char smem[];
    __shared__ int sh_scan[8];
    const int x = blockIdx.x & 7, j = blockIdx.x >> 3;  // workgroups go to the XCDs round-robin by id
    const int ndx = (mp.nd_blocks + 7) >> 3;
    if (j >= ndx) {
        // the prefill grid is sized for every slot being in the prefill phase; the surplus leaves at once
        if constexpr (D == 512) prefill_wide_body<T, QS>(pp, (j - ndx) * 8 + x, smem, sh_scan);
        else prefill_body<D, T, QS>(pp, (j - ndx) * 8 + x, smem, sh_scan);
        return;
    }
    const int d = j * 8 + x;
    if (d >= mp.nd_blocks) return;
    if constexpr (D == 512) {
        decode_worker_body<D, CL, T, 4, QS, MIXED_DECODE_PF>(pd, d, reinterpret_cast<float*>(smem));
    } else {
        if (mp.pair_path) {
            decode_pair_body<D, CL, T, QS>(pd, d, reinterpret_cast<float*>(smem));
        } else {
            decode_worker_body<D, CL, T, 1, QS>(pd, d * 4 + (int)(threadIdx.x >> 6), nullptr);
        }
    }
}

template <int D, class T>
__global__ __launch_bounds__(256) void attn_mixed_combine(const AttnParams pp, const AttnParams pd, const MixedPlan mp) {
    __shared__ int sh_scan[8];
    __shared__ DecodeCombineSmem<D> sm;
    if ((int)blockIdx.x < mp.combine_pf) {
        const int tblocks = (pp.Tq + pfc_rows(D) - 1) / pfc_rows(D);
        prefill_combine_body<D, T>(pp, blockIdx.x % tblocks, (blockIdx.x / tblocks) % pp.H, blockIdx.x / (tblocks * pp.H), sh_scan);
        return;
    }
    const int d = blockIdx.x - mp.combine_pf, rows = pd.R * pd.Tq;
    decode_combine_body<D>(pd, d / rows, d % rows, sm);
}

template <int D, int CL, class T, bool QS>
static hipError_t launch_mixed_t(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream) {
    constexpr int smem_pf = D == 512 ? PW_SMEM : 4 * PfSmem<D>::TILE;
    constexpr int smem_pair = D == 512 ? 2 * 4 * 8 * 64 * (int)sizeof(float) : dec_pair_smem<D>();  // 512: the workers' exchange buffers
    constexpr int smem = smem_pf > smem_pair ? smem_pf : smem_pair;
    static uint64_t attr_done = 0;
    hipError_t e = allow_dynamic_smem(reinterpret_cast<const void*>(&attn_mixed_kernel<D, CL, T, QS>), smem, attr_done);
    if (e != hipSuccess) return e;
    const int grid = 8 * (mp.npx + (mp.nd_blocks + 7) / 8);
    if (pp.kernel_mask & 1) G4B_LAUNCH_DOMINANT((attn_mixed_kernel<D, CL, T, QS>), dim3(grid), dim3(256), smem, stream, pp, pd, mp);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if ((pp.kernel_mask & 2) && mp.combine_pf + mp.combine_dec > 0)
        hipLaunchKernelGGL((attn_mixed_combine<D, T>), dim3(mp.combine_pf + mp.combine_dec), dim3(256), 0, stream, pp, pd, mp);
    return hipGetLastError();
}

template <int D, class T>
static hipError_t launch_mixed_dtype(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream) {
    const int rows = pd.R * pd.Tq;
    if (pp.q_split) {
        if (rows <= 4) return launch_mixed_t<D, 4, T, true>(pp, pd, mp, stream);
        if (rows <= 8) return launch_mixed_t<D, 2, T, true>(pp, pd, mp, stream);
        return launch_mixed_t<D, 1, T, true>(pp, pd, mp, stream);
    }
    if (rows <= 4) return launch_mixed_t<D, 4, T, false>(pp, pd, mp, stream);
    if (rows <= 8) return launch_mixed_t<D, 2, T, false>(pp, pd, mp, stream);
    return launch_mixed_t<D, 1, T, false>(pp, pd, mp, stream);
}

}  // namespace g4b
