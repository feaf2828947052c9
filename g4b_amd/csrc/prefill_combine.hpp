// Second kernel of a prefill-shaped launch whose keys were split over several workgroups.
#pragma once
#include "common.hpp"

namespace g4b {

// Merge the key splits of a prefill-shaped launch: a lane per four output columns of a row, PFC_ROWS rows per
// workgroup, every load of a row independent of the others.
constexpr int PFC_ROWS = 8;
// SPANS: the launch cut pairs of query tiles into key spans (AttnParams::pair_split): a split may have no rows for a
// query tile, or have written them straight to o, and says so in its sums.  Otherwise every split has written its
// rows, and their loads are issued with the loads of the sums instead of behind them: one round trip to memory less.
template <int D, int NS, class T, bool SPANS>
G4B_DEV void prefill_combine_rows(const AttnParams& p, int a_idx, int b, int h, int tb, int nsplit) {
    constexpr int LPR = D / 4;      // lanes per row
    constexpr int RPP = 256 / LPR;  // rows per pass
    const int r_in = threadIdx.x / LPR, d0 = (threadIdx.x % LPR) * 4;
#pragma unroll
    for (int pass = 0; pass < PFC_ROWS / RPP; ++pass) {
        const int t = tb * PFC_ROWS + pass * RPP + r_in;
        if (t >= p.Tq) continue;
        float ms[NS], ls[NS];
        f4 ov[NS];
        bool final_row = false;  // a workgroup that held every key tile of the row's query tile has written o itself
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int64_t prow = ((int64_t)(a_idx * nsplit + min(s, nsplit - 1)) * p.H + h) * p.Tq + t;  // clamped, masked below
            ms[s] = p.part_ml[prow * 2];
            ls[s] = (s < nsplit) ? p.part_ml[prow * 2 + 1] : 0.f;
            final_row |= ls[s] < 0.f;
        }
        if constexpr (SPANS)
            if (final_row) continue;
        // spans without key tiles of the row's query tile left (0, 0) and no sums: only what was written is read
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int64_t prow = ((int64_t)(a_idx * nsplit + min(s, nsplit - 1)) * p.H + h) * p.Tq + t;
            const f4 zero = {0.f, 0.f, 0.f, 0.f};
            if (SPANS ? ls[s] > 0.f : s < nsplit) {
                float x[4];
                load_f32<4>(p.part_o, prow * D + d0, T::dt, x);
                ov[s] = f4{x[0], x[1], x[2], x[3]};
            } else {
                ov[s] = zero;
            }
        }
        float mref = -INFINITY;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (ls[s] > 0.f) mref = fmaxf(mref, ms[s]);
        f4 acc = {0.f, 0.f, 0.f, 0.f};
        float l = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (ls[s] > 0.f) {
                const float w = ls[s] * fast_exp2(ms[s] - mref);  // the split's rows were normalised by its sum
                acc += ov[s] * w;
                l += w;
            }
        const float inv = l > 0.f ? 1.f / l : 0.f;
        const int64_t ooff = (int64_t)b * p.o_s[0] + (int64_t)h * p.o_s[1] + (int64_t)t * p.o_s[2] + d0;
        store4(p.o, ooff, p.o_dt, acc * inv);
    }
}

// Workgroups the merge kernel of a split prefill-shaped launch needs (0 = the launch never splits).
inline int prefill_combine_grid_of(const AttnParams& p, int slots) {
    if (slots <= 1) return 0;
    const int items = p.B < slots / 2 ? p.B : slots / 2;  // more active slots than this are never split
    return items * p.H * ((p.Tq + PFC_ROWS - 1) / PFC_ROWS);
}
inline int prefill_combine_grid(const AttnParams& p) { return prefill_combine_grid_of(p, p.part_o ? p.split_slots : 1); }

// NSMAX: the most key splits the launch can have (its split_slots, which the host knows; the split count itself follows
// the number of in-phase slots, which only the device knows).  The wide variants hold up to 16 partial rows per lane
// and set the kernel's register count; a launch that cannot need them takes a kernel without them, twice as many of
// whose workgroups fit a compute unit (the merge of the S = 2048 launch ran its 2048 workgroups in two rounds).
template <int D, class T, int NSMAX = 16>
G4B_DEV void prefill_combine_body(const AttnParams& p, const int bid, int* sh_scan) {
    const int tblocks = (p.Tq + PFC_ROWS - 1) / PFC_ROWS;
    const int a_idx = bid / (p.H * tblocks), h = (bid / tblocks) % p.H, tb = bid % tblocks;
    int n_active;
    const int b = nth_active_slot(p, a_idx, n_active, sh_scan);
    const int nsplit = prefill_splits(p.split_slots, n_active);
    if (b < 0 || nsplit == 1) return;
    if (nsplit <= 2) {
        if (p.pair_split) prefill_combine_rows<D, 2, T, true>(p, a_idx, b, h, tb, nsplit);
        else prefill_combine_rows<D, 2, T, false>(p, a_idx, b, h, tb, nsplit);
    } else if constexpr (NSMAX >= 4) {
        if (nsplit <= 4) {
            if (p.pair_split) prefill_combine_rows<D, 4, T, true>(p, a_idx, b, h, tb, nsplit);
            else prefill_combine_rows<D, 4, T, false>(p, a_idx, b, h, tb, nsplit);
        } else if constexpr (NSMAX >= 8) {
            if (nsplit <= 8) {
                if (p.pair_split) prefill_combine_rows<D, 8, T, true>(p, a_idx, b, h, tb, nsplit);
                else prefill_combine_rows<D, 8, T, false>(p, a_idx, b, h, tb, nsplit);
            }
            else if constexpr (NSMAX >= 16) prefill_combine_rows<D, 16, T, false>(p, a_idx, b, h, tb, nsplit);  // (pairs are cut into five spans at most)
        }
    }
}

template <int D, class T, int NSMAX>
__global__ __launch_bounds__(256) void attn_prefill_combine(const AttnParams p) {
    __shared__ int sh_scan[8];
    prefill_combine_body<D, T, NSMAX>(p, blockIdx.x, sh_scan);
}
// The merge kernel for a launch whose partial buffers hold `slots` (slot, split) pairs.
template <int D, class T>
inline void launch_prefill_combine(const AttnParams& p, int slots, hipStream_t stream) {
    const dim3 grid(prefill_combine_grid_of(p, slots)), block(256);
    if (slots <= 2) hipLaunchKernelGGL((attn_prefill_combine<D, T, 2>), grid, block, 0, stream, p);
    else if (slots <= 4) hipLaunchKernelGGL((attn_prefill_combine<D, T, 4>), grid, block, 0, stream, p);
    else if (slots <= 8) hipLaunchKernelGGL((attn_prefill_combine<D, T, 8>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_prefill_combine<D, T, 16>), grid, block, 0, stream, p);
}


}  // namespace g4b
