// Second kernel of a prefill-shaped launch whose keys were split over several workgroups.
#pragma once
#include "common.hpp"

namespace g4b {

// Merge the key splits of a prefill-shaped launch.  The kernel is bound by the instructions it issues, not by its bytes
// (a thread has a handful of them to merge): a lane takes eight output columns of a row -- one 16-byte load per split --
// a workgroup pfc_rows(D) rows of a head, every load of those rows is in flight before the first is used, and the
// workgroup's place comes from a three-dimensional grid instead of divisions of a linear id.
__host__ __device__ constexpr int pfc_rows(int D) { return D >= 512 ? 8 : 16; }

// SPANS: the launch cut pairs of query tiles into key spans (AttnParams::pair_split): a split may have no rows for a
// query tile, or have written them straight to o, and says so in its sums.  Without SPANS every split has written its
// rows, and they are asked for together with the sums: one round trip to memory less than asking behind the sums.  With
// SPANS the same is done where most splits are expected to hold rows (guess_rows: the later, heavier tile of a causal
// pair, or any tile under a per-query window); what comes back for a split that wrote nothing is whatever the buffer
// held and is cleared before use.  The earlier tile of a causal pair nearly always lies in one span, which wrote it to
// o, so only its sums are read, and rows that turn out to be needed after all are asked for behind them.  The guess
// decides how long the merge takes, never what it computes.
// Addresses are a workgroup-uniform 64-bit base per split plus one 32-bit offset per lane, the same for every split.
template <int D, int NS, class T, bool SPANS>
G4B_DEV void prefill_combine_rows(const AttnParams& p, int a_idx, int b, int h, int tb, int nsplit, bool guess_rows) {
    constexpr int ROWS = pfc_rows(D);
    constexpr int LPR = D / 8;      // lanes per row
    constexpr int RPP = 256 / LPR;  // rows per pass
    constexpr int PASSES = ROWS / RPP;
    static_assert(ROWS % RPP == 0, "whole passes");
    const int r_in = threadIdx.x / LPR, d0 = (threadIdx.x % LPR) * 8;
    const int64_t split_rows = (int64_t)p.H * p.Tq;  // rows of one split
    const int64_t row_base = ((int64_t)a_idx * nsplit * p.H + h) * p.Tq;  // row of token 0, split 0
    const char* const o_base = reinterpret_cast<const char*>(p.part_o) + row_base * (D * 2);
    const char* const ml_base = reinterpret_cast<const char*>(p.part_ml) + row_base * 8;
    int t[PASSES];
    // byte offsets of a lane's row (clamped to the last one: loaded twice, stored once); 32 bits are plenty: only
    // launches whose query tiles do not fill the chip are split (api.hip::prefill_split_slots), a few thousand tokens
    uint32_t o_off[PASSES], ml_off[PASSES];
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        t[pass] = tb * ROWS + pass * RPP + r_in;
        const uint32_t tc = (uint32_t)min(t[pass], p.Tq - 1);
        o_off[pass] = tc * (uint32_t)(D * 2) + (uint32_t)(d0 * 2);
        ml_off[pass] = tc * 8u;
    }
    u2 sums[PASSES][NS];
    u4 rows[PASSES][NS];
    auto load_rows = [&](int pass, int s) {
        rows[pass][s] = ld_vec<false>(reinterpret_cast<const u4*>(o_base + (int64_t)s * split_rows * (D * 2) + o_off[pass]));
    };
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            sums[pass][s] = u2{0u, 0u};
            rows[pass][s] = u4{0u, 0u, 0u, 0u};
        }
        if (s < nsplit) {  // (uniform)
#pragma unroll
            for (int pass = 0; pass < PASSES; ++pass)
                sums[pass][s] = ld_vec<false>(reinterpret_cast<const u2*>(ml_base + (int64_t)s * split_rows * 8 + ml_off[pass]));
            if (!SPANS || guess_rows) {
#pragma unroll
                for (int pass = 0; pass < PASSES; ++pass) load_rows(pass, s);
            }
        }
    }
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        float ms[NS], ls[NS];
        bool final_row = false;  // a workgroup that held every key tile of the row's query tile has written o itself
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const uint32_t m_bits = sums[pass][s][0], l_bits = sums[pass][s][1];
            ms[s] = __builtin_bit_cast(float, m_bits);
            ls[s] = __builtin_bit_cast(float, l_bits);
            final_row |= ls[s] < 0.f;
        }
        if (t[pass] >= p.Tq || (SPANS && final_row)) continue;
        if constexpr (SPANS) {
            // spans without key tiles of the row's query tile left (0, 0) and no rows
            if (guess_rows) {
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int i = 0; i < 4; ++i) rows[pass][s][i] = ls[s] > 0.f ? rows[pass][s][i] : 0u;
            } else {
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    if (ls[s] > 0.f) load_rows(pass, s);
            }
        }
        float mref = -INFINITY;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (ls[s] > 0.f) mref = fmaxf(mref, ms[s]);
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float l = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            // (a split's rows were normalised by its sum; rows of a split without keys are zeros and weigh nothing)
            const float w = ls[s] > 0.f ? ls[s] * fast_exp2(ms[s] - mref) : 0.f;
            l += w;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t two = rows[pass][s][i];
                acc[2 * i] += T::lo(two) * w;
                acc[2 * i + 1] += T::hi(two) * w;
            }
        }
        const float inv = l > 0.f ? __builtin_amdgcn_rcpf(l) : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= inv;
        store_n<8>(p.o, (int64_t)b * p.o_s[0] + (int64_t)h * p.o_s[1] + (int64_t)t[pass] * p.o_s[2] + d0, p.o_dt, acc);
    }
}

// Workgroups of the merge of a split prefill-shaped launch, as (row blocks, heads, slots); x = 0: the launch never splits.
inline dim3 prefill_combine_grid_of(const AttnParams& p, int slots, int D) {
    if (slots <= 1) return dim3(0, 1, 1);
    const int items = p.B < slots / 2 ? p.B : slots / 2;  // more active slots than this are never split
    return dim3((p.Tq + pfc_rows(D) - 1) / pfc_rows(D), p.H, items);
}
inline int prefill_combine_blocks(const AttnParams& p, int D) {
    const dim3 g = prefill_combine_grid_of(p, p.part_o ? p.split_slots : 1, D);
    return (int)(g.x * g.y * g.z);
}

// NSMAX: the most key splits the launch can have (its split_slots, which the host knows; the split count itself follows
// the number of in-phase slots, which only the device knows).  The wide variants hold up to 16 partial rows per lane
// and pass, which sets the kernel's register count; a launch that cannot need them takes a kernel without them, more
// of whose workgroups fit a compute unit.  (tb, h, a_idx) = row block, head, in-phase slot.
template <int D, class T, int NSMAX = 16>
G4B_DEV void prefill_combine_body(const AttnParams& p, int tb, int h, int a_idx, int* sh_scan) {
    int n_active;
    const int b = nth_active_slot(p, a_idx, n_active, sh_scan);
    const int nsplit = n_active == 1 ? min(p.split_slots, 16) : prefill_splits(p.split_slots, n_active);
    if (b < 0 || nsplit <= 1) return;
    bool guess_rows = false;
    if (p.pair_split) {
        // (the kernel that cuts pairs into spans gives a query tile 128 / R tokens, R a power of two)
        const int tok_shift = 8 - __ffs(p.R);
        const int nq = (p.Tq + (1 << tok_shift) - 1) >> tok_shift;
        guess_rows = p.qwin > 0 || ((tb * pfc_rows(D)) >> tok_shift) >= nq / 2;
    }
    if (nsplit <= 2) {
        if (p.pair_split) prefill_combine_rows<D, 2, T, true>(p, a_idx, b, h, tb, nsplit, guess_rows);
        else prefill_combine_rows<D, 2, T, false>(p, a_idx, b, h, tb, nsplit, guess_rows);
    } else if constexpr (NSMAX >= 4) {
        if (nsplit <= 4) {
            if (p.pair_split) prefill_combine_rows<D, 4, T, true>(p, a_idx, b, h, tb, nsplit, guess_rows);
            else prefill_combine_rows<D, 4, T, false>(p, a_idx, b, h, tb, nsplit, guess_rows);
        } else if constexpr (NSMAX >= 8) {
            if (nsplit <= 8) {
                if (p.pair_split) prefill_combine_rows<D, 8, T, true>(p, a_idx, b, h, tb, nsplit, guess_rows);
                else prefill_combine_rows<D, 8, T, false>(p, a_idx, b, h, tb, nsplit, guess_rows);
            } else if constexpr (NSMAX >= 16) {
                prefill_combine_rows<D, 16, T, false>(p, a_idx, b, h, tb, nsplit, guess_rows);  // (pairs are cut into five spans at most)
            }
        }
    }
}

template <int D, class T, int NSMAX>
__global__ __launch_bounds__(256) void attn_prefill_combine(const AttnParams p) {
    __shared__ int sh_scan[8];
    prefill_combine_body<D, T, NSMAX>(p, blockIdx.x, blockIdx.y, blockIdx.z, sh_scan);
}
// The merge kernel for a launch whose partial buffers hold `slots` (slot, split) pairs.
template <int D, class T>
inline void launch_prefill_combine(const AttnParams& p, int slots, hipStream_t stream) {
    const dim3 grid = prefill_combine_grid_of(p, slots, D), block(256);
    if (slots <= 2) hipLaunchKernelGGL((attn_prefill_combine<D, T, 2>), grid, block, 0, stream, p);
    else if (slots <= 4) hipLaunchKernelGGL((attn_prefill_combine<D, T, 4>), grid, block, 0, stream, p);
    else if (slots <= 8) hipLaunchKernelGGL((attn_prefill_combine<D, T, 8>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_prefill_combine<D, T, 16>), grid, block, 0, stream, p);
}


}  // namespace g4b
