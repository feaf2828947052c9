// Pieces the two prefill kernels (head dimensions 128/256 and 512) share: which item a workgroup works on, where a key
// tile sits in the ring, the mask of an edge tile, the lazy rescaling of the accumulators and the dma chunk issue.
#pragma once
#include "common.hpp"
#include "prefill_map.hpp"

namespace g4b {

// The item(s) of workgroup `bid`: head = (active slot a_idx, kv head g, key split), rank among the head's workgroups.
struct PfWork {
    int nsplit, nq_tiles, rank, split, g, a_idx, b;  // b: slot index
    bool valid;
};
// Every thread of the workgroup calls it (it scans the slots' phases); sh: 8 ints of LDS.  paired: the kernel gives a
// workgroup pf_items_per_workgroup query tiles.
G4B_DEV PfWork pf_select_work(const AttnParams& p, int bid, int rows_per_workgroup, bool paired, int* sh) {
    PfWork w;
    w.valid = false;
    int n_active;
    nth_active_slot(p, -1, n_active, sh);
    if (n_active == 0) return w;
    const int tokb = rows_per_workgroup / p.R;
    w.nsplit = prefill_splits(p.part_o ? p.split_slots : 1, n_active);
    w.nq_tiles = (p.Tq + tokb - 1) / tokb;
    const PfMap map = pf_map(n_active * p.G * w.nsplit, paired ? pf_ranks(w.nsplit, w.nq_tiles, false, n_active * p.G) : w.nq_tiles);
    if (bid >= map.grid) return w;
    int head;
    pf_item(map, bid, head, w.rank, p.qwin > 0);
    if (w.rank >= map.nq) return w;
    w.split = head % w.nsplit;
    w.g = (head / w.nsplit) % p.G;
    w.a_idx = head / (w.nsplit * p.G);
    w.b = nth_active_slot(p, w.a_idx, n_active, sh);  // workgroup-uniform
    w.valid = true;
    return w;
}

// Where the keys of a slot sit: logical key j (clamped to the window) is ring row (ring_start + j) mod KV_CTX.
struct PfRing {
    int window, ring_start, kv_ctx;
    uint32_t row_bytes;
    G4B_DEV uint32_t key_off(int j) const {  // byte offset of logical key j in the (slot, kv head) block of the cache
        j = min(max(j, 0), window - 1);
        int r = ring_start + j;
        r = (r >= kv_ctx) ? r - kv_ctx : r;
        return (uint32_t)r * row_bytes;
    }
    // Ring row of the first key of the tile [jb, jb + bn) when its keys lie inside the window and do not straddle the
    // ring seam (then its rows are consecutive in memory), else -1.
    G4B_DEV int plain_row0(int jb, int bn) const {
        if (jb + bn > window) return -1;
        int r0 = ring_start + jb;
        r0 = (r0 >= kv_ctx) ? r0 - kv_ctx : r0;
        return (r0 + bn <= kv_ctx) ? r0 : -1;
    }
};

// Mask one 32-key block of S^T held as 16 accumulator values per lane: element i of lane half h2 is key
// jb + 8 * (i / 4) + 4 * h2 + i % 4; keys outside [lo_r, hi_r) of the lane's row become -inf.
G4B_DEV void pf_mask_block(f16v& s, int jb, int h2, int lo_r, int hi_r) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int j = jb + 8 * (i >> 2) + 4 * h2 + (i & 3);
        if (j < lo_r || j >= hi_r) s[i] = -INFINITY;
    }
}

// Lazy rescaling of the online softmax: the reference point m_run of a row's exponentials only moves when the row
// maximum mx outgrows it by more than 2^PF_TAU, so P stays below 2^PF_TAU and the accumulators are rarely touched.
// The accumulators (f16v acc[DT]) live in AGPRs; spelling the read-scale-write out keeps the copies inside this rarely
// taken branch instead of on the main path.  A macro, not a function: handed the accumulator array by reference the
// compiler allocates the main loop's registers differently, which cost the 128/256 kernel 4 % when it was measured.
#define G4B_PF_LAZY_RESCALE(acc, DT, m_run, l_run, mx)                                                       \
    do {                                                                                                     \
        const bool grow_ = (mx) > (m_run) + PF_TAU;                                                          \
        if (__any(grow_)) {                                                                                  \
            const float m_new_ = grow_ ? (mx) : (m_run);                                                     \
            const float alpha_ = grow_ ? fast_exp2((m_run) - (mx)) : 1.f; /* 0 on a row's first keys */      \
            const bool touch_ = grow_ && ((m_run) != -INFINITY);                                             \
            (m_run) = m_new_;                                                                                \
            (l_run) *= alpha_;                                                                               \
            if (__any(touch_)) {                                                                             \
                _Pragma("unroll") for (int i_ = 0; i_ < (DT); ++i_)                                          \
                    _Pragma("unroll") for (int j_ = 0; j_ < 16; ++j_) {                                      \
                        float t_, r_;                                                                        \
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t_) : "a"((acc)[i_][j_]));           \
                        t_ *= alpha_;                                                                        \
                        asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(r_) : "v"(t_));                     \
                        (acc)[i_][j_] = r_;                                                                  \
                    }                                                                                        \
            }                                                                                                \
        }                                                                                                    \
    } while (0)

// Chunk i of a tile's direct-to-LDS loads: four chunks share one M0 base, the instruction offset moves source and
// destination alike.
G4B_DEV void pf_dma_chunk(int i, const char* src, uint32_t ofs, uint32_t dst) {
    if ((i & 3) == 0) dma_set_base(dst + i * 1024);
    if ((i & 3) == 0) dma16_to_lds_at<0>(src, ofs);
    if ((i & 3) == 1) dma16_to_lds_at<1024>(src, ofs);
    if ((i & 3) == 2) dma16_to_lds_at<2048>(src, ofs);
    if ((i & 3) == 3) dma16_to_lds_at<3072>(src, ofs);
}

}  // namespace g4b
