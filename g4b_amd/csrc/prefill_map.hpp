// Work-item bookkeeping shared by the prefill kernels and their launcher.
#pragma once
#include "common.hpp"

namespace g4b {

constexpr int PF_BM = 128;     // query rows per workgroup
constexpr int PF_BN = 64;      // keys per tile of the 128 / 256 kernel
constexpr float PF_TAU = 8.f;  // log2 of the growth of a row maximum that triggers a rescale

// Linear workgroup id -> (head, query tile rank).  "Heads" are (active slot, kv head, key split) triples.  Workgroups
// are handed to the 8 XCDs round-robin by their linear id and every XCD has an L2 of its own, so the ids are mapped
// such that an XCD walks the K/V of as few heads as possible, its workgroups start at the same key and advance
// together (one fetch from memory serves the XCD), the heaviest (latest) query tiles start first, and the XCDs get
// equal shares.
struct PfMap {
    int heads, nq, mode, grid;
};
__host__ __device__ inline PfMap pf_map(int heads, int nq) {
    PfMap m;
    m.heads = heads;
    m.nq = nq;
    if (heads <= 8 && 8 % heads == 0) {
        const int share = 8 / heads;
        m.mode = 1;
        m.grid = 8 * ((nq + share - 1) / share);
    } else {
        m.mode = (heads % 8 == 0) ? 2 : 0;
        m.grid = heads * nq;
    }
    return m;
}
// blocked: a per-query window shorter than the span makes a query tile read only the keys around it, so the XCDs
// that share a head take contiguous runs of its query tiles (each then fetches its own part of K/V) instead of taking
// the tiles in turn (which suits the causal prefix that every tile reads).
__host__ __device__ inline void pf_item(const PfMap& map, int f, int& head, int& rank, bool blocked = false) {
    const int x = f & 7, j = f >> 3;
    if (map.mode == 1) {  // heads divide 8: 8 / heads XCDs share a head
        const int share = 8 / map.heads;
        head = x % map.heads;
        rank = blocked ? (x / map.heads) * (map.grid >> 3) + j : j * share + x / map.heads;
    } else if (map.mode == 2) {  // 8 divides heads: every XCD owns heads / 8 heads
        head = (j % (map.heads / 8)) * 8 + x;
        rank = j / (map.heads / 8);
    } else {
        head = f % map.heads;
        rank = f / map.heads;
    }
}

// Query tiles per workgroup of the 128/256 kernel.  A launch pairs the r-th heaviest query tile of a head with the
// r-th lightest in one workgroup: equal work for every pair under the causal mask, and half as many workgroup starts.
// When the pairs are fewer than the compute units, the key tiles of a pair -- the heavy tile's, then the light
// tile's -- are one list that is cut into nsplit equal spans, one workgroup each (pair_split; without it a launch
// that splits keys gives every workgroup one query tile and a uniform share of its keys, which suits query tiles of
// equal work: a chunk on a long context).
// A launch whose query tiles are no more than the compute units (PF_FILL) stays one tile per workgroup: pairs would
// leave half of the chip idle (eight slots with a 512-token chunk each are 256 tiles).  unsplit_heads = in-phase slots
// x kv heads.
constexpr int PF_FILL = 256;
__host__ __device__ inline int pf_items_per_workgroup(int nsplit, int nq, bool pair_split, int unsplit_heads) {
    if (nq < 2) return 1;
    if (pair_split) return 2;
    return (nsplit == 1 && unsplit_heads * nq > PF_FILL) ? 2 : 1;
}
// Ranks (workgroups) per head: query tiles, or pairs of them.
__host__ __device__ inline int pf_ranks(int nsplit, int nq, bool pair_split, int unsplit_heads) {
    return pf_items_per_workgroup(nsplit, nq, pair_split, unsplit_heads) == 2 ? (nq + 1) / 2 : nq;
}

// The spans of a pair's key-tile list (pair_split): n_first tiles of the first query tile, then n_second of the second,
// cut into nsplit spans; visit(k, begin, end) is called for span k = 0 .. nsplit - 1 in order.  Spans of equal cost,
// not of equal length: a query tile costs a workgroup about four key tiles' time besides its key tiles (staging, Q,
// first scores, epilogue), and the span in which the list passes from the first query tile to the second pays that
// twice.  With equal lengths the workgroups of that span finished 12 % after the others (S = 4096: 101 against 89 us;
// costs of 3, 5, 6 and 8 tiles measured worse).
constexpr int PF_ITEM_COST = 4;
template <class Visit>
__host__ __device__ inline void pf_pair_spans(int n_first, int n_second, int nsplit, Visit&& visit) {
    const int n_all = n_first + n_second;
    const int target = (n_all + PF_ITEM_COST * (nsplit + 1) + nsplit - 1) / nsplit;
    int pos = 0;
    for (int k = 0; k < nsplit; ++k) {
        int end = pos + target - PF_ITEM_COST;
        if (pos < n_first && end > n_first && n_second > 0) end = end - PF_ITEM_COST > n_first ? end - PF_ITEM_COST : n_first;
        end = end > pos ? end : pos;
        end = (k == nsplit - 1 || end > n_all) ? n_all : end;
        visit(k, pos, end);
        pos = end;
    }
}
// Grid for the worst case over the number of slots that turn out to be in phase; the kernels read that number on
// the device and surplus workgroups leave at once.  paired: the kernel gives a workgroup pf_items_per_workgroup tiles.
inline int prefill_grid(const AttnParams& p, int bm = PF_BM, bool paired = true) {
    const int tokb = bm / p.R;
    const int nq = (p.Tq + tokb - 1) / tokb;
    const int slots = p.part_o ? p.split_slots : 1;
    int blocks = 0;
    auto grid_for = [&](int n) {
        const int ns = prefill_splits(slots, n);
        return pf_map(n * p.G * ns, paired ? pf_ranks(ns, nq, p.pair_split != 0, n * p.G) : nq).grid;
    };
    // keys are only split while 2 * n <= slots and the XCD-sharing map (up to 8 heads) rounds its grid up; beyond both
    // the grid grows with n except where the tiles start to be paired (n * G * nq passing PF_FILL), so the candidates
    // are the small n, the last n before the pairing, and n = B
    const int n_small = slots / 2 + 1 > 8 ? slots / 2 + 1 : 8;
    for (int n = 1; n <= n_small && n <= p.B; ++n) blocks = grid_for(n) > blocks ? grid_for(n) : blocks;
    const int n_unpaired = PF_FILL / (p.G * nq);
    if (n_unpaired >= 1) blocks = grid_for(n_unpaired < p.B ? n_unpaired : p.B) > blocks ? grid_for(n_unpaired < p.B ? n_unpaired : p.B) : blocks;
    const int g_all = grid_for(p.B);
    return g_all > blocks ? g_all : blocks;
}

}  // namespace g4b
