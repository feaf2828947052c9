// Prefill (and chunked-prefill) attention for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (slot, kv head) pair: all R = H/G query
// heads of the group for 128/R consecutive tokens, so a staged K/V tile serves the whole GQA
// group.  Each wave owns 32 rows.  The KV loop walks 64-key tiles from the first tile any row
// of the workgroup can see to the causal diagonal; tiles entirely inside every row's range run
// without masks, edge tiles (sliding-window lower edge, causal diagonal, window end) compare
// per element.
//
// Staging.  K and V tiles are double-buffered in LDS and both travel global -> LDS directly
// (global_load_lds_dwordx4: no registers, no LDS stores).  Rows stay row-major and unpadded; the
// 16-byte pieces of a row are XOR-swizzled by choosing which global piece each lane fetches:
// K with (row & 15), read back with ds_read_b128 as the A operand of S^T = K Q^T; V with
// 4 * (row & 7) (whole 64-byte groups move), read back with ds_read_b64_tr_b16, which transposes
// 4 keys x 16 columns inside each 16-lane group and so delivers V^T fragments without a transpose
// pass.  Both read patterns are bank-conflict free.  The direct loads are issued a few at a time
// between MFMA steps so the address unit never queues a burst.
//
// Math per tile and wave: S^T[64 keys x 32 rows] = K Q^T and O^T[D x 32 rows] += V^T P on
// v_mfma_f32_32x32x16 (fp16 or bf16 operands, fp32 accumulate).  Q stays in registers as the B
// operand; P never leaves registers: the accumulator layout of S^T is the B-operand layout of
// the second product once the key order inside each 16-key group of V^T is permuted to match.
// The loop is software pipelined: S(kt+1) is computed while the softmax of S(kt) runs.  LDS
// operand reads are volatile asm issued a fixed number of steps ahead of their MFMA and retired
// with explicit lgkmcnt waits.  Softmax is online in fp32 with exp2 and scale*log2(e) folded into
// one FMA; the row statistics live one row per lane pair (lane, lane^32); accumulators are
// rescaled lazily.
#pragma once
#include "common.hpp"
#include "prefill_combine.hpp"
#include "prefill_map.hpp"

namespace g4b {

constexpr int PF_PD = 6;       // LDS operand fetches in flight (issued and retired in pairs)

template <int D>
struct PfSmem {
    static constexpr int ROW = D * 2;  // bytes per K or V row, in memory and in LDS
    static constexpr int TILE = PF_BN * ROW;
    static constexpr int VSWZ = (D >= 256) ? 7 : 3;  // (V row & VSWZ) selects the 64-byte group swizzle
};

// The small pieces this kernel has in common with the head-dimension-512 kernel (work selection, ring arithmetic, edge
// mask, lazy rescaling, chunk issue; prefill_common.hpp) are spelled out here on purpose: routed through the shared
// helpers the compiler allocates the main loop's registers differently and the S = 8192 launch measured 2 to 4 %
// slower on the same board, helper by helper.
//
// QS: the query is wider than the cache type (fp32 scratchpads over a 16-bit cache) and enters S^T = K Q^T as two
// B operands, the rounded value and its rounding error, against the same K fragments.
// The body of workgroup `bid` of a launch (256 threads).  smem: 4 * PfSmem<D>::TILE bytes of LDS, 16-byte aligned;
// sh_scan: 8 ints of LDS.
// PS: the launch pairs query tiles although it splits keys (AttnParams::pair_split); a variant of its own because the
// few scalars it adds to the set-up of a query tile change the register allocation of the main loop (the unsplit
// S = 8192 launch measured 0.5 % slower with them compiled in).
template <int D, class T, bool QS, bool PS = false>
G4B_DEV void prefill_body(const AttnParams& p, const int bid, char* smem, int* sh_scan) {
    using SM = PfSmem<D>;
    constexpr int KSTEPS = D / 16;               // contraction steps of the first product
    constexpr int DT = D / 32;                   // 32-row tiles of O^T
    constexpr int CHUNKS = SM::TILE / 1024 / 4;  // 1 KiB direct-to-LDS loads per wave and tile (K or V)
    constexpr int ROWS_PER_CHUNK = 1024 / SM::ROW;
    constexpr int PIECES = D / 8;
    constexpr int QK_STEPS = 2 * KSTEPS;  // MFMAs of S^T = K Q^T per tile; step idx -> (c = idx/2, key tile mt = idx%2)
    constexpr int PV_STEPS = 4 * DT;      // MFMAs of O^T += V^T P per tile; step idx -> (key group idx/DT, d tile idx%DT)
    constexpr int N1 = 8;                 // QK steps issued next to the row-max part of the softmax
    static_assert(PF_PD == 6, "the wait ladders are written for three pairs of fetches in flight");

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n32 = lane & 31, h2 = lane >> 5;
    const int R = p.R, Tq = p.Tq, KV_CTX = p.KV_CTX;
    const int TOKB = PF_BM / R;
    // The work list is built from the slots that are in phase, so a launch with few of them (one prefill chunk in a
    // batch of decoding slots) can split every item's keys over several workgroups and still fill the chip.
    // A launch of up to 64 slots reads every slot's data in one round, lane l slot l: the in-phase slots are a ballot
    // away, and the slot this workgroup works on is a lane read instead of a second round of loads behind the first.
    int n_active;
    SlotInfo mine = {};
    unsigned long long in_phase = 0;
    if (p.B <= 64) {
        if (lane < p.B) mine = slot_info(p, lane);
        in_phase = __ballot(mine.active);
        n_active = __popcll(in_phase);
    } else {
        nth_active_slot(p, -1, n_active, sh_scan);
    }
    if (n_active == 0) return;
    const int nsplit = prefill_splits(p.part_o ? p.split_slots : 1, n_active);
    const int nq_tiles = (Tq + TOKB - 1) / TOKB;
    constexpr bool pair_split = PS;
    const PfMap map = pf_map(n_active * p.G * nsplit, pf_ranks(nsplit, nq_tiles, pair_split, n_active * p.G));
    if (bid >= map.grid) return;
    int head, rank;
    pf_item(map, bid, head, rank, p.qwin > 0);
    if (rank >= map.nq) return;
    // Unsplit launches give a workgroup two query tiles of its head, the rank-th from the end and the rank-th from the
    // start: under the causal mask their key ranges add up to the same length for every workgroup, and the second
    // item starts without a new workgroup having to be placed, scan the slots and set its staging up.
    const int ipw = pf_items_per_workgroup(nsplit, nq_tiles, pair_split, n_active * p.G);
    // (with a per-query window every tile has the same work: neighbours are paired instead, whose key ranges overlap)
    const bool near_pair = ipw == 2 && p.qwin > 0;
    const int qtile_first = near_pair ? min(2 * rank + 1, nq_tiles - 1) : nq_tiles - 1 - rank;
    const int qtile_second = near_pair ? 2 * rank : rank;
    const int n_items = (ipw == 2 && qtile_second != qtile_first) ? 2 : 1;
    const int split = head % nsplit, g = (head / nsplit) % p.G, a_idx = head / (nsplit * p.G);
    int b;  // workgroup-uniform
    SlotInfo si;
    if (p.B <= 64) {
        const unsigned long long hit = __ballot(mine.active && __popcll(in_phase & ((1ull << lane) - 1ull)) == a_idx);
        b = __ffsll((long long)hit) - 1;  // a_idx < n_active: the grid map hands out no other
        si = slot_info_of_lane(mine, b);
    } else {
        b = nth_active_slot(p, a_idx, n_active, sh_scan);
        si = slot_info(p, b);
    }

    // Key splits: the key tiles of the workgroup's query tiles -- the first tile's, then the second's -- are one list
    // that is cut into nsplit equal spans; this workgroup owns span `split` (tiles [span0, span1) of the list).
    auto tile_span = [&](int qtile, int& count) {
        const int t0 = qtile * TOKB, t1 = min(t0 + TOKB, Tq) - 1;
        int lo, hi, unused;
        row_range(p, si, t0, lo, unused);
        row_range(p, si, t1, unused, hi);
        count = hi > lo ? (hi - 1) / PF_BN - lo / PF_BN + 1 : 0;
    };
    int n_first = 0, n_second = 0, span0 = 0, span1 = 0;
    if constexpr (PS) {
        if (nsplit > 1) {
            tile_span(qtile_first, n_first);
            if (n_items == 2) tile_span(qtile_second, n_second);
        }
        pf_pair_spans(n_first, n_second, nsplit, [&](int k, int begin, int end) {  // the same walk in every workgroup of the pair
            if (k == split) {
                span0 = begin;
                span1 = end;
            }
        });
    }

    const char* kbase = static_cast<const char*>(p.k) + ((int64_t)b * p.k_sb + (int64_t)g * KV_CTX * D) * 2;
    const char* vbase = static_cast<const char*>(p.v) + ((int64_t)b * p.v_sb + (int64_t)g * KV_CTX * D) * 2;
    auto key_off = [&](int j) -> uint32_t {  // byte offset of logical key j (clamped to the window) in the ring
        j = min(max(j, 0), si.window - 1);
        int r = si.ring_start + j;
        r = (r >= KV_CTX) ? r - KV_CTX : r;
        return (uint32_t)r * (uint32_t)SM::ROW;
    };

    // ---- staging ------------------------------------------------------------------------------------------
    // LDS map: K stages at [0, 2*TILE), V stages at [2*TILE, 4*TILE).  Wave `wave` moves chunks
    // wave*CHUNKS .. +CHUNKS of each tile; chunk c covers bytes [c*1024, +1024) of the tile, lane l its piece l.
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;  // LDS byte address of the dynamic segment
    const int st_row_in_chunk = lane / PIECES;        // 0 .. ROWS_PER_CHUNK-1
    const int st_piece_lds = lane % PIECES;           // 16-byte piece position inside the LDS row
    auto st_row = [&](int i) { return (wave * CHUNKS + i) * ROWS_PER_CHUNK + st_row_in_chunk; };
    auto k_piece = [&](int row) { return st_piece_lds ^ (row & 15); };
    auto v_piece = [&](int row) { return st_piece_lds ^ (4 * (row & SM::VSWZ)); };
    // A tile is "plain" when its 64 keys lie inside the window and do not straddle the ring seam: then its rows
    // are consecutive in memory and every lane's source offset is a loop constant added to one scalar base.
    // Only the first / last tiles of a slot and the one on the seam take the general path with per-row clamping.
    uint32_t k_const[CHUNKS], v_const[CHUNKS];
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
        const int row = st_row(i);
        // chunk i is issued with instruction offset (i % 4) KiB, which moves source and destination alike
        k_const[i] = (uint32_t)row * SM::ROW + (uint32_t)k_piece(row) * 16u - (uint32_t)(i & 3) * 1024u;
        v_const[i] = (uint32_t)row * SM::ROW + (uint32_t)v_piece(row) * 16u - (uint32_t)(i & 3) * 1024u;
    }
    auto plain_row0 = [&](int kt) -> int {  // ring row of the tile's first key, or -1
        const int jb = kt * PF_BN;
        if (jb + PF_BN > si.window) return -1;
        int r0 = si.ring_start + jb;
        r0 = (r0 >= KV_CTX) ? r0 - KV_CTX : r0;
        return (r0 + PF_BN <= KV_CTX) ? r0 : -1;
    };
    // Source of K or V tile kt as scalar base + per-lane byte offsets (the instruction offset of chunk i comes on
    // top: on the general path the base is lowered by 3 KiB so that the lane offsets stay non-negative).
    auto tile_src = [&](int kt, bool is_v, const char*& src, uint32_t(&ofs)[CHUNKS]) {
        const int r0 = plain_row0(kt);
        const char* base = is_v ? vbase : kbase;
        if (r0 >= 0) {
            src = base + (int64_t)r0 * SM::ROW;
#pragma unroll
            for (int i = 0; i < CHUNKS; ++i) ofs[i] = is_v ? v_const[i] : k_const[i];
        } else {
            src = base - 3072;
#pragma unroll
            for (int i = 0; i < CHUNKS; ++i) {
                const int row = st_row(i);
                ofs[i] = key_off(kt * PF_BN + row) + (uint32_t)(is_v ? v_piece(row) : k_piece(row)) * 16u + 3072u -
                         (uint32_t)(i & 3) * 1024u;
            }
        }
    };
    const uint32_t wave_chunk0 = (uint32_t)__builtin_amdgcn_readfirstlane(wave) * (CHUNKS * 1024);
    // chunk i of a tile: four chunks share one M0 base
    auto dma_chunk = [&](int i, const char* src, const uint32_t(&ofs)[CHUNKS], uint32_t dst) {
        if ((i & 3) == 0) dma_set_base(dst + i * 1024);
        if ((i & 3) == 0) dma16_to_lds_at<0>(src, ofs[i]);
        if ((i & 3) == 1) dma16_to_lds_at<1024>(src, ofs[i]);
        if ((i & 3) == 2) dma16_to_lds_at<2048>(src, ofs[i]);
        if ((i & 3) == 3) dma16_to_lds_at<3072>(src, ofs[i]);
    };
    auto stage_whole_tile = [&](int kt, bool is_v, int stage) {  // prologue only: all chunks at once
        const char* src;
        uint32_t ofs[CHUNKS];
        tile_src(kt, is_v, src, ofs);
        const uint32_t dst = lds0 + (is_v ? 2 * SM::TILE : 0) + stage * SM::TILE + wave_chunk0;
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) dma_chunk(i, src, ofs, dst);
    };

    // ---- operand read offsets (bytes from the start of a stage pair) ----------------------------------------
    // K^T step (mt, c): row mt*32 + n32, piece 2c + h2, swizzled with (row & 15) = (n32 & 15)
    uint32_t koff[8];
#pragma unroll
    for (int c8 = 0; c8 < 8; ++c8) koff[c8] = (uint32_t)n32 * SM::ROW + (uint32_t)(((2 * c8 + h2) ^ (n32 & 15)) * 16);
    // V^T fragment of step (cu, dt): d = 32dt + n32, keys {16cu + 4h2 + 0..3, 16cu + 8 + 4h2 + 0..3} (the order in
    // which this lane half holds P), fetched with two transposing reads.  Inside a 16-lane group, lane 4r + q
    // points at columns 4q..4q+3 of key r of the block and receives the group's column (lane % 16) of 4 keys.
    const int tr_r = (lane & 15) >> 2, tr_q = lane & 3, tr_dhalf = (lane >> 4) & 1;
    const int tr_key = 4 * h2 + tr_r;  // key (mod 16) this lane points at
    uint32_t voff[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int piece = dt * 4 + tr_dhalf * 2 + (tr_q >> 1);
        voff[dt] = 2 * SM::TILE + (uint32_t)tr_key * SM::ROW + (uint32_t)((piece ^ (4 * (tr_key & SM::VSWZ))) * 16) +
                   (uint32_t)(tr_q & 1) * 8u;
    }
    // Operand reads are issued as volatile asm, PF_PD steps ahead of the MFMA that consumes them, and
    // retired with explicit lgkmcnt waits: LDS returns data in order, so "at most n outstanding" is exact
    // for the oldest read whatever else the compiler has in flight.
    uint32_t kaddr[8], vaddr[DT];
    auto k_issue = [&](int idx) -> u4 {  // needs kaddr[] of the stage
        const int c = idx >> 1, mt = idx & 1;
        return lds_read16(kaddr[c & 7], mt * 32 * SM::ROW + (c >> 3) * 256);
    };
    struct VFrag {
        u2 lo, hi;
    };
    auto v_issue = [&](int idx) -> VFrag {  // needs vaddr[] of the stage
        const int cu = idx / DT, dt = idx % DT;
        VFrag f;
        f.lo = lds_read8_tr16(vaddr[dt], cu * 16 * SM::ROW);
        f.hi = lds_read8_tr16(vaddr[dt], (cu * 16 + 8) * SM::ROW);
        return f;
    };
    // Reads are retired a pair at a time; `left` = pairs of the same sequence issued after the one being retired
    // (a constant after unrolling).
    auto wait_pair = [&](u4& a0, u4& a1, int left) {
        if (left >= 2) lds_wait_pair<4>(a0, a1);
        else if (left == 1) lds_wait_pair<2>(a0, a1);
        else lds_wait_pair<0>(a0, a1);
    };
    auto wait_pair2 = [&](VFrag& f0, VFrag& f1, int left) {  // every fragment is two reads
        if (left >= 2) lds_wait4<8>(f0.lo, f0.hi, f1.lo, f1.hi);
        else if (left == 1) lds_wait4<4>(f0.lo, f0.hi, f1.lo, f1.hi);
        else lds_wait4<0>(f0.lo, f0.hi, f1.lo, f1.hi);
    };
#pragma unroll
    for (int item = 0; item < 2; ++item) {
    if (item >= n_items) break;
    if (item > 0) __syncthreads();  // every wave has read its rows of the previous item back from LDS
    const int qtile = item == 0 ? qtile_first : qtile_second;
    const int tok0 = qtile * TOKB;
    const int tok_last = min(tok0 + TOKB, Tq) - 1;
    // key range of the workgroup and the range that every row shares
    int lo_wg, hi_wg, lo_max, hi_min;
    row_range(p, si, tok0, lo_wg, hi_min);
    row_range(p, si, tok_last, lo_max, hi_wg);

    // this lane's row
    const int rrow = wave * 32 + n32;
    const int hh = rrow / TOKB;
    const int ti = tok0 + rrow % TOKB;
    const bool row_ok = ti < Tq;
    int lo_r = 0, hi_r = 0;
    if (row_ok) row_range(p, si, ti, lo_r, hi_r);

    const int64_t qoff = (int64_t)b * p.q_s[0] + (int64_t)(g * R + hh) * p.q_s[1] + (int64_t)ti * p.q_s[2];

    f16v acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;  // exponent reference in log2 units (scaled), running sum (this lane's keys)
    bool have_keys = !PS;                  // the span holds tiles of this query tile
    bool whole = false;                    // ... all of them: the rows are final and go straight to o

    if (hi_wg > lo_wg) {
        // this workgroup's share of the item's key tiles
        int kt0 = lo_wg / PF_BN, kt1 = (hi_wg - 1) / PF_BN;
        if (nsplit > 1) {
            if constexpr (PS) {
                const int base = item == 0 ? 0 : n_first, n = item == 0 ? n_first : n_second;
                whole = span0 <= base && span1 - base >= n;  // the span holds every key tile of this query tile
                kt1 = kt0 + min(span1 - base, n) - 1;
                kt0 = kt0 + max(span0 - base, 0);
            } else {
                const int n = kt1 - kt0 + 1;
                kt1 = kt0 + (split + 1) * n / nsplit - 1;
                kt0 = kt0 + split * n / nsplit;
            }
        }
        if (kt1 >= kt0) {
        if constexpr (PS) have_keys = true;

        // ---- prologue: K(kt0), K(kt0+1), V(kt0) staged; S(kt0) computed --------------------------------
        stage_whole_tile(kt0, false, 0);
        stage_whole_tile(kt0 + 1, false, 1);
        stage_whole_tile(kt0, true, 0);
        // Q as B operand: lane (row n32, half h2), step c: d = 16c + 8*h2 .. +8 (loaded behind the staging loads)
        u4 qf[KSTEPS];
        u4 qf_lo[QS ? KSTEPS : 1];
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c) {
            u4 z = {0, 0, 0, 0};
            if constexpr (QS) {
                qf[c] = z;
                qf_lo[c] = z;
                if (row_ok) load8_split<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt, qf[c], qf_lo[c]);
            } else {
                qf[c] = row_ok ? load8_as<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt) : z;
            }
        }
        vm_wait_all();
        __syncthreads();
        f16v s_cur[2];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            s_cur[0][j] = 0.f;
            s_cur[1][j] = 0.f;
        }
        {
#pragma unroll
            for (int c8 = 0; c8 < 8; ++c8) kaddr[c8] = lds0 + koff[c8];
            u4 abuf[PF_PD];
#pragma unroll
            for (int i = 0; i < PF_PD; ++i) abuf[i] = k_issue(i);
#pragma unroll
            for (int idx = 0; idx < QK_STEPS; idx += 2) {
                u4 a0 = abuf[idx % PF_PD], a1 = abuf[(idx + 1) % PF_PD];
                wait_pair(a0, a1, (QK_STEPS - 2 - idx) / 2);
                if (idx + PF_PD < QK_STEPS) {
                    abuf[idx % PF_PD] = k_issue(idx + PF_PD);
                    abuf[(idx + 1) % PF_PD] = k_issue(idx + 1 + PF_PD);
                }
                if constexpr (QS) {
                    s_cur[0] = T::mfma32(a0, qf_lo[idx >> 1], s_cur[0]);
                    s_cur[1] = T::mfma32(a1, qf_lo[idx >> 1], s_cur[1]);
                }
                s_cur[0] = T::mfma32(a0, qf[idx >> 1], s_cur[0]);
                s_cur[1] = T::mfma32(a1, qf[idx >> 1], s_cur[1]);
            }
        }
        __syncthreads();  // every wave is done with K stage 0 before the loop refills it

        // One tile: softmax of S(kt) and O += V(kt) P, overlapped with S(kt+1) = K(kt+1) Q^T.
        // par = (kt - kt0) & 1: V(kt) sits in V stage par, K(kt+1) in K stage par^1; K(kt+2) is fetched into K
        // stage par and V(kt+1) into V stage par^1 while this tile computes.  The tiles after the last one are
        // fetched (addresses are clamped to the window) and multiplied too; nobody reads the results.
        for (int kt = kt0; kt <= kt1; ++kt) {
            const int par = (kt - kt0) & 1;
            // Sources of K(kt+2) and V(kt+1).  The loads themselves are issued a few at a time between the MFMA
            // steps below so that the address unit is never handed more than one instruction per wave at once.
            const char *ksrc, *vsrc;
            uint32_t kofs[CHUNKS], vofs[CHUNKS];
            tile_src(kt + 2, false, ksrc, kofs);
            tile_src(kt + 1, true, vsrc, vofs);
            const uint32_t kdst = lds0 + par * SM::TILE + wave_chunk0;
            const uint32_t vdst = lds0 + 2 * SM::TILE + (par ^ 1) * SM::TILE + wave_chunk0;
            {
                const uint32_t kb = lds0 + (par ^ 1) * SM::TILE, vb = lds0 + par * SM::TILE;
#pragma unroll
                for (int c8 = 0; c8 < 8; ++c8) kaddr[c8] = kb + koff[c8];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) vaddr[dt] = vb + voff[dt];  // voff includes the 2*TILE base
            }

            // ---- edge tiles only: mask S(kt) before anything else so the rest of the tile is one straight block
            const int jb = kt * PF_BN;
            if ((jb < lo_max) || (jb + PF_BN > hi_min)) {
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int j = jb + mt * 32 + 8 * (i >> 2) + 4 * h2 + (i & 3);
                        if (j < lo_r || j >= hi_r) s_cur[mt][i] = -INFINITY;
                    }
            }

            f16v s_nxt[2];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                s_nxt[0][j] = 0.f;
                s_nxt[1][j] = 0.f;
            }
            u4 abuf[PF_PD];
#pragma unroll
            for (int i = 0; i < PF_PD; ++i) abuf[i] = k_issue(i);
            auto qk_pair = [&](int idx) {  // steps idx (key tile 0) and idx + 1 (key tile 1) of contraction step idx / 2
                u4 a0 = abuf[idx % PF_PD], a1 = abuf[(idx + 1) % PF_PD];
                wait_pair(a0, a1, (QK_STEPS - 2 - idx) / 2);
                if (idx + PF_PD < QK_STEPS) {
                    abuf[idx % PF_PD] = k_issue(idx + PF_PD);
                    abuf[(idx + 1) % PF_PD] = k_issue(idx + 1 + PF_PD);
                }
                if constexpr (QS) {
                    s_nxt[0] = T::mfma32(a0, qf_lo[idx >> 1], s_nxt[0]);
                    s_nxt[1] = T::mfma32(a1, qf_lo[idx >> 1], s_nxt[1]);
                }
                s_nxt[0] = T::mfma32(a0, qf[idx >> 1], s_nxt[0]);
                s_nxt[1] = T::mfma32(a1, qf[idx >> 1], s_nxt[1]);
                // One direct load per pair: K(kt+2) first (its stage was released by the barrier that ended the
                // previous tile and it is needed first), then V(kt+1).  Issued this early, the loads have the rest
                // of the tile to land before the closing barrier waits for them.
                if (idx / 2 < CHUNKS) dma_chunk(idx / 2, ksrc, kofs, kdst);
                if (idx / 2 >= CHUNKS && idx / 2 < 2 * CHUNKS)
                    dma_chunk(idx / 2 - CHUNKS, vsrc, vofs, vdst);
            };
#pragma unroll
            for (int idx = 0; idx < N1; idx += 2) qk_pair(idx);

            // ---- softmax, part 1: row maximum --------------------------------------------------------------
            float mx = fmaxf(s_cur[0][0], s_cur[1][0]);
#pragma unroll
            for (int i = 1; i < 16; ++i) mx = fmaxf(mx, fmaxf(s_cur[0][i], s_cur[1][i]));
            mx = half_swap_max(mx) * p.c;  // scale > 0: max commutes with the scaling

            // Lazy rescaling: the reference point m_run of the exponentials only moves when the row maximum
            // outgrows it by more than 2^PF_TAU, so P stays below 2^PF_TAU and the accumulators are rarely touched.
            const bool grow = mx > m_run + PF_TAU;
            if (__any(grow)) {
                const float m_new = grow ? mx : m_run;
                const float alpha = grow ? fast_exp2(m_run - mx) : 1.f;  // 0 on a row's first keys
                const bool touch = grow && (m_run != -INFINITY);
                m_run = m_new;
                l_run *= alpha;
                if (__any(touch)) {
                    // The accumulators live in AGPRs.  Spelling the read-scale-write out keeps the copies inside
                    // this rarely taken branch instead of on the main path.
#pragma unroll
                    for (int i = 0; i < DT; ++i)
#pragma unroll
                        for (int j = 0; j < 16; ++j) {
                            float t, r;
                            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(acc[i][j]));
                            t *= alpha;
                            asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(r) : "v"(t));
                            acc[i][j] = r;
                        }
                }
            }

            // ---- softmax, part 2: exponentials, row sums, P in MFMA operand layout ---------------------------
            const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
            float psum = 0.f;
            u4 pf[2][2];  // [key tile][16-key group] -> 8 keys of this lane half
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    float e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = fast_exp2(__builtin_fmaf(s_cur[mt][8 * u + j], p.c, -m_safe));
                    pf[mt][u] = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
                    // the row sum adds up the rounded values the second product uses
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t w = pf[mt][u][j];
                        psum = T::sum2(w, psum);
                    }
                    // a quarter of the remaining K Q^T steps next to each quarter of the exponentials
#pragma unroll
                    for (int q = 0; q < (QK_STEPS - N1) / 4; q += 2) qk_pair(N1 + (mt * 2 + u) * ((QK_STEPS - N1) / 4) + q);
                }
            l_run += psum;

            // ---- O^T += V^T P : (key group) outer, d tile inner -> consecutive MFMAs are independent ----------
            {
                VFrag vbuf[PF_PD];
#pragma unroll
                for (int i = 0; i < PF_PD; ++i) vbuf[i] = v_issue(i);
#pragma unroll
                for (int idx = 0; idx < PV_STEPS; idx += 2) {
                    VFrag f0 = vbuf[idx % PF_PD], f1 = vbuf[(idx + 1) % PF_PD];
                    wait_pair2(f0, f1, (PV_STEPS - 2 - idx) / 2);
                    if (idx + PF_PD < PV_STEPS) {
                        vbuf[idx % PF_PD] = v_issue(idx + PF_PD);
                        vbuf[(idx + 1) % PF_PD] = v_issue(idx + 1 + PF_PD);
                    }
                    const int cu = idx / DT, dt = idx % DT;  // DT is even: both steps share the key group
                    const u4 a0 = {f0.lo[0], f0.lo[1], f0.hi[0], f0.hi[1]};
                    const u4 a1 = {f1.lo[0], f1.lo[1], f1.hi[0], f1.hi[1]};
                    acc[dt] = T::mfma32(a0, pf[cu >> 1][cu & 1], acc[dt]);
                    acc[dt + 1] = T::mfma32(a1, pf[cu >> 1][cu & 1], acc[dt + 1]);
                }
            }
            vm_wait_all();
            __syncthreads();
            s_cur[0] = s_nxt[0];
            s_cur[1] = s_nxt[1];
        }
        }
    }

    // ---- epilogue ---------------------------------------------------------------------------------------
    // Lane (row n32, half h2) holds columns d = 32*dt + 8*(i/4) + 4*h2 + i%4 of its row.  The wave turns its 32 x D
    // block around in LDS (its own 32 * D * 4 bytes of the staging area, free after the loop's last barrier; 16-byte
    // pieces XOR-swizzled with the row so that neither side conflicts) and stores whole rows: one instruction covers
    // 64 / (D/4) complete rows instead of touching 32 rows at 8 or 16 bytes each.
    const float l_tot = half_swap_sum(l_run);
    const bool partial = nsplit > 1 && !whole;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;  // a key split's rows are normalised too: they are kept in 16 bits
    char* wbase = smem + wave * (32 * D * 4);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            f4 v = {acc[dt][4 * q4] * inv, acc[dt][4 * q4 + 1] * inv, acc[dt][4 * q4 + 2] * inv, acc[dt][4 * q4 + 3] * inv};
            const int pc = 8 * dt + 2 * q4 + h2;
            *reinterpret_cast<f4*>(wbase + n32 * (D * 4) + ((pc ^ (n32 & 15)) * 16)) = v;
        }
    if (nsplit > 1 && h2 == 0 && row_ok) {
        // (reference, sum) of this key split's rows; a negative sum tells the merge kernel that the row is final
        const int64_t prow = ((int64_t)(a_idx * nsplit + split) * p.H + (g * R + hh)) * Tq + ti;
        p.part_ml[prow * 2] = (m_run == -INFINITY) ? 0.f : m_run;
        p.part_ml[prow * 2 + 1] = whole ? -1.f : l_tot;
    }
    constexpr int LPR = D / 4;       // lanes that cover a row, 16 bytes of fp32 each
    constexpr int RPI = 64 / LPR;    // rows per store instruction
    const int tokb_shift = __ffs(TOKB) - 1;  // TOKB = 128 / R is a power of two
    // Both destinations are rows of D elements at (head, token): the split's [pair][H][Tq][D] block in the cache's type,
    // or o with the caller's strides and type.  A wave has its SIMD to itself here, so every instruction of this loop is
    // four cycles of the workgroup's time: rows go eight at a time, their LDS reads first and in one block, the wave
    // index is a scalar (a row's head, token and 64-bit offset are then scalar arithmetic), the type is chosen per
    // batch and the rows of a batch are one offset plus a stride apart.  Row by row -- read, wait, compute the offset,
    // choose the type, convert, store -- the 32 rows of a wave took 3.2 us before the stores themselves.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int sub = lane / LPR, pc = lane % LPR;  // row inside an instruction's RPI rows, 16-byte piece of the row
    void* dst;
    int64_t head_stride, row_stride, base_off;
    if (partial) {
        dst = p.part_o;
        head_stride = (int64_t)Tq * D;
        row_stride = D;
        base_off = ((int64_t)(a_idx * nsplit + split) * p.H + g * R) * head_stride;
    } else {
        dst = p.o;
        head_stride = p.o_s[1];
        row_stride = p.o_s[2];
        base_off = (int64_t)b * p.o_s[0] + (int64_t)(g * R) * p.o_s[1];
    }
    auto store_rows = [&](auto nt, const int dt) {
        constexpr bool NT = decltype(nt)::value;
#pragma unroll 1
        for (int i0 = 0; i0 < 32 / RPI; i0 += 8) {
            f4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int row = (i0 + j) * RPI + sub;
                v[j] = *reinterpret_cast<const f4*>(wbase + row * (D * 4) + ((pc ^ (row & 15)) * 16));
            }
            const int rs = wave_u * 32 + i0 * RPI;  // first row of the batch
            if (TOKB >= 8 * RPI) {
                // the batch lies inside one head: consecutive tokens, one stride apart
                const int hr = rs >> tokb_shift, tr0 = tok0 + (rs & (TOKB - 1));
                const int64_t off0 = base_off + (int64_t)hr * head_stride + (int64_t)tr0 * row_stride;
                const int64_t lane_off = (int64_t)sub * row_stride + pc * 4;
                const int n_ok = Tq - tr0 - sub;  // token tr0 + j * RPI + sub is inside while j * RPI < n_ok
                if (dt == DT_F32) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j * RPI < n_ok) store4<NT>(dst, off0 + (int64_t)(j * RPI) * row_stride + lane_off, DT_F32, v[j]);
                } else if (dt == DT_F16) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j * RPI < n_ok) store4<NT>(dst, off0 + (int64_t)(j * RPI) * row_stride + lane_off, DT_F16, v[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j * RPI < n_ok) store4<NT>(dst, off0 + (int64_t)(j * RPI) * row_stride + lane_off, DT_BF16, v[j]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int rr = rs + j * RPI + sub;
                    const int hr = rr >> tokb_shift, tr = tok0 + (rr & (TOKB - 1));
                    if (tr < Tq) store4<NT>(dst, base_off + (int64_t)hr * head_stride + (int64_t)tr * row_stride + pc * 4, dt, v[j]);
                }
            }
        }
    };
    if (partial) {
        // this key split's result, normalised by its own sum; a span without tiles of this query tile leaves (0, 0) in
        // part_ml only
        if (have_keys) store_rows(std::false_type{}, T::dt);
    } else {
        // written once and not read here again: non-temporal, so that the rows do not displace K/V tiles in L2
        // (S = 8192 0.5 % faster, the 512-key sliding window 3.7 %; the same hint on the Q loads cost 1.3 .. 4 %)
        store_rows(std::true_type{}, p.o_dt);
    }
    }
}

template <int D, class T, bool QS, bool PS = false>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const AttnParams p) {
    extern __shared__ __align__(16) char smem[];
    __shared__ int sh_scan[8];
    prefill_body<D, T, QS, PS>(p, blockIdx.x, smem, sh_scan);
}

}  // namespace g4b
