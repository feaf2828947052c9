// Prefill (and chunked-prefill) attention for head dimension 512 on gfx950.
//
// Same decomposition as the 128/256 kernel: one workgroup (4 waves) owns 128 query rows of one (slot, kv head) pair
// and each wave 32 of them, so a staged K/V tile serves the whole GQA group.  A wave's 32 x 512 output block fills
// the accumulator register file (256 registers) and its Q block takes 128 of the 256 vector registers, which leaves
// room for one score tile and a short operand pipeline: tiles are 32 keys (K and V double-buffered in LDS, 128 KiB),
// the first product runs as one chain of 32 MFMAs, and there is no overlap of the next tile's scores with this tile's
// softmax.  Address arithmetic that the other kernel keeps in registers across the loop is recomputed where used.
//
// Staging, operand layouts and masks are those of the 128/256 kernel: direct global -> LDS loads (rows row-major and
// unpadded, 16-byte pieces XOR-swizzled through the choice of the source piece), K read with ds_read_b128 as the A
// operand, V read with ds_read_b64_tr_b16, v_mfma_f32_32x32x16, P kept in registers, exp2 softmax in fp32 with lazy
// rescaling.  The next tile's loads are issued one per two MFMA steps of the first product and waited for at the
// barrier that closes the tile.
//
// QS (a query wider than the cache type, to enter K Q^T unrounded): there is no register left for a second Q block,
// so a wave owns 16 rows and the 32 columns of its B operand hold their rounded values (columns 0..15) and their
// rounding errors (columns 16..31); a workgroup covers 64 rows.  The two halves of S^T are added across the lane pair
// (n, n + 16) right after the first product, each lane of the pair keeping the sums of 16 of the tile's 32 keys: the
// four lanes of a row (n, n + 16, n + 32, n + 48) then hold eight keys each, which is the B operand of
// v_mfma_f32_16x16x32 -- the second product runs on 16-column tiles (32 MFMAs of half the cycles, accumulators in
// 128 registers) instead of computing every row twice on 32-column ones, and the softmax handles every score once.
#pragma once
#include "common.hpp"
#include "prefill_combine.hpp"
#include "prefill_common.hpp"

namespace g4b {

constexpr int PW_D = 512;                // head dimension
constexpr int PW_BN = 32;                // keys per tile
constexpr int PW_BM = PF_BM;             // query rows per workgroup (half of it for a split query)
constexpr int PW_ROW = PW_D * 2;         // bytes per K or V row
constexpr int PW_TILE = PW_BN * PW_ROW;  // bytes per staged tile
constexpr int PW_SMEM = 4 * PW_TILE;
constexpr int PW_PD = 4;                 // LDS operand fetches in flight

// Sum over the lane pair (l, l ^ 16): v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even
// rows of its second, leaving (row 0, row 0, row 2, row 2) and (row 1, row 1, row 3, row 3).
G4B_DEV float row16_pair_sum(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

G4B_DEV float row16_pair_max(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
// a of the even 16-lane rows plus the pair lane's a, b of the odd rows plus the pair lane's b: lane l of an even row
// receives a(l) + a(l + 16), lane l + 16 receives b(l) + b(l + 16).
G4B_DEV float row16_pair_sum_split(float a, float b) {
    const u2 r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b), false, false);
    const uint32_t r0 = r[0], r1 = r[1];  // (a.row0, b.row0, a.row2, b.row2), (a.row1, b.row1, a.row3, b.row3)
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

// The body of workgroup `bid` of a launch (256 threads).  smem: PW_SMEM bytes of LDS, 16-byte aligned; sh_scan: 8 ints.
template <class T, bool QS>
G4B_DEV void prefill_wide_body(const AttnParams& p, const int bid, char* smem, int* sh_scan) {
    constexpr int D = PW_D, ROW = PW_ROW, TILE = PW_TILE;
    constexpr int KSTEPS = D / 16;           // contraction steps of the first product
    constexpr int DT = D / 32;               // 32-row tiles of O^T
    constexpr int CHUNKS = TILE / 1024 / 4;  // 1 KiB direct-to-LDS loads per wave and tile: one K or V row each
    constexpr int PV_STEPS = 2 * DT;         // (16-key group, d tile)
    static_assert(CHUNKS == 8 && KSTEPS == 4 * CHUNKS, "one direct load per four steps of the first product");

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n32 = lane & 31, h2 = lane >> 5;
    const int R = p.R, Tq = p.Tq, KV_CTX = p.KV_CTX;
    constexpr int WROWS = QS ? 16 : 32;  // query rows per wave
    constexpr int BM = 4 * WROWS;
    const int TOKB = BM / R;
    const PfWork work = pf_select_work(p, bid, BM, false, sh_scan);
    if (!work.valid) return;
    const int nsplit = work.nsplit, qtile = work.nq_tiles - 1 - work.rank;  // heaviest (latest) query tiles first
    const int split = work.split, g = work.g, a_idx = work.a_idx, b = work.b;

    const SlotInfo si = slot_info(p, b);
    const PfRing ring{si.window, si.ring_start, KV_CTX, (uint32_t)ROW};
    const int tok0 = qtile * TOKB;
    const int tok_last = min(tok0 + TOKB, Tq) - 1;
    int lo_wg, hi_wg, lo_max, hi_min;
    row_range(p, si, tok0, lo_wg, hi_min);
    row_range(p, si, tok_last, lo_max, hi_wg);

    // this lane's row
    const int rrow = wave * WROWS + (QS ? (n32 & 15) : n32);
    const int hh = rrow / TOKB;
    const int ti = tok0 + rrow % TOKB;
    const bool row_ok = ti < Tq;
    int lo_r = 0, hi_r = 0;
    if (row_ok) row_range(p, si, ti, lo_r, hi_r);
    const int64_t qoff = (int64_t)b * p.q_s[0] + (int64_t)(g * R + hh) * p.q_s[1] + (int64_t)ti * p.q_s[2];

    f16v acc[QS ? 1 : DT];  // 256 accumulator registers: the whole AGPR file
#pragma unroll
    for (int i = 0; i < (QS ? 1 : DT); ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    // split query: O^T as 32 tiles of 16 d x 16 rows; lane (row n16, group kg = lane / 16) holds d = 16 blk + 4 kg + 0..3
    constexpr int NB16 = D / 16;
    f4 acc16[QS ? NB16 : 1];
#pragma unroll
    for (int i = 0; i < (QS ? NB16 : 1); ++i) acc16[i] = f4{0.f, 0.f, 0.f, 0.f};
    const int n16 = lane & 15, u16 = (lane >> 4) & 1, kg = lane >> 4;
    float m_run = -INFINITY, l_run = 0.f;

    if (hi_wg > lo_wg) {
        const char* kbase = static_cast<const char*>(p.k) + ((int64_t)b * p.k_sb + (int64_t)g * KV_CTX * D) * 2;
        const char* vbase = static_cast<const char*>(p.v) + ((int64_t)b * p.v_sb + (int64_t)g * KV_CTX * D) * 2;

        // ---- staging: K stages at [0, 2*TILE), V stages at [2*TILE, 4*TILE); wave w moves rows 8w .. 8w+7 of a tile,
        // lane l the 16-byte piece that lands at position l of the LDS row.  Source offsets are recomputed where they
        // are used (two or three integer operations) instead of living in registers across the loop.
        const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
        const int wrow0 = wave * CHUNKS;
        auto src_piece = [&](int row, bool is_v) { return is_v ? (lane ^ (4 * (row & 7))) : (lane ^ (row & 15)); };
        struct TileSrc {
            const char* src;  // scalar base
            int kt, plain;
        };
        auto tile_src = [&](int kt, bool is_v) -> TileSrc {
            const int r0 = ring.plain_row0(kt * PW_BN, PW_BN);
            const char* base = is_v ? vbase : kbase;
            TileSrc t;
            t.kt = kt;
            t.plain = r0 >= 0;
            // general path: the base is lowered by 3 KiB so that the lane offsets stay non-negative under the
            // instruction offsets
            t.src = (r0 >= 0) ? base + (int64_t)r0 * ROW : base - 3072;
            return t;
        };
        auto chunk_ofs = [&](const TileSrc& t, int i, bool is_v) -> uint32_t {
            const int row = wrow0 + i;
            const uint32_t pc = (uint32_t)src_piece(row, is_v) * 16u;
            if (t.plain) return (uint32_t)row * ROW + pc - (uint32_t)(i & 3) * 1024u;
            return ring.key_off(t.kt * PW_BN + row) + pc + 3072u - (uint32_t)(i & 3) * 1024u;
        };
        const uint32_t wave_chunk0 = (uint32_t)__builtin_amdgcn_readfirstlane(wave) * (CHUNKS * 1024);
        auto dma_chunk = [&](int i, const TileSrc& t, bool is_v, uint32_t dst) {
            pf_dma_chunk(i, t.src, chunk_ofs(t, i, is_v), dst);
        };

        // ---- operand read offsets --------------------------------------------------------------------------
        // K^T step c: key row n32, piece 2c + h2 swizzled with (row & 15); c / 8 becomes an instruction offset
        uint32_t koff[8];
#pragma unroll
        for (int c8 = 0; c8 < 8; ++c8) koff[c8] = (uint32_t)n32 * ROW + (uint32_t)(((2 * c8 + h2) ^ (n32 & 15)) * 16);
        // V^T fragment of step (cu, dt): d = 32*dt + n32, keys {16cu + 4h2 + 0..3, 16cu + 8 + 4h2 + 0..3}.  The swizzle
        // only touches the low three bits of dt; dt / 8 becomes an instruction offset.
        const int tr_r = (lane & 15) >> 2, tr_q = lane & 3, tr_dhalf = (lane >> 4) & 1;
        const int tr_key = 4 * h2 + tr_r;
        uint32_t voff[8];
#pragma unroll
        for (int d8 = 0; d8 < 8; ++d8) {
            const int piece = d8 * 4 + tr_dhalf * 2 + (tr_q >> 1);
            voff[d8] = 2 * TILE + (uint32_t)tr_key * ROW + (uint32_t)((piece ^ (4 * (tr_key & 7))) * 16) + (uint32_t)(tr_q & 1) * 8u;
        }
        // split query: V^T fragment of d tile blk for lane group kg: d = 16 blk + n16, keys {16 u16 + 4 h2 + 0..3, the same
        // + 8}; the swizzle touches bits 1..3 of blk, blk / 16 becomes an instruction offset
        uint32_t voff16[QS ? 16 : 1];
        if constexpr (QS) {
            const int key = 16 * u16 + tr_key;
#pragma unroll
            for (int bl = 0; bl < 16; ++bl) {
                const int piece = 2 * bl + (tr_q >> 1);
                voff16[bl] = 2 * TILE + (uint32_t)key * ROW + (uint32_t)((piece ^ (4 * (key & 7))) * 16) + (uint32_t)(tr_q & 1) * 8u;
            }
        }
        uint32_t stage_base = lds0;
        auto k_issue = [&](int c) -> u4 { return lds_read16(stage_base + koff[c & 7], (c >> 3) * 256); };
        struct VFrag {
            u2 lo, hi;
        };
        auto v_issue = [&](int idx) -> VFrag {
            const int cu = idx / DT, dt = idx % DT;
            VFrag f;
            f.lo = lds_read8_tr16(stage_base + voff[dt & 7], cu * 16 * ROW + (dt >> 3) * 512);
            f.hi = lds_read8_tr16(stage_base + voff[dt & 7], (cu * 16 + 8) * ROW + (dt >> 3) * 512);
            return f;
        };
        auto v_issue16 = [&](int blk) -> VFrag {
            VFrag f;
            f.lo = lds_read8_tr16(stage_base + voff16[blk & 15], (blk >> 4) * 512);
            f.hi = lds_read8_tr16(stage_base + voff16[blk & 15], 8 * ROW + (blk >> 4) * 512);
            return f;
        };
        auto wait_pair = [&](u4& a0, u4& a1, int left) {
            if (left >= 1) lds_wait_pair<2>(a0, a1);
            else lds_wait_pair<0>(a0, a1);
        };
        auto wait_pair2 = [&](VFrag& f0, VFrag& f1, int left) {
            if (left >= 1) lds_wait4<4>(f0.lo, f0.hi, f1.lo, f1.hi);
            else lds_wait4<0>(f0.lo, f0.hi, f1.lo, f1.hi);
        };

        int kt0 = lo_wg / PW_BN, kt1 = (hi_wg - 1) / PW_BN;
        if (nsplit > 1) {
            const int n = kt1 - kt0 + 1;
            kt1 = kt0 + (split + 1) * n / nsplit - 1;
            kt0 = kt0 + split * n / nsplit;
        }
        if (kt1 >= kt0) {
            // ---- prologue: K(kt0) and V(kt0) staged, Q in registers
            {
                const TileSrc tk = tile_src(kt0, false), tv = tile_src(kt0, true);
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) dma_chunk(i, tk, false, lds0 + wave_chunk0);
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) dma_chunk(i, tv, true, lds0 + 2 * TILE + wave_chunk0);
            }
            u4 qf[KSTEPS];  // B operand: lane (row n32, half h2), step c: d = 16c + 8*h2 .. +8
#pragma unroll
            for (int c = 0; c < KSTEPS; ++c) {
                u4 z = {0, 0, 0, 0};
                if constexpr (QS) {
                    u4 qh = z, ql = z;
                    if (row_ok) load8_split<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt, qh, ql);
                    qf[c] = (n32 < 16) ? qh : ql;
                } else {
                    qf[c] = row_ok ? load8_as<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt) : z;
                }
            }
            vm_wait_all();
            __syncthreads();

            for (int kt = kt0; kt <= kt1; ++kt) {
                const int par = (kt - kt0) & 1;
                // K(kt+1) and V(kt+1) go into the other stage pair, which every wave left at the last barrier.  Tiles
                // past the last one are fetched as well (addresses are clamped to the window); nobody reads them.
                const TileSrc tk = tile_src(kt + 1, false), tv = tile_src(kt + 1, true);
                const uint32_t kdst = lds0 + (par ^ 1) * TILE + wave_chunk0;
                const uint32_t vdst = lds0 + 2 * TILE + (par ^ 1) * TILE + wave_chunk0;
                stage_base = lds0 + par * TILE;

                // ---- S^T = K Q^T
                f16v s;
#pragma unroll
                for (int j = 0; j < 16; ++j) s[j] = 0.f;
                {
                    u4 abuf[PW_PD];
#pragma unroll
                    for (int i = 0; i < PW_PD; ++i) abuf[i] = k_issue(i);
#pragma unroll
                    for (int idx = 0; idx < KSTEPS; idx += 2) {
                        u4 a0 = abuf[idx % PW_PD], a1 = abuf[(idx + 1) % PW_PD];
                        wait_pair(a0, a1, (KSTEPS - 2 - idx) / 2);
                        if (idx + PW_PD < KSTEPS) {
                            abuf[idx % PW_PD] = k_issue(idx + PW_PD);
                            abuf[(idx + 1) % PW_PD] = k_issue(idx + 1 + PW_PD);
                        }
                        s = T::mfma32(a0, qf[idx], s);
                        s = T::mfma32(a1, qf[idx + 1], s);
                        // one direct load per pair of steps: the 8 K rows first, then the 8 V rows
                        if (idx / 2 < CHUNKS) dma_chunk(idx / 2, tk, false, kdst);
                        else dma_chunk(idx / 2 - CHUNKS, tv, true, vdst);
                    }
                }

                const int jb = kt * PW_BN;
                if constexpr (QS) {
                    // K q_hi + K q_lo: lane (n16, u16, h2) keeps score j of key jb + 16 u16 + 8 (j / 4) + 4 h2 + j % 4
                    float t[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float a = s[j], b8 = s[j + 8];
                        t[j] = row16_pair_sum_split(a, b8);
                    }
                    if ((jb < lo_max) || (jb + PW_BN > hi_min)) {  // edge tiles: mask
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const int key = jb + 16 * u16 + 8 * (j >> 2) + 4 * h2 + (j & 3);
                            if (key < lo_r || key >= hi_r) t[j] = -INFINITY;
                        }
                    }
                    float mx = t[0];
#pragma unroll
                    for (int j = 1; j < 8; ++j) mx = fmaxf(mx, t[j]);
                    mx = half_swap_max(row16_pair_max(mx)) * p.c;  // over the four lanes of the row
                    {   // lazy rescaling (G4B_PF_LAZY_RESCALE for the 16-column accumulators)
                        const bool grow = mx > m_run + PF_TAU;
                        if (__any(grow)) {
                            const float alpha = grow ? fast_exp2(m_run - mx) : 1.f;  // 0 on a row's first keys
                            const bool touch = grow && (m_run != -INFINITY);
                            m_run = grow ? mx : m_run;
                            l_run *= alpha;
                            if (__any(touch)) {
#pragma unroll
                                for (int i = 0; i < NB16; ++i) acc16[i] = acc16[i] * alpha;
                            }
                        }
                    }
                    const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
                    float e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = fast_exp2(__builtin_fmaf(t[j], p.c, -m_safe));
                    const u4 pf = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
                    float psum = 0.f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t w = pf[j];
                        psum = T::sum2(w, psum);  // the row sum adds up the rounded values the second product uses
                    }
                    l_run += psum;

                    // ---- O^T += V^T P on 16 x 16 tiles: lane group kg contracts its eight keys
                    VFrag vbuf[PW_PD];
#pragma unroll
                    for (int i = 0; i < PW_PD; ++i) vbuf[i] = v_issue16(i);
#pragma unroll
                    for (int idx = 0; idx < NB16; idx += 2) {
                        VFrag f0 = vbuf[idx % PW_PD], f1 = vbuf[(idx + 1) % PW_PD];
                        wait_pair2(f0, f1, (NB16 - 2 - idx) / 2);
                        if (idx + PW_PD < NB16) {
                            vbuf[idx % PW_PD] = v_issue16(idx + PW_PD);
                            vbuf[(idx + 1) % PW_PD] = v_issue16(idx + 1 + PW_PD);
                        }
                        const u4 a0 = {f0.lo[0], f0.lo[1], f0.hi[0], f0.hi[1]};
                        const u4 a1 = {f1.lo[0], f1.lo[1], f1.hi[0], f1.hi[1]};
                        acc16[idx] = T::mfma16(a0, pf, acc16[idx]);
                        acc16[idx + 1] = T::mfma16(a1, pf, acc16[idx + 1]);
                    }
                } else {
                    // ---- edge tiles: mask
                    if ((jb < lo_max) || (jb + PW_BN > hi_min)) {
                        pf_mask_block(s, jb, h2, lo_r, hi_r);
                    }

                    // ---- online softmax with lazy rescaling (the exponent reference moves only when the maximum outgrows
                    // it by more than 2^PF_TAU)
                    float mx = s[0];
#pragma unroll
                    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
                    mx = half_swap_max(mx) * p.c;
                    G4B_PF_LAZY_RESCALE(acc, DT, m_run, l_run, mx);
                    const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
                    float psum = 0.f;
                    u4 pf[2];  // [16-key group] -> 8 keys of this lane half
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        float e[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) e[j] = fast_exp2(__builtin_fmaf(s[8 * u + j], p.c, -m_safe));
                        pf[u] = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint32_t w = pf[u][j];
                            psum = T::sum2(w, psum);  // the row sum adds up the rounded values the second product uses
                        }
                    }
                    l_run += psum;

                    // ---- O^T += V^T P
                    {
                        VFrag vbuf[PW_PD];
#pragma unroll
                        for (int i = 0; i < PW_PD; ++i) vbuf[i] = v_issue(i);
#pragma unroll
                        for (int idx = 0; idx < PV_STEPS; idx += 2) {
                            VFrag f0 = vbuf[idx % PW_PD], f1 = vbuf[(idx + 1) % PW_PD];
                            wait_pair2(f0, f1, (PV_STEPS - 2 - idx) / 2);
                            if (idx + PW_PD < PV_STEPS) {
                                vbuf[idx % PW_PD] = v_issue(idx + PW_PD);
                                vbuf[(idx + 1) % PW_PD] = v_issue(idx + 1 + PW_PD);
                            }
                            const int cu = idx / DT, dt = idx % DT;  // DT is even: both steps share the key group
                            const u4 a0 = {f0.lo[0], f0.lo[1], f0.hi[0], f0.hi[1]};
                            const u4 a1 = {f1.lo[0], f1.lo[1], f1.hi[0], f1.hi[1]};
                            acc[dt] = T::mfma32(a0, pf[cu], acc[dt]);
                            acc[dt + 1] = T::mfma32(a1, pf[cu], acc[dt + 1]);
                        }
                    }
                }
                vm_wait_all();
                __syncthreads();
            }
        }
    }

    // ---- epilogue: the wave turns its 32 x 512 block around in LDS, 256 columns at a time (32 KiB of the staging
    // area per wave, free after the loop's last barrier), and stores 1 KiB row halves
    const float l_tot = QS ? half_swap_sum(row16_pair_sum(l_run)) : half_swap_sum(l_run);
    const bool partial = nsplit > 1;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;  // a key split's rows are normalised too: they are kept in 16 bits
    char* wbase = smem + wave * (32 * 256 * 4);
    if (partial && h2 == 0 && row_ok && (!QS || n32 < 16)) {
        const int64_t prow = ((int64_t)(a_idx * nsplit + split) * p.H + (g * R + hh)) * Tq + ti;
        p.part_ml[prow * 2] = (m_run == -INFINITY) ? 0.f : m_run;
        p.part_ml[prow * 2 + 1] = l_tot;
    }
    const int tokb_shift = __ffs(TOKB) - 1;  // TOKB = BM / R is a power of two
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // a row's head, token and offset are scalar arithmetic then
    // both destinations are rows of D elements at (head, token): the split's [pair][H][Tq][D] block in the cache's type,
    // or o with the caller's strides and type
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
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if constexpr (QS) {
#pragma unroll
            for (int bl = 0; bl < 16; ++bl) {  // d = 256 half + 16 bl + 4 kg + 0..3: piece 4 bl + kg of the row's half
                const int pc = 4 * bl + kg;
                *reinterpret_cast<f4*>(wbase + n16 * 1024 + ((pc ^ n16) * 16)) = acc16[half * 16 + bl] * inv;
            }
        } else {
#pragma unroll
            for (int d8 = 0; d8 < 8; ++d8)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int dt = half * 8 + d8;
                    f4 v = {acc[dt][4 * q4] * inv, acc[dt][4 * q4 + 1] * inv, acc[dt][4 * q4 + 2] * inv, acc[dt][4 * q4 + 3] * inv};
                    const int pc = 8 * d8 + 2 * q4 + h2;
                    *reinterpret_cast<f4*>(wbase + n32 * 1024 + ((pc ^ (n32 & 15)) * 16)) = v;
                }
        }
        // Rows go eight at a time, their LDS reads first and in one block; the type is chosen per batch and the rows of
        // a batch are one scalar offset plus a stride apart (a wave has its SIMD to itself here: row by row -- read,
        // wait, compute the offset, choose the type, convert, store -- every row paid the LDS latency and some thirty
        // instructions by itself).
        auto store_rows = [&](auto nt, const int dt) {
            constexpr bool NT = decltype(nt)::value;
#pragma unroll 1
            for (int r0 = 0; r0 < WROWS; r0 += 8) {
                f4 v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)  // 64 lanes x 16 bytes = 256 fp32 columns of one row
                    v[j] = *reinterpret_cast<const f4*>(wbase + (r0 + j) * 1024 + ((lane ^ ((r0 + j) & 15)) * 16));
                const int rs = wave_u * WROWS + r0;  // first row of the batch
                if (TOKB >= 8) {
                    // the batch lies inside one head: consecutive tokens, one stride apart
                    const int hr = rs >> tokb_shift, tr0 = tok0 + (rs & (TOKB - 1));
                    const int64_t off0 = base_off + (int64_t)hr * head_stride + (int64_t)tr0 * row_stride + half * 256;
                    const int n_ok = Tq - tr0;
                    if (dt == DT_F32) {
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (j < n_ok) store4<NT>(dst, off0 + (int64_t)j * row_stride + lane * 4, DT_F32, v[j]);
                    } else if (dt == DT_F16) {
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (j < n_ok) store4<NT>(dst, off0 + (int64_t)j * row_stride + lane * 4, DT_F16, v[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (j < n_ok) store4<NT>(dst, off0 + (int64_t)j * row_stride + lane * 4, DT_BF16, v[j]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int rr = rs + j;
                        const int hr = rr >> tokb_shift, tr = tok0 + (rr & (TOKB - 1));
                        if (tr < Tq)
                            store4<NT>(dst, base_off + (int64_t)hr * head_stride + (int64_t)tr * row_stride + half * 256 + lane * 4, dt, v[j]);
                    }
                }
            }
        };
        // written once and not read here again: o goes out non-temporal, so that the rows do not displace K/V tiles in
        // L2 (S = 8192 0.5 % faster, the 512-key sliding window 3.7 %; the same hint on the Q loads cost 1.3 .. 4 %)
        if (partial) store_rows(std::false_type{}, T::dt);
        else store_rows(std::true_type{}, p.o_dt);
    }
}

template <class T, bool QS>
__global__ __launch_bounds__(256) void attn_prefill_wide_kernel(const AttnParams p) {
    extern __shared__ __align__(16) char smem[];
    __shared__ int sh_scan[8];
    prefill_wide_body<T, QS>(p, blockIdx.x, smem, sh_scan);
}

}  // namespace g4b
