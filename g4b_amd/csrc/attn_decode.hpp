// Decode attention for gfx950: the query block of one (slot, kv head) pair is at most 16 rows
// (R = H/G heads x Tq tokens), the KV cache is streamed from HBM exactly once per pair.
//
// Work decomposition.  Every in-phase slot contributes ceil(keys / 32) tiles per kv head; the
// tiles of all pairs form one flat list that is dealt to NW single-wave workgroups in contiguous
// runs (worker w owns flat tiles [begin(w), begin(w+1)), TileShares below: equal shares, or 26 : 24
// between workers on even and odd XCDs).  The split is computed on the device from
// time_dim_sizes, so the grid is static while the balance follows the real lengths.  A worker
// whose range covers a whole pair writes the output directly; otherwise it leaves an
// un-normalised fp32 partial (acc, running max, running sum) in workspace slot (w + pair) and a
// second kernel merges the partials of each pair.  Launches whose window is at most 512 keys take a one-kernel
// variant instead (attn_decode_pair: four waves per pair, merged through LDS).
//
// Tile math (one wave, 32 keys).  S^T = K Q^T and O^T += V^T P run on v_mfma_f32_16x16x32.
// The 16 output columns carry (row, class) pairs: the D/8 16-byte pieces of a key row are dealt
// round-robin to CL classes, lane quad members read neighbouring pieces (64 contiguous bytes per
// quad, 256 per key row and instruction), and the diagonal (class == class) blocks of the MFMA
// result summed over the CL lanes of a row give the dot product.  P stays in registers: the
// score layout of the first MFMA is the B-operand layout of the second, with the key order of the
// contraction chosen to match.  V^T operands are built with an in-lane 8x8 16-bit transpose.
#pragma once
#ifndef G4B_DEC_LD
#define G4B_DEC_LD ld16_stream
#endif
#include "common.hpp"

namespace g4b {

constexpr int DEC_TILE = 32;  // keys per wave iteration

G4B_DEV int slot_tiles(const SlotInfo& s) { return (s.window - s.klo + DEC_TILE - 1) / DEC_TILE; }
G4B_DEV int slot_tiles(const AttnParams& p, int b) { return slot_tiles(slot_info(p, b)); }
// Share-out of the flat tile list over nw workers.  The odd XCDs of the chip stream from HBM more slowly than the even
// ones (a decode batch with equal shares: workers on XCDs 0, 2, 4, 6 took 148 .. 160 us, those on 1, 3, 5, 7
// 165 .. 172 us, on three boxes, and the slow half followed the hardware when the shares were swapped), and a launch
// lasts as long as its slowest worker, so a worker on an even XCD gets 25 + XCD_SKEW parts of the list for every
// 25 - XCD_SKEW on an odd one (batch of 64: 0.820 -> 0.835 of 8 TB/s; the odd XCDs still finish last, more slowly per
// tile while the even ones take more of the memory system, so the gain is the shorter tail, not the 8 %).  Worker w
// starts at tile floor(total * cum(w) / cum(nw)), cum(w) = 25 w + e(w) being the parts of the workers before it;
// unweighted (parity unknown, or fewer than two tiles per worker, where a share could come out empty) cum(w) = w.
constexpr int XCD_SKEW = 1;  // parts out of 25 taken from an odd XCD's worker and given to an even one's (2 measured the same, 3 worse)
struct TileShares {
    int total, nw, shift;  // shift < 0: equal shares
    uint32_t cn;           // cum(nw)
    bool small;            // total * cum(nw) fits 32 bits
    __host__ __device__ uint32_t cum(int w) const {
        if (shift < 0) return (uint32_t)w;
        const int period = 2 << shift, r = w & (period - 1);
        return 25u * (uint32_t)w + (uint32_t)(XCD_SKEW * (r <= period / 2 ? r : period - r));
    }
    __host__ __device__ int64_t begin(int w) const {  // first tile of worker w; begin(nw) = total
        const uint32_t c = cum(w);
        if (small) return (int64_t)((uint32_t)total * c / cn);  // the common case in 32-bit arithmetic throughout
        return (int64_t)((uint64_t)total * c / cn);
    }
    __host__ __device__ int owner(int64_t x) const {  // the worker that owns tile x: the largest w with begin(w) <= x
        uint32_t c;
        if (small) c = ((uint32_t)(x + 1) * cn - 1u) / (uint32_t)total;
        else c = (uint32_t)(((uint64_t)(x + 1) * cn - 1u) / (uint32_t)total);
        if (shift < 0) return (int)c;
        int w = (int)(c / 25u);  // c < 25 nw + 4
        if (cum(w) > c) --w;
        return w;
    }
};
// num_workers: the launch's worker count; xcd_shift: AttnParams::xcd_shift.  (Host-callable so that the arithmetic the
// workers and the merge kernel share can be brute-forced on the CPU.)
__host__ __device__ inline TileShares make_tile_shares(int num_workers, int xcd_shift, int total) {
    TileShares s;
    s.total = total;
    s.nw = num_workers < total ? num_workers : total;  // never more workers than tiles: every worker below nw owns >= 1 tile
    s.shift = (xcd_shift >= 0 && total >= 2 * s.nw) ? xcd_shift : -1;
    s.cn = s.cum(s.nw);
    s.small = (uint64_t)(uint32_t)total * s.cn < ((uint64_t)1 << 32);
    return s;
}
G4B_DEV TileShares tile_shares(const AttnParams& p, int total) { return make_tile_shares(p.NW, p.xcd_shift, total); }
template <int CL>
G4B_DEV float pick(const f4& c, int e, int cls) {
    // element e*CL + cls of c without dynamic register indexing
    if constexpr (CL == 1) {
        return c[e];
    } else if constexpr (CL == 2) {
        return cls ? c[2 * e + 1] : c[2 * e];
    } else {
        float lo = (cls & 1) ? c[1] : c[0];
        float hi = (cls & 1) ? c[3] : c[2];
        return (cls & 2) ? hi : lo;
    }
}

// One segment: tiles [t0, t1) of pair (bb, g) whose slot has tlb tiles per kv head.  Worker w
// writes the output itself when the segment is the whole pair, else partial slot (w + pair).
//
// DH > 1: the workgroup has DH waves and wave hv owns columns [hv*D/DH, (hv+1)*D/DH) of the head dimension: its share
// of q, of every K and V row and of the output.  The waves add their partial dot products through LDS once per tile
// and then run the same softmax, so the register tiling is that of head dimension D/DH.
//
// lds_part != nullptr: the un-normalised result goes to that LDS block ([16 rows][D] floats, then [16 rows][2] of
// (reference, sum)) whatever the segment covers; the caller merges the blocks of its waves.
//
// QS: the query is wider than the cache type and enters the first product as two operands (rounded value, rounding
// error), so the scores see the unrounded query.
//
// PF: key tiles whose loads are in flight ahead of the arithmetic.  One leaves a streaming worker's registers to its
// 32 KB tile and is all that a launch of a thousand workers needs; in a mixed launch, where the stream has part of the
// chip and the kernel's register budget is that of the prefill body anyway, a worker asks for two tiles at a time.
template <int D, int CL, class T, int DH, bool QS, int PF = 1>
G4B_DEV void decode_segment(const AttnParams& p, const SlotInfo& si, int w, int bb, int g, int t0, int t1, int tlb,
                            float* xch, float* lds_part = nullptr) {
    constexpr int DL = D / DH;         // columns this wave owns
    constexpr int E = 4 / CL;          // scores a lane keeps per 16-row MFMA tile
    constexpr int KT = 16 / CL;        // keys per MFMA tile
    constexpr int NT = DEC_TILE / KT;  // MFMA tiles per 32 keys
    constexpr int PIECES = DL / 8;     // 16-byte pieces of a key row this wave reads
    constexpr int NC = PIECES / (4 * CL);
    constexpr int DC = DL / 128;
    constexpr int ROWB = D * 2;  // bytes per cache row
    static_assert(NC >= 1 && DC >= 1, "head dim too small for this tiling");
    const int lane = threadIdx.x & 63;
    const int hv = (DH > 1) ? (int)(threadIdx.x >> 6) : 0;
    const int m16 = lane & 15, g4 = lane >> 4;
    const int cls = m16 % CL;
    const int G = p.G, Tq = p.Tq;
    const int NR = p.R * Tq;

    const int KV_CTX = p.KV_CTX;
    const char* kbase =
        static_cast<const char*>(p.k) + ((int64_t)bb * p.k_sb + (int64_t)g * KV_CTX * D + hv * DL) * 2;
    const char* vbase =
        static_cast<const char*>(p.v) + ((int64_t)bb * p.v_sb + (int64_t)g * KV_CTX * D + hv * DL) * 2;

    // this lane's query row (as MFMA column n = m16 = row*CL + cls)
    const int row = m16 / CL;
    const bool row_ok = row < NR;
    const int hh = row_ok ? row / Tq : 0;
    const int ti = row_ok ? row % Tq : 0;
    int lo_r, hi_r;
    row_range(p, si, ti, lo_r, hi_r);
    int lo_max, hi_min, dummy;
    row_range(p, si, Tq - 1, lo_max, dummy);
    row_range(p, si, 0, dummy, hi_min);

    u4 qf[NC];
    u4 qf_lo[QS ? NC : 1];
    {
        const int64_t qoff =
            (int64_t)bb * p.q_s[0] + (int64_t)(g * p.R + hh) * p.q_s[1] + (int64_t)ti * p.q_s[2] + hv * DL;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int piece = cls + CL * g4 + 4 * CL * c;
            u4 z = {0, 0, 0, 0};
            if constexpr (QS) {
                qf[c] = z;
                qf_lo[c] = z;
                if (row_ok) load8_split<T>(p.q, qoff + piece * 8, p.q_dt, qf[c], qf_lo[c]);
            } else {
                qf[c] = row_ok ? load8_as<T>(p.q, qoff + piece * 8, p.q_dt) : z;
            }
        }
    }

    // byte offset of (logical key j, 16-byte piece) in the ring; j clamped to the window
    auto key_off = [&](int j) -> uint32_t {
        j = min(j, si.window - 1);
        int r = si.ring_start + j;
        r = (r >= KV_CTX) ? r - KV_CTX : r;
        return (uint32_t)r * ROWB;
    };

    u4 kreg[PF][NT][NC];
    u4 vreg[PF][DC][8];
    auto load_k = [&](int t, auto buf) {
        const int jb = si.klo + t * DEC_TILE;
#pragma unroll
        for (int tau = 0; tau < NT; ++tau) {
            const uint32_t ro = key_off(jb + tau * KT + m16 / CL);
#pragma unroll
            for (int c = 0; c < NC; ++c)
                kreg[decltype(buf)::value][tau][c] = G4B_DEC_LD(kbase, ro + (uint32_t)(cls + CL * g4 + 4 * CL * c) * 16u);
        }
    };
    auto load_v = [&](int t, auto buf) {
        const int jb = si.klo + t * DEC_TILE;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t ro = key_off(jb + (s / E) * KT + g4 * E + (s % E));
#pragma unroll
            for (int dc = 0; dc < DC; ++dc)
                vreg[decltype(buf)::value][dc][s] = G4B_DEC_LD(vbase, ro + (uint32_t)(m16 + 16 * dc) * 16u);
        }
    };

    float m_run = -INFINITY, l_run = 0.f;
    f4 acc[DC * 8];
#pragma unroll
    for (int i = 0; i < DC * 8; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};

    static_assert(PF == 1 || PF == 2, "one or two tiles ahead");
    load_k(t0, std::integral_constant<int, 0>{});
    load_v(t0, std::integral_constant<int, 0>{});
    if constexpr (PF == 2) {
        if (t0 + 1 < t1) {
            load_k(t0 + 1, std::integral_constant<int, 1>{});
            load_v(t0 + 1, std::integral_constant<int, 1>{});
        }
    }
    if constexpr (DH > 1) __syncthreads();  // the exchange buffers of the previous segment are free
    // one key tile: the tile in buffer `buf`, whose next occupant (tile t + PF) is asked for as soon as the buffer is read
    auto tile = [&](int t, auto buf) {
        constexpr int BUF = decltype(buf)::value;
        const int jb = si.klo + t * DEC_TILE;
        // ---- S^T = K Q^T -------------------------------------------------------
        float sc[8];
#pragma unroll
        for (int tau = 0; tau < NT; ++tau) {
            f4 c4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if constexpr (QS) c4 = T::mfma16(kreg[BUF][tau][c], qf_lo[c], c4);
                c4 = T::mfma16(kreg[BUF][tau][c], qf[c], c4);
            }
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float x = pick<CL>(c4, e, cls);
                if constexpr (CL >= 2) x += quad_xor1(x);
                if constexpr (CL == 4) x += quad_xor2(x);
                sc[tau * E + e] = x * p.c;
            }
        }
        if (t + PF < t1) load_k(t + PF, buf);
        if constexpr (DH > 1) {
            // add the other waves' partial dot products; buffers alternate so one barrier per tile is enough
            float* xb = xch + (t & 1) * (DH * 8 * 64);
#pragma unroll
            for (int s = 0; s < 8; ++s) xb[(hv * 8 + s) * 64 + lane] = sc[s];
            __syncthreads();
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                float x = 0.f;
#pragma unroll
                for (int h = 0; h < DH; ++h) x += xb[(h * 8 + s) * 64 + lane];  // same order in every wave
                sc[s] = x;
            }
        }

        // ---- online softmax (per row; a row's keys are spread over the 4 lane groups)
        if (jb < lo_max || jb + DEC_TILE > hi_min) {
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int j = jb + (s / E) * KT + g4 * E + (s % E);
                if (j < lo_r || j >= hi_r) sc[s] = -INFINITY;
            }
        }
        float mx = sc[0];
#pragma unroll
        for (int s = 1; s < 8; ++s) mx = fmaxf(mx, sc[s]);
        mx = half_swap_max(row_swap_max(mx));  // over the lanes l, l ^ 16, l ^ 32, l ^ 48 that share a query row
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float ps[8], psum = 0.f;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            ps[s] = fast_exp2(sc[s] - m_safe);
            psum += ps[s];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        const u4 pf = {T::pack2(ps[0], ps[1]), T::pack2(ps[2], ps[3]), T::pack2(ps[4], ps[5]), T::pack2(ps[6], ps[7])};
        // (nothing to rescale on the first tile, and on most later ones no row's maximum has moved)
        if (t > t0 && __any(alpha != 1.f)) {
#pragma unroll
            for (int i = 0; i < DC * 8; ++i) acc[i] *= alpha;
        }

        // ---- O^T += V^T P ------------------------------------------------------
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            u4 vt[8];
            transpose8x8_b16(vreg[BUF][dc], vt);
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) acc[dc * 8 + jj] = T::mfma16(vt[jj], pf, acc[dc * 8 + jj]);
        }
        if (t + PF < t1) load_v(t + PF, buf);
    };
    for (int t = t0; t < t1; t += PF) {
        tile(t, std::integral_constant<int, 0>{});
        if constexpr (PF == 2) {
            if (t + 1 < t1) tile(t + 1, std::integral_constant<int, 1>{});
        }
    }

    // ---- epilogue -----------------------------------------------------------------
    const float l_tot = half_swap_sum(row_swap_sum(l_run));
    const bool whole = (t0 == 0 && t1 == tlb) && lds_part == nullptr;
    if (row_ok) {
        if (whole) {
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            const int64_t ooff =
                (int64_t)bb * p.o_s[0] + (int64_t)(g * p.R + hh) * p.o_s[1] + (int64_t)ti * p.o_s[2];
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    float v8[8];
#pragma unroll
                    for (int jj = 0; jj < 8; ++jj) v8[jj] = pick<CL>(acc[dc * 8 + jj], e, cls) * inv;
                    const int d0 = hv * DL + 128 * dc + (4 * g4 + e * CL + cls) * 8;
                    store8(p.o, ooff + d0, p.o_dt, v8);
                }
            }
        } else {
            const int64_t slot = (int64_t)w + (int64_t)bb * G + g;
            float* po = lds_part ? lds_part + row * D : p.part_o + (slot * NR + row) * D;
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    float v8[8];
#pragma unroll
                    for (int jj = 0; jj < 8; ++jj) v8[jj] = pick<CL>(acc[dc * 8 + jj], e, cls);
                    const int d0 = hv * DL + 128 * dc + (4 * g4 + e * CL + cls) * 8;
                    store8(po, d0, DT_F32, v8);
                }
            }
            if (cls == 0 && g4 == 0 && hv == 0) {
                float* pm = lds_part ? lds_part + 16 * D + row * 2 : p.part_ml + (slot * NR + row) * 2;
                pm[0] = m_run;
                pm[1] = l_tot;
            }
        }
    }
}

// Worker w of a launch: its share of the flat tile list.  Called by every wave of the worker (DH of them); xch is the
// worker's exchange buffer when DH > 1.
template <int D, int CL, class T, int DH, bool QS, int PF = 1>
G4B_DEV void decode_worker_body(const AttnParams& p, int w, float* xch) {
    const int lane = threadIdx.x & 63;  // every wave of the worker does the same bookkeeping
    const int B = p.B, G = p.G;

    if (p.NW == 0) {
        // no workspace: worker w owns the whole pair w
        if (w >= B * G) return;
        const int bb = w / G, g = w % G;
        const SlotInfo si = slot_info(p, bb);
        const int tlb = slot_tiles(si);
        if (tlb > 0) {
            decode_segment<D, CL, T, DH, QS, PF>(p, si, w, bb, g, 0, tlb, tlb, xch);
        } else if (si.active && (DH == 1 || threadIdx.x < 64)) {  // one wave of the worker
            // in-phase slot without any visible key: defined as zeros (no merge kernel runs on this path)
            const int NR = p.R * p.Tq;
            for (int idx = lane; idx < NR * (D / 4); idx += 64) {
                const int row = idx / (D / 4), c4 = idx % (D / 4);
                const int64_t ooff = (int64_t)bb * p.o_s[0] + (int64_t)(g * p.R + row / p.Tq) * p.o_s[1] +
                                     (int64_t)(row % p.Tq) * p.o_s[2];
                store4(p.o, ooff + c4 * 4, p.o_dt, f4{0.f, 0.f, 0.f, 0.f});
            }
        }
        return;
    }

    if (B == 1) {
        // A single slot (single-sequence decode: a launch of a few microseconds that is all latency): its tile count is
        // the whole list, so the sums and prefix sums over the slots and the search for the slot fall away.
        const SlotInfo si = slot_info(p, 0);
        const int tlb = slot_tiles(si);
        const TileShares shares = tile_shares(p, G * tlb);
        if (w >= shares.nw) return;  // (also: no tiles at all)
        const int64_t ws = shares.begin(w), we = shares.begin(w + 1);
        for (int g = (int)(ws / tlb); g < G && (int64_t)g * tlb < we; ++g) {
            const int64_t fs = (int64_t)g * tlb;
            const int t0 = (int)(max(ws, fs) - fs);
            const int t1 = (int)(min(we, fs + tlb) - fs);
            if (t1 > t0) decode_segment<D, CL, T, DH, QS, PF>(p, si, w, 0, g, t0, t1, tlb, xch);
        }
        return;
    }

    // ---- flat tile list: total, then this worker's range ------------------------------------
    // lane l keeps what it read of slot l (the first 64 slots) for the second pass and for the segments
    int total = 0, tl_first = 0;
    SlotInfo si_first = {};
    for (int b0 = 0; b0 < B; b0 += 64) {
        const int b = b0 + lane;
        int tl = 0;
        if (b < B) {
            const SlotInfo s = slot_info(p, b);
            tl = slot_tiles(s);
            if (b0 == 0) si_first = s;
        }
        if (b0 == 0) tl_first = tl;
        total += G * tl;
    }
    total = wave_sum_i(total);
    const TileShares shares = tile_shares(p, total);
    if (w >= shares.nw) return;
    const int64_t ws = shares.begin(w);
    const int64_t we = shares.begin(w + 1);

    int carry = 0;
    for (int b0 = 0; b0 < B; b0 += 64) {
        const int bl = b0 + lane;
        const int tl = b0 == 0 ? tl_first : ((bl < B) ? slot_tiles(p, bl) : 0);
        const int cnt = G * tl;
        const int incl = wave_incl_scan_i(cnt, lane);
        const int excl = carry + incl - cnt;
        const bool hit = cnt > 0 && (int64_t)excl < we && (int64_t)excl + cnt > ws;
        uint64_t mask = __ballot(hit);
        while (mask) {
            const int src = __builtin_ctzll(mask);
            mask &= mask - 1;
            const int bb = b0 + src;
            const int ex = __builtin_amdgcn_readlane(excl, src);
            const int tlb = __builtin_amdgcn_readlane(tl, src);
            const SlotInfo si = b0 == 0 ? slot_info_of_lane(si_first, src) : slot_info(p, bb);
            for (int g = 0; g < G; ++g) {
                const int64_t fs = (int64_t)ex + (int64_t)g * tlb;
                const int t0 = (int)(max(ws, fs) - fs);
                const int t1 = (int)(min(we, fs + tlb) - fs);
                if (t1 > t0) decode_segment<D, CL, T, DH, QS, PF>(p, si, w, bb, g, t0, t1, tlb, xch);
            }
        }
        carry += __builtin_amdgcn_readlane(incl, 63);
        if ((int64_t)carry >= we) break;
    }
}

template <int D, int CL, class T, int DH, bool QS>
__global__ __launch_bounds__(64 * DH, 1) void attn_decode_worker(const AttnParams p) {
    __shared__ float xch_buf[DH > 1 ? 2 * DH * 8 * 64 : 1];
    decode_worker_body<D, CL, T, DH, QS>(p, blockIdx.x, xch_buf);
}

// Short windows (a sliding-window layer: at most a few dozen tiles per pair): one workgroup of four waves per (slot, kv
// head) pair, each wave a quarter of the pair's tiles, merged through LDS in the same launch.  With so little work per
// pair the two-kernel path is all latency (worker prologue, partials out and back in, second launch).
constexpr int DEC_PAIR_WAVES = 4;
template <int D>
constexpr int dec_pair_smem() { return DEC_PAIR_WAVES * (16 * D + 32) * (int)sizeof(float); }

template <int D, int CL, class T, bool QS>
G4B_DEV void decode_pair_body(const AttnParams& p, int pair, float* pair_smem) {
    constexpr int BLK = 16 * D + 32;  // floats per wave block
    const int tid = threadIdx.x, wave = tid >> 6;
    const int bb = pair / p.G, g = pair % p.G;
    const SlotInfo si = slot_info(p, bb);
    if (!si.active) return;
    const int NR = p.R * p.Tq;
    const int tl = slot_tiles(si);
    float* mine = pair_smem + wave * BLK;
    const int t0 = wave * tl / DEC_PAIR_WAVES, t1 = (wave + 1) * tl / DEC_PAIR_WAVES;
    if (t1 > t0) {
        decode_segment<D, CL, T, 1, QS>(p, si, 0, bb, g, t0, t1, tl, nullptr, mine);
    } else if ((tid & 63) < 16) {
        mine[16 * D + (tid & 63) * 2] = -INFINITY;  // this wave brought no keys
        mine[16 * D + (tid & 63) * 2 + 1] = 0.f;
    }
    __syncthreads();
    // merge: a thread per four output columns of a row
    constexpr int LPR = D / 4;
    for (int item = tid; item < NR * LPR; item += 64 * DEC_PAIR_WAVES) {
        const int row = item / LPR, c4 = item % LPR;
        float mref = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_PAIR_WAVES; ++w) mref = fmaxf(mref, pair_smem[w * BLK + 16 * D + row * 2]);
        const float msafe = (mref == -INFINITY) ? 0.f : mref;
        f4 acc = {0.f, 0.f, 0.f, 0.f};
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_PAIR_WAVES; ++w) {
            const float m = pair_smem[w * BLK + 16 * D + row * 2];
            if (m != -INFINITY) {
                const float e = fast_exp2(m - msafe);
                acc += *reinterpret_cast<const f4*>(pair_smem + w * BLK + row * D + c4 * 4) * e;
                l += pair_smem[w * BLK + 16 * D + row * 2 + 1] * e;
            }
        }
        const float inv = l > 0.f ? 1.f / l : 0.f;
        const int64_t ooff =
            (int64_t)bb * p.o_s[0] + (int64_t)(g * p.R + row / p.Tq) * p.o_s[1] + (int64_t)(row % p.Tq) * p.o_s[2];
        store4(p.o, ooff + c4 * 4, p.o_dt, acc * inv);
    }
}

template <int D, int CL, class T, bool QS>
__global__ __launch_bounds__(64 * DEC_PAIR_WAVES, 1) void attn_decode_pair(const AttnParams p) {
    extern __shared__ __align__(16) float pair_smem[];
    decode_pair_body<D, CL, T, QS>(p, blockIdx.x, pair_smem);
}

// Merge the partials of each (slot, kv head) pair: one workgroup of 256 threads per (pair, query row).  The workers
// that own tiles of the pair are spread over the four waves and their loads are independent, so the merge costs a few
// memory round trips however many workers a long slot was dealt to.
template <int D>
struct DecodeCombineSmem {
    float sm_max[4];
    float sm_l[4];
    f4 sm_acc[4][D / 4];
};
template <int D>
G4B_DEV void decode_combine_body(const AttnParams& p, int pair, int row, DecodeCombineSmem<D>& sm) {
    float(&sm_max)[4] = sm.sm_max;
    float(&sm_l)[4] = sm.sm_l;
    f4(&sm_acc)[4][D / 4] = sm.sm_acc;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = pair / p.G, g = pair % p.G;
    const int B = p.B, G = p.G;
    const int NR = p.R * p.Tq;

    // flat start of this pair and total tile count (same arithmetic as the workers), computed by every wave
    int before = 0, total = 0;
    SlotInfo si_first = {};  // lane l keeps what it read of slot l (the first 64 slots)
    if (B == 1) {  // a single slot: nothing to sum (the launch is all latency, and this is a dozen instructions of it)
        si_first = slot_info(p, 0);
        total = G * slot_tiles(si_first);
    }
    for (int b0 = 0; b0 < (B == 1 ? 0 : B); b0 += 64) {
        const int x = b0 + lane;
        int c = 0;
        if (x < B) {
            const SlotInfo s = slot_info(p, x);
            c = G * slot_tiles(s);
            if (b0 == 0) si_first = s;
        }
        total += c;
        before += (x < b) ? c : 0;
    }
    if (B > 1) {
        total = wave_sum_i(total);
        before = wave_sum_i(before);
    }

    const SlotInfo si = B == 1 ? si_first : (b < 64 ? slot_info_of_lane(si_first, b) : slot_info(p, b));
    if (!si.active) return;
    const int tl = slot_tiles(si);
    const int64_t ooff = (int64_t)b * p.o_s[0] + (int64_t)(g * p.R + row / p.Tq) * p.o_s[1] + (int64_t)(row % p.Tq) * p.o_s[2];
    if (tl == 0) {
        // in-phase slot without any visible key: defined as zeros
        if (tid < D / 4) store4(p.o, ooff + tid * 4, p.o_dt, f4{0.f, 0.f, 0.f, 0.f});
        return;
    }
    if (p.NW == 0) return;  // one wave owned the whole pair
    const TileShares shares = tile_shares(p, total);
    const int64_t fs = (int64_t)before + (int64_t)g * tl;
    const int w0 = shares.owner(fs), w1 = shares.owner(fs + tl - 1);
    if (w0 == w1) return;  // a single worker owned the pair and wrote the output itself

    // partial of worker w for this pair and row: slot w + pair
    auto ml_of = [&](int w) { return p.part_ml + (((int64_t)w + pair) * NR + row) * 2; };
    // Wave k takes workers w0 + k, w0 + k + 4, ...; a lane owns four output columns.  Every wave sums its workers
    // against a reference of its own (the largest one it has seen, -inf marks a worker without keys for the row), so
    // that nothing waits for a first pass over all references; the four waves are merged through LDS at the end.
    constexpr int LPR = D / 4 < 64 ? D / 4 : 64;  // lanes that hold a row
    constexpr int NV = D / 4 / LPR;               // float4 pieces per lane: piece v covers columns (v*64 + lane)*4..+3
    constexpr int UN = NV == 1 ? 16 : 8;          // workers whose loads are in flight together
    f4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = f4{0.f, 0.f, 0.f, 0.f};
    float l = 0.f, ref = -INFINITY;
    for (int wb = w0 + wave; wb <= w1; wb += 4 * UN) {
        float wgt[UN], lw[UN];
        f4 ov[UN][NV];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int w = min(wb + 4 * u, w1);  // clamped loads, masked below
            const float* ml = ml_of(w);
            wgt[u] = ml[0];
            lw[u] = ml[1];
            const float* po = p.part_o + (((int64_t)w + pair) * NR + row) * D;
#pragma unroll
            for (int v = 0; v < NV; ++v)
                ov[u][v] = (lane < LPR) ? *reinterpret_cast<const f4*>(po + (v * 64 + lane) * 4) : f4{0.f, 0.f, 0.f, 0.f};
        }
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (wb + 4 * u <= w1) bm = fmaxf(bm, wgt[u]);
        if (bm > ref) {  // the same in every lane
            const float a = fast_exp2(ref - bm);  // 0 while ref is -inf
#pragma unroll
            for (int v = 0; v < NV; ++v) acc[v] = acc[v] * a;
            l *= a;
            ref = bm;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const bool live = (wb + 4 * u <= w1) && (wgt[u] != -INFINITY);
            if (live) {
                const float e = fast_exp2(wgt[u] - ref);
#pragma unroll
                for (int v = 0; v < NV; ++v) acc[v] += ov[u][v] * e;
                l += lw[u] * e;
            }
        }
    }
    if (lane < LPR) {
#pragma unroll
        for (int v = 0; v < NV; ++v) sm_acc[wave][v * 64 + lane] = acc[v];
    }
    if (lane == 0) {
        sm_l[wave] = l;
        sm_max[wave] = ref;
    }
    __syncthreads();
    if (tid < D / 4) {
        const float mref = fmaxf(fmaxf(sm_max[0], sm_max[1]), fmaxf(sm_max[2], sm_max[3]));
        f4 r = {0.f, 0.f, 0.f, 0.f};
        float lt = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float e = sm_max[k] == -INFINITY ? 0.f : fast_exp2(sm_max[k] - mref);
            r += sm_acc[k][tid] * e;
            lt += sm_l[k] * e;
        }
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        store4(p.o, ooff + tid * 4, p.o_dt, r * inv);
    }
}

template <int D>
__global__ __launch_bounds__(256) void attn_decode_combine(const AttnParams p) {
    __shared__ DecodeCombineSmem<D> sm;
    decode_combine_body<D>(p, blockIdx.x, blockIdx.y, sm);
}

}  // namespace g4b
