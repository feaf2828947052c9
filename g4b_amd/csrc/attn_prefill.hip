// Prefill (and chunked-prefill) attention for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (slot, kv head) pair: all R = H/G query
// heads of the group for 128/R consecutive tokens, so a staged K/V tile serves the whole GQA
// group.  Each wave owns 32 rows.  The KV loop walks 64-key tiles from the first tile any row
// of the workgroup can see to the causal diagonal; tiles entirely inside every row's range run
// without masks, edge tiles (sliding-window lower edge, causal diagonal, window end) compare
// per element.
//
// Staging.  Tiles are double-buffered in LDS.  K goes global -> LDS directly
// (global_load_lds_dwordx4, no registers): rows stay row-major and unpadded, the 16-byte pieces
// of a row are XOR-swizzled with (row & 15) by choosing which global piece each lane fetches.
// V passes through registers for an in-lane 8x8 16-bit transpose and is stored as V^T
// ([d][key], 128-byte rows) with the 16-byte column groups XOR-swizzled.  Both are read back
// with conflict-free ds_read_b128 directly in MFMA operand layout.
//
// Math per tile and wave: S^T[64 keys x 32 rows] = K Q^T and O^T[D x 32 rows] += V^T P on
// v_mfma_f32_32x32x16 (fp16 or bf16 operands, fp32 accumulate).  Q stays in registers as the B
// operand; P never leaves registers: the accumulator layout of S^T is the B-operand layout of
// the second product once the key order inside each 16-key group of V^T is permuted to match.
// LDS operand reads run a fixed number of steps ahead of the MFMAs that consume them.
// Softmax is online in fp32 with exp2 and scale*log2(e) folded into one FMA; the row statistics
// live one row per lane pair (lane, lane^32).
#include "common.hpp"
#include "launch.hpp"

namespace g4b {

constexpr int PF_BM = 128;  // query rows per workgroup
constexpr int PF_BN = 64;   // keys per tile
constexpr int PF_PD = 4;    // LDS operand reads in flight ahead of the MFMA that uses them
constexpr float PF_TAU = 8.f;  // log2 of the growth of a row maximum that triggers a rescale

template <int D>
struct PfSmem {
    static constexpr int KROW = D * 2;  // bytes per K row in LDS (unpadded, swizzled)
    static constexpr int KBYTES = PF_BN * KROW;
    static constexpr int VROW = PF_BN * 2;  // bytes per V^T row (64 keys), swizzled
    static constexpr int VBYTES = D * VROW;
    static constexpr int STAGE = KBYTES + VBYTES;
};

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

template <int D, class T>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const AttnParams p) {
    using SM = PfSmem<D>;
    extern __shared__ __align__(16) char smem[];
    constexpr int KSTEPS = D / 16;  // contraction steps of the first product
    constexpr int DT = D / 32;      // 32-row tiles of O^T
    constexpr int KCHUNKS = SM::KBYTES / 1024 / 4;  // 1 KiB direct-to-LDS loads per wave and tile
    constexpr int ROWS_PER_CHUNK = 1024 / SM::KROW;
    constexpr int PIECES = D / 8;
    constexpr int VSEG = D / 8;                 // 8-wide d segments per row
    constexpr int VITEMS = (PF_BN / 8) * VSEG;  // (8-key group, d segment) items per tile
    static_assert(VITEMS <= 256, "one V item per thread");

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n32 = lane & 31, h2 = lane >> 5;
    const int R = p.R, Tq = p.Tq, KV_CTX = p.KV_CTX;
    const int TOKB = PF_BM / R;
    const int qtile = (int)gridDim.x - 1 - (int)blockIdx.x;  // heaviest (latest) tiles first
    const int g = blockIdx.y, b = blockIdx.z;

    const SlotInfo si = slot_info(p, b);
    if (!si.active) return;

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
    const int64_t ooff = (int64_t)b * p.o_s[0] + (int64_t)(g * R + hh) * p.o_s[1] + (int64_t)ti * p.o_s[2];

    f16v acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;  // running max in log2 units (scaled), running sum (this lane's keys)

    if (hi_wg > lo_wg) {
        // Q as B operand: lane (row n32, half h2), step c: d = 16c + 8*h2 .. +8
        u4 qf[KSTEPS];
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c) {
            u4 z = {0, 0, 0, 0};
            qf[c] = row_ok ? load8_as<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt) : z;
        }

        const char* kbase = static_cast<const char*>(p.k) + ((int64_t)b * p.k_sb + (int64_t)g * KV_CTX * D) * 2;
        const char* vbase = static_cast<const char*>(p.v) + ((int64_t)b * p.v_sb + (int64_t)g * KV_CTX * D) * 2;
        auto key_off = [&](int j) -> uint32_t {
            j = min(max(j, 0), si.window - 1);
            int r = si.ring_start + j;
            r = (r >= KV_CTX) ? r - KV_CTX : r;
            return (uint32_t)r * (uint32_t)(D * 2);
        };

        // ---- staging roles ------------------------------------------------------------------------
        // K: wave `wave` issues KCHUNKS direct loads; chunk c covers LDS bytes [c*1024, +1024) of the K tile.
        const int k_row_in_chunk = lane / PIECES;  // 0 .. ROWS_PER_CHUNK-1
        const int k_piece_lds = lane % PIECES;
        // V: thread item = (8-key group q8, d segment)
        const int v_q8 = tid / VSEG, v_dseg = tid % VSEG;
        const bool v_item = (VITEMS == 256) || tid < VITEMS;
        u4 vst[8];

        // A tile is "plain" when its 64 keys lie inside the window and do not straddle the ring seam: then its rows
        // are consecutive in memory and every lane's source offset is a loop constant added to one scalar base.
        // Only the first / last tiles of a slot and the one on the seam take the general path with per-row clamping.
        uint32_t k_const[KCHUNKS], v_const[8];
#pragma unroll
        for (int i = 0; i < KCHUNKS; ++i) {
            const int row = (wave * KCHUNKS + i) * ROWS_PER_CHUNK + k_row_in_chunk;
            k_const[i] = (uint32_t)row * SM::KROW + (uint32_t)(k_piece_lds ^ (row & 15)) * 16u;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            v_const[j] = (uint32_t)((v_q8 >> 1) * 16 + (v_q8 & 1) * 4 + 8 * (j >> 2) + (j & 3)) * SM::KROW + (uint32_t)v_dseg * 16u;
        auto plain_row0 = [&](int kt) -> int {  // ring row of the tile's first key, or -1
            const int jb = kt * PF_BN;
            if (jb + PF_BN > si.window) return -1;
            int r0 = si.ring_start + jb;
            r0 = (r0 >= KV_CTX) ? r0 - KV_CTX : r0;
            return (r0 + PF_BN <= KV_CTX) ? r0 : -1;
        };
        auto issue_k = [&](int kt, int stage) {
            const int jb = kt * PF_BN;
            char* ks = smem + stage * SM::KBYTES;
            const int r0 = plain_row0(kt);
            if (r0 >= 0) {
                const char* tb = kbase + (int64_t)r0 * SM::KROW;
#pragma unroll
                for (int i = 0; i < KCHUNKS; ++i)
                    __builtin_amdgcn_global_load_lds((gptr_t)(tb + k_const[i]), (lptr_t)(ks + (wave * KCHUNKS + i) * 1024), 16, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < KCHUNKS; ++i) {
                    const int chunk = wave * KCHUNKS + i;
                    const int row = chunk * ROWS_PER_CHUNK + k_row_in_chunk;
                    const int piece = k_piece_lds ^ (row & 15);
                    const char* src = kbase + key_off(jb + row) + (uint32_t)piece * 16u;
                    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(ks + chunk * 1024), 16, 0, 0);
                }
            }
        };
        auto issue_v = [&](int kt) {
            const int jb = kt * PF_BN;
            const int r0 = plain_row0(kt);
            if (r0 >= 0) {
                const char* tb = vbase + (int64_t)r0 * SM::KROW;
                if (v_item) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) vst[j] = ld16(tb, v_const[j]);
                }
            } else {
                // 8-key group q8: 16-key group q8/2, half q8 & 1; slot j -> key 8*(j/4) + 4*half + j%4
                const int kb16 = jb + (v_q8 >> 1) * 16 + (v_q8 & 1) * 4;
                if (v_item) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        vst[j] = ld16(vbase, key_off(kb16 + 8 * (j >> 2) + (j & 3)) + (uint32_t)v_dseg * 16u);
                }
            }
        };
        auto store_v = [&](int stage) {
            char* vs = smem + 2 * SM::KBYTES + stage * SM::VBYTES;
            if (v_item) {
                u4 vt[8];
                transpose8x8_b16(vst, vt);
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    const int d = v_dseg * 8 + jj;
                    const int slot = v_q8 ^ ((jj ^ v_dseg) & 7);
                    *reinterpret_cast<u4*>(vs + d * SM::VROW + slot * 16) = vt[jj];
                }
            }
        };

        // ---- operand read offsets ------------------------------------------------------------------
        // LDS map: K stages at [0, 2*KBYTES), V^T stages at [2*KBYTES, 2*KBYTES + 2*VBYTES).
        // K^T step (mt, c): row mt*32 + n32, piece 2c + h2, swizzled with (row & 15) = (n32 & 15)
        uint32_t koff[8];
#pragma unroll
        for (int c8 = 0; c8 < 8; ++c8) koff[c8] = (uint32_t)n32 * SM::KROW + (uint32_t)(((2 * c8 + h2) ^ (n32 & 15)) * 16);
        // V^T step (dt, mt, u): row d = 32*dt + n32, column group (4*mt + 2*u + h2) ^ swz(d)
        uint32_t voff[2][4];
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const int d = par * 32 + n32;
            const int sw = (d ^ (d >> 3)) & 7;
#pragma unroll
            for (int cu = 0; cu < 4; ++cu) voff[par][cu] = 2 * SM::KBYTES + (uint32_t)n32 * SM::VROW + (uint32_t)(((2 * cu + h2) ^ sw) * 16);
        }
        constexpr int QK_STEPS = 2 * KSTEPS;  // MFMAs of S^T = K Q^T per tile; step idx -> (c = idx/2, key tile mt = idx%2)
        constexpr int PV_STEPS = 4 * DT;      // MFMAs of O^T += V^T P per tile; step idx -> (key group idx/DT, d tile idx%DT)
        const uint32_t lds0 = (uint32_t)(uintptr_t)smem;  // LDS byte address of the dynamic segment
        // Operand reads are issued as volatile asm, PF_PD steps ahead of the MFMA that consumes them, and
        // retired with explicit lgkmcnt waits: LDS returns data in order, so "at most n outstanding" is exact
        // for the oldest read whatever else the compiler has in flight.
        uint32_t kaddr[8], vaddr[2][4];
        // `left` = reads of the same sequence issued after the one being retired (a constant after unrolling)
        auto wait_left = [&](u4& a, int left) {
            static_assert(PF_PD == 4, "wait ladder below is written for 4 reads in flight");
            if (left >= 3) lds_wait<3>(a);
            else if (left == 2) lds_wait<2>(a);
            else if (left == 1) lds_wait<1>(a);
            else lds_wait<0>(a);
        };
        auto k_issue = [&](int idx) -> u4 {  // needs kaddr[] of the stage
            const int c = idx >> 1, mt = idx & 1;
            return lds_read16(kaddr[c & 7], mt * 32 * SM::KROW + (c >> 3) * 256);
        };
        auto v_issue = [&](int idx) -> u4 {
            const int cu = idx / DT, dt = idx % DT;
            return lds_read16(vaddr[dt & 1][cu], dt * 32 * SM::VROW);
        };

        const int kt0 = lo_wg / PF_BN, kt1 = (hi_wg - 1) / PF_BN;

        // ---- prologue: K(kt0), K(kt0+1), V(kt0) staged; S(kt0) computed --------------------------------
        issue_k(kt0, 0);
        issue_k(kt0 + 1, 1);
        issue_v(kt0);
        store_v(0);
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
            for (int idx = 0; idx < QK_STEPS; ++idx) {
                u4 a = abuf[idx % PF_PD];
                wait_left(a, QK_STEPS - 1 - idx);
                if (idx + PF_PD < QK_STEPS) abuf[idx % PF_PD] = k_issue(idx + PF_PD);
                s_cur[idx & 1] = T::mfma32(a, qf[idx >> 1], s_cur[idx & 1]);
            }
        }
        __syncthreads();  // every wave is done with K stage 0 before the loop refills it

        // One tile: softmax of S(kt) and O += V(kt) P, overlapped with S(kt+1) = K(kt+1) Q^T.
        // par = (kt - kt0) & 1: V(kt) sits in V stage par, K(kt+1) in K stage par^1; K(kt+2) is fetched into K
        // stage par and V(kt+1) into V stage par^1 while this tile computes.
        for (int kt = kt0; kt <= kt1; ++kt) {
            constexpr int N1 = 8;  // QK steps issued next to the row-max part of the softmax
            const int par = (kt - kt0) & 1;
            // the tiles after the last one are fetched (addresses are clamped to the window) and multiplied too;
            // nobody reads the results
            // Sources of K(kt+2) and V(kt+1): scalar base + per-lane offset (loop constants on plain tiles).  The
            // loads themselves are issued a few at a time between the MFMA steps below so that the address unit is
            // never handed more than one instruction per wave at once.
            const char* ksrc = kbase;
            const char* vsrc = vbase;
            uint32_t kofs[KCHUNKS], vofs[8];
            {
                const int rk = plain_row0(kt + 2), rv = plain_row0(kt + 1);
                if (rk >= 0) {
                    ksrc = kbase + (int64_t)rk * SM::KROW;
#pragma unroll
                    for (int i = 0; i < KCHUNKS; ++i) kofs[i] = k_const[i];
                } else {
#pragma unroll
                    for (int i = 0; i < KCHUNKS; ++i) {
                        const int row = (wave * KCHUNKS + i) * ROWS_PER_CHUNK + k_row_in_chunk;
                        kofs[i] = key_off((kt + 2) * PF_BN + row) + (uint32_t)(k_piece_lds ^ (row & 15)) * 16u;
                    }
                }
                if (rv >= 0) {
                    vsrc = vbase + (int64_t)rv * SM::KROW;
#pragma unroll
                    for (int j = 0; j < 8; ++j) vofs[j] = v_const[j];
                } else {
                    const int kb16 = (kt + 1) * PF_BN + (v_q8 >> 1) * 16 + (v_q8 & 1) * 4;
#pragma unroll
                    for (int j = 0; j < 8; ++j) vofs[j] = key_off(kb16 + 8 * (j >> 2) + (j & 3)) + (uint32_t)v_dseg * 16u;
                }
            }
            const uint32_t kdst = lds0 + par * SM::KBYTES + (uint32_t)__builtin_amdgcn_readfirstlane(wave) * (KCHUNKS * 1024);
            {
                const uint32_t kb = lds0 + (par ^ 1) * SM::KBYTES, vb = lds0 + par * SM::VBYTES;
#pragma unroll
                for (int c8 = 0; c8 < 8; ++c8) kaddr[c8] = kb + koff[c8];
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int cu = 0; cu < 4; ++cu) vaddr[q][cu] = vb + voff[q][cu];  // voff includes the 2*KBYTES base
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
            u4 abuf[PF_PD];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                s_nxt[0][j] = 0.f;
                s_nxt[1][j] = 0.f;
            }
#pragma unroll
            for (int i = 0; i < PF_PD; ++i) abuf[i] = k_issue(i);
            auto qk_step = [&](int idx) {
                u4 a = abuf[idx % PF_PD];
                wait_left(a, QK_STEPS - 1 - idx);
                if (idx + PF_PD < QK_STEPS) abuf[idx % PF_PD] = k_issue(idx + PF_PD);
                s_nxt[idx & 1] = T::mfma32(a, qf[idx >> 1], s_nxt[idx & 1]);
                // one of the eight V(kt+1) row loads every few steps of the second part
                constexpr int VSTRIDE = (QK_STEPS - N1) / 8;
                if (idx >= N1 && (idx - N1) % VSTRIDE == 0 && (idx - N1) / VSTRIDE < 8) {
                    if (v_item) vst[(idx - N1) / VSTRIDE] = gload16_async(vsrc, vofs[(idx - N1) / VSTRIDE]);
                }
            };
#pragma unroll
            for (int idx = 0; idx < N1; ++idx) qk_step(idx);

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
                    for (int j = 0; j < 8; ++j) {
                        e[j] = fast_exp2(__builtin_fmaf(s_cur[mt][8 * u + j], p.c, -m_safe));
                        psum += e[j];
                    }
                    pf[mt][u] = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
                    // six of the remaining K Q^T steps next to each quarter of the exponentials
#pragma unroll
                    for (int q = 0; q < (QK_STEPS - N1) / 4; ++q) qk_step(N1 + (mt * 2 + u) * ((QK_STEPS - N1) / 4) + q);
                }
            l_run += psum;

            // ---- O^T += V^T P : (key group) outer, d tile inner -> consecutive MFMAs are independent ----------
            {
                u4 vbuf[PF_PD];
#pragma unroll
                for (int i = 0; i < PF_PD; ++i) vbuf[i] = v_issue(i);
#pragma unroll
                for (int idx = 0; idx < PV_STEPS; ++idx) {
                    u4 a = vbuf[idx % PF_PD];
                    wait_left(a, PV_STEPS - 1 - idx);
                    if (idx + PF_PD < PV_STEPS) vbuf[idx % PF_PD] = v_issue(idx + PF_PD);
                    const int cu = idx / DT, dt = idx % DT;
                    acc[dt] = T::mfma32(a, pf[cu >> 1][cu & 1], acc[dt]);
                    // one of the K(kt+2) direct-to-LDS loads every other step of the first half
                    if (idx % 2 == 0 && idx / 2 < KCHUNKS) dma16_to_lds(ksrc, kofs[idx / 2], kdst + (idx / 2) * 1024);
                }
            }
            vm_wait8<KCHUNKS>(vst);  // the V loads were issued before the K loads
            store_v(par ^ 1);
            vm_wait_all();
            __syncthreads();
            s_cur[0] = s_nxt[0];
            s_cur[1] = s_nxt[1];
        }
    }

    // ---- epilogue: lane (row n32, half h2) holds d = 32*dt + 8*(i/4) + 4*h2 + i%4 -----------------
    float l_tot = l_run + __shfl_xor(l_run, 32);
    if (row_ok) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                f4 v = {acc[dt][4 * q4] * inv, acc[dt][4 * q4 + 1] * inv, acc[dt][4 * q4 + 2] * inv, acc[dt][4 * q4 + 3] * inv};
                store4(p.o, ooff + dt * 32 + 8 * q4 + 4 * h2, p.o_dt, v);
            }
    }
}

template <int D, class T>
static hipError_t launch_prefill_t(const AttnParams& p, hipStream_t stream) {
    const int TOKB = PF_BM / p.R;
    dim3 grid((p.Tq + TOKB - 1) / TOKB, p.G, p.B);
    const int smem = 2 * PfSmem<D>::STAGE;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_kernel<D, T>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL((attn_prefill_kernel<D, T>), grid, dim3(256), smem, stream, p);
    return hipGetLastError();
}

hipError_t launch_attn_prefill(const AttnParams& p, int D, int kv_dt, hipStream_t stream) {
    if (kv_dt == DT_F16) {
        if (D == 256) return launch_prefill_t<256, F16>(p, stream);
        if (D == 128) return launch_prefill_t<128, F16>(p, stream);
    } else {
        if (D == 256) return launch_prefill_t<256, BF16>(p, stream);
        if (D == 128) return launch_prefill_t<128, BF16>(p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace g4b
