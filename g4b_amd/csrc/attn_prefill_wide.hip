// Prefill (and chunked-prefill) attention for head dimension 512 on gfx950.
//
// A 32-row wave of the 128/256 kernel would need 128 registers of Q and 256 of output accumulators, so here the head
// dimension is split over a pair of waves.  One workgroup (4 waves) owns 64 query rows of one (slot, kv head) pair:
// wave w works on row block w / 2 (32 rows) and on columns [256 * (w % 2), +256) of the head dimension, its share of
// Q, of every K and V row and of the output.  Per 32-key tile a wave computes the partial product S^T = K Q^T over
// its 256 columns, the two waves of a pair add their partials through LDS and then run the same online softmax on the
// same numbers, and each accumulates O^T += V^T P for its own 256 output columns.
//
// Staging, operand layouts and masks are those of the 128/256 kernel: K and V tiles double-buffered in LDS by direct
// global -> LDS loads (rows row-major and unpadded, 16-byte pieces XOR-swizzled through the choice of the source
// piece), K read with ds_read_b128 as the A operand, V read with ds_read_b64_tr_b16, v_mfma_f32_32x32x16, P kept in
// registers, exp2 softmax in fp32 with lazy rescaling.  The next tile's loads are issued one per MFMA step of the
// first product and waited for at the barrier that closes the tile.
#include "common.hpp"
#include "launch.hpp"
#include "prefill_combine.hpp"
#include "prefill_map.hpp"

namespace g4b {

constexpr int PW_D = 512;                    // head dimension
constexpr int PW_DL = 256;                   // columns per wave
constexpr int PW_BN = 32;                    // keys per tile
constexpr int PW_BM = 64;                    // query rows per workgroup
constexpr int PW_ROW = PW_D * 2;             // bytes per K or V row
constexpr int PW_TILE = PW_BN * PW_ROW;      // bytes per staged tile
constexpr int PW_XCH = 4 * 16 * 64 * 4;      // partial scores of the four waves
constexpr int PW_SMEM = 4 * PW_TILE + PW_XCH;
constexpr int PW_PD = 6;                     // LDS operand fetches in flight

template <class T>
__global__ __launch_bounds__(256) void attn_prefill_wide_kernel(const AttnParams p) {
    extern __shared__ __align__(16) char smem[];
    constexpr int D = PW_D, DL = PW_DL, ROW = PW_ROW, TILE = PW_TILE;
    constexpr int KSTEPS = DL / 16;         // contraction steps of the first product (per wave)
    constexpr int DT = DL / 32;             // 32-row tiles of this wave's part of O^T
    constexpr int CHUNKS = TILE / 1024 / 4;  // 1 KiB direct-to-LDS loads per wave and tile: one K or V row each
    constexpr int PV_STEPS = 2 * DT;        // (16-key group, d tile)
    static_assert(CHUNKS == 8 && KSTEPS == 2 * CHUNKS, "one direct load per step of the first product");

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int rb = wave >> 1, hv = wave & 1;
    const int n32 = lane & 31, h2 = lane >> 5;
    const int R = p.R, Tq = p.Tq, KV_CTX = p.KV_CTX;
    const int TOKB = PW_BM / R;
    __shared__ int sh_scan[8];
    int n_active;
    nth_active_slot(p, -1, n_active, sh_scan);
    if (n_active == 0) return;
    const int nsplit = prefill_splits(p.part_o ? p.split_slots : 1, n_active);
    const PfMap map = pf_map(n_active * p.G * nsplit, (Tq + TOKB - 1) / TOKB);
    if ((int)blockIdx.x >= map.grid) return;
    int head, rank;
    pf_item(map, blockIdx.x, head, rank);
    if (rank >= map.nq) return;
    const int qtile = map.nq - 1 - rank;
    const int split = head % nsplit, g = (head / nsplit) % p.G, a_idx = head / (nsplit * p.G);
    const int b = nth_active_slot(p, a_idx, n_active, sh_scan);  // workgroup-uniform

    const SlotInfo si = slot_info(p, b);
    const int tok0 = qtile * TOKB;
    const int tok_last = min(tok0 + TOKB, Tq) - 1;
    int lo_wg, hi_wg, lo_max, hi_min;
    row_range(p, si, tok0, lo_wg, hi_min);
    row_range(p, si, tok_last, lo_max, hi_wg);

    // this lane's row
    const int rrow = rb * 32 + n32;
    const int hh = rrow / TOKB;
    const int ti = tok0 + rrow % TOKB;
    const bool row_ok = ti < Tq;
    int lo_r = 0, hi_r = 0;
    if (row_ok) row_range(p, si, ti, lo_r, hi_r);
    const int64_t qoff = (int64_t)b * p.q_s[0] + (int64_t)(g * R + hh) * p.q_s[1] + (int64_t)ti * p.q_s[2] + hv * DL;

    f16v acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    if (hi_wg > lo_wg) {
        const char* kbase = static_cast<const char*>(p.k) + ((int64_t)b * p.k_sb + (int64_t)g * KV_CTX * D) * 2;
        const char* vbase = static_cast<const char*>(p.v) + ((int64_t)b * p.v_sb + (int64_t)g * KV_CTX * D) * 2;
        auto key_off = [&](int j) -> uint32_t {  // byte offset of logical key j (clamped to the window) in the ring
            j = min(max(j, 0), si.window - 1);
            int r = si.ring_start + j;
            r = (r >= KV_CTX) ? r - KV_CTX : r;
            return (uint32_t)r * (uint32_t)ROW;
        };

        // ---- staging: K stages at [0, 2*TILE), V stages at [2*TILE, 4*TILE); wave w moves rows 8w .. 8w+7 of a tile,
        // lane l the 16-byte piece that lands at position l of the LDS row
        const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
        auto st_row = [&](int i) { return wave * CHUNKS + i; };
        auto k_piece = [&](int row) { return lane ^ (row & 15); };
        auto v_piece = [&](int row) { return lane ^ (4 * (row & 7)); };
        uint32_t k_const[CHUNKS], v_const[CHUNKS];
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const int row = st_row(i);
            // chunk i is issued with instruction offset (i % 4) KiB, which moves source and destination alike
            k_const[i] = (uint32_t)row * ROW + (uint32_t)k_piece(row) * 16u - (uint32_t)(i & 3) * 1024u;
            v_const[i] = (uint32_t)row * ROW + (uint32_t)v_piece(row) * 16u - (uint32_t)(i & 3) * 1024u;
        }
        auto plain_row0 = [&](int kt) -> int {  // ring row of the tile's first key when its rows are consecutive, or -1
            const int jb = kt * PW_BN;
            if (jb + PW_BN > si.window) return -1;
            int r0 = si.ring_start + jb;
            r0 = (r0 >= KV_CTX) ? r0 - KV_CTX : r0;
            return (r0 + PW_BN <= KV_CTX) ? r0 : -1;
        };
        auto tile_src = [&](int kt, bool is_v, const char*& src, uint32_t(&ofs)[CHUNKS]) {
            const int r0 = plain_row0(kt);
            const char* base = is_v ? vbase : kbase;
            if (r0 >= 0) {
                src = base + (int64_t)r0 * ROW;
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) ofs[i] = is_v ? v_const[i] : k_const[i];
            } else {
                src = base - 3072;  // keeps the lane offsets non-negative under the instruction offsets
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) {
                    const int row = st_row(i);
                    ofs[i] = key_off(kt * PW_BN + row) + (uint32_t)(is_v ? v_piece(row) : k_piece(row)) * 16u + 3072u -
                             (uint32_t)(i & 3) * 1024u;
                }
            }
        };
        const uint32_t wave_chunk0 = (uint32_t)__builtin_amdgcn_readfirstlane(wave) * (CHUNKS * 1024);
        auto dma_chunk = [&](int i, const char* src, const uint32_t(&ofs)[CHUNKS], uint32_t dst) {
            if ((i & 3) == 0) dma_set_base(dst + i * 1024);
            if ((i & 3) == 0) dma16_to_lds_at<0>(src, ofs[i]);
            if ((i & 3) == 1) dma16_to_lds_at<1024>(src, ofs[i]);
            if ((i & 3) == 2) dma16_to_lds_at<2048>(src, ofs[i]);
            if ((i & 3) == 3) dma16_to_lds_at<3072>(src, ofs[i]);
        };

        // ---- operand read offsets --------------------------------------------------------------------------
        // K^T step c: key row n32, piece 32*hv + 2c + h2 swizzled with (row & 15); c / 8 becomes an instruction offset
        uint32_t koff[8];
#pragma unroll
        for (int c8 = 0; c8 < 8; ++c8)
            koff[c8] = (uint32_t)n32 * ROW + (uint32_t)hv * (DL * 2) + (uint32_t)(((2 * c8 + h2) ^ (n32 & 15)) * 16);
        // V^T fragment of step (cu, dt): d = 256*hv + 32*dt + n32, keys {16cu + 4h2 + 0..3, 16cu + 8 + 4h2 + 0..3}
        const int tr_r = (lane & 15) >> 2, tr_q = lane & 3, tr_dhalf = (lane >> 4) & 1;
        const int tr_key = 4 * h2 + tr_r;
        uint32_t voff[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int piece = hv * (DL / 8) + dt * 4 + tr_dhalf * 2 + (tr_q >> 1);
            voff[dt] = 2 * TILE + (uint32_t)tr_key * ROW + (uint32_t)((piece ^ (4 * (tr_key & 7))) * 16) + (uint32_t)(tr_q & 1) * 8u;
        }
        uint32_t kaddr[8], vaddr[DT];
        auto k_issue = [&](int c) -> u4 { return lds_read16(kaddr[c & 7], (c >> 3) * 256); };
        struct VFrag {
            u2 lo, hi;
        };
        auto v_issue = [&](int idx) -> VFrag {
            const int cu = idx / DT, dt = idx % DT;
            VFrag f;
            f.lo = lds_read8_tr16(vaddr[dt], cu * 16 * ROW);
            f.hi = lds_read8_tr16(vaddr[dt], (cu * 16 + 8) * ROW);
            return f;
        };
        auto wait_pair = [&](u4& a0, u4& a1, int left) {
            if (left >= 2) lds_wait_pair<4>(a0, a1);
            else if (left == 1) lds_wait_pair<2>(a0, a1);
            else lds_wait_pair<0>(a0, a1);
        };
        auto wait_pair2 = [&](VFrag& f0, VFrag& f1, int left) {
            if (left >= 2) lds_wait4<8>(f0.lo, f0.hi, f1.lo, f1.hi);
            else if (left == 1) lds_wait4<4>(f0.lo, f0.hi, f1.lo, f1.hi);
            else lds_wait4<0>(f0.lo, f0.hi, f1.lo, f1.hi);
        };
        float* xch = reinterpret_cast<float*>(smem + 4 * TILE);

        int kt0 = lo_wg / PW_BN, kt1 = (hi_wg - 1) / PW_BN;
        if (nsplit > 1) {
            const int n = kt1 - kt0 + 1;
            kt1 = kt0 + (split + 1) * n / nsplit - 1;
            kt0 = kt0 + split * n / nsplit;
        }
        if (kt1 >= kt0) {
            // ---- prologue: K(kt0) and V(kt0) staged, this wave's half of Q in registers
            {
                const char* src;
                uint32_t ofs[CHUNKS];
                tile_src(kt0, false, src, ofs);
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) dma_chunk(i, src, ofs, lds0 + wave_chunk0);
                tile_src(kt0, true, src, ofs);
#pragma unroll
                for (int i = 0; i < CHUNKS; ++i) dma_chunk(i, src, ofs, lds0 + 2 * TILE + wave_chunk0);
            }
            u4 qf[KSTEPS];  // B operand: lane (row n32, half h2), step c: d = 256*hv + 16c + 8*h2 .. +8
#pragma unroll
            for (int c = 0; c < KSTEPS; ++c) {
                u4 z = {0, 0, 0, 0};
                qf[c] = row_ok ? load8_as<T>(p.q, qoff + c * 16 + h2 * 8, p.q_dt) : z;
            }
            vm_wait_all();
            __syncthreads();

            for (int kt = kt0; kt <= kt1; ++kt) {
                const int par = (kt - kt0) & 1;
                // K(kt+1) and V(kt+1) go into the other stage pair, which every wave left at the last barrier.  Tiles
                // past the last one are fetched as well (addresses are clamped to the window); nobody reads them.
                const char *ksrc, *vsrc;
                uint32_t kofs[CHUNKS], vofs[CHUNKS];
                tile_src(kt + 1, false, ksrc, kofs);
                tile_src(kt + 1, true, vsrc, vofs);
                const uint32_t kdst = lds0 + (par ^ 1) * TILE + wave_chunk0;
                const uint32_t vdst = lds0 + 2 * TILE + (par ^ 1) * TILE + wave_chunk0;
                {
                    const uint32_t sb = lds0 + par * TILE;
#pragma unroll
                    for (int c8 = 0; c8 < 8; ++c8) kaddr[c8] = sb + koff[c8];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) vaddr[dt] = sb + voff[dt];  // voff includes the 2*TILE base
                }

                // ---- partial S^T = K Q^T over this wave's columns; two chains so consecutive MFMAs are independent
                f16v s0, s1;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    s0[j] = 0.f;
                    s1[j] = 0.f;
                }
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
                        s0 = T::mfma32(a0, qf[idx], s0);
                        s1 = T::mfma32(a1, qf[idx + 1], s1);
                        if (idx < CHUNKS) {
                            dma_chunk(idx, ksrc, kofs, kdst);
                            dma_chunk(idx + 1, ksrc, kofs, kdst);
                        } else {
                            dma_chunk(idx - CHUNKS, vsrc, vofs, vdst);
                            dma_chunk(idx + 1 - CHUNKS, vsrc, vofs, vdst);
                        }
                    }
                }
                // ---- the pair adds its partials: same operands, same order, so both waves hold the same scores
                float sc[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    sc[j] = s0[j] + s1[j];
                    xch[(wave * 16 + j) * 64 + lane] = sc[j];
                }
                __syncthreads();
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float mine = sc[j], other = xch[((wave ^ 1) * 16 + j) * 64 + lane];
                    sc[j] = mine + other;  // commutative: bit-identical in both waves
                }

                // ---- edge tiles: mask
                const int jb = kt * PW_BN;
                if ((jb < lo_max) || (jb + PW_BN > hi_min)) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int j = jb + 8 * (i >> 2) + 4 * h2 + (i & 3);
                        if (j < lo_r || j >= hi_r) sc[i] = -INFINITY;
                    }
                }

                // ---- online softmax with lazy rescaling (exponent reference moves only when the maximum outgrows it
                // by more than 2^PF_TAU)
                float mx = sc[0];
#pragma unroll
                for (int i = 1; i < 16; ++i) mx = fmaxf(mx, sc[i]);
                mx = half_swap_max(mx) * p.c;
                const bool grow = mx > m_run + PF_TAU;
                if (__any(grow)) {
                    const float m_new = grow ? mx : m_run;
                    const float alpha = grow ? fast_exp2(m_run - mx) : 1.f;
                    const bool touch = grow && (m_run != -INFINITY);
                    m_run = m_new;
                    l_run *= alpha;
                    if (__any(touch)) {
#pragma unroll
                        for (int i = 0; i < DT; ++i)
#pragma unroll
                            for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
                    }
                }
                const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
                float psum = 0.f;
                u4 pf[2];  // [16-key group] -> 8 keys of this lane half
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    float e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = fast_exp2(__builtin_fmaf(sc[8 * u + j], p.c, -m_safe));
                    pf[u] = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t w = pf[u][j];
                        psum = T::sum2(w, psum);  // the row sum adds up the rounded values the second product uses
                    }
                }
                l_run += psum;

                // ---- O^T += V^T P for this wave's columns
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
                vm_wait_all();
                __syncthreads();
            }
        }
    }

    // ---- epilogue: the wave turns its 32 x 256 block around in LDS (32 KiB of the staging area per wave, free after
    // the loop's last barrier) and stores whole 1 KiB row halves
    const float l_tot = half_swap_sum(l_run);
    const bool partial = nsplit > 1;
    const float inv = partial ? 1.f : (l_tot > 0.f ? 1.f / l_tot : 0.f);
    char* wbase = smem + wave * (32 * DL * 4);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            f4 v = {acc[dt][4 * q4] * inv, acc[dt][4 * q4 + 1] * inv, acc[dt][4 * q4 + 2] * inv, acc[dt][4 * q4 + 3] * inv};
            const int pc = 8 * dt + 2 * q4 + h2;
            *reinterpret_cast<f4*>(wbase + n32 * (DL * 4) + ((pc ^ (n32 & 15)) * 16)) = v;
        }
    if (partial && h2 == 0 && hv == 0 && row_ok) {
        const int64_t prow = ((int64_t)(a_idx * nsplit + split) * p.H + (g * R + hh)) * Tq + ti;
        p.part_ml[prow * 2] = (m_run == -INFINITY) ? 0.f : m_run;
        p.part_ml[prow * 2 + 1] = l_tot;
    }
    const int tokb_shift = __ffs(TOKB) - 1;  // TOKB = 64 / R is a power of two
#pragma unroll 4
    for (int row = 0; row < 32; ++row) {
        const int pc = lane;  // 64 lanes x 16 bytes = the wave's 256 fp32 columns of one row
        const int rr = rb * 32 + row;
        const int hr = rr >> tokb_shift, tr = tok0 + (rr & (TOKB - 1));
        const f4 v = *reinterpret_cast<const f4*>(wbase + row * (DL * 4) + ((pc ^ (row & 15)) * 16));
        if (tr < Tq) {
            if (partial) {
                const int64_t prow = ((int64_t)(a_idx * nsplit + split) * p.H + (g * R + hr)) * Tq + tr;
                *reinterpret_cast<f4*>(p.part_o + prow * D + hv * DL + pc * 4) = v;
            } else {
                const int64_t off = (int64_t)b * p.o_s[0] + (int64_t)(g * R + hr) * p.o_s[1] + (int64_t)tr * p.o_s[2];
                store4(p.o, off + hv * DL + pc * 4, p.o_dt, v);
            }
        }
    }
}

template <class T>
static hipError_t launch_prefill_wide_t(const AttnParams& p, hipStream_t stream) {
    const int slots = p.part_o ? p.split_slots : 1;
    const int blocks = prefill_grid(p, PW_BM);
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_wide_kernel<T>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, PW_SMEM);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    if (p.kernel_mask & 1) hipLaunchKernelGGL((attn_prefill_wide_kernel<T>), dim3(blocks), dim3(256), PW_SMEM, stream, p);
    if (slots > 1 && (p.kernel_mask & 2)) {
        const int items = min(p.B, slots / 2);  // more active slots than this are never split
        hipLaunchKernelGGL((attn_prefill_combine<PW_D>), dim3(items * p.H * ((p.Tq + PFC_ROWS - 1) / PFC_ROWS)), dim3(256), 0,
                           stream, p);
    }
    return hipGetLastError();
}

hipError_t launch_attn_prefill_wide(const AttnParams& p, int kv_dt, hipStream_t stream) {
    return kv_dt == DT_F16 ? launch_prefill_wide_t<F16>(p, stream) : launch_prefill_wide_t<BF16>(p, stream);
}

}  // namespace g4b
