// Prefill (and chunked-prefill) attention for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (slot, kv head) pair: all R = H/G query
// heads of the group for 128/R consecutive tokens, so a staged K/V tile serves the whole GQA
// group.  Each wave owns 32 rows.  The KV loop walks 64-key tiles from the first tile any row
// of the workgroup can see to the causal diagonal; tiles entirely inside every row's range run
// without masks, edge tiles (sliding-window lower edge, causal diagonal, window end) compare
// per element.  Tiles are double-buffered in LDS: K row-major with a 16-byte row pad, V
// transposed ([d][key]) with an XOR swizzle of the 16-byte column groups, both read back with
// conflict-free ds_read_b128 in MFMA operand layout.
//
// Math per tile and wave: S^T[64 keys x 32 rows] = K Q^T and O^T[D x 32 rows] += V^T P on
// v_mfma_f32_32x32x16 (fp16 or bf16 operands, fp32 accumulate).  Q stays in registers as the B
// operand; P never leaves registers: the accumulator layout of S^T is the B-operand layout of
// the second product once the key order inside each 16-key group of V^T is permuted to match.
// Softmax is online in fp32 with exp2 and scale*log2(e) folded into one multiplier; the row
// statistics live one row per lane pair (lane, lane^32).
#include "common.hpp"
#include "launch.hpp"

namespace g4b {

constexpr int PF_BM = 128;  // query rows per workgroup
constexpr int PF_BN = 64;   // keys per tile

template <int D>
struct PfSmem {
    static constexpr int KROW = D * 2 + 16;  // bytes per K row in LDS
    static constexpr int KBYTES = PF_BN * KROW;
    static constexpr int VROW = PF_BN * 2;  // bytes per V^T row (64 keys), swizzled, unpadded
    static constexpr int VBYTES = D * VROW;
    static constexpr int STAGE = KBYTES + VBYTES;
};

template <int D, class T>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const AttnParams p) {
    using SM = PfSmem<D>;
    extern __shared__ __align__(16) char smem[];
    constexpr int KSTEPS = D / 16;  // contraction steps of the first product
    constexpr int DT = D / 32;      // 32-row tiles of O^T
    constexpr int PIECES = D / 8;   // 16-byte pieces per cache row
    constexpr int KLD = PF_BN * PIECES / 256;  // 16-byte K loads per thread and tile
    constexpr int VSEG = D / 8;                // 8-wide d segments per row
    constexpr int VITEMS = (PF_BN / 8) * VSEG;     // (8-key group, d segment) items per tile
    constexpr int VLD = (VITEMS + 255) / 256;      // items per thread

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
    int lo_wg, hi_wg, lo_max, hi_min, dummy;
    row_range(p, si, tok0, lo_wg, hi_min);
    row_range(p, si, tok_last, lo_max, hi_wg);
    (void)dummy;

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
    float m_run = -INFINITY, l_run = 0.f;

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

        // staging roles
        const int k_piece = tid % PIECES, k_row0 = tid / PIECES;  // rows k_row0 + (256/PIECES)*i
        constexpr int KROWSTEP = 256 / PIECES;

        u4 kst[KLD];
        u4 vst[VLD][8];
        auto load_tile = [&](int kt) {
            const int jb = kt * PF_BN;
#pragma unroll
            for (int i = 0; i < KLD; ++i) kst[i] = ld16(kbase, key_off(jb + k_row0 + KROWSTEP * i) + (uint32_t)k_piece * 16u);
#pragma unroll
            for (int it = 0; it < VLD; ++it) {
                const int item = tid + 256 * it;
                const int q8 = item / VSEG, dseg = item % VSEG;
                // 8-key group q8 of the tile: 16-key group q8/2, half hsel = q8 & 1; slot j -> key 8*(j/4) + 4*hsel + j%4
                const int kb16 = jb + (q8 >> 1) * 16 + (q8 & 1) * 4;
                if (item < VITEMS) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        vst[it][j] = ld16(vbase, key_off(kb16 + 8 * (j >> 2) + (j & 3)) + (uint32_t)dseg * 16u);
                }
            }
        };
        auto store_tile = [&](int stage) {
            char* ks = smem + stage * SM::STAGE;
            char* vs = ks + SM::KBYTES;
#pragma unroll
            for (int i = 0; i < KLD; ++i)
                *reinterpret_cast<u4*>(ks + (k_row0 + KROWSTEP * i) * SM::KROW + k_piece * 16) = kst[i];
#pragma unroll
            for (int it = 0; it < VLD; ++it) {
                const int item = tid + 256 * it;
                const int q8 = item / VSEG, dseg = item % VSEG;
                if (item >= VITEMS) continue;
                u4 vt[8];
                transpose8x8_b16(vst[it], vt);
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    const int d = dseg * 8 + jj;
                    const int slot = q8 ^ ((d ^ (d >> 3)) & 7);
                    *reinterpret_cast<u4*>(vs + d * SM::VROW + slot * 16) = vt[jj];
                }
            }
        };

        const int kt0 = lo_wg / PF_BN, kt1 = (hi_wg - 1) / PF_BN;
        load_tile(kt0);
        store_tile(0);
        __syncthreads();

        for (int kt = kt0; kt <= kt1; ++kt) {
            const int stage = (kt - kt0) & 1;
            const char* ks = smem + stage * SM::STAGE;
            const char* vs = ks + SM::KBYTES;
            if (kt < kt1) load_tile(kt + 1);

            // ---- S^T = K Q^T : 2 key tiles of 32 -------------------------------------------
            f16v s[2];
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
                for (int j = 0; j < 16; ++j) s[mt][j] = 0.f;
                const char* krow = ks + (mt * 32 + n32) * SM::KROW + h2 * 16;
#pragma unroll
                for (int c = 0; c < KSTEPS; ++c) {
                    const u4 a = *reinterpret_cast<const u4*>(krow + c * 32);
                    s[mt] = T::mfma32(a, qf[c], s[mt]);
                }
            }

            // ---- online softmax ---------------------------------------------------------------
            const int jb = kt * PF_BN;
            const bool edge = (jb < lo_max) || (jb + PF_BN > hi_min);
            float mx = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float x = s[mt][i] * p.c;
                    if (edge) {
                        const int j = jb + mt * 32 + 8 * (i >> 2) + 4 * h2 + (i & 3);
                        if (j < lo_r || j >= hi_r) x = -INFINITY;
                    }
                    s[mt][i] = x;
                    mx = fmaxf(mx, x);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_safe);
            m_run = m_new;
            float psum = 0.f;
            u4 pf[2][2];  // [key tile][16-key group] -> 8 keys of this lane half
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    float e[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        e[j] = fast_exp2(s[mt][8 * u + j] - m_safe);
                        psum += e[j];
                    }
                    pf[mt][u] = u4{T::pack2(e[0], e[1]), T::pack2(e[2], e[3]), T::pack2(e[4], e[5]), T::pack2(e[6], e[7])};
                }
            l_run = l_run * alpha + psum;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int i = 0; i < DT; ++i) acc[i] *= alpha;
            }

            // ---- O^T += V^T P -------------------------------------------------------------------
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 32 + n32;
                const int sw = (d ^ (d >> 3)) & 7;
                const char* vrow = vs + d * SM::VROW;
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const int slot = (mt * 4 + u * 2 + h2) ^ sw;
                        const u4 a = *reinterpret_cast<const u4*>(vrow + slot * 16);
                        acc[dt] = T::mfma32(a, pf[mt][u], acc[dt]);
                    }
            }

            if (kt < kt1) store_tile(stage ^ 1);
            __syncthreads();
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
