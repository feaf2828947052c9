// Attention for the shapes and types the tuned kernels are not built for: any head dimension that is a multiple of 8
// (up to 1024), any number of query heads per kv head, an fp32 KV cache (the reference's G4B_DTKV_FP32 switch,
// g4b/models/gemma4e.py:32), and STAGE_ON_BAND on its own (g4b/kernels/fa2.py:15,399-435).  Same window / ring / phase
// semantics as the tuned kernels (g4b/kernels/fa2.py:52-96,332-335), evaluated per query row as one key range.
//
// All arithmetic is fp32 on the vector ALU (no operand is rounded, so USE_FP32_DOT holds trivially).  One workgroup of
// four waves serves up to four query heads of one kv head at one (slot, query position) -- they see the same keys, so
// K and V rows are loaded once for all of them; the waves take the 64-key chunks of the range in turn.  Within a
// chunk a lane owns one key for K Q^T (the query row sits in LDS, read as a broadcast) and eight output columns for
// P V (several keys per pass when the head dimension is below 512).  The four online-softmax states meet in LDS in a
// fixed order, so results do not depend on timing.  The path is correct and reasonably parallel, not tuned: Gemma-4's
// shapes never reach it.
#include "launch.hpp"

namespace g4b {

namespace {

constexpr int GEN_MAX_D = 1024;
constexpr int GEN_WAVES = 4;

G4B_DEV float wave_max64(float v) {
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) v = fmaxf(v, __shfl_xor(v, s));
    return v;
}
G4B_DEV float wave_sum64(float v) {
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) v += __shfl_xor(v, s);
    return v;
}

template <int NQ>
struct GenericSmem {
    float q[NQ][GEN_MAX_D];               // the query rows times scale * log2(e)
    float part[GEN_WAVES][GEN_MAX_D];     // per wave: [key sub-group][D] un-normalised sums of one head (sub-groups * D <= 1024)
    float m[NQ][GEN_WAVES], l[NQ][GEN_WAVES];
};

}  // namespace

// NQ query heads of one kv head at one query position per workgroup: they see the same keys, so every K and V row is
// loaded once for all of them.
template <int NQ>
__global__ __launch_bounds__(64 * GEN_WAVES) void attn_generic_kernel(const AttnParams p, const int D, const int kv_dt,
                                                                       const int band) {
    __shared__ GenericSmem<NQ> sm;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // blockIdx.x = ((b * G + g) * Tq + i) * (R / NQ) + head group: the heads of one kv head and one position are neighbours
    const int ngrp = p.R / NQ;
    int idx = blockIdx.x;
    const int r0 = (idx % ngrp) * NQ;
    idx /= ngrp;
    const int i = idx % p.Tq;
    idx /= p.Tq;
    const int g = idx % p.G;
    const int b = idx / p.G;
    const int h0 = g * p.R + r0;

    if (p.phase_arr[(int64_t)b * p.ph_s] != (uint8_t)p.phase) return;  // o stays as it is (fa2.py:332-335)
    int tds = max(p.tds[(int64_t)b * p.tds_s], 0);
    int W = p.win_arr ? p.win_arr[(int64_t)b * p.win_s] : p.W;
    W = min(max(W, 0), p.KV_CTX);
    const int window = min(tds, W);
    const int ring_start = (tds - window) % p.KV_CTX;
    const int qb = window - p.Tq;  // logical key aligned with query 0 (fa2.py:55)
    const int qp = qb + i;
    int lo = 0, hi = window;
    if (p.stage != STAGE_FULL) hi = min(window, qp + 1);
    if (p.stage == STAGE_ON_BAND) lo = max(0, qb + (i / band) * band);  // the diagonal block of the row's tile (fa2.py:56,61)
    if (p.qwin > 0) lo = max(lo, qp - p.qwin + 1);
    hi = max(hi, lo);

    const int nchunk = D >> 3;  // 8-column pieces of a row
    for (int t = tid; t < NQ * nchunk; t += 64 * GEN_WAVES) {
        const int n = t / nchunk, c = t % nchunk;
        float x[8];
        load_f32<8>(p.q, (int64_t)b * p.q_s[0] + (int64_t)(h0 + n) * p.q_s[1] + (int64_t)i * p.q_s[2] + c * 8, p.q_dt, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) sm.q[n][c * 8 + e] = x[e] * p.c;
    }
    __syncthreads();

    // P V ownership: kpp keys per pass, lane = (key sub-group sk, piece c); cpl pieces per lane when D > 512
    const int kpp = nchunk >= 64 ? 1 : 64 / nchunk;
    const int cpl = (nchunk + 63) >> 6;
    const int sk = nchunk >= 64 ? 0 : lane / nchunk;
    const int c0 = nchunk >= 64 ? lane : lane % nchunk;
    const bool pv_lane = sk < kpp;

    const char* kbase = static_cast<const char*>(p.k);
    const char* vbase = static_cast<const char*>(p.v);
    const int esz = kv_dt == DT_F32 ? 4 : 2;
    const int64_t k_slot = ((int64_t)b * p.k_sb + (int64_t)g * p.KV_CTX * D) * esz;
    const int64_t v_slot = ((int64_t)b * p.v_sb + (int64_t)g * p.KV_CTX * D) * esz;

    float m[NQ], l[NQ];
    float acc[NQ][2][8];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        m[n] = -INFINITY;
        l[n] = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[n][u][e] = 0.f;
    }

    for (int j0 = lo + wave * 64; j0 < hi; j0 += 64 * GEN_WAVES) {
        const int nk = min(64, hi - j0);
        // ---- scores: one key per lane
        const bool valid = lane < nk;
        int row = ring_start + j0 + (valid ? lane : 0);
        if (row >= p.KV_CTX) row -= p.KV_CTX;
        const void* krow = kbase + k_slot + (int64_t)row * D * esz;
        float s[NQ];
#pragma unroll
        for (int n = 0; n < NQ; ++n) s[n] = 0.f;
        for (int c = 0; c < nchunk; ++c) {
            float kx[8];
            load_f32<8>(krow, c * 8, kv_dt, kx);
#pragma unroll
            for (int n = 0; n < NQ; ++n) {
                const f4 qa = *reinterpret_cast<const f4*>(&sm.q[n][c * 8]);
                const f4 qc = *reinterpret_cast<const f4*>(&sm.q[n][c * 8 + 4]);
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s0 = fmaf(kx[e], qa[e], s0);
                    s1 = fmaf(kx[4 + e], qc[e], s1);
                }
                s[n] += s0 + s1;
            }
        }
        float pj[NQ];
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            const float sv = valid ? s[n] : -INFINITY;
            const float m_new = fmaxf(m[n], wave_max64(sv));  // finite: lane 0 is valid
            const float alpha = exp2f(m[n] - m_new);          // 0 on the first chunk
            pj[n] = exp2f(sv - m_new);                        // 0 for lanes past the range
            l[n] = l[n] * alpha + wave_sum64(pj[n]);
            m[n] = m_new;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[n][u][e] *= alpha;
        }
        // ---- P V: kpp keys per pass
        for (int jj = 0; jj < nk; jj += kpp) {
            const int kk = jj + sk;
            float pk[NQ];
#pragma unroll
            for (int n = 0; n < NQ; ++n) pk[n] = __shfl(pj[n], kk & 63);
            if (pv_lane && kk < nk) {
                int vr = ring_start + j0 + kk;
                if (vr >= p.KV_CTX) vr -= p.KV_CTX;
                const void* vrow = vbase + v_slot + (int64_t)vr * D * esz;
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int c = c0 + u * 64;
                    if (u < cpl && c < nchunk) {
                        float vx[8];
                        load_f32<8>(vrow, c * 8, kv_dt, vx);
#pragma unroll
                        for (int n = 0; n < NQ; ++n)
#pragma unroll
                            for (int e = 0; e < 8; ++e) acc[n][u][e] = fmaf(pk[n], vx[e], acc[n][u][e]);
                    }
                }
            }
        }
    }

    // ---- the four waves' states meet in LDS, one head after the other
    if (lane == 0) {
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            sm.m[n][wave] = m[n];
            sm.l[n][wave] = l[n];
        }
    }
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        if (n > 0) __syncthreads();  // the previous head's sums have been read
        if (pv_lane) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int c = c0 + u * 64;
                if (u < cpl && c < nchunk) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) sm.part[wave][sk * D + c * 8 + e] = acc[n][u][e];
                }
            }
        }
        __syncthreads();
        if (tid < nchunk) {
            float M = -INFINITY;
#pragma unroll
            for (int w = 0; w < GEN_WAVES; ++w) M = fmaxf(M, sm.m[n][w]);
            float L = 0.f, out[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = 0.f;
            for (int w = 0; w < GEN_WAVES; ++w) {
                const float mw = sm.m[n][w];
                if (mw == -INFINITY) continue;  // the wave saw no key
                const float f = exp2f(mw - M);
                L += f * sm.l[n][w];
                for (int s2 = 0; s2 < kpp; ++s2)
#pragma unroll
                    for (int e = 0; e < 8; ++e) out[e] = fmaf(f, sm.part[w][s2 * D + tid * 8 + e], out[e]);
            }
            // a row that sees no key is written as zeros, like the tuned kernels
            const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] *= inv;
            store8(p.o, (int64_t)b * p.o_s[0] + (int64_t)(h0 + n) * p.o_s[1] + (int64_t)i * p.o_s[2] + tid * 8, p.o_dt, out);
        }
    }
}

hipError_t launch_attn_generic(const AttnParams& p, int D, int kv_dt, int on_band_block, hipStream_t stream) {
    if (D < 8 || D % 8 || D > GEN_MAX_D) return hipErrorInvalidValue;
    // query heads per workgroup: as many as share the K/V loads, unless that leaves the chip short of workgroups
    // (decode-shaped launches: 64 slots x 8 heads measured 0.30 ms one head per workgroup, 0.34 ms four)
    int nq = p.R % 4 == 0 ? 4 : (p.R % 2 == 0 ? 2 : 1);
    while (nq > 1 && (int64_t)p.B * (p.H / nq) * p.Tq < 1024) nq /= 2;
    const int64_t blocks = (int64_t)p.B * (p.H / nq) * p.Tq;
    if (blocks < 1 || blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    if (!(p.kernel_mask & 1)) return hipSuccess;
    const dim3 grid((unsigned)blocks), block(64 * GEN_WAVES);
    const int band = on_band_block > 0 ? on_band_block : 1;
    if (nq == 4) G4B_LAUNCH_DOMINANT(attn_generic_kernel<4>, grid, block, 0, stream, p, D, kv_dt, band);
    else if (nq == 2) G4B_LAUNCH_DOMINANT(attn_generic_kernel<2>, grid, block, 0, stream, p, D, kv_dt, band);
    else G4B_LAUNCH_DOMINANT(attn_generic_kernel<1>, grid, block, 0, stream, p, D, kv_dt, band);
    return hipGetLastError();
}

}  // namespace g4b
