// q/k RMSNorm + rotary embedding for gfx950, optionally fused with the ring append of the rotated K and of V.
//
// An element-wise, HBM-bound pass: a thread owns 16 bytes' worth of consecutive columns j.. of the first half of a head
// (eight for 16-bit scratchpads, four for fp32 ones) and their partners j + D/2..; it evaluates sin/cos of its angles once (full-precision sincosf: positions reach
// tens of thousands of radians) and then walks over the query heads and the kv heads of its (slot, token), so the
// angles are shared by every head as in the reference.  A wave's loads and stores are contiguous runs per half row;
// a workgroup covers 256 / (threads per token) tokens of one slot.  With the append fused, rotated K goes straight into the ring
// in the cache's dtype (one rounding) and V is copied / normalised by the same threads: the K and V scratch rows are
// read once and nothing is read back.
#include "common.hpp"
#include "launch.hpp"

namespace g4b {

// One head row, in two steps so that the loads of several rows can be in flight before any of them is stored
// (the rows are rewritten in place, so the compiler may not move a load above an earlier store by itself).
template <int N>
struct RopeRow {
    float x1[N], x2[N];
};
template <int N>
G4B_DEV void rope_row_load(RopeRow<N>& r, const void* x, int64_t xo, int x_dt, int half) {
    // ordinary (cached) accesses on purpose: the scratchpads come from the projection kernels just before and q goes
    // to the attention kernel just after; non-temporal ones measured 0.63 -> 0.55 of the HBM peak at 8192 tokens (the
    // 184 MB working set sits in the last-level cache) and only pay beyond it (0.68 -> 0.79 at 131072 tokens)
    load_f32<N>(x, xo, x_dt, r.x1);
    load_f32<N>(x, xo + half, x_dt, r.x2);
}
template <int N>
G4B_DEV void rope_row_finish(const RopeRow<N>& r, void* x, int64_t xo, int x_dt, float inv_rms, const float (&w1)[N],
                             const float (&w2)[N], const float (&sn)[N], const float (&cs)[N], int half, bool writeback,
                             void* cache, int64_t co, int cache_dt) {
    float y1[N], y2[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        // rope.py:33-37: x *= inv_rms * w, then the rotation, all in fp32
        const float a = r.x1[i] * (inv_rms * w1[i]);
        const float b = r.x2[i] * (inv_rms * w2[i]);
        y1[i] = cs[i] * a - sn[i] * b;
        y2[i] = cs[i] * b + sn[i] * a;
    }
    if (writeback) {
        store_n<N>(x, xo, x_dt, y1);
        store_n<N>(x, xo + half, x_dt, y2);
    }
    if (cache) {
        store_n<N>(cache, co, cache_dt, y1);
        store_n<N>(cache, co + half, cache_dt, y2);
    }
}

// CPT = columns of each half of a head row per thread: 8 when every scratchpad is 16-bit, 4 when any is fp32 (the
// engine's), so that a thread's access is 16 bytes either way and a wave's one contiguous run per half row.
template <int CPT>
__global__ __launch_bounds__(256) void rope_kernel(const RopeParams p) {
    const int b = blockIdx.y;
    const int half = p.D / 2;
    const int tpr = half / CPT;          // threads per token
    const int rows = 256 / tpr;          // tokens per workgroup
    // Workgroups go to the 8 XCDs round-robin by id, and the odd XCDs stream from HBM more slowly than the even ones
    // (attn_decode.hpp): a launch of many token blocks deals 26 of every 50 to the even workgroups, so that both
    // halves of the chip finish together; the odd workgroups left over leave at once.
    int block = blockIdx.x;
    if (p.even_blocks > 0) {
        const int k = block >> 1;
        if (block & 1) {
            block = p.even_blocks + k;
        } else {
            if (k >= p.even_blocks) return;
            block = k;
        }
    }
    const int tt = block * rows + threadIdx.x / tpr;
    const int j0 = (threadIdx.x % tpr) * CPT;
    // threads beyond rows * tpr (tpr does not divide 256) would alias the next workgroup's first token
    if ((int)threadIdx.x >= rows * tpr || tt >= p.t) return;

    const int32_t off = p.offsets[(int64_t)b * p.off_s];
    const float pos = (float)(off + tt);  // rope.py:180: integer position, converted once
    float sn[CPT], cs[CPT], qw1[CPT], qw2[CPT], kw1[CPT], kw2[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        // rope.py:183-186: the angle is the fp32 product; its sine and cosine are wanted to fp32 accuracy although the
        // angle reaches tens of thousands of radians.  The reduction to half turns is done in fp64 (three instructions)
        // instead of the general-purpose large-argument path of sincosf.
        const float theta = pos * p.freqs[(int64_t)(j0 + i) * p.freqs_s];
        double half_turns = (double)theta * 0.31830988618379067154;  // theta / pi
        half_turns -= 2.0 * __builtin_rint(half_turns * 0.5);          // now in [-1, 1]
        sincospif((float)half_turns, &sn[i], &cs[i]);
        qw1[i] = p.q_w[(int64_t)(j0 + i) * p.q_w_s];
        qw2[i] = p.q_w[(int64_t)(j0 + i + half) * p.q_w_s];
        kw1[i] = p.k_w[(int64_t)(j0 + i) * p.k_w_s];
        kw2[i] = p.k_w[(int64_t)(j0 + i + half) * p.k_w_s];
    }

    const bool append = p.k_cache && (!p.phase_arr || p.phase_arr[(int64_t)b * p.ph_s] == (uint8_t)p.phase);
    int64_t ring_row = 0;
    if (append) {
        ring_row = ((int64_t)tt + off) % p.T;
        if (ring_row < 0) ring_row += p.T;
    }
    const bool k_back = !p.k_cache || p.k_writeback;
    const bool with_v = append && p.v;

    // Row jobs of this (slot, token): H query heads, G key heads, G value heads.  They are dealt round-robin to the
    // gridDim.z workgroups that share the (slot, token block), which keeps more independent loads in flight than one
    // thread walking all of them; the angles are recomputed by each, which costs nothing next to the memory traffic.
    const int jobs = p.H + p.G + (with_v ? p.G : 0);
    for (int job = blockIdx.z; job < jobs; job += gridDim.z) {
        if (job < p.H) {
            // up to eight query heads at a time (this workgroup's heads are job, job + z, ...)
            constexpr int NB = 8;
            RopeRow<CPT> qrows[NB];
            float rs[NB];
            const int step = gridDim.z;
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int h = job + u * step;
                if (h < p.H) {
                    rs[u] = p.q_rsos[(int64_t)b * p.q_rsos_s[0] + (int64_t)h * p.q_rsos_s[1] + (int64_t)tt * p.q_rsos_s[2]];
                    rope_row_load<CPT>(qrows[u], p.q, (int64_t)b * p.q_s[0] + (int64_t)h * p.q_s[1] + (int64_t)tt * p.q_s[2] + j0, p.q_dt, half);
                }
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int h = job + u * step;
                if (h < p.H) {
                    const float inv = 1.0f / __builtin_sqrtf(rs[u] / (float)p.D + p.eps);
                    rope_row_finish<CPT>(qrows[u], p.q, (int64_t)b * p.q_s[0] + (int64_t)h * p.q_s[1] + (int64_t)tt * p.q_s[2] + j0, p.q_dt,
                                         inv, qw1, qw2, sn, cs, half, true, nullptr, 0, 0);
                }
            }
            // skip the heads handled above; the loop increment adds one more step
            int last = job;
            for (int u = 1; u < NB; ++u)
                if (job + u * step < p.H) last = job + u * step;
            job = last;
        } else if (job < p.H + p.G) {
            const int g = job - p.H;
            const float r = p.k_rsos[(int64_t)b * p.k_rsos_s[0] + (int64_t)g * p.k_rsos_s[1] + (int64_t)tt * p.k_rsos_s[2]];
            const float inv = 1.0f / __builtin_sqrtf(r / (float)p.D + p.eps);
            const int64_t xo = (int64_t)b * p.k_s[0] + (int64_t)g * p.k_s[1] + (int64_t)tt * p.k_s[2] + j0;
            const int64_t co = (int64_t)b * p.k_cache_sb + ((int64_t)g * p.T + ring_row) * p.D + j0;
            RopeRow<CPT> row;
            rope_row_load<CPT>(row, p.k, xo, p.k_dt, half);
            rope_row_finish<CPT>(row, p.k, xo, p.k_dt, inv, kw1, kw2, sn, cs, half, k_back, append ? p.k_cache : nullptr, co, p.cache_dt);
        } else {
            // V: the token's threads cover the row in runs of D/2 columns (Dv may differ from D)
            const int g = job - p.H - p.G;
            float inv = 1.f;
            if (p.v_rsos) {
                const float r = p.v_rsos[(int64_t)b * p.v_rsos_s[0] + (int64_t)g * p.v_rsos_s[1] + (int64_t)tt * p.v_rsos_s[2]];
                inv = 1.0f / __builtin_sqrtf(r / (float)p.Dv + p.eps);
            }
            for (int col = j0; col < p.Dv; col += half) {
                float vx[CPT];
                load_f32<CPT>(p.v, (int64_t)b * p.v_s[0] + (int64_t)g * p.v_s[1] + (int64_t)tt * p.v_s[2] + col, p.v_dt, vx);
#pragma unroll
                for (int i = 0; i < CPT; ++i) vx[i] *= inv;
                store_n<CPT>(p.v_cache, (int64_t)b * p.v_cache_sb + ((int64_t)g * p.T + ring_row) * p.Dv + col, p.cache_dt, vx);
            }
        }
    }
}

hipError_t launch_rope(const RopeParams& p, hipStream_t stream) {
    const bool any_f32 = p.q_dt == DT_F32 || p.k_dt == DT_F32 || (p.v && p.v_dt == DT_F32);
    const int cpt = (any_f32 && p.D <= 2048) ? 4 : 8;  // a token has at most 256 threads
    const int rows = 256 / (p.D / (2 * cpt));
    const int blocks = (p.t + rows - 1) / rows;
    // launches of a few tokens (decode): split the row jobs of a token up to four ways to get the chip busy at all;
    // otherwise a thread walks all heads of its token, which are neighbours in the engine's [B, t, heads, D] layout
    const int jobs = p.H + 2 * p.G;
    int z = 1;
    while (z < 4 && z * 2 <= jobs && (int64_t)blocks * p.B * z < 256) z *= 2;
    RopeParams pk = p;
    pk.even_blocks = (p.xcd_weighted && blocks >= 128) ? (blocks * 26 + 49) / 50 : 0;
    dim3 grid(pk.even_blocks ? 2 * pk.even_blocks : blocks, p.B, z);
    if (cpt == 4) G4B_LAUNCH_DOMINANT(rope_kernel<4>, grid, dim3(256), 0, stream, pk);
    else G4B_LAUNCH_DOMINANT(rope_kernel<8>, grid, dim3(256), 0, stream, pk);
    return hipGetLastError();
}

__global__ void rope_frequencies_kernel(float* out, const float* scalars, int n, int64_t out_s, int64_t sc_s, float log2_base) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    // rope.py:279-286: 1 / exp2(log2(base) * (j / n)), optionally divided by a per-frequency scalar
    float f = 1.0f / exp2f(log2_base * ((float)j / (float)n));
    if (scalars) f /= scalars[(int64_t)j * sc_s];
    out[(int64_t)j * out_s] = f;
}

hipError_t launch_rope_frequencies(float* out, const float* scalars, int n, int64_t out_s, int64_t sc_s, float log2_base,
                                   hipStream_t stream) {
    hipLaunchKernelGGL(rope_frequencies_kernel, dim3((n + 127) / 128), dim3(128), 0, stream, out, scalars, n, out_s, sc_s, log2_base);
    return hipGetLastError();
}

}  // namespace g4b
