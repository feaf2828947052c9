// q/k RMSNorm + rotary embedding for gfx950, optionally fused with the ring append of the rotated K and of V.
//
// An element-wise, HBM-bound pass: a thread owns eight consecutive columns j..j+7 of the first half of a head and
// their partners j + D/2..; it evaluates sin/cos of its eight angles once (full-precision sincosf: positions reach
// tens of thousands of radians) and then walks over the query heads and the kv heads of its (slot, token), so the
// angles are shared by every head as in the reference.  Loads and stores are 16- or 32-byte vectors per half row;
// a workgroup covers 256 / (D/16) tokens of one slot.  With the append fused, rotated K goes straight into the ring
// in the cache's dtype (one rounding) and V is copied / normalised by the same threads: the K and V scratch rows are
// read once and nothing is read back.
#include "common.hpp"
#include "launch.hpp"

namespace g4b {

G4B_DEV void load8_f32(const void* base, int64_t elem_off, int dt, float (&v)[8]) {
    if (dt == DT_F32) {
        const f4* src = reinterpret_cast<const f4*>(static_cast<const float*>(base) + elem_off);
        const f4 a = src[0], c = src[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = a[i];
            v[4 + i] = c[i];
        }
    } else {
        const u4 raw = *reinterpret_cast<const u4*>(static_cast<const uint16_t*>(base) + elem_off);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = raw[i];
            v[2 * i] = dt == DT_F16 ? F16::lo(w) : BF16::lo(w);
            v[2 * i + 1] = dt == DT_F16 ? F16::hi(w) : BF16::hi(w);
        }
    }
}

// One head row, in two steps so that the loads of several rows can be in flight before any of them is stored
// (the rows are rewritten in place, so the compiler may not move a load above an earlier store by itself).
struct RopeRow {
    float x1[8], x2[8];
};
G4B_DEV void rope_row_load(RopeRow& r, const void* x, int64_t xo, int x_dt, int half) {
    load8_f32(x, xo, x_dt, r.x1);
    load8_f32(x, xo + half, x_dt, r.x2);
}
G4B_DEV void rope_row_finish(const RopeRow& r, void* x, int64_t xo, int x_dt, float inv_rms, const float (&w1)[8],
                             const float (&w2)[8], const float (&sn)[8], const float (&cs)[8], int half, bool writeback,
                             void* cache, int64_t co, int cache_dt) {
    float y1[8], y2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        // rope.py:33-37: x *= inv_rms * w, then the rotation, all in fp32
        const float a = r.x1[i] * (inv_rms * w1[i]);
        const float b = r.x2[i] * (inv_rms * w2[i]);
        y1[i] = cs[i] * a - sn[i] * b;
        y2[i] = cs[i] * b + sn[i] * a;
    }
    if (writeback) {
        store8(x, xo, x_dt, y1);
        store8(x, xo + half, x_dt, y2);
    }
    if (cache) {
        store8(cache, co, cache_dt, y1);
        store8(cache, co + half, cache_dt, y2);
    }
}

__global__ __launch_bounds__(256) void rope_kernel(const RopeParams p) {
    const int b = blockIdx.y;
    const int half = p.D / 2;
    const int tpr = p.D / 16;            // threads per token (eight columns of each half per thread)
    const int rows = 256 / tpr;          // tokens per workgroup
    const int tt = blockIdx.x * rows + threadIdx.x / tpr;
    const int j0 = (threadIdx.x % tpr) * 8;
    // threads beyond rows * tpr (D / 16 does not divide 256) would alias the next workgroup's first token
    if ((int)threadIdx.x >= rows * tpr || tt >= p.t) return;

    const int32_t off = p.offsets[(int64_t)b * p.off_s];
    const float pos = (float)(off + tt);  // rope.py:180: integer position, converted once
    float sn[8], cs[8], qw1[8], qw2[8], kw1[8], kw2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
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
            // up to four query heads at a time (this workgroup's heads are job, job + z, ...)
            constexpr int NB = 4;
            RopeRow rows[NB];
            float rs[NB];
            const int step = gridDim.z;
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int h = job + u * step;
                if (h < p.H) {
                    rs[u] = p.q_rsos[(int64_t)b * p.q_rsos_s[0] + (int64_t)h * p.q_rsos_s[1] + (int64_t)tt * p.q_rsos_s[2]];
                    rope_row_load(rows[u], p.q, (int64_t)b * p.q_s[0] + (int64_t)h * p.q_s[1] + (int64_t)tt * p.q_s[2] + j0, p.q_dt, half);
                }
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int h = job + u * step;
                if (h < p.H) {
                    const float inv = 1.0f / __builtin_sqrtf(rs[u] / (float)p.D + p.eps);
                    rope_row_finish(rows[u], p.q, (int64_t)b * p.q_s[0] + (int64_t)h * p.q_s[1] + (int64_t)tt * p.q_s[2] + j0, p.q_dt,
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
            RopeRow row;
            rope_row_load(row, p.k, xo, p.k_dt, half);
            rope_row_finish(row, p.k, xo, p.k_dt, inv, kw1, kw2, sn, cs, half, k_back, append ? p.k_cache : nullptr, co, p.cache_dt);
        } else {
            // V: thread (token, j0) owns columns [2*j0, 2*j0 + 16) of the row while they exist; Dv may exceed D
            const int g = job - p.H - p.G;
            float inv = 1.f;
            if (p.v_rsos) {
                const float r = p.v_rsos[(int64_t)b * p.v_rsos_s[0] + (int64_t)g * p.v_rsos_s[1] + (int64_t)tt * p.v_rsos_s[2]];
                inv = 1.0f / __builtin_sqrtf(r / (float)p.Dv + p.eps);
            }
            for (int c = j0 * 2; c < p.Dv; c += p.D) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int col = c + 8 * s;
                    if (col < p.Dv) {
                        float v8[8];
                        load8_f32(p.v, (int64_t)b * p.v_s[0] + (int64_t)g * p.v_s[1] + (int64_t)tt * p.v_s[2] + col, p.v_dt, v8);
#pragma unroll
                        for (int i = 0; i < 8; ++i) v8[i] *= inv;
                        store8(p.v_cache, (int64_t)b * p.v_cache_sb + ((int64_t)g * p.T + ring_row) * p.Dv + col, p.cache_dt, v8);
                    }
                }
            }
        }
    }
}

hipError_t launch_rope(const RopeParams& p, hipStream_t stream) {
    const int rows = 256 / (p.D / 16);
    const int blocks = (p.t + rows - 1) / rows;
    // launches of a few tokens (decode): split the row jobs of a token up to four ways to get the chip busy at all;
    // otherwise a thread walks all heads of its token, which are neighbours in the engine's [B, t, heads, D] layout
    const int jobs = p.H + 2 * p.G;
    int z = 1;
    while (z < 4 && z * 2 <= jobs && (int64_t)blocks * p.B * z < 256) z *= 2;
    dim3 grid(blocks, p.B, z);
    G4B_LAUNCH_DOMINANT(rope_kernel, grid, dim3(256), 0, stream, p);
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
