// KV ring append and decode-state advance for gfx950.  Both are index kernels: the ring row of
// new token t of slot b is (t + cache_offsets[b]) mod T and must be bit-exact; values are copied
// (or scaled by the weightless RMSNorm factor rsqrt(rsos / D + eps) in fp32) and rounded once
// into the cache dtype.
#include "common.hpp"
#include "launch.hpp"

namespace g4b {

// One thread moves N consecutive elements, 16 bytes of the wider of the two types (N = 4 when the scratchpad or the
// cache is fp32, else 8), so a wave reads and writes contiguous runs; a workgroup of 256 threads covers 256 * N
// elements of the [G, t, D] block of one slot.
template <int N>
__global__ __launch_bounds__(256) void kv_append_kernel(const KvAppendParams p) {
    const int b = blockIdx.y;
    if (p.phase_arr && p.phase_arr[(int64_t)b * p.ph_s] != (uint8_t)p.phase) return;
    const int64_t off = p.off_is_i64 ? static_cast<const int64_t*>(p.offsets)[(int64_t)b * p.off_s]
                                     : (int64_t) static_cast<const int32_t*>(p.offsets)[(int64_t)b * p.off_s];
    const int segs = p.D / N;
    const int64_t n = (int64_t)p.G * p.t * segs;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int seg = (int)(idx % segs);
    const int tt = (int)((idx / segs) % p.t);
    const int g = (int)(idx / ((int64_t)segs * p.t));
    int64_t row = (tt + off) % p.T;
    if (row < 0) row += p.T;

    const int64_t xo = (int64_t)b * p.x_s[0] + (int64_t)g * p.x_s[1] + (int64_t)tt * p.x_s[2] + seg * N;
    float v[N];
    load_f32<N>(p.x, xo, p.x_dt, v);
    if (p.x_rsos) {
        const float r = p.x_rsos[(int64_t)b * p.rsos_s[0] + (int64_t)g * p.rsos_s[1] + (int64_t)tt * p.rsos_s[2]];
        const float inv = 1.0f / __builtin_sqrtf(r / (float)p.D + p.eps);
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] *= inv;
    }
    const int64_t co = (int64_t)b * p.cache_sb + ((int64_t)g * p.T + row) * p.D + seg * N;
    store_n<N>(p.cache, co, p.cache_dt, v);
}

hipError_t launch_kv_append(const KvAppendParams& p, hipStream_t stream) {
    const int N = (p.x_dt == DT_F32 || p.cache_dt == DT_F32) ? 4 : 8;
    const int64_t n = (int64_t)p.G * p.t * (p.D / N);
    dim3 grid((unsigned)((n + 255) / 256), p.B);
    if (N == 4) hipLaunchKernelGGL(kv_append_kernel<4>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(kv_append_kernel<8>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void advance_decode_state_kernel(const AdvanceParams p) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= p.B) return;
    if (p.user_phase[(int64_t)b * p.ph_s] != 2) return;  // decode-phase slots only
    p.input_token_ids[(int64_t)b * p.in_s1] = p.out_token_ids[(int64_t)b * p.out_s0];
    p.cache_offsets[(int64_t)b * p.off_s] += 1;
    p.time_dim_sizes[(int64_t)b * p.tds_s] += 1;
}

hipError_t launch_advance_decode_state(const AdvanceParams& p, hipStream_t stream) {
    hipLaunchKernelGGL(advance_decode_state_kernel, dim3((p.B + 255) / 256), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace g4b
