// Host-side launchers implemented by the kernel translation units.
#pragma once
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.hpp"

namespace g4b {

// Profiling aid: when the calling thread has armed a pair of events, the dominant kernel of the next launcher call is
// dispatched with them (hipExtLaunchKernelGGL stamps the events with the begin and the end of that dispatch, so their
// difference is the kernel's own duration, without the gaps an event pair recorded around the launch includes).
struct ProfileEvents {
    hipEvent_t start = nullptr, stop = nullptr;
};
inline thread_local ProfileEvents g_profile_events;
#define G4B_LAUNCH_DOMINANT(kernel, grid, block, smem, stream, ...)                                                    \
    do {                                                                                                               \
        if (g4b::g_profile_events.start) {                                                                             \
            hipExtLaunchKernelGGL(kernel, grid, block, smem, stream, g4b::g_profile_events.start,                      \
                                  g4b::g_profile_events.stop, 0, __VA_ARGS__);                                         \
            g4b::g_profile_events = g4b::ProfileEvents{};                                                              \
        } else {                                                                                                       \
            hipLaunchKernelGGL(kernel, grid, block, smem, stream, __VA_ARGS__);                                        \
        }                                                                                                              \
    } while (0)

// Raise a kernel's dynamic shared memory limit once per device (the attribute belongs to the function on the current
// device).  `done` is the call site's bit mask of devices already served.
inline hipError_t allow_dynamic_smem(const void* kernel, int bytes, uint64_t& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && ((done >> dev) & 1)) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && dev >= 0 && dev < 64) done |= 1ull << dev;
    return e;
}

// Decode-shaped launches, host-side choice (static in the launch arguments, so a recorded graph keeps it): the
// one-kernel variant (a workgroup of four waves per (slot, kv head) pair, merged through LDS) when no slot can bring
// more than DEC_PAIR_MAX_KEYS keys (four tiles per wave; beyond that the waves' sequential tiles cost more than the
// second launch saves).
constexpr int DEC_PAIR_MAX_KEYS = 512;
inline bool decode_pair_path(const AttnParams& p, int D) {
    return D <= 256 && p.win_arr == nullptr && (p.W < p.KV_CTX ? p.W : p.KV_CTX) <= DEC_PAIR_MAX_KEYS;
}

// rows = (H/G) * Tq <= 16, D in {128, 256, 512}; kv_dt in {DT_F16, DT_BF16}
hipError_t launch_attn_decode(const AttnParams& p, int D, int kv_dt, hipStream_t stream);
// any Tq; (H/G) must divide 128; D in {128, 256}
hipError_t launch_attn_prefill(const AttnParams& p, int D, int kv_dt, hipStream_t stream);
// any Tq; (H/G) must divide 128; D = 512
hipError_t launch_attn_prefill_wide(const AttnParams& p, int kv_dt, hipStream_t stream);

// any Tq, any H/G, D a multiple of 8 up to 1024, kv_dt also DT_F32, STAGE_ON_BAND with its block size: plain fp32 kernel
hipError_t launch_attn_generic(const AttnParams& p, int D, int kv_dt, int on_band_block, hipStream_t stream);

// One launch for the prefill-phase slots (pp: rows > 16) and the decode-phase slots (pd: rows <= 16) of a batch.
struct MixedPlan {
    int npx;          // prefill workgroups per XCD (grid slots; the prefill body drops the surplus)
    int nd_blocks;    // decode workgroups
    int pair_path;    // 1: short-window decode, one workgroup per (slot, kv head) pair
    int combine_pf;   // merge workgroups of the prefill half
    int combine_dec;  // merge workgroups of the decode half
};
// head dimension 256
hipError_t launch_attn_mixed_f16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream);
hipError_t launch_attn_mixed_bf16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream);
// head dimension 512
hipError_t launch_attn_mixed_d512_f16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream);
hipError_t launch_attn_mixed_d512_bf16(const AttnParams& pp, const AttnParams& pd, const MixedPlan& mp, hipStream_t stream);

struct KvAppendParams {
    const void* x;
    void* cache;
    const void* offsets;    // int32 or int64
    const float* x_rsos;    // optional [B,G,t] row sums of squares
    const uint8_t* phase_arr;  // optional
    int64_t x_s[4];
    int64_t rsos_s[3];
    int64_t cache_sb;  // batch stride of the cache (elements)
    int64_t off_s, ph_s;
    int32_t x_dt, cache_dt, off_is_i64;
    int32_t B, G, t, T, D;
    int32_t phase;
    float eps;
};
hipError_t launch_kv_append(const KvAppendParams& p, hipStream_t stream);

struct AdvanceParams {
    int32_t* input_token_ids;  // [t, B], row 0 written
    const int32_t* out_token_ids;  // [B, >=1], column 0 read
    int32_t* cache_offsets;
    int32_t* time_dim_sizes;
    const uint8_t* user_phase;
    int64_t in_s1, out_s0, off_s, tds_s, ph_s;
    int32_t B;
};
hipError_t launch_advance_decode_state(const AdvanceParams& p, hipStream_t stream);

struct RopeParams {
    void* q;
    void* k;
    const float* freqs;
    const int32_t* offsets;
    const float* q_rsos;
    const float* k_rsos;
    const float* q_w;
    const float* k_w;
    const void* v;          // optional: fused append
    const float* v_rsos;    // optional
    void* k_cache;          // optional: fused append
    void* v_cache;
    const uint8_t* phase_arr;  // optional
    int64_t q_s[4], k_s[4], v_s[4];
    int64_t q_rsos_s[3], k_rsos_s[3], v_rsos_s[3];
    int64_t freqs_s, q_w_s, k_w_s, off_s, ph_s;
    int64_t k_cache_sb, v_cache_sb;
    int32_t q_dt, k_dt, v_dt, cache_dt;
    int32_t B, H, G, t, D, Dv, T;
    int32_t phase, k_writeback;
    int32_t xcd_weighted;  // 1: workgroup i of a grid runs on an XCD of the parity of i, and the even XCDs get 26 blocks of 50
    int32_t even_blocks;  // rope_kernel: token blocks dealt to the even workgroups (0: workgroup i takes token block i)
    float eps;
};
hipError_t launch_rope(const RopeParams& p, hipStream_t stream);
hipError_t launch_rope_frequencies(float* out, const float* scalars, int n, int64_t out_s, int64_t sc_s, float log2_base,
                                   hipStream_t stream);

}  // namespace g4b
