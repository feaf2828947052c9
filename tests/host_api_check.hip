// Host-side driver for the sanitizer build (g4b_amd/build.py --asan, tests/test_host_sanitizers.py): every entry point of
// the C ABI is called with argument blocks that the host-side validation must refuse, so the checks, the size
// arithmetic and the error formatting run under AddressSanitizer and UndefinedBehaviorSanitizer.  The kernel launchers
// are replaced by stand-ins that abort: nothing here may reach a launch (the pointers are not device memory).
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../g4b_amd/csrc/launch.hpp"
#include "../include/g4b_attn.h"

namespace g4b {
[[noreturn]] static void reached(const char* what) {
    fprintf(stderr, "host_api_check: validation let a launch through (%s)\n", what);
    abort();
}
hipError_t launch_attn_decode(const AttnParams&, int, int, hipStream_t) { reached("decode"); }
hipError_t launch_attn_prefill(const AttnParams&, int, int, hipStream_t) { reached("prefill"); }
hipError_t launch_attn_prefill_wide(const AttnParams&, int, hipStream_t) { reached("prefill 512"); }
hipError_t launch_attn_generic(const AttnParams&, int, int, int, hipStream_t) { reached("generic"); }
hipError_t launch_attn_mixed_f16(const AttnParams&, const AttnParams&, const MixedPlan&, hipStream_t) { reached("mixed"); }
hipError_t launch_attn_mixed_bf16(const AttnParams&, const AttnParams&, const MixedPlan&, hipStream_t) { reached("mixed"); }
hipError_t launch_attn_mixed_d512_f16(const AttnParams&, const AttnParams&, const MixedPlan&, hipStream_t) { reached("mixed"); }
hipError_t launch_attn_mixed_d512_bf16(const AttnParams&, const AttnParams&, const MixedPlan&, hipStream_t) { reached("mixed"); }
hipError_t launch_kv_append(const KvAppendParams&, hipStream_t) { reached("append"); }
hipError_t launch_advance_decode_state(const AdvanceParams&, hipStream_t) { reached("advance"); }
hipError_t launch_rope(const RopeParams&, hipStream_t) { reached("rope"); }
hipError_t launch_rope_frequencies(float*, const float*, int, int64_t, int64_t, float, hipStream_t) { reached("rope frequencies"); }
}  // namespace g4b

static long checks = 0, bad = 0;
static void expect(int got, int want, const char* what) {
    ++checks;
    if (got != want || (want != G4B_OK && strlen(g4b_last_error()) == 0)) {
        ++bad;
        printf("%s: status %d, expected %d (\"%s\")\n", what, got, want, g4b_last_error());
    }
}

// an argument block that would pass: B=4 slots, H=8, G=2, Tq, D, ring of 4096 rows
static g4b_attn_args good(int Tq, int D) {
    g4b_attn_args a;
    memset(&a, 0, sizeof(a));
    a.q = a.k_cache = a.v_cache = a.o = reinterpret_cast<void*>(4096);
    a.time_dim_sizes = reinterpret_cast<const int32_t*>(4096);
    a.user_phase = reinterpret_cast<const uint8_t*>(4096);
    a.B = 4, a.H = 8, a.G = 2, a.Tq = Tq, a.D = D, a.KV_CTX = 4096;
    const int64_t qs[4] = {(int64_t)8 * Tq * D, (int64_t)Tq * D, D, 1};
    for (int i = 0; i < 4; ++i) a.q_stride[i] = a.o_stride[i] = qs[i];
    a.k_stride_b = a.v_stride_b = (int64_t)2 * 4096 * D;
    a.time_dim_sizes_stride = a.user_phase_stride = 1;
    a.ctx_window_size = 4096, a.phase = 2, a.stage = G4B_STAGE_CAUSAL, a.scale = 1.f;
    return a;
}

int main() {
    expect(g4b_attn_forward(nullptr, nullptr), G4B_ERR_INVALID_ARGUMENT, "NULL block");
    expect(g4b_attn_forward_static_scratch(nullptr, nullptr), G4B_ERR_INVALID_ARGUMENT, "NULL block, static scratch");
    expect(g4b_attn_forward_mixed(nullptr, nullptr, nullptr), G4B_ERR_INVALID_ARGUMENT, "NULL blocks, mixed");
    for (int Tq : {1, 3, 64, 512, 8192})
        for (int D : {8, 64, 128, 256, 512, 1024}) {
            g4b_attn_args a = good(Tq, D);
#define REJECT(mutation, status, what) { g4b_attn_args b = a; mutation; expect(g4b_attn_forward(&b, nullptr), status, what); }
            REJECT(b.q = nullptr, G4B_ERR_INVALID_ARGUMENT, "q NULL")
            REJECT(b.user_phase = nullptr, G4B_ERR_INVALID_ARGUMENT, "user_phase NULL")
            REJECT(b.q_dtype = 9, G4B_ERR_INVALID_ARGUMENT, "q dtype")
            REJECT(b.kv_dtype = -1, G4B_ERR_INVALID_ARGUMENT, "kv dtype")
            REJECT(b.B = 0, G4B_ERR_INVALID_ARGUMENT, "B = 0")
            REJECT(b.H = 7, G4B_ERR_INVALID_ARGUMENT, "H % G")
            REJECT(b.D = D + 4, G4B_ERR_UNSUPPORTED, "D % 8")
            REJECT(b.D = 2048, G4B_ERR_UNSUPPORTED, "D > 1024")
            REJECT(b.B = 70000, G4B_ERR_UNSUPPORTED, "B > 65535")
            REJECT(b.ctx_window_size = 0, G4B_ERR_INVALID_ARGUMENT, "W = 0")
            REJECT(b.ctx_window_size = 4097, G4B_ERR_INVALID_ARGUMENT, "W > KV_CTX")
            REJECT(b.stage = 0, G4B_ERR_INVALID_ARGUMENT, "stage")
            REJECT(b.stage = G4B_STAGE_ON_BAND, G4B_ERR_INVALID_ARGUMENT, "on-band without a block size")
            REJECT(b.phase = 256, G4B_ERR_INVALID_ARGUMENT, "phase")
            REJECT(b.query_window = -1, G4B_ERR_INVALID_ARGUMENT, "query window")
            REJECT(b.scale = 0.f, G4B_ERR_INVALID_ARGUMENT, "scale 0")
            REJECT(b.scale = -1.f, G4B_ERR_INVALID_ARGUMENT, "scale < 0")
            REJECT(b.q_stride[3] = 2, G4B_ERR_INVALID_ARGUMENT, "q inner stride")
            REJECT(b.o_stride[1] = 4, G4B_ERR_INVALID_ARGUMENT, "o stride % 8")
            REJECT(b.q = reinterpret_cast<void*>(4100), G4B_ERR_INVALID_ARGUMENT, "q alignment")
            REJECT(b.k_stride_b = 8, G4B_ERR_INVALID_ARGUMENT, "cache slot stride")
            REJECT(b.num_workers = -3, G4B_ERR_INVALID_ARGUMENT, "num_workers")
            REJECT(b.KV_CTX = 1 << 30; b.ctx_window_size = 1; b.k_stride_b = b.v_stride_b = INT64_MAX / 2 & ~7ll, G4B_ERR_UNSUPPORTED, "2 GiB per (slot, kv head)")
            REJECT(b.B = 60000; b.G = 40000; b.H = 40000; b.D = 8; b.KV_CTX = b.ctx_window_size = 1 << 20;
                   b.k_stride_b = b.v_stride_b = (int64_t)40000 * (1 << 20) * 8, G4B_ERR_UNSUPPORTED, "tile count beyond 32 bits")
            if ((a.H / a.G) * Tq <= 16 && (D == 128 || D == 256 || D == 512)) {
                REJECT(b.workspace = reinterpret_cast<void*>(4096); b.workspace_bytes = 16, G4B_ERR_WORKSPACE, "workspace too small")
                g4b_attn_args b = a;
                b.num_workers = 1 << 20;
                expect(g4b_attn_forward_static_scratch(&b, nullptr), G4B_ERR_WORKSPACE, "static scratch too small");
            }
            {
                g4b_attn_args b = a;
                b.workspace = reinterpret_cast<void*>(4096);
                expect(g4b_attn_forward_static_scratch(&b, nullptr), G4B_ERR_INVALID_ARGUMENT, "static scratch with a workspace");
            }
#undef REJECT
            // size queries never fail: they return 0 for what never uses a workspace
            ++checks;
            const uint64_t w = g4b_attn_workspace_bytes(4, 8, 2, Tq, D, 0);
            if ((D != 128 && D != 256 && D != 512) != (w == 0) && Tq <= 2) {
                ++bad;
                printf("workspace bytes Tq=%d D=%d: %llu\n", Tq, D, (unsigned long long)w);
            }
            (void)g4b_attn_mixed_workspace_bytes(33, 8, 2, 512, 1, D, 32768, 32768, 0, 0);
            // mixed launch: the halves must share the caches and differ in phase
            g4b_attn_args pf = good(512, 256), dec = good(1, 256);
            pf.phase = 1;
            { g4b_attn_args d2 = dec; d2.k_cache = reinterpret_cast<void*>(8192); expect(g4b_attn_forward_mixed(&pf, &d2, nullptr), G4B_ERR_INVALID_ARGUMENT, "mixed: caches differ"); }
            { g4b_attn_args d2 = dec; d2.phase = 1; expect(g4b_attn_forward_mixed(&pf, &d2, nullptr), G4B_ERR_INVALID_ARGUMENT, "mixed: same phase"); }
            { expect(g4b_attn_forward_mixed(&dec, &pf, nullptr), G4B_ERR_INVALID_ARGUMENT, "mixed: halves swapped"); }
            { g4b_attn_args p2 = good(512, 128), d2 = good(1, 128); p2.phase = 1; expect(g4b_attn_forward_mixed(&p2, &d2, nullptr), G4B_ERR_UNSUPPORTED, "mixed: head dim 128"); }
        }
    g4b_kv_append_args k;
    memset(&k, 0, sizeof(k));
    expect(g4b_kv_append(nullptr, nullptr), G4B_ERR_INVALID_ARGUMENT, "append NULL");
    expect(g4b_kv_append(&k, nullptr), G4B_ERR_INVALID_ARGUMENT, "append zero block");
    k.x = k.cache_offsets = reinterpret_cast<void*>(4096);
    k.cache = reinterpret_cast<void*>(4096);
    k.B = 2, k.G = 2, k.t = 20, k.T = 17, k.D = 64;
    k.x_stride[0] = 2 * 20 * 64, k.x_stride[1] = 20 * 64, k.x_stride[2] = 64, k.x_stride[3] = 1;
    k.cache_stride_b = 2 * 17 * 64, k.cache_offsets_stride = 1;
    expect(g4b_kv_append(&k, nullptr), G4B_ERR_INVALID_ARGUMENT, "append t > T");
    g4b_advance_args adv;
    memset(&adv, 0, sizeof(adv));
    expect(g4b_advance_decode_state(&adv, nullptr), G4B_ERR_INVALID_ARGUMENT, "advance zero block");
    g4b_rope_args r;
    memset(&r, 0, sizeof(r));
    expect(g4b_rope(&r, nullptr), G4B_ERR_INVALID_ARGUMENT, "rope zero block");
    expect(g4b_rope_frequencies(nullptr, nullptr, 0, 1, 1, 1e6f, nullptr), G4B_ERR_INVALID_ARGUMENT, "rope frequencies");
    float ms[4];
    expect(g4b_profile_end(ms, 4), G4B_ERR_INVALID_ARGUMENT, "profile_end without begin");
    printf("%ld checks, %ld bad\n", checks, bad);
    return bad ? 1 : 0;
}
