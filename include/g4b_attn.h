/*
 * g4b_attn.h -- C ABI of libg4b_attn.so: the attention hot path of the g4b inference engine
 * (flash attention over the per-slot ring KV cache, KV append, decode-state advance) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - Every pointer is a device pointer owned by the caller; the library never allocates,
 *     frees or synchronises (the scratch of g4b_attn_forward_static_scratch is an array in the
 *     library's device image, not an allocation).  Work is enqueued on `stream` (a hipStream_t passed as void*;
 *     NULL = the default stream) and is legal inside stream capture.  One exception, once per GPU: the first
 *     decode-shaped attention or rope launch (or g4b_static_scratch_init) outside stream capture runs a 64-workgroup
 *     kernel that reports which XCD each workgroup ran on and waits for it on `stream`; the streaming kernels weight
 *     their work shares by the answer.  Launches captured before that keep equal shares.
 *   - Environment switches, read when the library is first used (counterparts of the reference's
 *     G4B_FA_FORCE_CONFIG / G4B_FA_PRINT_CONFIG, g4b/kernels/fa2.py:148-150,691-700): G4B_ATTN_NUM_WORKERS=n sets the
 *     default worker count of decode-shaped launches (and the size g4b_attn_workspace_bytes reports for it);
 *     G4B_ATTN_XCD_SHARES=0 forces equal work shares, =1 the weighted ones without asking the hardware;
 *     G4B_ATTN_PRINT_PLAN=1 prints one line per attention launch on stderr (kernel family, grid, workers, splits).
 *   - Strides are in ELEMENTS, as in the reference's launch adapter (g4b/kernels/utils.py:87-127).
 *   - Entry points return G4B_OK (0) or a negative g4b_status.  Arguments are validated on the
 *     host before anything is launched; g4b_last_error() returns a thread-local message for the
 *     last failure.
 *   - dtype codes: G4B_DT_F16, G4B_DT_BF16, G4B_DT_F32.
 */
#ifndef G4B_ATTN_H
#define G4B_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define G4B_ATTN_ABI_VERSION 4

enum g4b_status {
    G4B_OK = 0,
    G4B_ERR_INVALID_ARGUMENT = -1, /* shape / stride / dtype / value check failed (reference: tl.static_assert) */
    G4B_ERR_UNSUPPORTED = -2,      /* valid in the reference, not built here (e.g. head_dim above 1024, a mixed launch at head_dim 128) */
    G4B_ERR_WORKSPACE = -3,        /* workspace missing or too small for the requested split-KV launch */
    G4B_ERR_LAUNCH = -4,           /* the HIP runtime refused the launch (no device, bad stream, ...) */
    G4B_ERR_BUSY = -5              /* g4b_attn_forward_static_scratch: the array is in use by unfinished work on another stream */
};

enum g4b_dtype { G4B_DT_F16 = 0, G4B_DT_BF16 = 1, G4B_DT_F32 = 2 };

/* g4b/kernels/fa2.py:14-16 */
enum g4b_stage { G4B_STAGE_FULL = 1, G4B_STAGE_ON_BAND = 2, G4B_STAGE_CAUSAL = 3 };
/* g4b/kernels/fa2.py:29-31 */
enum g4b_phase { G4B_PHASE_UNALLOCATED = 0, G4B_PHASE_PREFILL = 1, G4B_PHASE_DECODE = 2 };

/*
 * g4b_attn_forward replaces flash_attention() = _attn_kernel + _reduce_split_kv_kernel
 * (g4b/kernels/fa2.py:634-715, 256-480, 546-631).
 *
 *   q, o          [B, H, Tq, D], any strides with last stride 1 (the engine passes permuted views
 *                 of [B, t, H, D] scratchpads, g4b/models/gemma4e.py:1031-1033); f16 / bf16 / f32.
 *   k_cache,      [B, G, KV_CTX, D], contiguous inside a slot (fa2.py:315-320), slot stride
 *   v_cache       k_stride_b / v_stride_b; f16 or bf16, or f32 (the reference's G4B_DTKV_FP32 debugging switch,
 *                 g4b/models/gemma4e.py:32).
 *   time_dim_sizes[B] int32: tokens in the slot after this step (fa2.py:52).
 *   user_phase    [B] uint8: slots whose value differs from `phase` are skipped and their rows of
 *                 `o` are left untouched (fa2.py:332-335).
 *   ctx_window_size  W <= KV_CTX: the launch sees the last min(tds, W) keys; logical key j is ring
 *                 row (max(tds - W, 0) + j) % KV_CTX; query i is aligned with logical key
 *                 min(tds, W) - Tq + i (fa2.py:53-56,75).
 *   stage         G4B_STAGE_CAUSAL (default of the reference), G4B_STAGE_FULL, or G4B_STAGE_ON_BAND: the diagonal
 *                 block alone (fa2.py:61,399-435), whose extent is the reference's autotuned Q_BLOCKSIZE_T and has to be
 *                 named here.
 *   on_band_block with G4B_STAGE_ON_BAND: Q_BLOCKSIZE_T (fa2.py:56,140-180; 1 in the reference's default configuration
 *                 list).  Query i then sees the keys of its own block of that many positions up to itself:
 *                 logical keys [q_t_base + (i / block) * block, q_t_base + i].  Ignored by the other stages.
 *   scale         softmax scale; the reference computes with 1.0 (fa2.py:89).
 *   query_window  0 = anchored window, the reference kernel's semantics.  > 0 additionally hides
 *                 keys with q_pos - k_pos >= query_window, the per-query sliding window of the CPU
 *                 reference's one-shot prefill (scripts/reference_impl.py:440-441).
 *   window_sizes  optional [B] int32 per-slot override of ctx_window_size (extension; NULL = none).
 *   workspace     device scratch for split-KV partials, >= g4b_attn_workspace_bytes(...) bytes, or
 *                 NULL: then a decode-shaped launch (R*Tq <= 16) uses one wave per (slot, kv head)
 *                 and a prefill-shaped launch one workgroup per (slot, kv head, query tile) however
 *                 few slots are in phase.  Contents are unspecified after the call (like
 *                 partial_o/l/m, fa2.py:643-645).  A decode-shaped launch with D <= 256,
 *                 ctx_window_size <= 512 and no window_sizes merges in LDS and never touches it.
 *   num_workers   0 = library default; otherwise the number of workers the decode key tiles are
 *                 dealt to (must not exceed the value the workspace was sized for).  A worker is one
 *                 wave, or a pair of waves when D = 512.  Ignored by
 *                 prefill-shaped launches, which choose their key split from the number of in-phase
 *                 slots on the device.
 *   use_fp32_dot  the reference's USE_FP32_DOT (fa2.py:85-88,126-129): 0 = the query is rounded to the cache's 16-bit
 *                 type before K Q^T, as the reference's `q.to(tl.float16)` does; non-zero = a query of a wider type
 *                 (f32 over any cache, f16 over a bf16 cache) enters K Q^T as the sum of two 16-bit operands, its
 *                 rounded value and its rounding error, so the scores are those of the unrounded query.  The engine
 *                 passes fp32 q with use_fp32_dot=True and scale 1.0 (g4b/models/gemma4e.py:30,606).  No effect when
 *                 q already has the cache's type.
 *   kernel_mask   profiling aid.  0 = run every kernel of the launch.  Otherwise bit 0 selects the
 *                 main attention kernel and bit 1 the split-merge kernel, so that each can be timed
 *                 on its own; results are only complete with both.
 *
 * The tuned kernels serve D in {128, 256, 512} with f16 / bf16 caches, the causal and full stages and, for
 * prefill-shaped launches ((H/G)*Tq > 16), H/G dividing 128 (64 at D = 512 with a split query): everything Gemma-4
 * and the reference's own test list (tests/compare_scripts/test_fa2.py:51-79) use.  Any other D that is a multiple of
 * 8 up to 1024, any other H/G, an f32 cache and G4B_STAGE_ON_BAND run on a plain fp32 kernel without matrix
 * instructions: same results to the same tolerance, a fraction of the speed, no workspace.
 *
 * Rows whose visible key set is empty (time_dim_sizes[b] == 0 on an in-phase slot) are written
 * as zeros; the reference leaves 0/0 there and its caller ignores them (g4b/scheduler.py:142-148).
 */
typedef struct g4b_attn_args {
    const void* q;
    const void* k_cache;
    const void* v_cache;
    void* o;
    const int32_t* time_dim_sizes;
    const uint8_t* user_phase;
    const int32_t* window_sizes;
    void* workspace;
    uint64_t workspace_bytes;
    int64_t q_stride[4];
    int64_t o_stride[4];
    int64_t k_stride_b;
    int64_t v_stride_b;
    int64_t time_dim_sizes_stride;
    int64_t user_phase_stride;
    int64_t window_sizes_stride;
    int32_t q_dtype;
    int32_t o_dtype;
    int32_t kv_dtype;
    int32_t B, H, G, Tq, D, KV_CTX;
    int32_t ctx_window_size;
    int32_t phase;
    int32_t stage;
    int32_t query_window;
    int32_t num_workers;
    int32_t kernel_mask;
    int32_t use_fp32_dot;
    int32_t on_band_block;
    float scale;
} g4b_attn_args;

int g4b_attn_forward(const g4b_attn_args* args, void* stream);

/* Bytes of workspace that let g4b_attn_forward split keys: for a decode-shaped launch (R*Tq <= 16)
 * over `num_workers` workers (0 = library default); for a prefill shape that brings fewer workgroups
 * per slot than the chip has compute units (chunked prefill, short prompts; sized by H, G, Tq, D
 * only) over several workgroups per query tile.  Returns 0 when the shape never uses a workspace.
 * Replaces the sizing of partial_o/l/m at g4b/models/gemma4e.py:43,819-821. */
uint64_t g4b_attn_workspace_bytes(int32_t B, int32_t H, int32_t G, int32_t Tq, int32_t D, int32_t num_workers);

/* The library default for num_workers on the current build (a multiple of the CU count) for D <= 256;
 * half of it for D = 512, whose workers are pairs of waves. */
int32_t g4b_attn_default_workers(void);

/*
 * g4b_attn_forward_mixed: one launch for a step that holds prefill-phase and decode-phase slots at once.  The
 * reference kernel skips per slot on user_phase[b] != PHASE (g4b/kernels/fa2.py:332-335), so such a step is two
 * flash_attention calls over the same batch tensors, one per phase, and its scheduler avoids the case altogether
 * (g4b/scheduler.py:66,96-98).  Here both calls are one grid: `prefill` is the argument block of the call whose query
 * block is a chunk ((H/G)*Tq > 16), `decode` the block of the call with one (or a few) query tokens per slot
 * ((H/G)*Tq <= 16); they must name the same caches, time_dim_sizes, user_phase, window_sizes, B, H, G, D, KV_CTX, cache
 * dtype and ctx_window_size and differ in q, o, Tq, strides and phase.  Results are those of the two calls.  The
 * workgroups of the two halves are dealt to different compute units, so the chunk's matrix work runs under the decode
 * stream's memory time.  Head dimensions 256 and 512.
 *   workspace     one buffer for both halves, passed in `prefill->workspace` (`decode->workspace` is ignored), at
 *                 least g4b_attn_mixed_workspace_bytes(...) bytes; NULL = neither half splits keys.
 *   num_workers   `decode->num_workers`: 0 = the library's share-out of the chip between the halves.
 */
int g4b_attn_forward_mixed(const g4b_attn_args* prefill, const g4b_attn_args* decode, void* stream);
uint64_t g4b_attn_mixed_workspace_bytes(int32_t B, int32_t H, int32_t G, int32_t Tq_prefill, int32_t Tq_decode, int32_t D,
                                        int32_t KV_CTX, int32_t ctx_window_size, int32_t has_window_sizes, int32_t num_workers);

/*
 * g4b_attn_forward_static_scratch: g4b_attn_forward for callers that cannot allocate.  It has no counterpart in the
 * reference; it is for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc, which
 * have no place to get the split-KV workspace from.  Same arguments and results as g4b_attn_forward with a workspace
 * of g4b_attn_workspace_bytes(...) bytes, except that `workspace` must be NULL: the split partials go to an array of
 * G4B_ATTN_STATIC_SCRATCH_BYTES bytes that is part of the library's device image (one copy per GPU the library runs
 * on, held until the process ends).  The call itself allocates and frees nothing.  A launch whose partials need more
 * than that is refused with G4B_ERR_WORKSPACE (the limit covers every prefill shape up to head dimension 512 and
 * decode batches of about a thousand (slot, kv head) pairs at the default worker count).  No kernel reads scratch
 * that the same call has not written, so nothing is cleared between calls; all calls on one GPU share the array, so
 * calls that overlap on one GPU would race.  The library remembers, per GPU, the stream of the last call that used the
 * array: a call on another stream while that stream still has unfinished work is refused with G4B_ERR_BUSY (wait for
 * the first stream, or give one of the calls a workspace through g4b_attn_forward).  Calls recorded into a graph are
 * not tracked -- whoever replays graphs concurrently keeps their launches apart.
 *
 * g4b_static_scratch_init looks the array's device address up for the current device (the first
 * g4b_attn_forward_static_scratch on a device does the same); call it once per device at load when the first launch
 * would otherwise happen under stream capture.
 */
#define G4B_ATTN_STATIC_SCRATCH_BYTES (68u << 20)
int g4b_attn_forward_static_scratch(const g4b_attn_args* args, void* stream);
int g4b_static_scratch_init(void);
uint64_t g4b_static_scratch_bytes(void);

/*
 * g4b_kv_append replaces add_kv_to_cache() (g4b/kernels/add_kv_to_cache.py:84-186):
 *   cache[b, g, (t + cache_offsets[b]) % T, :] = x[b, g, t, :] * (x_rsos ? rsqrt(x_rsos[b,g,t] / D + eps) : 1)
 * for slots with user_phase[b] == phase (all slots when user_phase is NULL).
 *   x [B,G,t,D] strided (last stride 1), f16/bf16/f32; cache [B,G,T,D] contiguous inside a slot,
 *   f16/bf16/f32; cache_offsets [B] int32 or int64; x_rsos [B,G,t] f32 strided or NULL; t <= T.
 */
typedef struct g4b_kv_append_args {
    const void* x;
    void* cache;
    const void* cache_offsets;
    const float* x_rsos;
    const uint8_t* user_phase;
    int64_t x_stride[4];
    int64_t x_rsos_stride[3];
    int64_t cache_stride_b;
    int64_t cache_offsets_stride;
    int64_t user_phase_stride;
    int32_t x_dtype;
    int32_t cache_dtype;
    int32_t cache_offsets_is_int64;
    int32_t B, G, t, T, D;
    int32_t phase;
    float rmsnorm_eps;
} g4b_kv_append_args;

int g4b_kv_append(const g4b_kv_append_args* args, void* stream);

/*
 * g4b_advance_decode_state replaces advance_decode_state()
 * (g4b/kernels/advance_decode_state.py:32-80): for slots with user_phase[b] == 2,
 *   input_token_ids[0, b] = out_token_ids[b, 0]; cache_offsets[b] += 1; time_dim_sizes[b] += 1.
 */
typedef struct g4b_advance_args {
    int32_t* input_token_ids;
    const int32_t* out_token_ids;
    int32_t* cache_offsets;
    int32_t* time_dim_sizes;
    const uint8_t* user_phase;
    int64_t input_token_ids_stride1;
    int64_t out_token_ids_stride0;
    int64_t cache_offsets_stride;
    int64_t time_dim_sizes_stride;
    int64_t user_phase_stride;
    int32_t B;
} g4b_advance_args;

int g4b_advance_decode_state(const g4b_advance_args* args, void* stream);

/*
 * g4b_rope replaces apply_rope() (g4b/kernels/rope.py:123-243): for x in (q, k), in place,
 *   x[b,h,t,:] <- rope(x[b,h,t,:] * rsqrt(x_rsos[b,h,t] / D + eps) * x_rmsnorm_w[:], theta[b,t,:])
 *   theta[b,t,j] = (time_dim_offsets[b] + t) * rope_freqs[j]  (fp32),  j < D/2
 *   rope(x)[j] = cos*x[j] - sin*x[j + D/2];   rope(x)[j + D/2] = cos*x[j + D/2] + sin*x[j]
 * on every slot (the reference's kernel has no phase skip).  With k_cache non-NULL the same launch also
 * does the two add_kv_to_cache() calls that follow it in the engine (g4b/models/gemma4e.py:575-590):
 *   k_cache[b, g, (t + time_dim_offsets[b]) % T, :] = rotated k[b,g,t,:]
 *   v_cache[b, g, (t + time_dim_offsets[b]) % T, :] = v[b,g,t,:] * (v_rsos ? rsqrt(v_rsos[b,g,t] / Dv + eps) : 1)
 * for slots with user_phase[b] == phase (all slots when user_phase is NULL); the rotated k is then written
 * back to k only if k_writeback != 0 (nothing in the engine reads it after the append).
 *   q [B,H,t,D], k [B,G,t,D], v [B,G,t,Dv]: strided, last stride 1, f16/bf16/f32; rope_freqs [D/2] f32;
 *   time_dim_offsets [B] int32; *_rsos [B,heads,t] f32 strided; *_rmsnorm_w [D] f32; caches [B,G,T,D(v)]
 *   contiguous inside a slot, f16/bf16/f32; D and Dv multiples of 16; t <= T.
 */
typedef struct g4b_rope_args {
    void* q;
    void* k;
    const float* rope_freqs;
    const int32_t* time_dim_offsets;
    const float* q_rsos;
    const float* k_rsos;
    const float* q_rmsnorm_w;
    const float* k_rmsnorm_w;
    const void* v;
    const float* v_rsos;
    void* k_cache;
    void* v_cache;
    const uint8_t* user_phase;
    int64_t q_stride[4];
    int64_t k_stride[4];
    int64_t v_stride[4];
    int64_t q_rsos_stride[3];
    int64_t k_rsos_stride[3];
    int64_t v_rsos_stride[3];
    int64_t rope_freqs_stride;
    int64_t q_rmsnorm_w_stride;
    int64_t k_rmsnorm_w_stride;
    int64_t time_dim_offsets_stride;
    int64_t user_phase_stride;
    int64_t k_cache_stride_b;
    int64_t v_cache_stride_b;
    int32_t q_dtype;
    int32_t k_dtype;
    int32_t v_dtype;
    int32_t cache_dtype;
    int32_t B, H, G, t, D, Dv, T;
    int32_t phase;
    int32_t k_writeback;
    float rmsnorm_eps;
} g4b_rope_args;

int g4b_rope(const g4b_rope_args* args, void* stream);

/*
 * g4b_rope_frequencies replaces populate_rope_frequencies() (g4b/kernels/rope.py:262-293), run once at load:
 *   out[j] = 1 / freq_base ** (j / n)  [/ freq_scalars[j]],  j < n;  out and freq_scalars are f32 device arrays.
 */
int g4b_rope_frequencies(float* out, const float* freq_scalars, int32_t n, int64_t out_stride,
                         int64_t freq_scalars_stride, float freq_base, void* stream);

/*
 * Profiling aid, no counterpart in the reference.  Between g4b_profile_begin() and g4b_profile_end() every
 * g4b_attn_forward and g4b_rope call of the calling thread has its dominant kernel (the streaming worker, the prefill
 * kernel, the rope kernel) dispatched with a pair of events that the runtime stamps with the begin and the end of that
 * dispatch: the kernel's own duration, as a kernel trace reports it, without the launch gaps an event pair recorded
 * around the call would include.  g4b_profile_end waits for the timed kernels, writes up to `capacity` durations in
 * milliseconds in call order (-1 for a call whose dominant kernel was masked out) and returns the number of timed
 * calls, or a negative g4b_status.  Events are created per call, so this is not for graph capture.
 */
int g4b_profile_begin(void);
int g4b_profile_end(float* ms, int32_t capacity);

/* Message of the calling thread's last failed call ("" if none). */
const char* g4b_last_error(void);

/* G4B_ATTN_ABI_VERSION the library was built with. */
int32_t g4b_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* G4B_ATTN_H */
