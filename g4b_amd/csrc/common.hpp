// Shared device helpers for the gfx950 attention kernels: vector types, MFMA wrappers for
// fp16 / bf16 operands, 16-byte global loads, wave64 cross-lane primitives, and the per-slot
// window arithmetic every kernel evaluates the same way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace g4b {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

enum : int { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2 };
enum : int { STAGE_FULL = 1, STAGE_ON_BAND = 2, STAGE_CAUSAL = 3 };

#define G4B_DEV __device__ __forceinline__

// ---- element types of the KV cache (and of the MFMA operands) ---------------------------------
struct F16 {
    static constexpr int dt = DT_F16;
    static G4B_DEV f4 mfma16(u4 a, u4 b, f4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    }
    static G4B_DEV f16v mfma32(u4 a, u4 b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    }
    static G4B_DEV uint32_t pack2(float lo, float hi) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    // acc + both halves of a packed pair, accumulated in fp32 (v_dot2_f32_f16 against (1, 1))
    static G4B_DEV float sum2(uint32_t w, float acc) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w), ones, acc, false);
    }
    static G4B_DEV float lo(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)); }
    static G4B_DEV float hi(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }
};

struct BF16 {
    static constexpr int dt = DT_BF16;
    static G4B_DEV f4 mfma16(u4 a, u4 b, f4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    }
    static G4B_DEV f16v mfma32(u4 a, u4 b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    }
    static G4B_DEV uint32_t pack2(float lo, float hi) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        b2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static G4B_DEV float sum2(uint32_t w, float acc) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        const b2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, w), ones, acc, false);
    }
    static G4B_DEV float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static G4B_DEV float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
};

// ---- memory ----------------------------------------------------------------------------------
G4B_DEV u4 ld16(const void* base, uint32_t byte_off) {
    return *reinterpret_cast<const u4*>(static_cast<const char*>(base) + byte_off);
}
// The same load marked non-temporal: the line is read once (a KV stream) and need not stay in the caches.
G4B_DEV u4 ld16_stream(const void* base, uint32_t byte_off) {
    return __builtin_nontemporal_load(reinterpret_cast<const u4*>(static_cast<const char*>(base) + byte_off));
}
G4B_DEV u4 ld16(const void* base, int64_t byte_off) {
    return *reinterpret_cast<const u4*>(static_cast<const char*>(base) + byte_off);
}

// A vector load / store that is marked non-temporal when NT: data touched once (scratchpads read by one pass, a KV
// stream) then passes through the caches without displacing what others re-read.
template <bool NT, class V>
G4B_DEV V ld_vec(const V* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}
template <bool NT, class V>
G4B_DEV void st_vec(V* p, V v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// Eight consecutive elements of a q/x row (dtype chosen at run time) as eight MFMA operand
// elements of type T, optionally pre-multiplied.
template <class T, bool NT = false>
G4B_DEV u4 load8_as(const void* base, int64_t elem_off, int dt) {
    if (dt == DT_F32) {
        const f4* p = reinterpret_cast<const f4*>(static_cast<const float*>(base) + elem_off);
        f4 a = ld_vec<NT>(p), b = ld_vec<NT>(p + 1);
        u4 r = {T::pack2(a[0], a[1]), T::pack2(a[2], a[3]), T::pack2(b[0], b[1]), T::pack2(b[2], b[3])};
        return r;
    }
    u4 raw = ld_vec<NT>(reinterpret_cast<const u4*>(static_cast<const uint16_t*>(base) + elem_off));
    if (dt == T::dt) return raw;
    u4 r;
    if (dt == DT_F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = T::pack2(F16::lo(raw[i]), F16::hi(raw[i]));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = T::pack2(BF16::lo(raw[i]), BF16::hi(raw[i]));
    }
    return r;
}

// The same eight elements as a pair of operands hi + lo: hi is the value rounded to T, lo the rounding error rounded
// to T again, so that K.hi + K.lo reproduces the product with the unrounded query to about twice T's mantissa.  For a
// source type that T holds exactly lo is zero.
template <class T>
G4B_DEV void load8_split(const void* base, int64_t elem_off, int dt, u4& hi, u4& lo) {
    float x[8];
    if (dt == DT_F32) {
        const f4* p = reinterpret_cast<const f4*>(static_cast<const float*>(base) + elem_off);
        const f4 a = p[0], b = p[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[i] = a[i];
            x[4 + i] = b[i];
        }
    } else {
        const u4 raw = *reinterpret_cast<const u4*>(static_cast<const uint16_t*>(base) + elem_off);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = raw[i];
            x[2 * i] = (dt == DT_F16) ? F16::lo(w) : BF16::lo(w);
            x[2 * i + 1] = (dt == DT_F16) ? F16::hi(w) : BF16::hi(w);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t h = T::pack2(x[2 * i], x[2 * i + 1]);
        hi[i] = h;
        lo[i] = T::pack2(x[2 * i] - T::lo(h), x[2 * i + 1] - T::hi(h));
    }
}

// Store eight consecutive output elements (dtype chosen at run time) from eight floats.
template <bool NT = false>
G4B_DEV void store8(void* base, int64_t elem_off, int dt, const float (&v)[8]) {
    if (dt == DT_F32) {
        f4* p = reinterpret_cast<f4*>(static_cast<float*>(base) + elem_off);
        f4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
        st_vec<NT>(p, a);
        st_vec<NT>(p + 1, b);
    } else if (dt == DT_F16) {
        u4 r = {F16::pack2(v[0], v[1]), F16::pack2(v[2], v[3]), F16::pack2(v[4], v[5]), F16::pack2(v[6], v[7])};
        st_vec<NT>(reinterpret_cast<u4*>(static_cast<uint16_t*>(base) + elem_off), r);
    } else {
        u4 r = {BF16::pack2(v[0], v[1]), BF16::pack2(v[2], v[3]), BF16::pack2(v[4], v[5]), BF16::pack2(v[6], v[7])};
        st_vec<NT>(reinterpret_cast<u4*>(static_cast<uint16_t*>(base) + elem_off), r);
    }
}

template <bool NT = false>
G4B_DEV void store4(void* base, int64_t elem_off, int dt, f4 v) {
    if (dt == DT_F32) {
        st_vec<NT>(reinterpret_cast<f4*>(static_cast<float*>(base) + elem_off), v);
    } else if (dt == DT_F16) {
        u2 r = {F16::pack2(v[0], v[1]), F16::pack2(v[2], v[3])};
        st_vec<NT>(reinterpret_cast<u2*>(static_cast<uint16_t*>(base) + elem_off), r);
    } else {
        u2 r = {BF16::pack2(v[0], v[1]), BF16::pack2(v[2], v[3])};
        st_vec<NT>(reinterpret_cast<u2*>(static_cast<uint16_t*>(base) + elem_off), r);
    }
}

// N consecutive elements (4 or 8; dtype chosen at run time) as floats: one 16-byte load per four fp32 values or eight
// 16-bit ones, so that the lanes of a wave read one contiguous run.
template <int N, bool NT = false>
G4B_DEV void load_f32(const void* base, int64_t elem_off, int dt, float (&v)[N]) {
    static_assert(N == 4 || N == 8, "4 or 8 elements");
    if (dt == DT_F32) {
        const f4* src = reinterpret_cast<const f4*>(static_cast<const float*>(base) + elem_off);
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            const f4 a = ld_vec<NT>(src + q);
#pragma unroll
            for (int i = 0; i < 4; ++i) v[4 * q + i] = a[i];
        }
    } else {
        uint32_t raw[N / 2];
        if constexpr (N == 8) {
            const u4 r = ld_vec<NT>(reinterpret_cast<const u4*>(static_cast<const uint16_t*>(base) + elem_off));
#pragma unroll
            for (int i = 0; i < 4; ++i) raw[i] = r[i];
        } else {
            const u2 r = ld_vec<NT>(reinterpret_cast<const u2*>(static_cast<const uint16_t*>(base) + elem_off));
            raw[0] = r[0];
            raw[1] = r[1];
        }
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            v[2 * i] = dt == DT_F16 ? F16::lo(raw[i]) : BF16::lo(raw[i]);
            v[2 * i + 1] = dt == DT_F16 ? F16::hi(raw[i]) : BF16::hi(raw[i]);
        }
    }
}
template <int N, bool NT = false>
G4B_DEV void store_n(void* base, int64_t elem_off, int dt, const float (&v)[N]) {
    if constexpr (N == 8) {
        store8<NT>(base, elem_off, dt, v);
    } else {
        const f4 x = {v[0], v[1], v[2], v[3]};
        store4<NT>(base, elem_off, dt, x);
    }
}

// ---- wave64 cross-lane -----------------------------------------------------------------------
template <int CTRL>
G4B_DEV float dpp_f(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
G4B_DEV float quad_xor1(float x) { return dpp_f<0xB1>(x); }  // quad_perm [1,0,3,2]
G4B_DEV float quad_xor2(float x) { return dpp_f<0x4E>(x); }  // quad_perm [2,3,0,1]

// Sum over the wave, in every lane, and inclusive prefix sum over the lanes.  Both stay in the vector ALU (DPP inside
// the rows of 16 lanes, then lane reads / row broadcasts across them): six dependent shuffles through the LDS crossbar
// were 0.3 us each at the head of every decode worker and merge workgroup.
template <int CTRL, int ROW_MASK = 0xf>
G4B_DEV int dpp_i0(int x) {  // lanes the pattern leaves without a source, or masks out, read 0
    return __builtin_amdgcn_update_dpp(0, x, CTRL, ROW_MASK, 0xf, false);
}
G4B_DEV int wave_sum_i(int v) {
    v += dpp_i0<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_i0<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_i0<0x141>(v);  // row_half_mirror
    v += dpp_i0<0x140>(v);  // row_mirror: every lane holds its row's sum
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
           __builtin_amdgcn_readlane(v, 48);
}
G4B_DEV int wave_incl_scan_i(int v, int /*lane*/) {
    v += dpp_i0<0x111>(v);       // row_shr:1
    v += dpp_i0<0x112>(v);       // row_shr:2
    v += dpp_i0<0x114>(v);       // row_shr:4
    v += dpp_i0<0x118>(v);       // row_shr:8: inclusive inside every row
    v += dpp_i0<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_i0<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}
// max / sum over the lanes l, l ^ 16: v_permlane16_swap exchanges the odd rows of its first operand with the even rows
// of its second, so that of the two results one is the lane's own value and the other its partner's.
G4B_DEV float row_swap_max(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
G4B_DEV float row_swap_sum(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

G4B_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max / sum over the lane pair (l, l ^ 32) without going through LDS: v_permlane32_swap exchanges the upper half
// of its first operand with the lower half of its second, leaving (low half, low half) and (high half, high half).
// The two results are copied into scalars before the bit casts: __builtin_bit_cast applied directly to an element of
// an ext_vector reads element 0 whatever the index.
G4B_DEV float half_swap_max(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
G4B_DEV float half_swap_sum(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    const u2 r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

// 16-byte LDS read issued where it is written (volatile asm), to be retired by lds_wait_pair<n> on the same value.
G4B_DEV u4 lds_read16(uint32_t lds_addr, int imm) {
    u4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(imm));
    return v;
}
// 16 bytes per lane from global memory straight into LDS: lane l lands at M0 + IMM + 16 * l and comes from
// scalar base + per-lane 32-bit offset + IMM (the instruction offset moves both ends; 0 <= IMM < 4096).  Completion
// is tracked by vmcnt.  dma_set_base loads M0; one base serves the loads that follow it until the next dma_set_base
// (nothing else in these kernels touches M0).
G4B_DEV void dma_set_base(uint32_t lds_base) { asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(lds_base) : "m0"); }
template <int IMM>
G4B_DEV void dma16_to_lds_at(const void* sbase, uint32_t voff) {
    static_assert(IMM >= 0 && IMM < 4096, "13-bit signed instruction offset");
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(voff), "s"(sbase), "n"(IMM) : "memory");
}
G4B_DEV void vm_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Transposing 8-byte LDS read of 16-bit elements (issued where it is written, retire with lds_wait4<n>).
// Inside every group of 16 lanes, lane s supplies the address of 4 consecutive elements E[s][0..3]; lane i receives
// E[i/4][i%4], E[4 + i/4][i%4], E[8 + i/4][i%4], E[12 + i/4][i%4].  With lane 4r+q pointing at columns 4q..4q+3 of row r
// of a 4 x 16 block, lane i receives column i of the four rows.
G4B_DEV u2 lds_read8_tr16(uint32_t lds_addr, int imm) {
    u2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(imm));
    return v;
}
// Wait until at most N LDS operations are outstanding; the values are tied so their consumers stay behind the wait.
template <int N>
G4B_DEV void lds_wait4(u2& a, u2& b, u2& c, u2& d) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N>
G4B_DEV void lds_wait_pair(u4& a, u4& b) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

// In-lane 8x8 transpose of 16-bit elements.  in[s] holds elements (s, 0..7); out[j] holds (0..7, j).
G4B_DEV void transpose8x8_b16(const u4 (&in)[8], u4 (&out)[8]) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t a = in[2 * t][w], b = in[2 * t + 1][w];
            out[2 * w][t] = __builtin_amdgcn_perm(b, a, 0x05040100u);      // low halves:  a.lo | b.lo << 16
            out[2 * w + 1][t] = __builtin_amdgcn_perm(b, a, 0x07060302u);  // high halves: a.hi | b.hi << 16
        }
    }
}

// ---- launch parameters shared by the attention kernels -----------------------------------------
struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const int32_t* tds;
    const uint8_t* phase_arr;
    const int32_t* win_arr;  // optional per-slot window sizes
    float* part_o;           // split partials.  Decode: [slot][row][D] un-normalised fp32; prefill: [slot][row][D] in the
                             // cache's 16-bit type, every row normalised by its own running sum
    float* part_ml;          // [slot][row][2] = (running max in log2 units, running sum)
    int64_t q_s[4], o_s[4];  // element strides of q and o ([B,H,Tq,D])
    int64_t k_sb, v_sb;      // batch strides of the caches (elements)
    int64_t tds_s, ph_s, win_s;
    int32_t q_dt, o_dt;
    int32_t B, H, G, R, Tq, KV_CTX;
    int32_t W, phase, stage, qwin;
    int32_t NW;  // number of decode workers (waves) the key tiles are dealt to
    int32_t split_slots;  // prefill: (active slot, key split) pairs the partial buffers hold; <= 1 = never split
    int32_t kernel_mask;  // bit 0: main kernel, bit 1: merge kernel
    int32_t q_split;      // 1: a query wider than the cache type enters K Q^T as a hi + lo pair of operands
    int32_t pair_split;   // 1: a prefill launch that splits keys still pairs query tiles (prefill_map.hpp)
    int32_t xcd_shift;    // decode workers: bit (worker >> xcd_shift) & 1 is the parity of the XCD the worker runs on;
                          // < 0: unknown, every worker gets the same share of the tiles
    float c;     // softmax scale * log2(e)
};

// What an attention launch reads of one slot.  window = min(tds, W) keys ending at the newest
// token; logical key j sits in ring row (ring_start + j) mod KV_CTX; query i is aligned with
// logical key qb + i.  [klo, window) is the union of the key ranges of all queries of the launch.
struct SlotInfo {
    int window, ring_start, qb, klo;
    bool active;
};

G4B_DEV SlotInfo slot_info(const AttnParams& p, int b) {
    SlotInfo s;
    s.active = p.phase_arr[(int64_t)b * p.ph_s] == (uint8_t)p.phase;
    int tds = p.tds[(int64_t)b * p.tds_s];
    int W = p.win_arr ? p.win_arr[(int64_t)b * p.win_s] : p.W;
    W = min(max(W, 0), p.KV_CTX);
    tds = max(tds, 0);
    s.window = s.active ? min(tds, W) : 0;
    int base = tds - min(tds, W);
    s.ring_start = base % p.KV_CTX;
    s.qb = s.window - p.Tq;
    int klo = 0;
    if (p.qwin > 0) klo = min(max(0, s.qb - p.qwin + 1), s.window);
    s.klo = klo;
    return s;
}

// What lane `src` of the wave holds, for every lane (src must be the same in all of them: a lane read, not a shuffle).
G4B_DEV SlotInfo slot_info_of_lane(const SlotInfo& s, int src) {
    SlotInfo r;
    r.window = __builtin_amdgcn_readlane(s.window, src);
    r.ring_start = __builtin_amdgcn_readlane(s.ring_start, src);
    r.qb = __builtin_amdgcn_readlane(s.qb, src);
    r.klo = __builtin_amdgcn_readlane(s.klo, src);
    r.active = __builtin_amdgcn_readlane((int)s.active, src) != 0;
    return r;
}
// Number of slots whose phase matches the launch (n_active) and the index of the a-th of them (-1 when a is out of
// range).  Every thread of a workgroup of NWAVES waves must call it; sh is workgroup-shared scratch of at least
// NWAVES + 1 ints.  Call it with a < 0 to count only.
template <int NWAVES>
G4B_DEV int nth_active_slot_t(const AttnParams& p, int a, int& n_active, int* sh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (p.B <= 64) {  // one ballot per wave answers both questions, no exchange between waves
        const bool act = lane < p.B && p.phase_arr[(int64_t)lane * p.ph_s] == (uint8_t)p.phase;
        const unsigned long long m = __ballot(act);
        n_active = __popcll(m);
        if (a < 0 || a >= n_active) return -1;
        const unsigned long long hit = __ballot(act && __popcll(m & ((1ull << lane) - 1ull)) == a);
        return __ffsll((long long)hit) - 1;
    }
    int base = 0;
    for (int c0 = 0; c0 < p.B; c0 += 64 * NWAVES) {
        const int b = c0 + tid;
        const bool act = b < p.B && p.phase_arr[(int64_t)b * p.ph_s] == (uint8_t)p.phase;
        const unsigned long long m = __ballot(act);
        if (lane == 0) sh[wave] = __popcll(m);
        __syncthreads();
        int before = base;
        for (int w = 0; w < wave; ++w) before += sh[w];
        int total = 0;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) total += sh[w];
        const int rank = before + __popcll(m & ((1ull << lane) - 1ull));
        if (act && rank == a) sh[NWAVES] = b;
        base += total;
        __syncthreads();
    }
    n_active = base;
    return (a >= 0 && a < base) ? sh[NWAVES] : -1;
}
G4B_DEV int nth_active_slot(const AttnParams& p, int a, int& n_active, int* sh) { return nth_active_slot_t<4>(p, a, n_active, sh); }


// Key splits per active slot of a prefill-shaped launch: the partial buffers hold split_slots (slot, split) pairs.
__host__ __device__ inline int prefill_splits(int split_slots, int n_active) {
    if (n_active < 1 || split_slots < 2 * n_active) return 1;
    const int s = split_slots / n_active;
    return s < 16 ? s : 16;
}

// Visible logical key range [lo, hi) of query i of a slot.
G4B_DEV void row_range(const AttnParams& p, const SlotInfo& s, int i, int& lo, int& hi) {
    int qp = s.qb + i;
    hi = (p.stage == STAGE_FULL) ? s.window : min(s.window, qp + 1);
    lo = (p.qwin > 0) ? max(0, qp - p.qwin + 1) : 0;
}

}  // namespace g4b
