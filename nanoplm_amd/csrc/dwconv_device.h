// Device-side building blocks of the varlen depthwise conv kernels (gfx950, wave64).
//
//  - RowVec<BF16, VEC>: one lane's slice of a token row (VEC adjacent channels) in its memory
//    format, with the widest load/store the slice allows (16 B for 8 bf16 / 4 fp32).
//  - SeqCursor: wave-uniform cursor over cu_seqlens; tells which [cs, ce) interval a row is in.
//
// The reference (peymanvahidi/nanoplm 0.1.6) has no counterpart: its packed path carries
// (total_tokens, hidden) activations and int32 cu_seqlens
// (src/nanoplm/pretraining/models/modern_bert/modeling.py:339, collator.py:322-325), which is the
// layout these helpers address.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nplm {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Two fp32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2 v = {lo, hi};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    __bf16 r = (__bf16)f;
    return __builtin_bit_cast(uint16_t, r);
}

// SwiGLU gate of the reference MLP (modeling.py:300-302: F.silu(gate) * x_proj), in fp32:
// sig = 1 / (1 + 2^(-g log2 e)); h = u * g * sig. Also what the backward needs of it.
__device__ __forceinline__ float sigmoid_f32(float g) {
    return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896341f * g));
}
__device__ __forceinline__ float gate_mul(float u, float g) { return u * g * sigmoid_f32(g); }

// ---------------------------------------------------------------------------------------------
// Buffer addressing. Row slices are moved with MUBUF instructions: address = descriptor base +
// scalar byte offset (the row, wave-uniform) + per-lane byte offset (the channel slice, constant for
// the whole kernel), so no vector ALU work goes into address arithmetic.
// ---------------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Raw (untyped, stride 0) buffer descriptor over `bytes` bytes at `base`; 0x00020000 = 32-bit data
// format word of gfx9-family descriptors.
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
// Descriptor over rows [row0, T) of a [T, row_bytes] tensor (capped at 4 GiB - 1).
__device__ __forceinline__ rsrc_t rows_rsrc(const void* tensor, int row0, int T, size_t row_bytes) {
    const size_t rem = (size_t)(T - row0) * row_bytes;
    const uint32_t n = rem > 0xffffffffull ? 0xffffffffu : (uint32_t)rem;
    return make_rsrc(reinterpret_cast<const char*>(tensor) + (size_t)row0 * row_bytes, n);
}

// Cache policy of the activation streams: the aux operand of the MUBUF builtins on gfx950 (bit 0 = sc0,
// bit 1 = nt, bit 4 = sc1). x, dy, y and dx are each touched once per call, plus the K-1 halo rows a
// neighbouring tile re-reads within the same round of tiles. Measured on MI355X at T=131072, C=1024, K=7, bf16
// (wall-clock forward+backward step on tensors no earlier kernel left in a cache; 244.8 us with no hints):
//   stores of y and dx non-temporal                      235.3 us (forward 95.0 -> 90.0, backward+finalize 149.5 -> 146.2)
//   + backward loads of rows only one tile reads, nt     234.8 us (backward+finalize 144.0); the Infinity Cache is then
//                                                         left to other tensors (with x still cached from the forward
//                                                         of the same step: 223.7 us)
//   backward x loads nt but dy loads plain               240.0 us
//   forward loads nt (all rows, or all but halo rows)    257.0 / 239.9 us: the forward slows from 90 to 100-103 us
//   sc0/sc1 variants of either                           no better than nt alone (235.2 - 237.7 us)
// The defaults below are the second line. (A plain copy kernel gains more from nt loads: 5.73 -> 6.27 TB/s.)
#ifndef NPLM_LOAD_AUX
#define NPLM_LOAD_AUX 0            // rows a neighbouring tile stages as well, and every load of the forward
#endif
#ifndef NPLM_LOAD_AUX_ONCE_FWD
#define NPLM_LOAD_AUX_ONCE_FWD NPLM_LOAD_AUX
#endif
#ifndef NPLM_LOAD_AUX_ONCE_BWD
#define NPLM_LOAD_AUX_ONCE_BWD 2   // nt
#endif
#ifndef NPLM_LOAD_AUX_ONCE_BWDX
#define NPLM_LOAD_AUX_ONCE_BWDX NPLM_LOAD_AUX_ONCE_BWD
#endif
#ifndef NPLM_STORE_AUX
#define NPLM_STORE_AUX 2           // nt
#endif
constexpr int kLoadAux = NPLM_LOAD_AUX;
constexpr int kLoadAuxOnceFwd = NPLM_LOAD_AUX_ONCE_FWD;   // LDS-staged forward: x rows only one tile reads
constexpr int kLoadAuxOnceBwd = NPLM_LOAD_AUX_ONCE_BWD;   // LDS-staged backward: dy rows only one tile reads
constexpr int kLoadAuxOnceBwdX = NPLM_LOAD_AUX_ONCE_BWDX; // LDS-staged backward: x rows (no halo)
constexpr int kStoreAux = NPLM_STORE_AUX;

// ---------------------------------------------------------------------------------------------
// RowVec: VEC adjacent channels of one row, as stored in memory.
// ---------------------------------------------------------------------------------------------
template <bool BF16, int VEC> struct RowVec;

// bf16, VEC even: VEC/2 dwords
template <int VEC> struct RowVec<true, VEC> {
    static_assert(VEC == 2 || VEC == 4 || VEC == 8, "bf16 VEC");
    static constexpr int NDW = VEC / 2;
    static constexpr int BYTES = VEC * 2;
    uint32_t d[NDW];
    __device__ __forceinline__ void load(const char* p) {
        if constexpr (NDW == 4) { uint4 t = *reinterpret_cast<const uint4*>(p); d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w; }
        else if constexpr (NDW == 2) { uint2 t = *reinterpret_cast<const uint2*>(p); d[0] = t.x; d[1] = t.y; }
        else { d[0] = *reinterpret_cast<const uint32_t*>(p); }
    }
    __device__ __forceinline__ void store(char* p) const {
        if constexpr (NDW == 4) { *reinterpret_cast<uint4*>(p) = make_uint4(d[0], d[1], d[2], d[3]); }
        else if constexpr (NDW == 2) { *reinterpret_cast<uint2*>(p) = make_uint2(d[0], d[1]); }
        else { *reinterpret_cast<uint32_t*>(p) = d[0]; }
    }
    __device__ __forceinline__ void bload(rsrc_t r, int voff, int soff) {
        if constexpr (NDW == 4) { u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, kLoadAux); d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w; }
        else if constexpr (NDW == 2) { u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, kLoadAux); d[0] = t.x; d[1] = t.y; }
        else { d[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, kLoadAux); }
    }
    __device__ __forceinline__ void bstore(rsrc_t r, int voff, int soff) const {
        if constexpr (NDW == 4) { u32x4 t = {d[0], d[1], d[2], d[3]}; __builtin_amdgcn_raw_buffer_store_b128(t, r, voff, soff, kStoreAux); }
        else if constexpr (NDW == 2) { u32x2 t = {d[0], d[1]}; __builtin_amdgcn_raw_buffer_store_b64(t, r, voff, soff, kStoreAux); }
        else { __builtin_amdgcn_raw_buffer_store_b32(d[0], r, voff, soff, kStoreAux); }
    }
    __device__ __forceinline__ void to_f32(float (&f)[VEC]) const {
#pragma unroll
        for (int i = 0; i < NDW; ++i) { f[2 * i] = bf16_lo(d[i]); f[2 * i + 1] = bf16_hi(d[i]); }
    }
    __device__ __forceinline__ void from_f32(const float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < NDW; ++i) d[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
    }
};
template <> struct RowVec<true, 1> {
    static constexpr int BYTES = 2;
    uint16_t h;
    __device__ __forceinline__ void load(const char* p) { h = *reinterpret_cast<const uint16_t*>(p); }
    __device__ __forceinline__ void store(char* p) const { *reinterpret_cast<uint16_t*>(p) = h; }
    __device__ __forceinline__ void bload(rsrc_t r, int voff, int soff) { h = __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, kLoadAux); }
    __device__ __forceinline__ void bstore(rsrc_t r, int voff, int soff) const { __builtin_amdgcn_raw_buffer_store_b16(h, r, voff, soff, kStoreAux); }
    __device__ __forceinline__ void to_f32(float (&f)[1]) const { f[0] = bf16_to_f32(h); }
    __device__ __forceinline__ void from_f32(const float (&f)[1]) { h = f32_to_bf16(f[0]); }
};
// fp32
template <int VEC> struct RowVec<false, VEC> {
    static_assert(VEC == 1 || VEC == 2 || VEC == 4, "fp32 VEC");
    static constexpr int BYTES = VEC * 4;
    float v[VEC];
    __device__ __forceinline__ void load(const char* p) {
        if constexpr (VEC == 4) { float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
        else if constexpr (VEC == 2) { float2 t = *reinterpret_cast<const float2*>(p); v[0] = t.x; v[1] = t.y; }
        else { v[0] = *reinterpret_cast<const float*>(p); }
    }
    __device__ __forceinline__ void store(char* p) const {
        if constexpr (VEC == 4) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
        else if constexpr (VEC == 2) { *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]); }
        else { *reinterpret_cast<float*>(p) = v[0]; }
    }
    __device__ __forceinline__ void bload(rsrc_t r, int voff, int soff) {
        if constexpr (VEC == 4) { u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, kLoadAux); v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y); v[2] = __uint_as_float(t.z); v[3] = __uint_as_float(t.w); }
        else if constexpr (VEC == 2) { u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, kLoadAux); v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y); }
        else { v[0] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, kLoadAux)); }
    }
    __device__ __forceinline__ void bstore(rsrc_t r, int voff, int soff) const {
        if constexpr (VEC == 4) { u32x4 t = {__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])}; __builtin_amdgcn_raw_buffer_store_b128(t, r, voff, soff, kStoreAux); }
        else if constexpr (VEC == 2) { u32x2 t = {__float_as_uint(v[0]), __float_as_uint(v[1])}; __builtin_amdgcn_raw_buffer_store_b64(t, r, voff, soff, kStoreAux); }
        else { __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v[0]), r, voff, soff, kStoreAux); }
    }
    __device__ __forceinline__ void to_f32(float (&f)[VEC]) const {
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = v[i];
    }
    __device__ __forceinline__ void from_f32(const float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = f[i];
    }
};

// ---------------------------------------------------------------------------------------------
// SeqCursor: which sequence interval [cs, ce) holds row t. Every member is wave-uniform (the
// callers derive t from blockIdx and a readfirstlane'd wave index), so the compiler keeps the
// cursor in scalar registers and reads cu through the scalar (read-only) data path.
//
// cu is used ONLY to mask taps, never to form an address, so a malformed cu cannot make the
// kernels read or write out of bounds. Rows below cu[0] or at/after cu[S] fall into one extra
// pseudo-sequence on that side.
// ---------------------------------------------------------------------------------------------
// One entry of cu as a scalar: on the device the value is forced into a scalar register, which keeps
// the whole cursor (and every comparison against it) off the vector ALU.
__host__ __device__ __forceinline__ int cu_at(const int32_t* __restrict__ cu, int i) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_readfirstlane(cu[i]);
#else
    return cu[i];
#endif
}

// cu read through scalar loads (s_load_dword, counted by lgkmcnt). What the compiler makes of cu_at() above is a vector
// load followed by v_readfirstlane whenever it cannot prove that nothing stored in the kernel aliases cu, and a wave
// that waits for that load (vmcnt) also waits for every direct global->LDS load and every store it has in flight.
// Kernels whose waves keep such operations in flight across their boundary lookups pass cu wrapped in this type.
struct ScalarCu {
    const int32_t* p;
};
__host__ __device__ __forceinline__ int cu_at(ScalarCu c, int i) {
#if defined(__HIP_DEVICE_COMPILE__)
    int v;
    const int32_t* a = c.p + i;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(a) : "memory");
    return v;
#else
    return c.p[i];
#endif
}

struct SeqCursor {
    int seq;  // index of the current interval; -1 / S for the pseudo-sequences at either end
    int cs;   // first row of the interval
    int ce;   // one past the last row

    // Position on the interval containing row t, searching cu[hint..S].
    template <typename CU>
    __host__ __device__ __forceinline__ void locate(CU cu, int S, int T, int t, int hint) {
        int lo = hint < 0 ? 0 : hint, hi = S;
        // first i in [lo, S) with cu[i+1] > t, else S
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (cu_at(cu, mid + 1) > t) hi = mid; else lo = mid + 1;
        }
        seq = lo;
        if (lo < S) { cs = cu_at(cu, lo); ce = cu_at(cu, lo + 1); }
        else        { cs = cu_at(cu, S);  ce = T; }
        if (cs > t) { ce = cs; cs = 0; seq = -1; }   // row lies before cu[0]
    }
    // Move forward until the interval contains row t (t must not decrease between calls).
    template <typename CU>
    __host__ __device__ __forceinline__ void advance(CU cu, int S, int T, int t) {
        while (t >= ce && seq < S) {
            ++seq;
            cs = ce;
            ce = (seq < S) ? cu_at(cu, seq + 1) : T;
        }
    }
};

// Which of the K taps of output row t stay inside the cursor's interval: bit m is set iff row
// t - P + m lies in [cs, ce). One scalar word (K <= 32) per row instead of two compares per tap;
// the kernels test its bits with scalar instructions and select, never multiply by zero.
template <int K>
__device__ __forceinline__ uint32_t row_tap_mask(const SeqCursor& sc, int t) {
    static_assert(K <= 32, "one mask bit per tap");
    constexpr int P = (K - 1) / 2;
    int lo = sc.cs - (t - P), hi = sc.ce - (t - P);     // valid taps: lo <= m < hi
    lo = lo < 0 ? 0 : lo;
    hi = hi > K ? K : hi;
    const uint32_t m = hi > lo ? (uint32_t)(((1ull << hi) - 1ull) & ~((1ull << lo) - 1ull)) : 0u;
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)m);
#else
    return m;
#endif
}

}  // namespace nplm
