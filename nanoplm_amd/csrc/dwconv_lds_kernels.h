// LDS-staged, software-pipelined kernels of the varlen depthwise conv (gfx950, wave64): both passes
// for K <= 9, the forward also for K = 15 and 31.
//
// A block owns tiles of R = RW*NRG consecutive token rows x one column block of NCW*64*VEC channels
// (1 KiB of every row of a 32-row tile at the default sizes). Its waves have two roles:
//
//   loader waves (NWL)   issue direct global->LDS loads (buffer_load ... lds, 16 B per lane,
//                        consecutive lanes consecutive addresses) for the NEXT tile and its K-1 halo
//                        rows, then wait for them. Every row of a tile is one contiguous run in HBM
//                        and is fetched once per block; no vector registers are involved.
//   compute waves        (NCW wave-columns x NRG row groups) work on the CURRENT tile out of LDS:
//                        each reads its RW+K-1 rows once, scatters every row into the RW accumulators
//                        it contributes to, and stores RW output rows.
//
// The two tiles live in two LDS buffers; one workgroup barrier per tile hands the freshly loaded
// buffer to the compute waves and the consumed one back to the loaders, so HBM traffic and
// arithmetic overlap inside one block. Blocks walk tiles in rounds of nbt (one tile per block and
// round): all resident blocks together sweep one compact window of rows, the access pattern HBM serves fastest,
// and the halo rows a block re-reads were fetched moments earlier by its neighbour.
//
// Backward: x and dy tiles are staged the same way; dx is written per tile, dw/db stay in registers
// across all tiles of the block and are combined as in the sliding-window kernels (row groups summed
// through LDS in fixed order, one slab per token-block, then dwconv_finalize_kernel). No atomics.
//
// Sequence boundaries: the cursor lookup for the NEXT tile (a chain of dependent scalar loads) runs
// where it costs least: in the forward on the loader waves, which idle while their loads are in
// flight and post the result in a small LDS mailbox (the forward's compute waves are themselves
// memory-bound through their stores); in the backward on the compute waves right before the tile
// barrier. A wave whose rows and taps all lie in one sequence takes an unmasked path. A wave that
// touches a boundary keeps the same unrolled schedule and selects every tap by a bit of its output
// row's tap mask (K = 31: one unmasked pass per sequence over that sequence's rows); that path must
// stay close to the unmasked one in cost, because tiles are dealt to blocks statically and a block's
// time is the sum of its tiles: a slow boundary path shows up as a long tail of the grid. For the
// same reason the tile slots rotate from round to round (lds_next_slot), so that boundaries at a
// regular period do not pile up on a few blocks.
//
// Every wave of a block executes exactly the same sequence of barriers: the trip counts depend only
// on blockIdx and the launch geometry.
//
// No counterpart in the reference (peymanvahidi/nanoplm 0.1.6 has no convolution); tensor contract:
// modeling.py:339,421-439 and collator.py:322-325,405-458.
#pragma once
#include <type_traits>
#include "dwconv_kernels.h"

namespace nplm {

struct LdsGeo {
    int32_t T, C, S;
    int32_t w_flags;    // W_BF16 | W_RESIDUAL
    int32_t ntiles;     // ceil(T / R)
    int32_t ncb, nbt;   // grid = ncb column blocks x nbt token blocks (nbt <= ntiles)
    int32_t xcd_group;  // > 0: runs of this many adjacent token-blocks share an XCD (and its L2)
    int32_t rot_step;   // per-round rotation of the tile slots, 0 <= rot_step < nbt
};

// blockIdx -> (column block, token block). Hardware deals consecutive workgroups round-robin to the
// 8 XCDs, each with its own L2. With xcd_group = G, the G token-blocks b/8*... of one XCD are
// adjacent tiles of the same column block, so G-1 of every G halo re-reads hit that XCD's L2 instead
// of going out to the fabric, while the XCDs still interleave finely (every G tiles) inside the one
// window of rows the grid is sweeping. Needs nbt % G == 0 and (ncb*nbt/8) % G == 0 (host-checked).
__device__ __forceinline__ void lds_block_coords(const LdsGeo& g, int& cb, int& tb) {
    const int b = (int)blockIdx.x;
    if (g.xcd_group > 0) {
        const int G = g.xcd_group;
        const int xcd = b & 7, l = b >> 3;
        const int k = l / G, r = l - k * G;
        const int chunk = k * 8 + xcd;
        cb = chunk % g.ncb;
        tb = (chunk / g.ncb) * G + r;
    } else {
        cb = b % g.ncb;
        tb = b / g.ncb;
    }
}

// Round r of the grid covers tiles r*nbt .. r*nbt + nbt-1, and token-block tb takes slot
// (tb + r*rot_step) mod nbt of them. Tiles are dealt statically (dw/db must not depend on timing), and
// without the rotation sequence boundaries that recur at a period dividing nbt tiles (equal-length
// sequences, padded batches) would all fall to the same few blocks, whose slower boundary path then
// becomes the tail of the whole grid. Adjacent token-blocks still take adjacent tiles (modulo the
// wrap), so the XCD grouping above keeps its halo sharing. The slot is carried from round to round
// (one add and a conditional subtract; rot_step < nbt).
__device__ __forceinline__ int lds_next_slot(const LdsGeo& g, int q) {
    q += g.rot_step;
    return q >= g.nbt ? q - g.nbt : q;
}
// First row of the tile in slot q of round r; T when the slot lies past the last tile (last round
// only): the block then idles through that round.
__device__ __forceinline__ int lds_tile_row0(const LdsGeo& g, int r, int q, int R) {
    const int tile = r * g.nbt + q;
    return tile < g.ntiles ? tile * R : g.T;
}

typedef __attribute__((address_space(3))) void lds_void;

// LDS a workgroup can have, and whether the forward's boundary mailbox fits behind `tile_bytes` of tiles.
constexpr int kLdsBytes = 160 * 1024;
constexpr bool lds_mail_fits(long long tile_bytes, int mail_bytes) { return tile_bytes + mail_bytes <= kLdsBytes; }

// s_waitcnt vmcnt(0) (expcnt / lgkmcnt untouched), gfx9 encoding.
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Compile-time shape of one kernel variant.
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, int NWL>
struct LdsShape {
    static constexpr int E = BF16 ? 2 : 4;
    static constexpr int P = (K - 1) / 2;
    static constexpr int NWC = NCW * NRG;               // compute waves
    static constexpr int NT = (NWC + NWL) * 64;         // threads per block
    static constexpr int R = RW * NRG;                  // output rows per tile
    static constexpr int NROWS = R + K - 1;             // staged rows per tile
    static constexpr int CB_BYTES = NCW * 64 * VEC * E; // bytes of a row in one column block
    static constexpr int CB_CH = NCW * 64 * VEC;        // channels in one column block
    static constexpr int NPIECE = (CB_BYTES + 1023) / 1024;   // direct loads (1 KiB each, the last may be partial) per staged row
    static constexpr bool WHOLE_PIECES = CB_BYTES % 1024 == 0;
    static constexpr int TILE_BYTES = NROWS * CB_BYTES;
    static constexpr int MAIL_BYTES = 2 * NRG * 16;     // forward: two sets of one 16-byte boundary record per row group
    static_assert(CB_BYTES % 256 == 0, "a column block is a whole number of 256-byte wave-columns");
    static_assert(NROWS * CB_BYTES <= 65536, "ds_read immediate offsets are 16 bit");
};

// Loader: stage rows first_row .. first_row+nrows-1 (clamped to [0,T)) x this block's column block of
// `src` into `dst` (row pitch CB_BYTES). (row, piece) pairs are dealt round-robin to the loader waves.
// One direct global->LDS load of 16 bytes per lane; `once` picks the cache policy of rows no other tile reads.
template <int ONCE_AUX>
__device__ __forceinline__ void load_to_lds(rsrc_t rs, char* d, int voff, int so, bool once) {
    if (kLoadAux != ONCE_AUX && once) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)d, 16, voff, so, 0, ONCE_AUX);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)d, 16, voff, so, 0, kLoadAux);
}

// `edge` = number of staged rows at either end that the neighbouring tile stages too (2P for a tile with its
// K-1 halo rows, 0 for a tile without halo).
template <typename SH, int ONCE_AUX>
__device__ __forceinline__ void stage_rows(const void* __restrict__ src, char* dst, int first_row, int nrows, int T,
                                           size_t row_bytes, int col_byte0, int valid_bytes, int lw, int nlw, int lane,
                                           int edge) {
    const int rb = first_row > 0 ? first_row : 0;
    const rsrc_t rs = rows_rsrc(src, rb, T, row_bytes);
    const int rowb = (int)row_bytes;
    const int voff = lane * 16;
    for (int pair = lw; pair < nrows * SH::NPIECE; pair += nlw) {
        const int j = pair / SH::NPIECE;
        const int p = pair % SH::NPIECE;
        const int so = (clamp_row(first_row + j, T) - rb) * rowb + col_byte0 + p * 1024;
        char* d = dst + j * SH::CB_BYTES + p * 1024;
        if (p * 1024 + voff < valid_bytes) load_to_lds<ONCE_AUX>(rs, d, voff, so, j >= edge && j < nrows - edge);
    }
}

// Same as stage_rows, but every loader wave issues exactly CNT loads (surplus slots repeat the last
// pair, lanes past the end of a narrow column block re-read its last 16 bytes), so that
// "all but the newest CNT loads have landed" is a compile-time s_waitcnt. Column blocks that are not
// a whole number of 1 KiB pieces mask the lanes past the end instead (their LDS slots belong to the
// next row); a piece with no lane left is then skipped, which only the plain "wait for all" tolerates.
template <typename SH, int CNT, int ONCE_AUX>
__device__ __forceinline__ void stage_rows_fixed(const void* __restrict__ src, char* dst, int first_row, int nrows, int T,
                                                 size_t row_bytes, int col_byte0, int valid_bytes, int lw, int nlw,
                                                 int lane, int edge) {
    const int rb = first_row > 0 ? first_row : 0;
    const rsrc_t rs = rows_rsrc(src, rb, T, row_bytes);
    const int rowb = (int)row_bytes;
    const int total = nrows * SH::NPIECE;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
        int pair = lw + i * nlw;
        pair = pair < total ? pair : total - 1;
        const int j = pair / SH::NPIECE;
        const int p = pair % SH::NPIECE;
        int boff = p * 1024 + lane * 16;
        const bool inside = boff < valid_bytes;
        boff = inside ? boff : valid_bytes - 16;
        const int so = (clamp_row(first_row + j, T) - rb) * rowb + col_byte0;
        char* d = dst + j * SH::CB_BYTES + p * 1024;
        if (SH::WHOLE_PIECES || inside) load_to_lds<ONCE_AUX>(rs, d, boff, so, j >= edge && j < nrows - edge);
    }
}

// s_waitcnt vmcnt(N) for a compile-time N < 64 (gfx9 encoding: bits 3:0 and 15:14).
template <int N>
__device__ __forceinline__ void wait_vmem_but() {
    static_assert(N >= 0 && N < 64, "vmcnt is 6 bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <bool BF16, int VEC>
__device__ __forceinline__ void lds_read_row(const char* p, float (&f)[VEC]) {
    RowVec<BF16, VEC> r;
    r.load(p);
    r.to_f32(f);
}

// The same through volatile address-space-3 accesses, for waves that also issue direct global->LDS loads: before an
// ordinary LDS access the compiler waits for every outstanding vector-memory operation of the wave (it cannot tell
// which LDS bytes a direct load writes); these accesses are left alone and the kernel orders them with its barriers.
template <bool BF16, int VEC>
__device__ __forceinline__ void lds_read_pinned_row(const char* p, float (&f)[VEC]) {
    RowVec<BF16, VEC> r;
    constexpr int NDW = RowVec<BF16, VEC>::BYTES / 4;
    static_assert(RowVec<BF16, VEC>::BYTES % 4 == 0, "whole dwords");
    uint32_t t[NDW];
    if constexpr (NDW == 2) {
        const u32x2 q = *(const volatile __attribute__((address_space(3))) u32x2*)p;
        t[0] = q.x; t[1] = q.y;
    } else {
#pragma unroll
        for (int i = 0; i < NDW; ++i) t[i] = ((const volatile __attribute__((address_space(3))) uint32_t*)p)[i];
    }
    __builtin_memcpy(&r, t, sizeof(t));
    r.to_f32(f);
}
template <bool PIN, bool BF16, int VEC>
__device__ __forceinline__ void lds_row(const char* p, float (&f)[VEC]) {
    if constexpr (PIN) lds_read_pinned_row<BF16, VEC>(p, f);
    else lds_read_row<BF16, VEC>(p, f);
}
template <bool PIN>
__device__ __forceinline__ float2 lds_pair(const float2* p) {
    if constexpr (PIN) {
        const u32x2 q = *(const volatile __attribute__((address_space(3))) u32x2*)p;
        return make_float2(__uint_as_float(q.x), __uint_as_float(q.y));
    } else {
        return *p;
    }
}
template <bool PIN>
__device__ __forceinline__ void lds_put_pair(float2* p, float a, float b) {
    if constexpr (PIN) {
        const u32x2 t = {__float_as_uint(a), __float_as_uint(b)};
        *(volatile __attribute__((address_space(3))) u32x2*)p = t;
    } else {
        *p = make_float2(a, b);
    }
}

// One lane's slice of a gated input row out of LDS: h[v] = u[v] * silu(g[v]).
template <bool BF16, int VEC>
__device__ __forceinline__ void lds_read_gated_row(const char* pu, const char* pg, float (&h)[VEC]) {
    float u[VEC], g[VEC];
    lds_read_row<BF16, VEC>(pu, u);
    lds_read_row<BF16, VEC>(pg, g);
#pragma unroll
    for (int v = 0; v < VEC; ++v) h[v] = gate_mul(u[v], g[v]);
}

// The expensive part of the boundary lookup: position the cursor on the sequence of row tf (a chain
// of dependent scalar loads). The compute waves run it for the NEXT tile right before the tile
// barrier, where they would otherwise idle until the loaders' data has landed.
// Returns true when every tap of rows tf .. tf+RW-1 lies inside that one sequence. Otherwise `nce`
// receives the end of the interval that follows the cursor's, so that crossing the (usually only)
// boundary inside the wave's rows costs no scalar load in the middle of the tile's arithmetic.
template <int RW, int P, typename CU>
__device__ __forceinline__ bool wave_locate(SeqCursor& sc, int& nce, CU cu, int S, int T, int tf) {
    if (tf >= T) return true;
    sc.locate(cu, S, T, tf, sc.seq < 0 ? 0 : sc.seq);
    const int tl = (tf + RW - 1 < T) ? tf + RW - 1 : T - 1;
    const bool in = (tf - P >= sc.cs) && (tl + P < sc.ce);
    if (!in) nce = (sc.seq + 1 < S) ? cu_at(cu, sc.seq + 2) : T;
    return in;
}
// wave_locate through a row whose sequence index is already known: `lo` is what SeqCursor::locate finds for row
// `anchor` <= tf (the first i in [0, S) with cu[i+1] > anchor, else S). cu[lo], cu[lo+1] and cu[lo+2] (indices clamped
// to S) are three independent scalar loads behind one wait, where the binary search is a chain of log2(S) dependent
// ones; the cursor then steps from the anchor's sequence to that of row tf (no step when both lie in one sequence).
template <int RW, int P>
__device__ __forceinline__ bool wave_locate_from(SeqCursor& sc, int& nce, const int32_t* __restrict__ cu, int S, int T, int anchor,
                                                 int tf, int lo) {
    if (tf >= T) return true;
    const int32_t* p0 = cu + (lo < S ? lo : S);
    const int32_t* p1 = cu + (lo + 1 < S ? lo + 1 : S);
    const int32_t* p2 = cu + (lo + 2 < S ? lo + 2 : S);
    int c0, c1, c2;
    asm volatile("s_load_dword %0, %3, 0x0\n\ts_load_dword %1, %4, 0x0\n\ts_load_dword %2, %5, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(c0), "=&s"(c1), "=&s"(c2) : "s"(p0), "s"(p1), "s"(p2) : "memory");
    sc.seq = lo;
    sc.cs = c0;                                  // cu[lo], or cu[S] for rows at or after the last sequence's end
    sc.ce = lo < S ? c1 : T;
    if (sc.cs > anchor) { sc.ce = sc.cs; sc.cs = 0; sc.seq = -1; }   // the anchor lies before cu[0]
    const bool stepped = tf >= sc.ce && sc.seq < S;
    sc.advance(ScalarCu{cu}, S, T, tf);
    const int tl = (tf + RW - 1 < T) ? tf + RW - 1 : T - 1;
    const bool in = (tf - P >= sc.cs) && (tl + P < sc.ce);
    if (!in) nce = (sc.seq + 1 >= S) ? T : (!stepped && sc.seq == lo) ? c2 : cu_at(ScalarCu{cu}, sc.seq + 2);
    return in;
}
// SeqCursor::advance that takes its first step from the prefetched `nce` (valid while `fresh`).
template <typename CU>
__device__ __forceinline__ void advance_prefetched(SeqCursor& sq, int nce, bool& fresh, CU cu, int S, int T, int t) {
    if (fresh && t >= sq.ce && sq.seq < S) {
        ++sq.seq;
        sq.cs = sq.ce;
        sq.ce = nce;
        fresh = false;
    }
    sq.advance(cu, S, T, t);
}

// Empty volatile asm that takes N registers in and out: orders the instructions that produce them
// before everything that follows (and compiler-level memory accesses do not move across it).
template <int N>
__device__ __forceinline__ void pin_regs(float (&r)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) asm volatile("" : "+v"(r[i]) : : "memory");
}

// Tap masks of a wave's RW output rows, for a wave whose rows touch a sequence boundary: bit m of
// vm[u] is set iff tap row (tf + u) - P + m lies inside the sequence of output row tf + u. Rows past
// the end of the tensor get an empty mask. `sc` (by value) must be positioned on row tf, `nce` is
// what wave_locate left.
template <int RW, int K, typename CU>
__device__ __forceinline__ void wave_tap_masks(SeqCursor sc, int nce, CU cu, int S, int T, int tf, uint32_t (&vm)[RW]) {
    bool fresh = true;
#pragma unroll
    for (int u = 0; u < RW; ++u) {
        const int t = tf + u;
        uint32_t m = 0;
        if (t < T) {
            advance_prefetched(sc, nce, fresh, cu, S, T, t);
            m = row_tap_mask<K>(sc, t);
        }
        vm[u] = m;
    }
}

// Long gated kernels (K >= 15): a wave reads RW+K-1 staged rows for RW output rows, so a gate evaluated as rows are
// read would be evaluated (RW+K-1)/RW times per element. Instead the loader waves, once a tile has landed, turn
// its u and g rows into h = u * silu(g) in place, in fp32: a lane takes EPL adjacent elements of a row (the same
// bytes of the u row and of the g row) and leaves the first half of its h values where its u elements were and
// the second half where its g elements were (fp32 activations: all of them where u was). The compute waves then
// read fp32 h and do no gate arithmetic (and no bf16 unpacking) at all.
template <typename SH, bool BF16>
__device__ __forceinline__ void gate_prepass(char* buf, int lw, int nlw, int lane) {
    constexpr int EPL = SH::CB_CH / 64;
    static_assert(EPL == 2 || EPL == 4 || EPL == 8, "elements per lane and row");
    for (int j = lw; j < SH::NROWS; j += nlw) {
        char* pu = buf + j * SH::CB_BYTES + lane * EPL * SH::E;
        char* pg = pu + SH::TILE_BYTES;
        float u[EPL], g[EPL], h[EPL];
        lds_read_row<BF16, EPL>(pu, u);
        lds_read_row<BF16, EPL>(pg, g);
#pragma unroll
        for (int i = 0; i < EPL; ++i) h[i] = gate_mul(u[i], g[i]);
        if constexpr (BF16) {
            RowVec<false, EPL / 2> lo, hi;
#pragma unroll
            for (int i = 0; i < EPL / 2; ++i) { lo.v[i] = h[i]; hi.v[i] = h[EPL / 2 + i]; }
            lo.store(pu);
            hi.store(pg);
        } else {
            RowVec<false, EPL> o;
#pragma unroll
            for (int i = 0; i < EPL; ++i) o.v[i] = h[i];
            o.store(pu);
        }
    }
}
// Byte offset inside a staged row of the fp32 h values of channels lc .. lc+VEC-1 of the column block.
template <typename SH, bool BF16, int VEC>
__device__ __forceinline__ int pregated_offset(int lc) {
    constexpr int EPL = SH::CB_CH / 64;
    if constexpr (BF16) {
        static_assert(VEC <= EPL / 2, "a lane's channels lie in one half of a pre-pass lane's elements");
        const int l = lc / EPL, r = lc % EPL;
        const bool second = r >= EPL / 2;
        return (second ? SH::TILE_BYTES : 0) + l * EPL * 2 + (r - (second ? EPL / 2 : 0)) * 4;
    } else {
        return lc * 4;
    }
}

// Workgroup barrier for LDS hand-over only. __syncthreads() carries release/acquire fences at workgroup scope, for
// which the compiler waits for every outstanding vector memory operation of the wave first: a loader wave would
// wait for the tile it has just put in flight, a compute wave for the acknowledgement of its stores. What the
// hand-over of a tile needs is that this wave's LDS operations have completed (lgkmcnt) and, for a loader wave, the
// landing of the tile it hands over, which it has waited for by count. The empty asm statements keep the compiler
// from moving memory accesses across.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Sums of 16 values over the 64 lanes of a wave as a reduce-scatter, 40 instructions instead of 16 x 6: the two halves
// of the wave exchange and add (v_permlane32_swap: lanes 0-31 go on with values 0-7, lanes 32-63 with 8-15), then the
// rows of each half (v_permlane16_swap: even rows go on with the lower four of their eight values, odd rows with the
// upper four), then four rotations inside every row of 16 lanes. Every lane of row r ends with the totals of values
// 4r .. 4r+3.
__device__ __forceinline__ void wave_sums16(const float (&v)[16], float (&out)[4]) {
    typedef unsigned u2x __attribute__((ext_vector_type(2)));
    float s1[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const u2x r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[j]), __float_as_uint(v[j + 8]), false, false);
        s1[j] = __uint_as_float(r.x) + __uint_as_float(r.y);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u2x r = __builtin_amdgcn_permlane16_swap(__float_as_uint(s1[j]), __float_as_uint(s1[j + 4]), false, false);
        float t = __uint_as_float(r.x) + __uint_as_float(r.y);
        t += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(t), 0x128, 0xF, 0xF, false));   // row_ror:8
        t += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(t), 0x124, 0xF, 0xF, false));   // row_ror:4
        t += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(t), 0x122, 0xF, 0xF, false));   // row_ror:2
        t += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(t), 0x121, 0xF, 0xF, false));   // row_ror:1
        out[j] = t;
    }
}

// LayerNorm folded into the conv kernels (NORM variants below): the conv runs over n = layer_norm(x; gamma, beta), x is
// the raw input and the row statistics come from `stats` (written by dwconv_ln_fwd_kernel or ln_stats_kernel,
// dwconv_ln_kernels.h); the waves normalise x rows as they read them out of LDS.
struct LnSide {
    const float* stats;    // [T][2] fp32 (mean, rstd)
    const void* gamma;     // [C], weight dtype
    const void* beta;      // [C] or null
    float* partial2;       // backward only: [nbt][2][C] partial sums of dgamma, dbeta
};

// =============================================================================================
// Forward
// =============================================================================================
// NBUF = 2: one tile in flight while one is consumed. NBUF = 3: two tiles in flight (the loaders wait
// only for the older one), which keeps HBM busy when a single tile's latency exceeds its compute time.
//
// GATED: x is z = [u | g] of shape [T, 2C] (the SwiGLU MLP's Wi output, modeling.py:300-302) and the
// conv runs over h = u * silu(g), formed in registers as rows are read out of LDS; a buffer then
// holds a u tile followed by a g tile, and y is still [T, C].
//
// NORM: y = conv(layer_norm(x)) (+ x: the residual flag then adds the raw centre row instead of raising the centre
// tap), for rows wider than the whole-row kernel of dwconv_ln_kernels.h takes; see LnSide.
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, int NWL, int NBUF, bool GATED = false, bool NORM = false>
__global__ void __launch_bounds__((NCW * NRG + NWL) * 64)
dwconv_fwd_lds_kernel(const void* __restrict__ x, const int32_t* __restrict__ cu, const void* __restrict__ w,
                      const void* __restrict__ b, void* __restrict__ y, const LdsGeo g, const LnSide ln) {
    static_assert(!NORM || (!GATED && K <= 9), "the LayerNorm variant is built for the plain short kernels");
    using SH = LdsShape<BF16, K, VEC, RW, NRG, NCW, NWL>;
    constexpr int P = SH::P, E = SH::E, R = SH::R;
    using Row = RowVec<BF16, VEC>;
    constexpr int CNT = (SH::NROWS * SH::NPIECE + NWL - 1) / NWL;     // loads per loader wave per tile and tensor
    constexpr int BUF_BYTES = SH::TILE_BYTES * (GATED ? 2 : 1);
    static_assert(NBUF == 2 || NBUF == 3, "two or three tile buffers");
    static_assert(NBUF == 2 || SH::WHOLE_PIECES, "three buffers count loads in flight: whole 1 KiB pieces only");
    static_assert(!GATED || NBUF == 2, "the gated forward is double-buffered");
    constexpr bool PREGATE = GATED && K >= 15;   // the loader waves form h in LDS (see gate_prepass)
    // Where LDS has 32 bytes to spare per row group, the loader waves (idle while their loads are in
    // flight) also run the boundary lookup for the next tile and leave the result in a mailbox behind
    // the tile buffers; the compute waves, whose stores make them as memory-bound as the loaders, then
    // pay one LDS read per tile instead of a chain of dependent scalar loads.
    constexpr bool MAIL = lds_mail_fits((long long)NBUF * BUF_BYTES, SH::MAIL_BYTES);
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];   // NBUF x BUF_BYTES (+ MAIL_BYTES)
    int4* box = reinterpret_cast<int4*>(lds_raw + NBUF * BUF_BYTES);  // [2][NRG] (cs, ce, nce, seq)
    // NORM: (mean, rstd) of a tile's staged rows travel with the tile, 8 bytes per row behind the buffers (and the
    // mailbox): the compute waves read them where they normalise a row, as vector operands, instead of holding two
    // scalars per staged row through the taps
    constexpr int ST_BYTES = (SH::NROWS * 8 + 15) & ~15;
    char* st_base = lds_raw + NBUF * BUF_BYTES + (MAIL ? SH::MAIL_BYTES : 0);

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const bool is_loader = wv >= SH::NWC;
    int cb, tb;
    lds_block_coords(g, cb, tb);
    const int T = g.T, S = g.S, C = g.C;
    const size_t row_bytes = (size_t)C * E;
    const int rowb = (int)row_bytes;
    const int col_byte0 = cb * SH::CB_BYTES;
    const int valid_bytes = (rowb - col_byte0 < SH::CB_BYTES) ? rowb - col_byte0 : SH::CB_BYTES;
    const int ntl = (g.ntiles + g.nbt - 1) / g.nbt;        // rounds of the grid, the same for every block
    const size_t in_row_bytes = GATED ? 2 * row_bytes : row_bytes;   // pitch of x (z when gated)
    auto stage_tile = [&](char* buf, int first_row) {
        if constexpr (PREGATE) {
            // Every staged row is loaded exactly once, by the loader wave that later rewrites it in place
            // (gate_prepass takes rows lw, lw + NWL, ... as these loads do). stage_rows_fixed pads every wave to the
            // same number of loads by loading the last row again: such a second copy, issued by another wave, can
            // land after the row's owner has turned it into h, and put the raw u and g back.
            static_assert(!PREGATE || SH::NPIECE == 1, "a staged row is one load");
            stage_rows<SH, kLoadAuxOnceFwd>(x, buf, first_row, SH::NROWS, T, in_row_bytes, col_byte0, valid_bytes, wv - SH::NWC, NWL,
                                            lane, 2 * P);
            stage_rows<SH, kLoadAuxOnceFwd>(x, buf + SH::TILE_BYTES, first_row, SH::NROWS, T, in_row_bytes, rowb + col_byte0,
                                            valid_bytes, wv - SH::NWC, NWL, lane, 2 * P);
            return;
        }
        stage_rows_fixed<SH, CNT, kLoadAuxOnceFwd>(x, buf, first_row, SH::NROWS, T, in_row_bytes, col_byte0, valid_bytes, wv - SH::NWC,
                                  NWL, lane, 2 * P);
        if constexpr (NORM) {
            // one dword per lane: lane l of a load takes float l of the tile's [NROWS][2] statistics (rows clamped like
            // the tile's own)
            if (wv == SH::NWC) {
                // descriptor based at the tile's first row (like the tile's own), so that the lane offsets stay small
                // whatever T is
                const int sb = first_row > 0 ? first_row : 0;
                const rsrc_t rst = rows_rsrc(ln.stats, sb, T, 8);
                char* d = st_base + (buf == lds_raw ? 0 : ST_BYTES);
#pragma unroll
                for (int l0 = 0; l0 < SH::NROWS * 2; l0 += 64) {
                    const int idx = l0 + lane;
                    if (idx < SH::NROWS * 2)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rst, (lds_void*)(d + l0 * 4), 4,
                                                                 ((clamp_row(first_row + idx / 2, T) - sb) * 2 + (idx & 1)) * 4, 0, 0, kLoadAux);
                }
            }
        }
        if constexpr (GATED)
            stage_rows_fixed<SH, CNT, kLoadAuxOnceFwd>(x, buf + SH::TILE_BYTES, first_row, SH::NROWS, T, in_row_bytes, rowb + col_byte0,
                                      valid_bytes, wv - SH::NWC, NWL, lane, 2 * P);
    };

    // compute-wave coordinates (meaningless but harmless for loader waves)
    const int wc = wv % NCW;
    const int rg = (wv / NCW) % NRG;
    const int cw = valid_bytes / E;                                  // channels in this column block
    const int lcol = (wc * 64 + lane) * VEC;
    const bool active = !is_loader && lcol < cw;
    const int lc0 = (lcol < cw) ? lcol : cw - VEC;
    const int c0 = cb * SH::CB_CH + lc0;
    const int out_voff = c0 * E;

    float wr[VEC][K];
    float bias[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bias[v] = 0.f;
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    // loader waves: locate the row groups of the tile that starts at row0 and post them in mailbox set `par`
    // (a loader takes row groups lw, lw + NWL, ... in rising order, so its cursor only moves forward)
    auto post_bounds = [&](int par, int row0) {
        if constexpr (MAIL) {
            for (int r = wv - SH::NWC; r < NRG; r += NWL) {
                const int tf = row0 + r * RW;
                int ne = 0;
                if (tf < T) {
                    sc.locate(cu, S, T, tf, sc.seq < 0 ? 0 : sc.seq);
                    ne = (sc.seq + 1 < S) ? cu_at(cu, sc.seq + 2) : T;
                }
                if (lane == 0) box[par * NRG + r] = make_int4(sc.cs, sc.ce, ne, sc.seq);
            }
        }
    };
    if (is_loader) {
        stage_tile(lds_raw, tb * R - P);     // round 0: tile tb (< nbt <= ntiles)
        post_bounds(0, tb * R);
        const int r1 = ntl > 1 ? lds_tile_row0(g, 1, lds_next_slot(g, tb), R) : T;
        if (NBUF == 3 && r1 < T) {
            stage_tile(lds_raw + BUF_BYTES, r1 - P);
            wait_vmem_but<CNT>();     // tile 0 has landed, tile 1 may still be in flight
        } else {
            wait_vmem_all();
        }
        if constexpr (PREGATE) gate_prepass<SH, BF16>(lds_raw, wv - SH::NWC, NWL, lane);
    } else {
        load_weights<VEC, K>(w, NORM ? (g.w_flags & ~W_RESIDUAL) : g.w_flags, c0, wr);
        if (b) {
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                bias[v] = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(b)[c0 + v])
                                   : reinterpret_cast<const float*>(b)[c0 + v];
        }
    }
    float gam[NORM ? VEC : 1], bet[NORM ? VEC : 1];
    const bool add_raw = NORM && (g.w_flags & W_RESIDUAL);
    if constexpr (NORM) {
        const bool wb = (g.w_flags & W_BF16) != 0;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            gam[v] = wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.gamma)[c0 + v]) : reinterpret_cast<const float*>(ln.gamma)[c0 + v];
            bet[v] = !ln.beta ? 0.f : wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.beta)[c0 + v]) : reinterpret_cast<const float*>(ln.beta)[c0 + v];
        }
    }
    bool interior = true;               // bounds of the wave's rows in the tile about to be computed
    int nce = 0;                        // (not interior) end of the interval after the cursor's
    if constexpr (!MAIL) {
        if (!is_loader) interior = wave_locate<RW, P>(sc, nce, cu, S, T, tb * R + rg * RW);
    }
    __syncthreads();

    int bcur = 0;                       // buffer of tile `it`
    int q = tb;                         // the block's slot in round `it`
    for (int it = 0; it < ntl; ++it) {
        const int t0 = lds_tile_row0(g, it, q, R);   // T when the block has no tile in the last round
        const int qn = lds_next_slot(g, q);
        char* cur = lds_raw + bcur * BUF_BYTES;
        if (is_loader) {
            // stage the tile of round it + NBUF - 1 into the buffer freed by the barrier that ended round
            // it - 1, then wait until the tile of round it + 1 has landed
            const int ahead = NBUF - 1;
            const int rn = it + ahead < ntl ? lds_tile_row0(g, it + ahead, NBUF == 3 ? lds_next_slot(g, qn) : qn, R) : T;
            if (rn < T) {
                const int bnew = (bcur + ahead) % NBUF;
                stage_tile(lds_raw + bnew * BUF_BYTES, rn - P);
            }
            if (it + 1 < ntl) post_bounds((it + 1) & 1, lds_tile_row0(g, it + 1, qn, R));
            if (NBUF == 3 && rn < T) wait_vmem_but<CNT>(); else wait_vmem_all();
            if constexpr (PREGATE) {
                if (rn < T) gate_prepass<SH, BF16>(lds_raw + ((bcur + 1) % NBUF) * BUF_BYTES, wv - SH::NWC, NWL, lane);
            }
        } else {
            const int tf = t0 + rg * RW;
            if (tf < T) {
                if constexpr (MAIL) {
                    const int4 m = box[(it & 1) * NRG + rg];
                    sc.cs = __builtin_amdgcn_readfirstlane(m.x);
                    sc.ce = __builtin_amdgcn_readfirstlane(m.y);
                    nce = __builtin_amdgcn_readfirstlane(m.z);
                    sc.seq = __builtin_amdgcn_readfirstlane(m.w);
                    const int tl = (tf + RW - 1 < T) ? tf + RW - 1 : T - 1;
                    interior = (tf - P >= sc.cs) && (tl + P < sc.ce);
                }
                float acc[RW][VEC];
#pragma unroll
                for (int u = 0; u < RW; ++u)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[u][v] = bias[v];
                const char* lp = cur + (rg * RW) * SH::CB_BYTES + (PREGATE ? pregated_offset<SH, BF16, VEC>(lc0) : lc0 * E);
                // LayerNorm: a staged row is normalised as it is read, after its raw values have joined the output row they
                // are the centre of
                const float2* stq = reinterpret_cast<const float2*>(st_base + bcur * ST_BYTES) + rg * RW;
                auto normalise = [&](int j, float (&xr)[VEC]) {
                    if constexpr (NORM) {
                        if (add_raw && j >= P && j < P + RW) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[j - P][v] += xr[v];
                        }
                        const float2 mr = stq[j];
                        const float a = mr.y, b2 = -mr.x * mr.y;
#pragma unroll
                        for (int v = 0; v < VEC; ++v) xr[v] = __builtin_fmaf(__builtin_fmaf(xr[v], a, b2), gam[v], bet[v]);
                    }
                };
                if (interior) {
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float xr[VEC];
                        if constexpr (PREGATE) lds_read_row<false, VEC>(lp + j * SH::CB_BYTES, xr);
                        else if constexpr (GATED) lds_read_gated_row<BF16, VEC>(lp + j * SH::CB_BYTES, lp + SH::TILE_BYTES + j * SH::CB_BYTES, xr);
                        else lds_read_row<BF16, VEC>(lp + j * SH::CB_BYTES, xr);
                        normalise(j, xr);
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[u][v] = __builtin_fmaf(wr[v][j - u], xr[v], acc[u][v]);
                            }
                        }
                    }
                } else if constexpr (K >= 15) {
                    // Long kernels, a sequence boundary inside the wave's window: one pass per sequence that owns
                    // output rows of the wave. A pass runs the unmasked schedule over the staged rows of
                    // its sequence only (whole rows are skipped by scalar branches, nothing is multiplied
                    // by zero) into a scratch set of accumulators, of which the sequence's own output
                    // rows are kept. Every staged row is read in at most one pass, so the path costs
                    // about what the unmasked one does, however many boundaries there are, and every
                    // output row sums its taps in the same order as on the other paths (same bits).
                    SeqCursor sq = sc;                      // positioned on row tf
                    int u0 = 0;                             // first output row not yet produced
                    bool fresh = true;
                    while (u0 < RW && tf + u0 < T) {
                        advance_prefetched(sq, nce, fresh, cu, S, T, tf + u0);
                        // staged rows (j <-> global row tf - P + j) and output rows of this sequence
                        int jlo = sq.cs - (tf - P), jhi = sq.ce - (tf - P), u1 = sq.ce - tf;
                        jlo = __builtin_amdgcn_readfirstlane(jlo < 0 ? 0 : jlo);
                        jhi = __builtin_amdgcn_readfirstlane(jhi > RW + K - 1 ? RW + K - 1 : jhi);
                        u1 = __builtin_amdgcn_readfirstlane(u1 > RW ? RW : u1);
                        float part[RW][VEC];
#pragma unroll
                        for (int u = 0; u < RW; ++u)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) part[u][v] = bias[v];
#pragma unroll
                        for (int j = 0; j < RW + K - 1; ++j) {
                            if (j >= jlo && j < jhi) {
                                float xr[VEC];
                                if constexpr (PREGATE) lds_read_row<false, VEC>(lp + j * SH::CB_BYTES, xr);
                                else if constexpr (GATED) lds_read_gated_row<BF16, VEC>(lp + j * SH::CB_BYTES, lp + SH::TILE_BYTES + j * SH::CB_BYTES, xr);
                                else lds_read_row<BF16, VEC>(lp + j * SH::CB_BYTES, xr);
#pragma unroll
                                for (int u = 0; u < RW; ++u) {
                                    if (j - u >= 0 && j - u < K) {
#pragma unroll
                                        for (int v = 0; v < VEC; ++v) part[u][v] = __builtin_fmaf(wr[v][j - u], xr[v], part[u][v]);
                                    }
                                }
                            }
                        }
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (u >= u0 && u < u1) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[u][v] = part[u][v];
                            }
                        }
                        u0 = u1;
                    }
                } else {
                    // Short kernels: the unmasked schedule with every tap selected (never multiplied by
                    // zero) by a bit of its output row's tap mask; cheaper than per-sequence passes here.
                    uint32_t vm[RW];
                    wave_tap_masks<RW, K>(sc, nce, cu, S, T, tf, vm);
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float xr[VEC];
                        if constexpr (GATED) lds_read_gated_row<BF16, VEC>(lp + j * SH::CB_BYTES, lp + SH::TILE_BYTES + j * SH::CB_BYTES, xr);
                        else lds_read_row<BF16, VEC>(lp + j * SH::CB_BYTES, xr);
                        normalise(j, xr);
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
                                const bool ok = (vm[u] >> (j - u)) & 1u;
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    const float xv = ok ? xr[v] : 0.f;
                                    acc[u][v] = __builtin_fmaf(wr[v][j - u], xv, acc[u][v]);
                                }
                            }
                        }
                    }
                }
                const rsrc_t ry = rows_rsrc(y, tf, T, row_bytes);
                Row o[RW];
#pragma unroll
                for (int u = 0; u < RW; ++u) o[u].from_f32(acc[u]);
                if (active) {
#pragma unroll
                    for (int u = 0; u < RW; ++u)
                        if (tf + u < T) o[u].bstore(ry, out_voff, u * rowb);
                }
            }
            if constexpr (!MAIL) {
                if (it + 1 < ntl) interior = wave_locate<RW, P>(sc, nce, cu, S, T, lds_tile_row0(g, it + 1, qn, R) + rg * RW);
            }
        }
        __syncthreads();   // next tile is in LDS; this tile's buffer may be overwritten
        bcur = (bcur + 1 == NBUF) ? 0 : bcur + 1;
        q = qn;
    }
}

// =============================================================================================
// Backward (fused)
// =============================================================================================
// Same arithmetic as the sliding-window backward: both gradients of row t read the one window of dy
// rows t-P .. t+P, and x only contributes its centre row:
//     dx[t] = sum_m w[K-1-m] * dy[t-P+m],   dw[K-1-m] += x[t] * dy[t-P+m],   db += dy[t].
// So only the dy tile carries halo rows; the x tile is exactly the R rows of the tile.
// LDS: [2 buffers][dy tile (R+K-1 rows), x tile (R rows, only when dw/db are wanted)].
//
// GATED: x is z = [u | g] of shape [T, 2C], the conv ran over h = u * silu(g), and dx is dz [T, 2C]:
// a buffer holds the dy tile, a u tile and a g tile; h rows (for dw) and the two halves of dz
//     du = dh * silu(g),   dg = dh * u * sig(g) * (1 + g * (1 - sig(g))),   dh = the conv's dx
// are formed in registers from the staged u and g rows.
//
// NORM: the conv ran over n = layer_norm(x; gamma, beta) (see LnSide) and x is
// the raw input: the wave normalises its x rows as it reads them, dx is the gradient with respect to n (fp32), and the
// block also sums the LayerNorm parameter gradients, which need that gradient in fp32 and the normalised rows:
//     dgamma[c] += dn[t,c] * xhat[t,c],   dbeta[c] += dn[t,c],   xhat = (x - mean) * rstd.
// They leave the block like dw/db, in a second slab of 2 x C floats per token block.
//
// WHOLE (with NORM; one column block that holds whole rows, NWL = 0): the block also forms LayerNorm's input gradient,
//     dx = rstd * (g - mean_c(g) - xhat * mean_c(g * xhat))  (+ dy with the residual flag),   g = gamma * dn,
// and dn never leaves it. A tile takes two phases around one more barrier: after the taps every wave reduces its rows'
// shares of sum_c g and sum_c g * xhat over its lanes (wave_sums16) and leaves them in LDS; after the barrier lane u of
// a wave adds the wave-columns' shares of row u and the wave writes dx of its rows. LDS behind the two buffers:
// [NCW][NRG][8] x (sum g, sum g * xhat), then two sets of (mean, rstd) per tile row, which arrive with the tile.
// There are no loader waves (SELF): every wave issues its share of the next tile's direct loads before it starts on
// the current tile and waits for them before it stores dx; its LDS accesses are pinned (lds_read_pinned_row), its
// boundary lookups scalar (ScalarCu), and the tile changes hands at an LDS-only barrier with the stores in flight.
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, int NWL, bool WDX, bool WDW, bool GATED = false, bool NORM = false,
          bool WHOLE = false>
__global__ void __launch_bounds__((NCW * NRG + NWL) * 64)
dwconv_bwd_lds_kernel(const void* __restrict__ x, const void* __restrict__ dy, const int32_t* __restrict__ cu,
                      const void* __restrict__ w, void* __restrict__ dx, float* __restrict__ partial, const LdsGeo g,
                      const LnSide ln) {
    static_assert(!NORM || (WDX && WDW && !GATED), "the LayerNorm variant produces every gradient of the plain conv");
    static_assert(!WHOLE || NORM, "whole rows: the LayerNorm variant with one column block");
    // NWL = 0: no loader waves; every wave stages its share of the next tile before it computes the current one, and
    // all its LDS accesses are pinned (see lds_read_pinned_row)
    constexpr bool SELF = NWL == 0;
    constexpr int NLW = SELF ? NCW * NRG : NWL;           // waves that stage
    static_assert(!SELF || WHOLE, "only the whole-row LayerNorm variant runs without loader waves");
    using SH = LdsShape<BF16, K, VEC, RW, NRG, NCW, NWL>;
    constexpr int P = SH::P, E = SH::E, R = SH::R;
    constexpr int XT_BYTES = R * SH::CB_BYTES;
    constexpr int BUF_BYTES = SH::TILE_BYTES + (WDW ? XT_BYTES : 0) * (GATED ? 2 : 1);
    static_assert(!GATED || (WDX && WDW), "the gated backward always produces dz, dw and db");
    using Row = RowVec<BF16, VEC>;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];   // 2 x BUF_BYTES

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const bool is_loader = !SELF && wv >= SH::NWC;
    int cb, tb;
    lds_block_coords(g, cb, tb);
    const int T = g.T, S = g.S, C = g.C;
    const size_t row_bytes = (size_t)C * E;
    const int rowb = (int)row_bytes;
    const int col_byte0 = cb * SH::CB_BYTES;
    const int valid_bytes = (rowb - col_byte0 < SH::CB_BYTES) ? rowb - col_byte0 : SH::CB_BYTES;
    const int ntl = (g.ntiles + g.nbt - 1) / g.nbt;        // rounds of the grid, the same for every block

    const int wc = wv % NCW;
    const int rg = (wv / NCW) % NRG;
    const int cw = valid_bytes / E;
    const int lcol = (wc * 64 + lane) * VEC;
    const bool active = !is_loader && lcol < cw;
    const int lc0 = (lcol < cw) ? lcol : cw - VEC;
    const int c0 = cb * SH::CB_CH + lc0;
    const int out_voff = c0 * E;
    const int lw = SELF ? wv : wv - SH::NWC;

    const size_t x_row_bytes = GATED ? 2 * row_bytes : row_bytes;    // pitch of x and dx (z and dz when gated)
    auto stage_x = [&](char* buf, int t0, int l, int nl) {
        stage_rows<SH, kLoadAuxOnceBwdX>(x, buf + SH::TILE_BYTES, t0, R, T, x_row_bytes, col_byte0, valid_bytes, l, nl, lane, 0);
        if constexpr (GATED)
            stage_rows<SH, kLoadAuxOnceBwdX>(x, buf + SH::TILE_BYTES + XT_BYTES, t0, R, T, x_row_bytes, rowb + col_byte0, valid_bytes, l, nl,
                           lane, 0);
    };
    auto stage_both = [&](char* buf, int t0) {
        // with two or more loader waves, even ones take the dy tile and odd ones the x tile(s)
        if constexpr (WDW && NLW >= 2) {
            if (lw & 1) stage_x(buf, t0, lw >> 1, NLW / 2);
            else        stage_rows<SH, kLoadAuxOnceBwd>(dy, buf, t0 - P, SH::NROWS, T, row_bytes, col_byte0, valid_bytes, lw >> 1, (NLW + 1) / 2, lane, 2 * P);
        } else {
            stage_rows<SH, kLoadAuxOnceBwd>(dy, buf, t0 - P, SH::NROWS, T, row_bytes, col_byte0, valid_bytes, lw, NLW, lane, 2 * P);
            if constexpr (WDW) stage_x(buf, t0, lw, NLW);
        }
        if constexpr (WHOLE) {
            // (mean, rstd) of the tile's rows travel with the tile: 8 bytes per row behind the buffers, one direct load of
            // one dword per lane (rows past the end read as zeros)
            if (lw == 0 && lane < R * 2) {
                char* d = lds_raw + 2 * BUF_BYTES + NCW * NRG * 64 + (buf == lds_raw ? 0 : R * 8);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rows_rsrc(ln.stats, t0, T, 8), (lds_void*)d, 4, lane * 4, 0, 0, kLoadAux);
            }
        }
    };

    float wr[VEC][K];
    float dwa[VEC][K];
    float dba[VEC];
    float dga[NORM ? VEC : 1], dbb[NORM ? VEC : 1], gam[NORM ? VEC : 1], bet[NORM ? VEC : 1];   // LayerNorm: sums and parameters
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        dba[v] = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) { dwa[v][k] = 0.f; wr[v][k] = 0.f; }
    }
    if constexpr (NORM) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            const bool wb = (g.w_flags & W_BF16) != 0;
            dga[v] = 0.f; dbb[v] = 0.f;
            const int c = c0 + v < C ? c0 + v : C - 1;
            if (WHOLE && !active) { gam[v] = 0.f; bet[v] = 0.f; continue; }     // copies of the last channels: out of the row sums
            gam[v] = wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.gamma)[c]) : reinterpret_cast<const float*>(ln.gamma)[c];
            bet[v] = !ln.beta ? 0.f : wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.beta)[c]) : reinterpret_cast<const float*>(ln.beta)[c];
        }
    }
    if (SELF || is_loader) stage_both(lds_raw, tb * R);
    if (!is_loader) {
        if constexpr (WDX) load_weights<VEC, K>(w, WHOLE ? (g.w_flags & ~W_RESIDUAL) : g.w_flags, c0, wr);
    }
    if (SELF || is_loader) wait_vmem_all();
    // WHOLE: the wave-columns' shares of the two row sums, [NCW][NRG][8 rows] x (sum g, sum g * xhat)
    static_assert(!WHOLE || RW <= 8, "the row sums of a wave are reduced sixteen at a time");
    constexpr int RED_BYTES = NCW * NRG * 8 * 8;
    float2* red2 = reinterpret_cast<float2*>(lds_raw + 2 * BUF_BYTES);
    // SELF: the boundary lookups go through scalar loads (see ScalarCu): the waves have stores and direct loads in flight
    std::conditional_t<SELF, ScalarCu, const int32_t*> cuq{cu};
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    bool interior = true;
    int nce = 0;
    // WHOLE: the sequence index of the first row of the block's tile in each of its first 64 rounds, found by 64 binary
    // searches side by side on the lanes of wave 0 and left in LDS behind the row statistics: the lookup of a wave's next
    // tile, which sits in every wave's chain from the taps to the row sums, is then one LDS read and three independent
    // scalar loads (wave_locate_from) instead of log2(S) dependent ones. With a handful of sequences the search stays.
    constexpr int TAB_TILES = 64;
    typedef volatile __attribute__((address_space(3))) int32_t lds_i32;
    lds_i32* seq_tab = (lds_i32*)(lds_raw + 2 * BUF_BYTES + RED_BYTES + 2 * R * 8);
    const bool use_tab = WHOLE && S >= 16;
    if constexpr (WHOLE) {
        if (use_tab && wv == 0) {
            int t = T;
            if (lane < ntl) {
                const int q_ = (int)(((long long)tb + (long long)lane * g.rot_step) % g.nbt);     // lds_next_slot, lane times
                const int tile = lane * g.nbt + q_;
                if (tile < g.ntiles) t = tile * R;
            }
            int lo = 0, hi = S;     // first i in [0, S) with cu[i + 1] > t, else S
            while (__builtin_amdgcn_ballot_w64(lo < hi) != 0) {
                if (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (cu[mid + 1] > t) hi = mid; else lo = mid + 1;
                }
            }
            seq_tab[lane] = lo;     // visible to the block after the barrier below
        }
    }
    // the boundary lookup of the wave's tile in round it + 1
    auto locate_next = [&](int it, int qn) __attribute__((always_inline)) {
        const int rn = lds_tile_row0(g, it + 1, qn, R);
        if constexpr (WHOLE) {
            if (use_tab && it + 1 < TAB_TILES)
                return wave_locate_from<RW, P>(sc, nce, cu, S, T, rn, rn + rg * RW, __builtin_amdgcn_readfirstlane(seq_tab[it + 1]));
        }
        return wave_locate<RW, P>(sc, nce, cuq, S, T, rn + rg * RW);
    };
    if (!is_loader) interior = wave_locate<RW, P>(sc, nce, cuq, S, T, tb * R + rg * RW);
    __syncthreads();

    int q = tb;                         // the block's slot in round `it`
    for (int it = 0; it < ntl; ++it) {
        const int t0 = lds_tile_row0(g, it, q, R);   // T when the block has no tile in the last round
        const int qn = lds_next_slot(g, q);
        char* cur = lds_raw + (it & 1) * BUF_BYTES;
        if (SELF || is_loader) {
            const int rn = it + 1 < ntl ? lds_tile_row0(g, it + 1, qn, R) : T;
            if (rn < T) stage_both(lds_raw + ((it + 1) & 1) * BUF_BYTES, rn);
            if constexpr (!SELF) {
                if constexpr (WHOLE) lds_barrier();      // the compute waves' exchange of row sums, with the loads in flight
                if (rn < T) wait_vmem_all();
            }
        }
        if (!is_loader) {
            const int tf = t0 + rg * RW;
            // WHOLE: dn of the wave's rows, kept across the exchange of the row sums; (mean, rstd) of the tile's rows
            float dnv[WHOLE ? RW : 1][VEC], xh[WHOLE ? RW : 1][VEC];       // ... and their normalised x
            bool located = false;       // WHOLE: the next tile's boundary lookup has been done (see emit_dx)
            bool fix_dw = false;        // boundary path: some x value of the wave's rows is Inf or NaN (see xbad there)
            const float2* stl = reinterpret_cast<const float2*>(lds_raw + 2 * BUF_BYTES + RED_BYTES) + (it & 1) * R;
            if (tf < T) {
                const int loff = (rg * RW) * SH::CB_BYTES + lc0 * E;
                const char* lpg = cur + loff;                      // dy: staged row j <-> global row tf - P + j
                const char* lpx = cur + SH::TILE_BYTES + loff;     // x : staged row u <-> global row tf + u
                const rsrc_t ro = rows_rsrc(dx, tf, T, x_row_bytes);
                // LayerNorm: (rstd, -mean * rstd) of the wave's x rows, wave-uniform: scalars loaded once per tile, or
                // (WHOLE, 16 rows per wave) read out of LDS wherever a row is normalised, where the loaders have put them
                float sa[NORM && !WHOLE ? RW : 1], sb[NORM && !WHOLE ? RW : 1];
                if constexpr (NORM && !WHOLE) {
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        const int tr = tf + u < T ? tf + u : T - 1;
                        const float mean = ln.stats[2 * (size_t)tr], rstd = ln.stats[2 * (size_t)tr + 1];
                        sa[u] = rstd;
                        sb[u] = -mean * rstd;
                    }
                }
                auto row_stats = [&](int u, float& a, float& b) {
                    if constexpr (WHOLE) {
                        const float2 mr = lds_pair<SELF>(stl + rg * RW + u);
                        a = mr.y;
                        b = -mr.x * mr.y;
                    } else {
                        a = sa[NORM ? u : 0];
                        b = sb[NORM ? u : 0];
                    }
                };
                // Gated: per element of the wave's x rows, the two factors everything else needs:
                //   gs = silu(g) / ... = g * sig(g)              (h = u * gs, du = dh * gs)
                //   gd = u * sig(g) * (1 + g * (1 - sig(g)))     (dg = dh * gd)
                float gs[GATED ? RW : 1][VEC], gd[GATED ? RW : 1][VEC];
                // x row u of the wave as the conv saw it (h when gated)
                auto read_x = [&](int u, float (&xv)[VEC]) {
                    if constexpr (GATED) {
                        float uu[VEC], gg[VEC];
                        lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, uu);
                        lds_row<SELF, BF16, VEC>(lpx + XT_BYTES + u * SH::CB_BYTES, gg);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            const float sg = sigmoid_f32(gg[v]);
                            gs[u][v] = gg[v] * sg;
                            gd[u][v] = uu[v] * sg * (1.f + gg[v] * (1.f - sg));
                            xv[v] = uu[v] * gs[u][v];
                        }
                    } else {
                        lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, xv);
                        if constexpr (NORM) {
                            float a, b;
                            row_stats(u, a, b);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) xv[v] = __builtin_fmaf(__builtin_fmaf(xv[v], a, b), gam[v], bet[v]);
                        }
                    }
                };
                // write the wave's dx rows (du and dg rows of dz when gated) from the conv's input gradient
                auto emit_dx = [&](float (&acc)[WDX ? RW : 1][VEC]) {
                    if constexpr (WHOLE) {
                        // The boundary lookup for the next tile (a chain of dependent scalar loads) goes here, between the
                        // taps and the row sums, where the other waves of the SIMD are at their arithmetic and not, as at
                        // the end of the tile, all at the same chain.
                        if (it + 1 < ntl) interior = locate_next(it, qn);
                        located = true;
                    }
                    if constexpr (WDX) {
                        const int xrowb = (int)x_row_bytes;
                        if constexpr (GATED) {
#pragma unroll
                            for (int u = 0; u < RW; ++u) {
                                float du[VEC], dg[VEC];
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    du[v] = acc[u][v] * gs[u][v];
                                    dg[v] = acc[u][v] * gd[u][v];
                                }
                                Row ou, og;
                                ou.from_f32(du);
                                og.from_f32(dg);
                                if (active && tf + u < T) {
                                    ou.bstore(ro, out_voff, u * xrowb);
                                    og.bstore(ro, out_voff + rowb, u * xrowb);
                                }
                            }
                        } else {
                            if constexpr (NORM) {
                                // the LayerNorm parameter gradients from the fp32 gradient of n and the normalised row
                                if constexpr (WHOLE) {
                                    // Straight-line code for all rows (no branch per row, so that the reads and the
                                    // reductions of different rows overlap): rows past the end of the last tile get a
                                    // zero gradient here and their statistics read as zeros, so they add nothing.
                                    if (tf + RW > T) {
#pragma unroll
                                        for (int u = 0; u < RW; ++u) {
                                            if (tf + u >= T) {
#pragma unroll
                                                for (int v = 0; v < VEC; ++v) acc[u][v] = 0.f;
                                            }
                                        }
                                    }
                                    float ps[16];       // (sum g, sum g * xhat) of row u at 2u, 2u + 1
#pragma unroll
                                    for (int i = 0; i < 16; ++i) ps[i] = 0.f;
#pragma unroll
                                    for (int u = 0; u < RW; ++u) {
                                        float xr[VEC], a, b;
                                        row_stats(u, a, b);
                                        lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, xr);
                                        // this lane's share of the two row sums LayerNorm's input gradient needs:
                                        // g = gamma * dn and g * xhat over the channels (gamma is 0 in lanes past the
                                        // row's end, which hold copies of the last channels)
#pragma unroll
                                        for (int v = 0; v < VEC; ++v) {
                                            const float xhat = __builtin_fmaf(xr[v], a, b);
                                            dga[v] = __builtin_fmaf(acc[u][v], xhat, dga[v]);
                                            dbb[v] += acc[u][v];
                                            const float gv = gam[v] * acc[u][v];
                                            dnv[u][v] = acc[u][v];
                                            xh[u][v] = xhat;
                                            ps[2 * u] += gv;
                                            ps[2 * u + 1] = __builtin_fmaf(gv, xhat, ps[2 * u + 1]);
                                        }
                                    }
                                    // over the wave's lanes: every lane of row r of the wave ends with the sums of rows 2r
                                    // and 2r + 1, and the first lane of the row leaves them for the other wave-columns
                                    float tot[4];
                                    wave_sums16(ps, tot);
                                    if ((lane & 15) == 0) {
                                        const u32x4 t = {__float_as_uint(tot[0]), __float_as_uint(tot[1]), __float_as_uint(tot[2]), __float_as_uint(tot[3])};
                                        *(volatile __attribute__((address_space(3))) u32x4*)(red2 + (wc * NRG + rg) * 8 + (lane >> 4) * 2) = t;
                                    }
                                } else {
#pragma unroll
                                    for (int u = 0; u < RW; ++u) {
                                        if (tf + u < T) {
                                            float xr[VEC], a, b;
                                            row_stats(u, a, b);
                                            lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, xr);
#pragma unroll
                                            for (int v = 0; v < VEC; ++v) {
                                                dga[v] = __builtin_fmaf(acc[u][v], __builtin_fmaf(xr[v], a, b), dga[v]);
                                                dbb[v] += acc[u][v];
                                            }
                                        }
                                    }
                                }
                            }
                            if constexpr (WHOLE) {
                                // dx waits for the other wave-columns' sums: after the barrier below
                            } else if constexpr (NORM) {
                                // the gradient of n leaves in fp32 whatever the activations are: the row pass that
                                // turns it into dx rounds once
                                const int nrowb = C * 4;
                                const rsrc_t rn = rows_rsrc(dx, tf, T, (size_t)nrowb);
                                RowVec<false, VEC> o[RW];
#pragma unroll
                                for (int u = 0; u < RW; ++u) o[u].from_f32(acc[u]);
                                if (active) {
#pragma unroll
                                    for (int u = 0; u < RW; ++u)
                                        if (tf + u < T) o[u].bstore(rn, c0 * 4, u * nrowb);
                                }
                            } else {
                                Row o[RW];
#pragma unroll
                                for (int u = 0; u < RW; ++u) o[u].from_f32(acc[u]);
                                if (active) {
#pragma unroll
                                    for (int u = 0; u < RW; ++u)
                                        if (tf + u < T) o[u].bstore(ro, out_voff, u * xrowb);
                                }
                            }
                        }
                    }
                };
                if (interior) {
                    float xc[WDW ? RW : 1][VEC];
                    if constexpr (WDW) {
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            read_x(u, xc[u]);
                            if (tf + u >= T) {     // rows past the end contribute nothing
#pragma unroll
                                for (int v = 0; v < VEC; ++v) xc[u][v] = 0.f;
                            }
                        }
                    }
                    float acc[WDX ? RW : 1][VEC];
                    if constexpr (WDX) {
#pragma unroll
                        for (int u = 0; u < RW; ++u)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[u][v] = 0.f;
                    }
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float gr[VEC];
                        lds_row<SELF, BF16, VEC>(lpg + j * SH::CB_BYTES, gr);
                        if constexpr (WDW) {
                            if (j >= P && j < P + RW) {   // centre row of output j - P (interior: always < T)
#pragma unroll
                                for (int v = 0; v < VEC; ++v) dba[v] += gr[v];
                            }
                        }
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    if constexpr (WDX) acc[u][v] = __builtin_fmaf(wr[v][K - 1 - (j - u)], gr[v], acc[u][v]);
                                    if constexpr (WDW) dwa[v][K - 1 - (j - u)] = __builtin_fmaf(xc[u][v], gr[v], dwa[v][K - 1 - (j - u)]);
                                }
                            }
                        }
                    }
                    emit_dx(acc);
                } else {
                    // A sequence boundary falls inside the wave's window: same unrolled schedule, every
                    // tap selected (never multiplied by 0) by bit m of its output row's tap mask.
                    uint32_t vm[RW];
                    wave_tap_masks<RW, K>(sc, nce, cuq, S, T, tf, vm);
                    float xc[WDW ? RW : 1][VEC];
                    // A masked tap enters the dw sums as x * (selected 0), which is NaN for an x that is Inf or NaN,
                    // where the definition drops the product. Such x values are rare enough to be handled apart: the
                    // wave tests its x rows (x * 0 summed up is NaN iff one of them is not finite), and if any is, the
                    // values in question run through the schedule as zeros and add_nonfinite_x below puts their
                    // valid products into the sums afterwards.
                    bool xbad = false;
                    if constexpr (WDW) {
#pragma unroll
                        for (int u = 0; u < RW; ++u) read_x(u, xc[u]);
                        float chk = 0.f;
#pragma unroll
                        for (int u = 0; u < RW; ++u)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) chk = __builtin_fmaf(xc[u][v], 0.f, chk);
                        xbad = __builtin_amdgcn_ballot_w64(chk != chk) != 0;
                        if (xbad) {
#pragma unroll
                            for (int u = 0; u < RW; ++u)
#pragma unroll
                                for (int v = 0; v < VEC; ++v) xc[u][v] = __builtin_isfinite(xc[u][v]) ? xc[u][v] : 0.f;
                        }
                    }
                    float acc[WDX ? RW : 1][VEC];
                    if constexpr (WDX) {
#pragma unroll
                        for (int u = 0; u < RW; ++u)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[u][v] = 0.f;
                    }
                    // one staged row ahead in registers; the scheduling fences keep the (already rare)
                    // path from hoisting every read and mask to the top and running out of registers
                    Row nxt;
                    if constexpr (!SELF) nxt.load(lpg);
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float gr[VEC];
                        if constexpr (SELF) {
                            lds_row<true, BF16, VEC>(lpg + j * SH::CB_BYTES, gr);
                        } else {
                            nxt.to_f32(gr);
                            if (j + 1 < RW + K - 1) nxt.load(lpg + (j + 1) * SH::CB_BYTES);
                        }
                        if constexpr (WDW) {
                            if (j >= P && j < P + RW) {   // centre tap of output j - P: valid iff that row exists
                                const bool okc = (vm[j - P] >> P) & 1u;
#pragma unroll
                                for (int v = 0; v < VEC; ++v) dba[v] += okc ? gr[v] : 0.f;
                            }
                        }
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
                                const bool ok = (vm[u] >> (j - u)) & 1u;
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    const float gv = ok ? gr[v] : 0.f;
                                    if constexpr (WDX) acc[u][v] = __builtin_fmaf(wr[v][K - 1 - (j - u)], gv, acc[u][v]);
                                    if constexpr (WDW) dwa[v][K - 1 - (j - u)] = __builtin_fmaf(xc[u][v], gv, dwa[v][K - 1 - (j - u)]);
                                }
                            }
                        }
                        // pin this row's arithmetic here: every accumulator passes through an empty
                        // volatile asm, so nothing of row j can sink below the read of row j + 2
                        if constexpr (WDX) {
#pragma unroll
                            for (int u = 0; u < RW; ++u)
                                if (j - u >= 0 && j - u < K) pin_regs<VEC>(acc[u]);
                        }
                        if constexpr (WDW) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) pin_regs<K>(dwa[v]);
                        }
                    }
                    emit_dx(acc);
                    fix_dw = xbad;
                }
            }
            if constexpr (WHOLE) {
                lds_barrier();
                if constexpr (SELF) wait_vmem_all();      // this wave's share of the next tile has landed (long ago)
                if (tf < T) {
                    // dx = rstd * (g - mean_c(g) - xhat * mean_c(g * xhat)) (+ dy: the residual connection's share)
                    const float inv_c = 1.f / (float)C;
                    const bool resid = (g.w_flags & W_RESIDUAL) != 0;
                    const char* lpc = cur + (rg * RW + P) * SH::CB_BYTES + lc0 * E;     // dy row of output row u: staged row u + P
                    const rsrc_t ro = rows_rsrc(dx, tf, T, row_bytes);
                    // lane u sums the wave-columns' shares of row u, in the order of the columns, and takes row u's rstd;
                    // the three per-row scalars are then read out of that lane
                    float s1 = 0.f, s2 = 0.f, ra = 0.f;
                    if (lane < RW) {
#pragma unroll
                        for (int c = 0; c < NCW; ++c) {
                            const float2 r = lds_pair<SELF>(red2 + (c * NRG + rg) * 8 + lane);
                            s1 += r.x;
                            s2 += r.y;
                        }
                        ra = lds_pair<SELF>(stl + rg * RW + lane).y;
                    }
                    s1 *= inv_c;
                    s2 *= -inv_c;
                    // straight-line arithmetic for all rows; only the store of a row past the end is skipped
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        {
                            const float m1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s1), u));
                            const float nm2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s2), u));
                            const float rstd = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ra), u));
                            float o[VEC];
#pragma unroll
                            for (int v = 0; v < VEC; ++v) o[v] = 0.f;
                            if (resid) lds_row<SELF, BF16, VEC>(lpc + u * SH::CB_BYTES, o);
#pragma unroll
                            for (int v = 0; v < VEC; ++v)
                                o[v] = __builtin_fmaf(rstd, __builtin_fmaf(nm2, xh[u][v], __builtin_fmaf(gam[v], dnv[u][v], -m1)), o[v]);
                            Row orow;
                            orow.from_f32(o);
                            if (active && tf + u < T) orow.bstore(ro, out_voff, u * rowb);
                        }
                    }
                }
            }
            // Boundary path, x rows that hold Inf or NaN (see xbad there): the products of those values with the dy rows
            // of their own sequence, one output row at a time, once everything else of the tile is done (the tile stays
            // in LDS until the barrier below). A rolled loop over the rows (their LDS addresses are formed at run time),
            // the taps unrolled, each behind a scalar branch on its bit of the row's tap mask; lanes whose x value is
            // finite keep their sums (their products went through the schedule).
            if constexpr (WDW) {
                if (fix_dw) {
                    const int loff = (rg * RW) * SH::CB_BYTES + lc0 * E;
                    const char* lpg = cur + loff;
                    const char* lpx = cur + SH::TILE_BYTES + loff;
                    SeqCursor sq = sc;
                    bool fresh = true;
#pragma nounroll
                    for (int u = 0; u < RW; ++u) {
                        const int t = tf + u;
                        if (t >= T) break;
                        advance_prefetched(sq, nce, fresh, cuq, S, T, t);
                        const uint32_t m = row_tap_mask<K>(sq, t);
                        float xv[VEC];
                        if constexpr (GATED) {
                            float uu[VEC], gg[VEC];
                            lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, uu);
                            lds_row<SELF, BF16, VEC>(lpx + XT_BYTES + u * SH::CB_BYTES, gg);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) xv[v] = gate_mul(uu[v], gg[v]);
                        } else {
                            lds_row<SELF, BF16, VEC>(lpx + u * SH::CB_BYTES, xv);
                            if constexpr (NORM) {
                                const float mean = ln.stats[2 * (size_t)t], rstd = ln.stats[2 * (size_t)t + 1];
#pragma unroll
                                for (int v = 0; v < VEC; ++v)
                                    xv[v] = __builtin_fmaf(__builtin_fmaf(xv[v], rstd, -mean * rstd), gam[v], bet[v]);
                            }
                        }
                        bool nf[VEC];
#pragma unroll
                        for (int v = 0; v < VEC; ++v) nf[v] = !__builtin_isfinite(xv[v]);
                        static_for<K>([&](auto kk_c) {
                            constexpr int kk = decltype(kk_c)::value;
                            if ((m >> kk) & 1u) {
                                float gr[VEC];
                                lds_row<SELF, BF16, VEC>(lpg + (u + kk) * SH::CB_BYTES, gr);
#pragma unroll
                                for (int v = 0; v < VEC; ++v)
                                    dwa[v][K - 1 - kk] = nf[v] ? __builtin_fmaf(xv[v], gr[v], dwa[v][K - 1 - kk]) : dwa[v][K - 1 - kk];
                            }
                        });
                    }
                }
            }
            if (!located && it + 1 < ntl) interior = locate_next(it, qn);
        }
        // SELF: every wave has waited for its share of the next tile before it stored dx, so the stores need not be
        // acknowledged before the tile changes hands (__syncthreads() would wait for them)
        if constexpr (SELF) lds_barrier(); else __syncthreads();
        q = qn;
    }

    if constexpr (!WDW) return;

    float* slab = partial + (size_t)tb * (K + 1) * C;
    if constexpr (NRG == 1) {
        // one row group: every (tap, channel) sum of the block already sits in exactly one lane
        if (active) {
#pragma unroll
            for (int kk = 0; kk <= K; ++kk) {
                float* dst = slab + (size_t)kk * C + c0;
#pragma unroll
                for (int v = 0; v < VEC; ++v) dst[v] = (kk < K) ? dwa[v][kk < K ? kk : 0] : dba[v];
            }
            if constexpr (NORM) {
                float* dst = ln.partial2 + (size_t)tb * 2 * C + c0;
#pragma unroll
                for (int v = 0; v < VEC; ++v) { dst[v] = dga[v]; dst[C + v] = dbb[v]; }
            }
        }
        return;
    }
    // ---- block-level pass: sum the NRG row groups of each wave-column, group order 0,1,2,... ----
    // The tiles are dead after the last barrier above. Every wave of row groups 1.. leaves all its sums in LDS, one
    // barrier, and the waves of row group 0 add them up and write the slab (one barrier for the whole pass: a barrier
    // per tap would also wait for the slab stores of the tap before, which end the kernel of every block at once).
    constexpr int NV = K + 1 + (NORM ? 2 : 0);
    static_assert((long long)NV * SH::NWC * VEC * 256 <= 2LL * BUF_BYTES, "the sums of all compute waves fit the dead tiles");
    float* red = reinterpret_cast<float*>(lds_raw);   // [NV][NWC][VEC][64]
    auto sum_of = [&](int kk, int v) __attribute__((always_inline)) {
        return (kk < K) ? dwa[v][kk < K ? kk : 0] : (kk == K) ? dba[v] : (kk == K + 1) ? dga[NORM ? v : 0] : dbb[NORM ? v : 0];
    };
    if (!is_loader && rg > 0) {
#pragma unroll
        for (int kk = 0; kk < NV; ++kk)
#pragma unroll
            for (int v = 0; v < VEC; ++v) red[((kk * SH::NWC + wv) * VEC + v) * 64 + lane] = sum_of(kk, v);
    }
    __syncthreads();
    if (!is_loader && rg == 0) {
#pragma unroll
        for (int kk = 0; kk < NV; ++kk) {
            float val[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) val[v] = sum_of(kk, v);
#pragma unroll
            for (int j = 1; j < NRG; ++j) {
                const int ow = j * NCW + wc;
#pragma unroll
                for (int v = 0; v < VEC; ++v) val[v] += red[((kk * SH::NWC + ow) * VEC + v) * 64 + lane];
            }
            if (active) {
                float* dst = kk <= K ? slab + (size_t)kk * C + c0 : ln.partial2 + ((size_t)tb * 2 + (kk - K - 1)) * C + c0;
#pragma unroll
                for (int v = 0; v < VEC; ++v) dst[v] = val[v];
            }
        }
    }
}

}  // namespace nplm
