// LDS-staged fused backward for K = 31 in which every wave computes and the two outputs have their own waves
// (gfx950, wave64).
//
// At K = 31 the backward issues 62 FMAs per element and is bound by the vector ALU. A SIMD issues FMAs near its rate
// (one v_fmac_f32 per 2.1 - 2.4 cycles, measured on register-only loops) only while 4 of its waves are in an FMA
// stream at once; one wave alone issues one per 5 cycles. That allows 128 registers per lane, where one wave holding K
// weights and K dw sums per channel needs 166, and it rules out idle loader waves, which cost as many registers as a
// compute wave. So here
//   * the two outputs go to two kinds of wave that share the staged dy tile:
//       role 0 (dx):    dx[t] = sum_m w[K-1-m] * dy[t-P+m]           holds K weights + RW row sums
//       role 1 (dw/db): dw[K-1-m] += x[t] * dy[t-P+m], db += dy[t]   holds K tap sums + RW x rows
//     Neither needs the other's registers, nothing is exchanged, and both run the same unrolled schedule over the
//     RW+K-1 staged rows of their RW output rows. dx sums its taps in the order of the sliding-window kernel (same bits).
//     Every SIMD runs two waves of each role (SplitShape::role_of).
//   * every wave computes. The dx waves also issue the direct global->LDS loads of the NEXT tile (dy with K-1 halo
//     rows, x without) into the other buffer, one load every few rows of their FMA schedule, and store an output row
//     as soon as its last tap is in; the dw/db waves never wait on memory.
//   * a wave lowers its priority as it advances through a tile, which keeps the 4 waves of a SIMD in step up to the
//     tile's barrier (the one synchronisation per tile: next tile landed, this tile's buffer free).
// Cycles per tile and SIMD at T = 131072, C = 2048, one sequence (s_memtime around the phases): 15300 with every wave
// loading at the top of the tile, roles on separate SIMDs' worth of waves and no priorities; 13300 as built, of which
// 11000 in the row schedules at 2.2 cycles per vector instruction (5100 per SIMD and tile, 3968 of them FMAs).
// Tiles, rounds, slot rotation and XCD grouping are those of the other LDS-staged kernels (dwconv_lds_kernels.h);
// dw/db leave the block as in those (row groups summed through LDS in fixed order, one slab per token block, then
// dwconv_finalize_kernel). No atomics; every sum has a fixed order.
//
// Sequence boundaries: a wave whose rows and taps all lie in one sequence runs unmasked. Otherwise it makes one pass
// per sequence that owns some of its output rows, over the staged rows of that sequence: the dx role skips the other
// rows by scalar branches and stores the sequence's output rows at the end of the pass; the dw role loads the x rows
// of the sequence (zero for the others), skips chunks of staged rows that hold none of the sequence's and masks
// single rows of another sequence inside a chunk (the mask rides on the bf16 -> fp32 conversion).
//
// The forward at these kernel sizes is the dx role alone on all 16 waves (taps in forward order, the bias as the row
// sums' start). Its gated form (input z = [u | g], conv over h = u * silu(g)) stages a u tile and a g tile, has the 16
// waves turn them into one fp32 h tile in place once per staged element, and runs the same schedules over that.
//
// No counterpart in the reference (peymanvahidi/nanoplm 0.1.6 has no convolution); tensor contract:
// modeling.py:339,421-439 and collator.py:322-325,405-458 (the gate product: modeling.py:300-302).
#pragma once
#include "dwconv_lds_kernels.h"

namespace nplm {

// FWD: the forward (y from x), which is the dx role alone on every wave, with the taps in forward order and the bias.
// GATED, backward: x is z = [u | g] of shape [T, 2C] and a buffer holds a u tile and a g tile behind the dy tile.
// FWD && GATED: x is z = [u | g] as well; a buffer holds a u tile and a g tile, both with their halo rows, which the waves
// turn into one fp32 h = u * silu(g) tile in place before the row schedules run (see gate_tile in split_role).
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, bool FWD = false, bool GATED = false>
struct SplitShape {
    static constexpr bool GF = FWD && GATED;
    static_assert(!GF || (BF16 ? VEC == 2 : VEC == 1), "gated forward: a lane's slice of a row is 4 bytes of u and 4 of g");
    static constexpr int E = BF16 ? 2 : 4;
    static constexpr int P = (K - 1) / 2;
    static constexpr int NROLE = FWD ? 1 : 2;
    static constexpr int NW = NCW * NROLE * NRG;           // waves per block (all compute)
    // wave -> (role, index within the role). The waves of a block go to the 4 SIMDs of a CU round-robin, so the role
    // changes within a residue class of the wave index mod 4: every SIMD then runs waves of both roles, and the
    // role with less work leaves its issue slots to the other instead of idling two of the four SIMDs.
    __device__ static constexpr int role_of(int wv) { return FWD ? 0 : (wv >> 2) & 1; }
    __device__ static constexpr int index_of(int wv) { return FWD ? wv : (wv & 3) | ((wv >> 3) << 2); }
    __device__ static constexpr int wave_of(int role, int idx) { return (idx & 3) | (role << 2) | ((idx >> 2) << 3); }
    static_assert(FWD || NW % 8 == 0, "roles alternate in groups of 4 waves");
    static constexpr int NT = NW * 64;
    static constexpr int R = RW * NRG;                     // output rows per tile
    static constexpr int NROWS = R + K - 1;                // staged dy (forward: x) rows per tile
    static constexpr int NJ = RW + K - 1;                  // of which a wave reads this many
    static constexpr int CB_BYTES = NCW * 64 * VEC * E;    // bytes of a row in one column block
    static constexpr int CB_CH = NCW * 64 * VEC;
    static constexpr int CPR = CB_BYTES / 16;              // 16-byte chunks per staged row
    static constexpr int IN_BYTES = NROWS * CB_BYTES;      // dy tile
    static constexpr int X_BYTES = FWD ? 0 : R * CB_BYTES; // backward: x tile, no halo (gated: the u tile, and as much again for g)
    static constexpr int BUF_BYTES = GF ? 2 * IN_BYTES : IN_BYTES + X_BYTES * (GATED ? 2 : 1);
    static constexpr int TAB_TILES = 64;                   // tiles of a block whose sequence index is looked up ahead
    static constexpr int LDS_BYTES = 2 * BUF_BYTES + TAB_TILES * 4;   // two tile buffers and that table
    static constexpr int RPL = 64 / CPR;                   // staged rows per 1 KiB load (64 lanes x 16 bytes)
    static constexpr int NLD_IN = (NROWS + RPL - 1) / RPL; // loads of a dy tile
    static constexpr int NLD_X1 = FWD ? 0 : (R + RPL - 1) / RPL;  // loads of an x tile (gated: of the u tile, of the g tile)
    static constexpr int NLD_X = GF ? NLD_IN : NLD_X1 * (GATED ? 2 : 1);  // gated forward: the g tile, like the u tile
    static constexpr int ROW_UNITS = NROWS * NCW;          // gated forward: (staged row, wave-column) pairs to gate
    static_assert(CB_BYTES == 256 || CB_BYTES == 512 || CB_BYTES == 1024, "a staged row is 16, 32 or 64 chunks");
    static_assert(NW <= 16, "at most 1024 threads per block");
    static_assert(LDS_BYTES <= kLdsBytes, "two tile buffers and the table must fit in LDS");
    static_assert(NJ * CB_BYTES <= 65536, "ds_read immediate offsets (a wave reads NJ rows from one base) are 16 bit");
    static_assert(NW * VEC * 64 * 4 <= LDS_BYTES, "the final reduction reuses the tile buffers");
    static_assert(NW == 16, "4 waves per SIMD and one block per CU");
};

// One lane's slice of a staged row, read with a volatile access: the compiler may neither hoist it out of its
// place in the unrolled schedule (all reads of a tile at the top would need NJ registers) nor merge it with
// the same read on another path.
template <bool BF16, int VEC>
__device__ __forceinline__ void lds_read_pinned(const char* p, RowVec<BF16, VEC>& r) {
    if constexpr (RowVec<BF16, VEC>::BYTES == 2) {
        r.h = *(const volatile __attribute__((address_space(3))) uint16_t*)p;
    } else if constexpr (RowVec<BF16, VEC>::BYTES == 8) {
        // one 8-byte access: as two dword reads the lanes' 8-byte stride puts them two to a bank in each
        const u32x2 t = *(const volatile __attribute__((address_space(3))) u32x2*)p;
        __builtin_memcpy(&r, &t, sizeof(t));
    } else {
        constexpr int NDW = RowVec<BF16, VEC>::BYTES / 4;
        uint32_t t[NDW];
#pragma unroll
        for (int i = 0; i < NDW; ++i) t[i] = ((const volatile __attribute__((address_space(3))) uint32_t*)p)[i];
        __builtin_memcpy(&r, t, sizeof(t));
    }
}

// The whole life of a wave of one role: its registers, its tile loop and (dw role) the block-level sum. The two roles
// are two instantiations that share no variable, so that the register allocator treats them apart (one function
// with both roles' K per-channel values meeting at every join needs 170 registers where either role needs 106).
// Both execute the same sequence of barriers.
// Backward: in = dy, other = x, out = dx, partial = dw/db slabs. Forward: in = x, out = y, bias may be null.
// GATED (backward): other = z = [u | g] [T, 2C], the conv ran over h = u * silu(g), out = dz [T, 2C]. The dw/db role
// forms h of its rows as it reads them; the dx role reads u and g of an output row when its last tap is in and stores
//     du = dh * g * sig(g),   dg = dh * u * sig(g) * (1 + g * (1 - sig(g))),   dh = the conv's input gradient.
// Each role evaluates the sigmoid of its rows itself (once per element and role): handing it over through LDS would
// need 8 bytes per element where u and g leave 4.
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, bool FWD, int ROLE, bool GATED = false>
__device__ __forceinline__ void split_role(const void* __restrict__ in, const void* __restrict__ other,
                                           const int32_t* __restrict__ cu, const void* __restrict__ w,
                                           const void* __restrict__ bias, void* __restrict__ out,
                                           float* __restrict__ partial, const LdsGeo& g) {
    using SH = SplitShape<BF16, K, VEC, RW, NRG, NCW, FWD, GATED>;
    constexpr int P = SH::P, E = SH::E, R = SH::R, NJ = SH::NJ, NROLE = SH::NROLE;
    using Row = RowVec<BF16, VEC>;
    using InRow = RowVec<BF16 && !(FWD && GATED), VEC>;              // a lane's slice of a staged row as the schedules read it
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];   // 2 x BUF_BYTES

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const int wc = SH::index_of(wv) % NCW;
    const int rg = SH::index_of(wv) / NCW;
    int cb, tb;
    lds_block_coords(g, cb, tb);
    const int T = g.T, S = g.S, C = g.C;
    const size_t row_bytes = (size_t)C * E;
    const int rowb = (int)row_bytes;
    const int col_byte0 = cb * SH::CB_BYTES;
    const int valid_bytes = (rowb - col_byte0 < SH::CB_BYTES) ? rowb - col_byte0 : SH::CB_BYTES;
    const int ntl = (g.ntiles + g.nbt - 1) / g.nbt;        // rounds of the grid, the same for every block

    const int cw = valid_bytes / E;
    const int lcol = (wc * 64 + lane) * VEC;
    const bool active = lcol < cw;
    const int lc0 = active ? lcol : cw - VEC;
    const int c0 = cb * SH::CB_CH + lc0;
    const int out_voff = c0 * E;
    constexpr bool GF = FWD && GATED;                      // gated forward: in = z [T, 2C], out = y [T, C]
    constexpr bool GB = GATED && !FWD;                     // gated backward: other = z, out = dz, both [T, 2C]
    const int xrowb = GB ? 2 * rowb : rowb;                // pitch of x and of the output (z and dz in the gated backward)
    const size_t x_row_bytes = GB ? 2 * row_bytes : row_bytes;
    const int in_rowb = GF ? 2 * rowb : rowb;              // pitch of the staged input with halo (z in the gated forward)
    const size_t in_row_bytes = GF ? 2 * row_bytes : row_bytes;

    // ---- staging: direct global->LDS loads of 1 KiB (64 lanes x 16 bytes = RPL adjacent rows of the column block) ----
    // A tile is one run of 16-byte chunks, dy rows first (NLD_IN loads), then x rows (NLD_X loads); load number
    // lw + n * NLW is the n-th of this wave. Each lane forms its own row offset. Rows outside [0, T) are not clamped:
    // their offsets fall outside the descriptor (or, on a tensor beyond 4 GiB, on other rows of it), so nothing faults,
    // and what lands in LDS for them is never used (a branch or a select, never a product, masks it).
    // The dx role stages the tiles: its waves have less to do per tile than the dw/db role's (no x rows to read, no
    // row masks), and a wave that stores dx and also waits for loads is the only kind that waits for store
    // acknowledgements at the tile's barrier; the dw/db role never waits on memory.
    // (In the forward every wave is of that kind.)
    // (Gated, where the dx role is the heavier one - the gate's derivative and two stores per output row - the dw/db role
    // staging the tiles instead measured 779 against 738 us at T=131072, C=2048, K=31.)
    constexpr bool LOADS = ROLE == 0;
    constexpr int NLW = SH::NW / NROLE;                                         // waves that stage tiles
    constexpr int NPW = (SH::NLD_IN + SH::NLD_X + NLW - 1) / NLW;               // loads per such wave and tile
    // A loader wave issues its loads of the next tile one at a time, every SSTEP staged rows of its FMA schedule.
    // (Issued all at once at the top of the tile they fill the CU's memory pipeline, and the wave stalls at their
    // issue for a sixth of the tile: 2500 of 15000 cycles measured.)
    constexpr int SSTEP = (NJ * 9 / 10) / NPW > 1 ? (NJ * 9 / 10) / NPW : 1;
    static_assert(NPW * SSTEP <= NJ, "a slot for every load");
    const int lw = rg * NCW + wc;                                               // this wave's index among them
    const int lrow = lane / SH::CPR, lchunk = lane % SH::CPR;
    const bool lane_ok = lchunk * 16 < valid_bytes;
    rsrc_t rs_in, rs_x;         // descriptors of the tile being staged
    int s_in = 0;               // byte offset of its first dy row from the descriptor's first row (negative in tile 0)
    char* nbuf = lds_raw;
    int lw_t = lw;              // lw, made opaque in every tile: see stage_begin
    const int v_lane = lrow * in_rowb + col_byte0 + lchunk * 16;
    const int v_lane_x = lrow * xrowb + col_byte0 + lchunk * 16;
    auto stage_begin = [&](char* buf, int t0) __attribute__((always_inline)) {
        const int rb = t0 - P > 0 ? t0 - P : 0;
        rs_in = rows_rsrc(in, rb, T, in_row_bytes);
        if constexpr (!FWD) rs_x = rows_rsrc(other, t0, T, x_row_bytes);
        s_in = (t0 - P - rb) * in_rowb;
        nbuf = buf;
        // everything a load derives from the wave's index is the same in every tile; computed once outside the tile
        // loop it would occupy some 50 scalar registers (NPW loads x flags and offsets) and push others into spills
        lw_t = lw;
        asm volatile("" : "+s"(lw_t));
    };
    auto stage_one = [&](int n) __attribute__((always_inline)) {
        const int gi = lw_t + n * NLW;
        if (gi < SH::NLD_IN) {
            const bool once = gi * SH::RPL >= 2 * P && gi * SH::RPL + SH::RPL <= SH::NROWS - 2 * P;   // no other tile stages it
            if (lane_ok && (SH::NROWS % SH::RPL == 0 || gi * SH::RPL + lrow < SH::NROWS))
                load_to_lds<FWD ? kLoadAuxOnceFwd : kLoadAuxOnceBwd>(rs_in, nbuf + gi * 1024, v_lane + (s_in + gi * (SH::RPL * in_rowb)), 0, once);
        } else if (GF && gi < 2 * SH::NLD_IN) {
            // gated forward: the g tile (the second half of every z row) behind the u tile, the same rows
            const int i = gi - SH::NLD_IN;
            const bool once = i * SH::RPL >= 2 * P && i * SH::RPL + SH::RPL <= SH::NROWS - 2 * P;
            if (lane_ok && (SH::NROWS % SH::RPL == 0 || i * SH::RPL + lrow < SH::NROWS))
                load_to_lds<kLoadAuxOnceFwd>(rs_in, nbuf + SH::IN_BYTES + i * 1024, v_lane + rowb + (s_in + i * (SH::RPL * in_rowb)), 0, once);
        } else if (!GF && gi < SH::NLD_IN + SH::NLD_X) {
            // gated: the loads of the u tile, then those of the g tile (the second half of every z row)
            const int i2 = gi - SH::NLD_IN;
            const bool gpart = GB && i2 >= SH::NLD_X1;
            const int i = gpart ? i2 - SH::NLD_X1 : i2;
            if (lane_ok && (R % SH::RPL == 0 || i * SH::RPL + lrow < R))
                load_to_lds<kLoadAuxOnceBwdX>(rs_x, nbuf + SH::IN_BYTES + (gpart ? SH::X_BYTES : 0) + i * 1024,
                                              v_lane_x + (gpart ? rowb : 0) + i * (SH::RPL * xrowb), 0, true);
        }
    };
    bool spread = false;        // the loads of the next tile are issued from inside the row schedule

    // role 0: a[v][m] = w[K-1-m], the weight of staged row u + m for output row u;   b = row sums of dx
    // role 1: a[v][m] = sum over rows of x[t] * dy[t-P+m] (= dw[K-1-m]);              b = x rows
    float a[VEC][K];
    float b[RW][VEC];
    float c[VEC];          // role 1: db; forward: the bias (what a row sum starts from); role 0 of the backward: zero
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        c[v] = 0.f;
#pragma unroll
        for (int m = 0; m < K; ++m) a[v][m] = 0.f;
    }
    auto pin_a = [&](auto v_c, auto m_c) __attribute__((always_inline)) {
        float& x = a[decltype(v_c)::value][decltype(m_c)::value];
        asm volatile("" : "+v"(x) : : "memory");
    };
    auto pin_b = [&](auto u_c, auto v_c) __attribute__((always_inline)) {
        float& x = b[decltype(u_c)::value][decltype(v_c)::value];
        asm volatile("" : "+v"(x) : : "memory");
    };
    // the sums row j touches: role 0 b[u][*], role 1 a[*][j-u], for every output row u with a tap on row j
    auto pin_row = [&](auto j_c) __attribute__((always_inline)) {
        constexpr int j = decltype(j_c)::value;
        static_for<RW>([&](auto u_c) __attribute__((always_inline)) {
            constexpr int u = decltype(u_c)::value;
            if constexpr (j - u >= 0 && j - u < K) {
                static_for<VEC>([&](auto v_c) __attribute__((always_inline)) {
                    if constexpr (ROLE == 0) pin_b(u_c, v_c);
                    else pin_a(v_c, std::integral_constant<int, j - u>{});
                });
            }
        });
    };
    if constexpr (ROLE == 0) {
        if (const int off = w_tap_off(g.w_flags); off == 0) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
#pragma unroll
                for (int m = 0; m < K; ++m) {
                    const size_t wi = (size_t)(c0 + v) * K + (FWD ? m : K - 1 - m);
                    a[v][m] = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[wi]) : reinterpret_cast<const float*>(w)[wi];
                }
            }
        } else {        // weight rows of K - 2 * off taps: the outer taps are zero, see W_TAP_OFF_SHIFT
            const int kw = K - 2 * off;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
#pragma unroll
                for (int m = 0; m < K; ++m) {
                    const int r = (FWD ? m : K - 1 - m) - off;
                    const bool tap = r >= 0 && r < kw;
                    const size_t wi = (size_t)(c0 + v) * kw + (tap ? r : 0);
                    const float t = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[wi]) : reinterpret_cast<const float*>(w)[wi];
                    a[v][m] = tap ? t : 0.f;
                }
            }
        }
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            if (g.w_flags & W_RESIDUAL) a[v][P] += 1.f;
            if (FWD && bias) c[v] = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(bias)[c0 + v]) : reinterpret_cast<const float*>(bias)[c0 + v];
        }
    }
    if constexpr (LOADS) {
        stage_begin(lds_raw, tb * R);
        for (int n = 0; n < NPW; ++n) stage_one(n);
    }
    // Entry l of seq_tab: the sequence index (what the binary search of SeqCursor::locate returns) of the first row of
    // the block's tile in round l, for the first TAB_TILES rounds: 64 searches side by side on the lanes of wave 0, once.
    // The lookup of the next tile at the end of every tile is then three independent scalar loads (wave_locate_from) and
    // not a chain of log2(S) dependent ones on which all 16 waves of the block wait at the same time, with nothing else
    // to issue (measured per wave and 64-row tile of the backward at T=131072, C=2048, 418 sequences: 1100-1400 of 13900
    // cycles). The table lives in LDS behind the tile buffers: as a register it would be live across the row schedules.
    // With a handful of sequences the binary search is two or three steps and stays (one long sequence, backward at
    // T=131072, C=2048: 457 us with it, 465 us through the table; 418 sequences: 498-518 against 489-497 us).
    typedef volatile __attribute__((address_space(3))) int32_t lds_i32;
    lds_i32* seq_tab = (lds_i32*)(lds_raw + 2 * SH::BUF_BYTES);
    const bool use_tab = S >= 16;
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
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    int nce = 0;
    bool interior = wave_locate<RW, P>(sc, nce, cu, S, T, tb * R + rg * RW);
    if constexpr (LOADS) wait_vmem_all();       // this wave's share of the first tile has landed
    __syncthreads();

    rsrc_t ro;                  // output rows of the wave in the current tile (dx role)
    const char* lpx_cur = lds_raw;     // x rows of the wave in the current tile: row u <-> global row tf + u (gated: u rows, g rows X_BYTES on)
    // dx role: output row u of the wave from its finished row sum (gated: the two halves of the dz row)
    auto emit_row = [&](int u, const float (&acc)[VEC]) __attribute__((always_inline)) {
        if constexpr (GB) {
            // (pinned reads: this wave has direct loads in flight, see lds_read_pinned)
            float uu[VEC], gg[VEC], du[VEC], dg[VEC];
            Row ru, rg_;
            lds_read_pinned<BF16, VEC>(lpx_cur + u * SH::CB_BYTES, ru);
            lds_read_pinned<BF16, VEC>(lpx_cur + SH::X_BYTES + u * SH::CB_BYTES, rg_);
            ru.to_f32(uu);
            rg_.to_f32(gg);
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float sg = sigmoid_f32(gg[v]);
                du[v] = acc[v] * (gg[v] * sg);
                dg[v] = acc[v] * (uu[v] * sg * (1.f + gg[v] * (1.f - sg)));
            }
            Row ou, og;
            ou.from_f32(du);
            og.from_f32(dg);
            if (active) {
                ou.bstore(ro, out_voff, u * xrowb);
                og.bstore(ro, out_voff + rowb, u * xrowb);
            }
        } else {
            Row o;
            o.from_f32(acc);
            if (active) o.bstore(ro, out_voff, u * xrowb);
        }
    };
    // dw role: x row u of the wave as the conv saw it (gated: h = u * silu(g))
    auto read_x_row = [&](int u, float (&xv)[VEC]) __attribute__((always_inline)) {
        if constexpr (GB) {
            float uu[VEC], gg[VEC];
            lds_read_row<BF16, VEC>(lpx_cur + u * SH::CB_BYTES, uu);
            lds_read_row<BF16, VEC>(lpx_cur + SH::X_BYTES + u * SH::CB_BYTES, gg);
#pragma unroll
            for (int v = 0; v < VEC; ++v) xv[v] = gate_mul(uu[v], gg[v]);
        } else {
            lds_read_row<BF16, VEC>(lpx_cur + u * SH::CB_BYTES, xv);
        }
    };
    // slot of the schedule after staged row j: the next load of the tile being staged
    auto slot = [&](auto j_c) __attribute__((always_inline)) {
        constexpr int j = decltype(j_c)::value;
        // A wave's priority falls as it advances through the tile (3 at the top, 0 in the last quarter), so the waves
        // of a SIMD that lag behind catch up and all reach the tile's barrier together. The arbiter otherwise favours
        // the same waves all the time, and the last one finishes alone at a quarter of the SIMD's issue rate.
        constexpr int Q = (NJ + 3) / 4;
        if constexpr (j % Q == Q - 1 && j / Q < 3) __builtin_amdgcn_s_setprio(2 - j / Q);
        if constexpr (LOADS && j % SSTEP == 0 && j / SSTEP < NPW) {
            if (spread) stage_one(j / SSTEP);
        }
    };

    // the unrolled schedule over staged rows [jlo, jhi) of the wave's window (all NJ rows when UNMASKED):
    // row j feeds output rows u = j-K+1 .. j with tap m = j - u
    auto run_rows = [&](const char* lp, auto unmasked_c, int jlo, int jhi) __attribute__((always_inline)) {
        constexpr bool UNMASKED = decltype(unmasked_c)::value;
        // Both forms keep two rows ahead in registers. A pass over the rows of one sequence (not UNMASKED) reads every
        // staged row all the same and skips only the arithmetic of the rows outside [jlo, jhi): a read that waits for
        // its row right before it is used leaves the wave idle for an LDS round trip per row, and a boundary wave that
        // runs late holds up its whole block at the tile's barrier.
        InRow nxt[2];
        lds_read_pinned(lp, nxt[0]);
        lds_read_pinned(lp + SH::CB_BYTES, nxt[1]);
        // (a compile-time loop: as an ordinary loop its unrolled body is too large for the unroller at K = 31, and
        // the register arrays would then be indexed at run time and live in scratch memory)
        static_for<NJ>([&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            // the scheduling barrier below keeps the compiler from hoisting all NJ reads to the top, which would not fit
            // the 128 registers of 4 waves per SIMD
            float gr[VEC];
            nxt[j & 1].to_f32(gr);
            if (j + 2 < NJ) lds_read_pinned(lp + (j + 2) * SH::CB_BYTES, nxt[j & 1]);
            if (UNMASKED || (j >= jlo && j < jhi)) {
#pragma unroll
                for (int u = 0; u < RW; ++u) {
                    if (j - u >= 0 && j - u < K) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) b[u][v] = __builtin_fmaf(a[v][j - u], gr[v], b[u][v]);
                    }
                }
                // pin this row's arithmetic here: every sum it touched passes through an empty volatile asm, which
                // is ordered with the (volatile) row reads, so the FMAs of row j stay between the reads of rows
                // j + 2 and j + 3
                if constexpr (UNMASKED) {
                    pin_row(j_c);
                    // output row j - (K-1) has all its taps: out it goes, long before the tile ends
                    if constexpr (j >= K - 1) emit_row(j - (K - 1), b[j - (K - 1)]);
                }
            }
            if constexpr (UNMASKED) slot(j_c);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // dw role: the staged rows in chunks of CH; a chunk with no row of the pass's sequence is skipped by one scalar
    // branch, inside a chunk a row of another sequence contributes a selected zero. (One branch per row, as in the
    // dx role, makes the register allocator keep two copies of the K tap sums per channel.) An interior tile is the
    // single pass over all rows.
    auto run_rows_chunked = [&](const char* lp, int jlo, int jhi) __attribute__((always_inline)) {
        constexpr int CH = 12, NCH = (NJ + CH - 1) / CH;
        // bit j: staged row j belongs to the pass (one scalar bit test per row, where two compares against the bounds
        // and their conjunction took 5 scalar instructions)
        static_assert(NJ < 64, "one mask bit per staged row");
        const int lo_ = jlo < 0 ? 0 : jlo, hi_ = jhi > NJ ? NJ : jhi;
        const uint64_t inmask = hi_ > lo_ ? (((1ull << hi_) - 1ull) & ~((1ull << lo_) - 1ull)) : 0ull;
        static_for<NCH>([&](auto ch_c) __attribute__((always_inline)) {
            constexpr int j0 = decltype(ch_c)::value * CH;
            constexpr int j1 = j0 + CH < NJ ? j0 + CH : NJ;
            if (j0 < jhi && j1 > jlo) {
                Row nxt[2];     // two rows ahead in registers, as in run_rows
                lds_read_pinned<BF16, VEC>(lp + j0 * SH::CB_BYTES, nxt[0]);
                if (j0 + 1 < j1) lds_read_pinned<BF16, VEC>(lp + (j0 + 1) * SH::CB_BYTES, nxt[1]);
                static_for<j1 - j0>([&](auto jj_c) __attribute__((always_inline)) {
                    constexpr int j = j0 + decltype(jj_c)::value;
                    const bool in = (inmask >> j) & 1ull;
                    float gr[VEC];
                    if constexpr (BF16 && VEC == 2) {
                        // the row mask rides on the bf16 -> fp32 conversion: the high half by an AND, the low half by a
                        // byte permute, both with a wave-uniform (scalar) second operand chosen by `in`
                        const uint32_t raw = nxt[(j - j0) & 1].d[0];
                        gr[1] = __uint_as_float(raw & (in ? 0xffff0000u : 0u));
                        gr[0] = __uint_as_float(__builtin_amdgcn_perm(raw, raw, in ? 0x01000c0cu : 0x0c0c0c0cu));
                        if (j + 2 < j1) lds_read_pinned<BF16, VEC>(lp + (j + 2) * SH::CB_BYTES, nxt[(j - j0) & 1]);
                    } else {
                        nxt[(j - j0) & 1].to_f32(gr);
                        if (j + 2 < j1) lds_read_pinned<BF16, VEC>(lp + (j + 2) * SH::CB_BYTES, nxt[(j - j0) & 1]);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) gr[v] = in ? gr[v] : 0.f;
                    }
                    if (j >= P && j < P + RW) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) c[v] += gr[v];
                    }
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        if (j - u >= 0 && j - u < K) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) a[v][j - u] = __builtin_fmaf(b[u][v], gr[v], a[v][j - u]);
                        }
                    }
                    pin_row(std::integral_constant<int, j>{});
                    slot(std::integral_constant<int, j>{});
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
        });
    };

    // Gated forward: the u and g rows of a landed tile become one fp32 h = u * silu(g) tile, once per staged element
    // (a gate evaluated as the schedules read their rows would be evaluated NJ / RW times per element). A unit of work
    // is one wave-column of one staged row, dealt round-robin to the waves: a lane takes its 4 bytes of u and of g
    // (two adjacent channels in bf16, one in fp32) and the wave leaves the fp32 values of the wave-column's first 64
    // channels in the unit's 256 bytes of the u tile and the rest in its 256 bytes of the g tile (fp32 activations: all
    // in the u tile), which is where the schedules' lanes read their slices. All reads of a unit are one instruction
    // of the wave and precede its writes, so the unit is turned in place. Volatile address-space-3 accesses: the waves
    // have stores of the previous tile in flight, and before an ordinary LDS access the compiler would wait for them.
    auto gate_tile = [&](char* buf) __attribute__((always_inline)) {
        typedef volatile __attribute__((address_space(3))) uint32_t lds_u32;
        for (int unit = wv; unit < SH::ROW_UNITS; unit += SH::NW) {
            char* pu = buf + (unit / NCW) * SH::CB_BYTES + (unit % NCW) * 256;
            char* pg = pu + SH::IN_BYTES;
            const uint32_t ru = *(lds_u32*)(pu + lane * 4), rg_ = *(lds_u32*)(pg + lane * 4);
            if constexpr (BF16) {
                const u32x2 h = {__float_as_uint(gate_mul(bf16_lo(ru), bf16_lo(rg_))), __float_as_uint(gate_mul(bf16_hi(ru), bf16_hi(rg_)))};
                *(volatile __attribute__((address_space(3))) u32x2*)((lane < 32 ? pu : pg) + (lane & 31) * 8) = h;
            } else {
                *(lds_u32*)(pu + lane * 4) = __float_as_uint(gate_mul(__uint_as_float(ru), __uint_as_float(rg_)));
            }
        }
    };
    // where a lane's slice of staged row 0 of the wave-column lies in a tile
    const int lane_off = !GF ? lc0 * E : wc * 256 + (BF16 ? (lane < 32 ? 0 : SH::IN_BYTES) + (lane & 31) * 8 : lane * 4);

    int q = tb;
    for (int it = 0; it < ntl; ++it) {
        const int t0 = lds_tile_row0(g, it, q, R);
        const int qn = lds_next_slot(g, q);
        char* cur = lds_raw + (it & 1) * SH::BUF_BYTES;
        const int rn = it + 1 < ntl ? lds_tile_row0(g, it + 1, qn, R) : T;
        const int tf = t0 + rg * RW;
        if constexpr (GF) {
            if (t0 < T) gate_tile(cur);
            lds_barrier();                          // every wave's share of h is written
        }
        __builtin_amdgcn_s_setprio(3);
        if constexpr (LOADS) {
            // an interior wave runs every row of its schedule exactly once: its loads go into the schedule's slots
            spread = rn < T && tf < T && interior;
            if (rn < T) {
                stage_begin(lds_raw + ((it + 1) & 1) * SH::BUF_BYTES, rn);
                if (!spread) {
                    for (int n = 0; n < NPW; ++n) stage_one(n);
                }
            }
        }
        if (tf < T) {
            const int loff = (rg * RW) * SH::CB_BYTES + lane_off;
            const char* lpi = cur + loff;                              // taps: staged row j <-> global row tf - P + j
            const char* lpx = cur + SH::IN_BYTES + loff;               // backward x: row u <-> global row tf + u
            lpx_cur = lpx;
            ro = rows_rsrc(out, tf, T, x_row_bytes);
            // role 0: store output rows [u0, u1) of the wave from b
            auto store_rows = [&](int u0, int u1) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < RW; ++u) {
                    if constexpr (GB) {
                        if (u >= u0 && u < u1) emit_row(u, b[u]);
                    } else {
                        Row o;
                        o.from_f32(b[u]);
                        if (u >= u0 && u < u1 && active) o.bstore(ro, out_voff, u * rowb);
                    }
                }
            };
            if constexpr (ROLE == 0) {
                if (interior) {
#pragma unroll
                    for (int u = 0; u < RW; ++u)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) b[u][v] = c[v];
                    run_rows(lpi, std::true_type{}, 0, NJ);
                } else {
                    SeqCursor sq = sc;                      // positioned on row tf
                    int u0 = 0;
                    bool fresh = true;
                    while (u0 < RW && tf + u0 < T) {
                        advance_prefetched(sq, nce, fresh, cu, S, T, tf + u0);
                        int jlo = sq.cs - (tf - P), jhi = sq.ce - (tf - P), u1 = sq.ce - tf;
                        jlo = __builtin_amdgcn_readfirstlane(jlo < 0 ? 0 : jlo);
                        jhi = __builtin_amdgcn_readfirstlane(jhi > NJ ? NJ : jhi);
                        u1 = __builtin_amdgcn_readfirstlane(u1 > RW ? RW : u1);
#pragma unroll
                        for (int u = 0; u < RW; ++u)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) b[u][v] = c[v];
                        run_rows(lpi, std::false_type{}, jlo, jhi);
                        store_rows(u0, u1);
                        u0 = u1;
                    }
                }
            } else {
                // The passes below mask by multiplying with zeros (x rows of other sequences are zeroed, dy rows of other
                // sequences are zeroed in the conversion), which turns an Inf or NaN on the other side into a NaN in a
                // tap sum the product does not belong to. A boundary wave therefore first tests the rows it is about to
                // use (the sum of their squares is finite iff all of them are; a finite value beyond 1e19 overflows it
                // and merely takes the slow path too) and, if any is not finite, forms its sums one output row at a
                // time with every product behind a scalar branch: same products, same order, nothing multiplied by 0.
                bool exact = false;
                if (!interior) {
                    float chk = 0.f;
                    auto add_sq = [&](const Row& r) __attribute__((always_inline)) {
                        if constexpr (BF16 && VEC == 2) {
                            const bf16x2 pr = __builtin_bit_cast(bf16x2, r.d[0]);
                            chk = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, chk, false);
                        } else {
                            float f[VEC];
                            r.to_f32(f);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) chk = __builtin_fmaf(f[v], f[v], chk);
                        }
                    };
                    static_for<NJ>([&](auto j_c) __attribute__((always_inline)) {
                        Row r;
                        r.load(lpi + decltype(j_c)::value * SH::CB_BYTES);
                        add_sq(r);
                    });
                    static_for<RW>([&](auto u_c) __attribute__((always_inline)) {
                        Row r;
                        r.load(lpx + decltype(u_c)::value * SH::CB_BYTES);
                        add_sq(r);
                        if constexpr (GB) {         // h = u * silu(g) is finite when u and g are (up to overflow, see above)
                            r.load(lpx + SH::X_BYTES + decltype(u_c)::value * SH::CB_BYTES);
                            add_sq(r);
                        }
                    });
                    exact = __builtin_amdgcn_ballot_w64(!__builtin_isfinite(chk)) != 0;
                }
                if (exact) {
                    SeqCursor sq = sc;
                    bool fresh = true;
#pragma nounroll
                    for (int u = 0; u < RW; ++u) {
                        const int t = tf + u;
                        if (t >= T) break;
                        advance_prefetched(sq, nce, fresh, cu, S, T, t);
                        int jlo = sq.cs - (tf - P), jhi = sq.ce - (tf - P);      // staged rows of row t's sequence
                        jlo = __builtin_amdgcn_readfirstlane(jlo < 0 ? 0 : jlo);
                        jhi = __builtin_amdgcn_readfirstlane(jhi > NJ ? NJ : jhi);
                        float xv[VEC], gc[VEC];
                        read_x_row(u, xv);
                        lds_read_row<BF16, VEC>(lpi + (u + P) * SH::CB_BYTES, gc);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) c[v] += gc[v];
                        static_for<K>([&](auto m_c) __attribute__((always_inline)) {
                            constexpr int m = decltype(m_c)::value;
                            if (u + m >= jlo && u + m < jhi) {
                                float gr[VEC];
                                lds_read_row<BF16, VEC>(lpi + (u + m) * SH::CB_BYTES, gr);
#pragma unroll
                                for (int v = 0; v < VEC; ++v) a[v][m] = __builtin_fmaf(xv[v], gr[v], a[v][m]);
                            }
                        });
                    }
                }
                // one code path for interior and boundary tiles (two regions that both update the K tap sums make the
                // register allocator keep them twice): one pass per sequence that owns output rows of the wave; an
                // interior tile is the single pass over all rows
                SeqCursor sq = sc;
                int u0 = exact ? RW : 0;
                bool fresh = true;
                while (u0 < RW && tf + u0 < T) {
                    int jlo = 0, jhi = NJ, u1 = RW;
                    if (!interior) {
                        advance_prefetched(sq, nce, fresh, cu, S, T, tf + u0);
                        jlo = sq.cs - (tf - P); jhi = sq.ce - (tf - P); u1 = sq.ce - tf;
                        jlo = __builtin_amdgcn_readfirstlane(jlo < 0 ? 0 : jlo);
                        jhi = __builtin_amdgcn_readfirstlane(jhi > NJ ? NJ : jhi);
                        u1 = __builtin_amdgcn_readfirstlane(u1 > RW ? RW : u1);
                    }
#pragma unroll
                    for (int u = 0; u < RW; ++u) read_x_row(u, b[u]);
                    if (!interior) {
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (!(u >= u0 && u < u1)) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) b[u][v] = 0.f;
                            }
                        }
                    }
                    run_rows_chunked(lpi, jlo, jhi);
                    u0 = u1;
                }
            }
        }
        if (it + 1 < ntl) {
            if (use_tab && it + 1 < SH::TAB_TILES)
                interior = wave_locate_from<RW, P>(sc, nce, cu, S, T, rn, rn + rg * RW, __builtin_amdgcn_readfirstlane(seq_tab[it + 1]));
            else
                interior = wave_locate<RW, P>(sc, nce, cu, S, T, rn + rg * RW);
        }
        if constexpr (LOADS) wait_vmem_all();   // this wave's share of the next tile has landed
        __syncthreads();   // so has everybody else's; this tile's buffer may be overwritten
        q = qn;
    }

    if constexpr (FWD) return;
    // ---- block-level pass: sum the NRG row groups of each wave-column, group order 0,1,2,... ----
    float* slab = partial + (size_t)tb * (K + 1) * C;
    float* red = reinterpret_cast<float*>(lds_raw);   // [NW][VEC][64]; the tiles are dead after the last barrier
#pragma unroll
    for (int i = 0; i <= K; ++i) {
        float val[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) val[v] = (i < K) ? a[v][i < K ? i : 0] : c[v];
        if (ROLE == 1 && rg > 0) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) red[(wv * VEC + v) * 64 + lane] = val[v];
        }
        __syncthreads();
        if (ROLE == 1 && rg == 0) {
#pragma unroll
            for (int j = 1; j < NRG; ++j) {
                const int ow = SH::wave_of(1, j * NCW + wc);
#pragma unroll
                for (int v = 0; v < VEC; ++v) val[v] += red[(ow * VEC + v) * 64 + lane];
            }
            if (active) {
                const int kk = (i < K) ? K - 1 - i : K;
                float* dst = slab + (size_t)kk * C + c0;
#pragma unroll
                for (int v = 0; v < VEC; ++v) dst[v] = val[v];
            }
        }
        __syncthreads();
    }
}

template <bool BF16, int K, int VEC, int RW, int NRG, int NCW>
__global__ void __launch_bounds__(NCW * 2 * NRG * 64)
dwconv_bwd_split_kernel(const void* __restrict__ x, const void* __restrict__ dy, const int32_t* __restrict__ cu,
                        const void* __restrict__ w, void* __restrict__ dx, float* __restrict__ partial, const LdsGeo g) {
    if (SplitShape<BF16, K, VEC, RW, NRG, NCW>::role_of(wave_id()) == 0)
        split_role<BF16, K, VEC, RW, NRG, NCW, false, 0>(dy, x, cu, w, nullptr, dx, partial, g);
    else
        split_role<BF16, K, VEC, RW, NRG, NCW, false, 1>(dy, x, cu, w, nullptr, dx, partial, g);
}

// x = z = [u | g] [T, 2C], dx = dz [T, 2C]
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW>
__global__ void __launch_bounds__(NCW * 2 * NRG * 64)
dwconv_bwd_split_gated_kernel(const void* __restrict__ z, const void* __restrict__ dy, const int32_t* __restrict__ cu,
                              const void* __restrict__ w, void* __restrict__ dz, float* __restrict__ partial, const LdsGeo g) {
    if (SplitShape<BF16, K, VEC, RW, NRG, NCW, false, true>::role_of(wave_id()) == 0)
        split_role<BF16, K, VEC, RW, NRG, NCW, false, 0, true>(dy, z, cu, w, nullptr, dz, partial, g);
    else
        split_role<BF16, K, VEC, RW, NRG, NCW, false, 1, true>(dy, z, cu, w, nullptr, dz, partial, g);
}

// x = z = [u | g] [T, 2C]: y = bias + conv(u * silu(g))
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW>
__global__ void __launch_bounds__(NCW * NRG * 64)
dwconv_fwd_split_gated_kernel(const void* __restrict__ z, const int32_t* __restrict__ cu, const void* __restrict__ w,
                              const void* __restrict__ bias, void* __restrict__ y, const LdsGeo g) {
    split_role<BF16, K, VEC, RW, NRG, NCW, true, 0, true>(z, nullptr, cu, w, bias, y, nullptr, g);
}

template <bool BF16, int K, int VEC, int RW, int NRG, int NCW>
__global__ void __launch_bounds__(NCW * NRG * 64)
dwconv_fwd_split_kernel(const void* __restrict__ x, const int32_t* __restrict__ cu, const void* __restrict__ w,
                        const void* __restrict__ bias, void* __restrict__ y, const LdsGeo g) {
    split_role<BF16, K, VEC, RW, NRG, NCW, true, 0>(x, nullptr, cu, w, bias, y, nullptr, g);
}

}  // namespace nplm
