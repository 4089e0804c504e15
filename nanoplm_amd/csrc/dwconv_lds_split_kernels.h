// LDS-staged fused backward for K = 31 in which every wave computes and the two outputs have their own waves
// (gfx950, wave64).
//
// At K = 31 the backward issues 62 FMAs per element and is bound by the vector ALU as much as by HBM. A SIMD issues
// FMAs near its rate only when 4 of its waves are in an FMA stream at once (measured on a register-only loop: one
// wave-instruction per 3.3 cycles with 2 waves per SIMD, per 2.4 with 4): that allows 128 registers per lane, where
// one wave holding K weights and K dw sums per channel needs 166, and it rules out idle loader waves, which cost as
// many registers as a compute wave. So here
//   * every wave computes, and at the top of a tile issues its share of the direct global->LDS loads of the NEXT
//     tile (dy with K-1 halo rows, x without) into the other buffer; the loads land while the tile is computed;
//   * the two outputs go to two kinds of wave that share the staged dy tile:
//       role 0 (dx):    dx[t] = sum_m w[K-1-m] * dy[t-P+m]           holds K weights + RW row sums
//       role 1 (dw/db): dw[K-1-m] += x[t] * dy[t-P+m], db += dy[t]   holds K tap sums + RW x rows
//     Neither needs the other's registers, nothing is exchanged, and both run the same unrolled schedule over the
//     RW+K-1 staged rows of their RW output rows. dx sums its taps in the order of the sliding-window kernel (same bits).
// Tiles, rounds, slot rotation and XCD grouping are those of the other LDS-staged kernels (dwconv_lds_kernels.h);
// dw/db leave the block as in those (row groups summed through LDS in fixed order, one slab per token block, then
// dwconv_finalize_kernel). No atomics; every sum has a fixed order.
//
// Sequence boundaries: a wave whose rows and taps all lie in one sequence runs unmasked. Otherwise it makes one pass
// per sequence that owns some of its output rows, over the staged rows of that sequence: the dx role skips the other
// rows by scalar branches and stores the sequence's output rows at the end of the pass; the dw role loads the x rows
// of the sequence (zero for the others), skips chunks of staged rows that hold none of the sequence's and selects a
// zero for single rows of another sequence inside a chunk.
//
// No counterpart in the reference (peymanvahidi/nanoplm 0.1.6 has no convolution); tensor contract:
// modeling.py:339,421-439 and collator.py:322-325,405-458.
#pragma once
#include "dwconv_lds_kernels.h"

namespace nplm {

template <bool BF16, int K, int VEC, int RW, int NRG, int NCW>
struct SplitShape {
    static constexpr int E = BF16 ? 2 : 4;
    static constexpr int P = (K - 1) / 2;
    static constexpr int NROLE = 2;
    static constexpr int NW = NCW * NROLE * NRG;           // waves per block (all compute)
    static constexpr int NT = NW * 64;
    static constexpr int R = RW * NRG;                     // output rows per tile
    static constexpr int NROWS = R + K - 1;                // staged dy rows per tile
    static constexpr int NJ = RW + K - 1;                  // of which a wave reads this many
    static constexpr int CB_BYTES = NCW * 64 * VEC * E;    // bytes of a row in one column block
    static constexpr int CB_CH = NCW * 64 * VEC;
    static constexpr int CPR = CB_BYTES / 16;              // 16-byte chunks per staged row
    static constexpr int IN_BYTES = NROWS * CB_BYTES;      // dy tile
    static constexpr int X_BYTES = R * CB_BYTES;           // x tile, no halo
    static constexpr int BUF_BYTES = IN_BYTES + X_BYTES;
    static constexpr int LDS_BYTES = 2 * BUF_BYTES;
    static_assert(CB_BYTES == 256 || CB_BYTES == 512 || CB_BYTES == 1024, "a staged row is 16, 32 or 64 chunks");
    static_assert(NW <= 16, "at most 1024 threads per block");
    static_assert(LDS_BYTES <= kLdsBytes, "two tile buffers must fit in LDS");
    static_assert(NJ * CB_BYTES <= 65536, "ds_read immediate offsets (a wave reads NJ rows from one base) are 16 bit");
    static_assert(NW * VEC * 64 * 4 <= LDS_BYTES, "the final reduction reuses the tile buffers");
};

// Stage rows first_row .. first_row+nrows-1 (clamped to [0,T)) x this block's column block of `src` into
// `dst` (row pitch CB_BYTES): the tile is one run of nrows*CPR 16-byte chunks, chunk 64*i + lane belongs
// to load i, and loads i = w0, w0 + nw, ... to this wave. A load covers 64/CPR adjacent rows, each lane
// forming its own (clamped) row offset. Staged rows in [edge, nrows-edge) are read by no other tile.
template <typename SH, int ONCE_AUX>
__device__ __forceinline__ void stage_rows_flat(const void* __restrict__ src, char* dst, int first_row, int nrows, int T,
                                                size_t row_bytes, int col_byte0, int valid_bytes, int w0, int nw, int lane,
                                                int edge) {
    constexpr int CPR = SH::CPR, RPL = 64 / CPR;          // rows per load
    const int rb = first_row > 0 ? first_row : 0;
    const rsrc_t rs = rows_rsrc(src, rb, T, row_bytes);
    const int rowb = (int)row_bytes;
    const int lrow = lane / CPR, lchunk = lane % CPR;
    const int nloads = (nrows + RPL - 1) / RPL;
    for (int i = w0; i < nloads; i += nw) {
        const int j = i * RPL + lrow;                    // staged row of this lane
        const int voff = (clamp_row(first_row + j, T) - rb) * rowb + col_byte0 + lchunk * 16;
        char* d = dst + i * 1024;                         // base of the load in LDS: lanes land 16 bytes apart
        const bool once = i * RPL >= edge && i * RPL + RPL <= nrows - edge;
        if (j < nrows && lchunk * 16 < valid_bytes) load_to_lds<ONCE_AUX>(rs, d, voff, 0, once);
    }
}

// One lane's slice of a staged row, read with a volatile access: the compiler may neither hoist it out of its
// place in the unrolled schedule (all reads of a tile at the top would need NJ registers) nor merge it with
// the same read on another path.
template <bool BF16, int VEC>
__device__ __forceinline__ void lds_read_pinned(const char* p, RowVec<BF16, VEC>& r) {
    if constexpr (RowVec<BF16, VEC>::BYTES == 2) {
        r.h = *(const volatile __attribute__((address_space(3))) uint16_t*)p;
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
// in = dy, other = x, out = dx, partial = dw/db slabs.
template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, int ROLE>
__device__ __forceinline__ void split_role(const void* __restrict__ in, const void* __restrict__ other,
                                           const int32_t* __restrict__ cu, const void* __restrict__ w,
                                           void* __restrict__ out, float* __restrict__ partial, const LdsGeo& g) {
    using SH = SplitShape<BF16, K, VEC, RW, NRG, NCW>;
    constexpr int P = SH::P, E = SH::E, R = SH::R, NJ = SH::NJ, NROLE = SH::NROLE;
    using Row = RowVec<BF16, VEC>;
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];   // 2 x BUF_BYTES

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const int wc = wv % NCW;
    const int rg = wv / (NCW * NROLE);
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

    auto stage_tile = [&](char* buf, int t0) __attribute__((always_inline)) {
        stage_rows_flat<SH, kLoadAuxOnceBwd>(in, buf, t0 - P, SH::NROWS, T, row_bytes, col_byte0, valid_bytes, wv, SH::NW, lane,
                                             2 * P);
        // the x loads start where the dy loads ended, so that both tensors spread over all waves
        constexpr int NLD = (SH::NROWS + 64 / SH::CPR - 1) / (64 / SH::CPR);
        const int w0x = (wv + SH::NW - NLD % SH::NW) % SH::NW;
        stage_rows_flat<SH, kLoadAuxOnceBwdX>(other, buf + SH::IN_BYTES, t0, R, T, row_bytes, col_byte0, valid_bytes, w0x,
                                              SH::NW, lane, 0);
    };

    // role 0: a[v][m] = w[K-1-m], the weight of staged row u + m for output row u;   b = row sums of dx
    // role 1: a[v][m] = sum over rows of x[t] * dy[t-P+m] (= dw[K-1-m]);              b = x rows
    float a[VEC][K];
    float b[RW][VEC];
    float c[VEC];          // role 0: zero (what a row sum starts from); role 1: db
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        c[v] = 0.f;
#pragma unroll
        for (int m = 0; m < K; ++m) a[v][m] = 0.f;
    }
    if constexpr (ROLE == 0) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
#pragma unroll
            for (int m = 0; m < K; ++m) {
                const size_t wi = (size_t)(c0 + v) * K + (K - 1 - m);
                float t = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[wi]) : reinterpret_cast<const float*>(w)[wi];
                if (m == P && (g.w_flags & W_RESIDUAL)) t += 1.f;
                a[v][m] = t;
            }
        }
    }
    stage_tile(lds_raw, tb * R);
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    int nce = 0;
    bool interior = wave_locate<RW, P>(sc, nce, cu, S, T, tb * R + rg * RW);
    wait_vmem_all();       // this wave's share of the first tile has landed
    __syncthreads();

    // the unrolled schedule over staged rows [jlo, jhi) of the wave's window (all NJ rows when UNMASKED):
    // row j feeds output rows u = j-K+1 .. j with tap m = j - u
    auto run_rows = [&](const char* lp, auto unmasked_c, auto role_c, int jlo, int jhi) __attribute__((always_inline)) {
        constexpr bool UNMASKED = decltype(unmasked_c)::value;
        constexpr int RROLE = decltype(role_c)::value;
        Row nxt[2];
        if constexpr (UNMASKED) {
            lds_read_pinned<BF16, VEC>(lp, nxt[0]);
            lds_read_pinned<BF16, VEC>(lp + SH::CB_BYTES, nxt[1]);
        }
        // (a compile-time loop: as an ordinary loop its unrolled body is too large for the unroller at K = 31, and
        // the register arrays would then be indexed at run time and live in scratch memory)
        static_for<NJ>([&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            if (UNMASKED || (j >= jlo && j < jhi)) {
                float gr[VEC];
                if constexpr (UNMASKED) {
                    // two rows ahead in registers; the scheduling barrier below keeps the compiler from hoisting
                    // all NJ reads to the top, which would not fit the 128 registers of 4 waves per SIMD
                    nxt[j & 1].to_f32(gr);
                    if (j + 2 < NJ) lds_read_pinned<BF16, VEC>(lp + (j + 2) * SH::CB_BYTES, nxt[j & 1]);
                } else {
                    lds_read_row<BF16, VEC>(lp + j * SH::CB_BYTES, gr);
                }
                if (RROLE == 1 && j >= P && j < P + RW) {   // centre row of output row j - P
#pragma unroll
                    for (int v = 0; v < VEC; ++v) c[v] += gr[v];
                }
#pragma unroll
                for (int u = 0; u < RW; ++u) {
                    if (j - u >= 0 && j - u < K) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            if (RROLE == 0) b[u][v] = __builtin_fmaf(a[v][j - u], gr[v], b[u][v]);
                            else a[v][j - u] = __builtin_fmaf(b[u][v], gr[v], a[v][j - u]);
                        }
                    }
                }
                // pin this row's arithmetic here: every sum it touched passes through an empty volatile asm, which
                // is ordered with the (volatile) row reads, so the FMAs of row j stay between the reads of rows
                // j + 2 and j + 3
                if constexpr (UNMASKED) {
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        if (j - u >= 0 && j - u < K) {
                            if (RROLE == 0) pin_regs<VEC>(b[u]);
                            else {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) asm volatile("" : "+v"(a[v][j - u]) : : "memory");
                            }
                        }
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // dw role at a boundary: the staged rows in chunks of CH; a chunk with no row of the pass's sequence is skipped by one
    // scalar branch, inside a chunk a row of another sequence contributes a selected zero. (One branch per row, as in
    // the dx role, makes the register allocator keep two copies of the K tap sums per channel.)
    auto run_rows_chunked = [&](const char* lp, int jlo, int jhi) __attribute__((always_inline)) {
        constexpr int CH = 12, NCH = (NJ + CH - 1) / CH;
        static_for<NCH>([&](auto ch_c) __attribute__((always_inline)) {
            constexpr int j0 = decltype(ch_c)::value * CH;
            constexpr int j1 = j0 + CH < NJ ? j0 + CH : NJ;
            if (j0 < jhi && j1 > jlo) {
                Row nxt[2];     // two rows ahead in registers, as in run_rows
                lds_read_pinned<BF16, VEC>(lp + j0 * SH::CB_BYTES, nxt[0]);
                if (j0 + 1 < j1) lds_read_pinned<BF16, VEC>(lp + (j0 + 1) * SH::CB_BYTES, nxt[1]);
                static_for<j1 - j0>([&](auto jj_c) __attribute__((always_inline)) {
                    constexpr int j = j0 + decltype(jj_c)::value;
                    const bool in = j >= jlo && j < jhi;
                    float gr[VEC];
                    nxt[(j - j0) & 1].to_f32(gr);
                    if (j + 2 < j1) lds_read_pinned<BF16, VEC>(lp + (j + 2) * SH::CB_BYTES, nxt[(j - j0) & 1]);
#pragma unroll
                    for (int v = 0; v < VEC; ++v) gr[v] = in ? gr[v] : 0.f;
                    if (j >= P && j < P + RW) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) c[v] += gr[v];
                    }
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        if (j - u >= 0 && j - u < K) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) {
                                a[v][j - u] = __builtin_fmaf(b[u][v], gr[v], a[v][j - u]);
                                asm volatile("" : "+v"(a[v][j - u]) : : "memory");
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
        });
    };

    int q = tb;
    for (int it = 0; it < ntl; ++it) {
        const int t0 = lds_tile_row0(g, it, q, R);
        const int qn = lds_next_slot(g, q);
        char* cur = lds_raw + (it & 1) * SH::BUF_BYTES;
        const int rn = it + 1 < ntl ? lds_tile_row0(g, it + 1, qn, R) : T;
        if (rn < T) stage_tile(lds_raw + ((it + 1) & 1) * SH::BUF_BYTES, rn);
        const int tf = t0 + rg * RW;
        if (tf < T) {
            const int loff = (rg * RW) * SH::CB_BYTES + lc0 * E;
            const char* lpi = cur + loff;                              // taps: staged row j <-> global row tf - P + j
            const char* lpx = cur + SH::IN_BYTES + loff;               // backward x: row u <-> global row tf + u
            const rsrc_t ro = rows_rsrc(out, tf, T, row_bytes);
            // role 0: store output rows [u0, u1) of the wave from b
            auto store_rows = [&](int u0, int u1) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < RW; ++u) {
                    Row o;
                    o.from_f32(b[u]);
                    if (u >= u0 && u < u1 && active) o.bstore(ro, out_voff, u * rowb);
                }
            };
            if constexpr (ROLE == 0) {
                if (interior) {
#pragma unroll
                    for (int u = 0; u < RW; ++u)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) b[u][v] = c[v];
                    run_rows(lpi, std::true_type{}, std::integral_constant<int, 0>{}, 0, NJ);
                    store_rows(0, RW);
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
                        run_rows(lpi, std::false_type{}, std::integral_constant<int, 0>{}, jlo, jhi);
                        store_rows(u0, u1);
                        u0 = u1;
                    }
                }
            } else {
                // one code path for interior and boundary tiles (two regions that both update the K tap sums make the
                // register allocator keep them twice): one pass per sequence that owns output rows of the wave; an
                // interior tile is the single pass over all rows
                SeqCursor sq = sc;
                int u0 = 0;
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
                    for (int u = 0; u < RW; ++u) {
                        lds_read_row<BF16, VEC>(lpx + u * SH::CB_BYTES, b[u]);
                        if (!(u >= u0 && u < u1)) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) b[u][v] = 0.f;
                        }
                    }
                    run_rows_chunked(lpi, jlo, jhi);
                    u0 = u1;
                }
            }
        }
        if (it + 1 < ntl) interior = wave_locate<RW, P>(sc, nce, cu, S, T, lds_tile_row0(g, it + 1, qn, R) + rg * RW);
        wait_vmem_all();   // this wave's share of the next tile has landed
        __syncthreads();   // so has everybody else's; this tile's buffer may be overwritten
        q = qn;
    }

    // ---- block-level pass: sum the NRG row groups of each role-1 wave-column, group order 0,1,2,... ----
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
                const int ow = (j * NROLE + 1) * NCW + wc;
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
    if ((wave_id() / NCW) % 2 == 0) split_role<BF16, K, VEC, RW, NRG, NCW, 0>(dy, x, cu, w, dx, partial, g);
    else split_role<BF16, K, VEC, RW, NRG, NCW, 1>(dy, x, cu, w, dx, partial, g);
}

}  // namespace nplm
