// LayerNorm fused into the forward of the varlen depthwise conv (gfx950, wave64), for rows that fit one column block.
//
//     n[t,c] = (x[t,c] - mean[t]) * rstd[t] * gamma[c] + beta[c]        mean, rstd over the C channels of row t
//     y[t,c] = b[c] + sum_k w[c,k] * n[t+k-P,c]  (+ x[t,c] with the residual flag)     inside the sequence of t
//
// The pre-norm block of the reference normalises the residual stream before every sub-module
// (src/nanoplm/pretraining/models/modern_bert/modeling.py:408-414) and adds the sub-module's output back to it; with a
// conv as the sub-module the unfused sequence is LayerNorm (read x, write n), conv (read n, write y), add (read x and
// y, write): 7 passes over [T, C], of which this kernel keeps 2 (read x, write y) and n is never in memory.
//
// A block owns whole rows (one column block: 2 KiB in 4 wave-columns and 16-row tiles, or, for fp32 rows, 4 KiB in 8
// wave-columns and tiles of 14 - K rows, see lds_ln_shape() and lds_ln_4k_shape()), so the row statistics come out of
// the staged tile.
// Three tile buffers: one being computed, one having its statistics taken, one in flight. A loader wave stages whole
// rows (rows lw, lw + NWL, ... of a tile), waits by count for its own loads of the tile before the newest one, and takes
// the statistics of exactly those rows while the compute waves are on the previous tile (a row is 2 x 64 chunks of
// 16 bytes; the rows' sums and then their squared deviations are reduced over the wave, see ln_stats_pass) and leaves
// (rstd, -mean * rstd, mean) per staged row in LDS, together with the sequence bounds of the tile's row groups. The
// compute waves normalise as they read (2 FMAs per value read), write (mean, rstd) of their own rows to `stats` in
// memory, which is what a LayerNorm backward needs, and otherwise run the forward of dwconv_lds_kernels.h: unmasked
// schedule inside a sequence, one select per tap at a boundary. Tiles, rounds, slot rotation and XCD grouping as in
// the other LDS-staged kernels.
// Measured (T=131072, C=1024, K=7, bf16, MI355X): 100 us, against 455 us for torch.layer_norm in bf16 + this
// library's conv + add, and 90 us for the conv alone; the vector ALU is the limit (statistics and normalisation of the
// K-1 halo rows of every 16-row tile included). fp32, C=1024 (rows of 4 KiB): 226 us against 174 us for the conv alone;
// there a tile period is as long as its loads take to arrive (13 staged rows per 7 output rows), not the vector ALU.
//
// No counterpart in the reference (peymanvahidi/nanoplm 0.1.6 has no convolution); the LayerNorm is
// torch.nn.LayerNorm's (modeling.py:408-414: eps and bias from the config, 1e-5 and none by default, modeling.py:51-52).
#pragma once
#include "dwconv_lds_kernels.h"

namespace nplm {

struct LnArgs {
    const void* gamma;   // [C], weight dtype
    const void* beta;    // [C] or null
    float* stats;        // [T][2] fp32 (mean, rstd) or null
    float eps;
};

// LDS accesses of the loader waves while their direct global->LDS loads of another buffer are in flight: through a
// volatile address-space-3 pointer. For an ordinary LDS access the compiler first waits for every outstanding vector
// memory operation (it cannot tell which LDS bytes a direct load will write), which would make the statistics of a
// tile wait for the tile in flight behind it.
template <bool BF16, int CE>
__device__ __forceinline__ void lds_read_chunk_pinned(const char* p, float (&f)[CE]) {
    static_assert(CE * (BF16 ? 2 : 4) == 16, "one 16-byte chunk");
    const u32x4 t = *(const volatile __attribute__((address_space(3))) u32x4*)p;
    if constexpr (BF16) {
        f[0] = bf16_lo(t.x); f[1] = bf16_hi(t.x); f[2] = bf16_lo(t.y); f[3] = bf16_hi(t.y);
        f[4] = bf16_lo(t.z); f[5] = bf16_hi(t.z); f[6] = bf16_lo(t.w); f[7] = bf16_hi(t.w);
    } else {
        f[0] = __uint_as_float(t.x); f[1] = __uint_as_float(t.y); f[2] = __uint_as_float(t.z); f[3] = __uint_as_float(t.w);
    }
}
__device__ __forceinline__ void lds_write16_pinned(void* p, float a, float b, float c, float d) {
    const u32x4 t = {__float_as_uint(a), __float_as_uint(b), __float_as_uint(c), __float_as_uint(d)};
    *(volatile __attribute__((address_space(3))) u32x4*)p = t;
}

template <int ROT>
__device__ __forceinline__ float dpp_row_ror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + ROT, 0xF, 0xF, false));
}
// Sums of up to four values over the 64 lanes of a wave as a reduce-scatter (see wave_sums16 in dwconv_lds_kernels.h):
// the halves of the wave exchange and add (values 0, 1 stay in lanes 0-31, values 2, 3 in lanes 32-63), then the rows of
// each half (even rows go on with the first of their two values, odd rows with the second), then four rotations inside
// every row of 16 lanes: every lane of row r ends with the total of value r. 10 instructions for all four.
__device__ __forceinline__ float wave_sums4(const float (&v)[4]) {
    typedef unsigned u2x __attribute__((ext_vector_type(2)));
    const u2x r02 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[0]), __float_as_uint(v[2]), false, false);
    const u2x r13 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[1]), __float_as_uint(v[3]), false, false);
    const float a = __uint_as_float(r02.x) + __uint_as_float(r02.y);
    const float b = __uint_as_float(r13.x) + __uint_as_float(r13.y);
    const u2x rr = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    float t = __uint_as_float(rr.x) + __uint_as_float(rr.y);
    t += dpp_row_ror<8>(t);
    t += dpp_row_ror<4>(t);
    t += dpp_row_ror<2>(t);
    t += dpp_row_ror<1>(t);
    return t;
}

// Statistics of NB staged rows of a loader wave (rows lw, lw + nlw, ...): two passes over the wave's registers - the
// rows' sums, reduced over the wave, give the means; the squared deviations from those means, reduced the same way,
// the variances - and (rstd, -mean * rstd, mean) per row left in LDS.
template <typename SH, bool BF16, int NB, bool FULLROW>
__device__ __forceinline__ void ln_stats_pass(const char* buf, float4* st, int lw, int nlw, int lane, int C, float eps) {
    static_assert(NB <= 4, "the rows of a loader wave are reduced four at a time");
    constexpr int CE = 16 / SH::E;                        // elements per 16-byte chunk
    constexpr int NCHB = SH::CB_BYTES / 1024;             // chunks per lane and row of a full column block
    const int rowb = C * SH::E;
    const float inv_c = 1.f / (float)C;
    float mean[NB], var[NB];
    // straight-line code (all reads first, four partial sums per row) so that the rows' dependency chains overlap; lanes
    // whose chunk lies past the end of a narrow row select zeros
    auto local = [&](auto full_c, auto nch_c) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_c)::value;
        constexpr int NCH = decltype(nch_c)::value;       // chunks per lane and row that hold values of the row
        float v[NB][NCH][CE];
#pragma unroll
        for (int r = 0; r < NB; ++r) {
            // (a slot past the wave's last row re-reads the tile's last row, whatever its state; its result is dropped)
            const int j = lw + r * nlw < SH::NROWS ? lw + r * nlw : SH::NROWS - 1;
#pragma unroll
            for (int i = 0; i < NCH; ++i) lds_read_chunk_pinned<BF16, CE>(buf + j * SH::CB_BYTES + (lane + 64 * i) * 16, v[r][i]);
        }
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < NB; ++r) {
            float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const bool ok = FULL || (lane + 64 * i) * 16 < rowb;
#pragma unroll
                for (int e = 0; e < CE; ++e) {
                    if (!FULL) v[r][i][e] = ok ? v[r][i][e] : 0.f;
                    p[e & 3] += v[r][i][e];
                }
            }
            s[r] = (p[0] + p[1]) + (p[2] + p[3]);
        }
        const float tot = wave_sums4(s);
#pragma unroll
        for (int r = 0; r < NB; ++r) mean[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tot), 16 * r)) * inv_c;
        float q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < NB; ++r) {
            float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const bool ok = FULL || (lane + 64 * i) * 16 < rowb;
#pragma unroll
                for (int e = 0; e < CE; ++e) {
                    float t = v[r][i][e] - mean[r];
                    if (!FULL) t = ok ? t : 0.f;
                    p[e & 3] = __builtin_fmaf(t, t, p[e & 3]);
                }
            }
            q[r] = (p[0] + p[1]) + (p[2] + p[3]);
        }
        const float tq = wave_sums4(q);
#pragma unroll
        for (int r = 0; r < NB; ++r) var[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tq), 16 * r)) * inv_c;
    };
    // rows that fill the column block, rows one KiB short of it (the last piece is then never staged), anything else
    if (FULLROW || rowb == SH::CB_BYTES) local(std::true_type{}, std::integral_constant<int, NCHB>{});
    else if (NCHB > 1 && rowb == SH::CB_BYTES - 1024) local(std::true_type{}, std::integral_constant<int, (NCHB > 1 ? NCHB - 1 : 1)>{});
    else local(std::false_type{}, std::integral_constant<int, NCHB>{});
#pragma unroll
    for (int r = 0; r < NB; ++r) {
        const int j = lw + r * nlw;
        const float rstd = __builtin_amdgcn_rsqf(var[r] + eps);
        if (lane == 0 && j < SH::NROWS) lds_write16_pinned(st + j, rstd, -mean[r] * rstd, mean[r], 0.f);
    }
}

// Stage rows first_row .. first_row+NROWS-1 (clamped to [0,T)) of `src` into `dst`, whole rows per loader wave: wave
// lw takes rows lw, lw + nlw, ... with all their 1 KiB pieces, so that its own loads are all it has to wait for
// before it reads those rows. Every wave issues exactly NB * np loads with all 64 lanes, np the number of 1 KiB pieces
// that hold part of a row (a slot past the wave's last row loads that row again; a lane past the end of a narrow row
// re-reads the row's last 16 bytes into the unused tail of its piece), so that "all but the newest tile's loads have
// landed" is an s_waitcnt with one of NPIECE immediates (wait_but_tile). LDS pieces past np are never written.
template <typename SH, int NB>
__device__ __forceinline__ void stage_whole_rows(const void* __restrict__ src, char* dst, int first_row, int T, size_t row_bytes,
                                                 int valid_bytes, int np, int lw, int nlw, int lane) {
    const int rb = first_row > 0 ? first_row : 0;
    const rsrc_t rs = rows_rsrc(src, rb, T, row_bytes);
    const int rowb = (int)row_bytes;
    const int last = lw + ((SH::NROWS - 1 - lw) / nlw) * nlw;             // the wave's last row (lw < nlw <= NROWS)
#pragma unroll
    for (int r = 0; r < NB; ++r) {
        const int j = lw + r * nlw <= last ? lw + r * nlw : last;
        const int so = (clamp_row(first_row + j, T) - rb) * rowb;
        const bool once = j >= 2 * SH::P && j < SH::NROWS - 2 * SH::P;   // no other tile stages this row
#pragma unroll
        for (int p = 0; p < SH::NPIECE; ++p) {
            if (p < np) {
                int boff = p * 1024 + lane * 16;
                boff = boff < valid_bytes ? boff : valid_bytes - 16;
                load_to_lds<kLoadAuxOnceFwd>(rs, dst + j * SH::CB_BYTES + p * 1024, boff, so, once);
            }
        }
    }
}

template <bool BF16, int K, int VEC, int RW, int NRG, int NCW, int NWL, bool FULLROW>
__global__ void __launch_bounds__((NCW * NRG + NWL) * 64)
dwconv_ln_fwd_kernel(const void* __restrict__ x, const int32_t* __restrict__ cu, const void* __restrict__ w,
                     const void* __restrict__ b, void* __restrict__ y, const LnArgs ln, const LdsGeo g) {
    using SH = LdsShape<BF16, K, VEC, RW, NRG, NCW, NWL>;
    constexpr int P = SH::P, E = SH::E, R = SH::R;
    constexpr int BUF_BYTES = SH::TILE_BYTES;
    constexpr int NBUF = 3;     // one tile computed, one having its statistics taken, one in flight
    constexpr int NB = (SH::NROWS + NWL - 1) / NWL;       // staged rows per loader wave
    using Row = RowVec<BF16, VEC>;
    static_assert(SH::CB_BYTES % 1024 == 0, "whole 1 KiB pieces");
    static_assert(NWL <= SH::NROWS, "every loader wave owns a row");
    // 3 x TILE_BYTES, then 3 x NROWS x (rstd, -mean*rstd, mean, 0), then 2 x NRG boundary records (cs, ce, nce, seq)
    extern __shared__ __attribute__((aligned(16))) char lds_raw[];
    float4* st_all = reinterpret_cast<float4*>(lds_raw + NBUF * BUF_BYTES);
    char* box = lds_raw + NBUF * BUF_BYTES + NBUF * SH::NROWS * 16;

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const bool is_loader = wv >= SH::NWC;
    int cb, tb;
    lds_block_coords(g, cb, tb);                           // ncb == 1: cb == 0
    const int T = g.T, S = g.S, C = g.C;
    const size_t row_bytes = (size_t)C * E;
    const int rowb = (int)row_bytes;
    const int valid_bytes = rowb;                          // <= CB_BYTES (host-checked)
    // 1 KiB pieces of a staged row that hold part of the row; FULLROW (rows that fill the column block, host-checked)
    // makes it, the counted wait and the statistics pass compile-time
    const int np = FULLROW ? SH::NPIECE : (rowb + 1023) >> 10;
    static_assert(SH::NPIECE <= 4, "wait_but_tile covers up to four pieces per row");
    // all of this wave's loads but the NB * np of the tile staged last have landed
    auto wait_but_tile = [&]() __attribute__((always_inline)) {
        if (np == 1) wait_vmem_but<NB>();
        else if (np == 2) wait_vmem_but<2 * NB>();
        else if (np == 3) wait_vmem_but<3 * NB>();
        else wait_vmem_but<4 * NB>();
    };
    const int ntl = (g.ntiles + g.nbt - 1) / g.nbt;

    const int wc = wv % NCW;
    const int rg = (wv / NCW) % NRG;
    const int lcol = (wc * 64 + lane) * VEC;
    const bool active = !is_loader && lcol < C;
    const int c0 = (lcol < C) ? lcol : C - VEC;
    const int out_voff = c0 * E;
    const bool residual = (g.w_flags & W_RESIDUAL) != 0;

    float wr[VEC][K];
    float bias[VEC], gam[VEC], bet[VEC];
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    // loader waves: locate the row groups of the tile that starts at row0 and post them in mailbox set `par` (a loader
    // takes row groups lw, lw + NWL, ... in rising order, so its cursor only moves forward). The compute waves then
    // issue no load of their own and never wait on the memory counter, which also counts their stores of y.
    auto post_bounds = [&](int par, int row0) {
        for (int r = wv - SH::NWC; r < NRG; r += NWL) {
            const int tf = row0 + r * RW;
            int ne = 0;
            if (tf < T) {
                sc.locate(cu, S, T, tf, sc.seq < 0 ? 0 : sc.seq);
                ne = (sc.seq + 1 < S) ? cu_at(cu, sc.seq + 2) : T;
            }
            if (lane == 0)
                lds_write16_pinned(box + (par * NRG + r) * 16, __int_as_float(sc.cs), __int_as_float(sc.ce), __int_as_float(ne),
                                   __int_as_float(sc.seq));
        }
    };
    if (is_loader) {
        const int lw = wv - SH::NWC;
        stage_whole_rows<SH, NB>(x, lds_raw, tb * R - P, T, row_bytes, valid_bytes, np, lw, NWL, lane);
        const int r1 = ntl > 1 ? lds_tile_row0(g, 1, lds_next_slot(g, tb), R) : T;
        if (r1 < T) stage_whole_rows<SH, NB>(x, lds_raw + BUF_BYTES, r1 - P, T, row_bytes, valid_bytes, np, lw, NWL, lane);
        post_bounds(0, tb * R);
        if (r1 < T) wait_but_tile(); else wait_vmem_all();           // this wave's rows of tile 0 have landed
        ln_stats_pass<SH, BF16, NB, FULLROW>(lds_raw, st_all, lw, NWL, lane, C, ln.eps);
    } else {
        load_weights<VEC, K>(w, g.w_flags & ~W_RESIDUAL, c0, wr);      // the identity is added from the raw x below
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            const bool wb = (g.w_flags & W_BF16) != 0;
            bias[v] = !b ? 0.f : wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(b)[c0 + v]) : reinterpret_cast<const float*>(b)[c0 + v];
            gam[v] = wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.gamma)[c0 + v]) : reinterpret_cast<const float*>(ln.gamma)[c0 + v];
            bet[v] = !ln.beta ? 0.f : wb ? bf16_to_f32(reinterpret_cast<const uint16_t*>(ln.beta)[c0 + v]) : reinterpret_cast<const float*>(ln.beta)[c0 + v];
        }
    }
    bool interior = true;
    int nce = 0;
    lds_barrier();

    int q = tb;
    int bcur = 0;               // buffer (and statistics set) of tile `it`
    for (int it = 0; it < ntl; ++it) {
        const int t0 = lds_tile_row0(g, it, q, R);
        const int qn = lds_next_slot(g, q);
        char* cur = lds_raw + bcur * BUF_BYTES;
        const float4* st = st_all + bcur * SH::NROWS;
        const int b1 = bcur + 1 == NBUF ? 0 : bcur + 1, b2 = b1 + 1 == NBUF ? 0 : b1 + 1;
        if (is_loader) {
            // tile it+2 into the buffer the last barrier freed; then the statistics of tile it+1, whose loads (issued
            // one round ago) are waited for by count, so that tile it+2 stays in flight meanwhile
            const int lw = wv - SH::NWC;
            const int r1 = it + 1 < ntl ? lds_tile_row0(g, it + 1, qn, R) : T;
            const int r2 = it + 2 < ntl ? lds_tile_row0(g, it + 2, lds_next_slot(g, qn), R) : T;
            if (r2 < T) stage_whole_rows<SH, NB>(x, lds_raw + b2 * BUF_BYTES, r2 - P, T, row_bytes, valid_bytes, np, lw, NWL, lane);
            if (r1 < T) post_bounds((it + 1) & 1, r1);
            if (r1 < T) {
                if (r2 < T) wait_but_tile(); else wait_vmem_all();
                ln_stats_pass<SH, BF16, NB, FULLROW>(lds_raw + b1 * BUF_BYTES, st_all + b1 * SH::NROWS, lw, NWL, lane, C, ln.eps);
            }
        } else {
            const int tf = t0 + rg * RW;
            if (tf < T && wc * 64 * VEC < C) {          // (a wave-column past the end of a narrow row has nothing to do)
                {
                    const u32x4 m = *(const volatile __attribute__((address_space(3))) u32x4*)(box + ((it & 1) * NRG + rg) * 16);
                    sc.cs = __builtin_amdgcn_readfirstlane((int)m.x);
                    sc.ce = __builtin_amdgcn_readfirstlane((int)m.y);
                    nce = __builtin_amdgcn_readfirstlane((int)m.z);
                    sc.seq = __builtin_amdgcn_readfirstlane((int)m.w);
                    const int tl = (tf + RW - 1 < T) ? tf + RW - 1 : T - 1;
                    interior = (tf - P >= sc.cs) && (tl + P < sc.ce);
                }
                float acc[RW][VEC];
#pragma unroll
                for (int u = 0; u < RW; ++u)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[u][v] = bias[v];
                const char* lp = cur + (rg * RW) * SH::CB_BYTES + c0 * E;
                const float4* sp = st + rg * RW;
                // (mean, rstd) of the wave's own rows for a LayerNorm backward, by the first wave-column
                if (ln.stats && wc == 0 && lane < RW && tf + lane < T) {
                    const u32x4 r = *(const volatile __attribute__((address_space(3))) u32x4*)(sp + P + lane);
                    ln.stats[2 * (size_t)(tf + lane)] = __uint_as_float(r.z);
                    ln.stats[2 * (size_t)(tf + lane) + 1] = __uint_as_float(r.x);
                }
                // staged row j of the wave's window: the raw values (for the residual) and the normalised ones
                auto read_row = [&](int j, float (&xr)[VEC], float (&nr)[VEC]) {
                    lds_read_pinned_row<BF16, VEC>(lp + j * SH::CB_BYTES, xr);
                    const u32x2 abu = *(const volatile __attribute__((address_space(3))) u32x2*)(sp + j);
                    const float2 ab = make_float2(__uint_as_float(abu.x), __uint_as_float(abu.y));
#pragma unroll
                    for (int v = 0; v < VEC; ++v) nr[v] = __builtin_fmaf(__builtin_fmaf(xr[v], ab.x, ab.y), gam[v], bet[v]);
                };
                if (interior) {
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float xr[VEC], nr[VEC];
                        read_row(j, xr, nr);
                        if (residual && j >= P && j < P + RW) {      // the centre row of output row j - P
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[j - P][v] += xr[v];
                        }
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[u][v] = __builtin_fmaf(wr[v][j - u], nr[v], acc[u][v]);
                            }
                        }
                    }
                } else {
                    // a boundary in the wave's window: every tap is selected (never multiplied by zero) by a bit of
                    // its output row's tap mask
                    uint32_t vm[RW];
                    wave_tap_masks<RW, K>(sc, nce, cu, S, T, tf, vm);
#pragma unroll
                    for (int j = 0; j < RW + K - 1; ++j) {
                        float xr[VEC], nr[VEC];
                        read_row(j, xr, nr);
                        if (residual && j >= P && j < P + RW) {
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[j - P][v] += xr[v];
                        }
#pragma unroll
                        for (int u = 0; u < RW; ++u) {
                            if (j - u >= 0 && j - u < K) {
                                const bool ok = (vm[u] >> (j - u)) & 1u;
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[u][v] = __builtin_fmaf(wr[v][j - u], ok ? nr[v] : 0.f, acc[u][v]);
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
        }
        lds_barrier();     // next tile and its statistics are in LDS; this tile's buffer may be overwritten
        bcur = b1;
        q = qn;
    }
}

// ---------------------------------------------------------------------------------------------
// LayerNorm backward with respect to its input, given the gradient dn of the normalised tensor (fp32: what the NORM
// variant of dwconv_bwd_lds_kernel writes as dx) and the row statistics of the forward:
//     g = gamma * dn,   dx = rstd * (g - mean_c(g) - xhat * mean_c(g * xhat))  (+ dy: the residual connection's share)
// The parameter gradients are summed by the conv backward. One wave per row (NCH 16-byte chunks per lane: rows of at
// most NCH KiB), 4 rows per block, blocks stride over the rows; four streams of [T, C].
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_allsum(float v) {
    v += dpp_row_ror<8>(v);
    v += dpp_row_ror<4>(v);
    v += dpp_row_ror<2>(v);
    v += dpp_row_ror<1>(v);
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (a + b) + (c + d);
}

// Row statistics for rows the whole-row kernel above does not take: one wave per row, the row in registers (NCH
// 16-byte chunks per lane: rows of at most NCH KiB), mean first and then the squared deviations from it.
template <bool BF16, int NCH>
__global__ void __launch_bounds__(256)
ln_stats_kernel(const void* __restrict__ x, float* __restrict__ stats, float eps, int T, int C) {
    constexpr int E = BF16 ? 2 : 4, CE = 16 / E;
    using Chunk = RowVec<BF16, CE>;
    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const int rowb = C * E;
    const float inv_c = 1.f / (float)C;
    for (int t = (int)blockIdx.x * 4 + wv; t < T; t += (int)gridDim.x * 4) {
        const char* row = reinterpret_cast<const char*>(x) + (size_t)t * rowb;
        float v[NCH][CE];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int off = (lane + 64 * i) * 16;
            if (off < rowb) {
                Chunk c;
                c.load(row + off);
                c.to_f32(v[i]);
#pragma unroll
                for (int e = 0; e < CE; ++e) s += v[i][e];
            }
        }
        const float mean = wave_allsum(s) * inv_c;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if ((lane + 64 * i) * 16 < rowb) {
#pragma unroll
                for (int e = 0; e < CE; ++e) {
                    const float d = v[i][e] - mean;
                    q = __builtin_fmaf(d, d, q);
                }
            }
        }
        const float rstd = __builtin_amdgcn_rsqf(wave_allsum(q) * inv_c + eps);
        if (lane == 0) {
            stats[2 * (size_t)t] = mean;
            stats[2 * (size_t)t + 1] = rstd;
        }
    }
}

template <bool BF16, int NCH>
__global__ void __launch_bounds__(256)
ln_bwd_dx_kernel(const void* __restrict__ x, const float* __restrict__ stats, const void* __restrict__ gamma, int w_flags,
                 const float* __restrict__ dn, const void* __restrict__ dy, void* __restrict__ dx, int T, int C) {
    constexpr int E = BF16 ? 2 : 4, CE = 16 / E;
    using Chunk = RowVec<BF16, CE>;
    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    const int rowb = C * E;
    const float inv_c = 1.f / (float)C;
    float gam[NCH][CE];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
#pragma unroll
        for (int e = 0; e < CE; ++e) {
            const int c = (lane + 64 * i) * CE + e;
            gam[i][e] = c >= C ? 0.f : (w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(gamma)[c])
                                                       : reinterpret_cast<const float*>(gamma)[c];
        }
    }
    for (int t = (int)blockIdx.x * 4 + wv; t < T; t += (int)gridDim.x * 4) {
        const float mean = stats[2 * (size_t)t], rstd = stats[2 * (size_t)t + 1];
        const float sb = -mean * rstd;
        const size_t row = (size_t)t * rowb;
        float gv[NCH][CE], xh[NCH][CE], res[NCH][CE];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int off = (lane + 64 * i) * 16;
            if (off < rowb) {
                Chunk cx;
                float xv[CE], dv[CE];
                cx.load(reinterpret_cast<const char*>(x) + row + off);
                cx.to_f32(xv);
                const float4* gp = reinterpret_cast<const float4*>(dn + (size_t)t * C + (lane + 64 * i) * CE);
#pragma unroll
                for (int e = 0; e < CE; e += 4) {
                    const float4 q = gp[e / 4];
                    dv[e] = q.x; dv[e + 1] = q.y; dv[e + 2] = q.z; dv[e + 3] = q.w;
                }
                if (dy) {
                    Chunk cr;
                    cr.load(reinterpret_cast<const char*>(dy) + row + off);
                    cr.to_f32(res[i]);
                }
#pragma unroll
                for (int e = 0; e < CE; ++e) {
                    if (!dy) res[i][e] = 0.f;
                    xh[i][e] = __builtin_fmaf(xv[e], rstd, sb);
                    gv[i][e] = gam[i][e] * dv[e];
                    s1 += gv[i][e];
                    s2 = __builtin_fmaf(gv[i][e], xh[i][e], s2);
                }
            }
        }
        const float m1 = wave_allsum(s1) * inv_c, m2 = wave_allsum(s2) * inv_c;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int off = (lane + 64 * i) * 16;
            if (off < rowb) {
                float o[CE];
#pragma unroll
                for (int e = 0; e < CE; ++e) o[e] = __builtin_fmaf(rstd, gv[i][e] - m1 - xh[i][e] * m2, res[i][e]);
                Chunk co;
                co.from_f32(o);
                co.store(reinterpret_cast<char*>(dx) + row + off);
            }
        }
    }
}

}  // namespace nplm
