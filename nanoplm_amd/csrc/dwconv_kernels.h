// Kernels of the varlen depthwise conv (gfx950, wave64): sliding-window forward, fused backward
// (dx + dw/db partials), partial-sum finalize, and runtime-K fallbacks.
//
// Work decomposition (forward and backward share it)
// --------------------------------------------------
//   thread-column : VEC adjacent channels, one lane; ncols = C / VEC
//   wave-column   : 64 adjacent thread-columns (64*VEC channels); nwc = ceil(ncols / 64)
//   tile          : R consecutive token rows; ntiles = ceil(T / R)
//   wave-item     : (tile, wave-column). A wave walks its tile top to bottom, holding the last
//                   K-1 rows in registers as fp32, so inside a tile every row is loaded once;
//                   only the K-1 rows around a tile edge are loaded by both neighbours.
//   block         : bw wave-columns x bt token slots (bw*bt waves).
//   grid          : ncb column-blocks x nbt token-blocks. Token slot s = tb*bt + tl walks tiles
//                   s, s + ntslots, s + 2*ntslots, ... (ntslots = nbt*bt), so at any moment the
//                   resident waves cover one contiguous window of rows that sweeps through the
//                   tensor, and the backward accumulates dw/db in registers over all its tiles.
//
// Sequence boundaries: the wave keeps a scalar cursor over cu (SeqCursor). A chunk of U output
// rows whose whole footprint [t-P, t+U-1+P] lies inside one sequence takes the unmasked path;
// otherwise every tap is selected (not multiplied) against [cs, ce) of its output row, so values
// from another sequence, NaN/Inf included, never enter a sum.
//
// No counterpart in the reference (peymanvahidi/nanoplm 0.1.6 has no convolution); the tensor
// contract is the packed path's: modeling.py:339,421-439 and collator.py:322-325,405-458.
#pragma once
#include <utility>

#include "dwconv_device.h"

namespace nplm {

// Sizes and launch geometry (everything that is not a pointer). Pointers are passed as separate
// __restrict__ kernel arguments so that cu is read through the scalar data path.
struct Geo {
    int32_t T, C, S;
    int32_t w_flags;       // W_BF16: weights/bias are bf16 (else fp32); W_RESIDUAL: the identity is added (see load_weights)
    int32_t R;             // rows per tile (multiple of U)
    int32_t ntiles;        // ceil(T / R)
    int32_t ncols;         // C / VEC
    int32_t nwc;           // ceil(ncols / 64)
    int32_t bw, bt;        // block = bw wave-columns x bt token slots
    int32_t ncb, nbt;      // grid = ncb x nbt blocks
    int32_t xcd_remap;     // 1: blocks that share an XCD get adjacent token-blocks (needs nblocks % 8 == 0)
};

__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// blockIdx -> (column-block, token-block). Hardware deals consecutive workgroups round-robin to the
// 8 XCDs; with xcd_remap, workgroups on one XCD get consecutive logical ids (measured slower on
// MI355X than the plain order, which keeps all XCDs inside one window of rows; kept as an option).
__device__ __forceinline__ void block_coords(const Geo& g, int& cb, int& tb) {
    int b = (int)blockIdx.x;
    if (g.xcd_remap) {
        const int per = (int)(gridDim.x >> 3);
        b = (b & 7) * per + (b >> 3);
    }
    cb = b % g.ncb;
    tb = b / g.ncb;
}

// Bits of the w_flags launch parameter.
constexpr int W_BF16 = 1;      // weights and bias are bf16 (otherwise fp32)
constexpr int W_RESIDUAL = 2;  // compute x + conv(x) (forward) / dy + conv^T(dy) (dx)
// A kernel built for K taps also runs a conv of K - 2 * off taps (the caller's weight rows are that long): taps
// off .. K-1-off carry the caller's weights, the outer ones are zero, and the reduction writes the inner rows of dw only.
constexpr int W_TAP_OFF_SHIFT = 8;
__host__ __device__ constexpr int w_tap_off(int w_flags) { return (w_flags >> W_TAP_OFF_SHIFT) & 0xff; }

// Weights of channels c0 .. c0+VEC-1 as fp32 registers. The fused residual costs nothing: the centre
// tap is valid for every row, so x + conv(x; w) = conv(x; w + delta_centre); one is added to the
// centre weight here (exact for bf16 weights, one fp32 rounding otherwise). dw does not read wr.
template <int VEC, int K>
__device__ __forceinline__ void load_weights(const void* __restrict__ w, int w_flags, int c0, float (&wr)[VEC][K]) {
    if (const int off = w_tap_off(w_flags); off != 0) {      // weight rows of K - 2 * off taps
        const int kw = K - 2 * off;
#pragma unroll
        for (int v = 0; v < VEC; ++v)
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int r = k - off;
                const size_t i = (size_t)(c0 + v) * kw + (r >= 0 && r < kw ? r : 0);
                const float t = (w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[i]) : reinterpret_cast<const float*>(w)[i];
                wr[v][k] = (r >= 0 && r < kw) ? t : 0.f;
            }
    } else if (w_flags & W_BF16) {
        const uint16_t* wp = reinterpret_cast<const uint16_t*>(w) + (size_t)c0 * K;
#pragma unroll
        for (int v = 0; v < VEC; ++v)
#pragma unroll
            for (int k = 0; k < K; ++k) wr[v][k] = bf16_to_f32(wp[v * K + k]);
    } else {
        const float* wp = reinterpret_cast<const float*>(w) + (size_t)c0 * K;
#pragma unroll
        for (int v = 0; v < VEC; ++v)
#pragma unroll
            for (int k = 0; k < K; ++k) wr[v][k] = wp[v * K + k];
    }
    if (w_flags & W_RESIDUAL) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) wr[v][(K - 1) / 2] += 1.f;
    }
}

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{}).
// Used where a loop variable must be a constant expression (register-ring slot numbers).
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

__device__ __forceinline__ int clamp_row(int r, int T) { return r < 0 ? 0 : (r >= T ? T - 1 : r); }

// Window storage. The K-1+U rows a chunk needs live in a ring of RING row slots; chunk number i of
// a tile starts at slot (i mod NPH) * U. When NPH * U >= K-1+U for some NPH <= 3 the chunk loop is
// unrolled NPH times and every slot index is a compile-time constant: no register moves at all.
// Otherwise (large K) NPH = 1 and the last K-1 rows are moved down after every chunk.
template <int K, int U> struct Ring {
    static constexpr int NEED = K - 1 + U;
    static constexpr int N3 = 1 + (K - 1 + U - 1) / U;          // phases so that (N3-1)*U >= K-1
    static constexpr bool ROTATE = (K > 1) && (N3 <= 3);
    static constexpr int NPH = ROTATE ? N3 : 1;
    static constexpr int RING = ROTATE ? N3 * U : NEED;
    static constexpr int slot(int ph, int j) { return (ph * U + j) % RING; }
};

// =============================================================================================
// Forward
// =============================================================================================
template <bool BF16, int K, int VEC, int U, int MAXT>
__global__ void __launch_bounds__(MAXT)
dwconv_fwd_kernel(const void* __restrict__ x, const int32_t* __restrict__ cu, const void* __restrict__ w,
                  const void* __restrict__ b, void* __restrict__ y, const Geo g) {
    constexpr int P = (K - 1) / 2;
    constexpr int E = BF16 ? 2 : 4;
    using Row = RowVec<BF16, VEC>;
    using RG = Ring<K, U>;

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    int cb, tb;
    block_coords(g, cb, tb);
    const int wc = cb * g.bw + (wv % g.bw);
    const int tslot = tb * g.bt + (wv / g.bw);
    const int ntslots = g.nbt * g.bt;
    if (wc >= g.nwc) return;

    const int col = wc * 64 + lane;
    const bool active = col < g.ncols;
    const int c0 = (active ? col : g.ncols - 1) * VEC;   // clamped: loads stay in bounds, stores are guarded
    const int lane_off = c0 * E;
    const size_t row_bytes = (size_t)g.C * E;
    const int rowb = (int)row_bytes;
    const int T = g.T, S = g.S, R = g.R;

    float wr[VEC][K];
    load_weights<VEC, K>(w, g.w_flags, c0, wr);
    float bias[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bias[v] = 0.f;
    if (b) {
#pragma unroll
        for (int v = 0; v < VEC; ++v)
            bias[v] = (g.w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(b)[c0 + v])
                               : reinterpret_cast<const float*>(b)[c0 + v];
    }

    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;

    for (int tile = tslot; tile < g.ntiles; tile += ntslots) {
        const int t0 = tile * R;
        const int t1 = (t0 + R < T) ? t0 + R : T;
        const int rb = (t0 - P > 0) ? t0 - P : 0;            // first row the descriptors cover
        const rsrc_t rx = rows_rsrc(x, rb, T, row_bytes);
        const rsrc_t ry = rows_rsrc(y, t0, T, row_bytes);

        float win[RG::RING][VEC];   // slot(ph, j) holds row tc - P + j
#pragma unroll
        for (int j = 0; j < K - 1; ++j) {
            Row r;
            r.bload(rx, lane_off, (clamp_row(t0 - P + j, T) - rb) * rowb);
            r.to_f32(win[RG::slot(0, j)]);
        }
        Row nxt[U];
#pragma unroll
        for (int u = 0; u < U; ++u) nxt[u].bload(rx, lane_off, (clamp_row(t0 + P + u, T) - rb) * rowb);
        sc.locate(cu, S, T, t0, sc.seq);

        int tc = t0;
        while (tc < t1) {
            static_for<RG::NPH>([&](auto ph_c) {
                constexpr int ph = decltype(ph_c)::value;
                if (tc < t1) {
#pragma unroll
                    for (int u = 0; u < U; ++u) nxt[u].to_f32(win[RG::slot(ph, K - 1 + u)]);
                    if (tc + U < t1) {
#pragma unroll
                        for (int u = 0; u < U; ++u)
                            nxt[u].bload(rx, lane_off, (clamp_row(tc + U + P + u, T) - rb) * rowb);
                    }
                    sc.advance(cu, S, T, tc);
                    Row o[U];
                    if (tc - P >= sc.cs && tc + U - 1 + P < sc.ce && tc + U <= t1) {
                        // whole footprint inside one sequence
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            float acc[VEC];
#pragma unroll
                            for (int v = 0; v < VEC; ++v) acc[v] = bias[v];
#pragma unroll
                            for (int k = 0; k < K; ++k)
#pragma unroll
                                for (int v = 0; v < VEC; ++v)
                                    acc[v] = __builtin_fmaf(wr[v][k], win[RG::slot(ph, u + k)][v], acc[v]);
                            o[u].from_f32(acc);
                        }
                        if (active) {
#pragma unroll
                            for (int u = 0; u < U; ++u) o[u].bstore(ry, lane_off, (tc + u - t0) * rowb);
                        }
                    } else {
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            const int t = tc + u;
                            if (t < t1) {
                                sc.advance(cu, S, T, t);
                                float acc[VEC];
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[v] = bias[v];
                                const uint32_t taps = row_tap_mask<K>(sc, t);
#pragma unroll
                                for (int k = 0; k < K; ++k) {
                                    const bool ok = (taps >> k) & 1u;      // row t + k - P is in t's sequence
#pragma unroll
                                    for (int v = 0; v < VEC; ++v) {
                                        const float xv = ok ? win[RG::slot(ph, u + k)][v] : 0.f;
                                        acc[v] = __builtin_fmaf(wr[v][k], xv, acc[v]);
                                    }
                                }
                                o[u].from_f32(acc);
                                if (active) o[u].bstore(ry, lane_off, (t - t0) * rowb);
                            }
                        }
                    }
                    if constexpr (!RG::ROTATE) {
#pragma unroll
                        for (int j = 0; j < K - 1; ++j)
#pragma unroll
                            for (int v = 0; v < VEC; ++v) win[j][v] = win[j + U][v];
                    }
                    tc += U;
                }
            });
        }
    }
}

// =============================================================================================
// Backward (fused): dx, plus per-block partial sums of dw and db
// =============================================================================================
// Both gradients of row t are written against the SAME window of dy rows t-P .. t+P (slot m holds
// dy[t-P+m]); only the centre row of x is needed, so x is read without any halo:
//     dx[t]      = sum_m w[K-1-m] * dy[t-P+m]
//     dw[K-1-m] += x[t] * dy[t-P+m]          (dw[k] = sum_t x[t] * dy[t-k+P], the same sum as
//                                             sum_t' dy[t'] * x[t'+k-P] with t = t'+k-P)
//     db        += dy[t]
// A tap is masked when row t-P+m lies outside the sequence of row t; the two rows of a product are
// always in the same sequence or the product is dropped, so the mask is the same in either form.
// Each wave keeps dw/db for its VEC channels in registers across all its tiles. At the end the bt
// waves of a block that share a wave-column are summed through LDS in fixed order (token slot
// 0,1,2,...), and the block writes one slab partial[tb][k][c]. No atomics.
// WDX / WDW select the outputs at compile time (dx only, dw/db only, or both).
// GATED: x is z = [u | g] of shape [T, 2C] (the SwiGLU MLP's Wi output, modeling.py:300-302), the conv ran over
// h = u * silu(g), and dx is dz [T, 2C] = [dh * silu(g) | dh * u * sig(g) * (1 + g * (1 - sig(g)))] with dh the
// conv's input gradient; h (for dw) and the two gate factors are formed once per element from the centre rows.
template <bool BF16, int K, int VEC, int U, int MAXT, bool WDX, bool WDW, bool GATED = false>
__global__ void __launch_bounds__(MAXT)
dwconv_bwd_kernel(const void* __restrict__ x, const void* __restrict__ dy, const int32_t* __restrict__ cu,
                  const void* __restrict__ w, void* __restrict__ dx, float* __restrict__ partial, const Geo g) {
    constexpr int P = (K - 1) / 2;
    constexpr int E = BF16 ? 2 : 4;
    using Row = RowVec<BF16, VEC>;
    using RG = Ring<K, U>;
    static_assert(!GATED || (WDX && WDW), "the gated backward always produces dz, dw and db");
    extern __shared__ float red[];   // [nwaves][VEC][64]

    const int lane = (int)(threadIdx.x & 63);
    const int wv = wave_id();
    int cb, tb;
    block_coords(g, cb, tb);
    const int wcl = wv % g.bw;
    const int tl = wv / g.bw;
    const int wc = cb * g.bw + wcl;
    const int tslot = tb * g.bt + tl;
    const int ntslots = g.nbt * g.bt;
    const bool wave_on = wc < g.nwc;   // idle waves still take part in the barriers below

    const int col = wc * 64 + lane;
    const bool active = wave_on && col < g.ncols;
    const int c0 = (active ? col : g.ncols - 1) * VEC;
    const int lane_off = c0 * E;
    const size_t row_bytes = (size_t)g.C * E;
    const int rowb = (int)row_bytes;
    const size_t x_row_bytes = GATED ? 2 * row_bytes : row_bytes;    // pitch of x and dx (z and dz when gated)
    const int xrowb = (int)x_row_bytes;
    const int T = g.T, S = g.S, R = g.R;

    float wr[VEC][K];
    if constexpr (WDX) load_weights<VEC, K>(w, g.w_flags, c0, wr);
    float dwa[VEC][K];
    float dba[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        dba[v] = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) dwa[v][k] = 0.f;
    }

    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;

    if (wave_on) {
        for (int tile = tslot; tile < g.ntiles; tile += ntslots) {
            const int t0 = tile * R;
            const int t1 = (t0 + R < T) ? t0 + R : T;
            const int rb = (t0 - P > 0) ? t0 - P : 0;
            const rsrc_t rg = rows_rsrc(dy, rb, T, row_bytes);   // dy rows from rb (window with halo)
            const rsrc_t rx = rows_rsrc(x, t0, T, x_row_bytes);  // x rows from t0 (centre rows only)
            const rsrc_t ro = rows_rsrc(dx, t0, T, x_row_bytes);

            float gw[RG::RING][VEC];   // slot(ph, j) holds dy row tc - P + j
#pragma unroll
            for (int j = 0; j < K - 1; ++j) {
                Row r;
                r.bload(rg, lane_off, (clamp_row(t0 - P + j, T) - rb) * rowb);
                r.to_f32(gw[RG::slot(0, j)]);
            }
            Row nx[WDW ? U : 1], nxg[GATED ? U : 1], ng[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                ng[u].bload(rg, lane_off, (clamp_row(t0 + P + u, T) - rb) * rowb);
                if constexpr (WDW) nx[u].bload(rx, lane_off, (clamp_row(t0 + u, T) - t0) * xrowb);
                if constexpr (GATED) nxg[u].bload(rx, lane_off + rowb, (clamp_row(t0 + u, T) - t0) * xrowb);
            }
            sc.locate(cu, S, T, t0, sc.seq);

            int tc = t0;
            while (tc < t1) {
                static_for<RG::NPH>([&](auto ph_c) {
                    constexpr int ph = decltype(ph_c)::value;
                    if (tc < t1) {
                        float xc[WDW ? U : 1][VEC];   // x rows tc .. tc+U-1 (h rows when gated)
                        // gated: gs = g * sig(g) (h = u * gs, du = dh * gs), gd = u * sig(g) * (1 + g * (1 - sig(g))) (dg = dh * gd)
                        float gs[GATED ? U : 1][VEC], gd[GATED ? U : 1][VEC];
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            ng[u].to_f32(gw[RG::slot(ph, K - 1 + u)]);
                            if constexpr (WDW) nx[u].to_f32(xc[u]);
                            if constexpr (GATED) {
                                float gg[VEC];
                                nxg[u].to_f32(gg);
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    const float sg = sigmoid_f32(gg[v]);
                                    gs[u][v] = gg[v] * sg;
                                    gd[u][v] = xc[u][v] * sg * (1.f + gg[v] * (1.f - sg));
                                    xc[u][v] *= gs[u][v];
                                }
                            }
                        }
                        if (tc + U < t1) {
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                ng[u].bload(rg, lane_off, (clamp_row(tc + U + P + u, T) - rb) * rowb);
                                if constexpr (WDW) nx[u].bload(rx, lane_off, (clamp_row(tc + U + u, T) - t0) * xrowb);
                                if constexpr (GATED) nxg[u].bload(rx, lane_off + rowb, (clamp_row(tc + U + u, T) - t0) * xrowb);
                            }
                        }
                        sc.advance(cu, S, T, tc);
                        Row o[WDX ? U : 1], og[GATED ? U : 1];
                        if (tc - P >= sc.cs && tc + U - 1 + P < sc.ce && tc + U <= t1) {
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                float acc[VEC];
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    acc[v] = 0.f;
                                    if constexpr (WDW) dba[v] += gw[RG::slot(ph, u + P)][v];
                                }
#pragma unroll
                                for (int m = 0; m < K; ++m)
#pragma unroll
                                    for (int v = 0; v < VEC; ++v) {
                                        const float gv = gw[RG::slot(ph, u + m)][v];
                                        if constexpr (WDX) acc[v] = __builtin_fmaf(wr[v][K - 1 - m], gv, acc[v]);
                                        if constexpr (WDW) dwa[v][K - 1 - m] = __builtin_fmaf(xc[u][v], gv, dwa[v][K - 1 - m]);
                                    }
                                if constexpr (GATED) {
                                    float du[VEC], dg[VEC];
#pragma unroll
                                    for (int v = 0; v < VEC; ++v) { du[v] = acc[v] * gs[u][v]; dg[v] = acc[v] * gd[u][v]; }
                                    o[u].from_f32(du);
                                    og[u].from_f32(dg);
                                } else if constexpr (WDX) {
                                    o[u].from_f32(acc);
                                }
                            }
                            if constexpr (WDX) {
                                if (active) {
#pragma unroll
                                    for (int u = 0; u < U; ++u) {
                                        o[u].bstore(ro, lane_off, (tc + u - t0) * xrowb);
                                        if constexpr (GATED) og[u].bstore(ro, lane_off + rowb, (tc + u - t0) * xrowb);
                                    }
                                }
                            }
                        } else {
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                const int t = tc + u;
                                if (t < t1) {
                                    sc.advance(cu, S, T, t);
                                    float acc[VEC];
#pragma unroll
                                    for (int v = 0; v < VEC; ++v) {
                                        acc[v] = 0.f;
                                        if constexpr (WDW) dba[v] += gw[RG::slot(ph, u + P)][v];
                                    }
                                    const uint32_t taps = row_tap_mask<K>(sc, t);
#pragma unroll
                                    for (int m = 0; m < K; ++m) {
                                        const bool ok = (taps >> m) & 1u;  // row t + m - P is in t's sequence
#pragma unroll
                                        for (int v = 0; v < VEC; ++v) {
                                            const float gv = ok ? gw[RG::slot(ph, u + m)][v] : 0.f;
                                            if constexpr (WDX) acc[v] = __builtin_fmaf(wr[v][K - 1 - m], gv, acc[v]);
                                            // x is selected too: an Inf or NaN in this row times the selected zero
                                            // would put a NaN into a tap sum the product does not belong to
                                            if constexpr (WDW) dwa[v][K - 1 - m] = __builtin_fmaf(ok ? xc[u][v] : 0.f, gv, dwa[v][K - 1 - m]);
                                        }
                                    }
                                    if constexpr (GATED) {
                                        float du[VEC], dg[VEC];
#pragma unroll
                                        for (int v = 0; v < VEC; ++v) { du[v] = acc[v] * gs[u][v]; dg[v] = acc[v] * gd[u][v]; }
                                        o[u].from_f32(du);
                                        og[u].from_f32(dg);
                                        if (active) {
                                            o[u].bstore(ro, lane_off, (t - t0) * xrowb);
                                            og[u].bstore(ro, lane_off + rowb, (t - t0) * xrowb);
                                        }
                                    } else if constexpr (WDX) {
                                        o[u].from_f32(acc);
                                        if (active) o[u].bstore(ro, lane_off, (t - t0) * rowb);
                                    }
                                }
                            }
                        }
                        if constexpr (!RG::ROTATE) {
#pragma unroll
                            for (int j = 0; j < K - 1; ++j)
#pragma unroll
                                for (int v = 0; v < VEC; ++v) gw[j][v] = gw[j + U][v];
                        }
                        tc += U;
                    }
                });
            }
        }
    }

    if constexpr (!WDW) return;

    // ---- block-level pass: sum the bt token slots of each wave-column, slot order 0,1,2,... ----
    float* slab = partial + (size_t)tb * (K + 1) * g.C;
#pragma unroll
    for (int kk = 0; kk <= K; ++kk) {
        float val[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) val[v] = (kk < K) ? dwa[v][kk < K ? kk : 0] : dba[v];
        if (tl > 0) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) red[(wv * VEC + v) * 64 + lane] = val[v];
        }
        __syncthreads();
        if (tl == 0) {
            for (int j = 1; j < g.bt; ++j) {
                const int ow = j * g.bw + wcl;
#pragma unroll
                for (int v = 0; v < VEC; ++v) val[v] += red[(ow * VEC + v) * 64 + lane];
            }
            if (active) {
                float* dst = slab + (size_t)kk * g.C + c0;
#pragma unroll
                for (int v = 0; v < VEC; ++v) dst[v] = val[v];
            }
        }
        __syncthreads();
    }
}

// =============================================================================================
// Finalize: dw[c][k] = sum_p partial[p][k][c], db[c] = sum_p partial[p][K][c], p in fixed order.
// Block = 64 outputs (adjacent c) x SPLIT groups of p; each group sums its contiguous share of p in
// order (loads issued 8 at a time), then group 0 adds the group sums in order.
// =============================================================================================
constexpr int FIN_SPLIT = 16;

// One block of the reduction: 64 consecutive (tap, channel) outputs, SPLIT groups of slabs summed in LDS.
// out_bf16: dw and db are bf16 buffers (the fp32 totals are rounded once, nearest-even, on store).
// tap_off: dw has rows of K - 2 * tap_off taps, slab rows tap_off .. K-1-tap_off (see W_TAP_OFF_SHIFT).
template <int SPLIT>
__device__ __forceinline__ void finalize_block(float (&red)[SPLIT][64], int block, const float* __restrict__ partial, int nbt, int C,
                                               int K, float* __restrict__ dw, float* __restrict__ db, int out_bf16 = 0,
                                               int tap_off = 0) {
    const int lane = (int)(threadIdx.x & 63);
    const int grp = (int)(threadIdx.x >> 6);
    const long long n_out = (long long)(K + 1) * C;
    const long long o = (long long)block * 64 + lane;   // o = kk*C + c
    const bool on = o < n_out;
    const int per = (nbt + SPLIT - 1) / SPLIT;
    const int p0 = grp * per;
    const int p1 = (p0 + per < nbt) ? p0 + per : nbt;
    float s = 0.f;
    if (on) {
        const float* src = partial + o;
        const size_t stride = (size_t)n_out;
        int p = p0;
        for (; p + 8 <= p1; p += 8) {
            float t[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) t[i] = src[(size_t)(p + i) * stride];
#pragma unroll
            for (int i = 0; i < 8; ++i) s += t[i];
        }
        for (; p < p1; ++p) s += src[(size_t)p * stride];
    }
    red[grp][lane] = s;
    __syncthreads();
    if (grp == 0 && on) {
        float tot = red[0][lane];
#pragma unroll
        for (int g = 1; g < SPLIT; ++g) tot += red[g][lane];
        const int kk = (int)(o / C);
        const int c = (int)(o - (long long)kk * C);
        const int kw = K - 2 * tap_off, r = kk - tap_off;
        const bool tap = dw && r >= 0 && r < kw;
        if (out_bf16) {
            if (kk < K) { if (tap) reinterpret_cast<uint16_t*>(dw)[(size_t)c * kw + r] = f32_to_bf16(tot); }
            else        { if (db) reinterpret_cast<uint16_t*>(db)[c] = f32_to_bf16(tot); }
        } else {
            if (kk < K) { if (tap) dw[(size_t)c * kw + r] = tot; }
            else        { if (db) db[c] = tot; }
        }
    }
}

template <int SPLIT>
__global__ void __launch_bounds__(64 * SPLIT) dwconv_finalize_kernel(const float* __restrict__ partial, int nbt, int C, int K,
                                                                     float* __restrict__ dw, float* __restrict__ db, int out_bf16,
                                                                     int tap_off) {
    __shared__ float red[SPLIT][64];
    finalize_block<SPLIT>(red, (int)blockIdx.x, partial, nbt, C, K, dw, db, out_bf16, tap_off);
}

// Two slab sets of the same launch in one reduction launch (the conv's dw/db and, as a conv of K2 = 1 tap, the
// LayerNorm's parameter gradients): the first `blocks_a` blocks take set a, the rest set b.
template <int SPLIT>
__global__ void __launch_bounds__(64 * SPLIT)
dwconv_finalize2_kernel(const float* __restrict__ pa, int Ka, float* __restrict__ dwa, float* __restrict__ dba, int blocks_a,
                        const float* __restrict__ pb, int Kb, float* __restrict__ dwb, float* __restrict__ dbb, int nbt, int C,
                        int out_bf16) {
    __shared__ float red[SPLIT][64];
    if ((int)blockIdx.x < blocks_a) finalize_block<SPLIT>(red, (int)blockIdx.x, pa, nbt, C, Ka, dwa, dba, out_bf16);
    else finalize_block<SPLIT>(red, (int)blockIdx.x - blocks_a, pb, nbt, C, Kb, dwb, dbb, out_bf16);
}

// =============================================================================================
// Runtime-K fallbacks (any odd K, any C): correct, not tuned. One wave per token row, lanes stride
// over channels.
// =============================================================================================
template <bool BF16>
__device__ __forceinline__ float ld_act(const void* p, size_t i) {
    if constexpr (BF16) return bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
    else return reinterpret_cast<const float*>(p)[i];
}
template <bool BF16>
__device__ __forceinline__ void st_act(void* p, size_t i, float f) {
    if constexpr (BF16) reinterpret_cast<uint16_t*>(p)[i] = f32_to_bf16(f);
    else reinterpret_cast<float*>(p)[i] = f;
}
__device__ __forceinline__ float ld_w(const void* p, int w_flags, size_t i) {
    return (w_flags & W_BF16) ? bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[i]) : reinterpret_cast<const float*>(p)[i];
}

// flip = 0: out[t] = b + sum_k w[k] * in[t+k-P]   (forward)
// flip = 1: out[t] =     sum_k w[k] * in[t-k+P]   (dx from dy)
template <bool BF16>
__global__ void dwconv_generic_rows_kernel(const void* in, const int32_t* __restrict__ cu, const void* w,
                                           const void* b, void* out, int T, int C, int S, int K,
                                           int w_flags, int flip) {
    const int P = (K - 1) / 2;
    const int lane = (int)(threadIdx.x & 63);
    const int wpb = (int)(blockDim.x >> 6);
    const int gw = (int)blockIdx.x * wpb + wave_id();
    const int nw = (int)gridDim.x * wpb;
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    for (int t = gw; t < T; t += nw) {
        sc.locate(cu, S, T, t, sc.seq);
        for (int c = lane; c < C; c += 64) {
            float acc = (b && !flip) ? ld_w(b, w_flags, c) : 0.f;
            for (int k = 0; k < K; ++k) {
                const int j = flip ? (t - k + P) : (t + k - P);
                // cu only masks; the explicit [0, T) test keeps a malformed cu from forming a bad address
                if (j >= sc.cs && j < sc.ce && j >= 0 && j < T) {
                    float wk = ld_w(w, w_flags, (size_t)c * K + k);
                    if (k == P && (w_flags & W_RESIDUAL)) wk += 1.f;
                    acc = __builtin_fmaf(wk, ld_act<BF16>(in, (size_t)j * C + c), acc);
                }
            }
            st_act<BF16>(out, (size_t)t * C + c, acc);
        }
    }
}

// partial[tb][kk][c] over the rows of token-block tb. grid = (nbt, ceil(C/256)); thread = channel.
template <bool BF16>
__global__ void dwconv_generic_dw_kernel(const void* x, const void* dy, const int32_t* __restrict__ cu,
                                         float* __restrict__ partial, int T, int C, int S, int K, int rows_per_block) {
    const int P = (K - 1) / 2;
    const int c = (int)(blockIdx.y * blockDim.x + threadIdx.x);
    const int tb = (int)blockIdx.x;
    const long long r0 = (long long)tb * rows_per_block;
    const int t0 = (int)(r0 < T ? r0 : T);
    const int t1 = (int)((r0 + rows_per_block < T) ? r0 + rows_per_block : T);
    float* slab = partial + (size_t)tb * (K + 1) * C;
    for (int kk = 0; kk <= K; ++kk) {
        float acc = 0.f;
        SeqCursor sc;
        sc.seq = 0; sc.cs = 0; sc.ce = 0;
        if (t0 < t1) sc.locate(cu, S, T, t0, 0);
        for (int t = t0; t < t1; ++t) {
            sc.advance(cu, S, T, t);
            if (c < C) {
                const float g = ld_act<BF16>(dy, (size_t)t * C + c);
                if (kk == K) acc += g;
                else {
                    const int j = t + kk - P;
                    if (j >= sc.cs && j < sc.ce && j >= 0 && j < T)
                        acc = __builtin_fmaf(g, ld_act<BF16>(x, (size_t)j * C + c), acc);
                }
            }
        }
        if (c < C) slab[(size_t)kk * C + c] = acc;
    }
}

}  // namespace nplm
