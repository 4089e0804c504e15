// Host-side internals of libnplm_dwconv: launch plans, the per-K launcher tables, and the
// geometry-override entry points used by the benchmark sweeps and the geometry tests.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "dwconv_kernels.h"
#include "dwconv_lds_kernels.h"
#include "dwconv_lds_split_kernels.h"
#include "dwconv_ln_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

// Launch-geometry overrides; a field left 0 keeps the library's default for that field.
typedef struct nplm_dwconv_tuning {
    int32_t vec;        // channels per lane (bf16: 1,2,4,8; fp32: 1,2,4)
    int32_t unroll;     // output rows per chunk (U); must be one the library was built with
    int32_t tile_rows;  // rows per tile (R), rounded up to a multiple of unroll
    int32_t bw;         // wave-columns per block (power of two)
    int32_t bt;         // token slots per block
    int32_t nbt;        // token-blocks in the grid
    int32_t xcd_remap;  // 1 = give each XCD a contiguous share of the token-blocks (off by default: measured slower)
    int32_t maxt;       // launch-bounds class (threads per block the kernel was compiled for)
    int32_t algo;       // 1 = sliding-window (register) kernels, 2 = LDS-staged pipelined kernels,
                        // 3 = role-split LDS-staged kernels (K = 31, 15)
    int32_t nwl;        // LDS kernels: loader waves per block
    int32_t nbuf;       // LDS forward: tile buffers (2 or 3)
    uint32_t flags;     // NPLM_DWCONV_RESIDUAL etc., as for the _ex entry points
    void* mid_event;    // backward: hipEvent_t recorded between the fused kernel and the finalize kernel
} nplm_dwconv_tuning;
// For algo 2 the fields mean: vec = channels per lane, unroll = rows per wave (RW), bt = row groups
// per block (tile rows = RW * bt), bw = wave-columns per block, nwl = loader waves, nbt = token
// blocks, xcd_remap = run length of adjacent tiles that share an XCD (0 = default 8, < 0 = off);
// tile_rows and maxt are ignored. Only shapes the library was built with exist.

// Same contracts as nplm_dwconv_fwd / nplm_dwconv_bwd, with geometry overrides. An override the
// build does not hold a kernel for yields -NPLM_DWCONV_ETUNING.
#define NPLM_DWCONV_ETUNING 8
int nplm_dwconv_fwd_tuned(const void* x, const int32_t* cu, const void* w, const void* b, void* y,
                          int64_t T, int32_t C, int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype,
                          void* stream, const nplm_dwconv_tuning* tune);
int nplm_dwconv_bwd_tuned(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx,
                          float* dw, float* db, void* workspace, size_t workspace_bytes, int64_t T,
                          int32_t C, int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype,
                          void* stream, const nplm_dwconv_tuning* tune);
// Token-blocks (= workspace slabs of (K'+1)*C floats, K' the kernel size that runs: K, or for an odd K <= 31 without
// kernels of its own the next of 3, 15, 31) a backward launch with these overrides uses.
int32_t nplm_dwconv_bwd_slabs(int64_t T, int32_t C, int32_t K, int32_t act_dtype, const nplm_dwconv_tuning* tune);
// The kernel size K' a plain or gated conv of K taps runs as (K itself for 3, 5, 7, 9, 15, 31 and above 31).
int32_t nplm_dwconv_exec_kernel_size(int32_t K);

// Host-side run of the kernels' boundary cursor (SeqCursor) over a HOST copy of cu: for rows
// t = start, start+step, ... < T writes the interval [cs, ce) the cursor reports, located afresh
// at `start` and every `relocate_every` rows (0 = never) and advanced in between -- the same two
// moves the kernels make at tile starts and inside tiles. Returns the number of rows written.
int64_t nplm_dwconv_debug_intervals(const int32_t* cu_host, int32_t S, int64_t T, int64_t start, int64_t step,
                                    int64_t relocate_every, int32_t* cs_out, int32_t* ce_out);

// Plain streaming copy of `bytes` bytes (multiple of 16, 16-byte aligned pointers) with one block
// per contiguous 16 KiB: the measuring stick for what a 1-read-1-write kernel reaches on this GPU and
// the known-size kernel that calibrates the profiler's HBM byte counters.
int nplm_dwconv_debug_copy(const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif

namespace nplm {

// The device pointers of one call (host-side bundle; kernels take them as separate arguments).
struct ConvPtrs {
    const void* x;
    const void* dy;
    const int32_t* cu;
    const void* w;
    const void* b;
    void* out;        // y (forward) or dx (backward)
    float* partial;   // backward: dw/db slabs
};

// One launcher per specialised kernel size, each in its own translation unit.
// Return hipErrorInvalidConfiguration when the (vec, unroll, maxt) combination is not built.
#define NPLM_DECLARE_K(KK)                                                                               \
    hipError_t launch_fwd_k##KK(bool bf16, int vec, int unroll, int maxt, const ConvPtrs& p, const Geo& g,   \
                                dim3 grid, dim3 block, hipStream_t s);                                       \
    hipError_t launch_bwd_k##KK(bool bf16, int vec, int unroll, int maxt, bool wdx, bool wdw,                \
                                const ConvPtrs& p, const Geo& g, dim3 grid, dim3 block, size_t shmem,        \
                                hipStream_t s);
// Which LDS kernel shape to launch (all are template parameters of the kernels).
struct LdsShapeSel {
    bool bf16;
    int vec, rw, nrg, ncw, nwl, nbuf;
};
#define NPLM_DECLARE_LDS_K(KK)                                                                            \
    hipError_t launch_fwd_lds_k##KK(const LdsShapeSel& sh, const ConvPtrs& p, const LdsGeo& g, dim3 grid, \
                                    hipStream_t s);                                                       \
    hipError_t launch_bwd_lds_k##KK(const LdsShapeSel& sh, bool wdx, bool wdw, const ConvPtrs& p,         \
                                    const LdsGeo& g, dim3 grid, hipStream_t s);
#define NPLM_DECLARE_LDS_GATED_K(KK)                                                                      \
    hipError_t launch_fwd_lds_gated_k##KK(bool bf16, bool narrow, const ConvPtrs& p, const LdsGeo& g, dim3 grid, \
                                          hipStream_t s);                                                 \
    hipError_t launch_bwd_lds_gated_k##KK(bool bf16, bool narrow, const ConvPtrs& p, const LdsGeo& g, dim3 grid, \
                                          hipStream_t s);
NPLM_DECLARE_LDS_GATED_K(3)
NPLM_DECLARE_LDS_GATED_K(5)
NPLM_DECLARE_LDS_GATED_K(7)
NPLM_DECLARE_LDS_GATED_K(9)
#undef NPLM_DECLARE_LDS_GATED_K
// long gated kernels: sliding-window fused backward with one channel per lane (rows the role-split kernel does not take),
hipError_t launch_bwd_gated_k15(bool bf16, int unroll, int maxt, const ConvPtrs& p, const Geo& g, dim3 grid, dim3 block,
                                size_t shmem, hipStream_t s);
hipError_t launch_bwd_gated_k31(bool bf16, int unroll, int maxt, const ConvPtrs& p, const Geo& g, dim3 grid, dim3 block,
                                size_t shmem, hipStream_t s);
// and LDS-staged forward with the gate formed in LDS by the loader waves (rows the role-split forward does not take)
hipError_t launch_fwd_lds_gated_k15(bool bf16, bool narrow, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_fwd_lds_gated_k31(bool bf16, bool narrow, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
// role-split LDS kernels at K = 31 and 15 (fixed shape per dtype, see lds_split_shape())
hipError_t launch_bwd_split_k31(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_fwd_split_k31(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_bwd_split_k15(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
// gated role-split forward (z = [u | g] in, y out), see lds_split_gated_fwd_shape()
hipError_t launch_fwd_split_gated_k31(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_fwd_split_gated_k15(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
// gated role-split backward (z = [u | g] in, dz out), see lds_split_gated_shape()
hipError_t launch_bwd_split_gated_k31(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_bwd_split_gated_k15(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
// LayerNorm-fused forward (dwconv_ln_kernels.h), K <= 9, fixed shape per dtype, see lds_ln_shape()
hipError_t launch_ln_fwd_k3(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_k5(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_k7(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_k9(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_4k_k3(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_4k_k5(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_4k_k7(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_4k_k9(bool bf16, const ConvPtrs& p, const LnArgs& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
// LayerNorm-fused backward for rows of one 2 KiB column block (the WHOLE variant of dwconv_bwd_lds_kernel): 8 wave-columns
// x 4 bytes per lane, 2 row groups of 8 rows (7 at K = 9, where 16 rows of x plus 24 of dy would not fit twice) and no
// loader waves: all 16 waves compute, each stages its share of the next tile first. Two (dy tile, x tile) pairs =
// 152 KiB at K = 7, plus 1.3 KiB for the exchange of the row sums and the tiles' row statistics. Measured at T=131072,
// C=1024, K=7, bf16 (whole call): 8 compute waves of 16 rows + 4 loader waves 271 us (8 loader waves: 497 us, the
// registers of 16 rows spill at 128 per wave; 12-row waves: 273 us).
// fp32 at K <= 7: 4 wave-columns x 8 bytes per lane and 4 row groups of 4 rows instead (T=131072, C=512, K=7: 163 against
// 178 us per call), as for the 4 KiB rows below.
constexpr LdsShapeSel lds_ln_bwd_shape(bool bf16, int K) {
    return (!bf16 && K <= 7) ? LdsShapeSel{false, 2, 4, 4, 4, 0, 2} : LdsShapeSel{bf16, bf16 ? 2 : 1, K <= 7 ? 8 : 7, 2, 8, 0, 2};
}
// The same for rows of up to 4 KiB (fp32 hidden sizes up to 1024 - the residual stream that torch.autocast leaves - and
// bf16 up to 2048): tiles of 8 (K = 3), 6 (K = 5, 7) or 5 (K = 9) rows, 144 KiB. bf16, and fp32 at K = 9: 16
// wave-columns x 4 bytes per lane, one row group. fp32 at K <= 7: 8 wave-columns x 8 bytes per lane, two row groups of
// 4 or 3 rows - half the LDS reads, stores and exchanged row sums per value (T=131072, C=1024, K=7: 354 against 393 us
// per call; C=768: 350 against 385 us). In bf16 that split (8 bytes = 4 channels per lane) spills at 128 registers.
constexpr bool lds_ln_bwd_wide_kernel_size(int K) { return K == 3 || K == 5 || K == 7 || K == 9; }
// fp32 rows of 2 to 3 KiB (hidden 768, the reference's default width, modeling.py:42) get a column block of their own:
// 6 wave-columns x 8 bytes per lane x 2 row groups (12 waves, none without channels) and, the rows being shorter,
// tiles of 12 (K = 3), 10 (K = 5, 7) or 8 (K = 9) rows in the same LDS.
constexpr bool lds_ln_bwd_rows3k(bool bf16, long long C) { return !bf16 && C * 4 > 2048 && C * 4 <= 3072; }
constexpr LdsShapeSel lds_ln_bwd_3k_shape(int K) { return LdsShapeSel{false, 2, K <= 3 ? 6 : K <= 7 ? 5 : 4, 2, 6, 0, 2}; }
constexpr LdsShapeSel lds_ln_bwd_wide_shape(bool bf16, int K) {
    return (!bf16 && K <= 7) ? LdsShapeSel{false, 2, K <= 3 ? 4 : 3, 2, 8, 0, 2}
                             : LdsShapeSel{bf16, bf16 ? 2 : 1, K <= 3 ? 8 : K <= 7 ? 6 : 5, 1, 16, 0, 2};
}
hipError_t launch_ln_bwd_whole4k_k3(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole4k_k5(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole4k_k7(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole4k_k9(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole_k3(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole_k5(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole_k7(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_whole_k9(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
// conv forward over layer_norm(x) with the statistics given (the NORM variant of dwconv_fwd_lds_kernel, default shape)
hipError_t launch_ln_fwd_wide_k3(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_wide_k5(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_wide_k7(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_fwd_wide_k9(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
// conv backward over layer_norm(x) (the NORM variant of dwconv_bwd_lds_kernel on the default backward shape)
hipError_t launch_ln_bwd_k3(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_k5(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_k7(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_ln_bwd_k9(bool bf16, const ConvPtrs& p, const LnSide& ln, const LdsGeo& g, dim3 grid, hipStream_t s);
hipError_t launch_fwd_split_k15(bool bf16, const ConvPtrs& p, const LdsGeo& g, dim3 grid, hipStream_t s);
NPLM_DECLARE_LDS_K(3)
NPLM_DECLARE_LDS_K(5)
NPLM_DECLARE_LDS_K(7)
NPLM_DECLARE_LDS_K(9)
NPLM_DECLARE_LDS_K(15)
NPLM_DECLARE_LDS_K(31)
#undef NPLM_DECLARE_LDS_K
NPLM_DECLARE_K(3)
NPLM_DECLARE_K(5)
NPLM_DECLARE_K(7)
NPLM_DECLARE_K(9)
NPLM_DECLARE_K(15)
NPLM_DECLARE_K(31)
#undef NPLM_DECLARE_K

// Widest lane slice (channels per lane) built for a (pass, dtype, K), default chunk length U and
// launch-bounds class for a (pass, K, VEC) — the single place both the instantiation lists and the
// planner read. Wider slices than these spill registers.
constexpr int max_vec(bool bwd, bool bf16, int K) {
    if (!bf16) return K >= 15 ? 1 : (bwd ? 2 : 4);
    if (K >= 31) return bwd ? 1 : 2;
    if (K >= 15) return bwd ? 2 : 4;
    return bwd ? 4 : 8;
}
constexpr int default_unroll(bool bwd, int K, int vec) {
    (void)bwd;
    if (K >= 15) return 8;
    return vec >= 8 ? 4 : 8;
}
// Kernel sizes the LDS-staged kernels are built for.
constexpr bool lds_kernel_size(int K) { return K == 3 || K == 5 || K == 7 || K == 9 || K == 15 || K == 31; }
// Default shapes: a block owns 1 KiB of every row of a tile of about 32 rows.
//   forward : 2 wave-columns x 8 bytes per lane, 4 row groups of 8 rows, 4 loader waves; two x tiles of
//             32 + K-1 rows (76 KiB of LDS at K = 7).
//   backward: 4 wave-columns x 4 bytes per lane, 3 row groups of 10 rows, 4 loader waves (16 waves, the most a
//             block can have); two (dy tile of 30 + K-1 rows, x tile of 30 rows) pairs = 132 KiB of the 160 KiB a
//             CU has. The backward issues 20 vector-ALU instructions per element (14 are the FMAs of dx and dw),
//             about 68 us per SIMD at the headline shape, so the compute waves need company to hide their LDS
//             latency: with 12 of them (3 per SIMD) backward + finalize takes 138.8 us where 8 waves of 16 rows
//             with 3 loader waves took 144.3 us (T=131072, C=1024, K=7, bf16; rows per wave 9 .. 12: 138.0 - 138.9 us;
//             3 loader waves: 146.2 us; 2: 155.0 us; 8 bytes per lane spill: 169 us and worse).
//             A third tile buffer was measured slower: 3 x 16-row tiles 179 us against 165 us for 2 x 16-row, 3 x
//             22-row tiles 162 us. So was the forward's boundary mailbox (loader waves running the lookup):
//             141.9 us against 138.8 us.
// Measured at T=131072, C=1024, K=7, bf16 against 16-row tiles on 2 KiB column blocks (the same bytes per
// tile, more halo rows per output row, twice the barriers), before the cache-policy hints: forward 98 -> 95 us.
constexpr LdsShapeSel lds_default_shape(bool bwd, bool bf16, int K) {
    if (K >= 15)   // long kernels: 32-row tiles of 16-row waves, so that tile + K-1 halo rows still fit twice
        return bwd ? LdsShapeSel{bf16, bf16 ? 2 : 1, 8, 2, 4, 4, 2} : LdsShapeSel{bf16, bf16 ? 2 : 1, 16, 2, 4, 4, 2};
    return bwd ? LdsShapeSel{bf16, bf16 ? 2 : 1, 10, 3, 4, 4, 2} : LdsShapeSel{bf16, bf16 ? 4 : 2, 8, 4, 2, 4, 2};
}
// Role-split LDS kernels at K = 31 and 15 (dwconv_lds_split_kernels.h): 512-byte column blocks (2 wave-columns x 4
// bytes per lane), 16 waves of 16 rows that all compute.
//   backward: 4 row groups x 2 roles, 64-row tiles, two (dy tile of 64 + K-1 rows, x tile of 64 rows) pairs (158 KiB
//     at K = 31).
//     T=131072, bf16, backward + finalize in us, sliding-window kernel -> this one: K=31, C=2048: one long sequence
//     677 -> 465, lengths 20 - 512 663 -> 500, the log-normal mix 720 -> 510; C=1024 lengths 20 - 512 376 -> 278.
//     K=15, C=2048: 354 -> 306, 390 -> 339, 385 -> 345; C=1024: 186 -> 156, 205 -> 180, 205 -> 177.
//   forward: 8 row groups, 128-row tiles, two x tiles of 128 + K-1 rows (158 KiB at K = 31). The library's choice
//     at K = 31 only: at K = 15 the forward with loader waves is faster (C=2048: 190 against 203 us).
struct SplitShapeSel {
    int vec, rw, nrg, ncw;
};
constexpr bool lds_split_kernel_size(int K) { return K == 31 || K == 15; }
constexpr SplitShapeSel lds_split_shape(bool fwd, bool bf16, int K) {
    (void)K;
    return SplitShapeSel{bf16 ? 2 : 1, 16, fwd ? 8 : 4, 2};
}
// Gated role-split backward (K = 31, 15): a buffer holds a u tile and a g tile behind the dy tile, so the tiles are
// shorter: two buffers of (R + K-1) + 2 R rows of 512 bytes fit the LDS with 4 row groups of 10 rows at K = 31
// (154 KiB) and of 12 rows at K = 15 (158 KiB).
// Measured at T=131072, C=2048, K=31, bf16 (backward + finalize, log-normal mix / one long sequence): 728 / 685 us;
// 256-byte column blocks with 8 row groups of 12 rows (96-row tiles) 721 / 673; 8 rows per wave 776 / 720; one channel
// per lane in 256-byte blocks with 16, 20, 24 rows per wave 784 / 732, 765 / 718, 771 / 702: rows per wave count, tile
// length does not. Both roles evaluate the gate's sigmoid (two quarter-rate instructions per element and role),
// which is what the kernel costs over the plain one (510 us).
constexpr SplitShapeSel lds_split_gated_shape(bool bf16, int K) { return SplitShapeSel{bf16 ? 2 : 1, K >= 31 ? 10 : 12, 4, 2}; }
// Gated role-split forward (K = 31, 15): a buffer holds a u tile and a g tile of R + K-1 rows each, which the waves turn
// into one fp32 h tile in place before the row schedules run. 256-byte column blocks (one wave-column) with 16 row
// groups of 8 rows: two buffers of 2 x 158 rows x 256 bytes = 158 KiB at K = 31. Measured at T=131072, C=2048, bf16
// against the LDS-staged forward with 8 loader waves that gate 32-row tiles (log-normal mix / one long sequence):
// K = 31 441 / 397 against 501 / 495 us, K = 15 372 / 340 against 420 / 419 us; y is the same bit for bit. At K = 15
// 9 rows per wave (144-row tiles) or 512-byte column blocks with 8 row groups measure the same (377-390 / 356-359 us).
constexpr SplitShapeSel lds_split_gated_fwd_shape(bool bf16, int K) {
    (void)K;
    return SplitShapeSel{bf16 ? 2 : 1, 8, 16, 1};
}
// LayerNorm-fused forward: one 2 KiB column block holds a whole row (C <= 1024 in bf16, 512 in fp32); 4 wave-columns x 8
// bytes per lane, 2 row groups of 8 rows (16-row tiles of K + 15 staged rows), 8 compute + 8 loader waves, three tiles
// (one computed, one having its row statistics taken by the loader waves, one in flight: 132 KiB at K = 7). With two
// 24-row tiles nothing is in flight while the statistics of a tile are taken, and the forward runs at 148 us instead of
// 108 us (T=131072, C=1024, K=7, bf16).
constexpr bool lds_ln_kernel_size(int K) { return K == 3 || K == 5 || K == 7 || K == 9; }
constexpr int kLnCbBytes = 2048;
constexpr LdsShapeSel lds_ln_shape(bool bf16) { return LdsShapeSel{bf16, bf16 ? 4 : 2, 8, 2, 4, 8, 3}; }
// fp32 rows of up to 4 KiB (C <= 1024, the residual stream under autocast): 8 wave-columns x 8 bytes per lane and one row
// group, so that three tiles of at most 13 staged rows fit the LDS (156 KiB): 14 - K rows per tile. Not for bf16 rows of
// that size (C <= 2048): twice the values per staged row, the loader waves' statistics pass spills at 128 registers and
// the kernel is slower than the statistics kernel + the normalising conv forward (352 against 303 us at C=2048, K=7).
constexpr LdsShapeSel lds_ln_4k_shape(bool bf16, int K) { return LdsShapeSel{bf16, bf16 ? 4 : 2, 14 - K, 1, 8, 8, 3}; }
// fp32 rows of 2 to 3 KiB (hidden 768): 6 wave-columns and three tiles of 17 staged rows x 3 KiB (18 - K rows per tile),
// 6 compute + 9 loader waves of two staged rows each.
constexpr bool lds_ln_rows3k(bool bf16, long long C) { return !bf16 && C * 4 > 2048 && C * 4 <= 3072; }
constexpr LdsShapeSel lds_ln_3k_shape(int K) { return LdsShapeSel{false, 2, 18 - K, 1, 6, 9, 3}; }
constexpr int kLdsDefaultCb = 1024;
// Rows that are not a whole number of 1 KiB column blocks leave the last one partly empty. Three more column-block
// widths cover the common cases (K <= 9):
//   backward, 768 bytes (C = 768 and 1152 in bf16, the reference's default hidden and intermediate widths,
//       modeling.py:42-43): 3 wave-columns x 4 bytes per lane, 4 row groups of 12 rows (48-row tiles, so that a
//       tile in flight is still ~75 KiB per CU); 12 compute + 4 loader waves, two (dy, x) tile pairs (153 KiB).
//       (3 row groups of 16 rows with 7 loader waves, 3 at K = 9 in bf16: C=768 K=7 120 against 112 us, K=9 135
//       against 112 us; C=1152 K=9 188 against 162 us.)
//   backward, 1280 bytes (C = 640, 1280 in bf16): 5 wave-columns x 4 bytes per lane, 2 row groups of 12 rows,
//       10 compute + 6 loader waves, 135 KiB.
//   forward, 2 KiB for rows between 1280 and 2047 bytes (C = 640 .. 1023 in bf16), which fill one such block
//       better than two of 1 KiB: 4 wave-columns x 8 bytes per lane, 2 row groups of 8 rows, 4 loader waves.
// Measured at T=131072, K=7, bf16 (us, default blocks -> these): backward C=768 140 -> 112, C=1152 200 -> 159,
// C=640 135 -> 106, C=1280 208 -> 193; forward C=768 83 -> 76. The forward gains nothing from 768-byte blocks
// (C=1152: 113 against 115, C=2304 at T=65536: 119 against 110).
constexpr LdsShapeSel lds_narrow_shape(bool bwd, bool bf16, int K, int cb_bytes) {
    if (!bwd) return LdsShapeSel{bf16, bf16 ? 4 : 2, 8, 2, 4, 4, 2};          // 2048, forward
    if (cb_bytes == 768) return LdsShapeSel{bf16, bf16 ? 2 : 1, 12, 4, 3, 4, 2};
    return LdsShapeSel{bf16, bf16 ? 2 : 1, 12, 2, 5, 6, 2};                  // 1280, backward
}
// 0 = the default column block, else 768 or 1280 (backward), 2048 (forward)
constexpr int lds_narrow_cb(bool bwd, int K, long long row_bytes) {
    if (K > 9 || row_bytes % kLdsDefaultCb == 0) return 0;
    if (!bwd) return (row_bytes >= 1280 && row_bytes < 2048) ? 2048 : 0;
    return row_bytes % 768 == 0 ? 768 : (row_bytes % 1280 == 0 ? 1280 : 0);
}
constexpr LdsShapeSel lds_shape_for(bool bwd, bool bf16, int K, long long row_bytes) {
    return lds_narrow_cb(bwd, K, row_bytes) ? lds_narrow_shape(bwd, bf16, K, lds_narrow_cb(bwd, K, row_bytes))
                                            : lds_default_shape(bwd, bf16, K);
}
// Gated kernels (z = [u | g] input): 1 KiB column blocks, so that a u tile and a g tile fit where the plain
// kernels hold one x tile: 4 wave-columns x 4 bytes per lane, 4 loader waves. The gate costs two transcendentals
// per element read, so the forward takes 32-row tiles of 2 row groups (16 rows per wave: the K-1 halo rows it
// re-gates weigh less; 2 x 2 x 38 KiB = 152 KiB of LDS at K = 7). The backward evaluates the gate on its x rows only
// (no halo) and its vector-ALU work (about 40 instructions per element) is what it has to hide behind the stream:
// 3 row groups, i.e. 12 compute waves, with as many rows per wave as 128 registers hold. Measured at T=131072,
// C=1024, bf16 against 2 row groups of 8 rows (backward + finalize, us): K = 5: 289 -> 240 with 7 rows per wave
// (8 rows: 257, 6: 277); K = 7: 294 -> 250 with 6 rows (7: 266, 8: 295, 5: 295); K = 9: 296 -> 272 with 5 rows (6: 281,
// 7: 296). The few registers these shapes spill (8 at K = 7, 21 at K = 9) cost less than the narrower tiles save.
// Rows that are a multiple of 768 bytes but not of 1 KiB (C = 1152 in bf16, the reference's default
// intermediate width) take 768-byte column blocks: 3 wave-columns; forward 2 row groups of 16 rows; backward
// 4 row groups (12 compute + 4 loader waves) of 8 rows (bf16: 6 at K = 7, 5 at K = 9). Measured at T=131072,
// C=1152, bf16 against 3 row groups of 8 rows with 3 loader waves (us): K = 3: 392 -> 292, 5: 383 -> 295, 7: 400 -> 292,
// 9: 350 -> 299.
// Long gated forward (K = 15, 31): 512-byte column blocks (2 wave-columns x 4 bytes per lane), 4 row groups of 8 rows,
// 8 loader waves that also form h = u * silu(g) in LDS once per staged element (gate_prepass; with 4 loader waves the
// pre-pass is the longer half of a tile: 745 against 599 us at T=131072, C=2048, K=31); two (u, g) tile pairs of
// 32 + K-1 rows = 124 KiB at K = 31.
constexpr bool lds_gated_narrow(long long row_bytes, int K = 7) { return K <= 9 && row_bytes % 768 == 0 && row_bytes % 1024 != 0; }
constexpr LdsShapeSel lds_gated_shape(bool bwd, bool bf16, bool narrow = false, int K = 7) {
    if (K >= 15) return LdsShapeSel{bf16, bf16 ? 2 : 1, 8, 4, 2, 8, 2};
    if (narrow)
        return bwd ? LdsShapeSel{bf16, bf16 ? 2 : 1, bf16 ? (K <= 5 ? 8 : K <= 7 ? 6 : 5) : 8, 4, 3, 4, 2}
                   : LdsShapeSel{bf16, bf16 ? 2 : 1, 16, 2, 3, 4, 2};
    // backward: 3 row groups (12 compute + 4 loader waves, 128 registers each); in bf16 the rows per wave shrink with K
    // so that the two cached gate factors per element still fit: 8, 7, 6, 5 rows at K = 3, 5, 7, 9
    if (bwd) return LdsShapeSel{bf16, bf16 ? 2 : 1, bf16 ? (K <= 3 ? 8 : K <= 5 ? 7 : K <= 7 ? 6 : 5) : 8, 3, 4, 4, 2};
    return LdsShapeSel{bf16, bf16 ? 2 : 1, 16, 2, 4, 4, 2};
}
constexpr bool lds_gated_kernel_size(int K, bool bwd) { return K == 3 || K == 5 || K == 7 || K == 9 || (!bwd && (K == 15 || K == 31)); }
constexpr bool long_gated_kernel_size(int K) { return K == 15 || K == 31; }   // backward: role-split kernel (GATED), else sliding-window
constexpr int default_maxt(bool bwd, int K, int vec) {
    (void)bwd; (void)K; (void)vec;
    return 256;
}

}  // namespace nplm
