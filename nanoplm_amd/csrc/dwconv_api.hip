// C ABI of libnplm_dwconv (see include/nplm_dwconv.h): argument checks, launch planning and
// dispatch to the per-K launchers. Host code only; the kernels live in dwconv_kernels.h and
// dwconv_lds_kernels.h.
//
// The entry points stand where a conv module's forward/backward would sit on the reference's
// packed path (src/nanoplm/pretraining/models/modern_bert/modeling.py:421-439; backward driven by
// src/nanoplm/pretraining/pure_pipeline.py:739-742). The reference holds no such op to replace.
#include <hip/hip_runtime.h>

#include <limits.h>
#include <stdlib.h>

#include <atomic>
#include <vector>

#include "../../include/nplm_dwconv.h"
#include "dwconv_internal.h"

// Scratch of nplm_dwconv_bwd_static: the dw/db partial-sum slabs of one backward call, for callers that
// cannot hand in a workspace they allocated. One copy per GPU, held until the process ends. Host code
// never uses this name as an address: static_scratch_for_current_device() asks the runtime where the
// current device's copy lives and the kernels are given that pointer.
static __device__ __align__(256) unsigned char scratch[NPLM_DWCONV_STATIC_SCRATCH_BYTES];

namespace nplm {
namespace {

constexpr int kVersion = 102;   // 0.1.2: odd kernel sizes up to 31 without kernels of their own run as the next built size

// MI355X: 256 CUs in 8 XCDs. Geometry is a pure function of the problem size so that the
// reduction order (and with it every output bit) is reproducible.
constexpr int kNumCU = 256;
constexpr int kNumXCD = 8;
constexpr long long kMaxRows = (long long)INT_MAX - (1 << 20);   // row arithmetic is int32 with tile-sized slack
constexpr int kMaxTileRows = 1 << 16;
constexpr size_t kSlabBudgetBytes = 16u << 20;   // cap on dw/db partials (written once, read once)

bool specialised_k(int K) { return K == 3 || K == 5 || K == 7 || K == 9 || K == 15 || K == 31; }
// The kernel size a plain conv of K taps runs as: an odd K below 31 without kernels of its own takes the next size that
// has them, with (exec - K) / 2 zero taps on either side (W_TAP_OFF_SHIFT); the caller's weight and dw rows stay K long.
// Runtime-K kernels (one wave per row) remain for K > 31.
int exec_kernel_size(int K) { return K > 31 || specialised_k(K) ? K : K < 3 ? 3 : K < 15 ? 15 : 31; }

int pow2_floor(int v) { int p = 1; while (p * 2 <= v) p *= 2; return p; }
int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

struct Plan {
    bool generic;
    int vec, unroll, maxt;
    int R, ntiles, ncols, nwc, bw, bt, ncb, nbt, remap;
};

int default_vec(bool bwd, bool bf16, int K) { return max_vec(bwd, bf16, K); }

// Largest VEC <= cap that divides C, keeps every row slice aligned, and still spreads a row over a
// whole wave (C / VEC >= 64) unless nothing smaller is left.
int pick_vec(bool bf16, int C, int cap, uintptr_t align_bits) {
    const int E = bf16 ? 2 : 4;
    const int vmax = bf16 ? 8 : 4;
    for (int v = (cap < vmax ? cap : vmax); v > 1; v >>= 1) {
        if (C % v) continue;
        if (align_bits % (uintptr_t)(v * E)) continue;
        if (C / v < 64) continue;
        return v;
    }
    return 1;
}

// tune may be null. Returns 0 or a negative argument error.
int make_plan(bool bwd, bool bf16, long long T, int C, int K, uintptr_t align_bits,
              const nplm_dwconv_tuning* tune, Plan* out) {
    Plan p{};
    nplm_dwconv_tuning z{};
    if (!tune) tune = &z;
    p.generic = !specialised_k(K);
    const int vcap = tune->vec > 0 ? tune->vec : default_vec(bwd, bf16, K);
    p.vec = p.generic ? 1 : pick_vec(bf16, C, vcap, align_bits);
    if (tune->vec > 0 && p.vec != tune->vec) return -NPLM_DWCONV_ETUNING;
    p.unroll = tune->unroll > 0 ? tune->unroll : default_unroll(bwd, K, p.vec);
    p.maxt = tune->maxt > 0 ? tune->maxt : default_maxt(bwd, K, p.vec);
    if (p.maxt < 64 || p.maxt > 1024 || p.maxt % 64) return -NPLM_DWCONV_ETUNING;
    // long kernels re-read K-1 halo rows per tile: longer tiles (measured at K=31: 256 rows beat 64 by 25 %)
    int R = tune->tile_rows > 0 ? tune->tile_rows : (K >= 15 ? 256 : (bwd ? 32 : 64));
    if (R > kMaxTileRows || p.unroll > 64) return -NPLM_DWCONV_ETUNING;
    R = ceil_div(R, p.unroll) * p.unroll;
    // row offsets inside a tile are 32-bit byte offsets
    const long long row_bytes = (long long)C * (bf16 ? 2 : 4);
    while ((long long)(R + K) * row_bytes >= INT_MAX && R > p.unroll) R = ceil_div(R / 2, p.unroll) * p.unroll;
    if ((long long)(R + K) * row_bytes >= INT_MAX) return -NPLM_DWCONV_ESHAPE;
    p.R = R;
    p.ntiles = ceil_div(T, R);
    p.ncols = C / p.vec;
    p.nwc = ceil_div(p.ncols, 64);
    const int wpb_max = p.maxt / 64;
    p.bt = tune->bt > 0 ? tune->bt : (bwd ? 4 : 2);
    if (p.bt > wpb_max) p.bt = wpb_max;
    p.bw = tune->bw > 0 ? tune->bw : pow2_floor(p.nwc);
    if (p.bw > wpb_max / p.bt) p.bw = wpb_max / p.bt;
    if (p.bw < 1 || (p.bw & (p.bw - 1))) return -NPLM_DWCONV_ETUNING;
    p.ncb = ceil_div(p.nwc, p.bw);
    // waves the grid is sized for: 2 per SIMD keep the HBM-bound kernels streaming; the long kernels
    // are ALU-bound and want every wave their registers allow (K=31 backward at C=2048: 848 -> 657 us)
    const int waves_per_cu = K >= 15 ? 32 : 8;
    int nbt = tune->nbt > 0 ? tune->nbt : (kNumCU * waves_per_cu) / (p.ncb * p.bw * p.bt);
    const int nbt_useful = ceil_div(p.ntiles, p.bt);
    if (nbt > nbt_useful) nbt = nbt_useful;
    if (bwd) {
        const size_t slab = (size_t)(K + 1) * C * sizeof(float);
        const long long cap = (long long)(kSlabBudgetBytes / slab);
        if (tune->nbt <= 0 && nbt > cap) nbt = (int)cap;
    }
    if (nbt < 1) nbt = 1;
    // keep the grid a multiple of the XCD count when it is large enough: every XCD gets equal work
    if (tune->nbt <= 0 && nbt >= kNumXCD) nbt -= nbt % kNumXCD;
    p.nbt = nbt;
    p.remap = (tune->xcd_remap == 1) && ((long long)p.ncb * p.nbt) % kNumXCD == 0;
    *out = p;
    return 0;
}

Geo make_geo(const Plan& p, long long T, int C, int S, int w_flags) {
    Geo g{};
    g.T = (int32_t)T; g.C = C; g.S = S; g.w_flags = w_flags;
    g.R = p.R; g.ntiles = p.ntiles; g.ncols = p.ncols; g.nwc = p.nwc;
    g.bw = p.bw; g.bt = p.bt; g.ncb = p.ncb; g.nbt = p.nbt; g.xcd_remap = p.remap;
    return g;
}

int check_common(long long T, int C, int K, int S, int act_dtype, int w_dtype) {
    if (T < 0 || T > kMaxRows || C < 1 || S < 0) return -NPLM_DWCONV_ESHAPE;
    if ((long long)C * K > INT_MAX / 8) return -NPLM_DWCONV_ESHAPE;
    if (K < 1 || K > NPLM_DWCONV_MAX_K || (K % 2) == 0) return -NPLM_DWCONV_EKSIZE;
    if ((act_dtype != NPLM_DWCONV_F32 && act_dtype != NPLM_DWCONV_BF16) ||
        (w_dtype != NPLM_DWCONV_F32 && w_dtype != NPLM_DWCONV_BF16))
        return -NPLM_DWCONV_EDTYPE;
    return 0;
}

hipError_t launch_fwd(int K, bool bf16, const Plan& p, const ConvPtrs& a, const Geo& g, hipStream_t s) {
    const dim3 grid(p.ncb * p.nbt), block(p.bw * p.bt * 64);
    switch (K) {
        case 3: return launch_fwd_k3(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
        case 5: return launch_fwd_k5(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
        case 7: return launch_fwd_k7(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
        case 9: return launch_fwd_k9(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
        case 15: return launch_fwd_k15(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
        case 31: return launch_fwd_k31(bf16, p.vec, p.unroll, p.maxt, a, g, grid, block, s);
    }
    return hipErrorInvalidConfiguration;
}
hipError_t launch_bwd(int K, bool bf16, const Plan& p, bool wdx, bool wdw, const ConvPtrs& a, const Geo& g,
                      hipStream_t s) {
    const dim3 grid(p.ncb * p.nbt), block(p.bw * p.bt * 64);
    const size_t shmem = (size_t)p.bw * p.bt * p.vec * 64 * sizeof(float);
    switch (K) {
        case 3: return launch_bwd_k3(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
        case 5: return launch_bwd_k5(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
        case 7: return launch_bwd_k7(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
        case 9: return launch_bwd_k9(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
        case 15: return launch_bwd_k15(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
        case 31: return launch_bwd_k31(bf16, p.vec, p.unroll, p.maxt, wdx, wdw, a, g, grid, block, shmem, s);
    }
    return hipErrorInvalidConfiguration;
}

// ---- LDS-staged pipelined kernels ---------------------------------------------------------------
constexpr size_t kLdsBytesPerCU = 160u << 10;

struct LdsPlan {
    LdsShapeSel sh;
    int R, ntiles, ncb, nbt, xcd_group, rot_step;
};

// Whether the LDS kernels can take this problem at all (16-byte row granularity, built kernel size).
bool lds_eligible(bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    const int E = bf16 ? 2 : 4;
    if (!lds_kernel_size(K) || T < 1) return false;
    if (((long long)C * E) % 16 || align_bits % 16) return false;
    return (long long)C * E >= 1024;
}

// Whether they are also the faster choice. A block owns one column block of its rows (1 KiB by default,
// see lds_shape_for) and the grid's time follows the number of column blocks, so a row that fills its
// column blocks poorly wastes lanes and loader slots. Measured on MI355X (T=131072, K=7, bf16 rows of
// 1024 .. 10240 bytes and fp32 rows of 1024 .. 8192 bytes): LDS-staged wins for a single column block
// filled to 5/8 or more; for several, the backward needs them filled to 4/5 on average, the forward only
// to 11/20; the sliding-window kernels win otherwise.
bool lds_preferred(bool bwd, bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    if (!lds_eligible(bf16, T, C, K, align_bits)) return false;
    if (K > 9 && bwd) return false;        // K = 15, 31: no single-role LDS backward (it does not fit the registers); see split_eligible
    const long long E = bf16 ? 2 : 4;
    const long long row_bytes = (long long)C * E;
    const LdsShapeSel sh = lds_shape_for(bwd, bf16, K, row_bytes);
    const long long cb_bytes = (long long)sh.ncw * 64 * sh.vec * E;
    const long long ncb = ceil_div(row_bytes, cb_bytes);
    if (ncb == 1) return row_bytes * 8 >= cb_bytes * 5;
    return bwd ? row_bytes * 5 >= ncb * cb_bytes * 4 : row_bytes * 20 >= ncb * cb_bytes * 11;
}

int make_lds_plan(bool bwd, bool bf16, long long T, int C, int K, const nplm_dwconv_tuning* tune, LdsPlan* out,
                  bool gated = false) {
    LdsPlan p{};
    nplm_dwconv_tuning z{};
    if (!tune) tune = &z;
    const int E = bf16 ? 2 : 4;
    p.sh = gated ? lds_gated_shape(bwd, bf16, lds_gated_narrow((long long)C * E, K), K) : lds_shape_for(bwd, bf16, K, (long long)C * E);
    if (tune->vec > 0) p.sh.vec = tune->vec;
    if (tune->unroll > 0) p.sh.rw = tune->unroll;
    if (tune->bt > 0) p.sh.nrg = tune->bt;
    if (tune->bw > 0) p.sh.ncw = tune->bw;
    if (tune->nwl > 0) p.sh.nwl = tune->nwl;
    if (tune->nbuf > 0 && !bwd) p.sh.nbuf = tune->nbuf;
    const long long cb_bytes = (long long)p.sh.ncw * 64 * p.sh.vec * E;
    const long long row_bytes = (long long)C * E;
    p.R = p.sh.rw * p.sh.nrg;
    const size_t tile_rows = gated ? (bwd ? (size_t)(p.R + K - 1) + 2 * (size_t)p.R : 2 * (size_t)(p.R + K - 1))
                                   : (size_t)(p.R + K - 1) + (bwd ? p.R : 0);
    const size_t shmem = (size_t)p.sh.nbuf * tile_rows * cb_bytes;
    if (shmem > kLdsBytesPerCU || cb_bytes % 256) return -NPLM_DWCONV_ETUNING;
    if ((long long)(p.R + K) * row_bytes * (gated ? 2 : 1) + 2 * row_bytes >= INT_MAX) return -NPLM_DWCONV_ESHAPE;
    p.ncb = ceil_div(row_bytes, cb_bytes);
    p.ntiles = ceil_div(T, p.R);
    int nbt = tune->nbt > 0 ? tune->nbt : kNumCU / p.ncb;
    if (nbt < 1) nbt = 1;
    if (nbt > p.ntiles) nbt = p.ntiles;
    if (bwd && tune->nbt <= 0) {
        const size_t slab = (size_t)(K + 1) * C * sizeof(float);
        const long long cap = (long long)(kSlabBudgetBytes / slab);
        if (nbt > cap && cap >= 1) nbt = (int)cap;
    }
    p.nbt = nbt;
    // adjacent tiles share an XCD in runs of G (tune->xcd_remap: 0 = default 8, > 0 = G, < 0 = off)
    int G = tune->xcd_remap == 0 ? 8 : (tune->xcd_remap > 0 ? tune->xcd_remap : 0);
    const long long nblocks = (long long)p.ncb * p.nbt;
    if (G > 0 && !(nblocks % kNumXCD == 0 && (nblocks / kNumXCD) % G == 0 && p.nbt % G == 0)) G = 0;
    p.xcd_group = G;
    // per-round rotation of the tile slots: an odd step near nbt / golden ratio, so that no short period of
    // sequence boundaries keeps landing on the same token-blocks
    p.rot_step = nbt > 2 ? (int)((long long)nbt * 618 / 1000) | 1 : 0;
    if (p.rot_step >= nbt) p.rot_step = nbt - 1;
    *out = p;
    return 0;
}

LdsGeo make_lds_geo(const LdsPlan& p, long long T, int C, int S, int w_flags) {
    LdsGeo g{};
    g.T = (int32_t)T; g.C = C; g.S = S; g.w_flags = w_flags;
    g.ntiles = p.ntiles; g.ncb = p.ncb; g.nbt = p.nbt; g.xcd_group = p.xcd_group; g.rot_step = p.rot_step;
    return g;
}

hipError_t launch_fwd_lds(int K, const LdsPlan& p, const ConvPtrs& a, const LdsGeo& g, hipStream_t s) {
    const dim3 grid(p.ncb * p.nbt);
    switch (K) {
        case 3: return launch_fwd_lds_k3(p.sh, a, g, grid, s);
        case 5: return launch_fwd_lds_k5(p.sh, a, g, grid, s);
        case 7: return launch_fwd_lds_k7(p.sh, a, g, grid, s);
        case 9: return launch_fwd_lds_k9(p.sh, a, g, grid, s);
        case 15: return launch_fwd_lds_k15(p.sh, a, g, grid, s);
        case 31: return launch_fwd_lds_k31(p.sh, a, g, grid, s);
    }
    return hipErrorInvalidConfiguration;
}
hipError_t launch_bwd_lds(int K, const LdsPlan& p, bool wdx, bool wdw, const ConvPtrs& a, const LdsGeo& g,
                          hipStream_t s) {
    const dim3 grid(p.ncb * p.nbt);
    switch (K) {
        case 3: return launch_bwd_lds_k3(p.sh, wdx, wdw, a, g, grid, s);
        case 5: return launch_bwd_lds_k5(p.sh, wdx, wdw, a, g, grid, s);
        case 7: return launch_bwd_lds_k7(p.sh, wdx, wdw, a, g, grid, s);
        case 9: return launch_bwd_lds_k9(p.sh, wdx, wdw, a, g, grid, s);
        case 15: return launch_bwd_lds_k15(p.sh, wdx, wdw, a, g, grid, s);
        case 31: return launch_bwd_lds_k31(p.sh, wdx, wdw, a, g, grid, s);
    }
    return hipErrorInvalidConfiguration;
}

// ---- role-split LDS-staged kernels at K = 31 and 15 (dwconv_lds_split_kernels.h) ---------------------
bool split_eligible(bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    const int E = bf16 ? 2 : 4;
    if (!lds_split_kernel_size(K) || T < 1) return false;
    if (((long long)C * E) % 16 || align_bits % 16) return false;
    const SplitShapeSel sh = lds_split_shape(false, bf16, K);      // the column block is the same in both passes
    return (long long)C * E >= (long long)sh.ncw * 64 * sh.vec * E;
}
int make_split_plan(bool fwd, bool bf16, long long T, int C, int K, const nplm_dwconv_tuning* tune, LdsPlan* out,
                    bool gated = false) {
    LdsPlan p{};
    nplm_dwconv_tuning z{};
    if (!tune) tune = &z;
    const int E = bf16 ? 2 : 4;
    const SplitShapeSel sh = !gated ? lds_split_shape(fwd, bf16, K) : fwd ? lds_split_gated_fwd_shape(bf16, K) : lds_split_gated_shape(bf16, K);
    const long long cb_bytes = (long long)sh.ncw * 64 * sh.vec * E;
    const long long row_bytes = (long long)C * E;
    p.R = sh.rw * sh.nrg;
    if ((long long)(p.R + K) * row_bytes * (gated ? 2 : 1) + 2 * row_bytes >= INT_MAX) return -NPLM_DWCONV_ESHAPE;
    p.ncb = ceil_div(row_bytes, cb_bytes);
    p.ntiles = ceil_div(T, p.R);
    int nbt = tune->nbt > 0 ? tune->nbt : kNumCU / p.ncb;     // one block of 16 waves per CU
    if (nbt < 1) nbt = 1;
    if (nbt > p.ntiles) nbt = p.ntiles;
    if (tune->nbt <= 0 && !fwd) {
        const long long cap = (long long)(kSlabBudgetBytes / ((size_t)(K + 1) * C * sizeof(float)));
        if (nbt > cap && cap >= 1) nbt = (int)cap;
    }
    p.nbt = nbt;
    int G = tune->xcd_remap == 0 ? 8 : (tune->xcd_remap > 0 ? tune->xcd_remap : 0);
    const long long nblocks = (long long)p.ncb * p.nbt;
    if (G > 0 && !(nblocks % kNumXCD == 0 && (nblocks / kNumXCD) % G == 0 && p.nbt % G == 0)) G = 0;
    p.xcd_group = G;
    p.rot_step = nbt > 2 ? (int)((long long)nbt * 618 / 1000) | 1 : 0;
    if (p.rot_step >= nbt) p.rot_step = nbt - 1;
    *out = p;
    return 0;
}

// algo requested by the caller (0 = library's choice) -> 1 sliding-window, 2 LDS-staged, 3 role-split LDS-staged.
// Measured on MI355X, bf16, T=131072:
//   K=7, C=1024: both passes are fastest LDS-staged (the chip sweeps one compact window of rows with every load of a
//     tile issued at once).
//   K=31 and K=15 backward (ALU-bound; one wave cannot hold the fused backward's registers): the role-split kernel,
//     when every output is asked for - C=2048, K=31: 510 us against 720 sliding-window on the log-normal length mix;
//     K=15: 345 against 385 (C=1024: 177 against 205). A backward asked for dx alone or dw/db alone takes the
//     sliding-window kernel, like everything the LDS kernels are not built for (other sizes, narrow or unaligned rows).
//   K=31 forward: the role-split kernel's dx role on every wave, 262 us against 299 LDS-staged with loader waves (C=2048).
//   K=15 forward: LDS-staged with loader waves, 190 us against 203 role-split and 227 sliding-window (C=2048).
int choose_algo(bool bwd, const nplm_dwconv_tuning* tune, bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    if (tune && tune->algo == 3) return split_eligible(bf16, T, C, K, align_bits) ? 3 : -NPLM_DWCONV_ETUNING;
    if (tune && tune->algo == 2) return lds_eligible(bf16, T, C, K, align_bits) ? 2 : -NPLM_DWCONV_ETUNING;
    if (tune && tune->algo == 1) return 1;
    if (split_eligible(bf16, T, C, K, align_bits) && (bwd || K == 31)) return 3;
    return lds_preferred(bwd, bf16, T, C, K, align_bits) ? 2 : 1;
}

// 256 threads x 4 x 16 B = one contiguous 16 KiB chunk per block
__global__ void __launch_bounds__(256) copy_chunks_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t nvec) {
    const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + u * 256 < nvec) v[u] = src[base + u * 256];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + u * 256 < nvec) dst[base + u * 256] = v[u];
}

__global__ void fill_zero_kernel(float* p, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}
__global__ void fill_zero16_kernel(uint16_t* p, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}
hipError_t fill_zero16(void* p, long long n, hipStream_t s) {
    if (!p || n <= 0) return hipSuccess;
    hipLaunchKernelGGL(fill_zero16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (uint16_t*)p, n);
    return hipGetLastError();
}
hipError_t fill_zero(float* p, long long n, hipStream_t s) {
    if (!p || n <= 0) return hipSuccess;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n);
    return hipGetLastError();
}

// launch flags of the kernels (W_BF16 | W_RESIDUAL) from the ABI's weight dtype and flags
// Shapes the gated (z = [u | g]) kernels are built for.
bool gated_supported(bool bwd, bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    const int E = bf16 ? 2 : 4;
    if (!lds_gated_kernel_size(K, bwd) || T < 1) return false;
    if (((long long)C * E) % 16 || align_bits % 16) return false;
    return (long long)C * E >= 1024;
}

// Long gated backward (K = 15, 31), role-split (dwconv_lds_split_kernels.h, GATED): rows of whole 16-byte chunks that fill
// at least one 512-byte column block, 16-byte aligned tensors. Measured at T=131072, C=2048, bf16, backward + finalize
// against the sliding-window kernel below (log-normal length mix / one long sequence): K=31 728 / 685 against 949 / 808 us,
// K=15 584 / 535 against 613 / 593 us; dz is the same bit for bit (same tap order).
bool split_gated_eligible(bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    return split_eligible(bf16, T, C, K, align_bits);
}
// Otherwise: the sliding-window kernel with one channel per lane; same shapes as the gated forward.
bool long_gated_bwd_supported(bool bf16, long long T, int C, int K, uintptr_t align_bits) {
    return long_gated_kernel_size(K) && gated_supported(false, bf16, T, C, K, align_bits);
}
int make_long_gated_plan(bool bf16, long long T, int C, int K, Plan* out) {
    nplm_dwconv_tuning t{};
    t.vec = 1;
    return make_plan(true, bf16, T, C, K, 0, &t, out);
}

int kernel_w_flags(int32_t w_dtype, uint32_t flags) {
    return (w_dtype == NPLM_DWCONV_BF16 ? W_BF16 : 0) | ((flags & NPLM_DWCONV_RESIDUAL) ? W_RESIDUAL : 0);
}

int fwd_impl(const void* x, const int32_t* cu, const void* w, const void* b, void* y, int64_t T, int32_t C,
             int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream,
             const nplm_dwconv_tuning* tune) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)NPLM_DWCONV_RESIDUAL) return -NPLM_DWCONV_EFLAGS;
    if (T == 0) return 0;
    if (!x || !cu || !w || !y) return -NPLM_DWCONV_ENULL;
    const int tap_off = (exec_kernel_size(K) - K) / 2;
    K = exec_kernel_size(K);        // from here on the kernel size that runs
    const int w_flags = kernel_w_flags(w_dtype, flags) | (tap_off << W_TAP_OFF_SHIFT);
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t E = bf16 ? 2 : 4;
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)y;
    if (bits % E) return -NPLM_DWCONV_EALIGN;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if (((uintptr_t)w | (uintptr_t)b) % WE || (uintptr_t)cu % 4) return -NPLM_DWCONV_EALIGN;
    hipStream_t s = (hipStream_t)stream;
    const int algo = choose_algo(false, tune, bf16, T, C, K, bits);
    if (algo < 0) return algo;
    if (algo == 3) {
        LdsPlan lp;
        rc = make_split_plan(true, bf16, T, C, K, tune, &lp);
        if (rc) return rc;
        const ConvPtrs la{x, nullptr, cu, w, b, y, nullptr};
        const LdsGeo lg = make_lds_geo(lp, T, C, S, w_flags);
        return (int)(K == 31 ? launch_fwd_split_k31(bf16, la, lg, dim3(lp.ncb * lp.nbt), s)
                             : launch_fwd_split_k15(bf16, la, lg, dim3(lp.ncb * lp.nbt), s));
    }
    if (algo == 2) {
        LdsPlan lp;
        rc = make_lds_plan(false, bf16, T, C, K, tune, &lp);
        if (rc) return rc;
        const ConvPtrs la{x, nullptr, cu, w, b, y, nullptr};
        const hipError_t e = launch_fwd_lds(K, lp, la, make_lds_geo(lp, T, C, S, w_flags), s);
        if (e == hipErrorInvalidConfiguration && tune) return -NPLM_DWCONV_ETUNING;
        return (int)e;
    }
    Plan p;
    rc = make_plan(false, bf16, T, C, K, bits, tune, &p);
    if (rc) return rc;
    if (p.generic) {
        const int wpb = 4;
        int blocks = ceil_div(T, wpb);
        if (blocks > kNumCU * 16) blocks = kNumCU * 16;
        if (bf16)
            hipLaunchKernelGGL(dwconv_generic_rows_kernel<true>, dim3(blocks), dim3(wpb * 64), 0, s, x, cu, w, b, y,
                               (int)T, C, S, K, w_flags, 0);
        else
            hipLaunchKernelGGL(dwconv_generic_rows_kernel<false>, dim3(blocks), dim3(wpb * 64), 0, s, x, cu, w, b, y,
                               (int)T, C, S, K, w_flags, 0);
        return (int)hipGetLastError();
    }
    const ConvPtrs a{x, nullptr, cu, w, b, y, nullptr};
    const hipError_t e = launch_fwd(K, bf16, p, a, make_geo(p, T, C, S, w_flags), s);
    if (e == hipErrorInvalidConfiguration && tune) return -NPLM_DWCONV_ETUNING;
    return (int)e;
}

int bwd_impl(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx, float* dw, float* db,
             void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K, int32_t S,
             int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream, const nplm_dwconv_tuning* tune) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)(NPLM_DWCONV_RESIDUAL | NPLM_DWCONV_GRADS_BF16)) return -NPLM_DWCONV_EFLAGS;
    const int out_bf16 = (flags & NPLM_DWCONV_GRADS_BF16) ? 1 : 0;      // dw, db are bf16 buffers
    hipStream_t s = (hipStream_t)stream;
    const bool want_red = dw || db;
    if (T == 0) {
        hipError_t e = out_bf16 ? fill_zero16(dw, (long long)C * K, s) : fill_zero(dw, (long long)C * K, s);
        if (e == hipSuccess) e = out_bf16 ? fill_zero16(db, C, s) : fill_zero(db, C, s);
        return (int)e;
    }
    const int tap_off = (exec_kernel_size(K) - K) / 2;
    K = exec_kernel_size(K);        // from here on the kernel size that runs (slabs of K + 1 rows; dw rows stay the caller's)
    const int w_flags = kernel_w_flags(w_dtype, flags) | (tap_off << W_TAP_OFF_SHIFT);
    if (!dx && !want_red) return 0;
    if (!dy || !cu || !w || (want_red && !x)) return -NPLM_DWCONV_ENULL;
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t E = bf16 ? 2 : 4;
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx;
    if (bits % E) return -NPLM_DWCONV_EALIGN;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if ((uintptr_t)w % WE || (uintptr_t)cu % 4 || ((uintptr_t)dw | (uintptr_t)db) % (out_bf16 ? 2 : 4)) return -NPLM_DWCONV_EALIGN;

    int algo = choose_algo(true, tune, bf16, T, C, K, bits);
    if (algo < 0) return algo;
    if (algo == 3 && !(dx && want_red)) {     // the role-split kernel is fused only: a partial request takes the others
        if (tune && tune->algo == 3) return -NPLM_DWCONV_ETUNING;
        algo = 1;
    }
    if (algo == 3) {
        LdsPlan lp;
        rc = make_split_plan(false, bf16, T, C, K, tune, &lp);
        if (rc) return rc;
        const size_t slab_bytes = (size_t)(K + 1) * C * sizeof(float);
        if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab_bytes * (size_t)lp.nbt)
            return -NPLM_DWCONV_EWORKSPACE;
        float* part = reinterpret_cast<float*>(workspace);
        const ConvPtrs la{x, dy, cu, w, nullptr, dx, part};
        const LdsGeo lg = make_lds_geo(lp, T, C, S, w_flags);
        const dim3 grid(lp.ncb * lp.nbt);
        hipError_t e = K == 31 ? launch_bwd_split_k31(bf16, la, lg, grid, s) : launch_bwd_split_k15(bf16, la, lg, grid, s);
        if (e != hipSuccess) return (int)e;
        if (tune && tune->mid_event) {
            e = hipEventRecord((hipEvent_t)tune->mid_event, s);
            if (e != hipSuccess) return (int)e;
        }
        const long long n_out = (long long)(K + 1) * C;
        hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)), dim3(64 * FIN_SPLIT), 0,
                           s, (const float*)part, lp.nbt, C, K, dw, db, out_bf16, tap_off);
        return (int)hipGetLastError();
    }
    if (algo == 2) {
        LdsPlan lp;
        rc = make_lds_plan(true, bf16, T, C, K, tune, &lp);
        if (rc) return rc;
        const size_t slab_bytes = (size_t)(K + 1) * C * sizeof(float);
        float* part = nullptr;
        if (want_red) {
            if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab_bytes * (size_t)lp.nbt)
                return -NPLM_DWCONV_EWORKSPACE;
            part = reinterpret_cast<float*>(workspace);
        }
        const ConvPtrs la{x, dy, cu, w, nullptr, dx, part};
        hipError_t e = launch_bwd_lds(K, lp, dx != nullptr, want_red, la,
                                      make_lds_geo(lp, T, C, S, w_flags), s);
        if (e == hipErrorInvalidConfiguration && tune) return -NPLM_DWCONV_ETUNING;
        if (e != hipSuccess) return (int)e;
        if (tune && tune->mid_event) {
            e = hipEventRecord((hipEvent_t)tune->mid_event, s);
            if (e != hipSuccess) return (int)e;
        }
        if (want_red) {
            const long long n_out = (long long)(K + 1) * C;
            hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)),
                               dim3(64 * FIN_SPLIT), 0, s, (const float*)part, lp.nbt, C, K, dw, db, out_bf16, tap_off);
            e = hipGetLastError();
        }
        return (int)e;
    }
    Plan p;
    rc = make_plan(true, bf16, T, C, K, bits, tune, &p);
    if (rc) return rc;
    if (!tune) {
        // never use more slabs than nplm_dwconv_bwd_workspace_bytes() promised for aligned inputs
        Plan nominal;
        rc = make_plan(true, bf16, T, C, K, 0, nullptr, &nominal);
        if (rc) return rc;
        if (p.nbt > nominal.nbt) {
            p.nbt = nominal.nbt;
            p.remap = p.remap && ((long long)p.ncb * p.nbt) % kNumXCD == 0;
        }
    }
    const size_t slab = (size_t)(K + 1) * C * sizeof(float);
    float* partial = nullptr;
    if (want_red) {
        if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab * (size_t)p.nbt)
            return -NPLM_DWCONV_EWORKSPACE;
        partial = reinterpret_cast<float*>(workspace);
    }

    if (p.generic) {
        if (dx) {
            const int wpb = 4;
            int blocks = ceil_div(T, wpb);
            if (blocks > kNumCU * 16) blocks = kNumCU * 16;
            if (bf16)
                hipLaunchKernelGGL(dwconv_generic_rows_kernel<true>, dim3(blocks), dim3(wpb * 64), 0, s, dy, cu, w,
                                   (const void*)nullptr, dx, (int)T, C, S, K, w_flags, 1);
            else
                hipLaunchKernelGGL(dwconv_generic_rows_kernel<false>, dim3(blocks), dim3(wpb * 64), 0, s, dy, cu, w,
                                   (const void*)nullptr, dx, (int)T, C, S, K, w_flags, 1);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return (int)e;
        }
        if (want_red) {
            const int rows = ceil_div(T, p.nbt);
            const dim3 grid(p.nbt, ceil_div(C, 256));
            if (bf16)
                hipLaunchKernelGGL(dwconv_generic_dw_kernel<true>, grid, dim3(256), 0, s, x, dy, cu, partial, (int)T, C,
                                   S, K, rows);
            else
                hipLaunchKernelGGL(dwconv_generic_dw_kernel<false>, grid, dim3(256), 0, s, x, dy, cu, partial, (int)T,
                                   C, S, K, rows);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return (int)e;
        }
    } else {
        const ConvPtrs a{x, dy, cu, w, nullptr, dx, partial};
        const hipError_t e = launch_bwd(K, bf16, p, dx != nullptr, want_red, a, make_geo(p, T, C, S, w_flags), s);
        if (e == hipErrorInvalidConfiguration && tune) return -NPLM_DWCONV_ETUNING;
        if (e != hipSuccess) return (int)e;
    }
    if (tune && tune->mid_event) {
        const hipError_t e = hipEventRecord((hipEvent_t)tune->mid_event, s);
        if (e != hipSuccess) return (int)e;
    }
    if (want_red) {
        const long long n_out = (long long)(K + 1) * C;
        hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)), dim3(64 * FIN_SPLIT), 0, s,
                           (const float*)partial, p.nbt, C, K, dw, db, out_bf16, tap_off);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

// Device address of `scratch` on the current device, looked up once per device and kept.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

hipError_t static_scratch_for_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(p, std::memory_order_release);   // every thread finds the same address
    }
    *out = p;
    return hipSuccess;
}

}  // namespace
}  // namespace nplm

// ---- LayerNorm-fused conv: shapes, geometry and the one-wave-per-row kernels' launchers ----------------------------
namespace nplm {
namespace {
// rows of one 2 KiB column block: one forward kernel that takes the statistics from the tile it has staged
bool ln_whole_rows(bool bf16, int C, int K, uintptr_t align_bits) {
    const long long row_bytes = (long long)C * (bf16 ? 2 : 4);
    return lds_ln_kernel_size(K) && row_bytes % 16 == 0 && row_bytes <= kLnCbBytes && align_bits % 16 == 0;
}
// forward, fp32 rows of up to 4 KiB: the same kernel with 6 or 8 wave-columns and shorter tiles, see lds_ln_3k_shape()
// and lds_ln_4k_shape()
bool ln_fwd_whole_4k(bool bf16, int C, int K, uintptr_t align_bits) {
    const long long row_bytes = (long long)C * 4;
    return !bf16 && lds_ln_kernel_size(K) && row_bytes % 16 == 0 && row_bytes > kLnCbBytes && row_bytes <= 2 * kLnCbBytes &&
           align_bits % 16 == 0;
}
// backward: rows of up to 4 KiB also fit a block, see lds_ln_bwd_wide_shape() and lds_ln_bwd_3k_shape()
bool ln_bwd_whole_4k(bool bf16, int C, int K, uintptr_t align_bits) {
    const long long row_bytes = (long long)C * (bf16 ? 2 : 4);
    return lds_ln_bwd_wide_kernel_size(K) && row_bytes % 16 == 0 && row_bytes > kLnCbBytes && row_bytes <= 4096 &&
           align_bits % 16 == 0;
}
// other rows of up to 8 KiB: a row-statistics kernel, then the conv forward that normalises as it reads (the forward
// asks ln_fwd_whole_4k first)
bool ln_wide_rows(bool bf16, int C, int K, uintptr_t align_bits) {
    const long long row_bytes = (long long)C * (bf16 ? 2 : 4);
    return lds_ln_kernel_size(K) && row_bytes % 16 == 0 && row_bytes > kLnCbBytes && row_bytes <= 8192 && align_bits % 16 == 0;
}
// 16-byte chunks per lane of the one-wave-per-row kernels: rows of at most 2, 4, 8 KiB
int ln_row_chunks(long long row_bytes) { return row_bytes <= 2048 ? 2 : row_bytes <= 4096 ? 4 : 8; }
int ln_row_blocks(long long T) {
    const int blocks = ceil_div(T, 4);
    return blocks > kNumCU * 8 ? kNumCU * 8 : blocks;
}
// the default shape of a pass as an explicit geometry, whatever lds_shape_for() would pick for the width
int make_default_lds_plan(bool bwd, bool bf16, long long T, int C, int K, LdsPlan* out) {
    nplm_dwconv_tuning t{};
    const LdsShapeSel sh = lds_default_shape(bwd, bf16, K);
    t.vec = sh.vec; t.unroll = sh.rw; t.bt = sh.nrg; t.bw = sh.ncw; t.nwl = sh.nwl; t.nbuf = sh.nbuf;
    return make_lds_plan(bwd, bf16, T, C, K, &t, out);
}
template <bool BF16>
hipError_t launch_ln_stats(int nch, const void* x, float* stats, float eps, long long T, int C, hipStream_t s) {
    const dim3 grid(ln_row_blocks(T)), block(256);
    if (nch == 2) hipLaunchKernelGGL((ln_stats_kernel<BF16, 2>), grid, block, 0, s, x, stats, eps, (int)T, C);
    else if (nch == 4) hipLaunchKernelGGL((ln_stats_kernel<BF16, 4>), grid, block, 0, s, x, stats, eps, (int)T, C);
    else hipLaunchKernelGGL((ln_stats_kernel<BF16, 8>), grid, block, 0, s, x, stats, eps, (int)T, C);
    return hipGetLastError();
}
template <bool BF16>
hipError_t launch_ln_bwd_dx(int nch, const void* x, const float* stats, const void* gamma, int w_flags, const float* dn,
                            const void* dy, void* dx, long long T, int C, hipStream_t s) {
    const dim3 grid(ln_row_blocks(T)), block(256);
    if (nch == 2) hipLaunchKernelGGL((ln_bwd_dx_kernel<BF16, 2>), grid, block, 0, s, x, stats, gamma, w_flags, dn, dy, dx, (int)T, C);
    else if (nch == 4) hipLaunchKernelGGL((ln_bwd_dx_kernel<BF16, 4>), grid, block, 0, s, x, stats, gamma, w_flags, dn, dy, dx, (int)T, C);
    else hipLaunchKernelGGL((ln_bwd_dx_kernel<BF16, 8>), grid, block, 0, s, x, stats, gamma, w_flags, dn, dy, dx, (int)T, C);
    return hipGetLastError();
}
}  // namespace
}  // namespace nplm

using namespace nplm;

extern "C" {

int nplm_dwconv_version(void) { return kVersion; }

int nplm_dwconv_gated_fwd(const void* z, const int32_t* cu, const void* w, const void* b, void* y, int64_t T,
                          int32_t C, int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype, uint32_t flags,
                          void* stream) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)NPLM_DWCONV_RESIDUAL) return -NPLM_DWCONV_EFLAGS;
    if (T == 0) return 0;
    if (!z || !cu || !w || !y) return -NPLM_DWCONV_ENULL;
    const int tap_flags = ((exec_kernel_size(K) - K) / 2) << W_TAP_OFF_SHIFT;
    K = exec_kernel_size(K);        // from here on the kernel size that runs
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if (((uintptr_t)w | (uintptr_t)b) % WE || (uintptr_t)cu % 4) return -NPLM_DWCONV_EALIGN;
    if (!gated_supported(false, bf16, T, C, K, (uintptr_t)z | (uintptr_t)y)) return -NPLM_DWCONV_EUNSUPPORTED;
    LdsPlan lp;
    if (long_gated_kernel_size(K) && split_gated_eligible(bf16, T, C, K, (uintptr_t)z | (uintptr_t)y)) {
        rc = make_split_plan(true, bf16, T, C, K, nullptr, &lp, true);
        if (rc) return rc;
        const ConvPtrs la{z, nullptr, cu, w, b, y, nullptr};
        const LdsGeo lg = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags) | tap_flags);
        const dim3 grid(lp.ncb * lp.nbt);
        return (int)(K == 31 ? launch_fwd_split_gated_k31(bf16, la, lg, grid, (hipStream_t)stream)
                             : launch_fwd_split_gated_k15(bf16, la, lg, grid, (hipStream_t)stream));
    }
    rc = make_lds_plan(false, bf16, T, C, K, nullptr, &lp, true);
    if (rc) return rc == -NPLM_DWCONV_ETUNING ? -NPLM_DWCONV_EUNSUPPORTED : rc;
    const ConvPtrs la{z, nullptr, cu, w, b, y, nullptr};
    const bool narrow = lds_gated_narrow((long long)C * (bf16 ? 2 : 4), K);
    const LdsGeo g = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags) | tap_flags);
    const dim3 grid(lp.ncb * lp.nbt);
    hipStream_t s = (hipStream_t)stream;
    switch (K) {
        case 15: return (int)launch_fwd_lds_gated_k15(bf16, narrow, la, g, grid, s);
        case 31: return (int)launch_fwd_lds_gated_k31(bf16, narrow, la, g, grid, s);
        case 3: return (int)launch_fwd_lds_gated_k3(bf16, narrow, la, g, grid, s);
        case 5: return (int)launch_fwd_lds_gated_k5(bf16, narrow, la, g, grid, s);
        case 7: return (int)launch_fwd_lds_gated_k7(bf16, narrow, la, g, grid, s);
        case 9: return (int)launch_fwd_lds_gated_k9(bf16, narrow, la, g, grid, s);
    }
    return -NPLM_DWCONV_EUNSUPPORTED;
}

// ---- LayerNorm-fused conv (dwconv_ln_kernels.h and the NORM variants of the LDS-staged kernels) ----------------------
int nplm_dwconv_ln_fwd(const void* x, const int32_t* cu, const void* ln_weight, const void* ln_bias, float eps,
                       const void* w, const void* b, void* y, float* stats, int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)NPLM_DWCONV_RESIDUAL) return -NPLM_DWCONV_EFLAGS;
    if (T == 0) return 0;
    if (!x || !cu || !w || !y || !ln_weight) return -NPLM_DWCONV_ENULL;
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t E = bf16 ? 2 : 4;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if (((uintptr_t)w | (uintptr_t)b | (uintptr_t)ln_weight | (uintptr_t)ln_bias) % WE || (uintptr_t)cu % 4 ||
        (uintptr_t)stats % 4 || ((uintptr_t)x | (uintptr_t)y) % E)
        return -NPLM_DWCONV_EALIGN;
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)y;
    hipStream_t s = (hipStream_t)stream;
    const ConvPtrs la{x, nullptr, cu, w, b, y, nullptr};
    const bool rows4k = ln_fwd_whole_4k(bf16, C, K, bits);
    if (!rows4k && ln_wide_rows(bf16, C, K, bits)) {
        if (!stats) return -NPLM_DWCONV_ENULL;      // the statistics pass between the two kernels through it
        LdsPlan lp;
        rc = make_default_lds_plan(false, bf16, T, C, K, &lp);
        if (rc) return rc == -NPLM_DWCONV_ETUNING ? -NPLM_DWCONV_EUNSUPPORTED : rc;
        const int nch = ln_row_chunks((long long)C * (long long)E);
        hipError_t e = bf16 ? launch_ln_stats<true>(nch, x, stats, eps, T, C, s) : launch_ln_stats<false>(nch, x, stats, eps, T, C, s);
        if (e != hipSuccess) return (int)e;
        const LnSide side{stats, ln_weight, ln_bias, nullptr};
        const LdsGeo g = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags));
        const dim3 grid(lp.ncb * lp.nbt);
        switch (K) {
            case 3: return (int)launch_ln_fwd_wide_k3(bf16, la, side, g, grid, s);
            case 5: return (int)launch_ln_fwd_wide_k5(bf16, la, side, g, grid, s);
            case 7: return (int)launch_ln_fwd_wide_k7(bf16, la, side, g, grid, s);
            case 9: return (int)launch_ln_fwd_wide_k9(bf16, la, side, g, grid, s);
        }
        return -NPLM_DWCONV_EUNSUPPORTED;
    }
    if (!rows4k && !ln_whole_rows(bf16, C, K, bits)) return -NPLM_DWCONV_EUNSUPPORTED;
    LdsPlan lp{};
    lp.sh = !rows4k ? lds_ln_shape(bf16) : lds_ln_rows3k(bf16, C) ? lds_ln_3k_shape(K) : lds_ln_4k_shape(bf16, K);
    lp.R = lp.sh.rw * lp.sh.nrg;
    lp.ncb = 1;
    lp.ntiles = ceil_div(T, lp.R);
    lp.nbt = lp.ntiles < kNumCU ? lp.ntiles : kNumCU;          // one block of 16 waves and three tiles per CU
    lp.xcd_group = (lp.nbt % (kNumXCD * 8) == 0) ? 8 : 0;
    // fp32 rows of 4 KiB: 6 of a tile's 13 staged rows are a neighbour's, and a neighbour on another XCD means reading them
    // from HBM again; 32 consecutive tiles per XCD instead of 8 (T=131072, C=1024, K=7: 217 against 222 us per call; the
    // other whole-row kernels, with longer tiles, measure the same either way)
    if (rows4k && lp.nbt % (kNumXCD * 32) == 0) lp.xcd_group = 32;
    lp.rot_step = lp.nbt > 2 ? (int)((long long)lp.nbt * 618 / 1000) | 1 : 0;
    if (lp.rot_step >= lp.nbt) lp.rot_step = lp.nbt - 1;
    const LnArgs ln{ln_weight, ln_bias, stats, eps};
    const LdsGeo g = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags));
    const dim3 grid(lp.nbt);
    if (rows4k) {
        switch (K) {
            case 3: return (int)launch_ln_fwd_4k_k3(bf16, la, ln, g, grid, s);
            case 5: return (int)launch_ln_fwd_4k_k5(bf16, la, ln, g, grid, s);
            case 7: return (int)launch_ln_fwd_4k_k7(bf16, la, ln, g, grid, s);
            case 9: return (int)launch_ln_fwd_4k_k9(bf16, la, ln, g, grid, s);
        }
        return -NPLM_DWCONV_EUNSUPPORTED;
    }
    switch (K) {
        case 3: return (int)launch_ln_fwd_k3(bf16, la, ln, g, grid, s);
        case 5: return (int)launch_ln_fwd_k5(bf16, la, ln, g, grid, s);
        case 7: return (int)launch_ln_fwd_k7(bf16, la, ln, g, grid, s);
        case 9: return (int)launch_ln_fwd_k9(bf16, la, ln, g, grid, s);
    }
    return -NPLM_DWCONV_EUNSUPPORTED;
}

// ---- backward of the LayerNorm-fused forward: conv backward over the re-normalised x (NORM variant of
// dwconv_bwd_lds_kernel: dn, dw, db and the LayerNorm parameter sums), then the LayerNorm input gradient ---------------
namespace {
bool ln_supported(bool bf16, int C, int K, uintptr_t align_bits) {
    return ln_whole_rows(bf16, C, K, align_bits) || ln_wide_rows(bf16, C, K, align_bits);
}
// workspace: [conv slabs: nbt x (K+1) x C][LayerNorm slabs: nbt x 2 x C][dn: T x C fp32], each part 256-byte aligned;
// rows of one 2 KiB column block finish dx inside the conv backward (the WHOLE variant) and need no dn
struct LnBwdLayout {
    LdsPlan lp;
    bool whole, whole4k;      // dx inside the conv backward: rows of one 2 KiB column block; rows of one 4 KiB block
    size_t conv_slabs, ln_slabs, dn, total;
};
int ln_bwd_layout(bool bf16, long long T, int C, int K, LnBwdLayout* out) {
    LnBwdLayout l{};
    l.whole4k = ln_bwd_whole_4k(bf16, C, K, 0);
    l.whole = l.whole4k || ln_whole_rows(bf16, C, K, 0);
    if (l.whole) {
        l.lp.sh = !l.whole4k ? lds_ln_bwd_shape(bf16, K) : lds_ln_bwd_rows3k(bf16, C) ? lds_ln_bwd_3k_shape(K) : lds_ln_bwd_wide_shape(bf16, K);
        l.lp.R = l.lp.sh.rw * l.lp.sh.nrg;
        l.lp.ncb = 1;
        l.lp.ntiles = ceil_div(T, l.lp.R);
        l.lp.nbt = l.lp.ntiles < kNumCU ? l.lp.ntiles : kNumCU;
        l.lp.xcd_group = (l.lp.nbt % (kNumXCD * 8) == 0) ? 8 : 0;
        // rows of 2 to 4 KiB: a tile is 5 to 10 rows behind K-1 halo rows of dy, and a neighbour on another XCD means reading
        // those from HBM again (fp32 C=1024, K=7: 6-row tiles, HBM-side reads 1.066 of x + dy with 8 consecutive tiles per
        // XCD); 32 consecutive tiles per XCD, as in the forward of these rows
        if (l.whole4k && l.lp.nbt % (kNumXCD * 32) == 0) l.lp.xcd_group = 32;
        l.lp.rot_step = l.lp.nbt > 2 ? (int)((long long)l.lp.nbt * 618 / 1000) | 1 : 0;
        if (l.lp.rot_step >= l.lp.nbt) l.lp.rot_step = l.lp.nbt - 1;
    } else {
        int rc = make_default_lds_plan(true, bf16, T, C, K, &l.lp);
        if (rc) return rc;
    }
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    l.conv_slabs = up((size_t)l.lp.nbt * (K + 1) * C * sizeof(float));
    l.ln_slabs = up((size_t)l.lp.nbt * 2 * C * sizeof(float));
    l.dn = l.whole ? 0 : up((size_t)T * C * sizeof(float));
    l.total = l.conv_slabs + l.ln_slabs + l.dn;
    *out = l;
    return 0;
}
}  // namespace

size_t nplm_dwconv_ln_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype) {
    if (check_common(T, C, K, 0, act_dtype, NPLM_DWCONV_F32) || T == 0) return 0;
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    if (!ln_supported(bf16, C, K, 0)) return 0;
    LnBwdLayout l;
    if (ln_bwd_layout(bf16, T, C, K, &l)) return 0;
    return l.total;
}

int nplm_dwconv_ln_bwd(const void* x, const void* dy, const int32_t* cu, const float* stats, const void* ln_weight,
                       const void* ln_bias, const void* w, void* dx, float* dw, float* db, float* dln_weight,
                       float* dln_bias, void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K,
                       int32_t S, int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)(NPLM_DWCONV_RESIDUAL | NPLM_DWCONV_GRADS_BF16)) return -NPLM_DWCONV_EFLAGS;
    const int out_bf16 = (flags & NPLM_DWCONV_GRADS_BF16) ? 1 : 0;      // dw, db, dln_weight, dln_bias are bf16 buffers
    hipStream_t s = (hipStream_t)stream;
    if (!dw || !db || !dln_weight) return -NPLM_DWCONV_ENULL;
    if (T == 0) {
        auto zero = [&](float* p, long long n) { return out_bf16 ? fill_zero16(p, n, s) : fill_zero(p, n, s); };
        hipError_t e = zero(dw, (long long)C * K);
        if (e == hipSuccess) e = zero(db, C);
        if (e == hipSuccess) e = zero(dln_weight, C);
        if (e == hipSuccess) e = zero(dln_bias, C);
        return (int)e;
    }
    if (!x || !dy || !cu || !stats || !ln_weight || !w || !dx) return -NPLM_DWCONV_ENULL;
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t E = bf16 ? 2 : 4;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if (((uintptr_t)w | (uintptr_t)ln_weight | (uintptr_t)ln_bias) % WE || ((uintptr_t)cu | (uintptr_t)stats) % 4 ||
        ((uintptr_t)dw | (uintptr_t)db | (uintptr_t)dln_weight | (uintptr_t)dln_bias) % (out_bf16 ? 2 : 4) ||
        ((uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx) % E)
        return -NPLM_DWCONV_EALIGN;
    if (!ln_supported(bf16, C, K, (uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx)) return -NPLM_DWCONV_EUNSUPPORTED;
    LnBwdLayout l;
    rc = ln_bwd_layout(bf16, T, C, K, &l);
    if (rc) return rc == -NPLM_DWCONV_ETUNING ? -NPLM_DWCONV_EUNSUPPORTED : rc;
    if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < l.total) return -NPLM_DWCONV_EWORKSPACE;
    char* ws = reinterpret_cast<char*>(workspace);
    float* part = reinterpret_cast<float*>(ws);
    float* part_ln = reinterpret_cast<float*>(ws + l.conv_slabs);
    float* dn = reinterpret_cast<float*>(ws + l.conv_slabs + l.ln_slabs);
    // the conv's own residual flag stays off: the identity branch bypasses the LayerNorm and joins where dx is formed
    // (the WHOLE variant takes the flag to mean exactly that)
    const int w_flags = kernel_w_flags(w_dtype, l.whole ? (flags & NPLM_DWCONV_RESIDUAL) : 0);
    const ConvPtrs la{x, dy, cu, w, nullptr, l.whole ? dx : (void*)dn, part};
    const LnSide ln{stats, ln_weight, ln_bias, part_ln};
    const LdsGeo g = make_lds_geo(l.lp, T, C, S, w_flags);
    const dim3 grid(l.lp.ncb * l.lp.nbt);
    hipError_t e = hipErrorInvalidConfiguration;
    if (l.whole4k) {
        switch (K) {
            case 3: e = launch_ln_bwd_whole4k_k3(bf16, la, ln, g, grid, s); break;
            case 5: e = launch_ln_bwd_whole4k_k5(bf16, la, ln, g, grid, s); break;
            case 7: e = launch_ln_bwd_whole4k_k7(bf16, la, ln, g, grid, s); break;
            case 9: e = launch_ln_bwd_whole4k_k9(bf16, la, ln, g, grid, s); break;
        }
    } else if (l.whole) {
        switch (K) {
            case 3: e = launch_ln_bwd_whole_k3(bf16, la, ln, g, grid, s); break;
            case 5: e = launch_ln_bwd_whole_k5(bf16, la, ln, g, grid, s); break;
            case 7: e = launch_ln_bwd_whole_k7(bf16, la, ln, g, grid, s); break;
            case 9: e = launch_ln_bwd_whole_k9(bf16, la, ln, g, grid, s); break;
        }
    } else {
        switch (K) {
            case 3: e = launch_ln_bwd_k3(bf16, la, ln, g, grid, s); break;
            case 5: e = launch_ln_bwd_k5(bf16, la, ln, g, grid, s); break;
            case 7: e = launch_ln_bwd_k7(bf16, la, ln, g, grid, s); break;
            case 9: e = launch_ln_bwd_k9(bf16, la, ln, g, grid, s); break;
        }
    }
    if (e != hipSuccess) return (int)e;
    // both slab sets in one launch; the LayerNorm slabs read as a conv of one tap: "dw" = d ln_weight, "db" = d ln_bias
    const int blocks_a = (int)(((long long)(K + 1) * C + 63) / 64), blocks_b = (int)((2LL * C + 63) / 64);
    hipLaunchKernelGGL(dwconv_finalize2_kernel<FIN_SPLIT>, dim3((unsigned)(blocks_a + blocks_b)), dim3(64 * FIN_SPLIT), 0, s,
                       (const float*)part, (int)K, dw, db, blocks_a, (const float*)part_ln, 1, dln_weight, dln_bias, l.lp.nbt, (int)C,
                       out_bf16);
    if (l.whole) return (int)hipGetLastError();
    const void* res = (flags & NPLM_DWCONV_RESIDUAL) ? dy : nullptr;
    const int nch = ln_row_chunks((long long)C * (long long)E);
    return (int)(bf16 ? launch_ln_bwd_dx<true>(nch, x, stats, ln_weight, w_flags, dn, res, dx, T, C, s)
                      : launch_ln_bwd_dx<false>(nch, x, stats, ln_weight, w_flags, dn, res, dx, T, C, s));
}

size_t nplm_dwconv_gated_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype) {
    if (check_common(T, C, K, 0, act_dtype, NPLM_DWCONV_F32) || T == 0) return 0;
    K = exec_kernel_size(K);        // the slabs have the rows of the kernel size that runs
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    if (long_gated_bwd_supported(bf16, T, C, K, 0)) {
        // enough for either kernel: which one runs also depends on pointer alignment, not known here
        Plan p;
        if (make_long_gated_plan(bf16, T, C, K, &p)) return 0;
        int slabs = p.nbt;
        LdsPlan lp;
        if (split_gated_eligible(bf16, T, C, K, 0) && make_split_plan(false, bf16, T, C, K, nullptr, &lp, true) == 0 && lp.nbt > slabs)
            slabs = lp.nbt;
        const size_t bytes = (size_t)slabs * (K + 1) * C * sizeof(float);
        return (bytes + 255) & ~(size_t)255;
    }
    if (!gated_supported(true, bf16, T, C, K, 0)) return 0;
    LdsPlan lp;
    if (make_lds_plan(true, bf16, T, C, K, nullptr, &lp, true)) return 0;
    const size_t bytes = (size_t)lp.nbt * (K + 1) * C * sizeof(float);
    return (bytes + 255) & ~(size_t)255;
}

int nplm_dwconv_gated_bwd(const void* z, const void* dy, const int32_t* cu, const void* w, void* dz, float* dw,
                          float* db, void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K,
                          int32_t S, int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream) {
    int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    if (flags & ~(uint32_t)(NPLM_DWCONV_RESIDUAL | NPLM_DWCONV_GRADS_BF16)) return -NPLM_DWCONV_EFLAGS;
    const int out_bf16 = (flags & NPLM_DWCONV_GRADS_BF16) ? 1 : 0;      // dw, db are bf16 buffers
    hipStream_t s = (hipStream_t)stream;
    if (!dw || !db) return -NPLM_DWCONV_ENULL;
    if (T == 0) {
        hipError_t e = out_bf16 ? fill_zero16(dw, (long long)C * K, s) : fill_zero(dw, (long long)C * K, s);
        if (e == hipSuccess) e = out_bf16 ? fill_zero16(db, C, s) : fill_zero(db, C, s);
        return (int)e;
    }
    if (!z || !dy || !cu || !w || !dz) return -NPLM_DWCONV_ENULL;
    const int tap_off = (exec_kernel_size(K) - K) / 2, tap_flags = tap_off << W_TAP_OFF_SHIFT;
    K = exec_kernel_size(K);        // from here on the kernel size that runs (slabs of K + 1 rows; dw rows stay the caller's)
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const uintptr_t WE = (w_dtype == NPLM_DWCONV_BF16) ? 2 : 4;
    if ((uintptr_t)w % WE || (uintptr_t)cu % 4 || ((uintptr_t)dw | (uintptr_t)db) % (out_bf16 ? 2 : 4)) return -NPLM_DWCONV_EALIGN;
    if (long_gated_kernel_size(K) && split_gated_eligible(bf16, T, C, K, (uintptr_t)z | (uintptr_t)dy | (uintptr_t)dz)) {
        LdsPlan lp;
        rc = make_split_plan(false, bf16, T, C, K, nullptr, &lp, true);
        if (rc) return rc;
        const size_t slab = (size_t)(K + 1) * C * sizeof(float);
        if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab * (size_t)lp.nbt) return -NPLM_DWCONV_EWORKSPACE;
        float* part = reinterpret_cast<float*>(workspace);
        const ConvPtrs la{z, dy, cu, w, nullptr, dz, part};
        const LdsGeo lg = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags) | tap_flags);
        const dim3 grid(lp.ncb * lp.nbt);
        hipError_t e = K == 31 ? launch_bwd_split_gated_k31(bf16, la, lg, grid, s) : launch_bwd_split_gated_k15(bf16, la, lg, grid, s);
        if (e != hipSuccess) return (int)e;
        const long long n_out = (long long)(K + 1) * C;
        hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)), dim3(64 * FIN_SPLIT), 0, s,
                           (const float*)part, lp.nbt, C, K, dw, db, out_bf16, tap_off);
        return (int)hipGetLastError();
    }
    if (long_gated_bwd_supported(bf16, T, C, K, (uintptr_t)z | (uintptr_t)dy | (uintptr_t)dz)) {
        Plan p;
        rc = make_long_gated_plan(bf16, T, C, K, &p);
        if (rc) return rc;
        const size_t slab = (size_t)(K + 1) * C * sizeof(float);
        if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab * (size_t)p.nbt) return -NPLM_DWCONV_EWORKSPACE;
        float* part = reinterpret_cast<float*>(workspace);
        const ConvPtrs a{z, dy, cu, w, nullptr, dz, part};
        const Geo g = make_geo(p, T, C, S, kernel_w_flags(w_dtype, flags) | tap_flags);
        const dim3 grid(p.ncb * p.nbt), block(p.bw * p.bt * 64);
        const size_t shmem = (size_t)p.bw * p.bt * p.vec * 64 * sizeof(float);
        hipError_t e = K == 15 ? launch_bwd_gated_k15(bf16, p.unroll, p.maxt, a, g, grid, block, shmem, s)
                               : launch_bwd_gated_k31(bf16, p.unroll, p.maxt, a, g, grid, block, shmem, s);
        if (e != hipSuccess) return (int)e;
        const long long n_out = (long long)(K + 1) * C;
        hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)), dim3(64 * FIN_SPLIT), 0, s,
                           (const float*)part, p.nbt, C, K, dw, db, out_bf16, tap_off);
        return (int)hipGetLastError();
    }
    if (!gated_supported(true, bf16, T, C, K, (uintptr_t)z | (uintptr_t)dy | (uintptr_t)dz)) return -NPLM_DWCONV_EUNSUPPORTED;
    LdsPlan lp;
    rc = make_lds_plan(true, bf16, T, C, K, nullptr, &lp, true);
    if (rc) return rc == -NPLM_DWCONV_ETUNING ? -NPLM_DWCONV_EUNSUPPORTED : rc;
    const size_t slab_bytes = (size_t)(K + 1) * C * sizeof(float);
    if (!workspace || (uintptr_t)workspace % 256 || workspace_bytes < slab_bytes * (size_t)lp.nbt)
        return -NPLM_DWCONV_EWORKSPACE;
    float* part = reinterpret_cast<float*>(workspace);
    const ConvPtrs la{z, dy, cu, w, nullptr, dz, part};
    const bool narrow = lds_gated_narrow((long long)C * (bf16 ? 2 : 4), K);
    const LdsGeo g = make_lds_geo(lp, T, C, S, kernel_w_flags(w_dtype, flags) | tap_flags);
    const dim3 grid(lp.ncb * lp.nbt);
    hipError_t e = hipErrorInvalidConfiguration;
    switch (K) {
        case 3: e = launch_bwd_lds_gated_k3(bf16, narrow, la, g, grid, s); break;
        case 5: e = launch_bwd_lds_gated_k5(bf16, narrow, la, g, grid, s); break;
        case 7: e = launch_bwd_lds_gated_k7(bf16, narrow, la, g, grid, s); break;
        case 9: e = launch_bwd_lds_gated_k9(bf16, narrow, la, g, grid, s); break;
    }
    if (e != hipSuccess) return (int)e;
    const long long n_out = (long long)(K + 1) * C;
    hipLaunchKernelGGL(dwconv_finalize_kernel<FIN_SPLIT>, dim3((unsigned)((n_out + 63) / 64)), dim3(64 * FIN_SPLIT), 0, s,
                       (const float*)part, lp.nbt, C, K, dw, db, out_bf16, tap_off);
    return (int)hipGetLastError();
}

const char* nplm_dwconv_strerror(int code) {
    if (code == 0) return "success";
    if (code > 0) return hipGetErrorString((hipError_t)code);
    switch (-code) {
        case NPLM_DWCONV_ENULL: return "nplm_dwconv: a required pointer is NULL";
        case NPLM_DWCONV_ESHAPE: return "nplm_dwconv: invalid sizes (need 0 <= T <= 2^31 - 2^20 - 1, C >= 1, S >= 0, C*K < 2^28)";
        case NPLM_DWCONV_EKSIZE: return "nplm_dwconv: kernel size must be odd and in [1, 255]";
        case NPLM_DWCONV_EDTYPE: return "nplm_dwconv: unknown element type (0 = fp32, 1 = bf16)";
        case NPLM_DWCONV_EALIGN: return "nplm_dwconv: pointer not aligned to its element size";
        case NPLM_DWCONV_EWORKSPACE: return "nplm_dwconv: workspace NULL, not 256-byte aligned, or too small";
        case NPLM_DWCONV_ECU: return "nplm_dwconv: cu_seqlens must start at 0, be non-decreasing and end at T";
        case NPLM_DWCONV_EFLAGS: return "nplm_dwconv: unknown bits set in flags";
        case NPLM_DWCONV_EUNSUPPORTED: return "nplm_dwconv: shape not supported by the fused (gated, LayerNorm) kernels";
        case NPLM_DWCONV_ESCRATCH: return "nplm_dwconv: the dw/db partial sums of this shape do not fit the library's static scratch (16 MiB); use nplm_dwconv_bwd_ex with a caller-owned workspace";
        case NPLM_DWCONV_ETUNING: return "nplm_dwconv: geometry override not available in this build";
    }
    return "nplm_dwconv: unknown error code";
}

int nplm_dwconv_fwd(const void* x, const int32_t* cu, const void* w, const void* b, void* y, int64_t T, int32_t C,
                    int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype, void* stream) {
    return fwd_impl(x, cu, w, b, y, T, C, K, S, act_dtype, w_dtype, 0, stream, nullptr);
}

int nplm_dwconv_fwd_ex(const void* x, const int32_t* cu, const void* w, const void* b, void* y, int64_t T, int32_t C,
                       int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream) {
    return fwd_impl(x, cu, w, b, y, T, C, K, S, act_dtype, w_dtype, flags, stream, nullptr);
}

int nplm_dwconv_fwd_tuned(const void* x, const int32_t* cu, const void* w, const void* b, void* y, int64_t T,
                          int32_t C, int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype, void* stream,
                          const nplm_dwconv_tuning* tune) {
    return fwd_impl(x, cu, w, b, y, T, C, K, S, act_dtype, w_dtype, tune ? tune->flags : 0u, stream, tune);
}

size_t nplm_dwconv_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype) {
    if (check_common(T, C, K, 0, act_dtype, NPLM_DWCONV_F32) || T == 0) return 0;
    K = exec_kernel_size(K);        // the slabs have the rows of the kernel size that runs
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    // enough for whichever kernel family the library picks for these sizes (the choice also depends
    // on pointer alignment, which is not known here)
    Plan p;
    if (make_plan(true, bf16, T, C, K, 0, nullptr, &p)) return 0;
    int slabs = p.nbt;
    if (choose_algo(true, nullptr, bf16, T, C, K, 0) == 2) {
        LdsPlan lp;
        if (make_lds_plan(true, bf16, T, C, K, nullptr, &lp) == 0 && lp.nbt > slabs) slabs = lp.nbt;
    }
    if (split_eligible(bf16, T, C, K, 0)) {
        LdsPlan lp;
        if (make_split_plan(false, bf16, T, C, K, nullptr, &lp) == 0 && lp.nbt > slabs) slabs = lp.nbt;
    }
    const size_t bytes = (size_t)slabs * (K + 1) * C * sizeof(float);
    return (bytes + 255) & ~(size_t)255;
}

int32_t nplm_dwconv_exec_kernel_size(int32_t K) { return exec_kernel_size(K); }

int32_t nplm_dwconv_bwd_slabs(int64_t T, int32_t C, int32_t K, int32_t act_dtype, const nplm_dwconv_tuning* tune) {
    if (check_common(T, C, K, 0, act_dtype, NPLM_DWCONV_F32) || T == 0) return 0;
    K = exec_kernel_size(K);
    const bool bf16 = act_dtype == NPLM_DWCONV_BF16;
    const int algo = choose_algo(true, tune, bf16, T, C, K, 0);
    if (algo < 0) return 0;
    if (algo == 3) {
        LdsPlan lp;
        if (make_split_plan(false, bf16, T, C, K, tune, &lp)) return 0;
        return lp.nbt;
    }
    if (algo == 2) {
        LdsPlan lp;
        if (make_lds_plan(true, bf16, T, C, K, tune, &lp)) return 0;
        return lp.nbt;
    }
    Plan p;
    if (make_plan(true, bf16, T, C, K, 0, tune, &p)) return 0;
    return p.nbt;
}

int nplm_dwconv_bwd(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx, float* dw, float* db,
                    void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K, int32_t S,
                    int32_t act_dtype, int32_t w_dtype, void* stream) {
    return bwd_impl(x, dy, cu, w, dx, dw, db, workspace, workspace_bytes, T, C, K, S, act_dtype, w_dtype, 0, stream,
                    nullptr);
}

int nplm_dwconv_bwd_ex(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx, float* dw, float* db,
                       void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream) {
    return bwd_impl(x, dy, cu, w, dx, dw, db, workspace, workspace_bytes, T, C, K, S, act_dtype, w_dtype, flags,
                    stream, nullptr);
}

int nplm_dwconv_bwd_static(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx, float* dw,
                           float* db, int64_t T, int32_t C, int32_t K, int32_t S, int32_t act_dtype, int32_t w_dtype,
                           uint32_t flags, void* stream) {
    const int rc = check_common(T, C, K, S, act_dtype, w_dtype);
    if (rc) return rc;
    void* ws = nullptr;
    size_t ws_bytes = 0;
    if (T > 0 && (dw || db)) {
        // the same number of slabs nplm_dwconv_bwd_ex would ask its caller for
        ws_bytes = nplm_dwconv_bwd_workspace_bytes(T, C, K, act_dtype);
        if (ws_bytes == 0 || ws_bytes > (size_t)NPLM_DWCONV_STATIC_SCRATCH_BYTES) return -NPLM_DWCONV_ESCRATCH;
        const hipError_t e = static_scratch_for_current_device(&ws);
        if (e != hipSuccess) return (int)e;
    }
    return bwd_impl(x, dy, cu, w, dx, dw, db, ws, ws_bytes, T, C, K, S, act_dtype, w_dtype, flags, stream, nullptr);
}

int nplm_dwconv_bwd_tuned(const void* x, const void* dy, const int32_t* cu, const void* w, void* dx, float* dw,
                          float* db, void* workspace, size_t workspace_bytes, int64_t T, int32_t C, int32_t K,
                          int32_t S, int32_t act_dtype, int32_t w_dtype, void* stream,
                          const nplm_dwconv_tuning* tune) {
    return bwd_impl(x, dy, cu, w, dx, dw, db, workspace, workspace_bytes, T, C, K, S, act_dtype, w_dtype,
                    tune ? tune->flags : 0u, stream, tune);
}

int nplm_dwconv_debug_copy(const void* src, void* dst, size_t bytes, void* stream) {
    if (!src || !dst) return -NPLM_DWCONV_ENULL;
    if (bytes % 16 || ((uintptr_t)src | (uintptr_t)dst) % 16) return -NPLM_DWCONV_EALIGN;
    if (bytes == 0) return 0;
    const size_t nvec = bytes / 16;
    hipLaunchKernelGGL(copy_chunks_kernel, dim3((unsigned)((nvec + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4*)src, (u32x4*)dst, nvec);
    return (int)hipGetLastError();
}

int64_t nplm_dwconv_debug_intervals(const int32_t* cu_host, int32_t S, int64_t T, int64_t start, int64_t step,
                                    int64_t relocate_every, int32_t* cs_out, int32_t* ce_out) {
    if (!cu_host || !cs_out || !ce_out || S < 0 || T < 0 || T > kMaxRows || start < 0 || step < 1) return -1;
    SeqCursor sc;
    sc.seq = 0; sc.cs = 0; sc.ce = 0;
    int64_t n = 0;
    for (int64_t t = start; t < T; t += step, ++n) {
        if (n == 0 || (relocate_every > 0 && n % relocate_every == 0))
            sc.locate(cu_host, S, (int)T, (int)t, sc.seq);
        else
            sc.advance(cu_host, S, (int)T, (int)t);
        cs_out[n] = sc.cs;
        ce_out[n] = sc.ce;
    }
    return n;
}

int nplm_dwconv_check_cu(const int32_t* cu, int32_t S, int64_t T, void* stream) {
    if (!cu) return -NPLM_DWCONV_ENULL;
    if (S < 0 || T < 0 || T > kMaxRows) return -NPLM_DWCONV_ESHAPE;
    std::vector<int32_t> h((size_t)S + 1);
    hipError_t e = hipMemcpyAsync(h.data(), cu, h.size() * sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return (int)e;
    if (h[0] != 0 || h[S] != (int32_t)T) return -NPLM_DWCONV_ECU;
    for (int32_t i = 0; i < S; ++i)
        if (h[i + 1] < h[i]) return -NPLM_DWCONV_ECU;
    return 0;
}

}  // extern "C"
