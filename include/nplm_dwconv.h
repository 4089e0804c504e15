/*
 * nplm_dwconv.h — C ABI of libnplm_dwconv.so: variable-length depthwise 1-D convolution over
 * packed sequences, forward and backward, for AMD MI355X (gfx950).
 *
 * The operator
 * ------------
 *   x, y, dy, dx : [T, C] row-major, contiguous (packed tokens x channels)
 *   w            : [C, K] row-major, K odd, P = (K-1)/2 (centred "same" padding)
 *   b            : [C] or NULL
 *   cu           : int32 [S+1], cu[0] = 0, non-decreasing, cu[S] = T. Sequence i owns rows
 *                  [cu[i], cu[i+1]). Zero-length sequences (cu[i] == cu[i+1]) are legal anywhere.
 *
 *   y [t,c] = b[c] + sum_k w[c,k] * x [t+k-P, c] * [s(t) <= t+k-P < e(t)]
 *   dx[t,c] =        sum_k w[c,k] * dy[t-k+P, c] * [s(t) <= t-k+P < e(t)]
 *   dw[c,k] = sum_t dy[t,c] * x[t+k-P, c] * [s(t) <= t+k-P < e(t)]
 *   db[c]   = sum_t dy[t,c]
 *   with [s(t), e(t)) the cu interval that contains row t. Taps never cross a sequence boundary
 *   (masked by selection, so a NaN/Inf in one sequence cannot reach another).
 *
 *   Kernel sizes: K = 3, 5, 7, 9, 15 and 31 have kernels of their own. Any other odd K <= 31 runs on the
 *   kernels of the next of 3, 15, 31 with zero taps on either side (w and dw keep rows of K taps; the
 *   workspace holds slabs of that size): for finite inputs the same sums with exact zeros added, so the
 *   same results; a NaN/Inf in x or dy then reaches the rows within that larger half-width of its own
 *   sequence (0 * Inf), never another sequence, and never a tap of dw that its products do not belong
 *   to. Odd K from 33 to NPLM_DWCONV_MAX_K run untuned kernels (one wave per row). The gated entry
 *   points take the same kernel sizes up to 31 the same way; the LayerNorm-fused ones K = 3, 5, 7, 9 only.
 *
 * Where this sits in the reference (peymanvahidi/nanoplm 0.1.6): the reference snapshot holds no
 * convolution; the ABI binds at the call site a conv module would occupy on the packed path,
 * src/nanoplm/pretraining/models/modern_bert/modeling.py:421-439 (encoder layer over x:[T,hidden]
 * with cu_seqlens), with the data contract of src/nanoplm/pretraining/collator.py:308-325
 * (cu_seqlens int32) and :405-458 (fixed-length cu_seqlens with trailing zero-length entries), and
 * the flat (total_tokens, hidden) layout of modeling.py:339,464. Each entry point below names the
 * autograd stage of that module it implements.
 *
 * Conventions
 * -----------
 *  - All pointers are DEVICE pointers owned by the caller. The library never allocates or frees
 *    device memory, keeps no pointer after return and has no mutable global state.
 *  - All work is enqueued asynchronously on `stream` (a hipStream_t passed as void*; NULL = the
 *    null stream). cu is read on the device: no host synchronisation.
 *  - Launch geometry depends only on (T, C, K, dtypes), never on timing: results are
 *    run-to-run bit-identical (no floating-point atomics anywhere).
 *  - Return value: 0 on success; < 0 an NPLM_DWCONV_E* argument error (nothing was launched);
 *    > 0 a hipError_t from a launch.
 *  - Preconditions NOT checked on the fast path (they would need a device read-back):
 *    cu[0] == 0, cu non-decreasing, cu[S] == T. Violations never cause out-of-bounds accesses
 *    (cu is only used to mask taps); rows outside [cu[0], cu[S]) are treated as one extra
 *    sequence on that side. nplm_dwconv_check_cu() verifies them with a read-back.
 */
#ifndef NPLM_DWCONV_H
#define NPLM_DWCONV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types for act_dtype / w_dtype */
#define NPLM_DWCONV_F32  0
#define NPLM_DWCONV_BF16 1

/* argument errors (returned negated: -NPLM_DWCONV_E...) */
#define NPLM_DWCONV_ENULL      1  /* a required pointer is NULL */
#define NPLM_DWCONV_ESHAPE     2  /* T < 0, T > 2^31 - 2^20 - 1, C < 1, S < 0, or C*K >= 2^28 */
#define NPLM_DWCONV_EKSIZE     3  /* K < 1, K even, or K > NPLM_DWCONV_MAX_K */
#define NPLM_DWCONV_EDTYPE     4  /* unknown act_dtype / w_dtype */
#define NPLM_DWCONV_EALIGN     5  /* activation pointer not aligned to its element size */
#define NPLM_DWCONV_EWORKSPACE 6  /* workspace NULL, misaligned (256 B) or smaller than required */
#define NPLM_DWCONV_ECU        7  /* check_cu: cu[0] != 0, cu decreasing, or cu[S] != T */
#define NPLM_DWCONV_EFLAGS     9  /* unknown bits set in `flags` (8 is used by the internal tuning interface) */
#define NPLM_DWCONV_EUNSUPPORTED 10 /* gated and LayerNorm entry points: shape outside what the fused kernels are built for */
#define NPLM_DWCONV_ESCRATCH   11 /* nplm_dwconv_bwd_static: the partial sums do not fit the static scratch */

/* flags of the _ex entry points */
#define NPLM_DWCONV_RESIDUAL 1u   /* fuse the residual connection: y = x + conv(x), dx = dy + conv^T(dy) */
#define NPLM_DWCONV_GRADS_BF16 2u /* backward entry points with a flags argument: the parameter gradients (dw, db, and
                                     dln_weight, dln_bias of nplm_dwconv_ln_bwd) point to bf16 buffers */

#define NPLM_DWCONV_MAX_K 255

/* Library version: major*10000 + minor*100 + patch. */
int nplm_dwconv_version(void);

/* Text for a return code of any entry point (argument errors and hipError_t values). */
const char* nplm_dwconv_strerror(int code);

/*
 * Forward: y = conv(x; w, b) per sequence.
 * Implements the module's forward at modeling.py:421-439 (x:[T,C] with cu_seqlens).
 * x, y: act_dtype; w, b: w_dtype (b may be NULL). bf16 activations are accumulated in fp32 and
 * rounded once (nearest-even) on store. T == 0 is a no-op.
 */
int nplm_dwconv_fwd(const void* x, const int32_t* cu, const void* w, const void* b, void* y,
                    int64_t T, int32_t C, int32_t K, int32_t S,
                    int32_t act_dtype, int32_t w_dtype, void* stream);

/*
 * Forward with flags. NPLM_DWCONV_RESIDUAL computes y = x + conv(x; w, b): the residual connection
 * around the module at its call site (x = x + conv(x, cu_seqlens) in the encoder layer,
 * modeling.py:421-439) without the extra pass over x and y an elementwise add would cost. The centre
 * tap is valid for every row, so the identity is folded into the centre weight in registers
 * (exact for bf16 weights; the sum is rounded once). flags == 0 is nplm_dwconv_fwd.
 */
int nplm_dwconv_fwd_ex(const void* x, const int32_t* cu, const void* w, const void* b, void* y,
                       int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * Bytes of device workspace nplm_dwconv_bwd needs for these sizes (fp32 partial sums of dw/db,
 * one slab per token-range block). Pure host arithmetic; 0 is returned for invalid sizes.
 */
size_t nplm_dwconv_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype);

/*
 * Backward: dx (act_dtype), dw [C,K] and db [C] (always fp32, fully overwritten) from x, dy.
 * Implements what autograd runs for the same module during loss.backward()
 * (src/nanoplm/pretraining/pure_pipeline.py:739-742). One fused pass reads x and dy once and
 * writes dx once; dw/db partials go to `workspace` (256-byte aligned, at least
 * nplm_dwconv_bwd_workspace_bytes() bytes, contents irrelevant on entry) and a second small
 * kernel sums them in a fixed order. dx, dw or db may each be NULL only if all of the outputs
 * it belongs with are skipped: dx == NULL skips dx; dw == NULL && db == NULL skips the
 * reductions (workspace may then be NULL). T == 0 zero-fills dw and db.
 */
int nplm_dwconv_bwd(const void* x, const void* dy, const int32_t* cu, const void* w,
                    void* dx, float* dw, float* db, void* workspace, size_t workspace_bytes,
                    int64_t T, int32_t C, int32_t K, int32_t S,
                    int32_t act_dtype, int32_t w_dtype, void* stream);

/*
 * Backward with flags. With NPLM_DWCONV_RESIDUAL, dx = dy + conv^T(dy; w) (the gradient of
 * x + conv(x) with respect to x); dw and db are those of the convolution and do not change.
 * With NPLM_DWCONV_GRADS_BF16, dw and db are bf16 buffers ([C,K] and [C], 2-byte aligned, passed
 * through the float* parameters): the sums are still formed in fp32 in the same fixed order and are
 * rounded once, nearest-even, as they are stored, which is what casting the fp32 results gives; it
 * saves a bf16 parameter's gradient the two cast kernels (autograd hands a parameter a gradient
 * of its own dtype: FSDP2 bf16 parameters, pure_pipeline.py:483-487). flags == 0 is nplm_dwconv_bwd.
 */
int nplm_dwconv_bwd_ex(const void* x, const void* dy, const int32_t* cu, const void* w,
                       void* dx, float* dw, float* db, void* workspace, size_t workspace_bytes,
                       int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * Backward for callers that cannot allocate: code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc, which therefore cannot produce the workspace nplm_dwconv_bwd_ex
 * asks for. No counterpart in the reference. Same arguments, kernels and results (bit for bit) as
 * nplm_dwconv_bwd_ex, minus the workspace: the dw/db partial sums go to a scratch array of
 * NPLM_DWCONV_STATIC_SCRATCH_BYTES that lives in the library's own device image, one copy per GPU,
 * held until the process ends. The call allocates and frees nothing. Its first use on a device looks
 * the array's address up (hipGetSymbolAddress) and keeps it, so make one call per device outside any
 * capture. Shapes whose partial sums need more than the array holds (C*(K'+1) above 4 Mi elements,
 * K' the kernel size that runs, see "Kernel sizes" above)
 * return -NPLM_DWCONV_ESCRATCH and launch nothing. Every call on a GPU shares that GPU's array: two
 * calls that overlap in time on one GPU (different streams, or threads) race on it and corrupt each
 * other's dw/db; calls on one stream, or otherwise ordered, are safe. Nothing in the array has to be
 * cleared between calls (every slab a call reads it has fully written first).
 */
#define NPLM_DWCONV_STATIC_SCRATCH_BYTES (16u << 20)
int nplm_dwconv_bwd_static(const void* x, const void* dy, const int32_t* cu, const void* w,
                           void* dx, float* dw, float* db,
                           int64_t T, int32_t C, int32_t K, int32_t S,
                           int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * Gated variants: the conv over h = x_proj * silu(gate) with the gate product fused into the conv's
 * loads, for a conv placed inside the SwiGLU MLP (ModernBertSwiGLUMLP.forward, modeling.py:300-302:
 * `x_proj, gate = self.Wi(x).chunk(2, dim=-1)`, then `F.silu(gate) * x_proj`).
 *   z, dz : [T, 2C] row-major, act_dtype; columns [0, C) are x_proj, columns [C, 2C) are gate
 *   y, dy : [T, C]
 *   y  = conv(h; w, b), h = z[:, :C] * silu(z[:, C:])           (h is formed in fp32, never stored)
 *   dz = [dh * silu(gate) | dh * x_proj * silu'(gate)], dh = conv^T(dy; w); dw, db as for conv(h)
 * This saves writing h and reading it back (forward) and the separate elementwise backward (backward).
 * Built for K in {3,5,7,9,15,31}, C * elemsize a multiple of 16 bytes and at least 1 KiB, 16-byte aligned
 * z / y / dy / dz; anything else returns -NPLM_DWCONV_EUNSUPPORTED and launches nothing (callers then
 * compose the unfused ops). `flags` as for nplm_dwconv_fwd_ex (the residual applies to h).
 * nplm_dwconv_gated_bwd_workspace_bytes returns 0 for unsupported shapes.
 */
int nplm_dwconv_gated_fwd(const void* z, const int32_t* cu, const void* w, const void* b, void* y,
                          int64_t T, int32_t C, int32_t K, int32_t S,
                          int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);
size_t nplm_dwconv_gated_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype);
int nplm_dwconv_gated_bwd(const void* z, const void* dy, const int32_t* cu, const void* w,
                          void* dz, float* dw, float* db, void* workspace, size_t workspace_bytes,
                          int64_t T, int32_t C, int32_t K, int32_t S,
                          int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * LayerNorm fused into the forward, for a conv that takes the place of a sub-module of the reference's pre-norm
 * encoder layer (ModernBertEncoderLayer.forward, modeling.py:404-438: `x + attn(attn_norm(x))`, the norm being a
 * torch.nn.LayerNorm over the hidden dimension, modeling.py:408-414):
 *   n = layer_norm(x; ln_weight, ln_bias, eps) over the C channels of a row (statistics and n in fp32, never stored)
 *   y = conv(n; w, b)            (+ x with NPLM_DWCONV_RESIDUAL: the identity is the raw x, not n)
 *   stats: [T][2] fp32, (mean, rstd) of every row - what nplm_dwconv_ln_bwd takes
 * x, y: act_dtype; ln_weight, ln_bias (may be NULL), w, b (may be NULL): w_dtype.
 * Built for K in {3,5,7,9}, rows in multiples of 16 bytes and 16-byte aligned x / y:
 *   rows of at most 2 KiB (C <= 1024 in bf16, 512 in fp32) and fp32 rows of at most 4 KiB (C <= 1024): one kernel
 *     whose blocks own whole rows and take the statistics from the tile they have staged; `stats` may be NULL;
 *   other rows of at most 8 KiB: a row-statistics kernel, then the conv kernel normalising as it reads; `stats` is
 *     required (it carries the statistics from the first kernel to the second; NULL returns -NPLM_DWCONV_ENULL).
 * Anything else returns -NPLM_DWCONV_EUNSUPPORTED and launches nothing (callers then run LayerNorm and
 * nplm_dwconv_fwd_ex).
 */
int nplm_dwconv_ln_fwd(const void* x, const int32_t* cu, const void* ln_weight, const void* ln_bias, float eps,
                       const void* w, const void* b, void* y, float* stats,
                       int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * Backward of nplm_dwconv_ln_fwd (same shapes, same -NPLM_DWCONV_EUNSUPPORTED rule; the reference would reach it
 * through autograd over torch.nn.LayerNorm, modeling.py:408-414).
 * From x, the row statistics the forward wrote and dy:
 *   dw, db                  the conv's parameter gradients over n = layer_norm(x) (n is recomputed, never stored)
 *   dln_weight, dln_bias    the LayerNorm's parameter gradients, fp32 [C] (dln_bias may be NULL)
 *   dx                      the LayerNorm's input gradient (+ dy with NPLM_DWCONV_RESIDUAL), act_dtype
 * Rows of at most 4 KiB: one kernel (the conv backward normalises x as it reads, its waves exchange the row sums of
 * the LayerNorm input gradient inside the block and write dx) and one small reduction of per-block partial sums.
 * Wider rows: the conv backward writes dn (the gradient of n, fp32) into the workspace and one more pass over
 * (x, dn, dy) rows forms dx. The workspace (nplm_dwconv_ln_bwd_workspace_bytes, 256-byte aligned; 0 for unsupported shapes) holds
 * the partial sums and, for the wider rows, dn (T x C x 4 bytes).
 */
size_t nplm_dwconv_ln_bwd_workspace_bytes(int64_t T, int32_t C, int32_t K, int32_t act_dtype);
int nplm_dwconv_ln_bwd(const void* x, const void* dy, const int32_t* cu, const float* stats,
                       const void* ln_weight, const void* ln_bias, const void* w,
                       void* dx, float* dw, float* db, float* dln_weight, float* dln_bias,
                       void* workspace, size_t workspace_bytes,
                       int64_t T, int32_t C, int32_t K, int32_t S,
                       int32_t act_dtype, int32_t w_dtype, uint32_t flags, void* stream);

/*
 * Debug helper: copies cu to the host (synchronises `stream`) and verifies the preconditions.
 * Returns 0, -NPLM_DWCONV_ECU, another argument error, or a hipError_t.
 */
int nplm_dwconv_check_cu(const int32_t* cu, int32_t S, int64_t T, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NPLM_DWCONV_H */
