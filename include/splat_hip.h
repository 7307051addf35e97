/*
 * splat_hip.h -- C ABI of libsplat_hip.so: SPLAT's ACSR sparse-attention forward path as
 * hand-written gfx950 (MI355X) HIP kernels.
 *
 * The reference (spikerheado1234/triton-fun, directory SPLAT/) has no FFI: its operator API is a
 * set of Python functions that launch Triton kernels.  Each entry point below replaces the device
 * work behind one of them and is what a ctypes / cffi stub in those Python functions binds:
 *
 *   splat_acsr_build      <- acsr_helpers.py:99-160   instantiate_metadata + create_acsr
 *   splat_mask_generate   <- acsr_helpers.py:18-55    create_*_mask (device-side equivalent)
 *   splat_acsr_build_pattern <- both of the above for the closed-form patterns, without the mask
 *   splat_sddmm           <- r_sddmm.py:15-115,171-184   rsddmm_kernel / rsddmm_launcher
 *   splat_softmax         <- r_softmax.py:16-59,126-150  r_softmax_1d_kernel / rsoftmax_launcher
 *   splat_spmm            <- r_spmm.py:13-126,148-164    r_spmm_kernel_row_maj_row_comp / rspmm_launcher
 *   splat_attention_fwd   <- r_attention.py:77-100    RegularAttention.forward (the three launches fused)
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless its comment says "host".
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only enqueue
 *     work; they never synchronise, never allocate or free device memory and never throw.
 *   - Return value: 0 on success; negative SPLAT_E_* for rejected arguments (nothing was
 *     launched); positive = the hipError_t reported by the launch.  splat_last_error() returns a
 *     thread-local, human readable description of the last non-zero return on this thread.
 *   - All metadata arrays are float32, exactly as acsr_helpers.py:148-156 stores them.
 *   - Compressed layout (r_sddmm.py:57-115, acsr_helpers.py:122-124): slot s of row r holds dense
 *     column c = sTod_lin[r] * (s + sTod_trans[r]); slots s >= nnz[r] are never written and never
 *     read.  A row's compressed slots may be the concatenation of several affine segments; segment
 *     k owns slots [slot_offset_k, slot_offset_k + nnz_k[r]).
 */
#ifndef SPLAT_HIP_H
#define SPLAT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPLAT_VERSION 900 /* major*10000 + minor*100 + patch; 0.2.0 added the planned forward, 0.3.0 splat_spmm_t, 0.4.0 splat_attention_fwd_stats, splat_sddmm_probs, 0.5.0 splat_attention_fwd_noalloc, 0.6.0 moved the two measurement aids out (libsplat_bench.so, splat_bench.h), 0.7.0 added splat_sddmm_planned, splat_spmm_planned, 0.8.0 splat_spmm_t_planned, 0.9.0 splat_attention_bwd_keys */

/* element types of q/k/v/score/output buffers */
#define SPLAT_F32 0
#define SPLAT_F16 1
#define SPLAT_BF16 2

/* negative return codes */
#define SPLAT_E_NULL (-1)        /* a required pointer is NULL */
#define SPLAT_E_SHAPE (-2)       /* a size is non-positive or out of the supported range */
#define SPLAT_E_DTYPE (-3)       /* unknown element type */
#define SPLAT_E_ALIGN (-4)       /* a pointer or stride is not aligned as the kernel requires */
#define SPLAT_E_UNSUPPORTED (-5) /* valid request that this build has no kernel for */

#define SPLAT_MAX_SEGMENTS 4

/* mask patterns for splat_mask_generate */
#define SPLAT_MASK_BLOCKED 0         /* acsr_helpers.py:18-34, p0 = p */
#define SPLAT_MASK_WINDOWED 1        /* acsr_helpers.py:36-44, p0 = p */
#define SPLAT_MASK_CAUSAL_WINDOWED 2 /* acsr_helpers.py:46-55, p0 = p */
#define SPLAT_MASK_DILATED 3         /* columns i - p0*p1/2 + p1*t, t in [0,p0): p0 = window, p1 = dilation */
#define SPLAT_MASK_STRIDED_LOCAL 4   /* columns (i-p0, i]: p0 = local width */
#define SPLAT_MASK_STRIDED_FAR 5     /* columns j <= i-p0 with j % p1 == p1-1: p0 = local width, p1 = stride */
#define SPLAT_MASK_TRANSPOSED 8      /* flag: the transpose of the pattern it is or-ed onto (row j keeps the rows of the pattern
                                        that keep column j); the backward pass needs the ACSR of the transposed mask */

/* One affine segment of an ACSR: the five per-row arrays create_acsr returns
 * (acsr_helpers.py:148-152) plus where the segment's slots start in a compressed row. */
typedef struct splat_acsr_seg {
    const float* dTos_lin;   /* [rows] dense->sparse linear term, 1/(b-a)            */
    const float* dTos_trans; /* [rows] dense->sparse translation, -a/(b-a)           */
    const float* sTod_lin;   /* [rows] sparse->dense linear term, b-a                */
    const float* sTod_trans; /* [rows] sparse->dense translation, a/(b-a)            */
    const float* nnz;        /* [rows] live slots of the row                          */
    const int32_t* first_col; /* [rows] optional (may be NULL): first live dense column of the
                                 row.  Used for rows with exactly one live column, whose stored
                                 translation acsr_helpers.py:126-130 hard-codes to 0.   */
    int32_t slot_offset;     /* first compressed slot of this segment (0 for one segment) */
    int32_t row_stride_hint; /* 0 or 1: none.  n > 1: every row's column step is n and its first column is
                                congruent to the row index modulo n (splat_acsr_build reports this in
                                summary[2..4]); kernels then group rows by phase.  Only affects speed. */
} splat_acsr_seg;

int splat_version(void);
const char* splat_last_error(void);

/* Build the ACSR of a rows x cols 0/1 byte mask (row pitch `ld` bytes).
 * Replaces instantiate_metadata/create_acsr, acsr_helpers.py:99-160; the float32 arrays are
 * bit-identical to what that code stores.
 *   dTos_lin..nnz      [rows]  float32 outputs
 *   span_start/end     [ceil(rows/block_height)] float32 outputs (acsr_helpers.py:135-140)
 *   row_first/row_last [rows]  int32 outputs, optional (NULL to skip): first / last nonzero
 *                      column (cols / -1 for an empty row); the tiling of r_sddmm.py:117-146 and
 *                      splat_acsr_seg.first_col are derived from them
 *   summary            [8] int32 output: [0] T = max row sum (acsr_helpers.py:153), [1] number of
 *                      rows that trip the reference's "Incorrect unpacking of affine-indices."
 *                      assertion (nnz > 1 but fewer than two entries equal to 1), [2] / [3] smallest / largest column
 *                      step over rows with nnz > 1 (INT32_MAX / 0 when there is none), [4] number of rows with
 *                      nnz > 1 whose first column is not congruent to the row index modulo the row's step,
 *                      [5..7] reserved.
 * Reads rows*ld bytes once; the caller reads `summary` back after synchronising the stream. */
int splat_acsr_build(const uint8_t* mask, int64_t rows, int64_t cols, int64_t ld,
                     int32_t block_height, float* dTos_lin, float* dTos_trans, float* sTod_lin,
                     float* sTod_trans, float* nnz, float* span_start, float* span_end,
                     int32_t* row_first, int32_t* row_last, int32_t* summary, void* stream);

/* Fill a rows x cols byte mask (row pitch ld) with one of the SPLAT_MASK_* patterns.
 * Device-side equivalent of the O(s^2) Python loops at acsr_helpers.py:18-55. */
int splat_mask_generate(uint8_t* mask, int64_t rows, int64_t cols, int64_t ld, int32_t pattern,
                        int64_t p0, int64_t p1, void* stream);

/* The ACSR of one of the closed-form s x s patterns above, without the mask: every row of such a pattern is an
 * arithmetic progression of columns, so what splat_acsr_build finds by scanning s*s bytes follows from
 * (pattern, p0, p1, row) directly.  Same outputs, bit for bit, as splat_mask_generate + splat_acsr_build
 * (instantiate_metadata / create_acsr, acsr_helpers.py:99-160, on create_*_mask, acsr_helpers.py:18-55), in
 * O(s) work and no s*s buffer: what makes L in the hundreds of thousands practical. */
int splat_acsr_build_pattern(int32_t pattern, int64_t s, int64_t p0, int64_t p1, int32_t block_height,
                             float* dTos_lin, float* dTos_trans, float* sTod_lin, float* sTod_trans,
                             float* nnz, float* span_start, float* span_end, int32_t* row_first,
                             int32_t* row_last, int32_t* summary, void* stream);

/* SDDMM: out[b,h,r,off+s] = scale * sum_k q[b,h,r,k] * kT[b,h,k,c(r,s)], s < nnz[r], per segment.
 * Replaces rsddmm_launcher / rsddmm_kernel, r_sddmm.py:15-115,171-184 (x = q, y = kT).
 *   q    element (b,h,r,k) at q   + b*q_sb + h*q_sh + r*q_sl + k            (unit stride in k)
 *   kT   element (b,h,k,c) at kT  + b*k_sb + h*k_sh + k*k_sd + c*k_sl       (k_sd==1 or k_sl==1)
 *   out  [B,H,L,T] contiguous, dtype `out_dtype`; q and kT have dtype `in_dtype`
 * Strides are in elements. */
int splat_sddmm(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out,
                const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t B, int32_t H,
                int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype,
                int32_t out_dtype, void* stream);

/* splat_sddmm whose stored value is exp(scale * score - lse[(b*H + h)*L + r]) instead of scale * score: the
 * row's softmax probabilities when lse is the row statistic of splat_attention_fwd_stats, written in one pass
 * (rsddmm_launcher followed by rsoftmax_launcher, r_attention.py:80-90, without the second pass over the
 * compressed matrix).  Used by the backward pass, which has the statistic from the forward. */
int splat_sddmm_probs(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                      int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out,
                      const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t B, int32_t H,
                      int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype,
                      int32_t out_dtype, const float* lse, void* stream);

/* splat_sddmm (lse == NULL) or splat_sddmm_probs (lse != NULL) with the mask's plan table: `plan` is what
 * splat_attention_plan wrote for the same segments and L (its per-block column ranges and per-row windows are those of
 * every tiled kernel here, not only the fused one).  The kernel for 16-bit types, d = 64 / 128 and launches of at least
 * 256 row blocks (or rows of at most 256 slots) then starts its copies after two scalar loads instead of deriving the plan from the ACSR arrays
 * (-7 % at B=2 H=32 L=8192 d=128 T=512, -18 % at B=4 H=16 L=4096 d=64 T=256); other shapes ignore the plan.  Same
 * results bit for bit.  A plan built from other metadata gives wrong scores but no access outside the buffers.
 * Replaces the same reference code as splat_sddmm (rsddmm_launcher, r_sddmm.py:153-188). */
int splat_sddmm_planned(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                        int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out,
                        const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t B, int32_t H,
                        int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype,
                        int32_t out_dtype, const float* lse /* may be NULL */, const void* plan,
                        int64_t plan_bytes, void* stream);

/* Row softmax over the live slots of compressed rows: y[bh,r,s] = exp(x[bh,r,s]-max_r)/sum_r.
 * Replaces rsoftmax_launcher / r_softmax_1d_kernel, r_softmax.py:16-59,126-150, applied to every
 * row.  x, y: [BH, L, T] contiguous; x may equal y (in place). */
int splat_softmax(const void* x, void* y, const splat_acsr_seg* segs /* host */, int32_t n_seg,
                  int64_t BH, int32_t L, int32_t T, int32_t in_dtype, int32_t out_dtype,
                  void* stream);

/* SpMM: out[b,h,r,:] = sum_{s<nnz[r]} p[b,h,r,off+s] * v[b,h,c(r,s),:], summed over segments.
 * Replaces rspmm_launcher / r_spmm_kernel_row_maj_row_comp, r_spmm.py:13-126,148-164.
 *   p    [B,H,L,T] contiguous compressed probabilities, dtype in_dtype
 *   v    element (b,h,c,n) at v + b*v_sb + h*v_sh + c*v_sl + n, dtype in_dtype
 *   out  [B,H,L,n_out] contiguous, dtype out_dtype */
int splat_spmm(const void* p, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out,
               const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t B, int32_t H,
               int32_t L, int32_t n_keys, int32_t n_out, int32_t T, int32_t in_dtype,
               int32_t out_dtype, void* stream);

/* splat_spmm with the mask's plan table (`plan` as in splat_sddmm_planned).  For 16-bit types and 64 or 128 output columns
 * this runs kernels of thin wavefronts (four per SIMD) that start from the table --
 * rows of at least 256 slots on 16-byte boundaries in compressed matrices of more than 192 MB through per-row rings of
 * aligned lines, everything else through a workgroup-wide tile: -20 % at B=2 H=32 L=8192 d=128 T=512, -23 % at B=4 H=16 L=4096 d=64 T=256, -40 % on rows
 * of 64 slots; masks of at least 256 slots per row whose rows all start on multiples of 8 positions of their block's walk
 * (blocked masks with large blocks) are better served by splat_spmm (the Python launcher looks that up in the table once
 * and picks).  Other shapes ignore the plan.  Same results as
 * splat_spmm up to the order of the float32 additions.  Replaces the same reference code (rspmm_launcher,
 * r_spmm.py:128-190). */
int splat_spmm_planned(const void* p, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out,
                       const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t B, int32_t H, int32_t L,
                       int32_t n_keys, int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype,
                       const void* plan, int64_t plan_bytes, void* stream);

/* Fused forward: out = softmax_over_live_columns(scale * q.kT) . v with online softmax; the
 * compressed score matrix is never written to memory.  Equals the composition
 * rsddmm_launcher -> rsoftmax_launcher -> rspmm_launcher of RegularAttention.forward
 * (r_attention.py:77-100).  d must be 64 or 128.  q, kT, v, out share `dtype`; layouts as in
 * splat_sddmm / splat_spmm, out element (b,h,r,n) at out + b*o_sb + h*o_sh + r*o_sl + n. */
int splat_attention_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                        int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                        int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb,
                        int64_t o_sh, int64_t o_sl, const splat_acsr_seg* segs /* host */,
                        int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d, float scale,
                        int32_t dtype, void* stream);

/* Plan of the fused forward for one mask: per 128-row block the key tiles it walks, per row its window in
 * tile positions.  splat_attention_fwd derives these from the ACSR arrays in every workgroup of every
 * launch; a module that attends with one mask many times (RegularAttention, r_attention.py:14-100, whose
 * constructor already holds every per-mask buffer) builds the plan once and calls
 * splat_attention_fwd_planned, whose workgroups start on their first tile after two small loads.
 * The reference has no counterpart (its kernels redo the affine index arithmetic per element).
 *
 * splat_attention_plan_bytes: size of the plan for these segments and L rows (0 for invalid arguments);
 *   host-only arithmetic, reads nothing on the device.
 * splat_attention_plan: fill `plan` (device memory, 16-byte aligned, plan_bytes >= the size above); the
 *   work is enqueued on `stream`, and forwards that use the plan must be ordered after it.
 * splat_attention_fwd_planned: as splat_attention_fwd, with the plan of the same segments and L; results
 *   are bit-identical to splat_attention_fwd.  A plan built from other segments or another L gives
 *   undefined results (only its size is checked). */
int64_t splat_attention_plan_bytes(const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t L);
int splat_attention_plan(const splat_acsr_seg* segs /* host */, int32_t n_seg, int32_t L, void* plan,
                         int64_t plan_bytes, void* stream);
int splat_attention_fwd_planned(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                                int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb,
                                int64_t o_sh, int64_t o_sl, const splat_acsr_seg* segs /* host */,
                                int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d, float scale,
                                int32_t dtype, const void* plan, int64_t plan_bytes, void* stream);

/* The fused forward that also hands out every row's softmax statistic: lse[(b*H + h)*L + r] = natural log of the
 * sum over the row's live columns of exp(scale * score), float32, so that the row's probabilities are
 * exp(scale * score - lse).  +inf for a row without live columns (its output row is zero).  That is what a
 * caller needs to merge partial results over disjoint key ranges (sequence shards) or to recompute the
 * probabilities in a backward pass without a second normalisation.  `plan` may be NULL (then as
 * splat_attention_fwd) or the plan of splat_attention_plan.  `out` is bit-identical to the other two
 * forwards'.  The reference has no counterpart: r_softmax.py:30-59 normalises in place and keeps neither the
 * row maximum nor the row sum. */
int splat_attention_fwd_stats(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                              int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                              int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb,
                              int64_t o_sh, int64_t o_sl, const splat_acsr_seg* segs /* host */,
                              int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d, float scale,
                              int32_t dtype, const void* plan, int64_t plan_bytes, float* lse,
                              void* stream);

/* The fused forward for callers that cannot allocate device memory or hold a plan buffer: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and
 * bit-identical results as splat_attention_fwd_planned, without the plan arguments: the plan is rebuilt by every call
 * into a buffer of SPLAT_STATIC_PLAN_BYTES that is part of the library's device image (each GPU the library runs on
 * holds one until the process ends), then the forward runs from it on the same stream.  The call allocates and frees
 * nothing.  Masks whose plan is larger (splat_attention_plan_bytes; 4256 bytes per 128-row block and segment) are
 * rejected with SPLAT_E_SHAPE.  All calls on one GPU share that one buffer: two calls whose work may overlap on a
 * GPU (different streams, different threads) race; order them.  The first call on a GPU for a given element type, head
 * size and K layout also looks up the buffer's address and raises its kernel's LDS limit, which are not stream
 * operations: make that call outside any stream capture (one eager warm-up call per configuration is enough; every
 * later call only enqueues two kernels and can be captured, and a replay rebuilds the plan it runs from). */
#define SPLAT_STATIC_PLAN_BYTES (4 << 20)
int splat_attention_fwd_noalloc(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                                int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb,
                                int64_t o_sh, int64_t o_sl, const splat_acsr_seg* segs /* host */,
                                int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d, float scale,
                                int32_t dtype, void* stream);

/* K^T [B, H, d, L] with unit stride along the keys (the layout the reference documents for `y`, r_sddmm.py:230-231) to
 * K [B, H, L, d] contiguous.  No counterpart in the reference, whose kernels only read the former: the kernels here read
 * that layout in dense runs of keys, so for rows that step over columns (dilated windows, strided far fields) the
 * Python launchers transpose K once per call with this and pass the result as a [B, H, d, L] view (unit stride along d).
 * kT_sb / kT_sh / kT_sd: element strides of batch, head and the d index (kT_sd >= L); k_rows 16-byte aligned. */
int splat_transpose_keys(const void* kT, int64_t kT_sb, int64_t kT_sh, int64_t kT_sd, void* k_rows, int32_t B,
                         int32_t H, int32_t L, int32_t d, int32_t dtype, void* stream);

/* ---- backward pass (the reference has none: r_attention.py:77-100 is forward only) ----
 * With S~ the compressed scores, P~ = softmax(S~), O = P~ . V:
 *   dP~ = splat_sddmm(x = dO, y = V viewed as [d, L])           dQ = splat_spmm(p = dS~, v = K)
 *   dS~ = splat_softmax_bwd(P~, dP~)                              dV = splat_spmm_t(P~, dO)
 *                                                                 dK = splat_spmm_t(dS~, Q)
 * The transposed products also need the ACSR of the transposed mask (splat_acsr_build on mask^T, whose rows are
 * affine for every pattern above): it says which rows a column meets.  splat_compressed_transpose stores a
 * compressed matrix in that ACSR's layout, after which splat_spmm with that ACSR gives the same products.
 *
 * splat_spmm_t: out[b, h, j, :] = sum over the rows i that keep column j of p[b, h, i, slot of j in row i] * x[b, h, i, :];
 *   p [B*H, L, T] compressed (layout of `segs`), x [B, H, L, n_out] by strides with unit stride along the last
 *   dimension, out [B*H, Lt, n_out] contiguous; segment k of `segs_t` must be the ACSR of the transpose of segment k
 *   of `segs` (Lt rows).  fp32 accumulation.
 * splat_softmax_bwd: ds[r, s] = p[r, s] * (dp[r, s] - sum_s' p[r, s'] dp[r, s']) * scale over the live slots of
 *   each row; [BH, L, T] contiguous, one dtype; ds may alias dp; dead slots are not touched.
 * splat_compressed_transpose: dst[bh, j, t] = src[bh, i(j, t), s(i, j)]: segment k of `segs_t` must be the ACSR of
 *   the transpose of segment k of `segs`; src [BH, L, T], dst [BH, Lt, Tt] contiguous, distinct, one dtype. */
int splat_softmax_bwd(const void* p, const void* dp, void* ds, const splat_acsr_seg* segs /* host */,
                      int32_t n_seg, int64_t BH, int32_t L, int32_t T, float scale, int32_t dtype,
                      void* stream);
int splat_spmm_t(const void* p, const void* x, int64_t x_sb, int64_t x_sh, int64_t x_sl, void* out,
                 const splat_acsr_seg* segs /* host */, const splat_acsr_seg* segs_t /* host */, int32_t n_seg,
                 int32_t B, int32_t H, int32_t L, int32_t Lt, int32_t n_out, int32_t T, int32_t in_dtype,
                 int32_t out_dtype, void* stream);
/* splat_spmm_t with the plan table of the TRANSPOSED mask (splat_attention_plan on `segs_t` with Lt rows; plan_bytes >=
 * splat_attention_plan_bytes(segs_t, n_seg, Lt), 16-byte aligned, device memory).  For 16-bit types of one kind for p, x
 * and out, n_out = 64 or 128, 16-byte aligned x rows, every segment with a first_col array and T >= 8
 * this runs a kernel of thin wavefronts (four per SIMD) that
 * starts from the table and keeps the tile loop's loads independent of one another: -31 % at B=2 H=32 L=8192 n_out=128
 * T=512 (dilated), -28 % at B=4 H=16 L=4096 n_out=64 T=256, -33 % on blocks of 512.  It is built for rows whose column
 * step equals the stride by which the transposed mask's rows are grouped (1 for windows and blocks, the dilation for
 * dilated windows); rows of another step are walked a second time entry by entry, which the general kernel does better
 * (the Python launcher picks by the metadata's largest step).  Other shapes ignore the plan.  Same results as
 * splat_spmm_t.  No counterpart in the reference (it has no backward pass). */
int splat_spmm_t_planned(const void* p, const void* x, int64_t x_sb, int64_t x_sh, int64_t x_sl, void* out,
                         const splat_acsr_seg* segs /* host */, const splat_acsr_seg* segs_t /* host */, int32_t n_seg,
                         int32_t B, int32_t H, int32_t L, int32_t Lt, int32_t n_out, int32_t T, int32_t in_dtype,
                         int32_t out_dtype, const void* plan_t, int64_t plan_bytes, void* stream);
int splat_compressed_transpose(const void* src, void* dst, const splat_acsr_seg* segs /* host */,
                               const splat_acsr_seg* segs_t /* host */, int32_t n_seg, int64_t BH,
                               int32_t L, int32_t T, int32_t Lt, int32_t Tt, int32_t dtype, void* stream);

/* The same backward pass in three launches of one kernel (two at d = 64) and without any compressed matrix in memory (no counterpart in
 * the reference, which is forward only: r_attention.py:77-100).  q, k, v, out (the forward's output) and dout (the
 * upstream gradient) are [B, H, L, d] views with unit stride along d (k is K itself, rows contiguous, not K^T);
 * lse [B, H, L] is the row statistic of splat_attention_fwd_stats for the same inputs; delta [B, H, L] float32 is
 * workspace (it receives rowsum(dout * out)); dq, dk, dv are contiguous [B, H, L, d].  segs / plan: the mask's ACSR and
 * its splat_attention_plan; segs_t / plan_t: the same for the transposed mask (keys as rows).  16-bit dtypes, d = 64 or
 * 128, scale > 0.  With P = exp(scale * q.k - lse) on the live columns:  dS = P * (dout.v - delta),
 * dq = scale * dS k,  dk = scale * dS^T q,  dv = P^T dout. */
int splat_attention_bwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* k, int64_t k_sb,
                        int64_t k_sh, int64_t k_sl, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl,
                        const void* out, int64_t o_sb, int64_t o_sh, int64_t o_sl, const void* dout, int64_t g_sb,
                        int64_t g_sh, int64_t g_sl, const float* lse, float* delta, void* dq, void* dk, void* dv,
                        const splat_acsr_seg* segs /* host */, int32_t n_seg, const void* plan, int64_t plan_bytes,
                        const splat_acsr_seg* segs_t /* host */, int32_t n_seg_t, const void* plan_t,
                        int64_t plan_t_bytes, int32_t B, int32_t H, int32_t L, int32_t d, float scale, int32_t dtype,
                        void* stream);

/* The keys' side of that pass for a list of rows of the transposed mask (no counterpart in the reference, which is forward
 * only: r_attention.py:77-100).  For transposed masks that keep a few keys with very long columns (a strided pattern's far
 * field: one key in 128 with up to L queries), whose walk by 128 consecutive keys runs almost empty tiles: the caller
 * leaves such a segment out of splat_attention_bwd's segs_t and lists its live rows here, cut into stretches of queries so
 * that many workgroups share the walk.  Row r of segs_t (n_rows rows, each an arithmetic progression of queries below L)
 * belongs to key key_of_row[r] (device int32 [n_rows]; values in [0, L), or negative for an empty padding row); dk_rows /
 * dv_rows (contiguous [B, H, n_rows, d], overwritten) receive every row's share of dk / dv.  With dk and dv given (contiguous
 * [B, H, L, d], as splat_attention_bwd wrote them for the other segments; both or neither), a second kernel adds the shares
 * onto them: rows k, k + rows_per_stretch, k + 2 rows_per_stretch, ... must then name the same key (one row per stretch,
 * the keys in the same order in every stretch, n_rows a multiple of rows_per_stretch) and the keys of one stretch must be
 * distinct; the shares are summed in fp32 together with the value already there and rounded once.  q, k, v, dout, lse as
 * for splat_attention_bwd; delta as splat_attention_bwd wrote it for the same inputs (earlier on the same stream); plan_t
 * is splat_attention_plan(segs_t, n_seg_t, n_rows). */
int splat_attention_bwd_keys(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* k, int64_t k_sb,
                             int64_t k_sh, int64_t k_sl, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl,
                             const void* dout, int64_t g_sb, int64_t g_sh, int64_t g_sl, const float* lse,
                             const float* delta, const int32_t* key_of_row, void* dk_rows, void* dv_rows,
                             const splat_acsr_seg* segs_t /* host */, int32_t n_seg_t, const void* plan_t,
                             int64_t plan_t_bytes, int32_t B, int32_t H, int32_t L, int32_t n_rows, int32_t d, float scale,
                             int32_t dtype, void* dk, void* dv, int32_t rows_per_stretch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPLAT_HIP_H */
