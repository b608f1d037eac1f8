/* corope_amd.h -- C ABI of the MI355X (gfx950) fused RoPE-attention library.
 *
 * The reference repository (Superposition09m/Co-RoPE) has no C or FFI boundary: its hot path
 * sits behind two torch.autograd.Function classes that launch Triton kernels.  This library
 * is the device side of the same two operators; the Python layer in co-rope_amd/ keeps the
 * reference's call surface and reaches these entry points through ctypes.
 *
 * Conventions (all entry points)
 *   - tensors are device pointers to contiguous row-major (B, H, N, D) bf16 storage;
 *     D is 64 or 128 (fused RoPE attention: also 256);
 *     pointers are 16-byte aligned;
 *   - freqs_cos / freqs_sin are fp32 tables with one row per position; only columns
 *     [0, D/2) are read; `freq_row_stride` is the distance between rows in elements
 *     (D for the reference's duplicated-half (N, D) table);
 *   - `lse` is the forward's per-row statistic M = log2(sum_j exp2(s_ij * sm_scale * log2 e)),
 *     shape (B, H, N) fp32 -- the same base-2 quantity the reference saves
 *     (fused-rope/fused_rope_attn.py:316-319);
 *   - the caller owns every buffer; the library never allocates or frees device memory and
 *     never synchronises; kernels are enqueued on `stream` (a hipStream_t, NULL = default);
 *   - every argument is validated before the first HIP call; return 0 on success or a
 *     negative COROPE_E_* code, with a message available from corope_amd_last_error().
 */
#ifndef COROPE_AMD_H
#define COROPE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define COROPE_OK 0
#define COROPE_E_BADARG (-1)      /* null pointer, non-positive size, bad scale */
#define COROPE_E_UNSUPPORTED (-2) /* head dim / group size / sequence length outside the built kernels */
#define COROPE_E_ALIGN (-3)       /* pointer not 16-byte aligned */
#define COROPE_E_LAUNCH (-4)      /* HIP reported an error at launch */

/* ABI version of this header (bumped on any signature change). */
int corope_amd_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char *corope_amd_last_error(void);

/* No entry point changes how later calls run: kernel forms (rows per workgroup item, rows per wave) are picked per call
 * from the shape, as the reference picks its tile sizes per shape (fused-rope/fused_rope_attn.py:163-183).  For diagnostics
 * the environment variables COROPE_AMD_TILE_ROWS (128 | 256) and COROPE_AMD_FWD_WAVE_ROWS (32 | 64 | 128), read once when the
 * library is loaded, override the pick for the whole process; results do not depend on them beyond rounding. */

/* Argument check only (no HIP call): what corope_rope_attn_fwd/bwd would return for these sizes. */
int corope_rope_attn_check(int B, int H, int N, int D, int64_t freq_row_stride, float sm_scale, int backward);

/* Argument check only (no HIP call) for corope_gqa_fwd. */
int corope_gqa_check(int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta);

/* cos/sin tables on the device: row r holds position pos0 + r, column i the angle (pos0 + r) * theta^(-2i/D);
 * width = D writes the reference's duplicated-half (n_pos, D) layout, width = D/2 the compact one.
 * Replaces precompute_freqs_cis (reference fused-rope/rope_attn_pytorch.py:10-49), which the reference runs as
 * torch ops on the device; pos0 > 0 gives a shard or a decode step its own slice of positions. */
int corope_rope_freqs(float *freqs_cos, float *freqs_sin, int n_pos, int D, int width, int64_t freq_row_stride,
                      int pos0, float theta, void *stream);

/* Fused RoPE flash-attention forward.
 * Replaces the launch of _attn_fwd in _attention.forward
 * (reference fused-rope/fused_rope_attn.py:222-320 kernel, :702-716 launch).
 * Writes o (B,H,N,D) bf16 and lse (B,H,N) fp32. */
int corope_rope_attn_fwd(const void *q, const void *k, const void *v,
                         const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                         void *o, float *lse,
                         int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Two-launch forward for long sequences: rotates K once into `workspace` (with the largest key norm of every
 * 64-key tile), then runs the attention kernel on the rotated copy, whose inner loop reads no cos/sin tables and
 * takes no data-dependent branch on tiles the norms prove harmless.  Same results as corope_rope_attn_fwd
 * (the rotated K is rounded to bf16 exactly as the single-launch kernel rounds it).  The reference rotates K
 * inside every program instead (fused-rope/fused_rope_attn.py:82-99); same launch site as above (:702-716).
 * workspace: device memory, 16-byte aligned, at least corope_rope_attn_fwd_workspace_bytes(B,H,N,D) bytes; it is
 * scratch, nothing in it has to survive the call. */
int64_t corope_rope_attn_fwd_workspace_bytes(int B, int H, int N, int D); /* -1 for unsupported sizes */
int corope_rope_attn_fwd_ws(const void *q, const void *k, const void *v,
                            const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                            void *o, float *lse,
                            int B, int H, int N, int D, float sm_scale, int causal,
                            void *workspace, int64_t workspace_bytes, void *stream);

/* The two-launch forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose forward allocates its outputs and
 * lets Triton allocate the rest.  Same kernels and same results, bit for bit, as corope_rope_attn_fwd_ws; the rotated
 * K and the per-tile key norms live in a buffer built into the library (one copy per GPU, held until the process ends,
 * corope_rope_attn_fwd_noalloc_max_bytes() = 65 MiB of it), so the call itself allocates and frees nothing.  Sizes whose
 * scratch (corope_rope_attn_fwd_workspace_bytes) exceeds that limit are refused with COROPE_E_UNSUPPORTED: the metric
 * shape B2 H32 N4096 D128 fits, B*H*N*D may reach about 34 million elements.  Nothing in the buffer has to start at zero
 * (the rotation pass writes every byte the attention kernel reads).  All calls on one GPU share that GPU's buffer:
 * calls that overlap in time on one GPU (different streams, or a captured graph replayed beside another call) race;
 * calls on one stream, or otherwise ordered, are safe. */
int64_t corope_rope_attn_fwd_noalloc_max_bytes(void);
int corope_rope_attn_fwd_noalloc(const void *q, const void *k, const void *v,
                                 const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                 void *o, float *lse,
                                 int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* y = scale * (half-layout rotation of x), x (B,H,N,D) bf16, fp32 arithmetic, rounded to bf16 once; tile_max (may be
 * NULL) receives [B*H][ceil(N/64)] floats, the largest norm of a row of y in every 64-row tile.  scale = 1 is
 * apply_rotary_emb (reference fused-rope/rope_attn_pytorch.py:71-84, rotate_half :52-68).  The "rotated" operands of the
 * *_prerotated entry points are: k_rot = this with scale 1, q_rot = this with scale = sm_scale * log2(e) -- the query side
 * carries the softmax temperature, so the scores leave the matrix cores in base-2 units (the reference folds the same
 * factor into k on the host for its backward, fused-rope/fused_rope_attn.py:746-748). */
int corope_rope_rotate(const void *x, const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                       void *y, float *tile_max, int B, int H, int N, int D, float scale, void *stream);

/* Attention on a K that corope_rope_rotate already rotated (k_rot, with its tile_max as tile_kmax): the second
 * launch of corope_rope_attn_fwd_ws on its own, for callers that keep the rotated K (a key cache) or time the two
 * launches separately.  q is still rotated inside the kernel; q_rot_out (may be NULL) receives the rotated q times
 * sm_scale * log2(e), the form the *_bwd_*_prerotated entry points take.
 * Same reference site as corope_rope_attn_fwd. */
int corope_rope_attn_fwd_prerotated(const void *q, const void *k_rot, const float *tile_kmax, const void *v,
                                    const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                    void *o, float *lse, void *q_rot_out,
                                    int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Forward for training: like corope_rope_attn_fwd_ws, but the rotated operands are outputs the caller keeps --
 * q_rot and k_rot, (B,H,N,D) bf16 -- so that the backward (corope_rope_attn_bwd_prerotated) needs no rotation pass and
 * the original q and k need not be saved (the reference saves q and k and re-rotates them in every inner iteration of
 * its backward, fused-rope/fused_rope_attn.py:718, :367-380).  tile_kmax: scratch, B*H*ceil(N/64) floats.
 * Same launch site as corope_rope_attn_fwd. */
int corope_rope_attn_fwd_train(const void *q, const void *k, const void *v,
                               const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                               void *o, float *lse, void *q_rot, void *k_rot, float *tile_kmax,
                               int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* delta[b,h,i] = sum_d o[b,h,i,d] * do[b,h,i,d]  (fp32).
 * Replaces _attn_bwd_preprocess (reference fused-rope/fused_rope_attn.py:324-337, launch :753-758). */
int corope_rope_attn_bwd_preprocess(const void *o, const void *d_o, float *delta,
                                    int B, int H, int N, int D, void *stream);

/* dV alone: one workgroup per key block, sweeping the query blocks that attend to it; recomputes P from q, k and lse.
 * Replaces the dV part of _attn_bwd_dkdv (reference fused-rope/fused_rope_attn.py:382-393, :571-572). */
int corope_rope_attn_bwd_dv(const void *q, const void *k, const void *d_o, const float *lse,
                            const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                            void *dv,
                            int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* dK alone: same sweep; recomputes P and dP, forms dS, un-rotates and scales dK in the epilogue.
 * Replaces the dK part of _attn_bwd_dkdv (reference fused-rope/fused_rope_attn.py:395-401, :573-579). */
int corope_rope_attn_bwd_dk(const void *q, const void *k, const void *v, const void *d_o,
                            const float *lse, const float *delta,
                            const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                            void *dk,
                            int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* dK and dV: corope_rope_attn_bwd_dv followed by corope_rope_attn_bwd_dk on the same stream (head dim 64: one
 * launch that computes both).
 * Replaces the _attn_bwd_dkdv half of _attn_bwd (reference fused-rope/fused_rope_attn.py:342-404,
 * :524-579) including the host-side K pre-scale (:746-748), which is folded into the kernels. */
int corope_rope_attn_bwd_dkdv(const void *q, const void *k, const void *v, const void *d_o,
                              const float *lse, const float *delta,
                              const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                              void *dk, void *dv,
                              int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* dQ: one workgroup per query block, sweeping the key blocks it attends to.
 * Replaces the _attn_bwd_dq half of _attn_bwd (reference fused-rope/fused_rope_attn.py:409-470, :592-649). */
int corope_rope_attn_bwd_dq(const void *q, const void *k, const void *v, const void *d_o,
                            const float *lse, const float *delta,
                            const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                            void *dq,
                            int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Whole backward = preprocess + dkdv + dq on one stream (what _attention.backward launches,
 * reference fused-rope/fused_rope_attn.py:725-777).  `delta` is caller-provided (B,H,N) fp32 scratch. */
int corope_rope_attn_bwd(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                         const float *lse, float *delta,
                         const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                         void *dq, void *dk, void *dv,
                         int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Backward on pre-rotated operands: q_rot and k_rot are copies of q and k that corope_rope_rotate rotated; the
 * kernels then read no cos/sin tables in their inner loops (the tables are still needed once per output row, to
 * rotate dK and dQ back).  Same results as the plain entry points (the rotated copies are rounded to bf16 exactly
 * as the kernels round them when they rotate a tile themselves).  Reference sites as for corope_rope_attn_bwd_dv,
 * _dk and _dq.  The dQ entry point takes o as well: NULL = delta is read (from the preprocess pass); non-NULL = delta is
 * computed from o and d_o for the rows each workgroup owns and WRITTEN to `delta`, which replaces the preprocess pass
 * (reference :324-337) when this launch comes before the dK launch. */
int corope_rope_attn_bwd_dv_prerotated(const void *q_rot, const void *k_rot, const void *d_o, const float *lse,
                                       const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                       void *dv,
                                       int B, int H, int N, int D, float sm_scale, int causal, void *stream);
int corope_rope_attn_bwd_dk_prerotated(const void *q_rot, const void *k_rot, const void *v, const void *d_o,
                                       const float *lse, const float *delta,
                                       const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                       void *dk,
                                       int B, int H, int N, int D, float sm_scale, int causal, void *stream);
/* dK and dV in one launch (S is recomputed once for both; the workgroup's V rows sit in LDS to make room for the two
 * sets of accumulators): the fused form of the two entry points above, same results bit for bit.  Replaces
 * _attn_bwd_dkdv (reference fused-rope/fused_rope_attn.py:342-404). */
int corope_rope_attn_bwd_dkdv_prerotated(const void *q_rot, const void *k_rot, const void *v, const void *d_o,
                                         const float *lse, const float *delta,
                                         const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                         void *dk, void *dv,
                                         int B, int H, int N, int D, float sm_scale, int causal, void *stream);
int corope_rope_attn_bwd_dq_prerotated(const void *q_rot, const void *k_rot, const void *v, const void *o,
                                       const void *d_o, const float *lse, float *delta,
                                       const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                       void *dq,
                                       int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Whole backward on rotated operands kept from corope_rope_attn_fwd_train (or made by corope_rope_rotate): preprocess,
 * dV, dK, dQ.  Replaces _attention.backward like corope_rope_attn_bwd (reference fused-rope/fused_rope_attn.py:720-777). */
int corope_rope_attn_bwd_prerotated(const void *q_rot, const void *k_rot, const void *v, const void *o, const void *d_o,
                                    const float *lse, float *delta,
                                    const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                    void *dq, void *dk, void *dv,
                                    int B, int H, int N, int D, float sm_scale, int causal, void *stream);

/* Whole backward for long sequences: rotates q and k once into `workspace`, then preprocess, dV, dK, dQ on the
 * rotated copies.  Replaces _attention.backward like corope_rope_attn_bwd (reference
 * fused-rope/fused_rope_attn.py:720-777).  workspace: device memory, 16-byte aligned, at least
 * corope_rope_attn_bwd_workspace_bytes(B,H,N,D) bytes, scratch. */
int64_t corope_rope_attn_bwd_workspace_bytes(int B, int H, int N, int D); /* -1 for unsupported sizes */
int corope_rope_attn_bwd_ws(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                            const float *lse, float *delta,
                            const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                            void *dq, void *dk, void *dv,
                            int B, int H, int N, int D, float sm_scale, int causal,
                            void *workspace, int64_t workspace_bytes, void *stream);

/* The operator on fp16 tensors -- the only dtype of the reference's kernels (fused-rope/fused_rope_attn.py:236,
 * verification.py:14): q, k, v, o, d_o, dq, dk, dv are fp16, the score products take fp16 operands, everything else
 * (tables, lse, delta, accumulation) is fp32 as above.  Same kernel sources as the bf16 entry points built for the other
 * element type.
 * Forward: k_rot == NULL: corope_rope_attn_fwd's single launch, with a true running maximum per 32-key half whenever a
 * probability would leave fp16's range.  k_rot != NULL ((B,Hkv,N,D) fp16 scratch, with tile_kmax (B,Hkv,ceil(N/64)) fp32):
 * the two-launch form as in corope_rope_attn_fwd_train / _gqa -- K rotated once into k_rot, then the pipelined attention
 * kernel, in which the unnormalised probabilities (up to 2^64: more binary orders than fp16 has) are bf16 and V is
 * converted to bf16 on its way into LDS, so that P V is a bf16 product; q_rot ((B,H,N,D) fp16, may be NULL) receives the
 * rotated Q times sm_scale*log2(e), and (q_rot, k_rot) are then the operands of a backward with prerotated = 1.
 * k_rot != NULL with tile_kmax == NULL: K is rotated once into k_rot and the single-launch kernel runs on the copy, without
 * the rotation in its loop and with its own bookkeeping -- P and V stay fp16, as in the reference -- and q_rot as above.
 * Backward: prerotated = 1: q, k are those rotated copies (dQ kernel, which computes delta on its way, then the fused dK+dV
 * kernel); else preprocess + dV + dK + dQ as in corope_rope_attn_bwd, or -- given a workspace of
 * corope_rope_attn_bwd_workspace_bytes (may be NULL) -- the rotation of q and k into it followed by the dQ and the fused
 * dK+dV kernel as in corope_rope_attn_bwd_ws, the faster form from N * D = 65536 on.  `delta` is (B,H,N) fp32 scratch.
 * k, v, dk, dv have Hkv heads (H a multiple of Hkv; Hkv = H: the reference's form), as in the grouped-query entry points below.
 * Replaces _attention.forward / .backward (fused-rope/fused_rope_attn.py:655-777) for callers that keep the reference's dtype. */
int corope_rope_attn_fwd_f16(const void *q, const void *k, const void *v,
                             const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                             void *o, float *lse, void *q_rot, void *k_rot, float *tile_kmax,
                             int B, int H, int Hkv, int N, int D, float sm_scale, int causal, void *stream);
int corope_rope_attn_bwd_f16(const void *q, const void *k, int prerotated, const void *v, const void *o, const void *d_o,
                             const float *lse, float *delta,
                             const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                             void *dq, void *dk, void *dv,
                             int B, int H, int Hkv, int N, int D, float sm_scale, int causal,
                             void *workspace, int64_t workspace_bytes, void *stream);

/* The forward on q, k, v that are strided views: `*_strides` = elements between batches, heads and rows of the
 * (B, H or Hkv, N, D) tensor (the last dimension contiguous; every stride a multiple of 8 elements, rows at least D apart) --
 * e.g. (N*H*D, D, H*D) for a (B, N, H, D) tensor viewed as (B, H, N, D).  The reference's forward kernel takes the strides
 * of q and k the same way (fused-rope/fused_rope_attn.py:709-710; its V and O go through contiguous descriptors, :245-251);
 * o, lse and the optional scratch are contiguous.  k_rot == NULL: single launch; k_rot != NULL: the two-launch form as
 * in corope_rope_attn_fwd_gqa (q_rot may be NULL; tile_kmax == NULL: the single-launch kernel on the rotated copy, as in
 * corope_rope_attn_fwd_f16); fp16 != 0: fp16 tensors as in corope_rope_attn_fwd_f16, else bf16. */
int corope_rope_attn_fwd_strided(const void *q, const int64_t *q_strides, const void *k, const int64_t *k_strides,
                                 const void *v, const int64_t *v_strides,
                                 const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                                 void *o, float *lse, void *q_rot, void *k_rot, float *tile_kmax,
                                 int B, int H, int Hkv, int N, int D, float sm_scale, int causal, int fp16, void *stream);

/* Grouped-query form of the operator: q (B,Hq,N,D), k and v (B,Hkv,N,D), Hq a multiple of Hkv; query head h reads
 * key/value head h / (Hq/Hkv); dk and dv (B,Hkv,N,D) are sums over the query heads of their group (the key block's
 * workgroup sweeps all of them, no atomics).  The reference's RoPE operator requires Hq == Hkv
 * (fused-rope/fused_rope_attn.py:657-661); the indexing follows its plain attention tutorial and the group
 * reduction its archived GQA experiment (assets/flashattn-gqa/triton_gqa.py:605-666).
 * forward: k_rot NULL = single launch (q_rot and tile_kmax must be NULL too); otherwise K is rotated into k_rot
 * (B,Hkv,N,D) with tile_kmax (B*Hkv*ceil(N/64) floats, scratch) and q_rot (may be NULL) receives the rotated q.
 * backward: prerotated != 0 means q and k are those rotated copies (fused dK+dV kernel); delta (B,Hq,N) is scratch. */
int corope_rope_attn_fwd_gqa(const void *q, const void *k, const void *v,
                             const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                             void *o, float *lse, void *q_rot, void *k_rot, float *tile_kmax,
                             int B, int Hq, int Hkv, int N, int D, float sm_scale, int causal, void *stream);
int corope_rope_attn_bwd_gqa(const void *q, const void *k, int prerotated, const void *v, const void *o, const void *d_o,
                             const float *lse, float *delta,
                             const float *freqs_cos, const float *freqs_sin, int64_t freq_row_stride,
                             void *dq, void *dk, void *dv,
                             int B, int Hq, int Hkv, int N, int D, float sm_scale, int causal, void *stream);

/* Co-RoPE grouped-query attention forward (causal only).
 * q: (B,Hq,N,D), k/v: (B,Hkv,N,D), o: (B,Hq,N,D), group size Hq/Hkv in [1, 8].
 * Replaces the launch of _corope_fwd_backbone in _attention.forward
 * (reference corope-exp/flash_attn_co_rope_gqa_triton.py:48-400 kernel, :428-450 launch);
 * the inverse frequencies theta^(-2d/D) the reference builds with torch (:428) are computed
 * on the host here and passed to the kernel by value.  Limits: B*Hkv*N < 2^31, N*D*2 bytes < 4 GiB. */
int corope_gqa_fwd(const void *q, const void *k, const void *v, void *o,
                   int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta, void *stream);

/* The same forward on fp16 tensors, the dtype of the reference's kernel and of its comparison script
 * (corope-exp/flash_attn_co_rope_gqa_triton.py:406-456, compare_corope.py:18): fp16 q, k, v, o; same kernel built for
 * fp16 elements (leader logits, scores and P V all on fp16 matrix-core operands).  The backward: corope_gqa_bwd_f16. */
int corope_gqa_fwd_f16(const void *q, const void *k, const void *v, void *o,
                       int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta, void *stream);

/* Bytes of device workspace corope_gqa_bwd needs for these sizes (-1 for sizes corope_gqa_check rejects):
 * packed lower-triangular N x N fp32 matrices (about N*N/2 + 32*N floats each): two per key/value head (accumulated
 * gates; gate gradients) and three per query head (attention weights; score gradients; dO V^T), plus N*D floats per
 * key/value head (the leader head's dq before its gate-path term is added). */
int64_t corope_gqa_bwd_workspace_bytes(int B, int Hq, int Hkv, int N, int D);

/* The smallest workspace corope_gqa_bwd accepts: the matrices of ONE (batch, key/value head) group, i.e. the figure above
 * divided by B*Hkv.  Groups are independent, so with a workspace between the two sizes the launch sequence runs once per
 * batch of as many groups as fit.  Fewer, larger passes are much faster, because two of the kernels spread over key blocks
 * x groups only: at B2 Hq32 Hkv8 N4096 D128 on MI355X 14.3 ms with all 16 groups in one pass (7.1 GiB), 31 ms with 4 per
 * pass (1.8 GiB), 94 ms with 1 (0.45 GiB) -- give it what memory allows.  -1 for sizes corope_gqa_check rejects. */
int64_t corope_gqa_bwd_min_workspace_bytes(int B, int Hq, int Hkv, int N, int D);

/* Co-RoPE grouped-query attention backward (causal only): dq (B,Hq,N,D), dk/dv (B,Hkv,N,D) from q, k, v and dO.
 * Replaces _attention.backward (reference corope-exp/flash_attn_co_rope_gqa_triton.py:459-577), which recomputes the
 * forward densely in PyTorch with (B,Hq,N,N,D/2) temporaries; the same gradients (including the path through the
 * leader head's gates, :548-561) are produced here with packed triangular N x N matrices of scalars in `workspace`.
 * Like the reference's, it needs neither the forward's output nor its row statistics; `o` may be NULL.  When the forward's output is
 * passed, rowsum(O o dO) serves as a reference value that keeps dQ accurate for rows dominated by a single key (the
 * result is mathematically the same with or without it).  The workspace need not be initialised and may be any size from
 * corope_gqa_bwd_min_workspace_bytes up (see there). */
int corope_gqa_bwd(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                   void *dq, void *dk, void *dv,
                   int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta,
                   void *workspace, int64_t workspace_bytes, void *stream);

/* The same for fp16 tensors, the dtype of the reference's callers (corope-exp/compare_corope.py:18): q, k, v, o, dO in and
 * dq, dk, dv out are fp16, every matrix-core operand is fp16, the workspace is the same size. */
int corope_gqa_bwd_f16(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                       void *dq, void *dk, void *dv,
                       int B, int Hq, int Hkv, int N, int D, float sm_scale, float theta,
                       void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* COROPE_AMD_H */
