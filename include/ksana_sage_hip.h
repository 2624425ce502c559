/*
 * libksana_sage_hip.so -- C ABI of the MI355X (gfx950) quantized "Sage" attention path.
 *
 * The reference (Tencent/KsanaDiT) has no FFI for this path: its Sage backend is a Python
 * adaptor around one third-party call,
 *     sageattn(q, k, v, tensor_layout="NHD", is_causal=...)
 *         ksana/operations/attention/backends/sage_attn.py:75-81
 * This library is what a Python backend class binds INSTEAD of that call.  The stage split
 * (quantize Q/K, quantize V, fused attention) follows the stages visible at the reference's
 * block-sparse sibling, ksana/operations/attention/backends/sage_sla.py:198-253.
 *
 * Conventions
 *   - every function returns 0 on success or a negative KSANA_SAGE_E* code; it never throws,
 *     exits or prints.  ksana_sage_last_error() gives the text for the calling thread.
 *   - all work is enqueued on `stream` (a hipStream_t passed as void*) and the call returns
 *     without synchronising.  The library allocates no device memory: the caller owns one
 *     workspace blob whose size and sub-buffer offsets come from ksana_sage_workspace_layout().
 *   - q, k, v, o are device pointers to [B, L, H, D] tensors of 16-bit floats (dtype below)
 *     with strides given in ELEMENTS in that index order; the D stride must be 1, the
 *     other strides multiples of 8 and the base pointers 16-byte aligned.
 *   - inputs are never written.  Calls that share a workspace must be ordered on one stream.
 */
#ifndef KSANA_SAGE_HIP_H
#define KSANA_SAGE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KSANA_SAGE_ABI_VERSION 20

/* element types of q/k/v/o */
#define KSANA_SAGE_BF16 0
#define KSANA_SAGE_FP16 1

/* error codes */
#define KSANA_SAGE_OK 0
#define KSANA_SAGE_EINVAL (-1)   /* bad shape, stride, alignment, dtype or null pointer      */
#define KSANA_SAGE_ENOTSUP (-2)  /* valid request this build does not implement (D != 128, sizes beyond its limits) */
#define KSANA_SAGE_EHIP (-3)     /* the HIP runtime reported an error at launch               */

/* flags of the attention entry points */
#define KSANA_SAGE_FLAG_PWL_EXP2 1 /* Default (flag clear): P = exp2(x) on the transcendental unit, then the  */
                                   /* hardware e4m3 cast.  Flag set: the e4m3 CODE of P is computed directly  */
                                   /* as rne(8*x + 55.5), i.e. exp2 with a piecewise-linear 3-bit mantissa:   */
                                   /* ~35 % fewer vector-ALU slots (about 1.2x faster), cos-sim to SDPA lower */
                                   /* by ~1.5e-4 and the worst element about 2x further out.                  */
#define KSANA_SAGE_FLAG_SMOOTH_V 2 /* ksana_sage_forward* only: quantize V with its channel means taken off   */
                                   /* (see ksana_sage_quant_v_smooth).                                        */

#define KSANA_SAGE_FLAG_WG_4_WAVES 4 /* attention entry points: force workgroups of 4 waves (128 query rows, two per   */
#define KSANA_SAGE_FLAG_WG_8_WAVES 8 /* compute unit) / of 8 waves (256 rows, one per unit) instead of the library's   */
                                     /* own choice (4 with a block mask, causal masking or Lk <= 1024).  Same results  */
                                     /* up to the rounding of the key-run merge; for measurements.                     */

/* rows per int8 scale: Q per token, K per 64 keys (sage_sla.py:190,204 uses (128, 64) off-Hopper;
 * the per-token Q scale is free in this kernel's operand layout and tighter) */
#define KSANA_SAGE_BLKQ 1
#define KSANA_SAGE_BLKK 64

#define KSANA_SAGE_FLAG_TILE_SKIP 16 /* attention entry points (not with KSANA_SAGE_FLAG_PWL_EXP2): a wave leaves out the  */
                                     /* exponentials and e4m3 conversions of a key tile whose scores lie more than 17     */
                                     /* octaves below the softmax reference point of each of its 32 rows.  Every          */
                                     /* probability byte of such a tile is the zero code, so the result is the same bits  */
                                     /* - the pvthreshold argument of the reference's sparse kernel (sage_sla.py:237-253; */
                                     /* the reference passes 1e6, i.e. "never"), at a threshold where nothing changes.    */
                                     /* Off by default: the test per tile costs ~7 % where no tile qualifies (flat         */
                                     /* attention); it pays where attention is peaked.                                     */

typedef struct ksana_sage_shape {
  int32_t B;   /* batch                                                     */
  int32_t Hq;  /* query heads                                               */
  int32_t Hkv; /* key/value heads; Hq % Hkv == 0                            */
  int32_t Lq;  /* query sequence length                                     */
  int32_t Lk;  /* key/value sequence length                                 */
  int32_t D;   /* head size: 128, or 64.  Rows of 64 channels are treated as    */
               /* rows of 128 whose upper half is zero (same workspace size,    */
               /* same kernels; o rows are 64 channels).  The folded norm /     */
               /* rotation step (ksana_sage_*_prep) needs 128.                  */
} ksana_sage_shape;

/* Byte offsets of the sub-buffers inside the workspace blob (each 256-byte aligned). */
typedef struct ksana_sage_ws_layout {
  uint64_t total_bytes;
  uint64_t q_i8;    /* int8  [B, Hq, LqPad, D] row-major, LqPad = ceil(Lq/128)*128, pad rows 0 */
  uint64_t q_scale; /* fp32  [B, Hq, LqPad]: one scale per query row                           */
  uint64_t k_i8;    /* int8  [B, Hkv, nkb, 8192] nkb = ceil(Lk/64): one 64x128 tile per block,  */
                    /*       stored in MFMA operand order (see ksanadit_amd/layout.py)          */
  uint64_t k_scale; /* fp32  [B, Hkv, nkb]                                                      */
  uint64_t k_mean;  /* fp32  [B, Hkv, D]: the channel mean AFTER rounding to the input dtype    */
  uint64_t v_fp8;   /* e4m3fn[B, Hkv, nkb, 8192]: V^T tile 128x64 in MFMA operand order         */
  uint64_t v_scale; /* fp32  [B, Hkv, D]                                                        */
  uint64_t v_inv;   /* fp32  [B, Hkv, D]: 448/amax used by the V quantizer                      */
  uint64_t k_part;  /* fp32  [B, Hkv, nch, D] nch = ceil(Lk/256): chunk sums of K               */
  uint64_t v_part;  /* fp32  [B, Hkv, nch, D]: chunk abs-max of V                               */
  uint64_t q_rms;   /* fp32  [B, Lq]: 1/sqrt(mean(q_row^2) + eps), written by the *_prep entry points */
  uint64_t k_rms;   /* fp32  [B, Lk]: the same for the key rows                                 */
  uint64_t v_mean;  /* fp32  [B, Hkv, D]: channel mean taken off V before scaling (rounded to the input */
                    /*       dtype; zeros without V smoothing); the attention adds it to its output     */
  uint64_t split_o; /* fp32  [256, 256, D]: scratch of the attention kernel - unnormalised accumulators */
                    /*       of workgroups whose key loop was cut into runs (see ksana_sage_attn_fwd)   */
  uint64_t split_ml;/* fp32  [256, 256, 2]: their running maxima and row sums                           */
  uint64_t k_sync;  /* int32 [2 * B*Hkv * 32 + 32]: per head a chunk counter and a ready flag (each in a 128-byte */
                    /*       line of its own) through which the workgroups of the one-read K quantizer meet, then */
                    /*       one status word                                                                       */
  uint64_t v_sync;  /* int32, the same for the one-read V quantizer                                                */
  int32_t lq_pad;
  int32_t nqb;
  int32_t nkb;
  int32_t nch;
} ksana_sage_ws_layout;

/* What WanSelfAttention.forward does to the q and k projections before it calls attention
 * (wan_model.py:163-174), for the *_prep entry points to apply while they read q and k:
 *   RMSNorm over the whole token row of H*D channels with an fp32 weight
 *     (norm_q / norm_k, wan_model.py:81-90; ops.py:62-72), then
 *   the 3-axis rotary embedding apply_default_rope(x, grid_sizes, freqs) (rope.py:61-128, one GPU).
 * Results are rounded to the tensor's half type after each of the two steps, as the separate
 * modules store them.  A NULL weight skips the norm of that tensor, NULL rope_freqs the rotation
 * (WanCrossAttention, wan_model.py:236-237, norms but does not rotate). */
typedef struct ksana_sage_prep {
  const float* q_norm_weight;  /* device, fp32 [Hq*D], 16-byte aligned, or NULL                          */
  const float* k_norm_weight;  /* device, fp32 [Hkv*D], 16-byte aligned, or NULL                         */
  float norm_eps;
  int32_t rope_rows;           /* rows of rope_freqs (1024 in the model, wan_model.py:679-681)           */
  const double* rope_freqs;    /* device, complex128 [rope_rows, D/2] as (re, im) pairs: the model's     */
                               /* `freqs` buffer (wan_model.py:677-684), 16-byte aligned, or NULL        */
  const int32_t* grid_sizes;   /* HOST array [B, 3]: (frames, height, width) per batch entry; the        */
                               /* reference reads it on the host as well (rope.py:107).  Needed with     */
                               /* rope_freqs; B <= 16; each extent <= rope_rows; F*H*W <= L              */
  /* kind == KSANA_SAGE_PREP_QWEN: what QwenDoubleStreamAttention.forward does to the joint q and k (text rows
   * first, image rows behind them, qwen/attention.py:340-357) instead of the Wan steps above:
   *   RMSNorm over the D channels of every head (norm_q / norm_k for the image rows, norm_added_q / norm_added_k for
   *     the text rows; float_rmsnorm of ops.py:62-72 with the statistic per head), then
   *   apply_rotary_emb_qwen (qwen/attention.py:31-59): pairs (x[2i], x[2i+1]) times one complex64 factor per
   *     (row, pair), image rows from rope_freqs_img, text rows from rope_freqs_txt.
   * q_norm_weight / k_norm_weight are then the IMAGE weights, fp32 [D]; the fields below the text side.  The caller
   * hands over the raw projections already concatenated (text first) - the concatenation the block performs anyway.
   * NULL weights skip the norm of that segment, NULL tables its rotation.  rope_freqs / grid_sizes are not used. */
  int32_t kind;                    /* KSANA_SAGE_PREP_WAN (0), _WAN_COMFY (1), _QWEN (2)                   */
  int32_t txt_len;                 /* rows [0, txt_len) are text, [txt_len, L) image                          */
  const float* q_norm_weight_txt;  /* device, fp32 [D], 16-byte aligned, or NULL                              */
  const float* k_norm_weight_txt;
  const float* rope_freqs_txt;     /* device, complex64 [txt_len, D/2] as (re, im), 16-byte aligned, or NULL  */
  const float* rope_freqs_img;     /* device, complex64 [L - txt_len, D/2]                                    */
  /* kind == KSANA_SAGE_PREP_WAN_COMFY: the Wan block with rope_func == "comfy" (wan_model.py:169-171): the norm as
   * for KSANA_SAGE_PREP_WAN, then apply_comfyui_rope (utils/rope.py:180-212): out[2i+e] = m[e][0]*x[2i] +
   * m[e][1]*x[2i+1] in fp32 with the 2x2 matrix of (row, pair i).  rope_rows is the table's row count here; rows at or
   * past it are left as they are (the identity padding of rope.py:133-148).  rope_freqs / grid_sizes are not used. */
  const float* rope_matrices;      /* device, fp32 [rope_rows, D/2, 2, 2]: the `freqs_cis` of EmbedND            */
                                   /* (rope.py:165-177) without its broadcast dims, 16-byte aligned, or NULL     */
} ksana_sage_prep;
#define KSANA_SAGE_PREP_WAN 0
#define KSANA_SAGE_PREP_WAN_COMFY 1
#define KSANA_SAGE_PREP_QWEN 2

/* Library identity.  No counterpart in the reference. */
int ksana_sage_abi_version(void);
const char* ksana_sage_last_error(void);

/* Process-wide settings of the one-read K / V quantizers (see ksana_sage_quant_status for what they are).  No
 * counterpart in the reference.
 *   one_read_stages: NULL = leave as it is; otherwise a string of the letters "k" and "v": the stages that take the
 *     one-read kernel when the shape allows ("" = neither).  First value: the environment variable
 *     KSANA_SAGE_ONE_READ, default "v"; the environment is read once, when the first call needs it.  K with a folded
 *     norm / rotation step always tries the one-read kernel.
 *   wait_ticks: KSANA_SAGE_KEEP = leave as it is; otherwise the bound, in 10 ns ticks, on a workgroup's wait for its
 *     head's statistic.  First value: KSANA_SAGE_WAIT_TICKS, default 200000 (2 ms; the kernels run 0.1 - 0.5 ms).
 *     A positive bound that expires makes the library take the two-pass kernels on that GPU from the next call on (the
 *     GPU evidently holds fewer workgroups at once than the launcher counted on, e.g. because it is shared; results
 *     are the same bits either way).  0 (give up at the first poll that finds the flag down) and negative values (do
 *     not poll: every workgroup but a head's last arriver recomputes the statistic from the input) exercise that path
 *     in tests and switch nothing off.
 * Every call also re-arms the one-read kernels on all GPUs. */
#define KSANA_SAGE_KEEP INT64_MIN
int ksana_sage_configure(const char* one_read_stages, int64_t wait_ticks);
/* The current settings, and whether the one-read kernels are switched off on the current GPU because a wait expired
 * there (any out-pointer may be NULL).  Reads host memory only; for logs and tests. */
int ksana_sage_one_read_state(int* one_read_k, int* one_read_v, int64_t* wait_ticks, int* demoted);
/* Host-side self-checks of the library's bookkeeping (today: that two instantiations of one kernel template keep
 * separate entries in the cache of resident-workgroup counts).  Touches no device; 0 = all passed. */
int ksana_sage_selftest(void);

/* Size/offsets of the scratch the stages below share.  Replaces the torch.empty calls the
 * reference makes for its quantized operands (sage_sla.py:222-227). */
int ksana_sage_workspace_layout(const ksana_sage_shape* shape, ksana_sage_ws_layout* out);

/* Q -> Walsh-Hadamard transform over D, times sm_scale*log2(e)/128, per-row int8 + fp32 scale.
 * Replaces the Q half of get_vanilla_qk_quant(q, k, km, 128, 64) (sage_sla.py:202-204). */
int ksana_sage_quant_q(const void* q, int dtype, const int64_t q_strides[4], const ksana_sage_shape* shape,
                       float sm_scale, void* workspace, void* stream);

/* K -> channel mean over the sequence (km = k.mean(-2), sage_sla.py:198), subtracted when
 * smooth_k != 0, then Walsh-Hadamard transform over D and per-64-row-block int8 + fp32 scale
 * (K half of sage_sla.py:202-204). */
int ksana_sage_quant_k(const void* k, int dtype, const int64_t k_strides[4], const ksana_sage_shape* shape,
                       int smooth_k, void* workspace, void* stream);

/* ksana_sage_quant_k for callers that cannot allocate device memory - code under HIP graph capture, tight serving
 * loops, harnesses that forbid it - and therefore cannot grow a workspace for a new shape's scratch.  No counterpart
 * in the reference.  Same arguments, same results bit for bit; the difference is where the kernels' scratch (the
 * per-256-row chunk sums behind the channel means) lives: not in the workspace's k_part area, which this call
 * leaves untouched, but in a 9 MiB array inside the library's own device image.  Limits: B * Hkv * ceil(Lk / 256)
 * <= 16384 and B * Hkv <= 4096 (KSANA_SAGE_ENOTSUP beyond).  The call allocates and frees nothing.  All calls on one GPU share that
 * array: calls that overlap on one GPU (different streams or threads) race and must be ordered by the caller.
 * Under graph capture: make one ordinary call on the device first (the first call looks the array's address up and
 * may load the code object, which a capturing stream can refuse).  The counters through which the workgroups of the
 * one-read kernel meet (KSANA_SAGE_ONE_READ=k) live in that array too: ksana_sage_quant_status, which reads the
 * workspace's words, says nothing about this call. */
int ksana_sage_quant_k_static(const void* k, int dtype, const int64_t k_strides[4], const ksana_sage_shape* shape,
                              int smooth_k, void* workspace, void* stream);

/* quant_q / quant_k with the step before attention folded in: q and k are the projections
 * viewed [B, L, H, D] (the H stride must be D: a token row is one contiguous run of H*D channels).
 * Replaces norm_q/norm_k + apply_default_rope + the quantizer of the path (wan_model.py:163-174
 * followed by sage_sla.py:198-204) without the two intermediate tensors: one extra read of the
 * input for the row statistic instead of two writes and two reads. */
int ksana_sage_quant_q_prep(const void* q, int dtype, const int64_t q_strides[4], const ksana_sage_shape* shape,
                            const ksana_sage_prep* prep, float sm_scale, void* workspace, void* stream);
int ksana_sage_quant_k_prep(const void* k, int dtype, const int64_t k_strides[4], const ksana_sage_shape* shape,
                            const ksana_sage_prep* prep, int smooth_k, void* workspace, void* stream);
/* The two calls above as one.  Same results in the same workspace areas; where q's token-row norm makes its kernel
 * take whole rows anyway, the row statistic of k rides along in that kernel instead of costing a pass over k of its
 * own.  What a caller that holds q and k together should use (the reference's block does: wan_model.py:163-174,
 * sage_sla.py:198-204 quantize both in one call). */
int ksana_sage_quant_qk_prep(const void* q, const void* k, int dtype, const int64_t q_strides[4],
                             const int64_t k_strides[4], const ksana_sage_shape* shape, const ksana_sage_prep* prep,
                             float sm_scale, int smooth_k, void* workspace, void* stream);

/* V -> transposed, padded, operand-ordered fp8 e4m3fn with one fp32 scale per (b, h, d).
 * Replaces transpose_pad_permute_cuda + scale_fuse_quant_cuda (sage_sla.py:222-228). */
int ksana_sage_quant_v(const void* v, int dtype, const int64_t v_strides[4], const ksana_sage_shape* shape,
                       void* workspace, void* stream);

/* The same with V smoothing when smooth_v != 0: the mean of every channel over the Lk rows (summed in the order
 * of the K mean, rounded to the input dtype) is subtracted in fp32 before the abs-max and the scaling, stored in
 * the workspace, and added back to the attention output (rows of P sum to one).  A channel that sits far from
 * zero then spends its e4m3 steps on the deviations instead of on the offset.  The `smooth_v` option of the
 * library behind the reference's call (sage_attn.py:75-81; off in that call, off by default here); one more
 * read of V.  smooth_v == 0 is ksana_sage_quant_v. */
int ksana_sage_quant_v_smooth(const void* v, int dtype, const int64_t v_strides[4], const ksana_sage_shape* shape,
                              int smooth_v, void* workspace, void* stream);

/* Block means for the sparse-linear backend's block map: out[b, h, i, :] = mean of x[b, i*rows_per_block : (i+1)*
 * rows_per_block, h, :] (the last block may be shorter), fp32 sum / number of rows, rounded to x's dtype; out is
 * [B, H, ceil(L / rows_per_block), D] in x's dtype, contiguous; x is [B, L, H, D] with `strides` like q/k/v (D = 128).
 * With centre != NULL (device, fp32 [B, H, D]) every x - centre is rounded to x's dtype before it is summed: the
 * reference pools `k - torch.mean(k, dim=-2, keepdim=True)`, a tensor in k's dtype (sage_sla.py:79-81); the k_mean
 * area of a workspace after ksana_sage_quant_k holds exactly that mean.  rows_per_block: a multiple of 32, <= 256.
 * Replaces the Triton kernel compress_kernel / mean_pool (sage_sla.py:43-75). */
int ksana_sage_block_means(const void* x, int dtype, const int64_t strides[4], int B, int H, int L, int rows_per_block,
                           const float* centre, void* out, void* stream);

/* ksana_sage_quant_q + ksana_sage_quant_k (smooth_k = 1) that take the sparse-linear backend's block averages along:
 * pooled_q [B, Hq, ceil(Lq / 128), 128] and pooled_k [B, Hkv, ceil(Lk / 64), 128] (device, `dtype`, contiguous) come
 * out bit for bit as ksana_sage_block_means(q, 128 rows) and ksana_sage_block_means(k, 64 rows, centre = the
 * workspace's k_mean) give them - the quantizers' workgroups are those blocks - without reading q and k once more.
 * Head size 128 only (KSANA_SAGE_ENOTSUP otherwise).  Replaces get_vanilla_qk_quant (sage_sla.py:202-204) together
 * with compress_kernel / mean_pool on q and on k - mean(k) (sage_sla.py:43-81). */
int ksana_sage_quant_qk_pooled(const void* q, const void* k, int dtype, const int64_t q_strides[4],
                               const int64_t k_strides[4], const ksana_sage_shape* shape, float sm_scale,
                               void* pooled_q, void* pooled_k, void* workspace, void* stream);

/* The second half of get_block_map (sage_sla.py:83-90) in one kernel: score = pooled_q pooled_k^T as a tensor of the
 * blocks' dtype, then per query block ones at the `keep` key blocks with the largest scores (of equal scores the
 * lower index wins; torch.topk, which the reference calls, leaves that open), zeros elsewhere.  pooled_q / pooled_k:
 * device, [B, H, nq, 128] / [B, H, nk, 128] in `dtype`, contiguous (what ksana_sage_block_means writes);
 * block_map: int8 [B, H, nq, nk], contiguous - the mask ksana_sage_attn_fwd_masked takes.  nk <= 1024
 * (KSANA_SAGE_ENOTSUP beyond).  Replaces a GEMM, torch.topk, zeros_like and scatter_. */
int ksana_sage_sla_block_map(const void* pooled_q, const void* pooled_k, int dtype, int B, int H, int nq, int nk,
                             int keep, int8_t* block_map, void* stream);

/* The linear-attention branch of the sparse-linear backend and what the backend does with it, in three kernels over
 * [B, L, H, D] tensors (D = 128; strides as for q/k/v), with phi = softmax over the channels of a row, rounded to the
 * tensors' dtype:
 *     kv = sum_l phi(k_l)^T v_l,  ksum = sum_l phi(k_l)                         (each rounded to the dtype)
 *     out_l = (phi(q_l) kv) / (1e-5 + phi(q_l) . ksum)                          sage_sla.py:135-139, 273-282
 *     out_l = out_l W^T + bias      when proj_weight != NULL (fp32 [128][128], (out, in); bias fp32 [128] or NULL):
 *                                   the block's proj_l layer, sage_sla.py:284-285, folded in as phi(q_l) (kv W^T)
 *     out_l += add_l                when add != NULL: the sparse branch's result, sage_sla.py:286
 * k and v are read once, q once; out may alias add.  sla_workspace: ksana_sage_sla_workspace_bytes(B, H, L) bytes of
 * device memory, 256-byte aligned (partial sums of kv per run of rows, added in a fixed order: repeated calls give
 * the same bits).  Replaces calc_linear and the two feature maps of the reference (five library kernels over
 * [B, H, L, D] intermediates there). */
int ksana_sage_sla_workspace_bytes(int B, int H, int L, uint64_t* bytes);
int ksana_sage_sla_linear(const void* q, const void* k, const void* v, int dtype, const int64_t q_strides[4],
                          const int64_t k_strides[4], const int64_t v_strides[4], int B, int H, int L,
                          const float* proj_weight, const float* proj_bias, const void* add,
                          const int64_t add_strides[4], void* out, const int64_t out_strides[4], void* sla_workspace,
                          void* stream);

/* Did a workgroup of the last ksana_sage_quant_k / ksana_sage_quant_v on this workspace give up waiting for the
 * others of its head?  Both quantizers can read their input once: a workgroup keeps its rows in registers while the
 * statistic of its head (channel means / column maxima) is gathered from all of them, and that wait is bounded by
 * a limit (2 ms by default, ksana_sage_configure) so that every kernel ends.  On a GPU the call has to itself the limit is never met.  Where it is
 * (a device shared with other work can hold fewer workgroups at once than the launcher counted on), the workgroup
 * takes the statistic from the input itself, in the specified order: the quantized operands are the same bits, the
 * call was slow, and the status word of the stage is 1.  SYNCHRONISES `stream`, then copies the two words: a call
 * for tests and diagnostics, not for the hot path.  No counterpart in the reference. */
int ksana_sage_quant_status(const void* workspace, const ksana_sage_shape* shape, void* stream, int* k_status,
                            int* v_status);

/* Fused attention on the quantized operands in `workspace`: INT8 QK^T, fp32 online softmax,
 * FP8 PV, output in `dtype` at [B, Lq, Hq, D] with `o_strides`.  Replaces the qattn.* kernel
 * call (sage_sla.py:237-253, dense form).  flags: KSANA_SAGE_FLAG_*.
 * When the number of 256-row query blocks times heads leaves a small remainder against the number of compute units,
 * the workgroups of that remainder are cut into runs of key tiles that fill the chip together, and a second small
 * kernel merges the runs (dense, non-causal calls only); the result is the same attention within rounding, and
 * repeated calls give identical bits.  The quantized operands in the workspace are only read; the runs' scratch
 * (split_o, split_ml) is the one part of it this call writes.
 * causal: non-zero lets query row i attend to keys [0, i] only (the is_causal of sage_attn.py:75-81 and of
 * sdpa.py:62-79), on top of k_lens and the block mask; for Lq != Lk the triangle is anchored at the top left corner,
 * as torch's scaled_dot_product_attention anchors it (sdpa.py:62-79 is the accuracy anchor of this path).  Lk <= 131072.
 * k_lens: NULL, or a device array of B int32: batch b attends to keys [0, k_lens[b]) only
 * (clamped to [0, Lk]; a batch without keys gets zeros).  Same meaning as the k_lens the
 * reference's callers pass (wan_model.py:182-189) and its variable-length backend honours
 * (flash_attn.py:131-139); the reference's Sage adaptor drops the argument (sage_attn.py:58-84),
 * which is what NULL reproduces.  The quantizers always see all Lk rows. */
int ksana_sage_attn_fwd(void* workspace, void* o, int dtype, const int64_t o_strides[4],
                        const ksana_sage_shape* shape, const int32_t* k_lens, int causal, int flags, void* stream);

/* ksana_sage_attn_fwd restricted by a block mask: block_mask is a device array of int8
 * [B, Hq, ceil(Lq/128), ceil(Lk/64)]; a non-zero entry lets the 128 query rows of its row attend to
 * the 64 keys of its column, zero hides them; dense inside a block.  mask_strides are the element
 * strides of the two leading dimensions (0 broadcasts over batch / heads); the last two dimensions
 * are contiguous.  Query rows whose mask row is all zero come out as zeros.  Lk <= 131072.
 * Replaces block_sparse_sage2_attn_cuda(q, k, v, mask_id=..., tensor_layout="NHD")
 * (radial_sage_attn.py:24,170-176: the same mask shape and block sizes); block_mask == NULL is
 * ksana_sage_attn_fwd.  Key tiles neither 128-row half of a 256-row workgroup asks for are skipped. */
int ksana_sage_attn_fwd_masked(void* workspace, void* o, int dtype, const int64_t o_strides[4],
                               const ksana_sage_shape* shape, const int8_t* block_mask,
                               const int64_t mask_strides[2], const int32_t* k_lens, int causal, int flags,
                               void* stream);

/* ksana_sage_attn_fwd_masked with a per-batch count of query rows as well: q_lens is NULL or a device array of B int32;
 * rows [0, q_lens[b]) of batch b (clamped to [0, Lq]) are computed, the rows from there to Lq are written as zeros and
 * cost nothing.  The q_lens of the reference's backends (flash_attn.py:120-124 packs the first q_lens[b] rows of every
 * batch entry before its variable-length call; sdpa.py:52-57 accepts and ignores the argument, like the Sage adaptor,
 * which NULL reproduces).  Everything else as in ksana_sage_attn_fwd_masked. */
int ksana_sage_attn_fwd_varlen(void* workspace, void* o, int dtype, const int64_t o_strides[4],
                               const ksana_sage_shape* shape, const int8_t* block_mask,
                               const int64_t mask_strides[2], const int32_t* q_lens, const int32_t* k_lens,
                               int causal, int flags, void* stream);

/* How ksana_sage_attn_fwd cuts `shape` on the current device (dense, non-causal calls): the 256-row query blocks
 * numbered *first_workgroup and up - numbering (b * Hq + h) * ceil(Lq/256) + block - have their key loop cut into
 * *runs runs; *runs == 0 means no cut.  For tools that want to mirror the kernel's rounding exactly (the test
 * emulation does); no counterpart in the reference. */
int ksana_sage_attn_key_split(const ksana_sage_shape* shape, int* first_workgroup, int* runs);

/* Measurement aid, no counterpart in the reference: launches `workgroups` workgroups of 8 waves that each issue, `steps`
 * times, the attention kernel's matrix instructions per key tile (8 INT8 + 5 FP8 MFMAs) on register operands and
 * nothing else.  `scratch` receives workgroups * 512 floats (so the work is not optimised away); *ops_per_launch is the
 * number of operations (multiply-add = 2) one launch performs.  Time it with events on `stream`: the rate is what the
 * matrix pipe sustains at the clock it holds under this load. */
int ksana_sage_mfma_probe(void* scratch, uint64_t scratch_bytes, int workgroups, int steps, void* stream,
                          double* ops_per_launch);

/* The whole path in one call: quant_q, quant_k, quant_v, attn_fwd on `stream`.
 * Replaces sageattn(q, k, v, tensor_layout="NHD", is_causal=causal) (sage_attn.py:75-81). */
int ksana_sage_forward(const void* q, const void* k, const void* v, void* o, int dtype,
                       const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                       const int64_t o_strides[4], const ksana_sage_shape* shape, const int32_t* k_lens,
                       float sm_scale, int smooth_k, int causal, int flags, void* workspace, void* stream);

/* ksana_sage_forward with q and k taken as projections and `prep` applied on the way in
 * (prep == NULL is ksana_sage_forward).  Replaces wan_model.py:163-174 + the attention call at :190. */
int ksana_sage_forward_prep(const void* q, const void* k, const void* v, void* o, int dtype,
                            const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                            const int64_t o_strides[4], const ksana_sage_shape* shape, const ksana_sage_prep* prep,
                            const int32_t* k_lens, float sm_scale, int smooth_k, int causal, int flags,
                            void* workspace, void* stream);

/* ksana_sage_forward with the block mask of ksana_sage_attn_fwd_masked. */
int ksana_sage_forward_masked(const void* q, const void* k, const void* v, void* o, int dtype,
                              const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                              const int64_t o_strides[4], const ksana_sage_shape* shape, const int8_t* block_mask,
                              const int64_t mask_strides[2], const int32_t* k_lens, float sm_scale, int smooth_k,
                              int causal, int flags, void* workspace, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KSANA_SAGE_HIP_H */
