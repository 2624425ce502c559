// Internal launch interface between the C ABI (sage_capi.hip) and the gfx950 kernels.
// Pointers are device pointers; strides are in elements; every launcher enqueues on `stream`
// and returns the hipError_t of the launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ksana_sage {

constexpr int kD = 128;          // head size the kernels are written for
constexpr int kBlkQ = 1;         // query rows per int8 scale (per token)
constexpr int kQPad = 128;       // stored query rows are padded to a multiple of this
constexpr int kBlkK = 64;        // key rows per int8 scale == key rows per LDS tile
constexpr int kMeanChunk = 256;  // rows per partial column sum
constexpr int kTileBytes = kBlkK * kD;  // one K (int8) or V^T (fp8) tile: 8192 bytes
constexpr int kAttnQPerWg = 256; // query rows per attention workgroup (8 waves x 32)

struct InTensor {
  const uint16_t* ptr;
  int64_t sB, sL, sH;  // element strides of [B, L, H, D]; D stride is 1
  int dtype;           // KSANA_SAGE_BF16 / KSANA_SAGE_FP16
  int D = 128;         // channels per row that exist: 128, or 64 (the kernels then read the upper 64 as zeros)
};

struct OutTensor {
  uint16_t* ptr;
  int64_t sB, sL, sH;
  int dtype;
};

// What the Wan block does to Q and K between the projection and attention, applied by the
// quantizer kernels to the channels they have just loaded (nullptr members switch a step off):
// RMSNorm over the whole token row (statistic precomputed per row), then the 3-axis rotary
// embedding with the model's complex128 table.
constexpr int kMaxPrepBatch = 16;
constexpr int kRopeSplit0 = 22, kRopeSplit1 = 43;  // pairs [0,22) turn with the frame, [22,43) row, [43,64) column
struct PrepParams {
  const float* inv_rms;  // [B, L]: 1 / sqrt(mean(x^2) + eps) of each token row; nullptr = no norm
  const float* weight;   // [H * 128] fp32 norm weight
  const double* freqs;   // [rows, 64] complex128 as (re, im); nullptr = no rotation
  int L;
  // kind 2, the Qwen-Image block (qwen/attention.py:340-353): RMSNorm over the 128 channels of every head (the
  // statistic is taken inside the kernel), one weight vector for the text rows [0, txt_len) and one for the image rows
  // behind them, then a rotation by one complex64 factor per (row, pair) from a table per segment.  A nullptr weight
  // / table switches that step off for its segment.
  int kind;  // 1: the Wan block (fields above and below), 2: the Qwen block (fields here), 3: the Wan block with
             // the rotation given as one 2x2 fp32 matrix per (row, pair) (`rot`, utils/rope.py:180-212)
  const float4* rot;  // kind 3: [rot_rows, 64] matrices (m00, m01, m10, m11); rows from rot_rows on are not rotated
  int rot_rows;
  int txt_len;
  float eps;
  const float* weight_txt;    // [128]
  const float* weight_img;    // [128]
  const float2* freqs_txt;    // [txt_len, 64] (re, im)
  const float2* freqs_img;    // [L - txt_len, 64]
  int grid[kMaxPrepBatch][3];  // (frames, height, width) per batch entry
  // Capacity (table rows) of the per-workgroup LDS copy of the rotation factors, filled in by the
  // launcher for its kernel's rows per workgroup; lds_frames == 0: read `freqs` directly.
  int lds_frames, lds_heights, lds_widths;
};
// inv_rms[b, l] from x[b, l, :H*128] (the row must be contiguous: sH == 128)
hipError_t launch_row_inv_rms(const InTensor& x, int B, int H, int L, float eps, float* inv_rms, hipStream_t s);

// column reductions over the sequence: op 0 = ordered fp32 sum, op 1 = max of |x|
// op 0: column sums, 1: column max |x|, 2: column max |x - centre[d]| (centre: [B, H, D])
hipError_t launch_col_partial(const InTensor& x, int B, int H, int L, int op, float* part, int nch, hipStream_t s,
                              const PrepParams* prep = nullptr, const float* centre = nullptr);
// status: nullptr, or the quantizer's status word to clear (see QuantSync)
hipError_t launch_k_mean_finalize(const float* part, int BH, int nch, int L, int dtype, int smooth, float* k_mean,
                                  hipStream_t s, int* status = nullptr);
// zero_mean: nullptr, or the [BH, D] mean slot to clear (V quantized without smoothing)
hipError_t launch_v_scale_finalize(const float* part, int BH, int nch, float* v_scale, float* v_inv, float* zero_mean,
                                   hipStream_t s, int* status = nullptr);
// pooled (quant_q and quant_k): nullptr, or where the averages of the blocks the kernel quantizes anyway - 128 query
// rows, 64 keys less their channel mean - go as [B, H, blocks, 128] of the input's half type, bit for bit what
// launch_block_means gives (head size 128, no prep)
hipError_t launch_quant_q(const InTensor& q, int B, int H, int L, int lq_pad, float premul, int8_t* q_i8,
                          float* q_scale, hipStream_t s, const PrepParams* prep = nullptr, uint16_t* pooled = nullptr);
// Q with a token-row norm (prep.inv_rms, prep.weight set; kinds 1 and 3): statistic and quantization from one pass over
// HBM, 32 whole token rows per workgroup; writes prep.inv_rms as launch_row_inv_rms would.  k_rows != nullptr: the
// statistic of rows [0, k_L) of that tensor (k_H heads of 128 channels, contiguous per row) goes to k_rms on the way.
hipError_t launch_quant_q_rows(const InTensor& q, int B, int H, int L, int lq_pad, float premul, float eps,
                               int8_t* q_i8, float* q_scale, hipStream_t s, const PrepParams& prep,
                               const InTensor* k_rows, int k_H, int k_L, float* k_rms);
hipError_t launch_quant_k(const InTensor& k, int B, int H, int L, int nkb, const float* k_mean, int8_t* k_tiles,
                          float* k_scale, hipStream_t s, const PrepParams* prep = nullptr, uint16_t* pooled = nullptr);
// v_mean: nullptr, or the channel means taken off before scaling (V smoothing)
hipError_t launch_quant_v(const InTensor& v, int B, int H, int L, int nkb, const float* v_inv, const float* v_mean,
                          uint8_t* v_tiles, hipStream_t s);

// Counters and flags of the one-read K / V quantizers, all zero before the launch (launch_clear_ints).  One
// word per head, kSyncStride words apart so that each sits in a cache line of its own.
constexpr int kSyncStride = 32;
constexpr int sync_words(int bh) { return 2 * bh * kSyncStride + kSyncStride; }  // counters, ready flags, status
struct QuantSync {
  int* k_counter;  // chunks of the head whose column sums are published
  int* k_ready;    // non-zero once the head's mean is published
  int* k_status;   // set to 1 if a workgroup gave up waiting (the results are then not to be trusted)
  int* v_counter;  // the same three for V: chunks whose column maxima are published,
  int* v_ready;    // scales published,
  int* v_status;   // a wait that ran into its limit
};
hipError_t launch_clear_ints(int* p, int n, hipStream_t s);

// Process-wide settings of the one-read quantizers.  Their first values come from the environment, read once when
// the first call needs them (KSANA_SAGE_ONE_READ: which of "k", "v" take the one-read kernels when the shape allows,
// default "v"; KSANA_SAGE_WAIT_TICKS: the bound below); configure_quant replaces them.
constexpr long long kDefaultWaitTicks = 200000;  // 2 ms at 100 MHz: ten to twenty times a healthy kernel's whole run
struct QuantOptions {
  bool one_read_k, one_read_v;
  // Wall-clock ticks (10 ns) a workgroup waits for its head's statistic before it takes it from the input itself.
  // > 0: a bound for production; an expiry also switches the one-read kernels off on that device (see
  // one_read_demoted).  0: give up at the first poll that finds the flag down; < 0: do not look at the flag at all,
  // every workgroup but the head's last arriver recomputes - both are for tests and switch nothing off.
  long long wait_ticks;
};
QuantOptions quant_options();
// stages == nullptr / keep_ticks: leave that setting as it is.  Also forgets every device's demotion.
void configure_quant(const char* stages, long long wait_ticks, bool keep_ticks);
// Has a workgroup's wait run into a bound > 0 on the current device since the last configure_quant?  The launchers
// then take the two-pass kernels there: a device that holds fewer workgroups than its occupancy figure promises
// (shared with other work) would pay the bound in every call.  `may_allocate` == false never creates the
// host-visible word the kernels report through (for callers that must not allocate): without it nothing is
// reported and the answer is false.
bool one_read_demoted(bool may_allocate = true);
// 0 when two kernel instantiations of one function-pointer type keep separate entries in the launchers' cache of
// resident-workgroup counts (a host-side self-check; touches no device)
int selftest_occupancy_cache();

// One-read quantizers: *used == false means the shape does not suit them and nothing was launched.
// `may_allocate`: see one_read_demoted.
hipError_t launch_quant_k_fused(const InTensor& k, int B, int H, int L, int nkb, int nch, int smooth, float* part,
                                float* k_mean, int8_t* k_tiles, float* k_scale, const QuantSync& sync, hipStream_t s,
                                const PrepParams* prep, bool* used, bool may_allocate = true);
hipError_t launch_quant_v_fused(const InTensor& v, int B, int H, int L, int nkb, int nch, float* part, float* v_scale,
                                float* v_inv, float* v_mean, uint8_t* v_tiles, const QuantSync& sync, hipStream_t s,
                                bool* used);

// out[b, h, blk, :] = mean of the rows of block blk (rows per block: a multiple of 32, at most 256) of x[b, :, h, :],
// of round_to_half(x - centre[b, h, :]) when centre != nullptr; out is [B, H, ceil(L / rows), 128] in x's half type
hipError_t launch_block_means(const InTensor& x, int B, int H, int L, int rows, const float* centre, uint16_t* out,
                              hipStream_t s);

// The linear-attention branch of the sparse-linear backend (sage_sla.hip).  part: [B * H][runs][128 * 128 + 128] fp32
// (plan_sla_runs gives runs); m_frag: [B * H][128 * 128] halves; ksum: [B * H][128] fp32.  proj_w: fp32 [128][128]
// (out, in) or nullptr; proj_b: fp32 [128] or nullptr; add: a [B, L, H, D] tensor added to the result, or nullptr.
void plan_sla_runs(int B, int H, int L, int* runs, int* rows_per_run);
struct OutTensor;
hipError_t launch_sla_linear(const InTensor& q, const InTensor& k, const InTensor& v, int B, int H, int L,
                             const float* proj_w, const float* proj_b, const InTensor* add, const OutTensor& out,
                             float* part, uint16_t* m_frag, float* ksum, hipStream_t s);

// int8 block_map[BH][nq][nk]: per query block ones at the `keep` key blocks with the largest pooled_q . pooled_k (half
// tensors [BH][n][128], contiguous); nk <= 1024
hipError_t launch_sla_block_map(const uint16_t* pooled_q, const uint16_t* pooled_k, int dtype, int BH, int nq, int nk, int keep,
                                int8_t* block_map, hipStream_t s);

struct AttnParams {
  const int8_t* q_i8;
  const float* q_scale;
  const int8_t* k_tiles;
  const float* k_scale;
  const uint8_t* v_tiles;
  const float* v_scale;
  const float* v_mean;  // [B, Hkv, D] added to every output row that saw a key (zeros without V smoothing)
  OutTensor o;
  int B, Hq, Hkv, Lq, Lk, lq_pad, nkb;
  int exact_exp2;  // 1: exp2 on the transcendental unit; 0: piecewise-linear e4m3 code (faster)
  const int32_t* k_lens;  // optional [B]: batch b attends to keys [0, clamp(k_lens[b], 0, Lk)); nullptr = all
  const int32_t* q_lens;  // optional [B]: query rows [0, clamp(q_lens[b], 0, Lq)) of batch b are computed, the rest zeros
  // optional block mask, int8 [B, Hq, ceil(Lq/128), ceil(Lk/64)] (rows contiguous): non-zero = the 128 query
  // rows attend to the 64 keys; nullptr = dense
  const int8_t* block_mask;
  int64_t mask_sB, mask_sH;  // element strides of the two leading dims (0 broadcasts)
  int causal;  // 1: query row i attends to keys [0, i] only (on top of k_lens and the block mask), whatever Lq and Lk
  // scratch for workgroups cut into runs of key tiles (nullptr: never cut): per partial 256 rows x 128 fp32
  // accumulators, and per row its running maximum and row sum; room for kMaxSplitPartials partials
  float* split_o;
  float* split_ml;
  int split_first_wg, n_split;  // filled in by the launcher
  int wg_waves;  // 0: the launcher picks the workgroup shape; 4 or 8: forced (for measurements and tests)
  int d_out;     // channels of an output row that exist: 128, or 64 (head size 64 runs zero-padded to 128)
  int tile_skip; // 1: a wave leaves out the exponentials of a key tile whose probabilities would all be the zero code
                 // (same bits; pays on peaked attention, costs ~7 % where no tile qualifies); 0: every tile in full
};
constexpr int kMaxSplitPartials = 256;  // (workgroups beyond the last full round) x (runs each) never exceeds this
constexpr int kMinTilesPerSplit = 8;    // a run shorter than this does not repay its prologue
constexpr int kMaskBlkQ = 128;           // query rows per mask row (two per workgroup)
constexpr int kSparseMaxKeyTiles = 2048; // key tiles per head with a block mask or causal masking (tile list lives in LDS)
hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t s);
// Which of `n_wg` dense workgroups the launcher cuts into runs of key tiles on the current device, and into how
// many: workgroups [*first_wg, n_wg) into *runs each; *runs == 0 means none.
void plan_key_split(int n_wg, int nkb, int* first_wg, int* runs);

}  // namespace ksana_sage
