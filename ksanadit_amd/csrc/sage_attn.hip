// Fused quantized attention for gfx950 (MI355X): INT8 QK^T and FP8 PV on MFMA, fp32 online
// softmax in registers.
//
// Work split.  One workgroup = 8 waves = 256 query rows of one (batch, head); each wave owns
// 32 query rows for the whole key loop.  Keys are consumed in tiles of 64 rows (= one int8
// K scale block; Q scales are per row, i.e. per lane), K and V^T tiles are copied asynchronously (global_load ... lds) into an 8-deep LDS ring shared by the 8 waves.
// Two waves share a SIMD, so one wave's softmax (VALU) overlaps the other's MFMAs.
//
// Fragment algebra (32x32 MFMA, lane l: l32 = l % 32, hh = l / 32):
//   S^T = K . Q^T   v_mfma_i32_32x32x32_i8   A = K rows, B = Q rows; both read 16 bytes at channel
//                   offset 32*s + 16*hh, so the contraction order is the same on both sides.
//                   Accumulator register r of sub-tile t holds key 32*t + 8*(r/4) + 4*hh + r%4
//                   for query l32: a lane owns ONE query column -> row max / row sum are
//                   register reductions plus a single lane<->lane+32 exchange.
//   O^T = V^T . P^T v_mfma_f32_32x32x64_f8f6f4   B = P packed to e4m3 straight from the S^T
//                   registers (byte 16*t + r); A = V^T tile whose bytes the quantizer already
//                   stored in that same key order, so P never goes through LDS.
//
// The int32 accumulators start at the bit pattern of 1.5 * 2^23 ("magic"): the result read
// as fp32 IS 12582912 + dot exactly (|dot| <= 127*127*128 < 2^22), which removes the
// int->float conversion from the softmax: p = exp2(fma(acc_as_float, sc, c)).
#include "sage_kernels.h"

#include <atomic>
#include <type_traits>

#include "../../include/ksana_sage_hip.h"

namespace ksana_sage {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Two shapes of workgroup: 8 waves = 256 query rows with an 8-stage tile ring (one workgroup holds a compute unit:
// every K/V tile copied serves 256 rows), and 4 waves = 128 query rows with a 4-stage ring, two of which share a
// compute unit - they run out of step, so one's prologue and epilogue hide under the other's key loop (what short key
// sequences need), and a workgroup is exactly one row of a block mask.
template <int kW>
struct WgShape {
  static_assert(kW == 8 || kW == 4, "workgroups of 8 or 4 waves");
  static constexpr int kThreads = kW * 64;
  static constexpr int kRows = kW * 32;                // query rows per workgroup
  static constexpr int kStages = kW == 8 ? 8 : 4;      // LDS ring (power of two): tiles j-1 .. j+kAhead live at step j
  static constexpr int kAhead = kW == 8 ? 4 : 2;       // global -> LDS copies are issued this many tiles ahead
  static constexpr int kCopies = 2 * (8 / kW);         // 1 KiB copy instructions per wave and tile (K and V^T halves)
  static constexpr int kRingBytes = kStages * 2 * kTileBytes;
  // The 4-wave shape keeps K tiles and V^T tiles in two rings of kStages slots each (same memory).  A K tile is
  // read one step BEFORE the step of its probabilities and its V^T tile one step AFTER, so in one ring of whole
  // tiles two K halves are always dead; in its own ring K can be requested kStages tiles ahead instead of two.
  // That matters where tiles miss the L2 (block masks): with two tiles ahead and every copy awaited at the end of the
  // step it was issued in, a copy has one step (about a microsecond) to arrive; now it has three.
  static constexpr bool kTwoRings = kW == 4;
  static constexpr int kAheadK = kTwoRings ? kStages : kAhead;
  // copies that may still be in flight at the barrier that ends a step: those of the newest (kAhead - 2) tiles in
  // one ring; with two rings everything issued in this step and the one before
  static constexpr int kInFlight = kTwoRings ? 2 * kCopies : kCopies * (kAhead - 2);
};
constexpr int kMagicI = 0x4B400000;       // bits of 12582912.0f = 1.5 * 2^23: fp32 values are 1 apart there
constexpr float kMagicF = 12582912.0f;
// Head size 64 runs on rows whose upper 64 channels are zeros before the Hadamard transform - and a copy of the lower
// 64 after it (H128 [x; 0] = [H64 x; H64 x]): the dot product over 128 channels is twice the one over the lower 64.
// The kernel then multiplies the lower half only and starts its accumulators at 1.5 * 2^24, where fp32 values are 2
// apart: the bits read as fp32 are 25165824 + 2 * dot, the full product, with no instruction spent on the doubling
// (|dot| <= 127 * 127 * 64 < 2^21).
constexpr int kMagicI2 = 0x4BC00000;      // bits of 25165824.0f = 1.5 * 2^24
constexpr float kMagicF2 = 25165824.0f;
// P is scaled by 2^6 before the e4m3 cast, and the reference point of a row (its "running maximum") is moved only when
// a tile's maximum exceeds it by more than kLazyMax octaves: probabilities then reach 2^(6 + 2.7) = 416 < 448, the
// largest e4m3 value, and the accumulators are rescaled in a few per cent of the steps instead of up to half of them
// (rows of flat attention set a new maximum every few tiles, by small amounts).  An e4m3 rounding does not depend on
// the power of two in front, so the result differs only where probabilities fall off the subnormal end, 2^-15 of the
// reference point.
// The piecewise-linear path keeps 2^8 and moves the reference point at every new maximum: its code formula is wrong
// for the subnormal codes (it fades them linearly), which must stay 2^-14 below the true maximum to be harmless.
constexpr float kPShift = 6.0f, kPShiftPwl = 8.0f;
constexpr float kLazyMax = 2.7f, kLazyMaxPwl = 0.0f;
constexpr int kStageBytes = 2 * kTileBytes;  // K tile + V tile
constexpr int kSparseMaxKeyTiles4 = 2048;    // 4-wave workgroups keep their tile list as 16-bit entries so that two fit a compute unit
constexpr int kMaxKeyTiles = 4096;           // K scales of one head are kept in LDS: Lk <= 262144
constexpr int kShortKeyTiles = 16;           // dense calls with at most this many key tiles (Lk <= 1024) take 4-wave workgroups
constexpr int kMidKeyTiles = 96;             // ... and up to this many (Lk <= 6144) when their 256-row grid fills the chip at least once
constexpr int kShortMaxKeyTiles = 2048;      // the most key tiles a dense 4-wave workgroup can hold scales for

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 16 bytes per lane from global memory straight into LDS at `lds_dst + 16 * lane` (lds_dst is
// wave-uniform).  Written as inline assembly on purpose: the compiler's wait-count model treats
// the builtin form as a possible LDS access through the flat path and from then on waits for
// ALL outstanding LDS reads before every use (lgkmcnt(0)), which serialises the operand
// prefetch.  The copy is tracked by hand instead (vmcnt, see tile_barrier).
// The global address is a wave-uniform base (scalar registers) plus a 32-bit per-lane offset.
// M0 is written and named as clobbered; the compiler remarks that M0 is a register it reserves (it re-materialises
// M0 before each of its own uses and never keeps a value live in it), which is the behaviour relied on here.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_copy16(const void* gbase, unsigned lane_off, const void* lds_dst) {
  const unsigned lds_off = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)lds_dst;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_off), "v"(lane_off), "s"(gbase)
               : "memory", "m0");
}
#pragma clang diagnostic pop

// Opaque use+def at this program point: keeps the optimizer from sinking the computation of
// `x` into a later basic block (it emits no instruction).
template <typename T>
__device__ __forceinline__ void pin(T& x) {
  asm volatile("" : "+v"(x));
}

template <int DT>
__device__ __forceinline__ uint2 half4(float a, float b, float c, float d) {
  uint32_t lo, hi;
  if constexpr (DT == KSANA_SAGE_BF16) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    b2 x = {(__bf16)a, (__bf16)b}, y = {(__bf16)c, (__bf16)d};
    lo = __builtin_bit_cast(uint32_t, x);
    hi = __builtin_bit_cast(uint32_t, y);
  } else {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 x = {(_Float16)a, (_Float16)b}, y = {(_Float16)c, (_Float16)d};
    lo = __builtin_bit_cast(uint32_t, x);
    hi = __builtin_bit_cast(uint32_t, y);
  }
  return make_uint2(lo, hi);
}
template <int DT>
__device__ __forceinline__ void store4(uint16_t* dst, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(dst) = half4<DT>(a, b, c, d);
}

// S^T tile (64 keys x 32 queries) of one wave: two 32-key sub-tiles, kG 32-channel steps (the channel groups that
// hold data: 4, or 2 for head size 64, whose upper 64 channels are zeros on both sides).
template <int kG>
__device__ __forceinline__ void qk_tile(const uint8_t* k_stage, int lane, const v4i (&qf)[4], const v16i& magic,
                                        v16i (&acc)[2]) {
  acc[0] = magic;
  acc[1] = magic;
#pragma unroll
  for (int s = 0; s < kG; ++s) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const v4i kf = *reinterpret_cast<const v4i*>(k_stage + ((t * 4 + s) * 64 + lane) * 16);
      acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[s], acc[t], 0, 0, 0);
    }
  }
}

// kSplit: the workgroup takes one of `p.n_split` equal runs of key tiles of its (head, query block) and leaves
// unnormalised accumulators, running maxima and row sums in the workspace for sage_attn_merge_kernel.  Used for
// the workgroups beyond the last full round of the chip, which would otherwise hold it for a whole round alone.
// kG: 32-channel groups the matrix instructions cover - 4, or 2 when the head size is 64 (rows run zero-extended to
// 128 channels and the operands keep their layout; see kMagicI2 for what is left out and why nothing is lost; the
// result equals the full-width code's up to the rounding of one constant in the exponent).
template <int DT, bool kPwlExp, bool kSparse, bool kSplit, int kW, bool kTileSkip, int kG, bool kCausal>
__global__ __launch_bounds__(kW * 64, kW == 8 ? 1 : 2) void sage_attn_fwd_kernel(const AttnParams p, int n_qwg,
                                                                                   int n_wg, int wg_per_xcd) {
  static_assert(!(kSparse && kSplit), "the key split is built for the dense loop only");
  static_assert(kSparse || !kCausal, "causal calls run through the tile list");
  // kCausal == false: the caller vouches that p.causal is 0, and everything that serves the diagonal (the per-wave
  // last tile, 32 lane masks held in scalar registers, the selects that blank a wave's probabilities past its rows)
  // is compiled out of the key loop
  const bool causal = kCausal && p.causal;
  static_assert(!kSplit || kW == 8, "the key split is built for 256-row workgroups");
  using Shape = WgShape<kW>;
  constexpr int kThreadsAttn = Shape::kThreads, kRowsWg = Shape::kRows, kStages = Shape::kStages, kAhead = Shape::kAhead;
  constexpr int kListMax = kW == 8 ? kSparseMaxKeyTiles : kSparseMaxKeyTiles4;
  static_assert(!(kTileSkip && kPwlExp), "the piecewise-linear code formula has its own zero point: no tiles are skipped there");
  static_assert(kG == 4 || kG == 2, "128 channels, or 64 zero-extended");
  constexpr int kMagicBits = kG == 4 ? kMagicI : kMagicI2;
  constexpr float kMagicVal = kG == 4 ? kMagicF : kMagicF2;
  int wg, split = 0;
  if constexpr (kSplit) {
    const int item = blockIdx.x / p.n_split;
    split = blockIdx.x - item * p.n_split;
    wg = p.split_first_wg + item;
  } else {
    // Consecutive workgroup ids land on consecutive XCDs (8 per chip, one L2 each).  Give every
    // XCD a contiguous run of (head, query block) pairs so the workgroups that stream the same
    // K/V tiles share one L2.
    const int xcd = blockIdx.x & 7;
    wg = xcd * wg_per_xcd + (blockIdx.x >> 3);
    if (wg >= n_wg) return;
  }
  const int bh = wg / n_qwg;
  int qwg = wg - bh * n_qwg;
  // causal: the later a query block, the more key tiles it walks - start the long ones first
  if (kSparse && causal) qwg = n_qwg - 1 - qwg;
  const int b = bh / p.Hq, h = bh - b * p.Hq;
  const int bhk = b * p.Hkv + h / (p.Hq / p.Hkv);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction: keep it scalar
  const int l32 = lane & 31, hh = lane >> 5;
  const int q0 = qwg * kRowsWg + wave * 32;
  // query rows [0, lq) of this batch take part: all of them, or the caller's per-batch count; the rows from lq up
  // to Lq exist in the output and are written as zeros
  int lq = p.Lq;
  if (p.q_lens != nullptr) lq = min(max(p.q_lens[b], 0), p.Lq);  // uniform: a scalar load
  const bool active = q0 < lq;  // wave-uniform; inactive waves only help move tiles

  // keys [0, lk) of this batch take part: all of them, or the caller's per-batch count
  int lk = p.Lk;
  if (p.k_lens != nullptr) lk = min(max(p.k_lens[b], 0), p.Lk);  // uniform: a scalar load
  auto write_zero_rows = [&]() {  // softmax over no key: the output rows are defined as zeros
    const int q = q0 + l32;
    if (q < p.Lq && 64 * hh < p.d_out) {
      uint4* orow = reinterpret_cast<uint4*>(p.o.ptr + b * p.o.sB + (int64_t)q * p.o.sL + h * p.o.sH + 64 * hh);
#pragma unroll
      for (int i = 0; i < 8; ++i) orow[i] = make_uint4(0, 0, 0, 0);
    }
  };
  int tile0 = 0;  // first key tile of this workgroup's run
  if constexpr (kSplit) {
    const int tiles = (lk + kBlkK - 1) / kBlkK;
    const int per = (tiles + p.n_split - 1) / p.n_split;
    tile0 = split * per;
    const int tile1 = min(tiles, tile0 + per);
    if (tile0 >= tile1 || qwg * kRowsWg >= lq) {  // nothing in this run (few tiles, a batch entry without keys, or no query row): an empty partial
      if (active) {
        const int row = wave * 32 + l32;
        float* po = p.split_o + ((int64_t)blockIdx.x * kAttnQPerWg + row) * kD + 64 * hh;
#pragma unroll
        for (int i = 0; i < 16; ++i) reinterpret_cast<float4*>(po)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (hh == 0) reinterpret_cast<float2*>(p.split_ml)[(int64_t)blockIdx.x * kAttnQPerWg + row] = make_float2(-INFINITY, 0.f);
      }
      return;
    }
    lk = min(lk, tile1 * kBlkK) - tile0 * kBlkK;  // from here on the run is the whole key sequence
  } else {
    if (lk == 0 || qwg * kRowsWg >= lq) {  // no key, or none of the workgroup's rows takes part
      write_zero_rows();
      return;
    }
  }

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // ---- Q fragments (B operand), 4 channel steps --------------------------------------
  v4i qf[4];
  float qs = 0.0f;
  if (active) {
    const int8_t* qrow = p.q_i8 + ((int64_t)bh * p.lq_pad + q0 + l32) * kD + 16 * hh;
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = s < kG ? *reinterpret_cast<const v4i*>(qrow + 32 * s) : v4i{0, 0, 0, 0};
    qs = p.q_scale[(int64_t)bh * p.lq_pad + q0 + l32];  // one scale per query row = per lane
  } else {
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = v4i{0, 0, 0, 0};
  }

  v16f oacc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
  float m_run = -INFINITY;  // running row max (log2 domain) of query l32
  // Row sums come from the matrix pipe too: an all-ones A operand (e4m3 1.0 = 0x38) makes every
  // row of `lacc` the sum over keys of the SAME e4m3-rounded P the numerator uses.  Only
  // register 0 is read (all 16 hold the same value), so only it is rescaled.
  v16f lacc;
#pragma unroll
  for (int r = 0; r < 16; ++r) lacc[r] = 0.0f;
  // eight registers on purpose: left as one constant the compiler keeps a single copy and rebuilds
  // the 8-register operand with seven moves in every step
  v8i ones;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    int one4 = 0x38383838;
    pin(one4);
    ones[r] = one4;
  }

  // kept opaque so the 16 registers stay resident instead of being rebuilt from constants
  // (8 moves) at every tile
  v16i magic;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int m = kMagicBits;
    pin(m);
    magic[r] = m;
  }

  const uint8_t* k_src = reinterpret_cast<const uint8_t*>(p.k_tiles) + ((int64_t)bhk * p.nkb + tile0) * kTileBytes;  // uniform
  const uint8_t* v_src = p.v_tiles + ((int64_t)bhk * p.nkb + tile0) * kTileBytes;
  const float* ks_ptr = p.k_scale + (int64_t)bhk * p.nkb + tile0;
  const int nkb = (lk + kBlkK - 1) / kBlkK;  // tiles this batch uses; p.nkb stays the per-head stride
  // K scales live in LDS behind the ring: a per-tile global load would share the in-order
  // vmcnt queue with the tile copies and stall on all of them
  // behind the ring: the head's V scales and V means (2 x 128 floats, read by the epilogue), then its K scales
  float* s_vs = reinterpret_cast<float*>(smem + kStages * kStageBytes);
  float* s_ks = s_vs + 2 * kD;

  // ---- block mask: the workgroup's list of key tiles ---------------------------------------
  // A mask row covers 128 query rows, a workgroup two of them (waves 0-3, waves 4-7).  Wave 0
  // compacts, in key order, the tiles either row asks for into LDS: entry = tile | row-0 flag
  // << 16 | row-1 flag << 17.  The loop below then walks list positions instead of tile
  // numbers; a wave whose row does not ask for a tile zeroes its probabilities for it and
  // leaves its running maximum alone, so the result is exactly the masked softmax.
  // Causal attention (key <= query row) runs through the same list: the workgroup lists the tiles up
  // to the one holding its last row, a wave leaves alone the tiles past its own last row, and the one
  // tile that straddles its rows' diagonal is masked element by element.
  // (one mask row per 4-wave workgroup: an entry is the tile number and fits 16 bits; with two mask rows per
  // workgroup it carries their two flags above the number)
  using ListEntry = typename std::conditional<kW == 4, uint16_t, int>::type;
  ListEntry* s_list = reinterpret_cast<ListEntry*>(s_ks + kListMax);
  int* s_count = reinterpret_cast<int*>(s_list + kListMax);
  int n_tiles = nkb;  // loop length: list entries with a mask, key tiles without
  // a wave's 32 rows start at a multiple of 32, so exactly one 64-key tile holds their diagonal
  const int my_last = (kSparse && causal) ? (q0 >> 6) : 0x7fffffff;
  if constexpr (kSparse) {
    if (wave == 0) {
      const int nqm = (p.Lq + kMaskBlkQ - 1) / kMaskBlkQ;
      const bool masked = p.block_mask != nullptr;
      constexpr int kMaskRows = kRowsWg / kMaskBlkQ;  // mask rows a workgroup covers: 2 or 1
      const int8_t* m0 = masked ? p.block_mask + b * p.mask_sB + h * p.mask_sH + (int64_t)(kMaskRows * qwg) * p.nkb : nullptr;
      const bool two = kMaskRows == 2 && 2 * qwg + 1 < nqm;
      const int wg_tiles = causal ? min(nkb, ((qwg * kRowsWg + kRowsWg - 1) >> 6) + 1) : nkb;
      int base = 0;
      // eight chunks of 64 tiles at a time: their mask bytes are requested together, so a list of 512 tiles costs
      // one memory latency instead of eight
      for (int jb = 0; jb < wg_tiles; jb += 512) {
        int8_t b0[8], b1[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int j = jb + 64 * c + lane;
          b0[c] = b1[c] = 1;
          if (masked && j < wg_tiles) {
            b0[c] = m0[j];
            if (two) b1[c] = m0[p.nkb + j];
          }
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int j = jb + 64 * c + lane;
          if (jb + 64 * c >= wg_tiles) break;  // uniform
          int f0 = 0, f1 = 0;
          if (j < wg_tiles) {
            f0 = b0[c] != 0;
            f1 = two && b1[c] != 0;
          }
          const bool keep = (f0 | f1) != 0;
          const unsigned long long bal = __ballot(keep);
          const int pre = __builtin_amdgcn_mbcnt_hi((unsigned)(bal >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)bal, 0));
          if (keep) s_list[base + pre] = static_cast<ListEntry>(kW == 4 ? j : (j | (f0 << 16) | (f1 << 17)));
          base += __popcll(bal);
        }
      }
      if (lane == 0) *s_count = base;
    }
    __syncthreads();
    n_tiles = __builtin_amdgcn_readfirstlane(*s_count);
    if (n_tiles == 0) {  // neither mask row allows any key
      write_zero_rows();
      return;
    }
  }
  // the head's K scales (in loop order: tile order, or the list's) and V scales / means go to LDS, once the first
  // tile copies are on their way, so that the loads' latencies overlap
  auto fill_scales = [&]() {
    // the V value is requested first and stored last: written where it is loaded, its load would only go out after
    // the K scales' loads had been awaited - a second memory latency in every workgroup's set-up
    float vsm = 0.0f;
    if (tid < 2 * kD) vsm = tid < kD ? p.v_scale[(int64_t)bhk * kD + tid] : p.v_mean[(int64_t)bhk * kD + tid - kD];
    if constexpr (kSparse) {
      for (int i = tid; i < n_tiles; i += kThreadsAttn) s_ks[i] = ks_ptr[s_list[i] & 0xffff];
    } else {
      for (int i = tid; i < nkb; i += kThreadsAttn) s_ks[i] = ks_ptr[i];
    }
    if (tid < 2 * kD) s_vs[tid] = vsm;
  };
  // Causal calls: the list is in key order, so the entries this wave takes part in (tile <= the one on its diagonal)
  // are the first n_mine, and the diagonal tile, if listed, is the last of them.  Both are found once here; the key
  // loop then compares loop positions instead of looking list entries up.
  int n_mine = n_tiles, jdiag = -1;  // wave-uniform
  if constexpr (kSparse) {
    if (causal) {
      if (p.block_mask == nullptr) {  // the list is 0, 1, 2, ...
        n_mine = min(n_tiles, my_last + 1);
      } else {
        int cnt = 0;
        for (int j0 = 0; j0 < n_tiles; j0 += 64) {
          const int jx = j0 + lane;
          const bool le = jx < n_tiles && (s_list[jx] & 0xffff) <= my_last;
          cnt += __popcll(__ballot(le));
        }
        n_mine = cnt;
      }
      if (n_mine > 0 && (__builtin_amdgcn_readfirstlane(s_list[n_mine - 1]) & 0xffff) == my_last) jdiag = n_mine - 1;
    }
  }
  // key tile behind loop position jj, and whether this wave's mask row asks for it
  auto tile_of = [&](int jj) -> int {
    if constexpr (kSparse) return __builtin_amdgcn_readfirstlane(s_list[jj]) & 0xffff;
    return jj;
  };
  auto mine_at = [&](int jj) -> bool {
    if constexpr (kSparse) {
      if constexpr (kW == 4 && !kCausal) return true;  // one mask row per workgroup: every listed tile is wanted
      if constexpr (kW == 4) return jj < n_mine;
      const int e = __builtin_amdgcn_readfirstlane(s_list[jj]);
      return ((e >> (16 + (wave >> 2))) & 1) != 0 && jj < n_mine;
    }
    return true;
  };
  // causal only: list position jj holds the tile on this wave's diagonal
  auto diag_at = [&](int jj) -> bool {
    if constexpr (kSparse && kCausal) return jj == jdiag;
    return false;
  };
  // scores of keys beyond the row's own position drop below every real score ...
  auto causal_half = [&](v16i blk, int t) -> v16i {
    // (pinned: the comparisons below are the same in every step, and hoisted out of the key loop they would sit in
    // 32 scalar register pairs for a block that runs once per wave)
    int row_local = (q0 & 63) + l32;
    pin(row_local);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      // all-ones where the key lies beyond the row
      const int beyond = (row_local - 4 * hh - (32 * t + 8 * (r >> 2) + (r & 3))) >> 31;
      blk[r] = (blk[r] & ~beyond) | ((kMagicBits - (1 << 22)) & beyond);
    }
    return blk;
  };
  auto causal_scores = [&](v16i (&blk)[2]) {
    blk[0] = causal_half(blk[0], 0);
    blk[1] = causal_half(blk[1], 1);
  };
  // ... and their probability bytes are cleared outright (code 0 is +0.0 in e4m3), so that a row
  // whose scale is zero does not count them either
  auto causal_probs = [&](v8i& pf) {
    int row_local = (q0 & 63) + l32;
    pin(row_local);
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      // bytes of the first min(max(n, 0), 4) keys of this dword stay
      const int n = min(max(row_local - 4 * hh - (32 * (w >> 2) + 8 * (w & 3)) + 1, 0), 4);
      const unsigned keep = n >= 4 ? 0xffffffffu : ((1u << (8 * n)) - 1u);
      pf[w] &= (int)keep;
    }
  };

  // ---- asynchronous tile copies: HBM/L2 -> LDS without passing through registers ----------
  // Each wave moves its 1 KiB slice of the K tile and of the V^T tile (lane i -> byte 16*i of
  // the slice).  Copies retire in issue order, so "at most 2*n outstanding" == "all but the
  // newest n tiles have landed".
  // keys >= lk live only in the last key tile, which (if the list holds it) is the last entry
  const bool has_tail = (lk & (kBlkK - 1)) != 0 && tile_of(n_tiles - 1) == nkb - 1;
  const int n_main = has_tail ? n_tiles - 1 : n_tiles;  // entries handled by the pipelined loop
  // LDS slot of a tile's K half / V^T half
  auto k_slot = [&](int tile) -> uint8_t* {
    if constexpr (Shape::kTwoRings) return smem + (tile & (kStages - 1)) * kTileBytes;
    return smem + (tile & (kStages - 1)) * kStageBytes;
  };
  auto v_slot = [&](int tile) -> uint8_t* {
    if constexpr (Shape::kTwoRings) return smem + (kStages + (tile & (kStages - 1))) * kTileBytes;
    return smem + (tile & (kStages - 1)) * kStageBytes + kTileBytes;
  };
  // clamped: past the end the last tile is copied again into a slot nobody reads any more,
  // which keeps the loop free of branches and the outstanding-copy count constant
  auto copy_tile_half = [&](const uint8_t* src, int jl, uint8_t* dst) {  // jl: key tile number, wave-uniform
#pragma unroll
    for (int c = 0; c < 8 / kW; ++c) {  // this wave's 1 KiB slices of the tile: slice c * kW + wave
      const int slice = c * kW + wave;
      lds_copy16(src + (int64_t)jl * kTileBytes, (unsigned)(slice * 64 + lane) * 16, dst + slice * 1024);
    }
  };
  auto copy_half = [&](const uint8_t* src, int tile, uint8_t* dst) {
    copy_tile_half(src, tile_of(min(tile, n_tiles - 1)), dst);
  };
  // With a tile list, the key tiles behind the loop positions whose copies the next steps issue are kept in scalar
  // registers: looked up in the step, a list entry costs an LDS read whose wait also drains the operand reads
  // requested just before it.  ahead[i] = tile at position j + kAhead + i for the step j about to run; a step
  // fetches the one entry that enters the window (position j + 1 + kAheadK) and takes it over at its end.
  constexpr int kWindow = Shape::kAheadK - kAhead + 1;
  int ahead[kWindow];
  if constexpr (kSparse) {
#pragma unroll
    for (int i = 0; i < kWindow; ++i) ahead[i] = tile_of(min(kAhead + i, n_tiles - 1));
  }
  // the copies of loop step j (step -1: nothing; the prologue below brings the first tiles in)
  auto issue_copy = [&](int j) {
    if constexpr (kSparse) {
      copy_tile_half(v_src, ahead[0], v_slot(j + kAhead));
      copy_tile_half(k_src, ahead[kWindow - 1], k_slot(j + Shape::kAheadK));
    } else {
      copy_half(v_src, j + kAhead, v_slot(j + kAhead));  // first: it is awaited first
      copy_half(k_src, j + Shape::kAheadK, k_slot(j + Shape::kAheadK));
    }
  };
  // wait until every copy except the newest Shape::kInFlight has landed, then meet the other waves.
  // Plain s_barrier: a fence here would drain ALL copies and undo the prefetch.
  auto tile_barrier = [&]() {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(Shape::kInFlight) : "memory");
  };

  // The compiler does not see the asynchronous copies in the memory-operation counter it models.  Every ordinary global
  // load of the set-up (Q fragments, scales) must therefore be known to have returned before the key loop starts:
  // left to itself the compiler would wait for "all but its n newest loads" at the first use of a loaded value
  // inside the loop, and drain the copies issued since.  The first copies go out first and everything is awaited
  // together.
  // The V^T slot of "tile -1" is read (times P = 0) by the first loop iteration: make it finite.
#pragma unroll
  for (int c = 0; c < 8 / kW; ++c)
    *reinterpret_cast<uint4*>(v_slot(-1) + (c * kThreadsAttn + tid) * 16) = make_uint4(0, 0, 0, 0);
  if constexpr (Shape::kTwoRings) {
#pragma unroll
    for (int t = 0; t < kAhead; ++t) copy_half(v_src, t, v_slot(t));
#pragma unroll
    for (int t = 0; t < Shape::kAheadK; ++t) copy_half(k_src, t, k_slot(t));
  } else {
#pragma unroll
    for (int t = 0; t < kAhead; ++t) {  // tile by tile: the oldest copies are the ones awaited
      copy_half(k_src, t, k_slot(t));
      copy_half(v_src, t, v_slot(t));
    }
  }
  fill_scales();
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the set-up's loads and, older than some of them, the copies
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  if (!active) {
    // same copy / barrier sequence as the active waves
    if constexpr (Shape::kTwoRings) __builtin_amdgcn_s_barrier();
    for (int j = 0; j < n_main; ++j) {
      // (looks the tiles up where they are needed: a wave without rows has nothing an LDS wait could hold up)
      copy_half(v_src, j + kAhead, v_slot(j + kAhead));
      copy_half(k_src, j + Shape::kAheadK, k_slot(j + Shape::kAheadK));
      tile_barrier();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (!kSplit) write_zero_rows();  // rows in [lq, Lq), if any (the merge kernel writes them for cut blocks)
    return;
  }

  auto scale_o = [&](float alpha) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
    lacc[0] *= alpha;
  };
  // max over the 16 keys one S^T register block holds for query l32, as two independent chains
  auto max8 = [&](const v16i& blk, int r0) {
    int m = max(max(blk[r0], blk[r0 + 1]), blk[r0 + 2]);
    m = max(max(m, blk[r0 + 3]), blk[r0 + 4]);
    m = max(max(m, blk[r0 + 5]), blk[r0 + 6]);
    return max(m, blk[r0 + 7]);
  };
  // this lane's maximum over a whole tile (32 of query l32's 64 keys)
  auto lane_max = [&](const v16i (&blk)[2]) {
    return max(max(max8(blk[0], 0), max8(blk[0], 8)), max(max8(blk[1], 0), max8(blk[1], 8)));
  };
  // new running max of query l32 given this lane's tile maximum; returns 2^(old max - new max)
  bool tile_is_nothing = false;  // set by update_max, per lane
  auto update_max = [&](int imax, float sc, float mneg) -> float {
    {
      // the other half of query l32's keys lives in lane l32 + 32
      int other = imax;
      const auto sw = __builtin_amdgcn_permlane32_swap(imax, other, false, false);
      imax = max(sw[0], sw[1]);
    }
    // the accumulator read as fp32 is magic + dot, so one fma gives sc * dot (mneg = -magic * sc)
    const float m_tile = __builtin_fmaf(__int_as_float(imax), sc, mneg);
    const float m_new = m_tile > m_run + (kPwlExp ? kLazyMaxPwl : kLazyMax) ? m_tile : m_run;  // -inf at the first tile: always taken
    const float alpha = fast_exp2(m_run - m_new);                     // exactly 1 where the reference point stays
    m_run = m_new;
    // Every probability of this row in this tile is below 2^(m_tile - m_run + shift).  Under 2^-10 (half the smallest
    // e4m3 subnormal; a tie goes to the even code, zero) each one converts to the zero code - taken with a margin of
    // one octave for the exponent's few units of rounding.
    tile_is_nothing = m_tile < m_run - (kPShift + 11.0f);
    return alpha;
  };
  // p = exp2(sc*dot - m_run + shift); the magic is folded into the constant c, which is off by
  // at most ~1.5 integer steps of the dot product
  auto p_of = [&](int acc_bits, float sc, float c) { return fast_exp2(__builtin_fmaf(__int_as_float(acc_bits), sc, c)); };
  // Four probabilities -> one dword of e4m3 codes (bytes in register order).
  //   exact:  p = exp2(x) on the transcendental unit, then the hardware e4m3 conversion;
  //   kPwlExp: the e4m3 CODE is computed directly, code = rne(8*x + 55.5) (saturating at 0): an
  //           e4m3 code is a 3-bit-mantissa logarithm, so this is exp2 with a piecewise-linear
  //           mantissa - two VALU slots per key instead of 3.5, no transcendental.  x <= 8.7 keeps
  //           the code <= 125, clear of the NaN code 127.
  auto pack4 = [&](int s0, int s1, int s2, int s3, float sc, float c) -> int {
    if constexpr (kPwlExp) {
      // here sc and c arrive pre-multiplied by 8, c with the +55.5 folded in
      unsigned w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s0), sc, c), 0, 0u);
      w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s1), sc, c), 1, w);
      w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s2), sc, c), 2, w);
      w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s3), sc, c), 3, w);
      return (int)w;
    } else {
      const float e0 = p_of(s0, sc, c), e1 = p_of(s1, sc, c), e2 = p_of(s2, sc, c), e3 = p_of(s3, sc, c);
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(e0, e1, __float_as_int(e0), false);  // both halves get written
      return __builtin_amdgcn_cvt_pk_fp8_f32(e2, e3, w, true);
    }
  };
  // O^T += V^T . P^T for one 32-channel slice
  auto pv_slice = [&](const uint8_t* vst, int dt, const v8i& pf) {
    const v4i lo = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 0) * 64 + lane) * 16);
    const v4i hi = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 1) * 64 + lane) * 16);
    const v8i vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    oacc[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf, oacc[dt], 0, 0, 0, 0, 0, 0);
  };
  // S^T chunk i of a step is (channel step i / 2, key half i % 2); the chunks of channel steps without data carry only
  // their share of the probabilities
  auto has_qk = [](int i) { return i >= 0 && i < 8 && (i >> 1) < kG; };

  v16i s_a[2], s_b[2];
  qk_tile<kG>(k_slot(0), lane, qf, magic, s_a);
  // two rings: step 0 requests K tile kStages into the slot of K tile 0, which every wave must have read by then
  if constexpr (Shape::kTwoRings) __builtin_amdgcn_s_barrier();
  if (diag_at(0)) causal_scores(s_a);
  int mx_cur = lane_max(s_a);  // this lane's maximum of the tile whose probabilities come next
  float ks_cur = s_ks[0];

  // Software pipeline, one key tile per step.  While this tile's probabilities are computed on
  // the VALU, the matrix pipe runs the S^T MFMAs of the NEXT tile and the PV MFMAs of the
  // PREVIOUS tile: every MFMA below is followed by the VALU work that hides it, LDS operands are
  // requested three MFMAs ahead, and sched_barrier pins that order.  The max reduction of the
  // next tile rides in the PV chunks, so a step starts with only the short finalisation.
  // Because PV lags one tile, so does the rescaling of O:
  //   at step j   O holds tiles <= j-2 relative to max m(j-2); alpha_prev = 2^(m(j-2) - m(j-1))
  //   step j      O *= alpha_prev (rare branch), then O += P(j-1) V(j-1), both relative to m(j-1)
  // LDS ring of 8 stages: tile j-1 (V), j (V next step), j+1 (K), j+2 .. j+4 (arriving).
  // probabilities of the previous and of the current tile swap registers every step, like s_a / s_b
  v8i pf_x = {0, 0, 0, 0, 0, 0, 0, 0}, pf_y = {0, 0, 0, 0, 0, 0, 0, 0};
  float alpha_prev = 1.0f;
  auto tile_step = [&](int j, v16i (&s_cur)[2], v16i (&s_nxt)[2], const v8i& pf_prev, v8i& pf) {
    const uint8_t* kst = k_slot(j + 1);
    const uint8_t* vst = v_slot(j - 1);
    auto k_frag = [&](int i) { return *reinterpret_cast<const v4i*>(kst + (((i & 1) * 4 + (i >> 1)) * 64 + lane) * 16); };
    auto v_frag = [&](int dt) {
      const v4i lo = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 0) * 64 + lane) * 16);
      const v4i hi = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 1) * 64 + lane) * 16);
      return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    v4i kf[4];
    v8i vf[4];
    // operands of the first three S^T MFMAs and the next tile's K scale: requested before the
    // dependent scalar work below, so their LDS latency is hidden behind it
    kf[0] = k_frag(0);
    kf[1] = k_frag(1);
    kf[2] = k_frag(2);  // (kG >= 2: chunks 0 .. 3 always exist)
    const float ks_nxt = s_ks[min(j + 1, n_tiles - 1)];
    int entering = 0;  // the list entry the next step's window gains; it arrives with the operands above
    if constexpr (kSparse) entering = s_list[min(j + 1 + Shape::kAheadK, n_tiles - 1)];
    const bool mine = mine_at(j);
    issue_copy(j);
    if (__any(alpha_prev < 1.0f)) scale_o(alpha_prev);
    // row sums of tile j-1: 64 matrix cycles that run under the max finalisation below
    lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pf_prev, lacc, 0, 0, 0, 0, 0, 0);
    const float sc = qs * ks_cur;
    const float mneg = -kMagicVal * sc;
    // a tile this wave's mask row does not ask for leaves the running maximum alone (wave-uniform
    // branch); its probabilities are zeroed where they are packed
    alpha_prev = mine ? update_max(mx_cur, sc, mneg) : 1.0f;
    // exponent of key r: x = sc*dot - m_run + shift, with the magic folded into the constant
    // (which is therefore off by at most ~1.5 integer steps of the dot product)
    const float c = ((kPwlExp ? kPShiftPwl : kPShift) - m_run) + mneg;
    const float scp = kPwlExp ? 8.0f * sc : sc;
    const float cp = kPwlExp ? __builtin_fmaf(8.0f, c, 55.5f) : c;
    int pm[4];
    // A tile whose scores lie more than 17 octaves under the reference point of every one of the wave's 32 rows: each
    // probability byte would be the zero code.  The wave then writes the zeros directly and leaves out the 64
    // exponentials and 32 conversions per lane (every chunk below tests this one scalar); the matrix work that
    // concerns the neighbouring tiles stays.  Same bits either way - the pvthreshold idea of the reference's sparse
    // kernel (sage_sla.py:237-253) with a threshold at which nothing changes.
    bool nothing = false;  // wave-uniform
    if constexpr (kTileSkip) nothing = mine && __all(tile_is_nothing);
    // The S^T chunks are short (a 32-cycle MFMA each): a wave inside them goes ahead of the SIMD's other
    // wave, which is usually in its PV chunks and has 64-cycle MFMAs to hide behind (measured: -1.3 %).
    __builtin_amdgcn_s_setprio(1);
    __builtin_amdgcn_sched_barrier(0);
    // 8 x [S^T MFMA of tile j+1 (32 matrix cycles) | 2 probabilities of tile j]
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int s = i >> 1, t = i & 1;
      if (i + 3 < 8) {
        if (has_qk(i + 3)) kf[(i + 3) & 3] = k_frag(i + 3);
      } else if (i + 3 - 8 < kG) {
        vf[i + 3 - 8] = v_frag(i + 3 - 8);
      }
      if (has_qk(i)) s_nxt[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i & 3], qf[s], s == 0 ? magic : s_nxt[t], 0, 0, 0);
      if constexpr (kPwlExp) {
        unsigned w = (i & 1) ? (unsigned)pf[i >> 1] : 0u;
        w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s_cur[0][2 * i]), scp, cp), (2 * i) & 3, w);
        w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(s_cur[0][2 * i + 1]), scp, cp), (2 * i + 1) & 3, w);
        int wi = (int)w;
        if (i & 1) pin(wi);
        pf[i >> 1] = wi;
      } else if (!nothing) {
        const float e0 = p_of(s_cur[0][2 * i], scp, cp), e1 = p_of(s_cur[0][2 * i + 1], scp, cp);
        if (i & 1) {
          int w = __builtin_amdgcn_cvt_pk_fp8_f32(e0, e1, pf[i >> 1], true);
          pin(w);
          pf[i >> 1] = w;
        } else {
          pf[i >> 1] = __builtin_amdgcn_cvt_pk_fp8_f32(e0, e1, __float_as_int(e0), false);  // both halves get written
        }
      } else {
        pf[i >> 1] = 0;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (kSparse) {  // rare, wave-uniform: the next tile is the one on this wave's diagonal
      if (j + 1 < n_tiles && diag_at(j + 1)) causal_scores(s_nxt);
    }
    __builtin_amdgcn_s_setprio(0);
    // 4 x [PV MFMA of tile j-1 (64 matrix cycles) | 4 probabilities of tile j | a quarter of
    // the max reduction of tile j+1, whose S^T MFMAs were issued at least one chunk ago]
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      if (dt == 0 && kG == 4) vf[3] = v_frag(3);
      if (dt < kG) oacc[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[dt], pf_prev, oacc[dt], 0, 0, 0, 0, 0, 0);
      int w = 0;
      if (!nothing) w = pack4(s_cur[1][4 * dt], s_cur[1][4 * dt + 1], s_cur[1][4 * dt + 2], s_cur[1][4 * dt + 3], scp, cp);
      pin(w);
      pf[4 + dt] = w;
      pm[dt] = max8(s_nxt[dt >> 1], (dt & 1) * 8);
      pin(pm[dt]);
      __builtin_amdgcn_sched_barrier(0);
    }
    mx_cur = max(max(pm[0], pm[1]), max(pm[2], pm[3]));
    ks_cur = ks_nxt;
    if constexpr (kSparse) {
#pragma unroll
      for (int i = 0; i + 1 < kWindow; ++i) ahead[i] = ahead[i + 1];
      ahead[kWindow - 1] = __builtin_amdgcn_readfirstlane(entering) & 0xffff;
      if (!mine) {  // wave-uniform and rare: a tile this wave's row does not take part in contributes nothing
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[i] = 0;
      }
      if (diag_at(j)) causal_probs(pf);
    }
    // after this barrier: tile j+2 is visible to every wave, and nobody reads tile j-1 any more
    tile_barrier();
  };

  {
    int j = 0;
    for (; j + 2 <= n_main; j += 2) {
      tile_step(j, s_a, s_b, pf_x, pf_y);
      tile_step(j + 1, s_b, s_a, pf_y, pf_x);
    }
    if (j < n_main) tile_step(j, s_a, s_b, pf_x, pf_y);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may outlive the workgroup's LDS
  if constexpr (Shape::kTwoRings) {
    // the peeled last tile's V^T half was requested two steps ago; the loop's last barrier vouches only for copies
    // three steps old, so the waves meet once more after each has seen its own copies land (uniform condition)
    if (has_tail) __builtin_amdgcn_s_barrier();
  }
  if (n_main > 0) {  // drain: PV of the last pipelined tile
    scale_o(alpha_prev);
    const uint8_t* vst = v_slot(n_main - 1);
    const v8i pf_last = (n_main & 1) ? pf_y : pf_x;  // written by the last step
#pragma unroll
    for (int dt = 0; dt < kG; ++dt) pv_slice(vst, dt, pf_last);
    lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pf_last, lacc, 0, 0, 0, 0, 0, 0);
  }
  if (has_tail && mine_at(n_tiles - 1)) {  // ragged last tile, not pipelined: mask keys >= lk
    const int j = nkb - 1, jj = n_tiles - 1;
    v16i (&s_cur)[2] = (n_main & 1) ? s_b : s_a;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = j * kBlkK + 32 * t + 8 * (r >> 2) + 4 * hh + (r & 3);
        if (key >= lk) s_cur[t][r] = kMagicBits - (1 << 22);  // below every real score
      }
    const float sc = qs * s_ks[jj];
    const float mneg = -kMagicVal * sc;
    scale_o(update_max(lane_max(s_cur), sc, mneg));
    const float c = ((kPwlExp ? kPShiftPwl : kPShift) - m_run) + mneg;
    const float scp = kPwlExp ? 8.0f * sc : sc;
    const float cp = kPwlExp ? __builtin_fmaf(8.0f, c, 55.5f) : c;
    v8i pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int w = pack4(s_cur[t][4 * g], s_cur[t][4 * g + 1], s_cur[t][4 * g + 2], s_cur[t][4 * g + 3], scp, cp);
        // zero the bytes of keys at or beyond lk (code 0 is +0.0 in e4m3)
        unsigned keep = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = j * kBlkK + 32 * t + 8 * g + 4 * hh + i;
          if (key < lk) keep |= 0xffu << (8 * i);
        }
        pf[4 * t + g] = w & (int)keep;
      }
    if (diag_at(jj)) causal_probs(pf);
    const uint8_t* vst = v_slot(jj);
#pragma unroll
    for (int dt = 0; dt < kG; ++dt) pv_slice(vst, dt, pf);
    lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pf, lacc, 0, 0, 0, 0, 0, 0);
  }

  if constexpr (kSplit) {
    // partial result of this run of keys: O^T and the row sum relative to the run's own maximum
    const int row = wave * 32 + l32;
    float* po = p.split_o + ((int64_t)blockIdx.x * kAttnQPerWg + row) * kD;
#pragma unroll
    for (int dt = 0; dt < kG; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<float4*>(po + 32 * dt + 8 * g + 4 * hh) =
            make_float4(oacc[dt][4 * g + 0], oacc[dt][4 * g + 1], oacc[dt][4 * g + 2], oacc[dt][4 * g + 3]);
    if (hh == 0) reinterpret_cast<float2*>(p.split_ml)[(int64_t)blockIdx.x * kAttnQPerWg + row] = make_float2(m_run, lacc[0]);
    return;
  }
  // ---- epilogue: O = O^T / rowsum * v_scale (+ the V mean), written [B, Lq, H, D] ---------------
  // A lane holds its query row in pieces of four channels; stored as they are, every store instruction would
  // touch 32 rows with 16 bytes each.  The rows go through LDS instead (the tile ring is free once every wave is
  // past its last tile) and leave as whole 256-byte rows, 16 bytes per lane.
  const int q = q0 + l32;
  // zero for a mask row that allows none of its keys (an empty sum, not 0/0) and for rows at or beyond lq
  const float inv_l = ((!kSparse || lacc[0] > 0.0f) && q < lq) ? 1.0f / lacc[0] : 0.0f;
  // the channel means the V quantizer took off come back here (rows of P sum to one); they are zeros without V
  // smoothing, and a row that saw no key stays zero
  const float keep_mean = inv_l != 0.0f ? 1.0f : 0.0f;
  constexpr int kPitch = 2 * kD + 16;  // bytes per staged row: 16 bytes of padding spread the rows over the banks
  // The lane's 16 quadruples of V scales are requested together and ahead of the barrier (the score registers are
  // free by now); read one quadruple at a time where they are used, every one of the 16 groups below would start
  // with an LDS round trip of its own.  Without V smoothing the means are all zero - seen here by the wave as a
  // whole - and their products and sums are left out (a zero output may then keep a minus sign it used to lose).
  const float4* vs4 = reinterpret_cast<const float4*>(s_vs);
  const float4* vm4 = reinterpret_cast<const float4*>(s_vs + kD);
  float4 s4a[16];
#pragma unroll
  for (int i = 0; i < 4 * kG; ++i) s4a[i] = vs4[(32 * (i >> 2) + 8 * (i & 3) + 4 * hh) >> 2];
  const float2 mm = reinterpret_cast<const float2*>(s_vs + kD)[lane];
  const bool has_mean = __any(mm.x != 0.0f || mm.y != 0.0f);  // wave-uniform
  __syncthreads();  // waves that ended early (no query rows) do not count
  uint8_t* stage = smem + wave * (32 * kPitch);
  if (!has_mean) {
#pragma unroll
    for (int i = 0; i < 4 * kG; ++i) {
      const int dt = i >> 2, g = i & 3;
      const int d = 32 * dt + 8 * g + 4 * hh;
      const float4 s4 = s4a[i];
      *reinterpret_cast<uint2*>(stage + l32 * kPitch + 2 * d) =
          half4<DT>(oacc[dt][4 * g + 0] * inv_l * s4.x, oacc[dt][4 * g + 1] * inv_l * s4.y,
                    oacc[dt][4 * g + 2] * inv_l * s4.z, oacc[dt][4 * g + 3] * inv_l * s4.w);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4 * kG; ++i) {
      const int dt = i >> 2, g = i & 3;
      const int d = 32 * dt + 8 * g + 4 * hh;
      const float4 s4 = s4a[i];
      const float4 m4 = vm4[d >> 2];
      *reinterpret_cast<uint2*>(stage + l32 * kPitch + 2 * d) =
          half4<DT>(oacc[dt][4 * g + 0] * inv_l * s4.x + m4.x * keep_mean, oacc[dt][4 * g + 1] * inv_l * s4.y + m4.y * keep_mean,
                    oacc[dt][4 * g + 2] * inv_l * s4.z + m4.z * keep_mean, oacc[dt][4 * g + 3] * inv_l * s4.w + m4.w * keep_mean);
    }
  }
  // LDS serves one wave's accesses in order: the reads below see the writes above
  uint16_t* obase = p.o.ptr + b * p.o.sB + h * p.o.sH;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int idx = i * 64 + lane, r = idx >> 4, c = idx & 15;  // row r of the wave, 16-byte piece c of it
    const uint4 piece = *reinterpret_cast<const uint4*>(stage + r * kPitch + 16 * c);
    if (q0 + r < p.Lq && 8 * c < p.d_out && 8 * c < 32 * kG) *reinterpret_cast<uint4*>(obase + (int64_t)(q0 + r) * p.o.sL + 8 * c) = piece;
  }
}

// Combines the partial results of the key runs: for every query row the run maxima are brought to a common one,
// then O = sum_i O_i 2^(m_i - m), l = sum_i l_i 2^(m_i - m), and the usual last step follows.
// grid = (items, 32), 256 threads: a thread owns one row and four channels of a 8-row slab.
template <int DT>
__global__ __launch_bounds__(256) void sage_attn_merge_kernel(const AttnParams p, int n_qwg) {
  const int item = blockIdx.x, wg = p.split_first_wg + item;
  const int bh = wg / n_qwg, qwg = wg - bh * n_qwg;
  const int b = bh / p.Hq, h = bh - b * p.Hq;
  const int bhk = b * p.Hkv + h / (p.Hq / p.Hkv);
  const int row = blockIdx.y * 8 + (threadIdx.x >> 5), d = (threadIdx.x & 31) * 4;
  const int q = qwg * kAttnQPerWg + row;
  if (q >= p.Lq || d >= p.d_out) return;
  uint16_t* orow = p.o.ptr + b * p.o.sB + (int64_t)q * p.o.sL + h * p.o.sH;
  if (p.q_lens != nullptr && q >= min(max(p.q_lens[b], 0), p.Lq)) {  // a row that does not take part: zeros
    *reinterpret_cast<uint2*>(orow + d) = make_uint2(0, 0);
    return;
  }
  const float2* ml = reinterpret_cast<const float2*>(p.split_ml) + (int64_t)item * p.n_split * kAttnQPerWg + row;
  const float* po = p.split_o + ((int64_t)item * p.n_split * kAttnQPerWg + row) * kD + d;
  float m = -INFINITY;
  for (int s = 0; s < p.n_split; ++s) m = fmaxf(m, ml[(int64_t)s * kAttnQPerWg].x);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float l = 0.0f;
  for (int s = 0; s < p.n_split; ++s) {
    const float2 e = ml[(int64_t)s * kAttnQPerWg];
    if (e.y == 0.0f) continue;  // an empty run (its maximum is -inf)
    const float w = fast_exp2(e.x - m);
    const float4 o = *reinterpret_cast<const float4*>(po + (int64_t)s * kAttnQPerWg * kD);
    acc.x += o.x * w, acc.y += o.y * w, acc.z += o.z * w, acc.w += o.w * w;
    l += e.y * w;
  }
  const float inv_l = l > 0.0f ? 1.0f / l : 0.0f;
  const float keep_mean = l > 0.0f ? 1.0f : 0.0f;
  const float4 s4 = *reinterpret_cast<const float4*>(p.v_scale + (int64_t)bhk * kD + d);
  const float4 m4 = *reinterpret_cast<const float4*>(p.v_mean + (int64_t)bhk * kD + d);
  store4<DT>(orow + d, acc.x * inv_l * s4.x + m4.x * keep_mean, acc.y * inv_l * s4.y + m4.y * keep_mean,
             acc.z * inv_l * s4.z + m4.z * keep_mean, acc.w * inv_l * s4.w + m4.w * keep_mean);
}

// dynamic LDS of one instantiation: tile ring + K scales (+ the tile list and its length with a mask or causal)
template <bool kSparse, int kW>
constexpr size_t max_lds() {
  return kSparse ? WgShape<kW>::kRingBytes + 1024 + (kW == 8 ? kSparseMaxKeyTiles * 8 : kSparseMaxKeyTiles4 * 6) + 1024
                 : WgShape<kW>::kRingBytes + 1024 + (kW == 8 ? kMaxKeyTiles : kShortMaxKeyTiles) * 4;
}

template <int DT, bool kPwlExp, bool kSparse, bool kSplit, int kW, bool kCausal, bool kTileSkip = false, int kG = 4>
hipError_t launch_variant(const AttnParams& p, dim3 grid, size_t lds, int n_qwg, int n_wg, int wg_per_xcd,
                          hipStream_t s) {
  // more than 64 KiB of dynamic LDS has to be requested per kernel, once per device
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> requested[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  if (!requested[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sage_attn_fwd_kernel<DT, kPwlExp, kSparse, kSplit, kW, kTileSkip, kG, kCausal>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)max_lds<kSparse, kW>());
    if (e != hipSuccess) return e;
    requested[dev].store(true, std::memory_order_release);
  }
  sage_attn_fwd_kernel<DT, kPwlExp, kSparse, kSplit, kW, kTileSkip, kG, kCausal><<<grid, dim3(kW * 64), lds, s>>>(p, n_qwg, n_wg, wg_per_xcd);
  return hipGetLastError();
}

// the (dtype, exp2 form, tile skip) instantiations behind one (mask, split, workgroup shape) choice
template <bool kSparse, bool kSplit, int kW, bool kCausal = false>
hipError_t launch_shape(const AttnParams& p, dim3 grid, size_t lds, int n_qwg, int n_wg, int wg_per_xcd, hipStream_t s) {
  const bool bf16 = p.o.dtype == KSANA_SAGE_BF16;
  // head size 64: the matrix instructions on the zero halves are left out (plain exact-exponential calls; the other
  // variants run the full-width code on the same operands, which gives the same bits)
  if (p.exact_exp2 && !p.tile_skip && p.d_out <= 64)
    return bf16 ? launch_variant<KSANA_SAGE_BF16, false, kSparse, kSplit, kW, kCausal, false, 2>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s)
                : launch_variant<KSANA_SAGE_FP16, false, kSparse, kSplit, kW, kCausal, false, 2>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
  if (p.exact_exp2 && p.tile_skip)
    return bf16 ? launch_variant<KSANA_SAGE_BF16, false, kSparse, kSplit, kW, kCausal, true>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s)
                : launch_variant<KSANA_SAGE_FP16, false, kSparse, kSplit, kW, kCausal, true>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
  if (p.exact_exp2)
    return bf16 ? launch_variant<KSANA_SAGE_BF16, false, kSparse, kSplit, kW, kCausal>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s)
                : launch_variant<KSANA_SAGE_FP16, false, kSparse, kSplit, kW, kCausal>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
  return bf16 ? launch_variant<KSANA_SAGE_BF16, true, kSparse, kSplit, kW, kCausal>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s)
              : launch_variant<KSANA_SAGE_FP16, true, kSparse, kSplit, kW, kCausal>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
}

// compute units of the current device (the size of one round of workgroups: one workgroup per unit)
int compute_units() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cached[dev].load(std::memory_order_acquire);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_release);
  }
  return n;
}

}  // namespace

// Dense calls that take 4-wave workgroups (n_wg8: their grid in 256-row workgroups): short key loops, where a
// workgroup's fixed costs weigh as much as its loop and hide under the compute unit's other workgroup - measured at
// B * H = 40 and 48: 32 tiles 14-19 % faster than 256-row workgroups, 64-68 tiles 2-6 %, 128 tiles 1-3 % slower.
// Beyond kShortKeyTiles only when the chip is full anyway: a grid of a few workgroups is better off cut into runs of
// keys, which only the 256-row shape does.
static bool dense_in_four_waves(int n_wg8, int nkb) {
  return nkb <= kShortKeyTiles || (nkb <= kMidKeyTiles && n_wg8 >= compute_units());
}

void plan_key_split(int n_wg, int nkb, int* first_wg, int* runs) {
  if (dense_in_four_waves(n_wg, nkb)) {  // these shapes run in 4-wave workgroups, which are never cut
    *first_wg = n_wg, *runs = 0;
    return;
  }
  const int cus = compute_units();
  const int rest = n_wg % cus;
  int n_split = 0;
  if (rest != 0 && 2 * rest <= cus) {
    n_split = min(min(cus / rest, kMaxSplitPartials / rest), nkb / kMinTilesPerSplit);
    if (n_split < 2) n_split = 0;
  }
  *first_wg = n_split ? n_wg - rest : n_wg;
  *runs = n_split;
}

// Workgroup shape for a call: 4-wave workgroups (two per compute unit) when a block mask or causal masking is
// involved (a workgroup is then one 128-row mask row, so no wave multiplies a tile only the neighbouring mask row
// asked for) and for short key sequences (dense_in_four_waves); 8-wave workgroups otherwise, which copy
// every K/V tile once per 256 rows instead of once per 128.  p.wg_waves (4 or 8) overrides the choice.
static int pick_wg_waves(const AttnParams& p) {
  if (p.wg_waves == 4 || p.wg_waves == 8) return p.wg_waves;
  const bool sparse = p.block_mask != nullptr || p.causal;
  if (sparse) return p.nkb <= kSparseMaxKeyTiles4 ? 4 : 8;
  const int n_wg8 = p.B * p.Hq * ((p.Lq + kAttnQPerWg - 1) / kAttnQPerWg);
  return dense_in_four_waves(n_wg8, p.nkb) ? 4 : 8;
}

hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t s) {
  if (p.nkb > kMaxKeyTiles) return hipErrorInvalidValue;
  const bool sparse = p.block_mask != nullptr || p.causal;
  if (sparse && p.nkb > kSparseMaxKeyTiles) return hipErrorInvalidValue;
  int waves = pick_wg_waves(p);
  if (waves == 4 && p.nkb > (sparse ? kSparseMaxKeyTiles4 : kShortMaxKeyTiles)) waves = 8;
  if (waves == 4) {
    const int n_qwg = (p.Lq + WgShape<4>::kRows - 1) / WgShape<4>::kRows;
    const int n_wg = p.B * p.Hq * n_qwg;
    const int wg_per_xcd = (n_wg + 7) / 8;
    const dim3 grid(wg_per_xcd * 8);
    if (sparse)
      return p.causal ? launch_shape<true, false, 4, true>(p, grid, max_lds<true, 4>(), n_qwg, n_wg, wg_per_xcd, s)
                      : launch_shape<true, false, 4, false>(p, grid, max_lds<true, 4>(), n_qwg, n_wg, wg_per_xcd, s);
    const size_t lds = WgShape<4>::kRingBytes + 1024 + (((size_t)p.nkb * 4 + 1023) & ~size_t(1023));
    return launch_shape<false, false, 4>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
  }
  const int n_qwg = (p.Lq + kAttnQPerWg - 1) / kAttnQPerWg;
  const int n_wg = p.B * p.Hq * n_qwg;
  const int wg_per_xcd = (n_wg + 7) / 8;
  const dim3 grid(wg_per_xcd * 8);
  // (tile lists in 256-row workgroups, by flag only: one instantiation serves causal and plain calls)
  if (sparse) return launch_shape<true, false, 8, true>(p, grid, max_lds<true, 8>(), n_qwg, n_wg, wg_per_xcd, s);
  // tile ring + the head's K scales (a multiple of 1 KiB keeps the request tidy)
  const size_t lds = WgShape<8>::kRingBytes + 1024 + (((size_t)p.nkb * 4 + 1023) & ~size_t(1023));
  // The workgroups beyond the last full round of the chip (one workgroup per compute unit) would hold it for a
  // whole round alone.  When they are few, each is cut into runs of key tiles that together fill a round, and a
  // small kernel merges the runs: 2568 workgroups are then 10 rounds and a bit instead of 11, 280 are 1.1 instead of 2.
  int n_full = n_wg, n_split = 0;
  if (p.split_o != nullptr) plan_key_split(n_wg, p.nkb, &n_full, &n_split);
  if (n_split == 0) return launch_shape<false, false, 8>(p, grid, lds, n_qwg, n_wg, wg_per_xcd, s);
  const int rest = n_wg - n_full;
  if (n_full > 0) {
    const int per_xcd = (n_full + 7) / 8;
    const hipError_t e = launch_shape<false, false, 8>(p, dim3(per_xcd * 8), lds, n_qwg, n_full, per_xcd, s);
    if (e != hipSuccess) return e;
  }
  AttnParams ps = p;
  ps.split_first_wg = n_full;
  ps.n_split = n_split;
  const hipError_t e = launch_shape<false, true, 8>(ps, dim3(rest * n_split), lds, n_qwg, n_wg, 0, s);
  if (e != hipSuccess) return e;
  if (p.o.dtype == KSANA_SAGE_BF16)
    sage_attn_merge_kernel<KSANA_SAGE_BF16><<<dim3(rest, kAttnQPerWg / 8), dim3(256), 0, s>>>(ps, n_qwg);
  else
    sage_attn_merge_kernel<KSANA_SAGE_FP16><<<dim3(rest, kAttnQPerWg / 8), dim3(256), 0, s>>>(ps, n_qwg);
  return hipGetLastError();
}

}  // namespace ksana_sage
