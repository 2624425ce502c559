// Fused quantized attention for gfx950 (MI355X): INT8 QK^T and FP8 PV on MFMA, fp32 online
// softmax in registers.
//
// Work split.  One workgroup = 8 waves = 256 query rows of one (batch, head); each wave owns
// 32 query rows for the whole key loop.  Keys are consumed in tiles of 64 rows (= one int8
// K scale block; Q scales are per row, i.e. per lane), K and V^T tiles are staged in a 3-deep LDS ring shared by the 8 waves.
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

#include <type_traits>

#include "../../include/ksana_sage_hip.h"

namespace ksana_sage {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kWaves = 8;
constexpr int kThreadsAttn = kWaves * 64;
constexpr int kMagicI = 0x4B400000;       // bits of 12582912.0f
constexpr float kMagicF = 12582912.0f;
constexpr float kPShift = 8.0f;           // P is scaled by 2^8 before the e4m3 cast
constexpr int kStageBytes = 2 * kTileBytes;  // K tile + V tile
constexpr int kStages = 3;                   // LDS ring: tile j (V), j+1 (K), j+2 (in flight)

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int DT>
__device__ __forceinline__ void store4(uint16_t* dst, float a, float b, float c, float d) {
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
  *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
}

// S^T tile (64 keys x 32 queries) of one wave: two 32-key sub-tiles, four 32-channel steps.
__device__ __forceinline__ void qk_tile(const uint8_t* k_stage, int lane, const v4i (&qf)[4], const v16i& magic,
                                        v16i (&acc)[2]) {
  acc[0] = magic;
  acc[1] = magic;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const v4i kf = *reinterpret_cast<const v4i*>(k_stage + ((t * 4 + s) * 64 + lane) * 16);
      acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[s], acc[t], 0, 0, 0);
    }
  }
}

template <int DT>
__global__ __launch_bounds__(kThreadsAttn) void sage_attn_fwd_kernel(const AttnParams p, int n_qwg, int n_wg,
                                                                     int wg_per_xcd) {
  // Consecutive workgroup ids land on consecutive XCDs (8 per chip, one L2 each).  Give every
  // XCD a contiguous run of (head, query block) pairs so the workgroups that stream the same
  // K/V tiles share one L2.
  const int xcd = blockIdx.x & 7;
  const int wg = xcd * wg_per_xcd + (blockIdx.x >> 3);
  if (wg >= n_wg) return;
  const int bh = wg / n_qwg, qwg = wg - bh * n_qwg;
  const int b = bh / p.Hq, h = bh - b * p.Hq;
  const int bhk = b * p.Hkv + h / (p.Hq / p.Hkv);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int q0 = qwg * kAttnQPerWg + wave * 32;
  const bool active = q0 < p.Lq;  // wave-uniform; inactive waves only help move tiles

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // ---- Q fragments (B operand), 4 channel steps --------------------------------------
  v4i qf[4];
  float qs = 0.0f;
  if (active) {
    const int8_t* qrow = p.q_i8 + ((int64_t)bh * p.lq_pad + q0 + l32) * kD + 16 * hh;
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = *reinterpret_cast<const v4i*>(qrow + 32 * s);
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
  float l_part[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // this lane's share of the running row sum

  v16i magic;
#pragma unroll
  for (int r = 0; r < 16; ++r) magic[r] = kMagicI;

  const uint8_t* k_src = reinterpret_cast<const uint8_t*>(p.k_tiles) + (int64_t)bhk * p.nkb * kTileBytes + tid * 16;
  const uint8_t* v_src = p.v_tiles + (int64_t)bhk * p.nkb * kTileBytes + tid * 16;
  const float* ks_ptr = p.k_scale + (int64_t)bhk * p.nkb;
  const int nkb = p.nkb;

  // ---- prologue: tiles 0 and 1 -> LDS stages 0 and 1; S^T of tile 0 --------------------
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (j < nkb) {
      const uint4 kreg = *reinterpret_cast<const uint4*>(k_src + (int64_t)j * kTileBytes);
      const uint4 vreg = *reinterpret_cast<const uint4*>(v_src + (int64_t)j * kTileBytes);
      *reinterpret_cast<uint4*>(smem + j * kStageBytes + tid * 16) = kreg;
      *reinterpret_cast<uint4*>(smem + j * kStageBytes + kTileBytes + tid * 16) = vreg;
    }
  }
  __syncthreads();

  const bool has_tail = (p.Lk & (kBlkK - 1)) != 0;  // keys >= Lk live only in the last tile
  const int n_main = has_tail ? nkb - 1 : nkb;       // tiles handled by the branch-free loop

  // HBM -> registers for tile j+2 (clamped: the last two iterations re-fetch the last tile into
  // a stage nobody reads any more, which keeps the loop body free of branches)
  auto fetch = [&](int j, uint4& kreg, uint4& vreg) {
    const int jl = min(j + 2, nkb - 1);
    kreg = *reinterpret_cast<const uint4*>(k_src + (int64_t)jl * kTileBytes);
    vreg = *reinterpret_cast<const uint4*>(v_src + (int64_t)jl * kTileBytes);
  };
  auto stash = [&](int j, const uint4& kreg, const uint4& vreg) {
    uint8_t* dst = smem + ((j + 2) % kStages) * kStageBytes;
    *reinterpret_cast<uint4*>(dst + tid * 16) = kreg;
    *reinterpret_cast<uint4*>(dst + kTileBytes + tid * 16) = vreg;
  };

  if (!active) {
    // same barrier sequence as the active waves, moving tiles only
    for (int j = 0; j < n_main; ++j) {
      uint4 kreg, vreg;
      fetch(j, kreg, vreg);
      stash(j, kreg, vreg);
      __syncthreads();
    }
    return;
  }

  // running max update for one tile; rescales O and the row sum when the max of any row moved
  auto update_max = [&](const v16i (&s_cur)[2], float sc) {
    int imax = s_cur[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) imax = max(imax, s_cur[t][r]);
    {
      // the other half of query l32's keys lives in lane l32 + 32
      int other = imax;
      const auto sw = __builtin_amdgcn_permlane32_swap(imax, other, false, false);
      imax = max(sw[0], sw[1]);
    }
    const float m_tile = (float)(imax - kMagicI) * sc;
    const float m_new = fmaxf(m_run, m_tile);
    if (__any(m_new > m_run)) {
      const float alpha = fast_exp2(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 4; ++i) l_part[i] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
      m_run = m_new;
    }
  };
  // P = exp2(sc*dot - m_run + shift) packed to e4m3 in MFMA operand order; the magic is folded
  // into the constant, which is off by at most ~1.5 integer steps of the dot product
  auto exp_and_pack = [&](const v16i (&s_cur)[2], float sc, v8i& pf, int j, auto is_tail) {
    const float c = (kPShift - m_run) - kMagicF * sc;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          e[i] = fast_exp2(__builtin_fmaf(__int_as_float(s_cur[t][4 * g + i]), sc, c));
          if constexpr (decltype(is_tail)::value) {
            const int key = j * kBlkK + 32 * t + 8 * g + 4 * hh + i;
            if (key >= p.Lk) e[i] = 0.0f;
          }
          l_part[i] += e[i];
        }
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(e[0], e[1], w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(e[2], e[3], w, true);
        pf[4 * t + g] = w;
      }
    }
  };
  // O^T += V^T . P^T
  auto pv_tile = [&](const uint8_t* vst, const v8i& pf) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const v4i lo = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 0) * 64 + lane) * 16);
      const v4i hi = *reinterpret_cast<const v4i*>(vst + ((dt * 2 + 1) * 64 + lane) * 16);
      const v8i vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      oacc[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf, oacc[dt], 0, 0, 0, 0, 0, 0);
    }
  };

  v16i s_a[2], s_b[2];
  qk_tile(smem, lane, qf, magic, s_a);

  // One full key tile.  The S^T MFMAs of the NEXT tile sit in the same basic block as this
  // tile's exponentials, so the scheduler can run them under the VALU work; the tile after
  // that travels HBM -> registers -> LDS meanwhile (3-stage ring).
  auto tile_step = [&](int j, v16i (&s_cur)[2], v16i (&s_nxt)[2]) {
    uint4 kreg, vreg;
    fetch(j, kreg, vreg);
    const float sc = qs * ks_ptr[j];
    update_max(s_cur, sc);
    // stage (j+1)%3 holds tile j+1 (stale bytes after the last tile: computed, never used)
    qk_tile(smem + ((j + 1) % kStages) * kStageBytes, lane, qf, magic, s_nxt);
    v8i pf;
    exp_and_pack(s_cur, sc, pf, j, std::false_type{});
    pv_tile(smem + (j % kStages) * kStageBytes + kTileBytes, pf);
    stash(j, kreg, vreg);
    // interleave: one MFMA (32 cycles of matrix pipe) per ~14 VALU instructions
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read (K fragment)
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, 14, 0);  // VALU (fma / exp2 / add / cvt)
    }
    // after this barrier: tile j+2 is visible, and nobody reads stage j%3 any more
    __syncthreads();
  };

  for (int j = 0; j < n_main; j += 2) {
    tile_step(j, s_a, s_b);
    if (j + 1 < n_main) tile_step(j + 1, s_b, s_a);
  }
  if (has_tail) {
    const int j = nkb - 1;
    v16i (&s_cur)[2] = (n_main & 1) ? s_b : s_a;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = j * kBlkK + 32 * t + 8 * (r >> 2) + 4 * hh + (r & 3);
        if (key >= p.Lk) s_cur[t][r] = kMagicI - (1 << 22);  // below every real score
      }
    const float sc = qs * ks_ptr[j];
    update_max(s_cur, sc);
    v8i pf;
    exp_and_pack(s_cur, sc, pf, j, std::true_type{});
    pv_tile(smem + (j % kStages) * kStageBytes + kTileBytes, pf);
  }

  // ---- epilogue: O = O^T / rowsum * v_scale, written [B, Lq, H, D] ----------------------
  const float l_lane = (l_part[0] + l_part[1]) + (l_part[2] + l_part[3]);
  const float l_tot = l_lane + __shfl_xor(l_lane, 32);
  const float inv_l = 1.0f / l_tot;
  const int q = q0 + l32;
  if (q < p.Lq) {
    uint16_t* orow = p.o.ptr + b * p.o.sB + (int64_t)q * p.o.sL + h * p.o.sH;
    const float* vs = p.v_scale + (int64_t)bhk * kD;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = 32 * dt + 8 * g + 4 * hh;
        const float4 s4 = *reinterpret_cast<const float4*>(vs + d);
        store4<DT>(orow + d, oacc[dt][4 * g + 0] * inv_l * s4.x, oacc[dt][4 * g + 1] * inv_l * s4.y,
                   oacc[dt][4 * g + 2] * inv_l * s4.z, oacc[dt][4 * g + 3] * inv_l * s4.w);
      }
    }
  }
}

}  // namespace

hipError_t launch_attn_fwd(const AttnParams& p, hipStream_t s) {
  const int n_qwg = (p.Lq + kAttnQPerWg - 1) / kAttnQPerWg;
  const int n_wg = p.B * p.Hq * n_qwg;
  const int wg_per_xcd = (n_wg + 7) / 8;
  const dim3 grid(wg_per_xcd * 8), block(kThreadsAttn);
  const size_t lds = kStages * kStageBytes;
  if (p.o.dtype == KSANA_SAGE_BF16)
    sage_attn_fwd_kernel<KSANA_SAGE_BF16><<<grid, block, lds, s>>>(p, n_qwg, n_wg, wg_per_xcd);
  else
    sage_attn_fwd_kernel<KSANA_SAGE_FP16><<<grid, block, lds, s>>>(p, n_qwg, n_wg, wg_per_xcd);
  return hipGetLastError();
}

}  // namespace ksana_sage
