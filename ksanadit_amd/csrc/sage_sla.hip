// The linear-attention branch of the sparse-linear ("SLA") backend for gfx950 (MI355X).
//
// Per (batch, head), with phi = softmax over the 128 channels of a row, rounded to the tensors' half type:
//   kv   = sum_l phi(k_l)^T v_l            [128 x 128]
//   ksum = sum_l phi(k_l)                  [128]
//   o_l  = (phi(q_l) kv) / (1e-5 + phi(q_l) . ksum)
// and, where the caller's projection is a plain linear layer, o_l W^T + bias folded in as phi(q_l) (kv W^T) / (...) +
// bias, plus an optional tensor added on the way out (the sparse branch's result).  This is calc_linear and what
// surrounds it in ksana/operations/attention/backends/sage_sla.py:135-139, 273-287 - there five library kernels over
// [B, H, L, D] intermediates, here one pass over k and v, a small finalisation, and one pass over q.
//
//   sla_kv_partial_kernel   reads k and v once; bf16 / fp16 MFMA; one partial kv and ksum per run of rows
//   sla_kv_finalize_kernel  adds the runs in order (repeatable bits), rounds to the half type as the reference's
//                           tensors are, multiplies by W^T, stores the matrix in MFMA operand order
//   sla_apply_kernel        reads q once, writes the result in [B, L, H, D]
#include "sage_kernels.h"

#include <atomic>

#include "../../include/ksana_sage_hip.h"

namespace ksana_sage {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kSlaThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;

template <int DT>
__device__ __forceinline__ v4f mfma16(const uint4& a, const uint4& b, const v4f& c) {
  if constexpr (DT == KSANA_SAGE_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}
template <int DT>
__device__ __forceinline__ v16f mfma32(const uint4& a, const uint4& b, const v16f& c) {
  if constexpr (DT == KSANA_SAGE_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

template <int DT>
__device__ __forceinline__ void widen8(const uint4& raw, float* out) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DT == KSANA_SAGE_BF16) {
      out[2 * i] = __uint_as_float(w[i] << 16);
      out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    } else {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      const h2 p = __builtin_bit_cast(h2, w[i]);
      out[2 * i] = (float)p[0];
      out[2 * i + 1] = (float)p[1];
    }
  }
}
// two fp32 values -> one dword of the half type (a in the low half)
template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (DT == KSANA_SAGE_BF16) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    const b2 p = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, p);
  } else {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 p = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, p);
  }
}
template <int DT>
__device__ __forceinline__ float round_half(float x) {
  if constexpr (DT == KSANA_SAGE_BF16) return (float)(__bf16)x;
  return (float)(_Float16)x;
}

// value of lane ^ M within the lane's group of 16, M = 1, 2, 4, 8 (DPP: quad permutes, half-row mirror, row rotation)
template <int M>
__device__ __forceinline__ float xor16(float v) {
  const int iv = __float_as_int(v);
  if constexpr (M == 1) return __int_as_float(__builtin_amdgcn_mov_dpp(iv, 0xB1, 0xF, 0xF, true));
  if constexpr (M == 2) return __int_as_float(__builtin_amdgcn_mov_dpp(iv, 0x4E, 0xF, 0xF, true));
  if constexpr (M == 8) return __int_as_float(__builtin_amdgcn_mov_dpp(iv, 0x128, 0xF, 0xF, true));  // row_ror:8
  const int t = __builtin_amdgcn_mov_dpp(iv, 0x141, 0xF, 0xF, true);                                // row_half_mirror
  return __int_as_float(__builtin_amdgcn_mov_dpp(t, 0x1B, 0xF, 0xF, true));                         // quad_perm [3,2,1,0]
}
__device__ __forceinline__ float max16(float v) {
  v = fmaxf(v, xor16<1>(v));
  v = fmaxf(v, xor16<2>(v));
  v = fmaxf(v, xor16<4>(v));
  return fmaxf(v, xor16<8>(v));
}
__device__ __forceinline__ float sum16(float v) {
  v += xor16<1>(v);
  v += xor16<2>(v);
  v += xor16<4>(v);
  return v + xor16<8>(v);
}

// ---------------------------------------------------------------------------------------------------------------
// kv and ksum over one run of rows of one head.  grid = (runs, H, B), 256 threads.
//
// A workgroup walks its rows 128 at a time, 32 per wave.  Lane (j = lane % 16, g = lane / 16) loads rows 8 g + i,
// i = 0 .. 7, channels 8 j .. 8 j + 7 of k and of v (16 bytes each; a load instruction covers four whole 256-byte
// rows).  The matrix instruction (16x16x32, contraction over 32 rows) wants, per lane, 8 consecutive ROWS of one
// channel: column t of the lane's 8 x 8 block - a matter of picking halves of registers, no data moves between
// lanes.  Tile t of the 128 phi(k) channels is therefore the strided set {8 j + t}, likewise tile u of the v
// channels {8 j + u}; the result is put back in order when it is written.
// The softmax of a row needs its 128 channels: 8 in the lane, the rest across the 16 lanes of its group (DPP).
// Operand fragments go through LDS so that every wave can use the rows of all four: wave w keeps the phi(k) tiles
// 2 w, 2 w + 1 against all eight v tiles (64 accumulator registers) and, against an all-ones operand, their row sums.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kSlaStepRows = 128;
constexpr int kSlaPartFloats = kD * kD + kD;  // one partial: kv, then ksum

template <int DT>
__global__ __launch_bounds__(kSlaThreads, 2) void sla_kv_partial_kernel(const uint16_t* __restrict__ k, int64_t ksB, int64_t ksL,
                                                                        int64_t ksH, const uint16_t* __restrict__ v,
                                                                        int64_t vsB, int64_t vsL, int64_t vsH, int H, int L,
                                                                        int rows_per_run, float* __restrict__ part) {
  const int run = blockIdx.x, h = blockIdx.y, b = blockIdx.z, runs = gridDim.x;
  const int t = threadIdx.x, lane = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int j = lane & 15, g = lane >> 4;
  const int r_begin = run * rows_per_run, r_end = min(L, r_begin + rows_per_run);
  const uint16_t* kb = k + b * ksB + h * ksH + 8 * j;
  const uint16_t* vb = v + b * vsB + h * vsH + 8 * j;
  // fragments in operand order: [wave whose rows][tile][lane] x 16 bytes
  __shared__ uint4 s_a[4 * 8 * 64];
  __shared__ uint4 s_b[4 * 8 * 64];
  v4f acc[2][8], accs[2];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    accs[m] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 8; ++u) acc[m][u] = v4f{0.f, 0.f, 0.f, 0.f};
  }
  uint4 ones;
  {
    const uint32_t one2 = DT == KSANA_SAGE_BF16 ? 0x3f803f80u : 0x3c003c00u;
    ones = make_uint4(one2, one2, one2, one2);
  }
  for (int r0 = r_begin; r0 < r_end; r0 += kSlaStepRows) {
    const int row0 = r0 + 32 * w + 8 * g;
    uint4 kx[8], vx[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      kx[i] = vx[i] = make_uint4(0, 0, 0, 0);
      if (row0 + i < r_end) {
        kx[i] = *reinterpret_cast<const uint4*>(kb + (int64_t)(row0 + i) * ksL);
        vx[i] = *reinterpret_cast<const uint4*>(vb + (int64_t)(row0 + i) * vsL);
      }
    }
    // phi(k): softmax over the row's 128 channels, rounded to the half type when it is packed
    float f[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float x[8];
      widen8<DT>(kx[i], x);
      float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
      mx = max16(mx);
      const float c = -mx * kLog2e;
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], kLog2e, c));
        sum += x[e];
      }
      sum = sum16(sum);
      const float inv = row0 + i < r_end ? __builtin_amdgcn_rcpf(sum) : 0.0f;  // rows past the run contribute nothing
#pragma unroll
      for (int e = 0; e < 8; ++e) f[i][e] = x[e] * inv;
    }
    // column t of the 8 x 8 block = the lane's fragment of tile t: rows 8 g .. 8 g + 7 of channel 8 j + t
#pragma unroll
    for (int tt = 0; tt < 8; ++tt) {
      const uint4 fa = make_uint4(pack2<DT>(f[0][tt], f[1][tt]), pack2<DT>(f[2][tt], f[3][tt]), pack2<DT>(f[4][tt], f[5][tt]),
                                  pack2<DT>(f[6][tt], f[7][tt]));
      s_a[(w * 8 + tt) * 64 + lane] = fa;
      // the same column of v: half (tt & 1) of dword tt / 2 of each row's register
      const uint32_t sel = (tt & 1) ? 0x07060302u : 0x05040100u;  // (high halves | low halves) of (src0, src1)
      auto dw = [&](const uint4& r) { return tt < 2 ? r.x : (tt < 4 ? r.y : (tt < 6 ? r.z : r.w)); };
      const uint4 fb = make_uint4(__builtin_amdgcn_perm(dw(vx[1]), dw(vx[0]), sel), __builtin_amdgcn_perm(dw(vx[3]), dw(vx[2]), sel),
                                  __builtin_amdgcn_perm(dw(vx[5]), dw(vx[4]), sel), __builtin_amdgcn_perm(dw(vx[7]), dw(vx[6]), sel));
      s_b[(w * 8 + tt) * 64 + lane] = fb;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {  // the 32 rows wave ks brought
      const uint4 a0 = s_a[(ks * 8 + 2 * w) * 64 + lane], a1 = s_a[(ks * 8 + 2 * w + 1) * 64 + lane];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint4 bu = s_b[(ks * 8 + u) * 64 + lane];
        acc[0][u] = mfma16<DT>(a0, bu, acc[0][u]);
        acc[1][u] = mfma16<DT>(a1, bu, acc[1][u]);
      }
      accs[0] = mfma16<DT>(a0, ones, accs[0]);
      accs[1] = mfma16<DT>(a1, ones, accs[1]);
    }
    __syncthreads();  // the fragments have been read: the next step may overwrite them
  }
  // accumulator register r of tile (m, u): phi(k) channel 8 * (4 g + r) + (2 w + m), v channel 8 * j + u
  float* out = part + (((int64_t)b * H + h) * runs + run) * kSlaPartFloats;
#pragma unroll
  for (int m = 0; m < 2; ++m) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ck = 8 * (4 * g + r) + 2 * w + m;
      float* orow = out + ck * kD + 8 * j;
      *reinterpret_cast<float4*>(orow) = make_float4(acc[m][0][r], acc[m][1][r], acc[m][2][r], acc[m][3][r]);
      *reinterpret_cast<float4*>(orow + 4) = make_float4(acc[m][4][r], acc[m][5][r], acc[m][6][r], acc[m][7][r]);
      if (j == 0) out[kD * kD + ck] = accs[m][r];  // every column of the all-ones product holds the row sum
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Per head: the runs' partial results added in run order; kv and ksum rounded to the half type (they are tensors of
// that type in the reference); then M = kv W^T (fp32 accumulation) where a projection is folded in, M = kv otherwise.
// M is stored for sla_apply_kernel's A operand: fragment (nt, s) = 64 lanes x 8 halves, lane (n = lane % 32,
// g = lane / 32) holding M[16 s + 8 g + i][32 nt + n], i = 0 .. 7.  grid = (8, B * H): 16 rows of kv per workgroup.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kFinRows = 16;  // rows of kv per workgroup

template <int DT>
__global__ __launch_bounds__(kSlaThreads) void sla_kv_finalize_kernel(const float* __restrict__ part, int runs,
                                                                      const float* __restrict__ proj_w,
                                                                      uint16_t* __restrict__ m_frag,
                                                                      float* __restrict__ ksum) {
  const int bh = blockIdx.y, d0 = blockIdx.x * kFinRows, t = threadIdx.x;
  __shared__ float s_kv[kFinRows * kD];
  const float* p = part + (int64_t)bh * runs * kSlaPartFloats;
  for (int idx = t; idx < kFinRows * kD; idx += kSlaThreads) {
    float a = 0.0f;
    for (int r = 0; r < runs; ++r) a = r == 0 ? p[d0 * kD + idx] : a + p[(int64_t)r * kSlaPartFloats + d0 * kD + idx];
    s_kv[idx] = round_half<DT>(a);
  }
  if (t < kFinRows) {
    float a = 0.0f;
    for (int r = 0; r < runs; ++r) a = r == 0 ? p[kD * kD + d0 + t] : a + p[(int64_t)r * kSlaPartFloats + kD * kD + d0 + t];
    ksum[bh * kD + d0 + t] = round_half<DT>(a);
  }
  __syncthreads();
  // thread t: output column n = t % 128 for the rows d0 + (t / 128), d0 + (t / 128) + 2, ...
  const int n = t & (kD - 1);
  float m[kFinRows / 2];
  if (proj_w != nullptr) {
#pragma unroll
    for (int i = 0; i < kFinRows / 2; ++i) m[i] = 0.0f;
    const float4* wr = reinterpret_cast<const float4*>(proj_w + n * kD);  // W[n][c]
    for (int c4 = 0; c4 < kD / 4; ++c4) {
      const float4 wv = wr[c4];
#pragma unroll
      for (int i = 0; i < kFinRows / 2; ++i) {
        const float* kr = s_kv + ((t >> 7) + 2 * i) * kD + 4 * c4;  // the same address in every lane: a broadcast
        m[i] = __builtin_fmaf(kr[0], wv.x, m[i]);
        m[i] = __builtin_fmaf(kr[1], wv.y, m[i]);
        m[i] = __builtin_fmaf(kr[2], wv.z, m[i]);
        m[i] = __builtin_fmaf(kr[3], wv.w, m[i]);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < kFinRows / 2; ++i) m[i] = s_kv[((t >> 7) + 2 * i) * kD + n];
  }
#pragma unroll
  for (int i = 0; i < kFinRows / 2; ++i) {
    const int d = d0 + (t >> 7) + 2 * i;
    const int nt = n >> 5, s = d >> 4, g = (d >> 3) & 1, e = d & 7, lane = 32 * g + (n & 31);
    uint16_t bits;
    if constexpr (DT == KSANA_SAGE_BF16)
      bits = __builtin_bit_cast(uint16_t, (__bf16)m[i]);
    else
      bits = __builtin_bit_cast(uint16_t, (_Float16)m[i]);
    m_frag[(int64_t)bh * kD * kD + ((nt * 8 + s) * 64 + lane) * 8 + e] = bits;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// out[b, l, h, :] = (phi(q_l) M) / (1e-5 + phi(q_l) . ksum) + bias (+ add[b, l, h, :]).
// grid = (ceil(L / (128 * blocks)), H, B), 256 threads; a workgroup stages M (32 KiB) in LDS once and walks `blocks`
// blocks of 128 rows, 32 per wave.  Lane (row = lane % 32, g = lane / 32) loads the channels 16 s + 8 g .. + 7 of its
// row, s = 0 .. 7 - half of the row, exactly its B operands of the 32x32x16 instruction (contraction over channels);
// the other half sits in lane + 32.  The product is taken transposed, out^T = M^T phi(q)^T, so that a lane ends up
// with channels of ONE row; the rows leave through LDS as whole 256-byte rows, 16 bytes per lane.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kApplyPitch = 2 * kD + 16;
constexpr int kApplyLds = kD * kD * 2 + 2 * kD * 4 + 4 * 32 * kApplyPitch;  // 68 608 bytes

template <int DT>
__global__ __launch_bounds__(kSlaThreads, 2) void sla_apply_kernel(const uint16_t* __restrict__ q, int64_t qsB, int64_t qsL,
                                                                   int64_t qsH, const uint16_t* __restrict__ m_frag,
                                                                   const float* __restrict__ ksum,
                                                                   const float* __restrict__ bias,
                                                                   const uint16_t* __restrict__ add, int64_t asB, int64_t asL,
                                                                   int64_t asH, uint16_t* __restrict__ out, int64_t osB,
                                                                   int64_t osL, int64_t osH, int H, int L, int blocks) {
  const int h = blockIdx.y, b = blockIdx.z, bh = b * H + h;
  const int t = threadIdx.x, lane = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  // dynamic LDS (kApplyLds bytes): M in operand order, ksum, bias, then one staging area per wave
  extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
  uint4* s_m = reinterpret_cast<uint4*>(s_dyn);
  float* s_ks = reinterpret_cast<float*>(s_dyn + kD * kD * 2);
  float* s_bias = s_ks + kD;
  constexpr int kPitch = kApplyPitch;  // bytes per staged row
  uint8_t* s_stage = s_dyn + kD * kD * 2 + 2 * kD * 4;
  {
    const uint4* src = reinterpret_cast<const uint4*>(m_frag + (int64_t)bh * kD * kD);
#pragma unroll
    for (int i = 0; i < 8; ++i) s_m[i * kSlaThreads + t] = src[i * kSlaThreads + t];
    if (t < kD) {
      s_ks[t] = ksum[bh * kD + t];
      s_bias[t] = bias != nullptr ? bias[t] : 0.0f;
    }
  }
  __syncthreads();
  uint8_t* stage = s_stage + w * (32 * kPitch);
  for (int blk = 0; blk < blocks; ++blk) {
    const int r0 = (blockIdx.x * blocks + blk) * 128 + 32 * w;
    if (r0 >= L) break;  // wave-uniform
    const int row = r0 + l32;
    const uint16_t* qr = q + b * qsB + (int64_t)row * qsL + h * qsH + 8 * g;
    uint4 raw[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) raw[s] = row < L ? *reinterpret_cast<const uint4*>(qr + 16 * s) : make_uint4(0, 0, 0, 0);
    // the pieces of `add` this lane will meet in the output loop below, requested now: they arrive under the
    // arithmetic instead of being waited for one by one between a load and its store
    uint16_t* ob = out + b * osB + h * osH;
    const uint16_t* ab = add != nullptr ? add + b * asB + h * asH : nullptr;
    uint4 other[8];
    if (ab != nullptr) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int idx = i * 64 + lane, r = idx >> 4, cc = idx & 15;
        other[i] = r0 + r < L ? *reinterpret_cast<const uint4*>(ab + (int64_t)(r0 + r) * asL + 8 * cc) : make_uint4(0, 0, 0, 0);
      }
    }
    float x[8][8];
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      widen8<DT>(raw[s], x[s]);
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, x[s][e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float c = -mx * kLog2e;
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x[s][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[s][e], kLog2e, c));
        sum += x[s][e];
      }
    sum += __shfl_xor(sum, 32);
    const float inv = __builtin_amdgcn_rcpf(sum);
    uint4 fq[8];
    float den = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      uint32_t pw[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float f0 = x[s][2 * e] * inv, f1 = x[s][2 * e + 1] * inv;
        pw[e] = pack2<DT>(f0, f1);
        den = __builtin_fmaf(f0, s_ks[16 * s + 8 * g + 2 * e], den);
        den = __builtin_fmaf(f1, s_ks[16 * s + 8 * g + 2 * e + 1], den);
      }
      fq[s] = make_uint4(pw[0], pw[1], pw[2], pw[3]);
    }
    den += __shfl_xor(den, 32);
    const float scale = __builtin_amdgcn_rcpf(1e-5f + den);
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      v16f acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; ++s) acc = mfma32<DT>(s_m[(nt * 8 + s) * 64 + lane], fq[s], acc);
      // register r: output channel 32 nt + 8 (r / 4) + 4 g + r % 4 of row l32
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = 32 * nt + 8 * q4 + 4 * g;
        const float4 bs = *reinterpret_cast<const float4*>(s_bias + n);
        const uint32_t lo = pack2<DT>(__builtin_fmaf(acc[4 * q4 + 0], scale, bs.x), __builtin_fmaf(acc[4 * q4 + 1], scale, bs.y));
        const uint32_t hi = pack2<DT>(__builtin_fmaf(acc[4 * q4 + 2], scale, bs.z), __builtin_fmaf(acc[4 * q4 + 3], scale, bs.w));
        *reinterpret_cast<uint2*>(stage + l32 * kPitch + 2 * n) = make_uint2(lo, hi);
      }
    }
    // LDS serves one wave's accesses in order: the reads below see the writes above
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = i * 64 + lane, r = idx >> 4, cc = idx & 15;  // row r of the wave, 16-byte piece cc of it
      uint4 piece = *reinterpret_cast<const uint4*>(stage + r * kPitch + 16 * cc);
      if (r0 + r < L) {
        if (ab != nullptr) {
          float a8[8], o8[8];
          widen8<DT>(piece, a8);
          widen8<DT>(other[i], o8);
          piece = make_uint4(pack2<DT>(a8[0] + o8[0], a8[1] + o8[1]), pack2<DT>(a8[2] + o8[2], a8[3] + o8[3]),
                             pack2<DT>(a8[4] + o8[4], a8[5] + o8[5]), pack2<DT>(a8[6] + o8[6], a8[7] + o8[7]));
        }
        *reinterpret_cast<uint4*>(ob + (int64_t)(r0 + r) * osL + 8 * cc) = piece;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The block map from the pooled blocks (get_block_map, sage_sla.py:83-90): score = pooled_q pooled_k^T as a tensor of
// the half type (fp32 accumulation, one rounding), then for every query block the `keep` key blocks with the largest
// scores get a one, the others a zero; of equal scores the lower index wins (what a stable descending sort gives;
// torch.topk leaves it open).  grid = (ceil(nq / 32), B * H), 256 threads; dynamic LDS 32 * nk_pad * 2 bytes.
//
// Scores: 32 query blocks x 32 key blocks per 32x32x16 matrix instruction, contraction over the 128 channels - both
// operands are 16-byte pieces of pooled rows as they lie in memory; wave w takes the key tiles w, w + 4, ...  Each
// score goes to LDS as a 16-bit key whose unsigned order is the order of the values.  Selection, one wave per 8 query
// blocks: the keep-th largest key by bisection over its 16 bits (count of keys >= candidate by ballots), then ones for
// the keys above it and for as many of its equals, lowest index first, as are still missing.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMapMaxKeyBlocks = 1024;

template <int DT>
__global__ __launch_bounds__(kSlaThreads) void sla_block_map_kernel(const uint16_t* __restrict__ pooled_q,
                                                                    const uint16_t* __restrict__ pooled_k, int nq, int nk,
                                                                    int nk_pad, int keep, int8_t* __restrict__ block_map) {
  extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
  uint16_t* s_key = reinterpret_cast<uint16_t*>(s_dyn);  // [32][nk_pad]
  const int bh = blockIdx.y, q0 = blockIdx.x * 32;
  const int t = threadIdx.x, lane = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const uint16_t* pq = pooled_q + ((int64_t)bh * nq + q0 + l32) * kD + 8 * g;
  const uint16_t* pk = pooled_k + (int64_t)bh * nk * kD + 8 * g;
  uint4 a[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) a[s] = q0 + l32 < nq ? *reinterpret_cast<const uint4*>(pq + 16 * s) : make_uint4(0, 0, 0, 0);
  for (int nt = w; nt * 32 < nk_pad; nt += 4) {
    const int kb = nt * 32 + l32;
    uint4 b[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) b[s] = kb < nk ? *reinterpret_cast<const uint4*>(pk + (int64_t)kb * kD + 16 * s) : make_uint4(0, 0, 0, 0);
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) acc = mfma32<DT>(a[s], b[s], acc);
    // register r: query block 8 (r / 4) + 4 g + r % 4 of the group, key block kb
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = 8 * (r >> 2) + 4 * g + (r & 3);
      uint32_t bits;
      if constexpr (DT == KSANA_SAGE_BF16)
        bits = __builtin_bit_cast(uint16_t, (__bf16)acc[r]);
      else
        bits = __builtin_bit_cast(uint16_t, (_Float16)acc[r]);
      const uint32_t key = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);  // unsigned order = value order
      s_key[m * nk_pad + kb] = (uint16_t)(kb < nk ? key : 0u);                    // padding sorts below everything
    }
  }
  __syncthreads();
  // a row's keys in registers: lane holds the keys lane + 64 i (0, the padding value, beyond nk)
  constexpr int kPerLane = kMapMaxKeyBlocks / 64;
  for (int mi = 0; mi < 8; ++mi) {
    const int m = 8 * w + mi;
    if (q0 + m >= nq) break;  // wave-uniform
    const uint16_t* row = s_key + m * nk_pad;
    int8_t* out = block_map + ((int64_t)bh * nq + q0 + m) * nk;
    uint32_t key[kPerLane];
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) key[i] = lane + 64 * i < nk ? row[lane + 64 * i] : 0u;
    uint32_t thr = 0;
    if (keep > 0 && keep < nk) {
      for (int bit = 15; bit >= 0; --bit) {
        const uint32_t cand = thr | (1u << bit);
        int count = 0;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) count += __popcll(__ballot(key[i] >= cand));  // padding keys are 0 < cand
        if (count >= keep) thr = cand;  // uniform
      }
    }
    int above = 0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) above += __popcll(__ballot(key[i] > thr));
    int missing = keep >= nk ? nk : (keep <= 0 ? 0 : keep - above);  // of the keys equal to thr, lowest index first
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int idx = lane + 64 * i;
      const bool in = idx < nk;
      const bool eq = in && key[i] == thr;
      const unsigned long long bal = __ballot(eq);
      const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(bal >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)bal, 0));
      const bool one = in && keep > 0 && (keep >= nk || key[i] > thr || (eq && rank < missing));
      if (in) out[idx] = one ? 1 : 0;
      missing -= __popcll(bal);
    }
  }
}

}  // namespace

// rows per run of sla_kv_partial_kernel, runs a multiple of 128 rows: as many runs per head as keep the whole grid
// within the 512 workgroups the chip holds at once (two per compute unit, 64 KiB of LDS each) - a few workgroups
// more than that and the launch takes two rounds for one round's work (520 workgroups: 212 us; 480: see profiles)
void plan_sla_runs(int B, int H, int L, int* runs, int* rows_per_run) {
  const int steps = (L + kSlaStepRows - 1) / kSlaStepRows;
  int n = 512 / max(1, B * H);
  n = max(1, min(n, steps));
  const int steps_per_run = (steps + n - 1) / n;
  *rows_per_run = steps_per_run * kSlaStepRows;
  *runs = (steps + steps_per_run - 1) / steps_per_run;
}

hipError_t launch_sla_linear(const InTensor& q, const InTensor& k, const InTensor& v, int B, int H, int L,
                             const float* proj_w, const float* proj_b, const InTensor* add, const OutTensor& out,
                             float* part, uint16_t* m_frag, float* ksum, hipStream_t s) {
  int runs = 1, rows_per_run = L;
  plan_sla_runs(B, H, L, &runs, &rows_per_run);
  const dim3 block(kSlaThreads);
  constexpr int kBlocks = 4;  // 128-row blocks per workgroup of the second pass (M is staged once per workgroup)
  const dim3 grid_apply(((L + 127) / 128 + kBlocks - 1) / kBlocks, H, B);
  {  // more than 64 KiB of dynamic LDS has to be requested per kernel, once per device
    static std::atomic<bool> requested[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!requested[dev].load(std::memory_order_acquire)) {
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sla_apply_kernel<KSANA_SAGE_BF16>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kApplyLds);
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sla_apply_kernel<KSANA_SAGE_FP16>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kApplyLds);
      if (e != hipSuccess) return e;
      requested[dev].store(true, std::memory_order_release);
    }
  }
  const uint16_t* add_ptr = add != nullptr ? add->ptr : nullptr;
  const int64_t asB = add ? add->sB : 0, asL = add ? add->sL : 0, asH = add ? add->sH : 0;
  if (q.dtype == KSANA_SAGE_BF16) {
    constexpr int DT = KSANA_SAGE_BF16;
    sla_kv_partial_kernel<DT><<<dim3(runs, H, B), block, 0, s>>>(k.ptr, k.sB, k.sL, k.sH, v.ptr, v.sB, v.sL, v.sH, H, L, rows_per_run, part);
    sla_kv_finalize_kernel<DT><<<dim3(kD / kFinRows, B * H), block, 0, s>>>(part, runs, proj_w, m_frag, ksum);
    sla_apply_kernel<DT><<<grid_apply, block, kApplyLds, s>>>(q.ptr, q.sB, q.sL, q.sH, m_frag, ksum, proj_b, add_ptr, asB, asL, asH, out.ptr,
                                                      out.sB, out.sL, out.sH, H, L, kBlocks);
  } else {
    constexpr int DT = KSANA_SAGE_FP16;
    sla_kv_partial_kernel<DT><<<dim3(runs, H, B), block, 0, s>>>(k.ptr, k.sB, k.sL, k.sH, v.ptr, v.sB, v.sL, v.sH, H, L, rows_per_run, part);
    sla_kv_finalize_kernel<DT><<<dim3(kD / kFinRows, B * H), block, 0, s>>>(part, runs, proj_w, m_frag, ksum);
    sla_apply_kernel<DT><<<grid_apply, block, kApplyLds, s>>>(q.ptr, q.sB, q.sL, q.sH, m_frag, ksum, proj_b, add_ptr, asB, asL, asH, out.ptr,
                                                      out.sB, out.sL, out.sH, H, L, kBlocks);
  }
  return hipGetLastError();
}

}  // namespace ksana_sage

namespace ksana_sage {
hipError_t launch_sla_block_map(const uint16_t* pooled_q, const uint16_t* pooled_k, int dtype, int BH, int nq, int nk, int keep,
                                int8_t* block_map, hipStream_t s) {
  if (nk > kMapMaxKeyBlocks) return hipErrorInvalidValue;
  const int nk_pad = (nk + 31) / 32 * 32;
  const dim3 grid((nq + 31) / 32, BH), block(kSlaThreads);
  const size_t lds = (size_t)32 * nk_pad * 2;
  if (dtype == KSANA_SAGE_BF16)
    sla_block_map_kernel<KSANA_SAGE_BF16><<<grid, block, lds, s>>>(pooled_q, pooled_k, nq, nk, nk_pad, keep, block_map);
  else
    sla_block_map_kernel<KSANA_SAGE_FP16><<<grid, block, lds, s>>>(pooled_q, pooled_k, nq, nk, nk_pad, keep, block_map);
  return hipGetLastError();
}
}  // namespace ksana_sage
