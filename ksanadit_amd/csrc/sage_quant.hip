// HBM-bound quantizer kernels for gfx950 (MI355X).
//
// Every kernel works on 128-channel rows of a [B, L, H, D] half tensor with the same thread
// mapping: 256 threads = 32 row slots x 8 lanes, each lane owning 16 consecutive channels
// (two 16-byte loads), so a wave reads four full 256-byte rows per load pair.
//
// The arithmetic is fixed to the last bit (it is compared bit-exactly with a PyTorch
// specification): plain IEEE fp32 add / sub / mul / div, round-half-even, no contraction.
#include "sage_kernels.h"

#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/ksana_sage_hip.h"

namespace ksana_sage {
namespace {

constexpr int kThreads = 256;
constexpr int kSlots = 32;  // row slots per workgroup

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
      h2 p = __builtin_bit_cast(h2, w[i]);
      out[2 * i] = (float)p[0];
      out[2 * i + 1] = (float)p[1];
    }
  }
}

// 16 channels of one row; rows at or beyond L read as zero.
template <int DT>
__device__ __forceinline__ void load_row16(const uint16_t* row_ptr, bool valid, float* out) {
  uint4 a = make_uint4(0, 0, 0, 0), b = make_uint4(0, 0, 0, 0);
  if (valid) {
    a = *reinterpret_cast<const uint4*>(row_ptr);
    b = *reinterpret_cast<const uint4*>(row_ptr + 8);
  }
  widen8<DT>(a, out);
  widen8<DT>(b, out + 8);
}

// 16 bytes of quantizer output.  Non-temporal: the tiles are written once and read next by another kernel, after
// half a gigabyte of other traffic; stores that do not linger in the caches on their way out measured 6 % off the
// three quantizers together (405 -> 380 us at B=1 H=40 L=32760), with the attention kernel's time unchanged.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_out16(void* p, uint4 v) {
  const u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p));
}

// The same row as it sits in memory (two 16-byte loads), for code that wants the next row in flight while it works
// on the current one.
__device__ __forceinline__ void fetch_row16(const uint16_t* row_ptr, bool valid, uint4 (&raw)[2]) {
  raw[0] = raw[1] = make_uint4(0, 0, 0, 0);
  if (valid) {
    raw[0] = *reinterpret_cast<const uint4*>(row_ptr);
    raw[1] = *reinterpret_cast<const uint4*>(row_ptr + 8);
  }
}

__device__ __forceinline__ float round_to_half_dtype(float x, int dtype) {
  if (dtype == KSANA_SAGE_BF16) return (float)(__bf16)x;
  return (float)(_Float16)x;
}

// ---------------------------------------------------------------------------------------
// The step before attention, on the 16 channels [16*c16, 16*c16+16) of head h, token `row`:
//   y = half( (x * inv_rms[row]) * weight[ch] )                         RMSNorm, fp32, in this order
//   (y[2i], y[2i+1]) -> half( float( (y[2i] + i*y[2i+1]) * freqs[p, i] ) )   rotation in fp64
// with p the token's frame / row / column index for pair i in [0,22) / [22,43) / [43,64).
// Each result is rounded to the tensor's half type exactly where a separate norm kernel and a
// separate rotation kernel would have stored it (the fp64 product first to fp32, as a
// conversion from double goes), so the quantizer sees the same bits.
// Tokens at or beyond frames*height*width are normed but not rotated.
// ---------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float through_half(float x) {
  // The fp32 value has to exist before it is narrowed: left alone, the compiler merges the
  // multiply that produced it with the conversion (v_fma_mixlo_f16), which rounds once
  // instead of twice and so differs from "compute in fp32, then store as half" in rare ties.
  asm volatile("" : "+v"(x));
  if constexpr (DT == KSANA_SAGE_BF16) return (float)(__bf16)x;
  return (float)(_Float16)x;
}

// Two values at a time: one packed conversion instead of two (bf16), the same roundings.
template <int DT>
__device__ __forceinline__ void through_half2(float& a, float& b) {
  asm volatile("" : "+v"(a), "+v"(b));  // as in through_half: the fp32 values exist before they are narrowed
  if constexpr (DT == KSANA_SAGE_BF16) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    const b2 p = {(__bf16)a, (__bf16)b};
    const uint32_t w = __builtin_bit_cast(uint32_t, p);
    a = __uint_as_float(w << 16);
    b = __uint_as_float(w & 0xffff0000u);
  } else {
    a = (float)(_Float16)a;
    b = (float)(_Float16)b;
  }
}

// Rotation factors for the rows of one workgroup, copied to LDS once.  The model's table is
// [position on an axis][64 pairs] of complex128; a lane needs 8 of them (128 bytes) per row, four
// times its payload, and fetched straight from the table those reads are 16 bytes out of 30-odd
// different cache lines per load instruction - the L1 tag rate, not HBM, then sets the pace.  The
// table is separable, so what a run of consecutive rows needs is small: the frames it touches
// (22 pairs each), the image rows it touches (21 pairs each) and every column (21 pairs each).
struct RopeLds {
  const double2* frame;   // [frames touched][22], first = frame f0
  const double2* height;  // [image rows touched][21], first = image row gr0 (counted across frames)
  const double2* width;   // [grid width][21]
  int f0, gr0;
};

constexpr int kRopeN0 = kRopeSplit0, kRopeN1 = kRopeSplit1 - kRopeSplit0, kRopeN2 = kD / 2 - kRopeSplit1;

// All threads of the workgroup call this; rows [row0, row0 + nrows) of batch entry b are the
// ones the workgroup will rotate.  Ends with a barrier.
__device__ __forceinline__ RopeLds stage_rope(const PrepParams& pp, int b, int row0, int nrows, double2* lds) {
  RopeLds rl;
  rl.frame = lds;
  rl.height = lds + pp.lds_frames * kRopeN0;
  rl.width = rl.height + pp.lds_heights * kRopeN1;
  const int gh = pp.grid[b][1], gw = pp.grid[b][2], plane = gh * gw;
  const int r1 = min(row0 + nrows, pp.grid[b][0] * plane);  // exclusive; rows from here on are not rotated
  rl.f0 = row0 / plane;
  rl.gr0 = row0 / gw;
  if (row0 < r1) {
    const double2* tab = reinterpret_cast<const double2*>(pp.freqs);
    const int nf = (r1 - 1) / plane - rl.f0 + 1, nh = (r1 - 1) / gw - rl.gr0 + 1;
    const int t = threadIdx.x, nt = blockDim.x;
    for (int idx = t; idx < nf * kRopeN0; idx += nt) {
      const int r = idx / kRopeN0, i = idx - r * kRopeN0;
      lds[idx] = tab[(int64_t)(rl.f0 + r) * (kD / 2) + i];
    }
    double2* hdst = lds + pp.lds_frames * kRopeN0;
    for (int idx = t; idx < nh * kRopeN1; idx += nt) {
      const int r = idx / kRopeN1, i = idx - r * kRopeN1;
      hdst[idx] = tab[(int64_t)((rl.gr0 + r) % gh) * (kD / 2) + kRopeSplit0 + i];
    }
    double2* wdst = hdst + pp.lds_heights * kRopeN1;
    for (int idx = t; idx < gw * kRopeN2; idx += nt) {
      const int r = idx / kRopeN2, i = idx - r * kRopeN2;
      wdst[idx] = tab[(int64_t)r * (kD / 2) + kRopeSplit1 + i];
    }
  }
  __syncthreads();
  return rl;
}

// n / d for 0 <= n < 2^24, 1 <= d: the fp32 quotient is off by at most one, fixed by the remainder test
__device__ __forceinline__ int small_div(int n, int d, int* rem) {
  int q = (int)(__int2float_rn(n) * __frcp_rn(__int2float_rn(d)));
  int r = n - q * d;
  if (r < 0) {
    --q;
    r += d;
  } else if (r >= d) {
    ++q;
    r -= d;
  }
  *rem = r;
  return q;
}

template <int M>
__device__ __forceinline__ float lane_xor(float v);

// The Qwen-Image block's step before attention on the 16 channels [16*c16, 16*c16+16) of one head of token `row`
// (the 8 lanes c16 = 0..7 of the row are adjacent):
//   y = half( (x * r) * weight[ch] ),  r = 1 / sqrt(mean_{128 channels}(x^2) + eps)
//       mean: every lane adds its 16 squares in channel order, the 8 lane sums meet in an adjacent-pair tree
//   (y[2i], y[2i+1]) -> half( (y[2i] + i*y[2i+1]) * freqs[row, i] )    complex64: four products, one subtraction and
//       one addition, each rounded to fp32
template <int DT>
__device__ __forceinline__ void prep16_qwen(float* x, const PrepParams& pp, int row, int c16) {
  const bool txt = row < pp.txt_len;
  const float* w = txt ? pp.weight_txt : pp.weight_img;
  if (w != nullptr) {
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; ++e) ss = e == 0 ? x[0] * x[0] : ss + x[e] * x[e];  // squares of half values are exact
    ss = ss + lane_xor<1>(ss);
    ss = ss + lane_xor<2>(ss);
    ss = ss + lane_xor<4>(ss);
    const float r = __fdiv_rn(1.0f, sqrtf(__fdiv_rn(ss, (float)kD) + pp.eps));
    const float4* w4 = reinterpret_cast<const float4*>(w + c16 * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float4 wj = w4[j];
      x[4 * j + 0] = (x[4 * j + 0] * r) * wj.x;
      x[4 * j + 1] = (x[4 * j + 1] * r) * wj.y;
      x[4 * j + 2] = (x[4 * j + 2] * r) * wj.z;
      x[4 * j + 3] = (x[4 * j + 3] * r) * wj.w;
      through_half2<DT>(x[4 * j + 0], x[4 * j + 1]);
      through_half2<DT>(x[4 * j + 2], x[4 * j + 3]);
    }
  }
  const float2* tab = txt ? pp.freqs_txt : pp.freqs_img;
  if (tab != nullptr) {
    const float4* t4 = reinterpret_cast<const float4*>(tab + (int64_t)(txt ? row : row - pp.txt_len) * (kD / 2) + c16 * 8);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float4 cs = t4[j];  // two factors: (re, im), (re, im)
      const float a0 = x[4 * j], b0 = x[4 * j + 1], a1 = x[4 * j + 2], b1 = x[4 * j + 3];
      x[4 * j + 0] = a0 * cs.x - b0 * cs.y;
      x[4 * j + 1] = a0 * cs.y + b0 * cs.x;
      x[4 * j + 2] = a1 * cs.z - b1 * cs.w;
      x[4 * j + 3] = a1 * cs.w + b1 * cs.z;
      through_half2<DT>(x[4 * j + 0], x[4 * j + 1]);
      through_half2<DT>(x[4 * j + 2], x[4 * j + 3]);
    }
  }
}

// The pieces of the Wan step on the 16 channels of a lane.
//   norm16:   y = half( (x * r) * weight[ch] ), r the row's 1 / sqrt(mean(x^2) + eps)
template <int DT>
__device__ __forceinline__ void norm16(float* x, float r, const float* w16) {
  const float4* w4 = reinterpret_cast<const float4*>(w16);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float4 w = w4[j];
    x[4 * j + 0] = (x[4 * j + 0] * r) * w.x;
    x[4 * j + 1] = (x[4 * j + 1] * r) * w.y;
    x[4 * j + 2] = (x[4 * j + 2] * r) * w.z;
    x[4 * j + 3] = (x[4 * j + 3] * r) * w.w;
    through_half2<DT>(x[4 * j + 0], x[4 * j + 1]);
    through_half2<DT>(x[4 * j + 2], x[4 * j + 3]);
  }
}
//   rotate_pair: (a, b) -> half( float( (a + i b) * (c + i s) ) ) in fp64, unfused
template <int DT>
__device__ __forceinline__ void rotate_pair(float& xa, float& xb, const double2 cs) {
  const double a = (double)xa, bb = (double)xb;
  const double re = a * cs.x - bb * cs.y;
  const double im = a * cs.y + bb * cs.x;
  xa = (float)re;
  xb = (float)im;
  through_half2<DT>(xa, xb);
}
//   comfy_pair: apply_comfyui_rope (utils/rope.py:180-212): out[2i+e] = m[e][0] * x[2i] + m[e][1] * x[2i+1] in fp32, the
//   first product rounded on its own, the second fused into the sum (what torch's mul followed by addcmul_ computes)
template <int DT>
__device__ __forceinline__ void comfy_pair(float& xa, float& xb, const float4 m) {
  const float a = xa, bb = xb;
  xa = __fmaf_rn(m.y, bb, __fmul_rn(m.x, a));
  xb = __fmaf_rn(m.w, bb, __fmul_rn(m.z, a));
  through_half2<DT>(xa, xb);
}

// Where the 8 rotation factors of lane c16 (pairs 8 * c16 + j) sit for a token at (frame f, image row hi, column wi):
// two of the table's three segments at most, the second from pair `split` on.  first / second are element indices of
// pair 8 * c16 + 0 as if the whole lane lay in that segment (the table is [position][64 pairs]).
struct RopeLaneIndex {
  int first, second, split;
};
__device__ __forceinline__ RopeLaneIndex rope_lane_index(int c16, int base_f, int base_h, int base_w) {
  const int i0 = c16 * 8, i7 = c16 * 8 + 7;
  RopeLaneIndex r;
  r.first = (i0 < kRopeSplit0 ? base_f : (i0 < kRopeSplit1 ? base_h : base_w)) + i0;
  r.second = (i7 < kRopeSplit0 ? base_f : (i7 < kRopeSplit1 ? base_h : base_w)) + i0;
  // pairs [0, 22) frame, [22, 43) image row, [43, 64) column: lane 2 changes segment at pair 22, lane 5 at pair 43
  r.split = c16 == 2 ? kRopeSplit0 - 16 : (c16 == 5 ? kRopeSplit1 - 40 : 8);
  return r;
}

// KIND: PrepParams::kind, a template argument so that every kernel instantiation carries the registers of its own
// variant only (with a run-time switch the three variants' table reads add up).
template <int DT, int KIND>
__device__ __forceinline__ void prep16(float* x, const PrepParams& pp, const RopeLds& rl, int b, int row, int h,
                                       int c16, bool staged = true, const float* row_rms = nullptr) {
  if constexpr (KIND == 2) {
    prep16_qwen<DT>(x, pp, row, c16);
    return;
  }
  if (pp.inv_rms != nullptr) {
    // (row_rms: the row's statistic where the caller holds it already, e.g. in LDS)
    const float r = row_rms != nullptr ? *row_rms : pp.inv_rms[(int64_t)b * pp.L + row];
    norm16<DT>(x, r, pp.weight + h * kD + c16 * 16);
  }
  if constexpr (KIND == 3) {
    if (pp.rot != nullptr && row < pp.rot_rows) {
      const float4* m4 = pp.rot + (int64_t)row * (kD / 2) + c16 * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) comfy_pair<DT>(x[2 * j], x[2 * j + 1], m4[j]);
    }
    return;
  }
  if (pp.freqs != nullptr) {
    const int gh = pp.grid[b][1], gw = pp.grid[b][2];
    const int plane = gh * gw;
    if (row < pp.grid[b][0] * plane) {
      int rem, wi;
      const int f = small_div(row, plane, &rem);
      const int hi = small_div(rem, gw, &wi);
      // one table, three segments; a lane's 8 pairs lie in two of them at most
      auto rotate = [&](const double2* tab, int base_f, int base_h, int base_w) {
        const RopeLaneIndex li = rope_lane_index(c16, base_f, base_h, base_w);
#pragma unroll
        for (int j = 0; j < 8; ++j) rotate_pair<DT>(x[2 * j], x[2 * j + 1], tab[(j < li.split ? li.first : li.second) + j]);
      };
      if (pp.lds_frames > 0 && staged)  // uniform (staged == false: a row outside the rows `rl` was staged for)
        rotate(rl.frame, (f - rl.f0) * kRopeN0,
               (int)(rl.height - rl.frame) + (f * gh + hi - rl.gr0) * kRopeN1 - kRopeSplit0,
               (int)(rl.width - rl.frame) + wi * kRopeN2 - kRopeSplit1);
      else
        rotate(reinterpret_cast<const double2*>(pp.freqs), f * (kD / 2), hi * (kD / 2), wi * (kD / 2));
    }
  }
}

// Dynamic LDS of the kernels that rotate: the staged factors.
extern __shared__ __attribute__((aligned(16))) double2 s_rope_tables[];

template <int PRE>
__device__ __forceinline__ RopeLds maybe_stage_rope(const PrepParams& pp, int b, int row0, int nrows) {
  RopeLds rl{};
  if constexpr (PRE == 1) {
    if (pp.freqs != nullptr && pp.lds_frames > 0) rl = stage_rope(pp, b, row0, nrows, s_rope_tables);
  }
  return rl;
}

// 1 / sqrt(mean(x^2) + eps) of every token row x[b, l, 0 : n8*8].  One wave per row: lane i takes the
// groups of 8 channels i, i+64, i+128, ... in order, adding the 8 squares of each one after the other
// (fp32, squares of half values are exact); the 64 lane sums meet in an adjacent-pair tree.  The order
// is part of the result.  grid = (ceil(L / 4), B), 256 threads.
// the statistic of one row, by one wave (every lane returns it)
template <int DT>
__device__ __forceinline__ float row_inv_rms_of(const uint16_t* base, int n8, float n_channels, float eps, int lane) {
  float acc = 0.0f;
  for (int g = lane; g < n8; g += 64) {
    float v[8];
    widen8<DT>(*reinterpret_cast<const uint4*>(base + g * 8), v);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = acc + v[e] * v[e];
  }
#pragma unroll
  for (int m = 1; m <= 32; m <<= 1) acc = acc + __shfl_xor(acc, m);
  // sqrtf, not __fsqrt_rn: the latter is the 1-ulp native instruction in this toolchain, the former is
  // correctly rounded (the build passes -fhip-fp32-correctly-rounded-divide-sqrt)
  return __fdiv_rn(1.0f, sqrtf(__fdiv_rn(acc, n_channels) + eps));
}

template <int DT>
__global__ __launch_bounds__(kThreads) void row_inv_rms_kernel(const uint16_t* __restrict__ x, int64_t sB, int64_t sL,
                                                               int L, int n8, float n_channels, float eps,
                                                               float* __restrict__ inv_rms) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), b = blockIdx.y;
  if (row >= L) return;
  const float r = row_inv_rms_of<DT>(x + b * sB + (int64_t)row * sL, n8, n_channels, eps, lane);
  if (lane == 0) inv_rms[(int64_t)b * L + row] = r;
}

// ---------------------------------------------------------------------------------------
// Column reduction over a chunk of 256 rows.  OP 0: fp32 sum in the frozen order (slot i%32
// sequential over the chunk's 8 row groups, then an adjacent-pair tree over the 32 slots).
// OP 1: max |x| (order free).  OP 2: max |x - centre[d]| over the rows that exist (V smoothing: the
// centre is the channel mean).  grid = (nch, H, B).
// ---------------------------------------------------------------------------------------
template <int DT, int OP, int PRE>
__global__ __launch_bounds__(kThreads) void col_partial_kernel(const uint16_t* __restrict__ x, int64_t sB, int64_t sL,
                                                               int64_t sH, int H, int L_all, int d_in, float* __restrict__ part,
                                                               int nch, const PrepParams pp,
                                                               const float* __restrict__ centre) {
  constexpr bool kSum = OP == 0;
  const int ch = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const uint16_t* base = x + b * sB + h * sH + c16 * 16;
  const RopeLds rl = maybe_stage_rope<PRE>(pp, b, ch * kMeanChunk, kMeanChunk);
  float acc[16];
  if constexpr (PRE) {
    float rows[kMeanChunk / kSlots][16];
#pragma unroll
    for (int i = 0; i < kMeanChunk / kSlots; ++i) {
      const int row = ch * kMeanChunk + i * kSlots + slot;
      load_row16<DT>(base + (int64_t)row * sL, row < L, rows[i]);
      if (row < L) prep16<DT, PRE>(rows[i], pp, rl, b, row, h, c16);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = kSum ? rows[0][e] : fabsf(rows[0][e]);
#pragma unroll
    for (int i = 1; i < kMeanChunk / kSlots; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = kSum ? acc[e] + rows[i][e] : fmaxf(acc[e], fabsf(rows[i][e]));
    }
  } else {
    // all sixteen loads of the lane are issued first and stay in flight as 16-bit values; they are widened and
    // folded in row order as they arrive (keeping them as fp32 costs twice the registers and a wave per SIMD)
    uint4 raw[kMeanChunk / kSlots][2];
#pragma unroll
    for (int i = 0; i < kMeanChunk / kSlots; ++i) {
      const int row = ch * kMeanChunk + i * kSlots + slot;
      raw[i][0] = raw[i][1] = make_uint4(0, 0, 0, 0);
      if (row < L) {
        raw[i][0] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL);
        raw[i][1] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL + 8);
      }
    }
    float cen[16];
    if constexpr (OP == 2) {
#pragma unroll
      for (int e = 0; e < 16; ++e) cen[e] = centre[((int64_t)b * H + h) * kD + c16 * 16 + e];
    }
#pragma unroll
    for (int i = 0; i < kMeanChunk / kSlots; ++i) {
      const int row = ch * kMeanChunk + i * kSlots + slot;
      float x[16];
      widen8<DT>(raw[i][0], x);
      widen8<DT>(raw[i][1], x + 8);
      if constexpr (OP == 2) {
        if (row < L) {
#pragma unroll
          for (int e = 0; e < 16; ++e) x[e] = x[e] - cen[e];
        }
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if (i == 0)
          acc[e] = kSum ? x[e] : fabsf(x[e]);
        else
          acc[e] = kSum ? acc[e] + x[e] : fmaxf(acc[e], fabsf(x[e]));
      }
    }
  }
  // slots of one wave differ in lane bits 3..5
#pragma unroll
  for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float o = __shfl_xor(acc[e], m);
      acc[e] = kSum ? acc[e] + o : fmaxf(acc[e], o);
    }
  }
  __shared__ float s_w[4][kD];
  const int wave = t >> 6, lane = t & 63;
  if (lane < 8) {
#pragma unroll
    for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = acc[e];
  }
  __syncthreads();
  if (t < kD) {
    const float lo = kSum ? s_w[0][t] + s_w[1][t] : fmaxf(s_w[0][t], s_w[1][t]);
    const float hi = kSum ? s_w[2][t] + s_w[3][t] : fmaxf(s_w[2][t], s_w[3][t]);
    part[(((int64_t)b * H + h) * nch + ch) * kD + t] = kSum ? lo + hi : fmaxf(lo, hi);
  }
}

// Finalisation of the column reductions.  grid = B*H, 1024 threads.  All chunk partials of the
// head are first pulled into LDS with independent, coalesced loads (the naive form - one
// dependent global load per chunk - costs a memory latency per chunk); 128 threads then combine
// them in increasing chunk order, which for the sum is part of the specification.
constexpr int kFinThreads = 1024;
constexpr int kFinMaxChunks = 96;  // partials staged per pass: 96 x 128 floats = 48 KiB of LDS

template <int OP>
__device__ __forceinline__ float combine_partials(const float* __restrict__ part, int nch, float* s_part) {
  const int d = threadIdx.x & (kD - 1);
  float acc = 0.0f;
  bool first = true;
  for (int c0 = 0; c0 < nch; c0 += kFinMaxChunks) {
    const int n = min(kFinMaxChunks, nch - c0);
    __syncthreads();
    // 96 x 128 floats by 1024 threads: twelve independent loads each, all in flight together
    float v[kFinMaxChunks * kD / kFinThreads];
#pragma unroll
    for (int j = 0; j < kFinMaxChunks * kD / kFinThreads; ++j) {
      const int idx = (int)threadIdx.x + kFinThreads * j;
      v[j] = idx < n * kD ? part[(int64_t)c0 * kD + idx] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < kFinMaxChunks * kD / kFinThreads; ++j) s_part[(int)threadIdx.x + kFinThreads * j] = v[j];
    __syncthreads();
    if (threadIdx.x < kD) {
      int c = 0;
      if (first) {
        acc = s_part[d];
        first = false;
        c = 1;
      }
      // chunk order is part of the specification for the sum; batches of 16 keep the LDS reads ahead of the adds
      for (; c + 16 <= n; c += 16) {
        float w[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i] = s_part[(c + i) * kD + d];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc = OP == 0 ? acc + w[i] : fmaxf(acc, w[i]);
      }
      for (; c < n; ++c) acc = OP == 0 ? acc + s_part[c * kD + d] : fmaxf(acc, s_part[c * kD + d]);
    }
  }
  return acc;
}

// chunk sums -> mean rounded to the input dtype, stored widened
__global__ __launch_bounds__(kFinThreads) void k_mean_finalize_kernel(const float* __restrict__ part, int nch, int L,
                                                                      int dtype, int smooth,
                                                                      float* __restrict__ k_mean, int* status) {
  __shared__ float s_part[kFinMaxChunks * kD];
  const int bh = blockIdx.x;
  if (status != nullptr && bh == 0 && threadIdx.x == 0) *status = 0;  // this path has no wait that could expire
  const float tot = combine_partials<0>(part + (int64_t)bh * nch * kD, nch, s_part);
  if (threadIdx.x < kD) {
    const float mean = __fdiv_rn(tot, (float)L);
    k_mean[bh * kD + threadIdx.x] = smooth ? round_to_half_dtype(mean, dtype) : 0.0f;
  }
}

// chunk abs-max -> scale and its inverse; `zero_mean` (optional) is the mean slot to clear when V is not smoothed
__global__ __launch_bounds__(kFinThreads) void v_scale_finalize_kernel(const float* __restrict__ part, int nch,
                                                                       float* __restrict__ v_scale,
                                                                       float* __restrict__ v_inv,
                                                                       float* __restrict__ zero_mean, int* status) {
  __shared__ float s_part[kFinMaxChunks * kD];
  const int bh = blockIdx.x;
  if (status != nullptr && bh == 0 && threadIdx.x == 0) *status = 0;
  const float amax = combine_partials<1>(part + (int64_t)bh * nch * kD, nch, s_part);
  if (threadIdx.x < kD) {
    const bool nz = amax > 0.0f;
    v_scale[bh * kD + threadIdx.x] = nz ? __fdiv_rn(amax, 448.0f) : 0.0f;
    v_inv[bh * kD + threadIdx.x] = nz ? __fdiv_rn(448.0f, amax) : 0.0f;
    if (zero_mean != nullptr) zero_mean[bh * kD + threadIdx.x] = 0.0f;
  }
}

// Value of lane (id ^ M) for M = 1, 2, 4, through DPP (the exchange then rides on the consuming
// VALU instruction instead of a round trip through the LDS crossbar).
//   quad_perm [1,0,3,2] = id ^ 1;  quad_perm [2,3,0,1] = id ^ 2;
//   row_half_mirror (id -> 7 - id within 8 lanes) followed by quad_perm [3,2,1,0] (id ^ 3) = id ^ 4.
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
  static_assert(M == 1 || M == 2 || M == 4, "only within groups of 8 lanes");
  const int iv = __float_as_int(v);
  if constexpr (M == 1) return __int_as_float(__builtin_amdgcn_mov_dpp(iv, 0xB1, 0xF, 0xF, true));
  if constexpr (M == 2) return __int_as_float(__builtin_amdgcn_mov_dpp(iv, 0x4E, 0xF, 0xF, true));
  const int t = __builtin_amdgcn_mov_dpp(iv, 0x141, 0xF, 0xF, true);
  return __int_as_float(__builtin_amdgcn_mov_dpp(t, 0x1B, 0xF, 0xF, true));
}

// One butterfly stage across lanes c16 and c16 ^ M: every lane takes `own + sign * other` with sign = -1 on the lane
// that holds the "b" half of a pair.  That lane ought to take `other - own`: it ends up with the negative of its
// value, exactly (a sum and its mirror image round alike).  Both lanes of any LATER stage's pair agree in bit M of
// c16, so they carry the same factor and the later butterfly is the mirror image of the right one as a whole: after
// the three stages a lane holds its transform times (-1)^popcount(c16), which the caller folds into the factor it
// multiplies with next (fwht_lane_sign).  Written this way the stage is one multiply-add per value whose first
// operand arrives through DPP - no separate sign flip, and no register written just ahead of the DPP read.
// The instruction is written out: the compiler keeps the DPP move and the multiply-add apart (two instructions per
// value).  Eight values per statement; `s_nop 1` in front gives the two wait states a DPP read needs after a
// vector-ALU write of the same register, whatever instruction the compiler placed just before; inside a statement
// every register is read at least eight instructions after it was written.
#define KSANA_FMAC_DPP8(CTRL)                                                                                      \
  "v_fmac_f32_dpp %0, %0, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %1, %1, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %2, %2, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %3, %3, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %4, %4, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %5, %5, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %6, %6, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"                                 \
  "v_fmac_f32_dpp %7, %7, %8 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1"
template <int M>
__device__ __forceinline__ void fwht_cross_stage(float* x, int c16) {
  const float sign = (c16 & M) ? -1.0f : 1.0f;
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    float* y = x + 8 * g;
    if constexpr (M == 1) {
      asm volatile("s_nop 1\n\t" KSANA_FMAC_DPP8("quad_perm:[1,0,3,2]")
                   : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]), "+v"(y[4]), "+v"(y[5]), "+v"(y[6]), "+v"(y[7])
                   : "v"(sign));
    } else if constexpr (M == 2) {
      asm volatile("s_nop 1\n\t" KSANA_FMAC_DPP8("quad_perm:[2,3,0,1]")
                   : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]), "+v"(y[4]), "+v"(y[5]), "+v"(y[6]), "+v"(y[7])
                   : "v"(sign));
    } else {
      // lane ^ 4 within 8 = row_half_mirror (lane -> 7 - lane) followed by quad_perm [3,2,1,0] (lane ^ 3)
      float t[8];
      asm volatile("s_nop 1\n\t"
                   "v_mov_b32_dpp %8, %0 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %9, %1 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %10, %2 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %11, %3 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %12, %4 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %13, %5 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %14, %6 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %15, %7 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %0, %8, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %1, %9, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %2, %10, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %3, %11, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %4, %12, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %5, %13, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %6, %14, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %7, %15, %16 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1"
                   : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]), "+v"(y[4]), "+v"(y[5]), "+v"(y[6]), "+v"(y[7]),
                     "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3]), "=&v"(t[4]), "=&v"(t[5]), "=&v"(t[6]), "=&v"(t[7])
                   : "v"(sign));
    }
  }
}

// The factor fwht128 leaves on the values of lane c16 (see fwht_cross_stage).
__device__ __forceinline__ float fwht_lane_sign(int c16) { return (__popc(c16 & 7) & 1) ? -1.0f : 1.0f; }

// Unnormalised Walsh-Hadamard transform of one 128-channel row held by 8 adjacent lanes x 16
// values (channel = 16*c16 + e), TIMES fwht_lane_sign(c16).  Butterflies (a, b) -> (a + b, a - b) with stride 1, 2,
// 4, 8 inside the lane, then 16, 32, 64 across lanes c16 ^ 1, ^ 2, ^ 4 - in exactly that order.
__device__ __forceinline__ void fwht128(float* x, int c16) {
#pragma unroll
  for (int s = 1; s < 16; s <<= 1) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if ((i & s) == 0) {
        const float a = x[i], b = x[i + s];
        x[i] = a + b;
        x[i + s] = a - b;
      }
    }
  }
  fwht_cross_stage<1>(x, c16);
  fwht_cross_stage<2>(x, c16);
  fwht_cross_stage<4>(x, c16);
}

// max over the workgroup of a non-negative per-thread value
__device__ __forceinline__ float block_max(float v, float* s_red) {
#pragma unroll
  for (int m = 1; m <= 32; m <<= 1) v = fmaxf(v, __shfl_xor(v, m));
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) s_red[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
}

// rne(x * inv) as int8, sixteen at a time, the product exact: one fused multiply-add onto 1.5 * 2^23, where the fp32
// grid is the integers, rounds the exact sum to nearest, ties to even, and leaves the two's-complement int8 in the low
// byte.  No clamp: |x| <= amax and inv = fl(127 / amax) keep |x * inv| below 127.5.  One instruction per value plus
// three byte-gathers per four.
__device__ __forceinline__ uint4 pack_int8x16(const float* x, float inv) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t z[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) z[j] = __float_as_uint(__fmaf_rn(x[4 * i + j], inv, 12582912.0f));
    const uint32_t lo = __builtin_amdgcn_perm(z[1], z[0], 0x0c0c0400u);  // bytes 0, 1 <- low bytes of z0, z1
    const uint32_t hi = __builtin_amdgcn_perm(z[3], z[2], 0x04000c0cu);  // bytes 2, 3 <- low bytes of z2, z3
    w[i] = lo | hi;
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Block mean from per-thread partial sums (thread = row slot x 16 channels; a slot has added its rows in increasing
// order): the 32 slots meet in an adjacent-pair tree - three steps inside a wave, the four waves through LDS - the sum
// is divided by the number of rows that exist and rounded to the half type.  The frozen order of the block averages
// (block_mean_kernel); the quantizers that take a block's average along use the same code, hence give the same bits.
template <int DT>
__device__ __forceinline__ void store_block_mean(float (&acc)[16], int t, float n_rows, uint16_t* __restrict__ out_row,
                                                 float (*s_w)[kD]) {
  const int c16 = t & 7;
#pragma unroll
  for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = acc[e] + __shfl_xor(acc[e], m);
  }
  const int wave = t >> 6, lane = t & 63;
  if (lane < 8) {
#pragma unroll
    for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = acc[e];
  }
  __syncthreads();
  if (t < kD) {
    const float sum = (s_w[0][t] + s_w[1][t]) + (s_w[2][t] + s_w[3][t]);
    const float mean = __fdiv_rn(sum, n_rows);
    uint16_t bits;
    if constexpr (DT == KSANA_SAGE_BF16) {
      bits = __builtin_bit_cast(uint16_t, (__bf16)mean);
    } else {
      bits = __builtin_bit_cast(uint16_t, (_Float16)mean);
    }
    out_row[t] = bits;
  }
}

// ---------------------------------------------------------------------------------------
// Q: Hadamard transform, fold sm_scale*log2(e)/128, one int8 scale per query row.  One
// workgroup handles 128 rows (4 per row slot).  grid = (lq_pad/128, H, B).  Output row-major
// int8 [B, H, lq_pad, 128] and fp32 [B, H, lq_pad]; rows at or beyond L come out as zeros.
// ---------------------------------------------------------------------------------------
// POOL: the workgroup's 128 rows are one block of the sparse-linear backend's block map; their average (of the input
// as it is) goes to pooled[b, h, blk, :] - what block_mean_kernel would read q a second time for.
template <int DT, int PRE, bool POOL = false>
__global__ __launch_bounds__(kThreads) void quant_q_kernel(const uint16_t* __restrict__ q, int64_t sB, int64_t sL,
                                                           int64_t sH, int H, int L_all, int d_in, int lq_pad, float premul,
                                                           int8_t* __restrict__ q_i8, float* __restrict__ q_scale,
                                                           const PrepParams pp, uint16_t* __restrict__ pooled = nullptr) {
  static_assert(!(POOL && PRE), "block averages are taken of the tensor as it is");
  const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const uint16_t* base = q + b * sB + h * sH + c16 * 16;
  constexpr int kRowsPerWg = 128, R = kRowsPerWg / kSlots;
  const int64_t bh = (int64_t)b * H + h;
  const RopeLds rl = maybe_stage_rope<PRE>(pp, b, blk * kRowsPerWg, kRowsPerWg);
  const float premul_lane = premul * fwht_lane_sign(c16);
  auto finish_row = [&](float* xr, int row) {
    fwht128(xr, c16);
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      xr[e] = xr[e] * premul_lane;
      amax = fmaxf(amax, fabsf(xr[e]));
    }
    amax = fmaxf(amax, lane_xor<1>(amax));
    amax = fmaxf(amax, lane_xor<2>(amax));
    amax = fmaxf(amax, lane_xor<4>(amax));
    const bool nz = amax > 0.0f;
    const float inv = nz ? __fdiv_rn(127.0f, amax) : 0.0f;
    if (c16 == 0) q_scale[bh * lq_pad + row] = nz ? __fdiv_rn(amax, 127.0f) : 0.0f;
    store_out16(q_i8 + (bh * lq_pad + row) * kD + c16 * 16, pack_int8x16(xr, inv));
  };
  if constexpr (PRE) {
    // The norm and the rotation are arithmetic-heavy (vector fp64): one row at a time with only the next row's two
    // loads in flight keeps the kernel at half the registers of "load all, then work", i.e. at twice the waves.
    uint4 nxt[2];
    fetch_row16(base + (int64_t)(blk * kRowsPerWg + slot) * sL, blk * kRowsPerWg + slot < L, nxt);
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int row = blk * kRowsPerWg + i * kSlots + slot;
      const uint4 cur0 = nxt[0], cur1 = nxt[1];
      if (i + 1 < R) fetch_row16(base + (int64_t)(row + kSlots) * sL, row + kSlots < L, nxt);
      float xr[16];
      widen8<DT>(cur0, xr);
      widen8<DT>(cur1, xr + 8);
      if (row < L) prep16<DT, PRE>(xr, pp, rl, b, row, h, c16);
      finish_row(xr, row);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    float x[R][16];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int row = blk * kRowsPerWg + i * kSlots + slot;
      load_row16<DT>(base + (int64_t)row * sL, row < L, x[i]);
    }
    if constexpr (POOL) {
      float acc[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = ((x[0][e] + x[1][e]) + x[2][e]) + x[3][e];
      static_assert(R == 4, "four rows per slot");
      __shared__ float s_w[4][kD];
      store_block_mean<DT>(acc, t, (float)min(kRowsPerWg, L_all - blk * kRowsPerWg),
                           pooled + (bh * gridDim.x + blk) * kD, s_w);
    }
#pragma unroll
    for (int i = 0; i < R; ++i) finish_row(x[i], blk * kRowsPerWg + i * kSlots + slot);
  }
}

// ---------------------------------------------------------------------------------------
// Q with a norm over the whole token row folded in (Wan), from ONE pass over HBM.  A workgroup takes 8 whole token
// rows, all heads.  First their statistics, as row_inv_rms_kernel takes them (one wave per row, two rows per wave,
// both at a time) - and, where the caller passes k, the statistics of the same rows of k, whose own quantizer then
// needs no statistic pass of its own.  Then the heads, four at a time: a row slot is (row, one of four heads), 8 lanes
// x 16 channels each, the next four heads' loads in flight while these are normed, rotated, transformed and packed.
// The rows are read a second time there, microseconds after the first: from the caches, not from HBM.  Small
// workgroups on purpose: several generations of them pass through a compute unit, so the memory-bound statistics of
// some run next to the arithmetic-bound heads of others.
// grid = (ceil(max(lq_pad, k_L) / 8), B).
// ---------------------------------------------------------------------------------------
constexpr int kRowsQ = 8;                   // token rows per workgroup
constexpr int kHeadsQ = kSlots / kRowsQ;    // heads in work at a time: 4
struct RowStatOf {  // the rows of another tensor whose statistic the kernel takes along (ptr == nullptr: none)
  const uint16_t* ptr;
  int64_t sB, sL;
  int L, n8;
  float n_channels;
  float* inv_rms;  // [B, L]
};

template <int DT, int KIND>
__global__ __launch_bounds__(kThreads) void quant_q_rows_kernel(const uint16_t* __restrict__ q, int64_t sB, int64_t sL,
                                                                int64_t sH, int H, int L, int lq_pad, float premul,
                                                                float eps, int8_t* __restrict__ q_i8,
                                                                float* __restrict__ q_scale, const PrepParams pp,
                                                                float* __restrict__ rms_out, const RowStatOf ks) {
  const int r0 = blockIdx.x * kRowsQ, b = blockIdx.y;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int wave = t >> 6, lane = t & 63;
  __shared__ float s_rms[kRowsQ];
  // ---- the rows' statistics: wave w takes rows 2 w and 2 w + 1 together (every row's sum adds its groups of 8
  // channels in the order of row_inv_rms_of) -------------------------------------------------------------------
  auto stats = [&](const uint16_t* x, int64_t xsB, int64_t xsL, int xL, int n8, float n_channels, float* out, bool keep) {
    constexpr int R = kRowsQ / 4;
    const int first = r0 + wave * R;
    if (first >= xL) return;  // wave-uniform
    const uint16_t* rbase = x + b * xsB + (int64_t)first * xsL;
    float acc[R];
#pragma unroll
    for (int i = 0; i < R; ++i) acc[i] = 0.0f;
#pragma unroll 4
    for (int g = lane; g < n8; g += 64) {
      uint4 raw[R];
#pragma unroll
      for (int i = 0; i < R; ++i)
        raw[i] = first + i < xL ? *reinterpret_cast<const uint4*>(rbase + i * xsL + g * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < R; ++i) {
        float v[8];
        widen8<DT>(raw[i], v);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i] = acc[i] + v[e] * v[e];
      }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
      float a = acc[i];
#pragma unroll
      for (int m = 1; m <= 32; m <<= 1) a = a + __shfl_xor(a, m);
      const float r = __fdiv_rn(1.0f, sqrtf(__fdiv_rn(a, n_channels) + eps));
      if (lane == 0 && first + i < xL) {
        out[(int64_t)b * xL + first + i] = r;
        if (keep) s_rms[wave * R + i] = r;
      }
    }
  };
  stats(q, sB, sL, L, H * (kD / 8), (float)(H * kD), rms_out, true);
  if (ks.ptr != nullptr) stats(ks.ptr, ks.sB, ks.sL, ks.L, ks.n8, ks.n_channels, ks.inv_rms, false);
  if (r0 >= lq_pad) return;  // rows that exist only in k
  __syncthreads();
  // ---- the heads, four at a time ------------------------------------------------------------------------------
  const int rloc = slot & (kRowsQ - 1), h0 = slot / kRowsQ;
  const int row = r0 + rloc;
  const bool live = row < L;
  // A token's rotation is the same for every head: the lane's 8 factors (pairs 8 * c16 + j of its row) are fetched
  // once, straight from the model's table (1 MiB, cache resident), and stay in registers for the whole head walk.
  bool rotates = false;
  double2 cs[KIND == 1 ? 8 : 1];
  float4 rm[KIND == 3 ? 8 : 1];
  if constexpr (KIND == 1) {
    if (pp.freqs != nullptr && live) {
      const int gh = pp.grid[b][1], gw = pp.grid[b][2], plane = gh * gw;
      if (row < pp.grid[b][0] * plane) {
        rotates = true;
        int rem, wi;
        const int f = small_div(row, plane, &rem);
        const int hi = small_div(rem, gw, &wi);
        const RopeLaneIndex li = rope_lane_index(c16, f * (kD / 2), hi * (kD / 2), wi * (kD / 2));
        const double2* tab = reinterpret_cast<const double2*>(pp.freqs);
#pragma unroll
        for (int j = 0; j < 8; ++j) cs[j] = tab[(j < li.split ? li.first : li.second) + j];
      }
    }
  } else {
    if (pp.rot != nullptr && live && row < pp.rot_rows) {
      rotates = true;
      const float4* m4 = pp.rot + (int64_t)row * (kD / 2) + c16 * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) rm[j] = m4[j];
    }
  }
  const float rinv = s_rms[rloc];
  const uint16_t* base = q + b * sB + (int64_t)row * sL + c16 * 16;
  const float premul_lane = premul * fwht_lane_sign(c16);
  uint4 nxt[2];
  fetch_row16(base + (int64_t)h0 * sH, live && h0 < H, nxt);
  for (int h = h0; h < H; h += kHeadsQ) {
    const uint4 cur0 = nxt[0], cur1 = nxt[1];
    if (h + kHeadsQ < H) fetch_row16(base + (int64_t)(h + kHeadsQ) * sH, live, nxt);
    float xr[16];
    widen8<DT>(cur0, xr);
    widen8<DT>(cur1, xr + 8);
    if (live) {
      norm16<DT>(xr, rinv, pp.weight + h * kD + c16 * 16);
      if (rotates) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if constexpr (KIND == 1) rotate_pair<DT>(xr[2 * j], xr[2 * j + 1], cs[j]);
          else comfy_pair<DT>(xr[2 * j], xr[2 * j + 1], rm[j]);
        }
      }
    }
    fwht128(xr, c16);
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      xr[e] = xr[e] * premul_lane;
      amax = fmaxf(amax, fabsf(xr[e]));
    }
    amax = fmaxf(amax, lane_xor<1>(amax));
    amax = fmaxf(amax, lane_xor<2>(amax));
    amax = fmaxf(amax, lane_xor<4>(amax));
    const bool nz = amax > 0.0f;
    const float inv = nz ? __fdiv_rn(127.0f, amax) : 0.0f;
    const int64_t bh = (int64_t)b * H + h;
    if (c16 == 0) q_scale[bh * lq_pad + row] = nz ? __fdiv_rn(amax, 127.0f) : 0.0f;
    store_out16(q_i8 + (bh * lq_pad + row) * kD + c16 * 16, pack_int8x16(xr, inv));
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ---------------------------------------------------------------------------------------
// K: subtract the channel mean, Hadamard transform, one int8 scale per 64-row block = one
// workgroup.  grid = (nkb, H, B).  The tile is written in the order
// the attention kernel's int8 MFMA consumes it: fragment (t = row/32, s = 32-channel step)
// is 64 lanes x 16 bytes, lane = 32*(16-channel half within the step) + row%32.
// ---------------------------------------------------------------------------------------
// POOL: the workgroup's 64 rows are one key block of the sparse-linear backend's block map; the average of
// k - mean(k), each difference rounded to the tensor's half type first as the reference forms it, goes to
// pooled[b, h, blk, :] - what block_mean_kernel would read k a third time for.
template <int DT, int PRE, bool POOL = false>
__global__ __launch_bounds__(kThreads) void quant_k_kernel(const uint16_t* __restrict__ k, int64_t sB, int64_t sL,
                                                           int64_t sH, int H, int L_all, int d_in, int nkb,
                                                           const float* __restrict__ k_mean,
                                                           int8_t* __restrict__ k_tiles, float* __restrict__ k_scale,
                                                           const PrepParams pp, uint16_t* __restrict__ pooled = nullptr) {
  static_assert(!(POOL && PRE), "block averages are taken of the tensor as it is");
  // Heads and batch entries from the last one down: this pass follows the column-sum pass over the same tensor, which
  // went upwards, so what that pass touched last - and the last-level cache may still hold - is read first.
  const int blk = blockIdx.x, h = (int)gridDim.y - 1 - (int)blockIdx.y, b = (int)gridDim.z - 1 - (int)blockIdx.z;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const int64_t bh = (int64_t)b * H + h;
  const uint16_t* base = k + b * sB + h * sH + c16 * 16;
  float km[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) km[e] = k_mean[bh * kD + c16 * 16 + e];
  constexpr int R = kBlkK / kSlots;
  const RopeLds rl = maybe_stage_rope<PRE>(pp, b, blk * kBlkK, kBlkK);
  float x[R][16];
  float amax = 0.0f;
  [[maybe_unused]] float pool_acc[16];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = blk * kBlkK + i * kSlots + slot;
    const bool valid = row < L;
    load_row16<DT>(base + (int64_t)row * sL, valid, x[i]);
    if constexpr (PRE) {
      if (valid) prep16<DT, PRE>(x[i], pp, rl, b, row, h, c16);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      x[i][e] = valid ? x[i][e] - km[e] : 0.0f;
    }
    if constexpr (POOL) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float d = valid ? through_half<DT>(x[i][e]) : 0.0f;
        pool_acc[e] = i == 0 ? d : pool_acc[e] + d;
      }
    }
    fwht128(x[i], c16);
#pragma unroll
    for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(x[i][e]));
  }
  if constexpr (POOL) {
    __shared__ float s_w[4][kD];
    store_block_mean<DT>(pool_acc, t, (float)min(kBlkK, L_all - blk * kBlkK), pooled + (bh * nkb + blk) * kD, s_w);
  }
  __shared__ float s_red[4];
  amax = block_max(amax, s_red);
  const bool nz = amax > 0.0f;
  const float inv = nz ? __fdiv_rn(127.0f, amax) : 0.0f;
  const float inv_lane = inv * fwht_lane_sign(c16);  // the transform left this lane's values times that sign
  if (t == 0) k_scale[bh * nkb + blk] = nz ? __fdiv_rn(amax, 127.0f) : 0.0f;
  int8_t* tile = k_tiles + (bh * nkb + blk) * (int64_t)kTileBytes;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int frag = i * 4 + (c16 >> 1);
    const int lane = (c16 & 1) * 32 + slot;
    store_out16(tile + (frag * 64 + lane) * 16, pack_int8x16(x[i], inv_lane));
  }
}

// ---------------------------------------------------------------------------------------
// V: one workgroup per 64-row block.  grid = (nkb, H, B).  Scales with 448/amax[d], converts
// to e4m3fn, transposes through LDS and writes the V^T tile in the order the fp8 MFMA
// consumes it: chunk (dt = d/32, tt = half of the 64 rows) is 64 lanes x 16 bytes,
// lane = 32*hh + d%32, byte r <-> row 32*tt + 8*(r/4) + 4*hh + r%4.
// ---------------------------------------------------------------------------------------
template <int DT, bool CENTRE>
__global__ __launch_bounds__(kThreads) void quant_v_kernel(const uint16_t* __restrict__ v, int64_t sB, int64_t sL,
                                                           int64_t sH, int H, int L_all, int d_in, int nkb,
                                                           const float* __restrict__ v_inv,
                                                           const float* __restrict__ v_mean,
                                                           uint8_t* __restrict__ v_tiles) {
  // (heads and batch entries from the last one down, like quant_k_kernel: the abs-max pass went upwards)
  const int blk = blockIdx.x, h = (int)gridDim.y - 1 - (int)blockIdx.y, b = (int)gridDim.z - 1 - (int)blockIdx.z;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const int64_t bh = (int64_t)b * H + h;
  const uint16_t* base = v + b * sB + h * sH + c16 * 16;
  constexpr int kStride = kD + 16;  // LDS row pitch in bytes
  __shared__ __attribute__((aligned(16))) uint8_t s_v[kBlkK * kStride];
  float inv[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) inv[e] = v_inv[bh * kD + c16 * 16 + e];
  float mean[16];
  if constexpr (CENTRE) {
#pragma unroll
    for (int e = 0; e < 16; ++e) mean[e] = v_mean[bh * kD + c16 * 16 + e];
  }
#pragma unroll
  for (int i = 0; i < kBlkK / kSlots; ++i) {
    const int r = i * kSlots + slot;
    const int row = blk * kBlkK + r;
    float x[16];
    load_row16<DT>(base + (int64_t)row * sL, row < L, x);
    if constexpr (CENTRE) {  // rows past the end stay zero
      if (row < L) {
#pragma unroll
        for (int e = 0; e < 16; ++e) x[e] = x[e] - mean[e];
      }
    }
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = fminf(fmaxf(x[4 * j + e] * inv[4 * j + e], -448.0f), 448.0f);
      int packed = 0;
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], packed, false);
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], packed, true);
      w[j] = (uint32_t)packed;
    }
    *reinterpret_cast<uint4*>(&s_v[r * kStride + c16 * 16]) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  __syncthreads();
  uint8_t* tile = v_tiles + (bh * nkb + blk) * (int64_t)kTileBytes;
#pragma unroll
  for (int i = 0; i < kTileBytes / 16 / kThreads; ++i) {
    const int oc = i * kThreads + t;
    const int dt = oc >> 7, tt = (oc >> 6) & 1, lane = oc & 63;
    const int hh = lane >> 5, d = dt * 32 + (lane & 31);
    uint32_t w[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint32_t acc = 0;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int row = 32 * tt + 8 * g + 4 * hh + c;
        acc |= (uint32_t)s_v[row * kStride + d] << (8 * c);
      }
      w[g] = acc;
    }
    store_out16(tile + oc * 16, make_uint4(w[0], w[1], w[2], w[3]));
  }
}


// ---------------------------------------------------------------------------------------
// One-read quantizers for K and V.
//
// The two-kernel form above reads K (and V) twice: once for the column statistic of the whole
// sequence, once to quantize.  Here a workgroup keeps its 256-row chunk in registers (as the 16-bit
// values it loaded: 64 registers per lane) across the point where the statistic of its head becomes
// known, so every input byte crosses the memory bus once:
//   1. load the chunk, reduce its columns, publish the chunk's partial result;
//   2. count the chunk in on its head's counter; the workgroup that finds itself last combines the
//      partial results (K: in chunk order, which is part of the specification; V: the maximum needs
//      no order and is taken with an atomic) and raises the head's ready flag;
//   3. every other workgroup of the head waits for the flag, then all of them quantize from registers.
// Waiting is safe because workgroups are dispatched in index order: a waiting workgroup only waits for
// workgroups with indices of the same head, all of which have been dispatched or are next in line on
// their part of the chip, and the launcher only picks this form when a head's chunks are a fraction
// of the workgroups the chip holds at once.  The wait is bounded by a wall-clock limit all the same (a device
// shared with other work may hold fewer workgroups than the launcher counted on): on expiry the workgroup
// records it in `status` and takes the head's statistic from the input itself - every chunk of the head, in the
// specified order - so every wave ends and the result is the same bits, only later.
// ---------------------------------------------------------------------------------------
constexpr int kChunkRowsPerSlot = kMeanChunk / kSlots;  // 8

// Opaque use+def: what was derived from the 16-bit values before this point (their fp32 forms) is not carried
// across it; only the 16-bit values themselves stay in registers.
__device__ __forceinline__ void forget_derived(uint4 (&raw)[kChunkRowsPerSlot][2]) {
#pragma unroll
  for (int i = 0; i < kChunkRowsPerSlot; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      asm volatile("" : "+v"(raw[i][j].x), "+v"(raw[i][j].y), "+v"(raw[i][j].z), "+v"(raw[i][j].w));
}

template <int DT>
__device__ __forceinline__ uint4 narrow8(const float* x) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DT == KSANA_SAGE_BF16) {
      // the values are exactly representable (they went through the half type): truncation is exact
      w[i] = (__float_as_uint(x[2 * i]) >> 16) | (__float_as_uint(x[2 * i + 1]) & 0xffff0000u);
    } else {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      h2 p = {(_Float16)x[2 * i], (_Float16)x[2 * i + 1]};
      w[i] = __builtin_bit_cast(uint32_t, p);
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Communication between workgroups (which may sit behind different L2 caches) goes through accesses that are
// coherent at device scope by themselves - relaxed device-scope atomics: stores write through, loads are served
// from the point of coherence - ordered by waiting for their completion (a workgroup-scope fence is that wait
// plus a compiler barrier).  Device-scope acquire / release fences are avoided on purpose: each one writes back or
// invalidates a whole L2, and a polling loop built on them starves the loads of every other workgroup.
__device__ __forceinline__ int load_shared_i32(const int* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared_f32(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void publish_f32(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// every memory access this wave has issued has completed - for the write-through stores and the atomics above:
// has reached the point of coherence - and the compiler moves no access across
__device__ __forceinline__ void complete_accesses() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }

struct HeadSync {
  int* counter;      // [B*H][kSyncStride] chunks counted in (one word per head, each in a cache line of its own)
  int* ready;        // [B*H][kSyncStride] set once the head's statistic is published
  int* status;       // [1]   set to 1 when a wait ran into its time limit
  long long limit;   // wall-clock ticks (100 MHz) a workgroup waits at most; 0 and negative: see QuantOptions
  int* host_word;    // nullptr, or a word in host memory the device can write: set to 1 when a bound > 0 expires
};

// Thread 0 waits until the head's ready flag is up (or the time limit passes), then the workgroup meets.  Returns
// true (to every thread) when the workgroup has to take the statistic from the input itself: the limit passed first,
// or the limit is negative, which means "do not even look".
__device__ __forceinline__ bool wait_for_head(const int* flag, const HeadSync& sy) {
  __shared__ int s_gave_up;
  if (threadIdx.x == 0) {
    int gave_up = 0;
    if (sy.limit < 0) {
      gave_up = 1;
    } else if (load_shared_i32(flag) < 1) {
      const long long t0 = wall_clock64();
      while (load_shared_i32(flag) < 1) {
        __builtin_amdgcn_s_sleep(16);  // ~0.5 us between polls
        if (wall_clock64() - t0 > sy.limit) {
          gave_up = 1;
          break;
        }
      }
    }
    if (gave_up) {
      __hip_atomic_store(sy.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (sy.limit > 0 && sy.host_word != nullptr)
        __hip_atomic_store(sy.host_word, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    s_gave_up = gave_up;
    complete_accesses();
  }
  __syncthreads();
  return s_gave_up != 0;
}

// Staging of one head's chunk partials for the workgroup that combines them: kFinStage chunks per
// pass (16 KiB of LDS), fetched with loads that are all in flight together; the next pass is fetched while this one
// is combined.
constexpr int kFinStage = 32;
constexpr int kFinLoads = kFinStage * kD / kThreads;  // per thread and pass: 32

__device__ __forceinline__ void fetch_partials(const float* hp, int c0, int nch, float (&v)[kFinLoads]) {
  const int n = (min(kFinStage, nch - c0)) * kD;
#pragma unroll
  for (int j = 0; j < kFinLoads; ++j) {
    const int idx = (int)threadIdx.x + kThreads * j;
    v[j] = idx < n ? load_shared_f32(hp + (int64_t)c0 * kD + idx) : 0.0f;
  }
}
__device__ __forceinline__ void stage_partials(const float (&v)[kFinLoads], float* s_part) {
#pragma unroll
  for (int j = 0; j < kFinLoads; ++j) s_part[(int)threadIdx.x + kThreads * j] = v[j];
}

// With the Wan step folded in the kernel is asked to fit three waves per SIMD (168 registers; it spills ten of them):
// a workgroup idles while it waits for its head's mean, and with two workgroups per compute unit instead of three
// the kernel measured 23 % slower.
template <int DT, int PRE>
__global__ __launch_bounds__(kThreads, PRE == 1 ? 3 : 1) void quant_k_fused_kernel(const uint16_t* __restrict__ k, int64_t sB, int64_t sL,
                                                                 int64_t sH, int H, int L_all, int d_in, int nkb, int nch,
                                                                 float* __restrict__ part, float* k_mean, int dtype,
                                                                 int smooth, int8_t* __restrict__ k_tiles,
                                                                 float* __restrict__ k_scale, const PrepParams pp,
                                                                 const HeadSync sy) {
  const int bh = blockIdx.x / nch, ch = blockIdx.x - bh * nch;
  const int b = bh / H, h = bh - b * H;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const int wave = t >> 6, lane = t & 63;
  const uint16_t* base = k + b * sB + h * sH + c16 * 16;
  const RopeLds rl = maybe_stage_rope<PRE>(pp, b, ch * kMeanChunk, kMeanChunk);
  __shared__ float s_w[4][kD];
  __shared__ float s_mean[kD];
  __shared__ float s_red[4][4];
  __shared__ int s_last;
  __shared__ float s_part[kFinStage * kD];

  // ---- 1. the chunk, and its column sums in the specified order -------------------------------
  // every load of the chunk goes out first (the rows stay in registers as 16-bit values until the end anyway): 16 KiB
  // per wave in flight; with the norm / rotation step each row is then worked on in place as it arrives
  uint4 raw[kChunkRowsPerSlot][2];
  float acc[16];
#pragma unroll
  for (int i = 0; i < kChunkRowsPerSlot; ++i) {
    const int row = ch * kMeanChunk + i * kSlots + slot;
    raw[i][0] = raw[i][1] = make_uint4(0, 0, 0, 0);
    if (row < L) {
      raw[i][0] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL);
      raw[i][1] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL + 8);
    }
  }
#pragma unroll
  for (int i = 0; i < kChunkRowsPerSlot; ++i) {
    const int row = ch * kMeanChunk + i * kSlots + slot;
    float x[16];
    widen8<DT>(raw[i][0], x);
    widen8<DT>(raw[i][1], x + 8);
    if constexpr (PRE) {
      if (row < L) prep16<DT, PRE>(x, pp, rl, b, row, h, c16);
      raw[i][0] = narrow8<DT>(x);
      raw[i][1] = narrow8<DT>(x + 8);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = i == 0 ? x[e] : acc[e] + x[e];
  }
  forget_derived(raw);
#pragma unroll
  for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = acc[e] + __shfl_xor(acc[e], m);
  }
  if (!smooth) {  // uniform: nothing is taken off, nothing to wait for
    if (t < kD) {
      s_mean[t] = 0.0f;
      if (ch == 0) k_mean[bh * kD + t] = 0.0f;
    }
    __syncthreads();
  } else {
  if (lane < 8) {
#pragma unroll
    for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = acc[e];
  }
  __syncthreads();
  if (t < kD) {
    publish_f32(part + ((int64_t)bh * nch + ch) * kD + t, (s_w[0][t] + s_w[1][t]) + (s_w[2][t] + s_w[3][t]));
    complete_accesses();  // the partial result is visible chip-wide before this chunk is counted in
  }
  __syncthreads();
  // ---- 2. count the chunk in; the last one of the head publishes the mean -----------------------
  if (t == 0) {
    const int before = __hip_atomic_fetch_add(sy.counter + bh * kSyncStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = before == nch - 1;
    complete_accesses();
  }
  __syncthreads();
  if (s_last) {  // uniform
    const float* hp = part + (int64_t)bh * nch * kD;
    float tot = 0.0f;
    float nxt[kFinLoads];
    fetch_partials(hp, 0, nch, nxt);
    for (int c0 = 0; c0 < nch; c0 += kFinStage) {
      const int n = min(kFinStage, nch - c0);
      __syncthreads();  // the previous pass has been read
      stage_partials(nxt, s_part);
      if (c0 + kFinStage < nch) fetch_partials(hp, c0 + kFinStage, nch, nxt);
      __syncthreads();
      if (t < kD) {
        // chunk order is part of the specification
        if (n == kFinStage) {
#pragma unroll 16
          for (int c = 0; c < kFinStage; ++c) tot = (c0 == 0 && c == 0) ? s_part[t] : tot + s_part[c * kD + t];
        } else {
          for (int c = 0; c < n; ++c) tot = (c0 == 0 && c == 0) ? s_part[t] : tot + s_part[c * kD + t];
        }
      }
    }
    if (t < kD) {
      const float mean = round_to_half_dtype(__fdiv_rn(tot, (float)L_all), dtype);
      s_mean[t] = mean;
      publish_f32(k_mean + bh * kD + t, mean);
      complete_accesses();
    }
    __syncthreads();
    if (t == 0) __hip_atomic_store(sy.ready + bh * kSyncStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    // ---- 3. everybody else waits for it -----------------------------------------------------------
    if (!wait_for_head(sy.ready + bh * kSyncStride, sy)) {
      if (t < kD) s_mean[t] = load_shared_f32(k_mean + bh * kD + t);
      __syncthreads();
    } else {
      // Uniform, and not taken on a device this call has to itself: the head's mean from the input, every chunk
      // summed and the chunks added up exactly as steps 1 and 2 do it.  (Rotation factors come from the table in
      // global memory: the staged ones cover this workgroup's own rows.)
      float tot = 0.0f;
      for (int c = 0; c < nch; ++c) {
        float a16[16];
#pragma unroll 1
        for (int i = 0; i < kChunkRowsPerSlot; ++i) {
          const int row = c * kMeanChunk + i * kSlots + slot;
          uint4 r[2];
          fetch_row16(base + (int64_t)row * sL, row < L, r);
          float x[16];
          widen8<DT>(r[0], x);
          widen8<DT>(r[1], x + 8);
          if constexpr (PRE) {
            if (row < L) prep16<DT, PRE>(x, pp, rl, b, row, h, c16, false);
          }
#pragma unroll
          for (int e = 0; e < 16; ++e) a16[e] = i == 0 ? x[e] : a16[e] + x[e];
        }
#pragma unroll
        for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
          for (int e = 0; e < 16; ++e) a16[e] = a16[e] + __shfl_xor(a16[e], m);
        }
        __syncthreads();  // s_w of the chunk before has been read
        if (lane < 8) {
#pragma unroll
          for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = a16[e];
        }
        __syncthreads();
        if (t < kD) {
          const float pc = (s_w[0][t] + s_w[1][t]) + (s_w[2][t] + s_w[3][t]);
          tot = c == 0 ? pc : tot + pc;
        }
      }
      if (t < kD) s_mean[t] = round_to_half_dtype(__fdiv_rn(tot, (float)L_all), dtype);
      __syncthreads();
    }
  }
  }
  // ---- 4. quantize the four 64-row tiles of the chunk from registers -----------------------------
#pragma unroll
  for (int tt = 0; tt < kMeanChunk / kBlkK; ++tt) {
    const int blk = ch * (kMeanChunk / kBlkK) + tt;
    if (blk >= nkb) break;  // uniform: the chunk's tail lies beyond the sequence
    float x[2][16];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = blk * kBlkK + i * kSlots + slot;
      widen8<DT>(raw[2 * tt + i][0], x[i]);
      widen8<DT>(raw[2 * tt + i][1], x[i] + 8);
#pragma unroll
      for (int e = 0; e < 16; ++e) x[i][e] = row < L ? x[i][e] - s_mean[c16 * 16 + e] : 0.0f;
      fwht128(x[i], c16);
#pragma unroll
      for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(x[i][e]));
    }
#pragma unroll
    for (int m = 1; m <= 32; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m));
    if (lane == 0) s_red[tt][wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(s_red[tt][0], s_red[tt][1]), fmaxf(s_red[tt][2], s_red[tt][3]));
    const bool nz = amax > 0.0f;
    const float inv = nz ? __fdiv_rn(127.0f, amax) : 0.0f;
    const float inv_lane = inv * fwht_lane_sign(c16);  // the transform left this lane's values times that sign
    if (t == 0) k_scale[(int64_t)bh * nkb + blk] = nz ? __fdiv_rn(amax, 127.0f) : 0.0f;
    int8_t* tile = k_tiles + ((int64_t)bh * nkb + blk) * (int64_t)kTileBytes;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int frag = i * 4 + (c16 >> 1);
      const int ln = (c16 & 1) * 32 + slot;
      store_out16(tile + (frag * 64 + ln) * 16, pack_int8x16(x[i], inv_lane));
    }
  }
}

// V: column abs-max of the whole sequence (the last workgroup of a head to arrive takes the maximum over the
// chunks' maxima - no order to respect - and publishes the scales), then per-channel e4m3 in the transposed tile
// order of quant_v_kernel.
template <int DT>
__global__ __launch_bounds__(kThreads) void quant_v_fused_kernel(const uint16_t* __restrict__ v, int64_t sB, int64_t sL,
                                                                 int64_t sH, int H, int L_all, int d_in, int nkb, int nch,
                                                                 float* __restrict__ part, float* v_scale, float* v_inv,
                                                                 float* __restrict__ v_mean,
                                                                 uint8_t* __restrict__ v_tiles, const HeadSync sy) {
  const int bh = blockIdx.x / nch, ch = blockIdx.x - bh * nch;
  const int b = bh / H, h = bh - b * H;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const int L = c16 * 16 < d_in ? L_all : 0;  // channels at or past d_in (head size 64) read as zero padding
  const int wave = t >> 6, lane = t & 63;
  const uint16_t* base = v + b * sB + h * sH + c16 * 16;
  __shared__ float s_w[4][kD];
  __shared__ float s_inv[kD];
  __shared__ int s_last;
  constexpr int kStride = kD + 16;  // LDS row pitch in bytes
  __shared__ __attribute__((aligned(16))) uint8_t s_v[2][kBlkK * kStride];

  uint4 raw[kChunkRowsPerSlot][2];
  float acc[16];
#pragma unroll
  for (int i = 0; i < kChunkRowsPerSlot; ++i) {
    const int row = ch * kMeanChunk + i * kSlots + slot;
    raw[i][0] = raw[i][1] = make_uint4(0, 0, 0, 0);
    if (row < L) {
      raw[i][0] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL);
      raw[i][1] = *reinterpret_cast<const uint4*>(base + (int64_t)row * sL + 8);
    }
    float x[16];
    widen8<DT>(raw[i][0], x);
    widen8<DT>(raw[i][1], x + 8);
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = i == 0 ? fabsf(x[e]) : fmaxf(acc[e], fabsf(x[e]));
  }
  forget_derived(raw);
#pragma unroll
  for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = fmaxf(acc[e], __shfl_xor(acc[e], m));
  }
  if (lane < 8) {
#pragma unroll
    for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = acc[e];
  }
  __syncthreads();
  if (t < kD) {
    publish_f32(part + ((int64_t)bh * nch + ch) * kD + t, fmaxf(fmaxf(s_w[0][t], s_w[1][t]), fmaxf(s_w[2][t], s_w[3][t])));
    complete_accesses();  // visible chip-wide before this chunk is counted in
  }
  __syncthreads();
  if (t == 0) {
    const int before = __hip_atomic_fetch_add(sy.counter + bh * kSyncStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = before == nch - 1;
    complete_accesses();
  }
  __syncthreads();
  if (s_last) {  // uniform
    // thread t: channel t % 128, chunks of parity t / 128; 32 loads in flight at a time
    const float* hp = part + (int64_t)bh * nch * kD + (t & (kD - 1));
    float m = 0.0f;
    for (int c0 = t >> 7; c0 < nch; c0 += 64) {
      float v32[32];
#pragma unroll
      for (int j = 0; j < 32; ++j) v32[j] = c0 + 2 * j < nch ? load_shared_f32(hp + (int64_t)(c0 + 2 * j) * kD) : 0.0f;
#pragma unroll
      for (int j = 0; j < 32; ++j) m = fmaxf(m, v32[j]);
    }
    __syncthreads();  // s_w was read above by every thread that needed it
    s_w[t >> 7][t & (kD - 1)] = m;
    __syncthreads();
    if (t < kD) {
      const float amax = fmaxf(s_w[0][t], s_w[1][t]);
      const bool nz = amax > 0.0f;
      const float inv = nz ? __fdiv_rn(448.0f, amax) : 0.0f;
      s_inv[t] = inv;
      publish_f32(v_inv + bh * kD + t, inv);
      v_scale[bh * kD + t] = nz ? __fdiv_rn(amax, 448.0f) : 0.0f;
      v_mean[bh * kD + t] = 0.0f;
      complete_accesses();
    }
    __syncthreads();
    if (t == 0) __hip_atomic_store(sy.ready + bh * kSyncStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    if (!wait_for_head(sy.ready + bh * kSyncStride, sy)) {
      if (t < kD) s_inv[t] = load_shared_f32(v_inv + bh * kD + t);
      __syncthreads();
    } else {
      // Uniform, and not taken on a device this call has to itself: the head's column maxima from the input (a
      // maximum needs no order), and from them the factor the last workgroup would have published.
      float m16[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) m16[e] = 0.0f;
      for (int row = slot; row < L; row += kSlots) {
        float x[16];
        widen8<DT>(*reinterpret_cast<const uint4*>(base + (int64_t)row * sL), x);
        widen8<DT>(*reinterpret_cast<const uint4*>(base + (int64_t)row * sL + 8), x + 8);
#pragma unroll
        for (int e = 0; e < 16; ++e) m16[e] = fmaxf(m16[e], fabsf(x[e]));
      }
#pragma unroll
      for (int m = 8; m <= 32; m <<= 1) {
#pragma unroll
        for (int e = 0; e < 16; ++e) m16[e] = fmaxf(m16[e], __shfl_xor(m16[e], m));
      }
      __syncthreads();  // s_w of step 1 has been read
      if (lane < 8) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s_w[wave][c16 * 16 + e] = m16[e];
      }
      __syncthreads();
      if (t < kD) {
        const float amax = fmaxf(fmaxf(s_w[0][t], s_w[1][t]), fmaxf(s_w[2][t], s_w[3][t]));
        s_inv[t] = amax > 0.0f ? __fdiv_rn(448.0f, amax) : 0.0f;
      }
      __syncthreads();
    }
  }
  float inv[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) inv[e] = s_inv[c16 * 16 + e];
#pragma unroll
  for (int tt = 0; tt < kMeanChunk / kBlkK; ++tt) {
    const int blk = ch * (kMeanChunk / kBlkK) + tt;
    if (blk >= nkb) break;  // uniform
    uint8_t* sv = s_v[tt & 1];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = i * kSlots + slot;
      float x[16];
      widen8<DT>(raw[2 * tt + i][0], x);
      widen8<DT>(raw[2 * tt + i][1], x + 8);
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = fminf(fmaxf(x[4 * j + e] * inv[4 * j + e], -448.0f), 448.0f);
        int packed = 0;
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], packed, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], packed, true);
        w[j] = (uint32_t)packed;
      }
      *reinterpret_cast<uint4*>(&sv[r * kStride + c16 * 16]) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    __syncthreads();  // two staging buffers: the one written two tiles ago was read before the last barrier
    uint8_t* tile = v_tiles + ((int64_t)bh * nkb + blk) * (int64_t)kTileBytes;
#pragma unroll
    for (int i = 0; i < kTileBytes / 16 / kThreads; ++i) {
      const int oc = i * kThreads + t;
      const int dt = oc >> 7, th = (oc >> 6) & 1, ln = oc & 63;
      const int hh = ln >> 5, d = dt * 32 + (ln & 31);
      uint32_t w[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t a = 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int row = 32 * th + 8 * g + 4 * hh + c;
          a |= (uint32_t)sv[row * kStride + d] << (8 * c);
        }
        w[g] = a;
      }
      store_out16(tile + oc * 16, make_uint4(w[0], w[1], w[2], w[3]));
    }
  }
}

// ---------------------------------------------------------------------------------------
// Block means: out[b, h, blk, d] = mean over the rows [blk * rows, min((blk + 1) * rows, L)) of x[b, :, h, d],
// optionally of x - centre[b, h, d] with each difference rounded to the tensor's half type first (the reference
// forms `k - mean(k)` as a half tensor before it pools it).  fp32 sum in a frozen order - row r of the block goes to
// slot r % 32, a slot adds its rows in increasing order, the 32 slots meet in an adjacent-pair tree - divided by the
// number of rows that exist and rounded to the half type.  One workgroup per block; rows <= 256, a multiple of 32.
// grid = (nblk, H, B).
// ---------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kThreads) void block_mean_kernel(const uint16_t* __restrict__ x, int64_t sB, int64_t sL,
                                                              int64_t sH, int H, int L, int rows,
                                                              const float* __restrict__ centre,
                                                              uint16_t* __restrict__ out) {
  const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t = threadIdx.x, slot = t >> 3, c16 = t & 7;
  const uint16_t* base = x + b * sB + h * sH + c16 * 16;
  const int64_t bh = (int64_t)b * H + h;
  float cen[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) cen[e] = centre != nullptr ? centre[bh * kD + c16 * 16 + e] : 0.0f;
  float acc[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
  for (int i = 0; i < rows / kSlots; ++i) {
    const int row = blk * rows + i * kSlots + slot;
    float v[16];
    load_row16<DT>(base + (int64_t)row * sL, row < L, v);
    if (centre != nullptr && row < L) {
#pragma unroll
      for (int e = 0; e < 16; ++e) v[e] = through_half<DT>(v[e] - cen[e]);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = i == 0 ? v[e] : acc[e] + v[e];
  }
  __shared__ float s_w[4][kD];
  store_block_mean<DT>(acc, t, (float)min(rows, L - blk * rows), out + (bh * gridDim.x + blk) * kD, s_w);
}

__global__ void clear_ints_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace

#define KSANA_DISPATCH_DT(dtype, ...)            \
  do {                                           \
    if ((dtype) == KSANA_SAGE_BF16) {            \
      constexpr int DT = KSANA_SAGE_BF16;        \
      __VA_ARGS__;                               \
    } else {                                     \
      constexpr int DT = KSANA_SAGE_FP16;        \
      __VA_ARGS__;                               \
    }                                            \
  } while (0)

// KIND as a compile-time constant for the three variants of the folded step (PrepParams::kind)
#define KSANA_DISPATCH_KIND(kind, ...)  \
  do {                                  \
    if ((kind) == 1) {                  \
      constexpr int KIND = 1;           \
      __VA_ARGS__;                      \
    } else if ((kind) == 2) {           \
      constexpr int KIND = 2;           \
      __VA_ARGS__;                      \
    } else {                            \
      constexpr int KIND = 3;           \
      __VA_ARGS__;                      \
    }                                   \
  } while (0)

// Sizes the LDS copy of the rotation factors for kernels that give `rows_per_wg` consecutive rows to
// a workgroup; returns the dynamic LDS bytes (0: the kernel reads the table directly).
static size_t plan_rope_lds(PrepParams* pp, int B, int rows_per_wg) {
  pp->lds_frames = pp->lds_heights = pp->lds_widths = 0;
  if (pp->kind == 2 || pp->freqs == nullptr) return 0;
  int nf = 0, nh = 0, nw = 0;
  for (int b = 0; b < B; ++b) {
    const int gh = pp->grid[b][1], gw = pp->grid[b][2];
    nf = max(nf, (rows_per_wg - 1) / (gh * gw) + 2);
    nh = max(nh, (rows_per_wg - 1) / gw + 2);
    nw = max(nw, gw);
  }
  const size_t bytes = ((size_t)nf * kRopeN0 + (size_t)nh * kRopeN1 + (size_t)nw * kRopeN2) * sizeof(double2);
  if (bytes > 48 * 1024) return 0;  // unusual grids (very wide, or planes of a few tokens): direct reads
  pp->lds_frames = nf, pp->lds_heights = nh, pp->lds_widths = nw;
  return bytes;
}

hipError_t launch_row_inv_rms(const InTensor& x, int B, int H, int L, float eps, float* inv_rms, hipStream_t s) {
  const dim3 grid((L + 3) / 4, B), block(kThreads);
  KSANA_DISPATCH_DT(x.dtype, (row_inv_rms_kernel<DT><<<grid, block, 0, s>>>(x.ptr, x.sB, x.sL, L, H * kD / 8,
                                                                            (float)(H * kD), eps, inv_rms)));
  return hipGetLastError();
}

hipError_t launch_col_partial(const InTensor& x, int B, int H, int L, int op, float* part, int nch, hipStream_t s,
                              const PrepParams* prep, const float* centre) {
  const dim3 grid(nch, H, B), block(kThreads);
  const PrepParams none{};
  KSANA_DISPATCH_DT(x.dtype, {
    if (op == 2)
      col_partial_kernel<DT, 2, 0><<<grid, block, 0, s>>>(x.ptr, x.sB, x.sL, x.sH, H, L, x.D, part, nch, none, centre);
    else if (op == 1)
      col_partial_kernel<DT, 1, 0><<<grid, block, 0, s>>>(x.ptr, x.sB, x.sL, x.sH, H, L, x.D, part, nch, none, nullptr);
    else if (prep == nullptr)
      col_partial_kernel<DT, 0, 0><<<grid, block, 0, s>>>(x.ptr, x.sB, x.sL, x.sH, H, L, x.D, part, nch, none, nullptr);
    else {
      PrepParams pp = *prep;
      const size_t lds = plan_rope_lds(&pp, B, kMeanChunk);
      KSANA_DISPATCH_KIND(pp.kind, (col_partial_kernel<DT, 0, KIND><<<grid, block, lds, s>>>(x.ptr, x.sB, x.sL, x.sH, H, L, x.D, part,
                                                                                        nch, pp, nullptr)));
    }
  });
  return hipGetLastError();
}

hipError_t launch_k_mean_finalize(const float* part, int BH, int nch, int L, int dtype, int smooth, float* k_mean,
                                  hipStream_t s, int* status) {
  k_mean_finalize_kernel<<<dim3(BH), dim3(kFinThreads), 0, s>>>(part, nch, L, dtype, smooth, k_mean, status);
  return hipGetLastError();
}

hipError_t launch_v_scale_finalize(const float* part, int BH, int nch, float* v_scale, float* v_inv, float* zero_mean,
                                   hipStream_t s, int* status) {
  v_scale_finalize_kernel<<<dim3(BH), dim3(kFinThreads), 0, s>>>(part, nch, v_scale, v_inv, zero_mean, status);
  return hipGetLastError();
}

hipError_t launch_quant_q(const InTensor& q, int B, int H, int L, int lq_pad, float premul, int8_t* q_i8,
                          float* q_scale, hipStream_t s, const PrepParams* prep, uint16_t* pooled) {
  const dim3 grid(lq_pad / 128, H, B), block(kThreads);
  const PrepParams none{};
  if (pooled != nullptr && (prep != nullptr || q.D != kD)) return hipErrorInvalidValue;
  KSANA_DISPATCH_DT(q.dtype, {
    if (pooled != nullptr)
      quant_q_kernel<DT, 0, true><<<grid, block, 0, s>>>(q.ptr, q.sB, q.sL, q.sH, H, L, q.D, lq_pad, premul, q_i8,
                                                              q_scale, none, pooled);
    else if (prep == nullptr)
      quant_q_kernel<DT, 0><<<grid, block, 0, s>>>(q.ptr, q.sB, q.sL, q.sH, H, L, q.D, lq_pad, premul, q_i8, q_scale,
                                                        none);
    else {
      PrepParams pp = *prep;
      const size_t lds = plan_rope_lds(&pp, B, 128);
      KSANA_DISPATCH_KIND(pp.kind, (quant_q_kernel<DT, KIND><<<grid, block, lds, s>>>(q.ptr, q.sB, q.sL, q.sH, H, L, q.D, lq_pad,
                                                                                 premul, q_i8, q_scale, pp)));
    }
  });
  return hipGetLastError();
}

hipError_t launch_quant_q_rows(const InTensor& q, int B, int H, int L, int lq_pad, float premul, float eps,
                               int8_t* q_i8, float* q_scale, hipStream_t s, const PrepParams& prep,
                               const InTensor* k_rows, int k_H, int k_L, float* k_rms) {
  RowStatOf ks{};
  if (k_rows != nullptr)
    ks = RowStatOf{k_rows->ptr, k_rows->sB, k_rows->sL, k_L, k_H * (kD / 8), (float)(k_H * kD), k_rms};
  const int rows = max(lq_pad, k_rows != nullptr ? k_L : 0);
  const dim3 grid((rows + kRowsQ - 1) / kRowsQ, B), block(kThreads);
  PrepParams pp = prep;
  float* rms_out = const_cast<float*>(pp.inv_rms);  // the caller's statistic area: written here, read by nobody else in this launch
  const size_t lds = 0;  // the rotation factors of a token are held in registers across its heads: nothing is staged
  KSANA_DISPATCH_DT(q.dtype, {
    if (pp.kind == 3)
      quant_q_rows_kernel<DT, 3><<<grid, block, lds, s>>>(q.ptr, q.sB, q.sL, q.sH, H, L, lq_pad, premul, eps, q_i8, q_scale, pp, rms_out, ks);
    else
      quant_q_rows_kernel<DT, 1><<<grid, block, lds, s>>>(q.ptr, q.sB, q.sL, q.sH, H, L, lq_pad, premul, eps, q_i8, q_scale, pp, rms_out, ks);
  });
  return hipGetLastError();
}

hipError_t launch_quant_k(const InTensor& k, int B, int H, int L, int nkb, const float* k_mean, int8_t* k_tiles,
                          float* k_scale, hipStream_t s, const PrepParams* prep, uint16_t* pooled) {
  const dim3 grid(nkb, H, B), block(kThreads);
  const PrepParams none{};
  if (pooled != nullptr && (prep != nullptr || k.D != kD)) return hipErrorInvalidValue;
  KSANA_DISPATCH_DT(k.dtype, {
    if (pooled != nullptr)
      quant_k_kernel<DT, 0, true><<<grid, block, 0, s>>>(k.ptr, k.sB, k.sL, k.sH, H, L, k.D, nkb, k_mean, k_tiles,
                                                              k_scale, none, pooled);
    else if (prep == nullptr)
      quant_k_kernel<DT, 0><<<grid, block, 0, s>>>(k.ptr, k.sB, k.sL, k.sH, H, L, k.D, nkb, k_mean, k_tiles, k_scale,
                                                        none);
    else {
      PrepParams pp = *prep;
      const size_t lds = plan_rope_lds(&pp, B, kBlkK);
      KSANA_DISPATCH_KIND(pp.kind, (quant_k_kernel<DT, KIND><<<grid, block, lds, s>>>(k.ptr, k.sB, k.sL, k.sH, H, L, k.D, nkb,
                                                                                 k_mean, k_tiles, k_scale, pp)));
    }
  });
  return hipGetLastError();
}

namespace {
constexpr int kMaxDevices = 64;

// Resident-workgroup counts the launchers have asked the runtime for, kept per (device, kernel address): every
// instantiation of a kernel template has its own register and LDS footprint, and all instantiations of one
// template share one function-pointer TYPE, so the address is the key.
class OccupancyCache {
 public:
  int find(int dev, const void* kernel) {
    std::lock_guard<std::mutex> lock(m_);
    for (int i = 0; i < n_; ++i)
      if (e_[i].dev == dev && e_[i].kernel == kernel) return e_[i].workgroups;
    return -1;
  }
  void put(int dev, const void* kernel, int workgroups) {
    std::lock_guard<std::mutex> lock(m_);
    for (int i = 0; i < n_; ++i)
      if (e_[i].dev == dev && e_[i].kernel == kernel) {
        e_[i].workgroups = workgroups;
        return;
      }
    if (n_ < kEntries) e_[n_++] = Entry{dev, kernel, workgroups};  // full: the answer is simply asked for again
  }

 private:
  struct Entry {
    int dev;
    const void* kernel;
    int workgroups;
  };
  static constexpr int kEntries = 256;
  std::mutex m_;
  Entry e_[kEntries];
  int n_ = 0;
};
OccupancyCache g_occupancy;

// Workgroups of `kernel` (256 threads, `lds` bytes of dynamic LDS) the current device holds at once.
// (0 when the runtime cannot tell: the caller then takes the two-pass kernels.)  The answer for a launch
// without dynamic LDS is kept per device and kernel.
template <typename K>
int resident_workgroups(K kernel, size_t lds) {
  int per_cu = 0, dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  const void* key = reinterpret_cast<const void*>(kernel);
  if (lds == 0) {
    const int c = g_occupancy.find(dev, key);
    if (c > 0) return c;
  }
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, lds) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (lds == 0 && per_cu * cus > 0) g_occupancy.put(dev, key, per_cu * cus);
  return per_cu * cus;
}

// ---- process-wide settings (see QuantOptions) ----------------------------------------------------------------
std::mutex g_opt_mutex;
bool g_opt_ready = false;
QuantOptions g_opt{false, true, kDefaultWaitTicks};

void parse_stages(const char* stages, QuantOptions* o) {
  o->one_read_k = strchr(stages, 'k') != nullptr;
  o->one_read_v = strchr(stages, 'v') != nullptr;
}
void options_from_environment_locked() {
  if (g_opt_ready) return;
  g_opt_ready = true;
  const char* e = getenv("KSANA_SAGE_ONE_READ");
  parse_stages(e ? e : "v", &g_opt);
  const char* w = getenv("KSANA_SAGE_WAIT_TICKS");
  if (w != nullptr && *w != 0) {
    char* end = nullptr;
    const long long v = strtoll(w, &end, 10);
    if (end != w) g_opt.wait_ticks = v;
  }
}

// One word of host memory per device that the device can write (pinned, mapped): a kernel whose wait expires sets it,
// the launchers read it as plain host memory - no copy, no synchronisation.  Allocated when a one-read kernel is first
// launched on the device by a caller that may allocate, and kept until the process ends.
struct HostWord {
  int* host = nullptr;
  int* dev = nullptr;
};
HostWord g_host_word[kMaxDevices];
std::mutex g_host_word_mutex;

HostWord host_word(bool may_allocate) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return HostWord{};
  std::lock_guard<std::mutex> lock(g_host_word_mutex);
  HostWord& w = g_host_word[dev];
  if (w.host == nullptr && may_allocate) {
    void* h = nullptr;
    void* d = nullptr;
    if (hipHostMalloc(&h, 64, hipHostMallocMapped) == hipSuccess) {
      *static_cast<volatile int*>(h) = 0;
      if (hipHostGetDevicePointer(&d, h, 0) == hipSuccess) {
        w.host = static_cast<int*>(h);
        w.dev = static_cast<int*>(d);
      } else {
        (void)hipGetLastError();
        (void)hipHostFree(h);
      }
    } else {
      (void)hipGetLastError();  // no word, no reports: the kernels still end and still give the same bits
    }
  }
  return w;
}

}  // namespace

QuantOptions quant_options() {
  std::lock_guard<std::mutex> lock(g_opt_mutex);
  options_from_environment_locked();
  return g_opt;
}

void configure_quant(const char* stages, long long wait_ticks, bool keep_ticks) {
  {
    std::lock_guard<std::mutex> lock(g_opt_mutex);
    options_from_environment_locked();
    if (stages != nullptr) parse_stages(stages, &g_opt);
    if (!keep_ticks) g_opt.wait_ticks = wait_ticks;
  }
  std::lock_guard<std::mutex> lock(g_host_word_mutex);
  for (HostWord& w : g_host_word)
    if (w.host != nullptr) *static_cast<volatile int*>(w.host) = 0;
}

bool one_read_demoted(bool may_allocate) {
  const HostWord w = host_word(may_allocate);
  return w.host != nullptr && *static_cast<volatile int*>(w.host) != 0;
}

int selftest_occupancy_cache() {
  OccupancyCache c;
  const void* a = reinterpret_cast<const void*>(&quant_k_fused_kernel<KSANA_SAGE_BF16, 1>);
  const void* b = reinterpret_cast<const void*>(&quant_k_fused_kernel<KSANA_SAGE_BF16, 2>);
  if (a == b) return 1;
  if (c.find(0, a) != -1) return 2;
  c.put(0, a, 768);
  if (c.find(0, a) != 768 || c.find(0, b) != -1 || c.find(1, a) != -1) return 3;
  c.put(0, b, 1024);
  c.put(1, a, 512);
  if (c.find(0, a) != 768 || c.find(0, b) != 1024 || c.find(1, a) != 512) return 4;
  c.put(0, a, 256);
  return c.find(0, a) == 256 && c.find(0, b) == 1024 ? 0 : 5;
}

hipError_t launch_block_means(const InTensor& x, int B, int H, int L, int rows, const float* centre, uint16_t* out,
                              hipStream_t s) {
  const dim3 grid((L + rows - 1) / rows, H, B), block(kThreads);
  KSANA_DISPATCH_DT(x.dtype, (block_mean_kernel<DT><<<grid, block, 0, s>>>(x.ptr, x.sB, x.sL, x.sH, H, L, rows, centre, out)));
  return hipGetLastError();
}

hipError_t launch_clear_ints(int* p, int n, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  clear_ints_kernel<<<dim3((n + 255) / 256), dim3(256), 0, s>>>(p, n);
  return hipGetLastError();
}

// The one-read forms are used when a head's chunks are at most half of what the chip holds at once (see the
// comment above the kernels); *used tells the caller whether anything was launched.
hipError_t launch_quant_k_fused(const InTensor& k, int B, int H, int L, int nkb, int nch, int smooth, float* part,
                                float* k_mean, int8_t* k_tiles, float* k_scale, const QuantSync& sync, hipStream_t s,
                                const PrepParams* prep, bool* used, bool may_allocate) {
  *used = false;
  if ((int64_t)B * H * nch > INT32_MAX) return hipSuccess;
  if (one_read_demoted(may_allocate)) return hipSuccess;
  const dim3 grid(B * H * nch), block(kThreads);
  const HeadSync sy{sync.k_counter, sync.k_ready, sync.k_status, quant_options().wait_ticks, host_word(false).dev};
  const PrepParams none{};
  hipError_t e = hipSuccess;
  KSANA_DISPATCH_DT(k.dtype, {
    if (prep == nullptr) {
      const int resident = resident_workgroups(quant_k_fused_kernel<DT, 0>, 0);
      if (2 * nch <= resident) {
        quant_k_fused_kernel<DT, 0><<<grid, block, 0, s>>>(k.ptr, k.sB, k.sL, k.sH, H, L, k.D, nkb, nch, part, k_mean,
                                                                k.dtype, smooth, k_tiles, k_scale, none, sy);
        *used = true;
      }
    } else {
      PrepParams pp = *prep;
      const size_t lds = plan_rope_lds(&pp, B, kMeanChunk);
      KSANA_DISPATCH_KIND(pp.kind, {
        // lds != 0 only for kind 1; the cached answer (lds == 0) is kept per kernel address
        if (2 * nch <= resident_workgroups(quant_k_fused_kernel<DT, KIND>, lds)) {
          quant_k_fused_kernel<DT, KIND><<<grid, block, lds, s>>>(k.ptr, k.sB, k.sL, k.sH, H, L, k.D, nkb, nch, part, k_mean,
                                                                   k.dtype, smooth, k_tiles, k_scale, pp, sy);
          *used = true;
        }
      });
    }
  });
  if (*used) e = hipGetLastError();
  return e;
}

hipError_t launch_quant_v_fused(const InTensor& v, int B, int H, int L, int nkb, int nch, float* part, float* v_scale,
                                float* v_inv, float* v_mean, uint8_t* v_tiles, const QuantSync& sync, hipStream_t s,
                                bool* used) {
  *used = false;
  if ((int64_t)B * H * nch > INT32_MAX) return hipSuccess;
  if (one_read_demoted()) return hipSuccess;
  const dim3 grid(B * H * nch), block(kThreads);
  const HeadSync sy{sync.v_counter, sync.v_ready, sync.v_status, quant_options().wait_ticks, host_word(false).dev};
  hipError_t e = hipSuccess;
  KSANA_DISPATCH_DT(v.dtype, {
    const int resident = resident_workgroups(quant_v_fused_kernel<DT>, 0);
    if (2 * nch <= resident) {
      quant_v_fused_kernel<DT><<<grid, block, 0, s>>>(v.ptr, v.sB, v.sL, v.sH, H, L, v.D, nkb, nch, part, v_scale, v_inv,
                                                       v_mean, v_tiles, sy);
      *used = true;
    }
  });
  if (*used) e = hipGetLastError();
  return e;
}

hipError_t launch_quant_v(const InTensor& v, int B, int H, int L, int nkb, const float* v_inv, const float* v_mean,
                          uint8_t* v_tiles, hipStream_t s) {
  const dim3 grid(nkb, H, B), block(kThreads);
  KSANA_DISPATCH_DT(v.dtype, {
    if (v_mean != nullptr)
      quant_v_kernel<DT, true><<<grid, block, 0, s>>>(v.ptr, v.sB, v.sL, v.sH, H, L, v.D, nkb, v_inv, v_mean, v_tiles);
    else
      quant_v_kernel<DT, false><<<grid, block, 0, s>>>(v.ptr, v.sB, v.sL, v.sH, H, L, v.D, nkb, v_inv, nullptr, v_tiles);
  });
  return hipGetLastError();
}

}  // namespace ksana_sage
