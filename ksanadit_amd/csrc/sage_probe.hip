// Matrix-pipe probe: the attention kernel's MFMA mix with nothing else around it.
//
// One wave issues, per step, the same thirteen matrix instructions the attention kernel issues per key tile - eight
// v_mfma_i32_32x32x32_i8 and five v_mfma_f32_32x32x64_f8f6f4 (four for O, one for the row sums) - on operands that
// stay in registers: no memory, no LDS, no vector-ALU work.  What it sustains is the ceiling the attention kernel's
// percentage of "peak" should be read against: the published 5.0e15 /s assumes a clock the chip does not hold under
// matrix load.
#include <hip/hip_runtime.h>

#include "../../include/ksana_sage_hip.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kProbeThreads = 512;  // 8 waves: two per SIMD, like the attention kernel

__global__ __launch_bounds__(kProbeThreads) void mfma_probe_kernel(float* out, int steps) {
  v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)threadIdx.x};
  v8i a8 = {0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838, 0x38383838};
  v8i b8 = {(int)(threadIdx.x & 7) * 0x08080808, 0, 0x38383838, 0, 0x30303030, 0, 0x28282828, 0};
  asm volatile("" : "+v"(a), "+v"(b), "+v"(a8), "+v"(b8));
  v16i s0, s1;
  v16f o0, o1, o2, o3, l;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    s0[r] = r, s1[r] = -r;
    o0[r] = o1[r] = o2[r] = o3[r] = l[r] = 0.0f;
  }
  for (int it = 0; it < steps; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, s1, 0, 0, 0);
    }
    o0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, o0, 0, 0, 0, 0, 0, 0);
    o1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, o1, 0, 0, 0, 0, 0, 0);
    o2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, o2, 0, 0, 0, 0, 0, 0);
    o3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, o3, 0, 0, 0, 0, 0, 0);
    l = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, l, 0, 0, 0, 0, 0, 0);
  }
  float acc = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc += (float)(s0[r] + s1[r]) + o0[r] + o1[r] + o2[r] + o3[r] + l[r];
  out[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = acc;
}

}  // namespace

extern "C" int ksana_sage_mfma_probe(void* scratch, uint64_t scratch_bytes, int workgroups, int steps, void* stream,
                                     double* ops_per_launch) {
  if (!scratch || workgroups < 1 || steps < 1 || !ops_per_launch) return KSANA_SAGE_EINVAL;
  if (scratch_bytes < (uint64_t)workgroups * kProbeThreads * sizeof(float)) return KSANA_SAGE_EINVAL;
  mfma_probe_kernel<<<dim3(workgroups), dim3(kProbeThreads), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<float*>(scratch), steps);
  // per wave and step: 8 x (2*32*32*32) integer + 5 x (2*32*32*64) fp8 multiply-adds counted as 2
  *ops_per_launch = (double)workgroups * (kProbeThreads / 64) * steps * (8.0 * 65536.0 + 5.0 * 131072.0);
  return hipGetLastError() == hipSuccess ? KSANA_SAGE_OK : KSANA_SAGE_EHIP;
}
