// Host-side check of the C ABI's argument validation, meant to be built with AddressSanitizer on the host pass
// (ksanadit_amd/build_host_check.py) and run on a machine without a GPU: every call below must be refused by the
// library before it touches a device, so whatever the host code reads on the way - shapes, strides, the descriptor
// of the step before attention, the host-resident grid sizes - is read under the sanitizer.  Exit code 0 = every
// call returned what it should; the sanitizer aborts the process on a bad access.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/ksana_sage_hip.h"

static int g_failed = 0;
#define EXPECT(call, want)                                                                        \
  do {                                                                                            \
    const int rc_ = (call);                                                                       \
    if (rc_ != (want)) {                                                                          \
      ++g_failed;                                                                                 \
      std::printf("line %d: %s -> %d (want %d): %s\n", __LINE__, #call, rc_, (want), ksana_sage_last_error()); \
    }                                                                                             \
  } while (0)

int main() {
  void* const fake = reinterpret_cast<void*>(0x1000);  // aligned and never dereferenced
  ksana_sage_shape s{1, 2, 2, 64, 64, 128};
  const int64_t st[4] = {64 * 2 * 128, 2 * 128, 128, 1};
  ksana_sage_ws_layout lay;
  EXPECT(ksana_sage_workspace_layout(nullptr, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_workspace_layout(&s, &lay), 0);
  if (lay.total_bytes == 0 || lay.nkb != 1 || lay.lq_pad != 128) ++g_failed, std::printf("layout of the small shape is off\n");
  ksana_sage_shape big{1, 40, 40, 32760, 32760, 128};
  EXPECT(ksana_sage_workspace_layout(&big, &lay), 0);
  ksana_sage_shape odd_d{1, 2, 2, 64, 64, 96};
  EXPECT(ksana_sage_workspace_layout(&odd_d, &lay), KSANA_SAGE_ENOTSUP);
  ksana_sage_shape gqa{1, 3, 2, 64, 64, 128};
  EXPECT(ksana_sage_workspace_layout(&gqa, &lay), KSANA_SAGE_EINVAL);

  EXPECT(ksana_sage_quant_q(nullptr, KSANA_SAGE_BF16, st, &s, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_k(fake, 7, st, &s, 1, fake, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_v(reinterpret_cast<void*>(0x1008), KSANA_SAGE_BF16, st, &s, fake, nullptr), KSANA_SAGE_EINVAL);
  const int64_t bad_d[4] = {64 * 2 * 128, 2 * 128, 128, 2};
  EXPECT(ksana_sage_quant_q(fake, KSANA_SAGE_BF16, bad_d, &s, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_q(fake, KSANA_SAGE_BF16, nullptr, &s, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_q(fake, KSANA_SAGE_BF16, st, &s, 0.1f, nullptr, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_k_static(fake, KSANA_SAGE_BF16, st, &s, 1, nullptr, nullptr), KSANA_SAGE_EINVAL);
  ksana_sage_shape many{1, 65, 65, 64, 65536, 128};
  EXPECT(ksana_sage_quant_k_static(fake, KSANA_SAGE_BF16, st, &many, 1, fake, nullptr), KSANA_SAGE_ENOTSUP);

  // the descriptor of the step before attention, with its host-resident grid sizes
  ksana_sage_prep prep;
  std::memset(&prep, 0, sizeof(prep));
  prep.norm_eps = 1e-6f;
  prep.q_norm_weight = reinterpret_cast<const float*>(0x1004);  // misaligned
  EXPECT(ksana_sage_quant_q_prep(fake, KSANA_SAGE_BF16, st, &s, &prep, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);
  std::memset(&prep, 0, sizeof(prep));
  prep.rope_freqs = reinterpret_cast<const double*>(0x1000);
  prep.rope_rows = 1024;  // a rotation without grid sizes
  EXPECT(ksana_sage_quant_k_prep(fake, KSANA_SAGE_BF16, st, &s, &prep, 1, fake, nullptr), KSANA_SAGE_EINVAL);
  std::vector<int32_t> grid = {2, 8, 8};  // exactly B * 3 values: reading past them is what the sanitizer would catch
  prep.grid_sizes = grid.data();
  EXPECT(ksana_sage_quant_k_prep(fake, KSANA_SAGE_BF16, st, &s, &prep, 1, fake, nullptr), KSANA_SAGE_EINVAL);  // 128 positions, 64 rows
  grid = {1, 8, 2000};  // an extent beyond the table
  prep.grid_sizes = grid.data();
  EXPECT(ksana_sage_quant_qk_prep(fake, fake, KSANA_SAGE_BF16, st, st, &s, &prep, 0.1f, 1, fake, nullptr), KSANA_SAGE_EINVAL);
  ksana_sage_shape two{2, 2, 2, 64, 64, 128};
  std::vector<int32_t> grid2 = {1, 8, 8, 1, 8, 9};  // the second batch entry is the bad one
  prep.grid_sizes = grid2.data();
  EXPECT(ksana_sage_forward_prep(fake, fake, fake, fake, KSANA_SAGE_BF16, st, st, st, st, &two, &prep, nullptr, 0.1f, 1, 0, 0, fake, nullptr),
         KSANA_SAGE_EINVAL);
  std::memset(&prep, 0, sizeof(prep));
  prep.kind = KSANA_SAGE_PREP_QWEN;
  prep.txt_len = 65;  // beyond the sequence
  prep.q_norm_weight = reinterpret_cast<const float*>(0x1000);
  EXPECT(ksana_sage_quant_q_prep(fake, KSANA_SAGE_BF16, st, &s, &prep, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);
  prep.kind = 9;
  EXPECT(ksana_sage_quant_q_prep(fake, KSANA_SAGE_BF16, st, &s, &prep, 0.1f, fake, nullptr), KSANA_SAGE_EINVAL);

  // attention entry points
  ksana_sage_shape long_k{1, 2, 2, 64, 131073, 128};
  EXPECT(ksana_sage_attn_fwd(fake, fake, KSANA_SAGE_BF16, st, &long_k, nullptr, 1, 0, nullptr), KSANA_SAGE_ENOTSUP);
  EXPECT(ksana_sage_attn_fwd(fake, fake, KSANA_SAGE_BF16, st, &s, nullptr, 0, 0x20, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_attn_fwd(fake, fake, KSANA_SAGE_BF16, st, &s, nullptr, 0, KSANA_SAGE_FLAG_TILE_SKIP | KSANA_SAGE_FLAG_PWL_EXP2, nullptr),
         KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_attn_fwd(fake, fake, KSANA_SAGE_BF16, st, &s, reinterpret_cast<const int32_t*>(0x1002), 0, 0, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_attn_fwd_masked(fake, fake, KSANA_SAGE_BF16, st, &s, reinterpret_cast<const int8_t*>(fake), nullptr, nullptr, 0, 0, nullptr),
         KSANA_SAGE_EINVAL);
  const int64_t neg[2] = {-1, 0};
  EXPECT(ksana_sage_attn_fwd_masked(fake, fake, KSANA_SAGE_BF16, st, &s, reinterpret_cast<const int8_t*>(fake), neg, nullptr, 0, 0, nullptr),
         KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_forward(fake, fake, nullptr, fake, KSANA_SAGE_BF16, st, st, st, st, &s, nullptr, 0.1f, 1, 0, 0, fake, nullptr), KSANA_SAGE_EINVAL);
  int first = -1, runs = -1;
  EXPECT(ksana_sage_attn_key_split(&s, &first, nullptr), KSANA_SAGE_EINVAL);

  // the sparse-linear backend's entry points
  uint64_t bytes = 0;
  EXPECT(ksana_sage_sla_workspace_bytes(1, 40, 32760, &bytes), 0);
  EXPECT(ksana_sage_sla_workspace_bytes(0, 40, 32760, &bytes), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_sla_linear(fake, fake, nullptr, KSANA_SAGE_BF16, st, st, st, 1, 2, 64, nullptr, nullptr, nullptr, nullptr, fake, st, fake, nullptr),
         KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_sla_block_map(fake, fake, KSANA_SAGE_BF16, 1, 2, 8, 2000, 3, reinterpret_cast<int8_t*>(fake), nullptr), KSANA_SAGE_ENOTSUP);
  EXPECT(ksana_sage_block_means(fake, KSANA_SAGE_BF16, st, 1, 2, 64, 48, nullptr, fake, nullptr), KSANA_SAGE_ENOTSUP);
  ksana_sage_shape d64{1, 2, 2, 64, 64, 64};
  EXPECT(ksana_sage_quant_qk_pooled(fake, fake, KSANA_SAGE_BF16, st, st, &d64, 0.1f, fake, fake, fake, nullptr), KSANA_SAGE_ENOTSUP);
  EXPECT(ksana_sage_quant_qk_pooled(fake, fake, KSANA_SAGE_BF16, st, st, &s, 0.1f, fake, nullptr, fake, nullptr), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_quant_qk_pooled(fake, nullptr, KSANA_SAGE_BF16, st, st, &s, 0.1f, fake, fake, fake, nullptr), KSANA_SAGE_EINVAL);

  // settings and self-checks
  EXPECT(ksana_sage_configure("kx", KSANA_SAGE_KEEP), KSANA_SAGE_EINVAL);
  EXPECT(ksana_sage_configure("kv", 123), 0);
  int k1 = 0, v1 = 0, dem = -1;
  int64_t ticks = 0;
  EXPECT(ksana_sage_one_read_state(&k1, &v1, &ticks, &dem), 0);
  if (!k1 || !v1 || ticks != 123 || dem != 0) ++g_failed, std::printf("settings did not stick\n");
  EXPECT(ksana_sage_selftest(), 0);
  if (ksana_sage_abi_version() != KSANA_SAGE_ABI_VERSION) ++g_failed, std::printf("ABI number differs from the header's\n");
  std::printf("host argument checks: %d failed\n", g_failed);
  return g_failed == 0 ? 0 : 1;
}
