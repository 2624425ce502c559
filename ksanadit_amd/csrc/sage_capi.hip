// C ABI of libksana_sage_hip.so: argument validation, workspace layout, kernel launches.
// Declarations and the reference call sites each entry point replaces: include/ksana_sage_hip.h.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/ksana_sage_hip.h"
#include "sage_kernels.h"

// Scratch of ksana_sage_quant_k_static: the chunk sums of K's channel means, [B * Hkv * ceil(Lk / 256)][128]
// fp32, followed by the counters and flags through which the workgroups of a head meet (cleared by a small kernel
// at the start of every call).  Device memory that belongs to the loaded code object: every GPU the library runs
// on holds its own copy (8.1 MiB) at its own address from the first launch on it until the process ends.  In host code the name below is
// only a handle for hipGetSymbolAddress - the device address it yields is what kernels are given.
constexpr int kStaticChunkRows = 16384;  // B * Hkv * ceil(Lk / 256) that fit
constexpr size_t kStaticPartFloats = (size_t)kStaticChunkRows * ksana_sage::kD;
constexpr int kStaticHeads = 4096;         // B * Hkv that fit
constexpr size_t kStaticSyncInts = ksana_sage::sync_words(kStaticHeads);  // per head a counter and a ready flag; a status word
static __device__ __align__(256) float scratch[kStaticPartFloats + kStaticSyncInts];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

uint64_t align256(uint64_t x) { return (x + 255u) & ~uint64_t(255); }

// Named ranges around the stages of a call (quantize, attention, ...) for a timeline viewer: roctx push / pop, looked
// up at run time in the profiler's marker library the first time they are wanted - only when the environment variable
// KSANA_SAGE_ROCTX is set to something other than 0 (read once), so a process that is not being profiled pays one
// branch per stage and links against nothing.
class StageRange {
 public:
  explicit StageRange(const char* name) : on_(enabled()) {
    if (on_) push_(name);
  }
  ~StageRange() {
    if (on_) pop_();
  }
  StageRange(const StageRange&) = delete;
  StageRange& operator=(const StageRange&) = delete;

 private:
  using Push = int (*)(const char*);
  using Pop = int (*)();
  static Push push_;
  static Pop pop_;
  static bool enabled() {
    static const bool on = [] {
      const char* e = getenv("KSANA_SAGE_ROCTX");
      if (e == nullptr || *e == 0 || strcmp(e, "0") == 0) return false;
      for (const char* lib : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
        if (void* h = dlopen(lib, RTLD_NOW | RTLD_GLOBAL)) {
          push_ = reinterpret_cast<Push>(dlsym(h, "roctxRangePushA"));
          pop_ = reinterpret_cast<Pop>(dlsym(h, "roctxRangePop"));
          if (push_ != nullptr && pop_ != nullptr) return true;
        }
      }
      return false;
    }();
    return on;
  }
  bool on_;
};
StageRange::Push StageRange::push_ = nullptr;
StageRange::Pop StageRange::pop_ = nullptr;

int check_shape(const ksana_sage_shape* s) {
  if (!s) return fail(KSANA_SAGE_EINVAL, "shape is null");
  if (s->B < 1 || s->Hq < 1 || s->Hkv < 1 || s->Lq < 1 || s->Lk < 1)
    return fail(KSANA_SAGE_EINVAL, "shape has a non-positive extent (B=%d Hq=%d Hkv=%d Lq=%d Lk=%d)", s->B, s->Hq,
                s->Hkv, s->Lq, s->Lk);
  if (s->Hq % s->Hkv != 0) return fail(KSANA_SAGE_EINVAL, "Hq=%d is not a multiple of Hkv=%d", s->Hq, s->Hkv);
  if (s->D != ksana_sage::kD && s->D != 64)
    return fail(KSANA_SAGE_ENOTSUP, "head size %d not supported (128, or 64 run zero-padded to 128)", s->D);
  if (s->Lk > 262144) return fail(KSANA_SAGE_ENOTSUP, "Lk=%d exceeds 262144 (K scales of one head are kept in LDS)", s->Lk);
  if ((int64_t)s->B * s->Hq > 65535 * 8 || s->Hq > 65535 || s->B > 65535)
    return fail(KSANA_SAGE_EINVAL, "B*H too large for the launch grid");
  // row numbers go through fp32 in the rotary step (exact below 2^24), and the kernels index workgroups with int32
  if (s->Lq > (1 << 24)) return fail(KSANA_SAGE_ENOTSUP, "Lq=%d exceeds %d", s->Lq, 1 << 24);
  const int64_t n_wg = (int64_t)s->B * s->Hq * ((s->Lq + ksana_sage::kAttnQPerWg - 1) / ksana_sage::kAttnQPerWg);
  if (n_wg > (INT64_C(1) << 31) / 8 - 8)
    return fail(KSANA_SAGE_ENOTSUP, "B*Hq*ceil(Lq/256) = %lld workgroups exceed the launch grid (%lld)",
                (long long)n_wg, (long long)((INT64_C(1) << 31) / 8 - 8));
  return 0;
}

int check_tensor(const char* name, const void* ptr, int dtype, const int64_t st[4], int B, int L, int H) {
  if (!ptr) return fail(KSANA_SAGE_EINVAL, "%s is null", name);
  if (dtype != KSANA_SAGE_BF16 && dtype != KSANA_SAGE_FP16) return fail(KSANA_SAGE_EINVAL, "%s: dtype %d unknown", name, dtype);
  if (!st) return fail(KSANA_SAGE_EINVAL, "%s: strides are null", name);
  if (st[3] != 1) return fail(KSANA_SAGE_EINVAL, "%s: D stride is %lld, must be 1", name, (long long)st[3]);
  if (reinterpret_cast<uintptr_t>(ptr) & 15u) return fail(KSANA_SAGE_EINVAL, "%s: pointer not 16-byte aligned", name);
  const int ext[3] = {B, L, H};
  for (int i = 0; i < 3; ++i) {
    if (st[i] < 0) return fail(KSANA_SAGE_EINVAL, "%s: negative stride", name);
    if (ext[i] > 1 && (st[i] % 8 != 0 || st[i] == 0))
      return fail(KSANA_SAGE_EINVAL, "%s: stride[%d]=%lld must be a non-zero multiple of 8", name, i, (long long)st[i]);
  }
  return 0;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(KSANA_SAGE_EHIP, "%s: %s", what, hipGetErrorString(e));
}

ksana_sage::InTensor in_tensor(const void* p, int dtype, const int64_t st[4], int D = ksana_sage::kD) {
  return ksana_sage::InTensor{static_cast<const uint16_t*>(p), st[0], st[1], st[2], dtype, D};
}

template <typename T>
T* ws_at(void* ws, uint64_t off) {
  return reinterpret_cast<T*>(static_cast<uint8_t*>(ws) + off);
}
template <typename T>
const T* ws_at(const void* ws, uint64_t off) {
  return reinterpret_cast<const T*>(static_cast<const uint8_t*>(ws) + off);
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(float** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(KSANA_SAGE_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(KSANA_SAGE_ENOTSUP, "device index %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(KSANA_SAGE_EHIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// The counter / ready / status words of the K and of the V quantizer inside their areas of sync_words(bhk) ints
ksana_sage::QuantSync sync_at(int* k_words, int* v_words, int bhk) {
  const int n = bhk * ksana_sage::kSyncStride;
  ksana_sage::QuantSync q{};
  if (k_words) q.k_counter = k_words, q.k_ready = k_words + n, q.k_status = k_words + 2 * n;
  if (v_words) q.v_counter = v_words, q.v_ready = v_words + n, q.v_status = v_words + 2 * n;
  return q;
}

// Which of K and V are quantized by the one-read kernels when the shape allows (otherwise by the two-pass ones): a
// process-wide setting (ksana_sage_configure; first value from the environment, read once)
bool one_read(char which) {
  const ksana_sage::QuantOptions o = ksana_sage::quant_options();
  return which == 'k' ? o.one_read_k : o.one_read_v;
}

int check_ws(const void* ws) {
  if (!ws) return fail(KSANA_SAGE_EINVAL, "workspace is null");
  if (reinterpret_cast<uintptr_t>(ws) & 255u) return fail(KSANA_SAGE_EINVAL, "workspace not 256-byte aligned");
  return 0;
}

int check_mask(const ksana_sage_shape* s, const int8_t* block_mask, const int64_t mask_st[2]) {
  if (!block_mask) return 0;
  if (!mask_st) return fail(KSANA_SAGE_EINVAL, "block_mask given without mask_strides");
  if (mask_st[0] < 0 || mask_st[1] < 0) return fail(KSANA_SAGE_EINVAL, "negative mask stride");
  if (s->Lk > ksana_sage::kSparseMaxKeyTiles * ksana_sage::kBlkK)
    return fail(KSANA_SAGE_ENOTSUP, "Lk=%d exceeds %d with a block mask (the tile list is kept in LDS)", s->Lk,
                ksana_sage::kSparseMaxKeyTiles * ksana_sage::kBlkK);
  return 0;
}

// Causal masking: query row i sees keys [0, i] (the triangle is anchored at the top left corner, as torch's SDPA
// anchors it when Lq != Lk); the kernel keeps its list of key tiles in LDS, which bounds Lk.
int check_causal(const ksana_sage_shape* s, int causal) {
  if (!causal) return 0;
  if (s->Lk > ksana_sage::kSparseMaxKeyTiles * ksana_sage::kBlkK)
    return fail(KSANA_SAGE_ENOTSUP, "Lk=%d exceeds %d with causal masking (the tile list is kept in LDS)", s->Lk,
                ksana_sage::kSparseMaxKeyTiles * ksana_sage::kBlkK);
  return 0;
}

int forward_impl(const void* q, const void* k, const void* v, void* o, int dtype, const int64_t q_st[4],
                 const int64_t k_st[4], const int64_t v_st[4], const int64_t o_st[4], const ksana_sage_shape* s,
                 const ksana_sage_prep* prep, const int8_t* block_mask, const int64_t mask_st[2],
                 const int32_t* k_lens, float sm_scale, int smooth_k, int causal, int flags, void* ws, void* stream);

// Validates `prep` for one tensor (`weight` is that tensor's norm weight) and fills the kernel-side
// parameters.  *out stays nullptr when there is nothing to apply.
int make_prep(const ksana_sage_prep* prep, const float* weight, const char* name, const int64_t st[4], int B, int L,
              int D, float* inv_rms, ksana_sage::PrepParams* pp, const ksana_sage::PrepParams** out) {
  *out = nullptr;
  if (!prep) return 0;
  if (D != ksana_sage::kD) return fail(KSANA_SAGE_ENOTSUP, "the folded norm / rotation step needs head size 128, got %d", D);
  if (prep->kind != KSANA_SAGE_PREP_WAN && prep->kind != KSANA_SAGE_PREP_WAN_COMFY && prep->kind != KSANA_SAGE_PREP_QWEN)
    return fail(KSANA_SAGE_EINVAL, "prep kind %d unknown", prep->kind);
  if (prep->kind == KSANA_SAGE_PREP_QWEN) {
    const bool is_q = name[0] == 'q';
    const float* w_txt = is_q ? prep->q_norm_weight_txt : prep->k_norm_weight_txt;
    if (!weight && !w_txt && !prep->rope_freqs_txt && !prep->rope_freqs_img) return 0;
    memset(pp, 0, sizeof(*pp));
    pp->L = L;
    pp->kind = 2;
    if (prep->txt_len < 0 || prep->txt_len > L)
      return fail(KSANA_SAGE_EINVAL, "txt_len=%d outside [0, %s length %d]", prep->txt_len, name, L);
    if (!(prep->norm_eps >= 0.0f)) return fail(KSANA_SAGE_EINVAL, "norm_eps must be >= 0");
    const void* ptrs[4] = {weight, w_txt, prep->rope_freqs_txt, prep->rope_freqs_img};
    for (const void* ptr : ptrs)
      if (reinterpret_cast<uintptr_t>(ptr) & 15u) return fail(KSANA_SAGE_EINVAL, "%s: a prep pointer is not 16-byte aligned", name);
    pp->txt_len = prep->txt_len;
    pp->eps = prep->norm_eps;
    pp->weight_img = weight;
    pp->weight_txt = w_txt;
    pp->freqs_txt = reinterpret_cast<const float2*>(prep->rope_freqs_txt);
    pp->freqs_img = reinterpret_cast<const float2*>(prep->rope_freqs_img);
    *out = pp;
    return 0;
  }
  const bool comfy = prep->kind == KSANA_SAGE_PREP_WAN_COMFY;
  if (!weight && !(comfy ? (const void*)prep->rope_matrices : (const void*)prep->rope_freqs)) return 0;
  memset(pp, 0, sizeof(*pp));
  pp->L = L;
  pp->kind = comfy ? 3 : 1;
  if (weight) {
    if (reinterpret_cast<uintptr_t>(weight) & 15u)
      return fail(KSANA_SAGE_EINVAL, "%s norm weight not 16-byte aligned", name);
    if (st[2] != ksana_sage::kD)
      return fail(KSANA_SAGE_EINVAL, "%s: RMSNorm over the token row needs the H stride to be %d, got %lld", name,
                  ksana_sage::kD, (long long)st[2]);
    if (!(prep->norm_eps >= 0.0f)) return fail(KSANA_SAGE_EINVAL, "norm_eps must be >= 0");
    pp->inv_rms = inv_rms;
    pp->weight = weight;
  }
  if (comfy) {
    if (prep->rope_matrices) {
      if (reinterpret_cast<uintptr_t>(prep->rope_matrices) & 15u)
        return fail(KSANA_SAGE_EINVAL, "rope_matrices not 16-byte aligned");
      if (prep->rope_rows < 1) return fail(KSANA_SAGE_EINVAL, "rope_rows must be positive");
      pp->rot = reinterpret_cast<const float4*>(prep->rope_matrices);
      pp->rot_rows = prep->rope_rows;
    }
  } else if (prep->rope_freqs) {
    if (reinterpret_cast<uintptr_t>(prep->rope_freqs) & 15u)
      return fail(KSANA_SAGE_EINVAL, "rope_freqs not 16-byte aligned");
    if (!prep->grid_sizes) return fail(KSANA_SAGE_EINVAL, "rope_freqs given without grid_sizes");
    if (B > ksana_sage::kMaxPrepBatch)
      return fail(KSANA_SAGE_ENOTSUP, "RoPE on the fly supports at most %d batch entries, got %d",
                  ksana_sage::kMaxPrepBatch, B);
    if (prep->rope_rows < 1) return fail(KSANA_SAGE_EINVAL, "rope_rows must be positive");
    for (int b = 0; b < B; ++b) {
      const int32_t* g = prep->grid_sizes + 3 * b;
      for (int a = 0; a < 3; ++a) {
        if (g[a] < 1 || g[a] > prep->rope_rows)
          return fail(KSANA_SAGE_EINVAL, "grid_sizes[%d][%d]=%d outside [1, rope_rows=%d]", b, a, g[a],
                      prep->rope_rows);
        pp->grid[b][a] = g[a];
      }
      if ((int64_t)g[0] * g[1] * g[2] > L)
        return fail(KSANA_SAGE_EINVAL, "grid_sizes[%d] = %dx%dx%d exceeds the %s sequence length %d", b, g[0], g[1],
                    g[2], name, L);
    }
    pp->freqs = prep->rope_freqs;
  }
  *out = pp;
  return 0;
}

}  // namespace

extern "C" {

int ksana_sage_abi_version(void) { return KSANA_SAGE_ABI_VERSION; }

const char* ksana_sage_last_error(void) { return g_err; }

int ksana_sage_configure(const char* one_read_stages, int64_t wait_ticks) {
  if (one_read_stages != nullptr)
    for (const char* c = one_read_stages; *c; ++c)
      if (*c != 'k' && *c != 'v') return fail(KSANA_SAGE_EINVAL, "one_read_stages \"%s\": letters k and v only", one_read_stages);
  ksana_sage::configure_quant(one_read_stages, wait_ticks, wait_ticks == KSANA_SAGE_KEEP);
  return 0;
}

int ksana_sage_one_read_state(int* one_read_k, int* one_read_v, int64_t* wait_ticks, int* demoted) {
  const ksana_sage::QuantOptions o = ksana_sage::quant_options();
  if (one_read_k) *one_read_k = o.one_read_k;
  if (one_read_v) *one_read_v = o.one_read_v;
  if (wait_ticks) *wait_ticks = o.wait_ticks;
  if (demoted) *demoted = ksana_sage::one_read_demoted(/*may_allocate=*/false) ? 1 : 0;
  return 0;
}

int ksana_sage_selftest(void) {
  const int rc = ksana_sage::selftest_occupancy_cache();
  return rc == 0 ? 0 : fail(KSANA_SAGE_EINVAL, "occupancy cache self-check failed at step %d", rc);
}

int ksana_sage_workspace_layout(const ksana_sage_shape* s, ksana_sage_ws_layout* out) {
  if (int rc = check_shape(s)) return rc;
  if (!out) return fail(KSANA_SAGE_EINVAL, "layout out-pointer is null");
  using namespace ksana_sage;
  ksana_sage_ws_layout l;
  memset(&l, 0, sizeof(l));
  l.lq_pad = (s->Lq + kQPad - 1) / kQPad * kQPad;
  l.nqb = l.lq_pad;  // one scale per (padded) query row
  l.nkb = (s->Lk + kBlkK - 1) / kBlkK;
  l.nch = (s->Lk + kMeanChunk - 1) / kMeanChunk;
  const uint64_t bhq = (uint64_t)s->B * s->Hq, bhk = (uint64_t)s->B * s->Hkv;
  uint64_t off = 0;
  auto take = [&](uint64_t bytes) {
    const uint64_t at = off;
    off = align256(off + bytes);
    return at;
  };
  l.q_i8 = take(bhq * l.lq_pad * kD);
  l.q_scale = take(bhq * l.nqb * 4);
  l.k_i8 = take(bhk * l.nkb * kTileBytes);
  l.k_scale = take(bhk * l.nkb * 4);
  l.k_mean = take(bhk * kD * 4);
  l.v_fp8 = take(bhk * l.nkb * kTileBytes);
  l.v_scale = take(bhk * kD * 4);
  l.v_inv = take(bhk * kD * 4);
  l.k_part = take(bhk * l.nch * kD * 4);
  l.v_part = take(bhk * l.nch * kD * 4);
  l.q_rms = take((uint64_t)s->B * s->Lq * 4);
  l.k_rms = take((uint64_t)s->B * s->Lk * 4);
  l.v_mean = take(bhk * kD * 4);
  l.split_o = take((uint64_t)kMaxSplitPartials * kAttnQPerWg * kD * 4);
  l.split_ml = take((uint64_t)kMaxSplitPartials * kAttnQPerWg * 2 * 4);
  l.k_sync = take((uint64_t)sync_words((int)bhk) * 4);
  l.v_sync = take((uint64_t)sync_words((int)bhk) * 4);
  l.total_bytes = off;
  *out = l;
  return 0;
}

int ksana_sage_quant_q(const void* q, int dtype, const int64_t st[4], const ksana_sage_shape* s, float sm_scale,
                       void* ws, void* stream) {
  return ksana_sage_quant_q_prep(q, dtype, st, s, nullptr, sm_scale, ws, stream);
}

// `k` != nullptr (the caller has checked k as a tensor): when q's path takes whole token rows anyway (a norm over the
// row), the row statistic of k is taken along and *k_rms_done says so
static int quant_q_impl(const void* q, int dtype, const int64_t st[4], const ksana_sage_shape* s,
                        const ksana_sage_prep* prep, float sm_scale, void* ws, void* stream, const void* k,
                        const int64_t k_st[4], bool* k_rms_done, uint16_t* pooled = nullptr) {
  const StageRange range("ksana_sage.quant_q");
  if (k_rms_done) *k_rms_done = false;
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_tensor("q", q, dtype, st, s->B, s->Lq, s->Hq)) return rc;
  if (int rc = check_ws(ws)) return rc;
  ksana_sage_ws_layout l;
  ksana_sage_workspace_layout(s, &l);
  ksana_sage::PrepParams pp;
  const ksana_sage::PrepParams* ppp = nullptr;
  if (int rc = make_prep(prep, prep ? prep->q_norm_weight : nullptr, "q", st, s->B, s->Lq, s->D, ws_at<float>(ws, l.q_rms),
                         &pp, &ppp))
    return rc;
  // one fp32 product, then an exact power of two (1/128 undoes the unnormalised Hadamard
  // transforms of Q and K): part of the quantizer specification
  const float premul = (sm_scale * 1.4426950408889634f) * 0.0078125f;
  if (ppp && ppp->inv_rms) {
    // a norm over the token row: statistic and quantization in one kernel that takes whole rows
    const bool take_k = k != nullptr && prep->k_norm_weight != nullptr && k_st[2] == ksana_sage::kD;
    const ksana_sage::InTensor kt = take_k ? in_tensor(k, dtype, k_st, s->D) : ksana_sage::InTensor{};
    hipError_t e = ksana_sage::launch_quant_q_rows(in_tensor(q, dtype, st, s->D), s->B, s->Hq, s->Lq, l.lq_pad, premul,
                                                   prep->norm_eps, ws_at<int8_t>(ws, l.q_i8), ws_at<float>(ws, l.q_scale),
                                                   static_cast<hipStream_t>(stream), *ppp, take_k ? &kt : nullptr,
                                                   s->Hkv, s->Lk, ws_at<float>(ws, l.k_rms));
    if (e != hipSuccess) return hip_fail(e, "quant_q (whole rows) launch");
    if (k_rms_done) *k_rms_done = take_k;
    return 0;
  }
  hipError_t e = ksana_sage::launch_quant_q(in_tensor(q, dtype, st, s->D), s->B, s->Hq, s->Lq, l.lq_pad, premul,
                                            ws_at<int8_t>(ws, l.q_i8), ws_at<float>(ws, l.q_scale),
                                            static_cast<hipStream_t>(stream), ppp, pooled);
  return e == hipSuccess ? 0 : hip_fail(e, "quant_q launch");
}

int ksana_sage_quant_q_prep(const void* q, int dtype, const int64_t st[4], const ksana_sage_shape* s,
                            const ksana_sage_prep* prep, float sm_scale, void* ws, void* stream) {
  return quant_q_impl(q, dtype, st, s, prep, sm_scale, ws, stream, nullptr, nullptr, nullptr);
}

int ksana_sage_quant_k(const void* k, int dtype, const int64_t st[4], const ksana_sage_shape* s, int smooth_k,
                       void* ws, void* stream) {
  return ksana_sage_quant_k_prep(k, dtype, st, s, nullptr, smooth_k, ws, stream);
}

// `part` == nullptr: the chunk sums and the counters go to the workspace's own k_part / k_sync areas
// `rms_done`: the row statistic of k (k_rms area) has been taken by the call before (quant_q_impl)
static int quant_k_impl(const void* k, int dtype, const int64_t st[4], const ksana_sage_shape* s,
                        const ksana_sage_prep* prep, int smooth_k, void* ws, float* part, int* sync_words,
                        void* stream, bool rms_done = false, bool may_allocate = true, uint16_t* pooled = nullptr) {
  const StageRange range("ksana_sage.quant_k");
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_tensor("k", k, dtype, st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = check_ws(ws)) return rc;
  ksana_sage_ws_layout l;
  ksana_sage_workspace_layout(s, &l);
  hipStream_t hs = static_cast<hipStream_t>(stream);
  const ksana_sage::InTensor kt = in_tensor(k, dtype, st, s->D);
  const int bhk = s->B * s->Hkv;
  if (part == nullptr) part = ws_at<float>(ws, l.k_part);
  if (sync_words == nullptr) sync_words = ws_at<int>(ws, l.k_sync);
  ksana_sage::PrepParams pp;
  const ksana_sage::PrepParams* ppp = nullptr;
  if (int rc = make_prep(prep, prep ? prep->k_norm_weight : nullptr, "k", st, s->B, s->Lk, s->D, ws_at<float>(ws, l.k_rms),
                         &pp, &ppp))
    return rc;
  hipError_t e = hipSuccess;
  if (ppp && ppp->inv_rms && !rms_done) {
    e = ksana_sage::launch_row_inv_rms(kt, s->B, s->Hkv, s->Lk, prep->norm_eps, ws_at<float>(ws, l.k_rms), hs);
    if (e != hipSuccess) return hip_fail(e, "k row statistic launch");
  }
  if ((one_read('k') || ppp != nullptr) && pooled == nullptr) {  // (block averages ride in the two-pass kernel)
    // one read of K: chunk sums, the head's mean and the quantization in one kernel, when the shape suits it (always
    // tried when the step before attention is applied on the way in: the rotation is then done once, not twice)
    e = ksana_sage::launch_clear_ints(sync_words, ksana_sage::sync_words(bhk), hs);
    if (e != hipSuccess) return hip_fail(e, "k counter clear launch");
    bool used = false;
    e = ksana_sage::launch_quant_k_fused(kt, s->B, s->Hkv, s->Lk, l.nkb, l.nch, smooth_k ? 1 : 0, part,
                                         ws_at<float>(ws, l.k_mean), ws_at<int8_t>(ws, l.k_i8),
                                         ws_at<float>(ws, l.k_scale), sync_at(sync_words, nullptr, bhk), hs, ppp, &used,
                                         may_allocate);
    if (e != hipSuccess) return hip_fail(e, "fused quant_k launch");
    if (used) return 0;
  }
  if (smooth_k) {
    e = ksana_sage::launch_col_partial(kt, s->B, s->Hkv, s->Lk, 0, part, l.nch, hs, ppp);
    if (e != hipSuccess) return hip_fail(e, "k column-sum launch");
  }
  e = ksana_sage::launch_k_mean_finalize(part, bhk, smooth_k ? l.nch : 0, s->Lk, dtype, smooth_k,
                                         ws_at<float>(ws, l.k_mean), hs, sync_at(sync_words, nullptr, bhk).k_status);
  if (e != hipSuccess) return hip_fail(e, "k mean finalize launch");
  e = ksana_sage::launch_quant_k(kt, s->B, s->Hkv, s->Lk, l.nkb, ws_at<float>(ws, l.k_mean),
                                 ws_at<int8_t>(ws, l.k_i8), ws_at<float>(ws, l.k_scale), hs, ppp, pooled);
  return e == hipSuccess ? 0 : hip_fail(e, "quant_k launch");
}

int ksana_sage_quant_k_prep(const void* k, int dtype, const int64_t st[4], const ksana_sage_shape* s,
                            const ksana_sage_prep* prep, int smooth_k, void* ws, void* stream) {
  return quant_k_impl(k, dtype, st, s, prep, smooth_k, ws, nullptr, nullptr, stream);
}

int ksana_sage_quant_qk_prep(const void* q, const void* k, int dtype, const int64_t q_st[4], const int64_t k_st[4],
                             const ksana_sage_shape* s, const ksana_sage_prep* prep, float sm_scale, int smooth_k,
                             void* ws, void* stream) {
  // k is checked before q's kernels go out: nothing is launched for a call that fails
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_tensor("k", k, dtype, k_st, s->B, s->Lk, s->Hkv)) return rc;
  {
    ksana_sage::PrepParams pp;
    const ksana_sage::PrepParams* ppp = nullptr;
    float dummy = 0.0f;  // only the validation matters here
    if (int rc = make_prep(prep, prep ? prep->k_norm_weight : nullptr, "k", k_st, s->B, s->Lk, s->D, &dummy, &pp, &ppp))
      return rc;
  }
  bool k_rms_done = false;
  if (int rc = quant_q_impl(q, dtype, q_st, s, prep, sm_scale, ws, stream, k, k_st, &k_rms_done)) return rc;
  return quant_k_impl(k, dtype, k_st, s, prep, smooth_k, ws, nullptr, nullptr, stream, k_rms_done);
}

int ksana_sage_quant_qk_pooled(const void* q, const void* k, int dtype, const int64_t q_st[4], const int64_t k_st[4],
                               const ksana_sage_shape* s, float sm_scale, void* pooled_q, void* pooled_k, void* ws,
                               void* stream) {
  if (int rc = check_shape(s)) return rc;
  if (s->D != ksana_sage::kD)
    return fail(KSANA_SAGE_ENOTSUP, "head size %d: the block averages are taken at head size %d only", s->D, ksana_sage::kD);
  if (pooled_q == nullptr || pooled_k == nullptr) return fail(KSANA_SAGE_EINVAL, "pooled_q / pooled_k is NULL");
  if ((reinterpret_cast<uintptr_t>(pooled_q) | reinterpret_cast<uintptr_t>(pooled_k)) & 1)
    return fail(KSANA_SAGE_EINVAL, "pooled_q / pooled_k is not 2-byte aligned");
  // k is checked before q's kernel goes out: nothing is launched for a call that fails
  if (int rc = check_tensor("k", k, dtype, k_st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = quant_q_impl(q, dtype, q_st, s, nullptr, sm_scale, ws, stream, nullptr, nullptr, nullptr,
                            static_cast<uint16_t*>(pooled_q)))
    return rc;
  return quant_k_impl(k, dtype, k_st, s, nullptr, 1, ws, nullptr, nullptr, stream, false, true,
                      static_cast<uint16_t*>(pooled_k));
}

int ksana_sage_quant_k_static(const void* k, int dtype, const int64_t st[4], const ksana_sage_shape* s, int smooth_k,
                              void* ws, void* stream) {
  if (int rc = check_shape(s)) return rc;
  const int64_t chunk_rows = (int64_t)s->B * s->Hkv * ((s->Lk + ksana_sage::kMeanChunk - 1) / ksana_sage::kMeanChunk);
  if (chunk_rows > kStaticChunkRows || (int64_t)s->B * s->Hkv > kStaticHeads)
    return fail(KSANA_SAGE_ENOTSUP,
                "B*Hkv*ceil(Lk/256) = %lld, B*Hkv = %lld: the library's own scratch holds %d chunk sums of %d heads; "
                "use ksana_sage_quant_k, whose scratch is part of the caller's workspace",
                (long long)chunk_rows, (long long)s->B * s->Hkv, kStaticChunkRows, kStaticHeads);
  // everything else is validated before the device is touched, like in ksana_sage_quant_k
  if (int rc = check_tensor("k", k, dtype, st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = check_ws(ws)) return rc;
  float* part = nullptr;
  if (int rc = static_scratch(&part)) return rc;
  // every chunk sum that is read is written earlier in the same call; the counters and flags behind the partial
  // sums are cleared by the call's first kernel
  return quant_k_impl(k, dtype, st, s, nullptr, smooth_k, ws, part, reinterpret_cast<int*>(part + kStaticPartFloats),
                      stream, false, /*may_allocate=*/false);
}

int ksana_sage_quant_v(const void* v, int dtype, const int64_t st[4], const ksana_sage_shape* s, void* ws,
                       void* stream) {
  return ksana_sage_quant_v_smooth(v, dtype, st, s, 0, ws, stream);
}

int ksana_sage_quant_v_smooth(const void* v, int dtype, const int64_t st[4], const ksana_sage_shape* s, int smooth_v,
                              void* ws, void* stream) {
  const StageRange range("ksana_sage.quant_v");
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_tensor("v", v, dtype, st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = check_ws(ws)) return rc;
  ksana_sage_ws_layout l;
  ksana_sage_workspace_layout(s, &l);
  hipStream_t hs = static_cast<hipStream_t>(stream);
  const ksana_sage::InTensor vt = in_tensor(v, dtype, st, s->D);
  const int bhk = s->B * s->Hkv;
  float* v_mean = ws_at<float>(ws, l.v_mean);
  hipError_t e = hipSuccess;
  if (!smooth_v && one_read('v')) {
    // one read of V: column maxima, scales and the quantization in one kernel, when the shape suits it
    int* words = ws_at<int>(ws, l.v_sync);
    e = ksana_sage::launch_clear_ints(words, ksana_sage::sync_words(bhk), hs);
    if (e != hipSuccess) return hip_fail(e, "v counter clear launch");
    bool used = false;
    e = ksana_sage::launch_quant_v_fused(vt, s->B, s->Hkv, s->Lk, l.nkb, l.nch, ws_at<float>(ws, l.v_part),
                                         ws_at<float>(ws, l.v_scale),
                                         ws_at<float>(ws, l.v_inv), v_mean, ws_at<uint8_t>(ws, l.v_fp8),
                                         sync_at(nullptr, words, bhk), hs, &used);
    if (e != hipSuccess) return hip_fail(e, "fused quant_v launch");
    if (used) return 0;
  }
  if (smooth_v) {
    e = ksana_sage::launch_col_partial(vt, s->B, s->Hkv, s->Lk, 0, ws_at<float>(ws, l.v_part), l.nch, hs);
    if (e != hipSuccess) return hip_fail(e, "v column sum launch");
    // the same finalisation as for K: the mean rounded to the input dtype
    e = ksana_sage::launch_k_mean_finalize(ws_at<float>(ws, l.v_part), bhk, l.nch, s->Lk, dtype, 1, v_mean, hs);
    if (e != hipSuccess) return hip_fail(e, "v mean finalize launch");
  }
  e = ksana_sage::launch_col_partial(vt, s->B, s->Hkv, s->Lk, smooth_v ? 2 : 1, ws_at<float>(ws, l.v_part), l.nch, hs,
                                     nullptr, smooth_v ? v_mean : nullptr);
  if (e != hipSuccess) return hip_fail(e, "v abs-max launch");
  // without smoothing the mean slot is cleared here: the attention adds whatever it holds
  e = ksana_sage::launch_v_scale_finalize(ws_at<float>(ws, l.v_part), s->B * s->Hkv, l.nch,
                                          ws_at<float>(ws, l.v_scale), ws_at<float>(ws, l.v_inv),
                                          smooth_v ? nullptr : v_mean, hs,
                                          sync_at(nullptr, ws_at<int>(ws, l.v_sync), bhk).v_status);
  if (e != hipSuccess) return hip_fail(e, "v scale finalize launch");
  e = ksana_sage::launch_quant_v(vt, s->B, s->Hkv, s->Lk, l.nkb, ws_at<float>(ws, l.v_inv),
                                 smooth_v ? v_mean : nullptr, ws_at<uint8_t>(ws, l.v_fp8), hs);
  return e == hipSuccess ? 0 : hip_fail(e, "quant_v launch");
}

int ksana_sage_quant_status(const void* ws, const ksana_sage_shape* s, void* stream, int* k_status, int* v_status) {
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_ws(ws)) return rc;
  if (!k_status || !v_status) return fail(KSANA_SAGE_EINVAL, "out-pointer is null");
  ksana_sage_ws_layout l;
  ksana_sage_workspace_layout(s, &l);
  const int bhk = s->B * s->Hkv;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  hipError_t e = hipStreamSynchronize(hs);
  if (e != hipSuccess) return hip_fail(e, "stream synchronize");
  const int at = 2 * bhk * ksana_sage::kSyncStride;
  e = hipMemcpy(k_status, ws_at<int>(ws, l.k_sync) + at, sizeof(int), hipMemcpyDeviceToHost);
  if (e != hipSuccess) return hip_fail(e, "status copy");
  e = hipMemcpy(v_status, ws_at<int>(ws, l.v_sync) + at, sizeof(int), hipMemcpyDeviceToHost);
  return e == hipSuccess ? 0 : hip_fail(e, "status copy");
}

int ksana_sage_block_means(const void* x, int dtype, const int64_t st[4], int B, int H, int L, int rows_per_block,
                           const float* centre, void* out, void* stream) {
  if (B < 1 || H < 1 || L < 1 || B > 65535 || H > 65535)
    return fail(KSANA_SAGE_EINVAL, "bad extent (B=%d H=%d L=%d)", B, H, L);
  if (rows_per_block < 32 || rows_per_block > 256 || rows_per_block % 32 != 0)
    return fail(KSANA_SAGE_ENOTSUP, "rows_per_block=%d: a multiple of 32 up to 256 is supported", rows_per_block);
  if (int rc = check_tensor("x", x, dtype, st, B, L, H)) return rc;
  if (!out || (reinterpret_cast<uintptr_t>(out) & 1u)) return fail(KSANA_SAGE_EINVAL, "out is null or misaligned");
  if (reinterpret_cast<uintptr_t>(centre) & 3u) return fail(KSANA_SAGE_EINVAL, "centre is not 4-byte aligned");
  hipError_t e = ksana_sage::launch_block_means(in_tensor(x, dtype, st), B, H, L, rows_per_block, centre,
                                                static_cast<uint16_t*>(out), static_cast<hipStream_t>(stream));
  return e == hipSuccess ? 0 : hip_fail(e, "block means launch");
}

static int sla_layout(int B, int H, int L, uint64_t* part, uint64_t* m_frag, uint64_t* ksum, uint64_t* total) {
  if (B < 1 || H < 1 || L < 1 || B > 65535 || H > 65535) return fail(KSANA_SAGE_EINVAL, "bad extent (B=%d H=%d L=%d)", B, H, L);
  int runs = 1, rows_per_run = L;
  ksana_sage::plan_sla_runs(B, H, L, &runs, &rows_per_run);
  const uint64_t bh = (uint64_t)B * H;
  uint64_t off = 0;
  *part = off, off = align256(off + bh * runs * (ksana_sage::kD * ksana_sage::kD + ksana_sage::kD) * 4);
  *m_frag = off, off = align256(off + bh * ksana_sage::kD * ksana_sage::kD * 2);
  *ksum = off, off = align256(off + bh * ksana_sage::kD * 4);
  *total = off;
  return 0;
}

int ksana_sage_sla_workspace_bytes(int B, int H, int L, uint64_t* bytes) {
  if (!bytes) return fail(KSANA_SAGE_EINVAL, "out-pointer is null");
  uint64_t a, b, c;
  return sla_layout(B, H, L, &a, &b, &c, bytes);
}

int ksana_sage_sla_linear(const void* q, const void* k, const void* v, int dtype, const int64_t q_st[4],
                          const int64_t k_st[4], const int64_t v_st[4], int B, int H, int L, const float* proj_weight,
                          const float* proj_bias, const void* add, const int64_t add_st[4], void* out,
                          const int64_t out_st[4], void* sla_workspace, void* stream) {
  const StageRange range("ksana_sage.sla_linear");
  uint64_t o_part, o_frag, o_ksum, total;
  if (int rc = sla_layout(B, H, L, &o_part, &o_frag, &o_ksum, &total)) return rc;
  if (int rc = check_tensor("q", q, dtype, q_st, B, L, H)) return rc;
  if (int rc = check_tensor("k", k, dtype, k_st, B, L, H)) return rc;
  if (int rc = check_tensor("v", v, dtype, v_st, B, L, H)) return rc;
  if (int rc = check_tensor("out", out, dtype, out_st, B, L, H)) return rc;
  if (add != nullptr)
    if (int rc = check_tensor("add", add, dtype, add_st, B, L, H)) return rc;
  if (int rc = check_ws(sla_workspace)) return rc;
  if ((reinterpret_cast<uintptr_t>(proj_weight) | reinterpret_cast<uintptr_t>(proj_bias)) & 15u)
    return fail(KSANA_SAGE_EINVAL, "projection weight / bias not 16-byte aligned");
  const ksana_sage::InTensor at = add != nullptr ? in_tensor(add, dtype, add_st) : ksana_sage::InTensor{};
  const ksana_sage::OutTensor ot{static_cast<uint16_t*>(out), out_st[0], out_st[1], out_st[2], dtype};
  hipError_t e = ksana_sage::launch_sla_linear(in_tensor(q, dtype, q_st), in_tensor(k, dtype, k_st), in_tensor(v, dtype, v_st), B, H, L,
                                               proj_weight, proj_bias, add != nullptr ? &at : nullptr, ot,
                                               ws_at<float>(sla_workspace, o_part), ws_at<uint16_t>(sla_workspace, o_frag),
                                               ws_at<float>(sla_workspace, o_ksum), static_cast<hipStream_t>(stream));
  return e == hipSuccess ? 0 : hip_fail(e, "sla linear branch launch");
}

int ksana_sage_sla_block_map(const void* pooled_q, const void* pooled_k, int dtype, int B, int H, int nq, int nk, int keep,
                             int8_t* block_map, void* stream) {
  if (B < 1 || H < 1 || nq < 1 || nk < 1 || (int64_t)B * H > 65535) return fail(KSANA_SAGE_EINVAL, "bad extent (B=%d H=%d nq=%d nk=%d)", B, H, nq, nk);
  if (dtype != KSANA_SAGE_BF16 && dtype != KSANA_SAGE_FP16) return fail(KSANA_SAGE_EINVAL, "dtype %d unknown", dtype);
  if (nk > 1024) return fail(KSANA_SAGE_ENOTSUP, "nk=%d key blocks exceed 1024 (a group's scores are kept in LDS)", nk);
  if (!pooled_q || !pooled_k || !block_map) return fail(KSANA_SAGE_EINVAL, "null pointer");
  if ((reinterpret_cast<uintptr_t>(pooled_q) | reinterpret_cast<uintptr_t>(pooled_k)) & 15u)
    return fail(KSANA_SAGE_EINVAL, "pooled blocks not 16-byte aligned");
  hipError_t e = ksana_sage::launch_sla_block_map(static_cast<const uint16_t*>(pooled_q), static_cast<const uint16_t*>(pooled_k),
                                                  dtype, B * H, nq, nk, keep, block_map, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? 0 : hip_fail(e, "block map launch");
}

int ksana_sage_attn_key_split(const ksana_sage_shape* s, int* first_workgroup, int* runs) {
  if (int rc = check_shape(s)) return rc;
  if (!first_workgroup || !runs) return fail(KSANA_SAGE_EINVAL, "out-pointer is null");
  const int n_qwg = (s->Lq + ksana_sage::kAttnQPerWg - 1) / ksana_sage::kAttnQPerWg;
  ksana_sage::plan_key_split(s->B * s->Hq * n_qwg, (s->Lk + ksana_sage::kBlkK - 1) / ksana_sage::kBlkK, first_workgroup,
                             runs);
  return 0;
}

int ksana_sage_attn_fwd(void* ws, void* o, int dtype, const int64_t o_st[4], const ksana_sage_shape* s,
                        const int32_t* k_lens, int causal, int flags, void* stream) {
  return ksana_sage_attn_fwd_masked(ws, o, dtype, o_st, s, nullptr, nullptr, k_lens, causal, flags, stream);
}

int ksana_sage_attn_fwd_masked(void* ws, void* o, int dtype, const int64_t o_st[4], const ksana_sage_shape* s,
                               const int8_t* block_mask, const int64_t mask_st[2], const int32_t* k_lens, int causal,
                               int flags, void* stream) {
  return ksana_sage_attn_fwd_varlen(ws, o, dtype, o_st, s, block_mask, mask_st, nullptr, k_lens, causal, flags, stream);
}

int ksana_sage_attn_fwd_varlen(void* ws, void* o, int dtype, const int64_t o_st[4], const ksana_sage_shape* s,
                               const int8_t* block_mask, const int64_t mask_st[2], const int32_t* q_lens,
                               const int32_t* k_lens, int causal, int flags, void* stream) {
  const StageRange range("ksana_sage.attention");
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_mask(s, block_mask, mask_st)) return rc;
  if (int rc = check_causal(s, causal)) return rc;
  if (flags & ~(KSANA_SAGE_FLAG_PWL_EXP2 | KSANA_SAGE_FLAG_WG_4_WAVES | KSANA_SAGE_FLAG_WG_8_WAVES | KSANA_SAGE_FLAG_TILE_SKIP))
    return fail(KSANA_SAGE_EINVAL, "unknown flag bits 0x%x", flags);
  if ((flags & KSANA_SAGE_FLAG_TILE_SKIP) && (flags & KSANA_SAGE_FLAG_PWL_EXP2))
    return fail(KSANA_SAGE_EINVAL, "KSANA_SAGE_FLAG_TILE_SKIP goes with the exact exponential only, not with KSANA_SAGE_FLAG_PWL_EXP2");
  if (int rc = check_tensor("o", o, dtype, o_st, s->B, s->Lq, s->Hq)) return rc;
  if (int rc = check_ws(ws)) return rc;
  if (reinterpret_cast<uintptr_t>(k_lens) & 3) return fail(KSANA_SAGE_EINVAL, "k_lens is not 4-byte aligned");
  if (reinterpret_cast<uintptr_t>(q_lens) & 3) return fail(KSANA_SAGE_EINVAL, "q_lens is not 4-byte aligned");
  ksana_sage_ws_layout l;
  ksana_sage_workspace_layout(s, &l);
  ksana_sage::AttnParams p;
  p.q_i8 = ws_at<int8_t>(ws, l.q_i8);
  p.q_scale = ws_at<float>(ws, l.q_scale);
  p.k_tiles = ws_at<int8_t>(ws, l.k_i8);
  p.k_scale = ws_at<float>(ws, l.k_scale);
  p.v_tiles = ws_at<uint8_t>(ws, l.v_fp8);
  p.v_scale = ws_at<float>(ws, l.v_scale);
  p.v_mean = ws_at<float>(ws, l.v_mean);
  p.split_o = ws_at<float>(ws, l.split_o);
  p.split_ml = ws_at<float>(ws, l.split_ml);
  p.split_first_wg = 0, p.n_split = 0;
  p.wg_waves = (flags & KSANA_SAGE_FLAG_WG_4_WAVES) ? 4 : ((flags & KSANA_SAGE_FLAG_WG_8_WAVES) ? 8 : 0);
  p.o = ksana_sage::OutTensor{static_cast<uint16_t*>(o), o_st[0], o_st[1], o_st[2], dtype};
  p.B = s->B, p.Hq = s->Hq, p.Hkv = s->Hkv, p.Lq = s->Lq, p.Lk = s->Lk;
  p.lq_pad = l.lq_pad, p.nkb = l.nkb;
  p.exact_exp2 = (flags & KSANA_SAGE_FLAG_PWL_EXP2) ? 0 : 1;
  p.k_lens = k_lens;
  p.q_lens = q_lens;
  p.block_mask = block_mask;
  p.mask_sB = block_mask ? mask_st[0] : 0;
  p.mask_sH = block_mask ? mask_st[1] : 0;
  p.causal = causal ? 1 : 0;
  p.d_out = s->D;
  p.tile_skip = (flags & KSANA_SAGE_FLAG_TILE_SKIP) ? 1 : 0;
  hipError_t e = ksana_sage::launch_attn_fwd(p, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? 0 : hip_fail(e, "attention launch");
}

int ksana_sage_forward(const void* q, const void* k, const void* v, void* o, int dtype, const int64_t q_st[4],
                       const int64_t k_st[4], const int64_t v_st[4], const int64_t o_st[4],
                       const ksana_sage_shape* s, const int32_t* k_lens, float sm_scale, int smooth_k, int causal,
                       int flags, void* ws, void* stream) {
  return ksana_sage_forward_prep(q, k, v, o, dtype, q_st, k_st, v_st, o_st, s, nullptr, k_lens, sm_scale, smooth_k,
                                 causal, flags, ws, stream);
}

int ksana_sage_forward_prep(const void* q, const void* k, const void* v, void* o, int dtype, const int64_t q_st[4],
                            const int64_t k_st[4], const int64_t v_st[4], const int64_t o_st[4],
                            const ksana_sage_shape* s, const ksana_sage_prep* prep, const int32_t* k_lens,
                            float sm_scale, int smooth_k, int causal, int flags, void* ws, void* stream) {
  return forward_impl(q, k, v, o, dtype, q_st, k_st, v_st, o_st, s, prep, nullptr, nullptr, k_lens, sm_scale, smooth_k,
                      causal, flags, ws, stream);
}

int ksana_sage_forward_masked(const void* q, const void* k, const void* v, void* o, int dtype, const int64_t q_st[4],
                              const int64_t k_st[4], const int64_t v_st[4], const int64_t o_st[4],
                              const ksana_sage_shape* s, const int8_t* block_mask, const int64_t mask_st[2],
                              const int32_t* k_lens, float sm_scale, int smooth_k, int causal, int flags, void* ws,
                              void* stream) {
  return forward_impl(q, k, v, o, dtype, q_st, k_st, v_st, o_st, s, nullptr, block_mask, mask_st, k_lens, sm_scale,
                      smooth_k, causal, flags, ws, stream);
}

}  // extern "C"

namespace {
int forward_impl(const void* q, const void* k, const void* v, void* o, int dtype, const int64_t q_st[4],
                 const int64_t k_st[4], const int64_t v_st[4], const int64_t o_st[4], const ksana_sage_shape* s,
                 const ksana_sage_prep* prep, const int8_t* block_mask, const int64_t mask_st[2],
                 const int32_t* k_lens, float sm_scale, int smooth_k, int causal, int flags, void* ws, void* stream) {
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_mask(s, block_mask, mask_st)) return rc;
  if (int rc = check_causal(s, causal)) return rc;
  // validate everything before the first launch so a bad argument leaves no partial work
  if (int rc = check_tensor("q", q, dtype, q_st, s->B, s->Lq, s->Hq)) return rc;
  if (int rc = check_tensor("k", k, dtype, k_st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = check_tensor("v", v, dtype, v_st, s->B, s->Lk, s->Hkv)) return rc;
  if (int rc = check_tensor("o", o, dtype, o_st, s->B, s->Lq, s->Hq)) return rc;
  if (int rc = check_ws(ws)) return rc;
  if (flags & ~(KSANA_SAGE_FLAG_PWL_EXP2 | KSANA_SAGE_FLAG_SMOOTH_V | KSANA_SAGE_FLAG_WG_4_WAVES | KSANA_SAGE_FLAG_WG_8_WAVES |
                KSANA_SAGE_FLAG_TILE_SKIP))
    return fail(KSANA_SAGE_EINVAL, "unknown flag bits 0x%x", flags);
  if (reinterpret_cast<uintptr_t>(k_lens) & 3) return fail(KSANA_SAGE_EINVAL, "k_lens is not 4-byte aligned");
  {
    ksana_sage::PrepParams pp;
    const ksana_sage::PrepParams* ppp = nullptr;
    float dummy = 0.0f;  // only the validation matters here
    if (int rc = make_prep(prep, prep ? prep->q_norm_weight : nullptr, "q", q_st, s->B, s->Lq, s->D, &dummy, &pp, &ppp))
      return rc;
    if (int rc = make_prep(prep, prep ? prep->k_norm_weight : nullptr, "k", k_st, s->B, s->Lk, s->D, &dummy, &pp, &ppp))
      return rc;
  }
  if (int rc = ksana_sage_quant_qk_prep(q, k, dtype, q_st, k_st, s, prep, sm_scale, smooth_k, ws, stream)) return rc;
  if (int rc = ksana_sage_quant_v_smooth(v, dtype, v_st, s, flags & KSANA_SAGE_FLAG_SMOOTH_V, ws, stream)) return rc;
  return ksana_sage_attn_fwd_masked(ws, o, dtype, o_st, s, block_mask, mask_st, k_lens, causal,
                                    flags & ~KSANA_SAGE_FLAG_SMOOTH_V, stream);
}
}  // namespace
