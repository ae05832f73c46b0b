// C-ABI layer of libmagi_attn: argument validation, error reporting, kernel dispatch.
#include <hip/hip_runtime.h>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "kernels.h"
#include "magi_attn.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(MAGI_EHIP, "%s: %s", what, hipGetErrorString(e));
}

std::atomic<uint64_t> g_launches{0};

// the caller's view of an argument struct must be this library's
template <class T>
bool same_layout(const T* p) { return p->struct_size == sizeof(T); }
#define MAGI_CHECK_LAYOUT(fn, p)                                                                            \
  if (!same_layout(p))                                                                                      \
    return fail(MAGI_EINVAL, fn ": struct_size %u, this library expects %zu (header / library version mismatch)", \
                (unsigned)(p)->struct_size, sizeof(*(p)))

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// compute units of the current device (asked once per device; 256 when the query fails)
int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// Scratch memory of magi_attn_fwd_static_scratch: the two words of the measured score bound (and room to spare).  One
// copy per GPU, held until the process ends; every call on a GPU shares it.
constexpr int SCRATCH_BYTES = 256;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// Device address of `scratch` on the current device (in host code the array's name is a stand-in, not an address):
// asked once per device with that device current, then kept.
std::mutex g_scratch_mutex;
void* g_scratch_ptr[64] = {nullptr};
int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= 64) return fail(MAGI_ENOSYS, "device index %d beyond the 64 this library keeps scratch pointers for", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(MAGI_EHIP, "hipGetSymbolAddress(scratch) returned no address");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MAGI_OK;
}

int attn_fwd_impl(const magi_attn_args* p, void* stream, float* workspace);

}  // namespace

extern "C" {

int magi_version(void) { return 103; }

uint64_t magi_launch_count(void) { return g_launches.load(std::memory_order_relaxed); }

const char* magi_last_error(void) { return g_err; }

int magi_attn_fwd(const magi_attn_args* p, void* stream) {
  if (!p) return fail(MAGI_EINVAL, "magi_attn_fwd: args is NULL");
  MAGI_CHECK_LAYOUT("magi_attn_fwd", p);
  return attn_fwd_impl(p, stream, p->workspace);
}

int magi_attn_fwd_static_scratch(const magi_attn_args* p, void* stream) {
  if (!p) return fail(MAGI_EINVAL, "magi_attn_fwd_static_scratch: args is NULL");
  MAGI_CHECK_LAYOUT("magi_attn_fwd_static_scratch", p);
  static_assert(4 * sizeof(float) <= SCRATCH_BYTES, "the measured score bound needs four words");
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != MAGI_OK) return rc;
  return attn_fwd_impl(p, stream, static_cast<float*>(ws));
}

}  // extern "C"

namespace {

int attn_fwd_impl(const magi_attn_args* p, void* stream, float* workspace) {
  if (p->D != 128) return fail(MAGI_ENOSYS, "magi_attn_fwd: head_dim %d not implemented (128 only)", p->D);
  if (p->dtype != MAGI_DTYPE_BF16 && p->dtype != MAGI_DTYPE_FP8_E4M3)
    return fail(MAGI_EINVAL, "magi_attn_fwd: unknown dtype %d", p->dtype);
  if (p->Hq <= 0 || p->Hkv <= 0 || p->Hq % p->Hkv != 0)
    return fail(MAGI_EINVAL, "magi_attn_fwd: Hq=%d must be a positive multiple of Hkv=%d", p->Hq, p->Hkv);
  if (p->total_q < 0 || p->total_k < 0 || p->n_ranges < 0 || p->max_seqlen_q < 0)
    return fail(MAGI_EINVAL, "magi_attn_fwd: negative size");
  if (p->ranges_mode != MAGI_RANGES_PAIRS && p->ranges_mode != MAGI_RANGES_CU)
    return fail(MAGI_EINVAL, "magi_attn_fwd: unknown ranges_mode %d", p->ranges_mode);
  if (p->n_ranges == 0 || p->total_q == 0 || p->max_seqlen_q == 0) return MAGI_OK;
  if (!p->q || !p->out || !p->q_ranges || !p->k_ranges) return fail(MAGI_EINVAL, "magi_attn_fwd: NULL q/out/ranges");
  const bool all_in_second = p->k2 && p->v2 && p->k_split == 0;  // an empty first segment may be NULL
  if (p->total_k > 0 && (!p->k || !p->v) && !all_in_second)
    return fail(MAGI_EINVAL, "magi_attn_fwd: NULL k/v with total_k > 0");
  const int esz = p->dtype == MAGI_DTYPE_BF16 ? 2 : 1;
  const int64_t row_elems = 16 / esz;  // 16-byte vectors
  if (p->q_stride_h % row_elems || p->q_stride_t % row_elems || p->k_stride_h % row_elems ||
      p->k_stride_t % row_elems || p->v_stride_h % row_elems || p->v_stride_t % row_elems || p->o_stride_h % 8 ||
      p->o_stride_t % 8)
    return fail(MAGI_EINVAL, "magi_attn_fwd: strides must keep rows 16-byte aligned");
  if (!aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->out) || !aligned16(p->k2) ||
      !aligned16(p->v2))
    return fail(MAGI_EINVAL, "magi_attn_fwd: q/k/v/out must be 16-byte aligned");
  if (p->q_stride_h < p->D || p->k_stride_h < p->D || p->v_stride_h < p->D || p->o_stride_h < p->D)
    return fail(MAGI_EINVAL, "magi_attn_fwd: head stride smaller than head_dim");
  if (p->q_stride_t < p->D || p->k_stride_t < p->D || p->v_stride_t < p->D || p->o_stride_t < p->D)
    return fail(MAGI_EINVAL, "magi_attn_fwd: token stride smaller than head_dim (rows may not overlap or run backwards)");
  // (the kernels address a 64-key tile with 32-bit byte offsets from its first row)
  if (p->k_stride_t > (1 << 23) || p->v_stride_t > (1 << 23))
    return fail(MAGI_ENOSYS, "magi_attn_fwd: k / v token strides above 2^23 elements are not implemented");
  if (p->dtype == MAGI_DTYPE_FP8_E4M3 && (p->flags & MAGI_ATTN_Q_PRESCALED))
    return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_Q_PRESCALED is a bf16 flag (fp8: MAGI_ATTN_FP8_POW2_PRESCALED)");
  if ((p->flags & MAGI_ATTN_FP8_FAST_EXP2) && !(p->dtype == MAGI_DTYPE_FP8_E4M3 && (p->flags & MAGI_ATTN_FP8_POW2_PRESCALED)))
    return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_FP8_FAST_EXP2 goes with fp8 and MAGI_ATTN_FP8_POW2_PRESCALED");
  if (p->dtype == MAGI_DTYPE_BF16 && (p->flags & MAGI_ATTN_FP8_POW2_PRESCALED))
    return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_FP8_POW2_PRESCALED is an fp8 flag");
  if (!(p->score_bound >= 0.f)) return fail(MAGI_EINVAL, "magi_attn_fwd: score_bound must be >= 0");
  const bool q_norm = p->q_norm_gamma != nullptr;
  if (q_norm) {
    if (p->dtype != MAGI_DTYPE_BF16 || (p->flags & MAGI_ATTN_Q_PRESCALED))
      return fail(MAGI_EINVAL, "magi_attn_fwd: q_norm takes raw bf16 q (no MAGI_ATTN_Q_PRESCALED)");
    if (!(p->score_bound > 0.f && p->score_bound <= MAGI_SCORE_BOUND_MAX))
      return fail(MAGI_ENOSYS, "magi_attn_fwd: q_norm is implemented for bounded scores (0 < score_bound <= %g)",
                  (double)MAGI_SCORE_BOUND_MAX);
    if (p->q_norm_kind != MAGI_NORM_LAYERNORM_1P && p->q_norm_kind != MAGI_NORM_RMSNORM_1P)
      return fail(MAGI_EINVAL, "magi_attn_fwd: q_norm_kind %d", p->q_norm_kind);
    if (!(p->q_norm_eps >= 0.f)) return fail(MAGI_EINVAL, "magi_attn_fwd: q_norm_eps");
    if (!aligned16(p->q_norm_gamma) || !aligned16(p->q_norm_beta))
      return fail(MAGI_EINVAL, "magi_attn_fwd: q_norm parameters must be 16-byte aligned");
  }
  if (p->score_bound > 0.f && p->dtype != MAGI_DTYPE_BF16)
    return fail(MAGI_EINVAL, "magi_attn_fwd: score_bound is a promise about bf16 inputs");
  const bool auto_bound = (p->flags & MAGI_ATTN_AUTO_BOUND) != 0;
  if (auto_bound) {
    if (p->dtype != MAGI_DTYPE_BF16 || p->score_bound > 0.f || q_norm || p->q_tile_rows != 0 ||
        (p->flags & MAGI_ATTN_BOUNDED_MFMA32))
      return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_AUTO_BOUND goes with bf16 and without score_bound, q_norm, "
                               "q_tile_rows and MAGI_ATTN_BOUNDED_MFMA32 (it measures the bound and picks the kernel itself)");
    if (!workspace || !aligned16(workspace))
      return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_AUTO_BOUND needs a 16-byte workspace on the device, 16-byte aligned");
  }
  if (p->out_group_heads < 0 || (p->out_group_heads > 0 && (p->Hq % p->out_group_heads || p->o_stride_g % 8)))
    return fail(MAGI_EINVAL, "magi_attn_fwd: out_group_heads must divide Hq and o_stride_g keep rows 16-byte aligned");
  int k_split = p->total_k;
  if (p->k2 || p->v2) {
    if (!p->k2 || !p->v2) return fail(MAGI_EINVAL, "magi_attn_fwd: k2 and v2 must be given together");
    if (p->k_split < 0 || p->k_split > p->total_k)
      return fail(MAGI_EINVAL, "magi_attn_fwd: k_split %d outside [0, total_k=%d]", p->k_split, p->total_k);
    k_split = p->k_split;
  }
  if (p->dtype == MAGI_DTYPE_FP8_E4M3) {
    if (!p->q_scale || !p->k_scale || !p->v_scale || p->scale_chunk_tokens <= 0)
      return fail(MAGI_EINVAL, "magi_attn_fwd: fp8 needs q/k/v scales and scale_chunk_tokens > 0");
    if ((p->k2_scale != nullptr) != (p->v2_scale != nullptr))
      return fail(MAGI_EINVAL, "magi_attn_fwd: k2_scale and v2_scale come together");
    if (p->k2_scale && (!p->k2 || p->k_split % p->scale_chunk_tokens))
      return fail(MAGI_EINVAL, "magi_attn_fwd: k2_scale / v2_scale need k2 / v2 and k_split on a scale-chunk boundary");
  }

  magi::AttnKernArgs a;
  std::memset(&a, 0, sizeof(a));
  a.q = static_cast<const char*>(p->q);
  a.k = static_cast<const char*>(p->k);
  a.v = static_cast<const char*>(p->v);
  a.k2 = static_cast<const char*>(p->k2);
  a.v2 = static_cast<const char*>(p->v2);
  a.out = static_cast<char*>(p->out);
  a.lse = p->lse;
  a.q_ranges = p->q_ranges;
  a.k_ranges = p->k_ranges;
  a.q_norm_gamma = p->q_norm_gamma;
  a.q_norm_beta = p->q_norm_beta;
  a.q_norm_eps = p->q_norm_eps;
  a.q_norm_kind = p->q_norm_kind;
  a.q_scale = p->q_scale;
  a.k_scale = p->k_scale;
  a.v_scale = p->v_scale;
  a.qs_t = p->q_stride_t * esz;
  a.qs_h = p->q_stride_h * esz;
  a.ks_t = p->k_stride_t * esz;
  a.ks_h = p->k_stride_h * esz;
  a.vs_t = p->v_stride_t * esz;
  a.vs_h = p->v_stride_h * esz;
  a.os_t = p->o_stride_t * 2;
  a.os_h = p->o_stride_h * 2;
  a.os_g = p->o_stride_g * 2;
  a.out_group = p->out_group_heads;
  a.total_q = p->total_q;
  a.total_k = p->total_k;
  a.k_split = k_split;
  a.n_ranges = p->n_ranges;
  a.ranges_mode = p->ranges_mode;
  // Kernel choice for bf16.
  //  * Scores with a promised bound (score_bound): the kernels without a running maximum that hold 64 query rows per
  //    wavefront; 256-row workgroups (4 waves, two per CU: the two waves of a SIMD belong to different workgroups
  //    and drift out of step, so one computes scores while the other is in its softmax) on v_mfma_f32_16x16x32
  //    (the part is power limited and that shape takes less energy per FLOP; measured +3 % on the 720p layer,
  //    between 0 and +6 % from box to box); the 32x32x16 form on request and for 512-row workgroups.
  //  * Otherwise 32 rows per wavefront with the online softmax: 384-row workgroups (12 waves, one workgroup per CU,
  //    every K / V tile fetched once for three times as many rows and one barrier per tile) pay on grids of many
  //    rounds with long key ranges (measured: +3 % at 43 rounds, +1 % at 9.4, -3 % at 5.3); small grids and short
  //    key ranges (cross attention) keep 128 rows (4 waves, three workgroups per CU).
  if (p->dtype == MAGI_DTYPE_FP8_E4M3 && p->q_tile_rows != 0 && p->q_tile_rows != 128)
    return fail(MAGI_EINVAL, "magi_attn_fwd: q_tile_rows %d (fp8: 128)", p->q_tile_rows);
  const bool promised = p->dtype == MAGI_DTYPE_BF16 && p->score_bound > 0.f && p->score_bound <= MAGI_SCORE_BOUND_MAX;
  const bool mfma32 = (p->flags & MAGI_ATTN_BOUNDED_MFMA32) != 0;
  if (mfma32 && !(promised && (p->flags & MAGI_ATTN_Q_PRESCALED)))
    return fail(MAGI_EINVAL, "magi_attn_fwd: MAGI_ATTN_BOUNDED_MFMA32 goes with bf16, MAGI_ATTN_Q_PRESCALED and a score_bound in force");
  a.Hq = p->Hq;
  a.Hkv = p->Hkv;
  a.G = p->Hq / p->Hkv;
  a.scale_chunk_tokens = p->scale_chunk_tokens;
  a.scale_split_chunk = 0x7fffffff;
  if (p->dtype == MAGI_DTYPE_FP8_E4M3 && p->k2_scale) {
    a.scale_split_chunk = p->k_split / p->scale_chunk_tokens;
    a.k2_scale_delta = (p->k2_scale - p->k_scale) - (long)a.scale_split_chunk * p->Hkv;
    a.v2_scale_delta = (p->v2_scale - p->v_scale) - (long)a.scale_split_chunk * p->Hkv;
  }
  const float scale = p->softmax_scale > 0.f ? p->softmax_scale : 1.0f / std::sqrt((float)p->D);
  a.scale_log2 = scale * 1.4426950408889634f;
  if (p->dtype == MAGI_DTYPE_BF16 && (p->flags & MAGI_ATTN_Q_PRESCALED)) a.scale_log2 = 1.f;  // q . k is the exp2 exponent
  // (with q_norm, or a score bound on unscaled q, the kernel multiplies q by scale_log2 itself while loading it, after
  // which the same holds)

  // One launch of `a` as the bounded-score kernel (bounded) or as the kernel without a promise about the scores.
  auto launch = [&](bool bounded) -> int {
    // a bound stated for unscaled q (what the reference's callers pass): the kernel applies the softmax scale while
    // it loads q, after which the scores are exp2 exponents as with MAGI_ATTN_Q_PRESCALED
    const bool scale_q = bounded && !q_norm && !(p->flags & MAGI_ATTN_Q_PRESCALED);
    a.block_m = 128;
    if (p->dtype == MAGI_DTYPE_BF16) {
      const double wg384 = (double)p->Hq * p->n_ranges * ((p->max_seqlen_q + 383) / 384);
      const bool long_keys = p->max_seqlen_k == 0 || p->max_seqlen_k >= 4096;  // (0 = not stated)
      if (bounded)
        a.block_m = 256;  // (512-row workgroups fetch half the tiles and measure 1 % slower: their two waves per SIMD march in step)
      else if (wg384 >= 9.0 * compute_units() && long_keys)
        a.block_m = 384;
      if (p->q_tile_rows != 0) {
        const int r = p->q_tile_rows;
        if ((q_norm || scale_q) && r != 256)
          return fail(MAGI_EINVAL, "magi_attn_fwd: q_tile_rows %d (with q_norm, or a score bound on unscaled q: 256)", r);
        if (bounded ? (r != 256 && r != 512) : (r != 128 && r != 384))
          return fail(MAGI_EINVAL, "magi_attn_fwd: q_tile_rows %d (bf16: 128 or 384; with a score bound: 256 or 512)", r);
        a.block_m = r;
      }
    }
    a.tiles_per_range = (p->max_seqlen_q + a.block_m - 1) / a.block_m;
    a.flags = p->flags | (bounded ? magi::ATTN_BOUNDED : 0) | (scale_q ? magi::ATTN_SCALE_Q : 0);
    const double total = (double)p->Hq * p->n_ranges * a.tiles_per_range;
    if (total > 2.0e9) return fail(MAGI_EINVAL, "magi_attn_fwd: grid too large (%.3g workgroups)", total);
    a.total_wgs = (unsigned)total;
    a.per_xcd = (a.total_wgs + 7u) / 8u;
    hipError_t e;
    if (p->dtype != MAGI_DTYPE_BF16)
      e = magi::launch_attn_fwd_fp8(a, static_cast<hipStream_t>(stream));
    else if (bounded && a.block_m == 256 && !mfma32)
      e = magi::launch_attn_fwd_bf16_x16(a, static_cast<hipStream_t>(stream));
    else if (bounded)
      e = magi::launch_attn_fwd_bf16_w64(a, static_cast<hipStream_t>(stream));
    else
      e = magi::launch_attn_fwd_bf16(a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "magi_attn_fwd launch");
    g_launches.fetch_add(1, std::memory_order_relaxed);
    return MAGI_OK;
  };

  if (!auto_bound) return launch(promised);

  // No promise about the scores: measure one.  Two streaming passes leave the largest squared length of a q row and
  // of a k row in the workspace (|q . k| <= |q| |k|); both attention kernels are launched behind them, each tests
  // the bound on the device and only the one it selects runs (the other returns at once).  No host synchronisation.
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned* ws = reinterpret_cast<unsigned*>(workspace);
  hipError_t e = magi::launch_gate_init(ws, st);
  if (e == hipSuccess) e = magi::launch_row_norm_max(a.q, a.qs_t, a.qs_h, p->total_q, p->Hq, ws, st);
  if (e == hipSuccess && k_split > 0) e = magi::launch_row_norm_max(a.k, a.ks_t, a.ks_h, k_split, p->Hkv, ws + 1, st);
  if (e == hipSuccess && p->total_k > k_split)
    e = magi::launch_row_norm_max(a.k2, a.ks_t, a.ks_h, p->total_k - k_split, p->Hkv, ws + 1, st);
  if (e != hipSuccess) return hip_fail(e, "magi_attn_fwd bound measurement");
  g_launches.fetch_add(2 + (k_split > 0) + (p->total_k > k_split), std::memory_order_relaxed);
  a.gate = workspace;
  a.gate_want = 1;
  int rc = launch(true);
  if (rc != MAGI_OK) return rc;
  a.gate_want = 0;
  return launch(false);
}

}  // namespace

extern "C" {

int magi_qk_prologue(const magi_prologue_args* p, void* stream) {
  if (!p) return fail(MAGI_EINVAL, "magi_qk_prologue: args is NULL");
  MAGI_CHECK_LAYOUT("magi_qk_prologue", p);
  if (p->D != 128) return fail(MAGI_ENOSYS, "magi_qk_prologue: head_dim %d not implemented (128 only)", p->D);
  if (p->S < 0 || p->Hq < 0 || p->Hkv < 0) return fail(MAGI_EINVAL, "magi_qk_prologue: negative size");
  if (p->S == 0 || p->Hq + p->Hkv == 0) return MAGI_OK;
  if (p->R2 < 0 || p->R2 % 8 || 2 * p->R2 > p->D)
    return fail(MAGI_EINVAL, "magi_qk_prologue: R2=%d must be a multiple of 8 with 2*R2 <= D", p->R2);
  if (p->norm_kind < 0 || p->norm_kind > 2) return fail(MAGI_EINVAL, "magi_qk_prologue: norm_kind %d", p->norm_kind);
  if (p->batch < 0) return fail(MAGI_EINVAL, "magi_qk_prologue: negative batch");
  if (p->Hq > 0 && (!p->q_raw || !p->q_out)) return fail(MAGI_EINVAL, "magi_qk_prologue: NULL q_raw/q_out");
  const bool out8 = p->out_dtype == MAGI_DTYPE_FP8_E4M3;
  if (p->out_dtype != MAGI_DTYPE_BF16 && !out8) return fail(MAGI_EINVAL, "magi_qk_prologue: out_dtype %d", p->out_dtype);
  if (p->Hkv > 0 && (!p->k_raw || (!p->v_raw && !out8))) return fail(MAGI_EINVAL, "magi_qk_prologue: NULL k_raw/v_raw");
  if (out8 && ((p->Hq > 0 && !(p->q_quant_scale > 0.f && std::isfinite(p->q_quant_scale))) ||
               (p->Hkv > 0 && !(p->k_quant_scale > 0.f && std::isfinite(p->k_quant_scale)))))
    return fail(MAGI_EINVAL, "magi_qk_prologue: e4m3 outputs need positive finite q_quant_scale / k_quant_scale");
  if (p->n_cache_rows < 0 || p->n_cache_rows > p->S)
    return fail(MAGI_EINVAL, "magi_qk_prologue: n_cache_rows %d outside [0, S=%d]", p->n_cache_rows, p->S);
  if (p->Hkv > 0 && p->n_cache_rows > 0 && !p->kv_out) return fail(MAGI_EINVAL, "magi_qk_prologue: NULL kv_out");
  if (p->Hkv > 0 && p->n_cache_rows < p->S && !p->kv_tail)
    return fail(MAGI_EINVAL, "magi_qk_prologue: kv_tail needed for rows >= n_cache_rows");
  if (p->norm_kind != MAGI_NORM_NONE && ((p->Hq > 0 && !p->gq) || (p->Hkv > 0 && !p->gk)))
    return fail(MAGI_EINVAL, "magi_qk_prologue: NULL gamma");
  if (p->R2 > 0 && p->rope && (reinterpret_cast<uintptr_t>(p->rope) & 15u))
    return fail(MAGI_EINVAL, "magi_qk_prologue: rope must be 16-byte aligned");
  if (p->q_raw_stride_t % 8 || p->k_raw_stride_t % 8 || p->v_raw_stride_t % 8 || p->kv_stride_t % 8 ||
      p->kv_tail_stride_t % 8)
    return fail(MAGI_EINVAL, "magi_qk_prologue: strides must keep rows 16-byte aligned");
  if (!aligned16(p->q_raw) || !aligned16(p->k_raw) || (!out8 && !aligned16(p->v_raw)) || !aligned16(p->q_out) ||
      !aligned16(p->kv_out) || !aligned16(p->kv_tail))
    return fail(MAGI_EINVAL, "magi_qk_prologue: buffers must be 16-byte aligned");

  magi::PrologueKernArgs a;
  std::memset(&a, 0, sizeof(a));
  a.q_raw = static_cast<const char*>(p->q_raw);
  a.k_raw = static_cast<const char*>(p->k_raw);
  a.v_raw = static_cast<const char*>(p->v_raw);
  a.rope = p->R2 > 0 ? p->rope : nullptr;
  a.gq = p->gq;
  a.bq = p->bq;
  a.gk = p->gk;
  a.bk = p->bk;
  a.q_out = static_cast<char*>(p->q_out);
  a.kv_out = static_cast<char*>(p->kv_out);
  a.kv_tail = static_cast<char*>(p->kv_tail);
  a.q_raw_stride_t = p->q_raw_stride_t * 2;
  a.k_raw_stride_t = p->k_raw_stride_t * 2;
  a.v_raw_stride_t = p->v_raw_stride_t * 2;
  a.kv_stride_t = p->kv_stride_t * (out8 ? 1 : 2);
  a.kv_tail_stride_t = p->kv_tail_stride_t * (out8 ? 1 : 2);
  a.out_fp8 = out8;
  a.q_inv_scale = out8 && p->Hq > 0 ? 1.f / p->q_quant_scale : 1.f;
  a.k_inv_scale = out8 && p->Hkv > 0 ? 1.f / p->k_quant_scale : 1.f;
  a.S = p->S;
  a.n_cache_rows = p->n_cache_rows;
  a.Hq = p->Hq;
  a.Hkv = p->Hkv;
  a.R2 = a.rope ? p->R2 : 0;
  a.norm_kind = p->norm_kind;
  a.eps = p->eps;
  a.batch = p->batch > 1 ? p->batch : 1;
  if (!(p->q_premul == p->q_premul) || std::fabs(p->q_premul) > 1e30f)
    return fail(MAGI_EINVAL, "magi_qk_prologue: q_premul is not finite");
  a.q_premul = p->q_premul == 0.f ? 1.f : p->q_premul;
  hipError_t e = magi::launch_prologue(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_qk_prologue launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_qkv_proj_prologue(const magi_qkv_proj_args* p, void* stream) {
  if (!p) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: args is NULL");
  MAGI_CHECK_LAYOUT("magi_qkv_proj_prologue", p);
  if (p->D != 128) return fail(MAGI_ENOSYS, "magi_qkv_proj_prologue: head_dim %d not implemented (128 only)", p->D);
  if (p->S < 0 || p->K <= 0 || p->Hq < 0 || p->Hkv < 0 || p->Hqx < 0)
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: bad size");
  const int heads = p->Hq + 2 * p->Hkv + p->Hqx;
  if (p->S == 0 || heads == 0) return MAGI_OK;
  if (p->K % 64) return fail(MAGI_ENOSYS, "magi_qkv_proj_prologue: K=%d is not a multiple of 64", p->K);
  if (heads % 2) return fail(MAGI_ENOSYS, "magi_qkv_proj_prologue: an odd number of heads (%d) is not implemented", heads);
  if (p->rope && p->R2 != 48 && p->R2 != 0)
    return fail(MAGI_ENOSYS, "magi_qkv_proj_prologue: R2=%d not implemented (48, or 0 / NULL rope for none)", p->R2);
  if (p->norm_kind < 0 || p->norm_kind > 2) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: norm_kind %d", p->norm_kind);
  if (p->batch < 0) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: negative batch");
  if (!p->x || !p->w) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: NULL x / w");
  if (p->x_stride < p->K || p->w_stride < p->K) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: row stride below K");
  if (p->Hq > 0 && !p->q_out) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: NULL q_out");
  if (p->Hqx > 0 && !p->qx_out) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: NULL qx_out");
  if (p->n_cache_rows < 0 || p->n_cache_rows > p->S)
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: n_cache_rows %d outside [0, S=%d]", p->n_cache_rows, p->S);
  if (p->Hkv > 0 && p->n_cache_rows > 0 && !p->kv_out) return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: NULL kv_out");
  if (p->Hkv > 0 && p->n_cache_rows < p->S && !p->kv_tail)
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: kv_tail needed for rows >= n_cache_rows");
  if (p->norm_kind != MAGI_NORM_NONE && ((p->Hq > 0 && !p->gq) || (p->Hkv > 0 && !p->gk)))
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: NULL gamma");
  if (p->x_stride % 8 || p->w_stride % 8 || p->kv_stride_t % 8 || p->kv_tail_stride_t % 8)
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: strides must keep rows 16-byte aligned");
  if (!aligned16(p->x) || !aligned16(p->w) || !aligned16(p->q_out) || !aligned16(p->kv_out) || !aligned16(p->kv_tail) ||
      !aligned16(p->qx_out) || !aligned16(p->rope) || !aligned16(p->gq) || !aligned16(p->bq) || !aligned16(p->gk) ||
      !aligned16(p->bk))
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: buffers must be 16-byte aligned");
  // (the loader addresses a workgroup's 256 rows with 32-bit byte offsets)
  if (p->x_stride > (1 << 21) || p->w_stride > (1 << 21))
    return fail(MAGI_ENOSYS, "magi_qkv_proj_prologue: row strides above 2^21 elements are not implemented");
  if (!(p->q_premul == p->q_premul) || std::fabs(p->q_premul) > 1e30f)
    return fail(MAGI_EINVAL, "magi_qkv_proj_prologue: q_premul is not finite");
  magi::QkvGemmKernArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = static_cast<const char*>(p->x);
  a.w = static_cast<const char*>(p->w);
  a.rope = (p->rope && p->R2 == 48) ? p->rope : nullptr;
  a.gq = p->gq;
  a.bq = p->bq;
  a.gk = p->gk;
  a.bk = p->bk;
  a.q_out = static_cast<char*>(p->q_out);
  a.kv_out = static_cast<char*>(p->kv_out);
  a.kv_tail = static_cast<char*>(p->kv_tail);
  a.qx_out = static_cast<char*>(p->qx_out);
  a.x_stride = p->x_stride * 2;
  a.w_stride = p->w_stride * 2;
  a.kv_stride_t = p->kv_stride_t * 2;
  a.kv_tail_stride_t = p->kv_tail_stride_t * 2;
  a.S = p->S;
  a.K = p->K;
  a.n_cache_rows = p->n_cache_rows;
  a.Hq = p->Hq;
  a.Hkv = p->Hkv;
  a.Hqx = p->Hqx;
  a.norm_kind = p->norm_kind;
  a.eps = p->eps;
  a.batch = p->batch > 1 ? p->batch : 1;
  a.q_premul = p->q_premul == 0.f ? 1.f : p->q_premul;
  hipError_t e = magi::launch_qkv_gemm_prologue(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_qkv_proj_prologue launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_layer_norm(const void* x, int64_t x_stride, const void* weight, const void* bias, int32_t params_fp32,
                    void* y, int64_t y_stride, int64_t rows, int32_t cols, float eps, void* stream) {
  if (rows < 0 || cols < 0) return fail(MAGI_EINVAL, "magi_layer_norm: negative size");
  if (rows == 0 || cols == 0) return MAGI_OK;
  if (cols % 8 || cols > 8192)
    return fail(MAGI_ENOSYS, "magi_layer_norm: cols %d not implemented (multiples of 8 up to 8192)", cols);
  if (!x || !y) return fail(MAGI_EINVAL, "magi_layer_norm: NULL x/y");
  if (x_stride < cols || y_stride < cols) return fail(MAGI_EINVAL, "magi_layer_norm: row stride below cols");
  if (x_stride % 8 || y_stride % 8 || !aligned16(x) || !aligned16(y))
    return fail(MAGI_EINVAL, "magi_layer_norm: rows must be 16-byte aligned");
  if (!(eps >= 0.f)) return fail(MAGI_EINVAL, "magi_layer_norm: eps");
  if (rows > 0x7fffffffLL * 4) return fail(MAGI_ENOSYS, "magi_layer_norm: more than 2^33 rows");  // (4 rows per workgroup)
  hipError_t e = magi::launch_layer_norm(static_cast<const char*>(x), x_stride * 2, weight, bias, params_fp32 != 0,
                                         static_cast<char*>(y), y_stride * 2, rows, cols, eps,
                                         static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_layer_norm launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_div_clamp_to_e4m3(const void* x, int64_t x_stride, const float* scale, int32_t scale_len, void* y,
                           int64_t y_stride, int64_t rows, int32_t cols, void* stream) {
  if (rows < 0 || cols < 0) return fail(MAGI_EINVAL, "magi_div_clamp_to_e4m3: negative size");
  if (rows == 0 || cols == 0) return MAGI_OK;
  if (cols % 8) return fail(MAGI_ENOSYS, "magi_div_clamp_to_e4m3: cols %d is not a multiple of 8", cols);
  if (!x || !y || !scale) return fail(MAGI_EINVAL, "magi_div_clamp_to_e4m3: NULL pointer");
  if (scale_len != 1 && scale_len != cols)
    return fail(MAGI_EINVAL, "magi_div_clamp_to_e4m3: scale_len %d (1, or cols = %d)", scale_len, cols);
  if (x_stride < cols || y_stride < cols) return fail(MAGI_EINVAL, "magi_div_clamp_to_e4m3: row stride below cols");
  if (x_stride % 8 || y_stride % 8 || !aligned16(x) || (reinterpret_cast<uintptr_t>(y) & 7u) || !aligned16(scale))
    return fail(MAGI_EINVAL, "magi_div_clamp_to_e4m3: rows of x must be 16-byte aligned, rows of y 8-byte, scale 16-byte");
  if (rows * (int64_t)(cols / 8) > 0x7fffffffLL * 256)
    return fail(MAGI_ENOSYS, "magi_div_clamp_to_e4m3: more than 2^39 groups of eight elements");
  hipError_t e = magi::launch_div_clamp(static_cast<const char*>(x), x_stride * 2, scale, scale_len != 1,
                                        static_cast<char*>(y), y_stride, rows, cols, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_div_clamp_to_e4m3 launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_head_norm(const void* x, int64_t x_stride_t, int64_t x_stride_h, const float* gamma, const float* beta,
                   void* y, int32_t S, int32_t H, int32_t D, int32_t norm_kind, float eps, void* stream) {
  if (D != 128) return fail(MAGI_ENOSYS, "magi_head_norm: head_dim %d not implemented (128 only)", D);
  if (S < 0 || H < 0) return fail(MAGI_EINVAL, "magi_head_norm: negative size");
  if (S == 0 || H == 0) return MAGI_OK;
  if (!x || !y) return fail(MAGI_EINVAL, "magi_head_norm: NULL x/y");
  if (norm_kind < 0 || norm_kind > 2) return fail(MAGI_EINVAL, "magi_head_norm: norm_kind %d", norm_kind);
  if (norm_kind != MAGI_NORM_NONE && !gamma) return fail(MAGI_EINVAL, "magi_head_norm: NULL gamma");
  if (x_stride_t % 8 || x_stride_h % 8 || !aligned16(x) || !aligned16(y))
    return fail(MAGI_EINVAL, "magi_head_norm: rows must be 16-byte aligned");
  hipError_t e = magi::launch_head_norm(static_cast<const char*>(x), x_stride_t * 2, x_stride_h * 2, gamma, beta,
                                        static_cast<char*>(y), S, H, norm_kind, eps, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_head_norm launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_apply_rotary(const void* x, const float* cos, const float* sin, void* y, int32_t B, int32_t S, int32_t H,
                      int32_t D, int32_t R2, int32_t is_bf16, void* stream) {
  if (B < 0 || S < 0 || H < 0 || D <= 0 || D % 2) return fail(MAGI_EINVAL, "magi_apply_rotary: bad shape");
  if (R2 < 0 || 2 * R2 > D) return fail(MAGI_EINVAL, "magi_apply_rotary: rotary_dim %d > head_dim %d", 2 * R2, D);
  if ((long)B * S * H == 0) return MAGI_OK;
  if (!x || !y || (R2 > 0 && (!cos || !sin))) return fail(MAGI_EINVAL, "magi_apply_rotary: NULL pointer");
  hipError_t e = magi::launch_rotary(x, cos, sin, y, B, S, H, D, R2, is_bf16, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "magi_apply_rotary launch");
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return MAGI_OK;
}

static int quantize_impl(const magi_quantize_args* p, void* stream, bool always_one_launch) {
  if (!p) return fail(MAGI_EINVAL, "magi_quantize_fp8: args is NULL");
  MAGI_CHECK_LAYOUT("magi_quantize_fp8", p);
  if (p->D != 128) return fail(MAGI_ENOSYS, "magi_quantize_fp8: head_dim %d not implemented (128 only)", p->D);
  if (p->T < 0 || p->H < 0 || p->chunk_tokens <= 0) return fail(MAGI_EINVAL, "magi_quantize_fp8: bad size");
  if (!(p->premul == p->premul) || p->premul == 0.f)
    return fail(MAGI_EINVAL, "magi_quantize_fp8: premul must be finite and non-zero");
  if (p->n_rows_first < 0 || p->n_rows_first > p->T)
    return fail(MAGI_EINVAL, "magi_quantize_fp8: n_rows_first %d outside [0, T=%d]", p->n_rows_first, p->T);
  if (p->n_rows_first < p->T && p->n_rows_first % p->chunk_tokens)
    return fail(MAGI_EINVAL, "magi_quantize_fp8: n_rows_first must be a multiple of chunk_tokens");
  if (p->T == 0 || p->H == 0) return MAGI_OK;
  if (p->H > 65535) return fail(MAGI_ENOSYS, "magi_quantize_fp8: more than 65535 heads");
  if (!p->x) return fail(MAGI_EINVAL, "magi_quantize_fp8: NULL pointer");
  if (p->n_rows_first > 0 && (!p->y || !p->scales)) return fail(MAGI_EINVAL, "magi_quantize_fp8: NULL pointer");
  if (p->n_rows_first < p->T && (!p->y2 || !p->scales2))
    return fail(MAGI_EINVAL, "magi_quantize_fp8: y2 / scales2 needed for rows >= n_rows_first");
  if (p->x_stride_t % 8 || p->x_stride_h % 8 || !aligned16(p->x) || !aligned16(p->y) || !aligned16(p->y2))
    return fail(MAGI_EINVAL, "magi_quantize_fp8: rows must be 16-byte aligned");
  int n_launches = 0;
  hipError_t e = magi::launch_quantize_fp8(static_cast<const char*>(p->x), p->x_stride_t * 2, p->x_stride_h * 2,
                                           static_cast<char*>(p->y), p->scales, p->T, p->H, p->chunk_tokens, p->premul,
                                           p->pow2_scales, p->n_rows_first, static_cast<char*>(p->y2), p->scales2,
                                           always_one_launch, compute_units(), static_cast<hipStream_t>(stream), &n_launches);
  if (e != hipSuccess) return hip_fail(e, "magi_quantize_fp8 launch");
  g_launches.fetch_add((uint64_t)n_launches, std::memory_order_relaxed);
  return MAGI_OK;
}

int magi_quantize_fp8_split(const magi_quantize_args* p, void* stream) { return quantize_impl(p, stream, true); }

int magi_quantize_fp8(const void* x, int64_t x_stride_t, int64_t x_stride_h, void* y, float* scales, int32_t T,
                      int32_t H, int32_t D, int32_t chunk_tokens, float premul, int32_t pow2_scales, void* stream) {
  magi_quantize_args q;
  std::memset(&q, 0, sizeof(q));
  q.struct_size = sizeof(q);
  q.x = x;
  q.x_stride_t = x_stride_t;
  q.x_stride_h = x_stride_h;
  q.T = T;
  q.H = H;
  q.D = D;
  q.chunk_tokens = chunk_tokens;
  q.premul = premul;
  q.pow2_scales = pow2_scales;
  q.y = y;
  q.scales = scales;
  q.n_rows_first = T;
  return quantize_impl(&q, stream, false);
}

}  // extern "C"
