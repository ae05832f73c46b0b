// Internal launch interface between the C-ABI layer (api.cpp) and the HIP kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace magi {

// Arguments of the range-attention forward kernels.  All strides are in BYTES.
struct AttnKernArgs {
  const char* q;
  const char* k;
  const char* v;
  const char* k2;
  const char* v2;
  char* out;
  float* lse;
  const int* q_ranges;
  const int* k_ranges;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  const float* q_norm_gamma;  // non-null: q is raw, normalise each (token, head) row while loading it
  const float* q_norm_beta;
  long qs_t, qs_h, ks_t, ks_h, vs_t, vs_h, os_t, os_h;
  // fp8, side segment with scale tables of its own: element offsets that lead from row c of k_scale / v_scale to
  // row c - scale_split_chunk of those tables (0 without them)
  long k2_scale_delta, v2_scale_delta;
  long os_g;     // byte stride between output head groups (out_group > 0)
  int out_group; // heads per output group, 0 = heads addressed by os_h alone
  int total_q, total_k, k_split;
  int n_ranges, ranges_mode, tiles_per_range;
  int block_m;  // q rows per workgroup (the launchers map it to an instantiation)
  int Hq, Hkv, G;
  int scale_chunk_tokens;
  int scale_split_chunk;  // first chunk served by the side segment's scale tables (INT_MAX without them)
  int flags;  // MAGI_ATTN_* bits of the public header, plus ATTN_BOUNDED / ATTN_SCALE_Q
  unsigned total_wgs, per_xcd;
  float scale_log2;  // softmax_scale * log2(e)
  float q_norm_eps;
  int q_norm_kind;  // MAGI_NORM_LAYERNORM_1P / MAGI_NORM_RMSNORM_1P
  // Measured score bound (MAGI_ATTN_AUTO_BOUND): gate[0] / gate[1] = the largest squared length of a q row / a k row
  // as launch_row_norm_max left them.  A kernel that is handed a gate first tests whether
  // sqrt(gate[0] gate[1]) * scale_log2 * 1.01 <= MAGI_SCORE_BOUND_MAX and runs only if the answer equals
  // gate_want (the bounded-score kernel: 1, the online-softmax kernel launched behind it: 0).  NULL: no test.
  const float* gate;
  int gate_want;
};


// internal flag: the caller promised bounded scores (magi_attn_args.score_bound within MAGI_SCORE_BOUND_MAX)
constexpr int ATTN_BOUNDED = 1 << 8;
// internal flag (with ATTN_BOUNDED): q is unscaled, the kernel multiplies it by scale_log2 while loading it
constexpr int ATTN_SCALE_Q = 1 << 9;

hipError_t launch_attn_fwd_bf16(const AttnKernArgs& a, hipStream_t stream);
hipError_t launch_attn_fwd_bf16_w64(const AttnKernArgs& a, hipStream_t stream);
hipError_t launch_attn_fwd_bf16_x16(const AttnKernArgs& a, hipStream_t stream);
hipError_t launch_attn_fwd_fp8(const AttnKernArgs& a, hipStream_t stream);
// ws[0..3] = 0 (a kernel, not a memset: the call may be under graph capture)
hipError_t launch_gate_init(unsigned* ws, hipStream_t stream);
// *out_bits = max(*out_bits, bit pattern of the largest sum of squares over a [T, H, 128] bf16 tensor's rows);
// strides in BYTES.  Bit patterns of non-negative floats order like the floats, and a NaN row ends up on top.
hipError_t launch_row_norm_max(const char* x, long stride_t, long stride_h, int T, int H, unsigned* out_bits,
                               hipStream_t stream);

struct PrologueKernArgs {
  const char* q_raw;
  const char* k_raw;
  const char* v_raw;
  const float* rope;
  const float* gq;
  const float* bq;
  const float* gk;
  const float* bk;
  char* q_out;
  char* kv_out;
  char* kv_tail;
  long q_raw_stride_t, k_raw_stride_t, v_raw_stride_t;  // bytes
  long kv_stride_t, kv_tail_stride_t;                   // bytes
  int S, n_cache_rows;
  int Hq, Hkv, R2;
  int norm_kind;
  float eps;
  int batch;
  float q_premul;  // factor on q before the bf16 rounding (1 = none)
  int out_fp8;     // q and k leave as e4m3 (kv_out / kv_tail then hold K rows only, strides in bytes); v untouched
  float q_inv_scale, k_inv_scale;  // out_fp8: 1 / the constant scale of q (after q_premul) and of k
};
hipError_t launch_prologue(const PrologueKernArgs& a, hipStream_t stream);

// The four projections as one GEMM with the prologue as its epilogue.  Strides in BYTES.
struct QkvGemmKernArgs {
  const char* x;  // [S, K] bf16
  const char* w;  // [(Hq + 2 Hkv + Hqx) * 128, K] bf16, rows ordered q | k | v | qx heads
  const float* rope;
  const float* gq;
  const float* bq;
  const float* gk;
  const float* bk;
  char* q_out;
  char* kv_out;
  char* kv_tail;
  char* qx_out;
  long x_stride, w_stride;
  long kv_stride_t, kv_tail_stride_t;
  int S, K, n_cache_rows;
  int Hq, Hkv, Hqx;
  int norm_kind;
  float eps;
  int batch;
  float q_premul;
  int n_row_tiles, n_col_tiles;  // filled by the launcher
};
hipError_t launch_qkv_gemm_prologue(const QkvGemmKernArgs& a, hipStream_t stream);

hipError_t launch_head_norm(const char* x, long x_stride_t, long x_stride_h, const float* gamma, const float* beta,
                            char* y, int S, int H, int norm_kind, float eps, hipStream_t stream);
hipError_t launch_layer_norm(const char* x, long x_stride, const void* w, const void* b, int params_fp32, char* y,
                             long y_stride, long rows, int cols, float eps, hipStream_t stream);
// y = e4m3(bf16(clamp(x / scale, +-448))): x [rows, cols] bf16, y [rows, cols] e4m3, strides in BYTES
hipError_t launch_div_clamp(const char* x, long x_stride, const float* scale, int per_column, char* y, long y_stride,
                            long rows, int cols, hipStream_t stream);
hipError_t launch_rotary(const void* x, const float* cos, const float* sin, void* y, int B, int S, int H, int D,
                         int R2, int is_bf16, hipStream_t stream);
// Rows below n_first go to y / scales, the rest (row index and chunk index counted from n_first, a multiple of
// chunk_tokens) to y2 / scales2.  one_launch: always the single-launch kernel (else only where it is the faster).
// *n_launches receives the number of kernels launched.
hipError_t launch_quantize_fp8(const char* x, long x_stride_t, long x_stride_h, char* y, float* scales, int T, int H,
                               int chunk_tokens, float premul, int pow2_scales, int n_first, char* y2, float* scales2,
                               bool one_launch, int compute_units, hipStream_t stream, int* n_launches);

}  // namespace magi
