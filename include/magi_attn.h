/*
 * libmagi_attn: C-ABI for the MAGI-1 DiT attention hot path on MI355X (gfx950).
 *
 * Every function returns 0 on success or a negative MAGI_E* code and never throws or
 * aborts; magi_last_error() returns a thread-local message for the last failure.  The
 * caller owns every device buffer; except where a function says otherwise the library
 * allocates no device memory, performs no host synchronisation and launches on the
 * stream it is given (hipStream_t passed as void*; NULL = the default stream).
 *
 * The reference has no FFI of its own: it binds four Python callables from third-party
 * CUDA packages.  Each entry point below names the reference call site it stands in for
 * (paths relative to the reference checkout).
 */
#ifndef MAGI_ATTN_H
#define MAGI_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MAGI_OK 0
#define MAGI_EINVAL (-22)   /* bad argument (shape, stride, alignment, dtype) */
#define MAGI_ENOSYS (-38)   /* configuration not implemented (e.g. head_dim != 128) */
#define MAGI_EHIP (-5)      /* a HIP runtime call failed; see magi_last_error() */

/* element types of q / k / v */
#define MAGI_DTYPE_BF16 0
#define MAGI_DTYPE_FP8_E4M3 1 /* OCP e4m3fn with per-(chunk, head) fp32 scales */

/* how q_ranges / k_ranges are encoded */
/* magi_attn_args.flags.  FP8_POW2_PRESCALED: every q/k/v scale is an exact power of two and q was multiplied by
 * softmax_scale * log2(e) before quantisation (magi_quantize_fp8 with pow2_scales = 1 and that premul).  The
 * scales then ride on the MFMA's block-scale operands and the kernel does no per-score multiply;
 * softmax_scale is ignored. */
#define MAGI_ATTN_FP8_POW2_PRESCALED 1
/* With FP8_POW2_PRESCALED: the probabilities are 2^floor(e) * (1 + frac(e)) instead of 2^e (e = the exp2 exponent
 * of a score relative to its row maximum), a piecewise-linear exp2 that costs one full-rate vector instruction per
 * score instead of the quarter-rate exponential this kernel is otherwise bound by.  At most 6.2 % above 2^e; the
 * row sums are taken from the same values, so the average excess cancels in the normalisation and a relative
 * spread of 2 % per weight remains, to be compared with the 2.7 % r.m.s. of rounding the probabilities to e4m3,
 * which both variants do.  lse is biased by up to +0.06 (natural log units).  An opt-in approximation: the modes
 * WITHOUT this flag evaluate the exponential exactly in fp32 ("softmax in fp32" of the fp8 benchmark configuration)
 * and are what FullyParallelAttention(attention_dtype="fp8") runs by default. */
#define MAGI_ATTN_FP8_FAST_EXP2 4
/* bf16 path: q already carries softmax_scale * log2(e) (magi_qk_prologue with q_premul set to it multiplies before
 * its one rounding to bf16, so nothing is lost), i.e. the scores q.k are exp2 exponents.  The kernel then skips the
 * per-score multiply and, where it has an instantiation for it, lets the score MFMAs accumulate onto the negated
 * running maximum; softmax_scale is ignored.  No counterpart in the reference, whose kernels take unscaled q. */
#define MAGI_ATTN_Q_PRESCALED 2
/* bf16 with MAGI_ATTN_Q_PRESCALED and a score_bound in force: run the bounded-score kernel on v_mfma_f32_32x32x16
 * instead of the default 16x16x32.  Same results up to the order of fp32 additions.  The default shape spends less
 * energy per FLOP, which is what counts on a part at its board power limit (+3 % on the 720p layer, 0 to +6 % from box
 * to box); the 32x32x16 form issues half as many MFMAs and is the better one where the clock, not the power, is
 * capped.  512-row workgroups (q_tile_rows) always use it. */
#define MAGI_ATTN_BOUNDED_MFMA32 8
/* bf16 without a score_bound: measure one.  Two streaming passes over q and k (256 bytes per (token, head) row: 0.3 ms
 * at the 720p shape) leave the largest squared row length of each in `workspace`; |q . k| <= |q| |k| for every pair,
 * so the bounded-score kernel and the online-softmax kernel are both launched behind them, each tests
 * max|q| max|k| softmax_scale log2(e) * 1.01 <= MAGI_SCORE_BOUND_MAX on the device, and only the one the test selects
 * runs (the other returns at once).  Five launches, no host synchronisation, capturable.  This is what the reference's
 * call sites get without any change to them: they pass QK-normed q and k and no bound (dit_module.py:1032-1043), and
 * the measured bound selects the kernel without a running maximum (15 % faster on the 720p layer).  Rows of k between
 * 0 and total_k that no range names are measured too (a looser bound, still a bound); a NaN anywhere selects the
 * online-softmax kernel.  Not with score_bound, q_norm, q_tile_rows or MAGI_ATTN_BOUNDED_MFMA32. */
#define MAGI_ATTN_AUTO_BOUND 16

#define MAGI_RANGES_PAIRS 0 /* int32 [n, 2]: range i = [r[2i], r[2i+1])          */
#define MAGI_RANGES_CU 1    /* int32 [n + 1] cumulative: range i = [r[i], r[i+1]) */

/* QK-norm kinds of the prologue */
#define MAGI_NORM_LAYERNORM_1P 0 /* (x-mean)/sqrt(var+eps) * (gamma+1) + beta */
#define MAGI_NORM_RMSNORM_1P 1   /* x/sqrt(mean(x^2)+eps) * (gamma+1)          */
#define MAGI_NORM_NONE 2

/* 100 * major + minor.  The layout of the argument structs below belongs to the version; every struct also starts
 * with its own size as the caller compiled it (struct_size = sizeof(the struct)), and an entry point that is handed
 * another size returns MAGI_EINVAL instead of reading fields the caller never wrote. */
int magi_version(void);
const char* magi_last_error(void);
/* Diagnostics: the number of kernel launches the library has issued in this process so far (all threads, all
 * entry points).  A caller can difference it around a piece of work to see how many launches that work costs. */
uint64_t magi_launch_count(void);

/*
 * Range attention forward (bf16 or fp8-e4m3 inputs, fp32 softmax, bf16 output).
 *
 *   for each i < n_ranges:
 *     out[q_range_i, h, :] = softmax(q[q_range_i, h] . k[k_range_i, h / (Hq/Hkv)]^T * scale) v[k_range_i, h / (Hq/Hkv)]
 *
 * with no mask inside a rectangle.  q ranges must be disjoint; rows of `out` that no range
 * covers are left untouched; a range with no keys writes zeros (and lse = -inf).
 *
 * Stands in for
 *   flex_flash_attn_func(q, k, v, q_ranges, k_ranges, max_seqlen_q, max_seqlen_k, softmax_scale, ...)
 *       inference/model/dit/dit_module.py:1032-1043, 1074-1085, 1111-1122
 *   flash_attn_func(q, k, v)                 inference/model/dit/dit_module.py:1062, 1090-1095  (one range)
 *   flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, ...)   dit_module.py:1124-1133 (MAGI_RANGES_CU)
 *
 * q   [total_q, Hq, D]   element strides q_stride_t (token), q_stride_h (head); D contiguous
 * k,v [total_k, Hkv, D]  element strides k_stride_t/h and v_stride_t/h.  K and V may alias one
 *                        interleaved KV-cache allocation [T, Hkv, 2D] (k = cache, v = cache + D):
 *                        the cache is read in place, which removes the prefix slice / cat /
 *                        contiguous copies of dit_module.py:915, 931, 945-946, 1027-1029.
 * k2,v2                  optional second segment (NULL to disable): key rows >= k_split are read
 *                        from k2/v2 at row (index - k_split) with the same strides.  This is how
 *                        "attend to the new KV without persisting it" (update_kv_cache == False,
 *                        dit_module.py:918-931) works without a copy.
 * out [total_q, Hq, D]   bf16, strides o_stride_t / o_stride_h
 * out_group_heads, o_stride_g   optional two-level head addressing of `out` (0 = off): head h is written at
 *                        (h / out_group_heads) * o_stride_g + (h % out_group_heads) * o_stride_h.  With 8 groups
 *                        the core and the cross attention write straight into the "(hn n hd)" buffer that
 *                        linear_proj consumes, which removes the concat + rearrange of attn_linear_proj
 *                        (inference/model/dit/dit_module.py:1332-1340).
 * lse                    optional fp32 [Hq, total_q] (NULL to skip): log sum exp of the scaled scores (natural log).
 *                        bf16 kernels sum the fp32 probabilities (within 1e-3 of the fp32 value; the bounded-score
 *                        kernel within 1e-5).  The fp8 kernel takes its row sums on the matrix pipe from the
 *                        probabilities AFTER their rounding to e4m3 (what the P V product uses): lse is within
 *                        2e-2 of the fp32 value in the exact-exponential modes, and up to 0.06 high with
 *                        MAGI_ATTN_FP8_FAST_EXP2.
 * q_ranges, k_ranges     DEVICE int32 arrays, encoding per ranges_mode; clamped to
 *                        [0,total_q] / [0,total_k] in the kernel
 * max_seqlen_q           upper bound of any q range length (host int; sizes the grid: rows of a range beyond
 *                        max_seqlen_q are NOT computed and stay untouched, without an error, because the ranges
 *                        live on the device and the call does not synchronise to read them)
 * q_scale,k_scale,v_scale  fp8 only: DEVICE fp32 [n_scale_chunks, H] with the scale of token t
 *                        at [t / scale_chunk_tokens, h]; NULL for bf16
 * softmax_scale          <= 0 selects D^-0.5
 * score_bound            0 = unknown.  > 0 (bf16 only): the caller's promise that every score satisfies
 *                        |q . k| * softmax_scale * log2(e) <= score_bound, i.e. a bound on the exp2 exponents
 *                        (with MAGI_ATTN_Q_PRESCALED the factor is already in q and the bound is on |q . k| itself).
 *                        Up to MAGI_SCORE_BOUND_MAX the softmax is then evaluated as 2^score / sum 2^score without a
 *                        running maximum (it is shift invariant, and 2^score can neither overflow nor lose its
 *                        leading terms in fp32 at such bounds): the same result with a third fewer vector
 *                        instructions, and room for kernels that hold 64 query rows per wavefront.  Unscaled q (no
 *                        MAGI_ATTN_Q_PRESCALED, what the reference's call sites pass) is multiplied by the scale
 *                        while the kernel loads it and rounded to bf16 a second time (2^-9 relative per element,
 *                        like the rounding q already carries).  QK-normed attention knows the bound from its norm
 *                        parameters:
 *                        |q| |k| <= (sqrt(D) max|gamma_q + 1| + |beta_q|) (sqrt(D) max|gamma_k + 1| + |beta_k|),
 *                        times the scale factor.  Larger bounds fall back to the running maximum.  A promise
 *                        that does not hold gives inf / nan or wrong rows, not a fault.  No counterpart in the
 *                        reference.
 * q_norm_gamma, q_norm_beta, q_norm_eps, q_norm_kind
 *                        optional (gamma NULL = off): q holds the RAW query projection and the kernel applies the
 *                        per-(token, head) norm of magi_head_norm (gamma stored zero-centred, beta may be NULL,
 *                        kind MAGI_NORM_LAYERNORM_1P or MAGI_NORM_RMSNORM_1P) in fp32 while it loads q, multiplies
 *                        by softmax_scale * log2(e) and rounds to bf16 once.  Stands in for q_layernorm_xattn in
 *                        get_xqkv (dit_module.py:1008) without the normalised copy of q ever reaching memory.
 *                        Needs bf16 inputs and a score_bound (stated for the normalised, scaled q); do not set
 *                        MAGI_ATTN_Q_PRESCALED (the raw q is not scaled).
 * q_tile_rows            0 = the library picks the workgroup shape from the size of the launch.  Otherwise the
 *                        number of query rows per workgroup to use: 128 or 384 (bf16), 256 or 512 (bf16 with a
 *                        score_bound in force and pre-scaled q; 256 with q_norm or unscaled q), 128 (fp8); anything
 *                        else is MAGI_EINVAL.  Results do not depend on
 *                        it beyond the order of fp32 additions; it exists so that every shipped workgroup shape
 *                        can be exercised on small inputs.
 */
#define MAGI_SCORE_BOUND_MAX 64.0f
typedef struct magi_attn_args {
  uint32_t struct_size; /* sizeof(magi_attn_args) */
  const void* q;
  const void* k;
  const void* v;
  const void* k2;
  const void* v2;
  void* out;
  float* lse;
  const int32_t* q_ranges;
  const int32_t* k_ranges;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  int64_t q_stride_t, q_stride_h;
  int64_t k_stride_t, k_stride_h;
  int64_t v_stride_t, v_stride_h;
  int64_t o_stride_t, o_stride_h;
  int32_t total_q, total_k, k_split;
  int32_t n_ranges, ranges_mode;
  int32_t max_seqlen_q, max_seqlen_k;
  int32_t Hq, Hkv, D;
  int32_t dtype;
  int32_t scale_chunk_tokens;
  float softmax_scale;
  int32_t flags; /* MAGI_ATTN_* bits */
  int32_t out_group_heads;
  int64_t o_stride_g;
  float score_bound;
  int32_t q_tile_rows;
  const float* q_norm_gamma;
  const float* q_norm_beta;
  float q_norm_eps;
  int32_t q_norm_kind;
  /* fp8, optional: scale rows of the side segment k2 / v2 in tables of their own, [chunks of the segment, Hkv],
   * row 0 = the chunk that starts at k_split (then a multiple of scale_chunk_tokens).  A caller that keeps
   * k_scale / v_scale next to a persistent cache can so attach rows it must not persist without rewriting the
   * cache's tables.  NULL (both): k_scale / v_scale are indexed across k_split as one table. */
  const float* k2_scale;
  const float* v2_scale;
  /* MAGI_ATTN_AUTO_BOUND: 16 bytes of DEVICE memory, 16-byte aligned, that the call may overwrite (the measured
   * bound; calls that overlap on the device need a workspace each).  NULL otherwise. */
  float* workspace;
} magi_attn_args;

int magi_attn_fwd(const magi_attn_args* args, void* stream);

/*
 * magi_attn_fwd for callers that cannot hand over a workspace and must not allocate one (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): args->workspace is ignored, and the scratch
 * memory of MAGI_ATTN_AUTO_BOUND is a 256-byte array that lives in the library's device image, one copy per GPU, held
 * until the process ends.  Its need does not grow with the problem (four words), so no size is refused for it.
 * Calls that overlap on one GPU (two streams, two threads) share the array and race: issue them on one stream, or
 * give the others a workspace through magi_attn_fwd.  Without MAGI_ATTN_AUTO_BOUND it is magi_attn_fwd.  Allocates
 * nothing, like every entry point of this library.  No counterpart in the reference.
 */
int magi_attn_fwd_static_scratch(const magi_attn_args* args, void* stream);

/*
 * Fused QK-norm + partial non-interleaved rotary + bf16 cast + KV-cache write, one pass.
 *
 * Stands in for get_q / get_k / get_v / get_kv after the linear layers
 * (inference/model/dit/dit_module.py:953-996: .float(), FusedLayerNorm :323-357, transpose,
 * flash_attn.layers.rotary.apply_rotary_emb :961/:978, .to(bf16), rearrange, cat) and for the
 * cache append of _full_adjust_key_and_value (dit_module.py:918-929).
 *
 * q_raw [S, Hq*D], k_raw / v_raw [S, Hkv*D]  bf16, token strides in elements
 * rope  [S / batch, 2*R2] fp32, sin in the first R2 columns, cos in the last R2 (dit_module.py:770, 1147);
 *       rotary_dim = 2*R2 <= D; NULL disables rotary
 * gq,bq,gk,bk  fp32 [D] norm parameters (gamma stored zero-centred); b* may be NULL
 * q_out [S, Hq, D] bf16 contiguous
 * q_premul  factor applied to q after norm and rotary, before the rounding to bf16 (0 = none, like 1); set it to
 *         softmax_scale * log2(e) when the attention call passes MAGI_ATTN_Q_PRESCALED
 * kv_out  row 0 of the destination for the first n_cache_rows tokens: [*, Hkv, 2D] with token
 *         stride kv_stride_t; K goes to [..., 0:D], V to [..., D:2D]
 * kv_tail destination of tokens >= n_cache_rows (same layout, row index t - n_cache_rows); may be
 *         NULL when n_cache_rows == S
 * out_dtype  MAGI_DTYPE_BF16 (0): as above.  MAGI_DTYPE_FP8_E4M3: the operands of the fp8 attention leave this
 *         pass directly, with no bf16 copy and no absmax pass:  q_out [S, Hq, D] = sat_e4m3(q * q_premul /
 *         q_quant_scale), and kv_out / kv_tail are K destinations [*, Hkv, D] e4m3 (token strides in elements)
 *         = sat_e4m3(k / k_quant_scale).  The two scales are constants of the call (use powers of two: the
 *         kernel multiplies by the reciprocal, which is then exact): a QK-normed row cannot exceed
 *         sqrt(D) max|gamma + 1| + |beta| in any element, before or after the rotation, so a scale chosen from
 *         the norm parameters never saturates, and e4m3 being a floating-point format a conservative scale
 *         costs no precision.  The attention call takes them as constant q_scale / k_scale tables.  V is not
 *         touched (v_raw may be NULL): it has no a-priori bound; magi_quantize_fp8_split takes it from v_raw.
 */
typedef struct magi_prologue_args {
  uint32_t struct_size; /* sizeof(magi_prologue_args) */
  const void* q_raw;
  const void* k_raw;
  const void* v_raw;
  const float* rope;
  const float* gq;
  const float* bq;
  const float* gk;
  const float* bk;
  void* q_out;
  void* kv_out;
  void* kv_tail;
  int64_t q_raw_stride_t, k_raw_stride_t, v_raw_stride_t;
  int64_t kv_stride_t, kv_tail_stride_t;
  int32_t S, n_cache_rows;
  int32_t Hq, Hkv, D, R2;
  int32_t norm_kind;
  float eps;
  int32_t batch; /* tokens are ordered (position, batch): rope row of token t is t / batch; 0 or 1 = no batch */
  float q_premul;
  int32_t out_dtype;
  float q_quant_scale, k_quant_scale;
} magi_prologue_args;

int magi_qk_prologue(const magi_prologue_args* args, void* stream);

/*
 * The four projections of the attention layer and the prologue in one launch: a bf16 GEMM
 *     [S, K] x [N, K]^T,  N = (Hq + 2 Hkv + Hqx) * 128,  rows of w ordered  q heads | k heads | v heads | qx heads
 * whose epilogue does to every (token, head) block of 128 columns what magi_qk_prologue does to the raw
 * projections: round to bf16 (the projection's output dtype), per-head norm, partial rotary, q_premul, cast, and
 * store q to q_out, k and v to the cache rows (kv_out / kv_tail as in magi_prologue_args), the cross-attention
 * q projection UNNORMALISED to qx_out [S, Hqx, D] (magi_attn_fwd normalises it while loading, q_norm_*).
 * Stands in for CustomLayerNormLinear's four linear layers after its LayerNorm
 * (inference/model/dit/dit_module.py:390-425: forward_q / forward_qx / forward_k / forward_v on the output of
 * forward_ln, called at :1153 and :954, 971, 986, 1007) followed by get_q / get_k / get_v (:953-996); the raw
 * projections never reach memory.  fp32 accumulation, so a raw value may differ from a library GEMM's by one bf16
 * rounding where the accumulation order decides it.
 * x [S, K] bf16 (row stride in elements), w [N, K] bf16; K a multiple of 64; Hq + 2 Hkv + Hqx even;
 * rope [S / batch, 96] fp32 (sin | cos) or NULL: this entry point implements rotary_dim 96 (R2 = 48) only.
 */
typedef struct magi_qkv_proj_args {
  uint32_t struct_size; /* sizeof(magi_qkv_proj_args) */
  const void* x;
  const void* w;
  int64_t x_stride, w_stride;
  int32_t S, K;
  int32_t Hq, Hkv, Hqx, D;
  const float* rope;
  int32_t R2;
  const float* gq;
  const float* bq;
  const float* gk;
  const float* bk;
  int32_t norm_kind;
  float eps;
  int32_t batch;
  float q_premul;
  void* q_out;
  void* kv_out;
  void* kv_tail;
  int64_t kv_stride_t, kv_tail_stride_t;
  int32_t n_cache_rows;
  void* qx_out;
} magi_qkv_proj_args;

int magi_qkv_proj_prologue(const magi_qkv_proj_args* args, void* stream);

/*
 * LayerNorm of the layer input over its last axis: x [rows, cols] bf16 -> y [rows, cols] bf16 with fp32
 * statistics, y = (x - mean) / sqrt(var + eps) * weight + bias (plain weight, not the "+1" form).
 * Stands in for torch.nn.LayerNorm in CustomLayerNormLinear.forward_ln (dit_module.py:401, 412-413;
 * first step of the layer forward, :1153).  weight / bias [cols] are bf16 (params_fp32 == 0, the
 * reference's params_dtype) or fp32; NULL weight = 1, NULL bias = 0.  Row strides in elements.
 * cols: multiples of 8 up to 8192.
 */
int magi_layer_norm(const void* x, int64_t x_stride, const void* weight, const void* bias, int32_t params_fp32,
                    void* y, int64_t y_stride, int64_t rows, int32_t cols, float eps, void* stream);

/*
 * The input quantiser of the reference's fp8 linear layers:
 *     y = e4m3fn( bf16( clamp( float(x) / scale, -448, 448 ) ) )
 * including the rounding to bf16 in the middle, which is part of the definition (a value may land on another e4m3
 * code than a direct conversion would give).  Stands in for div_clamp_to (inference/model/dit/dit_module.py:364-384)
 * as PerTensorQuantizedFp8Linear.forward applies it to the normalised hidden states ahead of bmm_fp8 (:445-456; the
 * q, qx, k and v projections of every layer but the first and the last under fp8_quant, :405-409).
 * x [rows, cols] bf16, y [rows, cols] e4m3 (row strides in elements); scale: DEVICE fp32, scale_len 1 (one value) or
 * cols (one per column).  cols a multiple of 8.
 */
int magi_div_clamp_to_e4m3(const void* x, int64_t x_stride, const float* scale, int32_t scale_len, void* y,
                           int64_t y_stride, int64_t rows, int32_t cols, void* stream);

/*
 * Per-head norm only (no rotary, no cache): x [S, H, D] bf16 -> y [S, H, D] bf16, computed in the
 * precision the reference uses for the cross-attention norms (bf16 in, fp32 statistics, bf16 out).
 * Stands in for q_layernorm_xattn / k_layernorm_xattn in get_xqkv (dit_module.py:1008, 1020).
 * x token stride / head stride in elements (K of the interleaved xattn KV projection has
 * head stride 2D); y is contiguous.
 */
int magi_head_norm(const void* x, int64_t x_stride_t, int64_t x_stride_h, const float* gamma, const float* beta,
                   void* y, int32_t S, int32_t H, int32_t D, int32_t norm_kind, float eps, void* stream);

/*
 * Non-interleaved rotary on the first 2*R2 features, any float dtype handled as fp32 or bf16.
 * Stands in for flash_attn.layers.rotary.apply_rotary_emb(x, cos, sin) (dit_module.py:961, 978).
 * x, y [B, S, H, D] contiguous; cos, sin [S, R2] fp32; is_bf16 selects the element type of x / y.
 */
int magi_apply_rotary(const void* x, const float* cos, const float* sin, void* y, int32_t B, int32_t S, int32_t H,
                      int32_t D, int32_t R2, int32_t is_bf16, void* stream);

/*
 * Per-(chunk, head) absmax scales and OCP e4m3fn quantisation for the fp8 attention path:
 * scale[c, h] = max(absmax over tokens of chunk c and D, tiny) * |premul| / 448, rounded UP to a power of two when
 * pow2_scales is set;  y = sat_e4m3(x * premul / scale).
 * The quantiser follows the reference's only fp8 convention, div_clamp_to
 * (dit_module.py:364-384: clamp to +-448, saturating e4m3fn), without its bf16 intermediate.
 * x [T, H, D] bf16 with strides; y [T, H, D] fp8 contiguous; scales fp32 [ceil(T/chunk_tokens), H].
 */
int magi_quantize_fp8(const void* x, int64_t x_stride_t, int64_t x_stride_h, void* y, float* scales, int32_t T,
                      int32_t H, int32_t D, int32_t chunk_tokens, float premul, int32_t pow2_scales, void* stream);

/*
 * The same quantiser with two destinations, as the KV-cache append has them (dit_module.py:918-929: rows that
 * are persisted go to the cache, the others only serve this call): tokens below n_rows_first go to y / scales,
 * the others to y2 / scales2 with row and chunk indices counted from n_rows_first (a multiple of chunk_tokens
 * unless it equals T; y / scales may be NULL when it is 0, y2 / scales2 when it is T).  Always ONE launch: a
 * workgroup per (chunk, head) takes the absmax, writes the scale and quantises, with no memory beyond x and the
 * outputs, so it suits groups the size of a video chunk; magi_quantize_fp8 switches to a multi-launch form for
 * large groups and gives the same bytes.
 */
typedef struct magi_quantize_args {
  uint32_t struct_size; /* sizeof(magi_quantize_args) */
  const void* x;
  int64_t x_stride_t, x_stride_h;
  int32_t T, H, D, chunk_tokens;
  float premul;
  int32_t pow2_scales;
  void* y;
  float* scales;
  int32_t n_rows_first;
  void* y2;
  float* scales2;
} magi_quantize_args;

int magi_quantize_fp8_split(const magi_quantize_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MAGI_ATTN_H */
