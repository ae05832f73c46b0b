// HBM-bound prologue kernels for gfx950: per-head QK norm + partial non-interleaved rotary +
// bf16 cast + KV-cache write in one pass, plus the norm-only and rotary-only variants.  With e4m3 outputs the
// same pass quantises q and k with constant scales (rows of a QK norm have a known bound, so no absmax pass is
// needed) and leaves v to the chunk quantiser.
//
// Layout: 8 lanes serve one (token, head) row of D = 128 elements, 16 elements (two 16-byte
// vectors) per lane, chosen so that a rotary pair (i, i + R2) lives in ONE lane: lanes
// j < R2/8 hold x[8j..8j+7] and x[R2+8j..R2+8j+7], the remaining lanes hold the pass-through
// tail in two consecutive vectors.  The rotation therefore needs no cross-lane traffic and the
// norm statistics need three butterfly steps.  A wavefront covers 8 rows, a workgroup 32; all
// global accesses are 16 bytes per lane and contiguous per row.
#include "kernels.h"

namespace magi {
namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int D = 128;
constexpr int THREADS = 256;
constexpr int GROUPS = THREADS / 8;  // rows in flight per workgroup

__device__ __forceinline__ void unpack8(const u32x4 v, float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __builtin_bit_cast(float, v[i] << 16);
    f[2 * i + 1] = __builtin_bit_cast(float, v[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ unsigned pack2(float a, float b) {
  f32x2 x = {a, b};
  bf16x2 r = __builtin_convertvector(x, bf16x2);
  return __builtin_bit_cast(unsigned, r);
}
__device__ __forceinline__ u32x4 pack8(const float* f) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = pack2(f[2 * i], f[2 * i + 1]);
  return v;
}
// 8 floats -> 8 saturating OCP e4m3fn bytes (the conversion itself does not saturate: clamp first)
__device__ __forceinline__ u32x2 pack8_e4m3(const float* f) {
  u32x2 o;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    float c[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = fminf(fmaxf(f[4 * j + i], -448.f), 448.f);
    int u = 0;
    u = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], u, false);
    u = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], u, true);
    o[j] = (unsigned)u;
  }
  return o;
}
__device__ __forceinline__ float group8_sum(float x) {
  x += __shfl_xor(x, 1);
  x += __shfl_xor(x, 2);
  x += __shfl_xor(x, 4);
  return x;
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) x += __shfl_xor(x, m);
  return x;
}

// Normalise the 16 values of this lane (8 lanes = one row of 128) in place.
__device__ __forceinline__ void norm16(float* x, const float* gam, const float* bet, int ea, int eb, int kind, float eps,
                                       bool has_beta) {
  if (kind == 2) return;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += x[i];
  float mean = 0.f;
  if (kind == 0) mean = group8_sum(s) * (1.f / D);
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float d = x[i] - mean;
    q += d * d;
  }
  const float rstd = __builtin_amdgcn_rsqf(group8_sum(q) * (1.f / D) + eps);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int e = (i < 8) ? ea + i : eb + (i - 8);
    float y = (x[i] - mean) * rstd * (gam[e] + 1.f);
    if (kind == 0 && has_beta) y += bet[e];
    x[i] = y;
  }
}

// TPB: tokens that share a workgroup (1, 2, 4 or 8).  OUT8: q and k leave as e4m3 bytes (q_out [S, Hq, D],
// K rows [*, Hkv, D] at kv_out / kv_tail), each multiplied by its constant inverse scale; v is not touched.
template <int TPB, bool OUT8>
__global__ __launch_bounds__(THREADS) void prologue_kernel(const PrologueKernArgs a) {
  __shared__ float s_par[4][D];  // gq, bq, gk, bk
  const int tid = threadIdx.x;
  // Everything a workgroup needs from memory is requested in one go: the norm parameters (two per thread, on their way
  // to LDS), the token's rotary row and each row group's first row; the barrier that publishes the parameters is where
  // they are waited for.  (Parameters, barrier, then the rows: two memory latencies in a workgroup that lives for
  // little more than that.)
  float par[4 * D / THREADS];
#pragma unroll
  for (int k = 0; k < 4 * D / THREADS; ++k) {
    const int i = tid + k * THREADS, which = i / D, e = i % D;
    const float* src = which == 0 ? a.gq : which == 1 ? a.bq : which == 2 ? a.gk : a.bk;
    par[k] = src ? src[e] : 0.f;
  }

  // The 32 row groups of the workgroup form tok_per_block teams of equal size, one token each, so that layers
  // with few heads (e.g. one rank's share of a head-parallel split: 8 rows per token) still fill the workgroup.
  const int j = tid & 7;
  constexpr int gpt = GROUPS / TPB;  // row groups per token
  const int team = TPB == 1 ? 0 : (tid >> 3) / gpt;  // (a constant keeps the token index in a scalar register)
  const int grp = (tid >> 3) % gpt;
  const int nr = a.R2 >> 3;  // lanes that hold rotary pairs
  const bool rot_lane = j < nr;
  const int ea = rot_lane ? 8 * j : 2 * a.R2 + 16 * (j - nr);  // first element of vector A
  const int eb = rot_lane ? a.R2 + 8 * j : ea + 8;             // first element of vector B
  const int U = a.Hq + (OUT8 ? 1 : 2) * a.Hkv;
  constexpr int ES = OUT8 ? 1 : 2;  // bytes per output element

  const int s = blockIdx.x * TPB + team;
  const bool live = s < a.S;
  float sn[8], cs[8];
  if (live && rot_lane && a.rope) {
    const float* rp = a.rope + (long)(s / a.batch) * (2 * a.R2);
    const f32x4 s0 = *(const f32x4*)(rp + 8 * j), s1 = *(const f32x4*)(rp + 8 * j + 4);
    const f32x4 c0 = *(const f32x4*)(rp + a.R2 + 8 * j), c1 = *(const f32x4*)(rp + a.R2 + 8 * j + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sn[i] = s0[i];
      sn[4 + i] = s1[i];
      cs[i] = c0[i];
      cs[4 + i] = c1[i];
    }
  }
  const int sc = live ? s : 0;  // (a valid row for the address arithmetic of a team past the end)
  char* kvrow = (sc < a.n_cache_rows) ? a.kv_out + (long)sc * a.kv_stride_t
                                      : a.kv_tail + (long)(sc - a.n_cache_rows) * a.kv_tail_stride_t;
  // row u of the token: 0 = q, 1 = k, 2 = v; where it comes from and where it goes
  auto locate = [&](int u, const char*& src, char*& dst, int& kind) __attribute__((always_inline)) {
    if (u < a.Hq) {
      kind = 0;
      src = a.q_raw + (long)sc * a.q_raw_stride_t + (long)u * (D * 2);
      dst = a.q_out + ((long)sc * a.Hq + u) * (D * ES);
    } else if (u < a.Hq + a.Hkv) {
      kind = 1;
      const int hh = u - a.Hq;
      src = a.k_raw + (long)sc * a.k_raw_stride_t + (long)hh * (D * 2);
      dst = kvrow + (long)hh * (OUT8 ? D : 2 * D * 2);
    } else {
      kind = 2;
      const int hh = u - a.Hq - a.Hkv;
      src = a.v_raw + (long)sc * a.v_raw_stride_t + (long)hh * (D * 2);
      dst = kvrow + (long)hh * (2 * D * 2) + D * 2;
    }
  };
  int u = grp;
  const char* src = nullptr;
  char* dst = nullptr;
  int kind = 0;
  u32x4 va = {0u, 0u, 0u, 0u}, vb = va;
  if (live && u < U) {
    locate(u, src, dst, kind);
    va = *(const u32x4*)(src + ea * 2);
    vb = *(const u32x4*)(src + eb * 2);
  }
#pragma unroll
  for (int k = 0; k < 4 * D / THREADS; ++k) {
    const int i = tid + k * THREADS;
    s_par[i / D][i % D] = par[k];
  }
  __syncthreads();
  if (!live) return;

  while (u < U) {
    // the next row of this group is requested before the current one is worked on
    const int u_next = u + gpt;
    const char* src_n = nullptr;
    char* dst_n = nullptr;
    int kind_n = 0;
    u32x4 va_n = va, vb_n = vb;
    if (u_next < U) {
      locate(u_next, src_n, dst_n, kind_n);
      va_n = *(const u32x4*)(src_n + ea * 2);
      vb_n = *(const u32x4*)(src_n + eb * 2);
    }
    if (kind == 2) {
      *(u32x4*)(dst + ea * 2) = va;
      *(u32x4*)(dst + eb * 2) = vb;
    } else {
      float x[16];
      unpack8(va, x);
      unpack8(vb, x + 8);
      norm16(x, s_par[2 * kind], s_par[2 * kind + 1], ea, eb, a.norm_kind, a.eps, true);
      if (rot_lane && a.rope) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float x1 = x[i], x2 = x[8 + i];
          x[i] = x1 * cs[i] - x2 * sn[i];
          x[8 + i] = x1 * sn[i] + x2 * cs[i];
        }
      }
      if (kind == 0 && a.q_premul != 1.f) {  // e.g. softmax_scale * log2(e), ahead of the one rounding to bf16
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] *= a.q_premul;
      }
      if constexpr (OUT8) {
        const float inv = kind == 0 ? a.q_inv_scale : a.k_inv_scale;
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] *= inv;
        *(u32x2*)(dst + ea) = pack8_e4m3(x);
        *(u32x2*)(dst + eb) = pack8_e4m3(x + 8);
      } else {
        *(u32x4*)(dst + ea * 2) = pack8(x);
        *(u32x4*)(dst + eb * 2) = pack8(x + 8);
      }
    }
    u = u_next;
    src = src_n;
    dst = dst_n;
    kind = kind_n;
    va = va_n;
    vb = vb_n;
  }
}

// x [S, H, 128] bf16 with strides -> y contiguous, norm only.
__global__ __launch_bounds__(THREADS) void head_norm_kernel(const char* x, long xs_t, long xs_h, const float* gamma,
                                                            const float* beta, char* y, int S, int H, int norm_kind,
                                                            float eps) {
  __shared__ float s_par[2][D];
  const int tid = threadIdx.x;
  for (int i = tid; i < 2 * D; i += THREADS) {
    const float* src = i < D ? gamma : beta;
    s_par[i / D][i % D] = src ? src[i % D] : 0.f;
  }
  __syncthreads();
  const int j = tid & 7;
  const long row = (long)blockIdx.x * GROUPS + (tid >> 3);
  if (row >= (long)S * H) return;
  const long s = row / H, h = row % H;
  const char* src = x + s * xs_t + h * xs_h;
  char* dst = y + row * (D * 2);
  const int ea = 16 * j, eb = ea + 8;
  float v[16];
  unpack8(*(const u32x4*)(src + ea * 2), v);
  unpack8(*(const u32x4*)(src + eb * 2), v + 8);
  norm16(v, s_par[0], s_par[1], ea, eb, norm_kind, eps, beta != nullptr);
  *(u32x4*)(dst + ea * 2) = pack8(v);
  *(u32x4*)(dst + eb * 2) = pack8(v + 8);
}

// Row LayerNorm of the layer input: one wavefront per row, the row held packed in registers as NV 16-byte
// vectors per lane (vector i of lane l covers elements (64 i + l) * 8 ...), fp32 statistics in two passes over
// the registers.  Weight and bias are read straight from global memory in the last pass (they stay in L1 / L2);
// a persistent variant that staged them in LDS once per workgroup measured 7-8 % slower.
template <int NV, bool PF32>
__global__ __launch_bounds__(THREADS) void layer_norm_kernel(const char* x, long xs, const char* w, const char* b,
                                                             char* y, long ys, long rows, int cols, float eps) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int nvec = cols >> 3;
  const float inv_n = 1.f / (float)cols;
  const long row = (long)blockIdx.x * (THREADS / 64) + (tid >> 6);
  if (row >= rows) return;
  const char* src = x + row * xs;
  u32x4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int vi = i * 64 + lane;
    raw[i] = vi < nvec ? *(const u32x4*)(src + (long)vi * 16) : u32x4{0u, 0u, 0u, 0u};
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    float f[8];
    unpack8(raw[i], f);
#pragma unroll
    for (int k = 0; k < 8; ++k) s += f[k];
  }
  const float mean = wave_sum(s) * inv_n;
  // the row stays packed between the passes (48 registers for 6144 columns instead of 96 more for its fp32
  // form): the empty asm makes the compiler unpack again rather than keep the first pass's values
#pragma unroll
  for (int i = 0; i < NV; ++i) asm volatile("" : "+v"(raw[i]));
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (i * 64 + lane < nvec) {
      float f[8];
      unpack8(raw[i], f);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float d = f[k] - mean;
        q += d * d;
      }
    }
  }
  const float rstd = __builtin_amdgcn_rsqf(wave_sum(q) * inv_n + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) asm volatile("" : "+v"(raw[i]));
  char* dst = y + row * ys;
  auto param8 = [&](const char* p, int vi, float* out) {  // elements 8 vi .. 8 vi + 7 of a parameter
    if (PF32) {
      const f32x4 lo = *(const f32x4*)(p + (long)vi * 32), hi = *(const f32x4*)(p + (long)vi * 32 + 16);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        out[k] = lo[k];
        out[4 + k] = hi[k];
      }
    } else {
      unpack8(*(const u32x4*)(p + (long)vi * 16), out);
    }
  };
  if (w && b) {  // the usual case, free of branches so that the parameter loads of all vectors go out together
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int vi = i * 64 + lane;
      if (vi < nvec) {
        float f[8], wf[8], bf[8];
        unpack8(raw[i], f);
        param8(w, vi, wf);
        param8(b, vi, bf);
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] = (f[k] - mean) * rstd * wf[k] + bf[k];
        *(u32x4*)(dst + (long)vi * 16) = pack8(f);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int vi = i * 64 + lane;
      if (vi < nvec) {
        float f[8], wf[8], bf[8];
        unpack8(raw[i], f);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          wf[k] = 1.f;
          bf[k] = 0.f;
        }
        if (w) param8(w, vi, wf);
        if (b) param8(b, vi, bf);
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] = (f[k] - mean) * rstd * wf[k] + bf[k];
        *(u32x4*)(dst + (long)vi * 16) = pack8(f);
      }
    }
  }
}

// Rotary only: x, y [B, S, H, D]; one thread per (row, pair).
template <bool BF16>
__global__ __launch_bounds__(THREADS) void rotary_kernel(const void* xin, const float* cosp, const float* sinp,
                                                         void* yout, long rows, int S, int H, int Dd, int R2) {
  const long gid = (long)blockIdx.x * THREADS + threadIdx.x;
  const int half = Dd / 2;  // threads per row: each handles elements p and p + half ... see below
  const long row = gid / half;
  const int p = (int)(gid % half);
  if (row >= rows) return;
  const long s = (row / H) % S;
  // thread p < R2 rotates the pair (p, p + R2); threads R2 <= p < half copy the tail two at a time
  auto ld = [&](long idx) -> float {
    if (BF16) return __builtin_bit_cast(float, (unsigned)((const unsigned short*)xin)[idx] << 16);
    return ((const float*)xin)[idx];
  };
  auto st = [&](long idx, float v) {
    if (BF16) {
      f32x2 t = {v, 0.f};
      bf16x2 r = __builtin_convertvector(t, bf16x2);
      ((unsigned short*)yout)[idx] = (unsigned short)(__builtin_bit_cast(unsigned, r) & 0xffffu);
    } else {
      ((float*)yout)[idx] = v;
    }
  };
  const long base = row * Dd;
  if (p < R2) {
    const float c = cosp[s * R2 + p], sn = sinp[s * R2 + p];
    const float x1 = ld(base + p), x2 = ld(base + R2 + p);
    st(base + p, x1 * c - x2 * sn);
    st(base + R2 + p, x1 * sn + x2 * c);
  } else {
    const int e = 2 * R2 + 2 * (p - R2);
    st(base + e, ld(base + e));
    st(base + e + 1, ld(base + e + 1));
  }
}

// div_clamp_to: y = e4m3(bf16(clamp(float(x) / scale, -448, 448))), the fp8 linears' input quantiser with its bf16
// intermediate (a double rounding that is part of the definition).  One thread per 8 consecutive elements of a row;
// scale: one value, or one per column.  IEEE division (the reference divides in fp32).
__global__ __launch_bounds__(THREADS) void div_clamp_kernel(const char* x, long xs, const float* scale, int per_column,
                                                            char* y, long ys, long rows, int cols8) {
  const long t = (long)blockIdx.x * THREADS + threadIdx.x;
  if (t >= rows * cols8) return;
  const long r = t / cols8;
  const int c = (int)(t - r * cols8);
  float f[8];
  unpack8(*(const u32x4*)(x + r * xs + (long)c * 16), f);
  float sc[8];
  if (per_column) {
    const f32x4 s0 = *(const f32x4*)(scale + 8 * c), s1 = *(const f32x4*)(scale + 8 * c + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = s0[i];
      sc[4 + i] = s1[i];
    }
  } else {
    const float s = scale[0];
#pragma unroll
    for (int i = 0; i < 8; ++i) sc[i] = s;
  }
  float q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float d = f[i] / sc[i];
    const float cl = d != d ? d : fminf(fmaxf(d, -448.f), 448.f);  // (a NaN stays a NaN, as torch.clamp leaves it)
    q[i] = (float)(__bf16)cl;                                     // the bf16 intermediate
  }
  u32x2 o;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    int u = 0;
    u = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j], q[4 * j + 1], u, false);
    u = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * j + 2], q[4 * j + 3], u, true);
    o[j] = (unsigned)u;
  }
  *(u32x2*)(y + r * ys + (long)c * 8) = o;
}

}  // namespace

hipError_t launch_div_clamp(const char* x, long x_stride, const float* scale, int per_column, char* y, long y_stride,
                            long rows, int cols, hipStream_t stream) {
  const long n = rows * (cols / 8);
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(div_clamp_kernel, dim3((unsigned)((n + THREADS - 1) / THREADS)), dim3(THREADS), 0, stream, x, x_stride,
                     scale, per_column, y, y_stride, rows, cols / 8);
  return hipGetLastError();
}

hipError_t launch_prologue(const PrologueKernArgs& a_in, hipStream_t stream) {
  if (a_in.S <= 0) return hipSuccess;
  const PrologueKernArgs& a = a_in;
  const int rows = a.Hq + (a.out_fp8 ? 1 : 2) * a.Hkv;
  int tpb = 1;
  while (tpb < 8 && 2 * tpb * rows <= GROUPS) tpb *= 2;
  const dim3 grid((unsigned)((a.S + tpb - 1) / tpb)), block(THREADS);
#define MAGI_PROLOGUE(TPB)                                                                  \
  do {                                                                                      \
    if (a.out_fp8)                                                                          \
      hipLaunchKernelGGL((prologue_kernel<TPB, true>), grid, block, 0, stream, a);          \
    else                                                                                    \
      hipLaunchKernelGGL((prologue_kernel<TPB, false>), grid, block, 0, stream, a);         \
  } while (0)
  switch (tpb) {
    case 1: MAGI_PROLOGUE(1); break;
    case 2: MAGI_PROLOGUE(2); break;
    case 4: MAGI_PROLOGUE(4); break;
    default: MAGI_PROLOGUE(8); break;
  }
#undef MAGI_PROLOGUE
  return hipGetLastError();
}

hipError_t launch_head_norm(const char* x, long x_stride_t, long x_stride_h, const float* gamma, const float* beta,
                            char* y, int S, int H, int norm_kind, float eps, hipStream_t stream) {
  const long rows = (long)S * H;
  if (rows <= 0) return hipSuccess;
  const unsigned grid = (unsigned)((rows + GROUPS - 1) / GROUPS);
  hipLaunchKernelGGL(head_norm_kernel, dim3(grid), dim3(THREADS), 0, stream, x, x_stride_t, x_stride_h, gamma, beta, y,
                     S, H, norm_kind, eps);
  return hipGetLastError();
}

hipError_t launch_layer_norm(const char* x, long x_stride, const void* w, const void* b, int params_fp32, char* y,
                             long y_stride, long rows, int cols, float eps, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  const int need = (cols / 8 + 63) / 64;  // 16-byte vectors per lane
  const dim3 grid((unsigned)((rows + THREADS / 64 - 1) / (THREADS / 64))), block(THREADS);
  const char* wp = static_cast<const char*>(w);
  const char* bp = static_cast<const char*>(b);
#define MAGI_LN(NV)                                                                                               \
  do {                                                                                                            \
    if (params_fp32)                                                                                              \
      hipLaunchKernelGGL((layer_norm_kernel<NV, true>), grid, block, 0, stream, x, x_stride, wp, bp, y, y_stride, \
                         rows, cols, eps);                                                                        \
    else                                                                                                          \
      hipLaunchKernelGGL((layer_norm_kernel<NV, false>), grid, block, 0, stream, x, x_stride, wp, bp, y,          \
                         y_stride, rows, cols, eps);                                                              \
  } while (0)
  if (need <= 2) MAGI_LN(2);
  else if (need <= 4) MAGI_LN(4);
  else if (need <= 6) MAGI_LN(6);
  else if (need <= 8) MAGI_LN(8);
  else if (need <= 12) MAGI_LN(12);
  else MAGI_LN(16);
#undef MAGI_LN
  return hipGetLastError();
}

hipError_t launch_rotary(const void* x, const float* cos, const float* sin, void* y, int B, int S, int H, int Dd, int R2,
                         int is_bf16, hipStream_t stream) {
  const long rows = (long)B * S * H;
  const long threads = rows * (Dd / 2);
  if (threads <= 0) return hipSuccess;
  const unsigned grid = (unsigned)((threads + THREADS - 1) / THREADS);
  if (is_bf16)
    hipLaunchKernelGGL(rotary_kernel<true>, dim3(grid), dim3(THREADS), 0, stream, x, cos, sin, y, rows, S, H, Dd, R2);
  else
    hipLaunchKernelGGL(rotary_kernel<false>, dim3(grid), dim3(THREADS), 0, stream, x, cos, sin, y, rows, S, H, Dd, R2);
  return hipGetLastError();
}

}  // namespace magi
