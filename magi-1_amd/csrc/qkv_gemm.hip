// The four projections of the attention layer as ONE bf16 GEMM whose epilogue is the prologue, for gfx950.
//
//   C[token][column] = sum_k X[token][k] W[column][k]        X [S, K] normalised hidden states, W [N, K]
//
// with the rows of W ordered [q heads | k heads | v heads | qx heads], 128 rows per head.  A column block of 128
// is one head, and a wavefront owns one head for 64 tokens, so everything the prologue does to a (token, head)
// row (round to bf16 as the projection's output would be, LayerNorm over the 128 features, partial rotary,
// factor on q, cast, store to q / the KV-cache rows / the raw cross-attention q) happens on the accumulators, and
// the raw projections never reach memory.
//
// Shape of the work.  Workgroup: 256 tokens x 256 columns (two heads), 8 wavefronts (2 per SIMD), wavefront
// (wn, wm) = head wn of the pair, tokens 64 wm .. +63.  K is walked in steps of 64: the X and W slices of a step
// (256 rows x 128 bytes each) are double buffered in LDS by direct global->LDS buffer loads, rows swizzled in
// 16-byte chunks (chunk ^ ((row >> 1) & 7)) so that the 16-byte operand reads of 16 consecutive rows fall on
// different banks.  The product is formed transposed, C^T = W X^T on v_mfma_f32_32x32x16_bf16 (W rows as the A
// operand, tokens as the B operand): a lane then holds ONE token per 32-token block and 64 of its 128 features
// (its partner in the other half wave the other 64), which is the layout the epilogue wants: the norm statistics
// need one exchange between the half waves, and a rotary pair (f, f + 48) lives in one lane.
// Per 64-step a wave issues 24 operand reads of 16 bytes for 32 MFMAs: 0.75 KB of LDS reads per MFMA, 96 bytes per
// clock and CU at the full MFMA rate, beside 32 for filling the slices.  The CU's LDS delivers about 157 bytes per
// clock to ds_read_b128 (measured with a read-only loop), so LDS bandwidth is what bounds this kernel; the library
// GEMM it competes with sits at the same wall with 128 x 128 per wavefront (0.5 KB per MFMA).
#include "attn_common.h"

#include <cstdlib>

namespace magi {
namespace {

constexpr int BM = 256;  // tokens per workgroup
constexpr int BNC = 256; // columns per workgroup (two heads)
constexpr int BK = 64;   // k per step
constexpr int ROWB = BK * 2;  // bytes per LDS row
constexpr int TILE = BM * ROWB;  // 32 KB per matrix per stage
constexpr int D = 128;
constexpr int R2 = 48;  // rotary pairs (the MAGI-1 layout: rotary_dim 96 of 128)

// MB: blocks of 32 tokens per wavefront.  MB = 2 (shipped): 8 wavefronts (two per SIMD), 128 accumulator registers
// each.  MB = 4: 4 wavefronts (one per SIMD) with 256 accumulator registers each, 0.5 instead of 0.75 KB of LDS
// operand reads per MFMA, but nothing to hide a wave's own waits behind; measured within 2 % of the other.
template <int MB>
__global__ __launch_bounds__(64 * (16 / MB), 1) void qkv_gemm_prologue_kernel(const QkvGemmKernArgs a) {
  constexpr int NWAVES = 16 / MB;
  constexpr int LOADS = 32 / NWAVES;  // wave-loads (8 rows each) per wave per matrix per step
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* const sX0 = smem;
  unsigned char* const sW0 = smem + TILE;
  unsigned char* const sX1 = smem + 2 * TILE;
  unsigned char* const sW1 = smem + 3 * TILE;
  unsigned char* const sJunk = smem + 4 * TILE;  // 1 KB that nothing reads (destination of the cache-warming loads)

  // ---- which tile: blockIdx % 8 is the XCD.  XCD x owns the token tiles x, x + 8, x + 16, ... (an even share for
  // every XCD whatever the tile count) and walks them in blocks of 8 x all column tiles, token tile fastest, so that
  // the ~32 workgroups it runs at a time share 8 X slices and 4 W slices through its L2 ----
  const int xcd = blockIdx.x & 7;
  const int t = blockIdx.x >> 3;
  const int per_block = 8 * a.n_col_tiles;
  const int qb = t / per_block, r = t % per_block;
  const int m_tile = (qb * 8 + (r & 7)) * 8 + xcd;
  const int n_tile = r >> 3;
  if (m_tile >= a.n_row_tiles) return;
  const int m0 = m_tile * BM;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, i = l & 31, g = l >> 5;
  const int wn = w & 1, wm = w >> 1;

  const int n_steps = a.K / BK;
  // ---- loader: a wave-load of 64 x 16 bytes fills 8 LDS rows; wave w takes row groups w, w + NWAVES, ...
  // of both matrices.  Lane l sits at row (l >> 3) of its group, slot l & 7, and fetches the logical chunk that
  // belongs there under the swizzle.
  const int lr = l >> 3, sl = l & 7;
  const int chunk = sl ^ ((4 * w + (lr >> 1)) & 7);
  const char* const xb = a.x + (long)m0 * a.x_stride;
  const char* const wb = a.w + (long)n_tile * BNC * a.w_stride;
  // rows past the end of X read as zeros through the descriptor's size
  const long x_valid = (long)(a.S - m0) * a.x_stride;
  const __amdgpu_buffer_rsrc_t rx =
      __builtin_amdgcn_make_buffer_rsrc((void*)xb, 0, (int)(x_valid < 0x7fffffffL ? x_valid : 0x7fffffffL), 0x00020000);
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)wb, 0, 0x7fffffff, 0x00020000);
  const unsigned vx = (unsigned)(8 * w + lr) * (unsigned)a.x_stride + (unsigned)(chunk * 16);
  const unsigned vw = (unsigned)(8 * w + lr) * (unsigned)a.w_stride + (unsigned)(chunk * 16);
  auto issue_pair = [&](int j, int kstep, unsigned char* sX, unsigned char* sW) __attribute__((always_inline)) {
    const unsigned kb = (unsigned)kstep * (unsigned)ROWB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, LDS_PTR(void, sX + (w + NWAVES * j) * 1024), 16, vx,
                                             (int)(kb + (unsigned)(8 * NWAVES * j) * (unsigned)a.x_stride), 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, LDS_PTR(void, sW + (w + NWAVES * j) * 1024), 16, vw,
                                             (int)(kb + (unsigned)(8 * NWAVES * j) * (unsigned)a.w_stride), 0, 0);
  };
  // Warm the caches for the slice after `kstep`: one 4-byte load per 128-byte row segment, issued BEHIND the loads of
  // slice `kstep` (loads complete in order, so the wait in front of the barrier can leave exactly these outstanding)
  // into LDS that nothing reads.  A slice is requested by the ~32 workgroups of an XCD at about the same time and
  // the first request goes to HBM (measured: 6 % on the 4-wavefront form, which has nothing to hide a wait behind;
  // no difference on the 8-wavefront form).  Always issued: the waits count them.
  auto issue_touch = [&](int kstep) __attribute__((always_inline)) {
    const unsigned kt = (unsigned)min(kstep + 1, n_steps - 1) * (unsigned)ROWB;
    if constexpr (MB == 4) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, LDS_PTR(void, sJunk), 4, (unsigned)tid * (unsigned)a.x_stride, (int)kt, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, LDS_PTR(void, sJunk + 256), 4, (unsigned)tid * (unsigned)a.w_stride, (int)kt, 0, 0);
    } else {
      if (w < 4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, LDS_PTR(void, sJunk), 4, (unsigned)tid * (unsigned)a.x_stride, (int)kt, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, LDS_PTR(void, sJunk + 256), 4, (unsigned)(tid - 256) * (unsigned)a.w_stride, (int)kt, 0, 0);
    }
  };
  constexpr int TOUCHES = MB == 4 ? 2 : 1;  // cache-warming loads per wave per step

  // ---- operand reads: row 32 blk + i of a slice, 16-byte chunk (2 kk + g) ^ ((i >> 1) & 7) ----
  const int sw = ((g ^ ((i >> 1) & 7)) << 4);
  const int base_w = (128 * wn + i) * ROWB + sw;  // + nb * 32 rows
  const int base_x = (32 * MB * wm + i) * ROWB + sw;   // + mb * 32 rows

  f32x16 acc[4][MB];  // [feature block of 32][token block of 32]
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[nb][mb][v] = 0.f;

  bf16x8 wf[2][4], xf[2][MB];  // two sets of operand fragments (one k block of 16 each)
  auto fetch = [&](const unsigned char* X, const unsigned char* W, int kk, int s) __attribute__((always_inline)) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) wf[s][nb] = *LDS_PTR(const bf16x8, W + ((base_w ^ (kk << 5)) + nb * 32 * ROWB));
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xf[s][mb] = *LDS_PTR(const bf16x8, X + ((base_x ^ (kk << 5)) + mb * 32 * ROWB));
    __builtin_amdgcn_sched_barrier(0);
  };
  // The MFMAs of the k block in set s in four groups (one feature block each), and behind every group a share of the
  // other work, so that the wave never goes long without issuing an MFMA:
  //  * the operand reads of the NEXT k block (kk_next of slices Xr / Wr, into the other set): the token fragments
  //    first, because the next block's first group needs all of them, then the feature fragments in the order of use;
  //  * if ld0 >= 0, the direct loads of the next slice: wave-load pairs ld0 + group, and behind the last pair the
  //    cache-warming loads.
  // The sched_barriers keep the compiler from gathering all this or sinking a read to its use.
  auto block = [&](int s, const unsigned char* Xr, const unsigned char* Wr, int kk_next, bool rd, int ld0 = -100,
                   int kstep = 0, unsigned char* Xl = nullptr, unsigned char* Wl = nullptr) __attribute__((always_inline)) {
    constexpr int NREAD = MB + 4;  // fragments per k block: x0 .. x(MB-1), w0 .. w3
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[s][nb], xf[s][mb], acc[nb][mb], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (rd) {
#pragma unroll
        for (int r = nb * NREAD / 4; r < (nb + 1) * NREAD / 4; ++r) {
          if (r < MB)
            xf[s ^ 1][r] = *LDS_PTR(const bf16x8, Xr + ((base_x ^ (kk_next << 5)) + r * 32 * ROWB));
          else
            wf[s ^ 1][r - MB] = *LDS_PTR(const bf16x8, Wr + ((base_w ^ (kk_next << 5)) + (r - MB) * 32 * ROWB));
        }
      }
      if (ld0 + nb >= 0 && ld0 + nb < LOADS && kstep < n_steps) issue_pair(ld0 + nb, kstep, Xl, Wl);
      if (ld0 + nb == LOADS - 1) issue_touch(kstep);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // The loop is rotated so that the matrix pipe has work across the barrier: a step's last k block (operands already
  // in registers) is multiplied AFTER the barrier that hands over the next slice, while the first operands of that
  // slice are read.  Before the barrier a wave waits for its own LDS reads (the slot it read is overwritten by the
  // loads issued after the barrier) and for its loads of the next slice.
#pragma unroll
  for (int j = 0; j < LOADS; ++j) issue_pair(j, 0, sX0, sW0);
  issue_touch(0);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(TOUCHES) : "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  fetch(sX0, sW0, 0, 0);
  auto step = [&](int ks, auto BUFC) __attribute__((always_inline)) {
    constexpr int BUF = decltype(BUFC)::value;
    const unsigned char* const X = BUF ? sX1 : sX0;
    const unsigned char* const W = BUF ? sW1 : sW0;
    unsigned char* const Xn = BUF ? sX0 : sX1;
    unsigned char* const Wn = BUF ? sW0 : sW1;
    const bool more = ks + 1 < n_steps;
    block(0, X, W, 1, true, 0, ks + 1, Xn, Wn);
    block(1, X, W, 2, true, LOADS > 4 ? 4 : -100, ks + 1, Xn, Wn);
    block(0, X, W, 3, true);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(TOUCHES) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    block(1, Xn, Wn, 0, more);
  };
  int ks = 0;
  for (; ks + 1 < n_steps; ks += 2) {
    step(ks, std::integral_constant<int, 0>{});
    step(ks + 1, std::integral_constant<int, 1>{});
  }
  if (ks < n_steps) step(ks, std::integral_constant<int, 0>{});

  // ---- epilogue: the prologue on the accumulators ----
  // register v of acc[nb][mb] = feature 32 nb + 8 (v >> 2) + 4 g + (v & 3) of token 32 mb + i
  const int head = 2 * n_tile + wn;
  int kind, hh;  // 0 = q, 1 = k, 2 = v, 3 = qx; head index within its kind
  if (head < a.Hq) {
    kind = 0;
    hh = head;
  } else if (head < a.Hq + a.Hkv) {
    kind = 1;
    hh = head - a.Hq;
  } else if (head < a.Hq + 2 * a.Hkv) {
    kind = 2;
    hh = head - a.Hq - a.Hkv;
  } else {
    kind = 3;
    hh = head - a.Hq - 2 * a.Hkv;
  }
  const bool normed = kind < 2 && a.norm_kind != 2;
  const float* const gam = kind == 0 ? a.gq : a.gk;
  const float* const bet = kind == 0 ? a.bq : a.bk;
  const float premul = kind == 0 ? a.q_premul : 1.f;
  int lane_e = l;
  asm volatile("" : "+v"(lane_e));
  const int ie = lane_e & 31, ge = lane_e >> 5;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int s = m0 + 32 * MB * wm + 32 * mb + ie;
    const bool row_ok = s < a.S;
    // the projection's output is a bf16 tensor in the reference: round once, as it would have been
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[nb][mb][v] = (float)(__bf16)acc[nb][mb][v];
    if (normed) {
      float sum = 0.f;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) sum += acc[nb][mb][v];
      sum += __shfl_xor(sum, 32);
      const float mean = a.norm_kind == 0 ? sum * (1.f / D) : 0.f;
      float sq = 0.f;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float d = acc[nb][mb][v] - mean;
          sq += d * d;
        }
      sq += __shfl_xor(sq, 32);
      const float rstd = __builtin_amdgcn_rsqf(sq * (1.f / D) + a.eps);
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int f = 32 * nb + 8 * q4 + 4 * ge;
          const f32x4 g4 = *(const f32x4*)(gam + f);
          f32x4 b4 = {0.f, 0.f, 0.f, 0.f};
          if (a.norm_kind == 0 && bet) b4 = *(const f32x4*)(bet + f);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[nb][mb][4 * q4 + e] = (acc[nb][mb][4 * q4 + e] - mean) * rstd * (g4[e] + 1.f) + b4[e];
        }
    }
    if (kind < 2 && a.rope) {
      // pairs (f, f + 48), f < 48: (nb 0, q4 0..1) with (nb 1, q4 2..3), (nb 0, q4 2..3) with (nb 2, q4 0..1),
      // (nb 1, q4 0..1) with (nb 2, q4 2..3); sin in the first 48 columns of the table row, cos in the last 48
      const float* const rp = a.rope + (long)((row_ok ? s : a.S - 1) / a.batch) * (2 * R2);
      auto rotate = [&](int nb1, int qa, int nb2, int qb) __attribute__((always_inline)) {
        const int f = 32 * nb1 + 8 * qa + 4 * ge;
        const f32x4 sn = *(const f32x4*)(rp + f), cs = *(const f32x4*)(rp + R2 + f);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x1 = acc[nb1][mb][4 * qa + e], x2 = acc[nb2][mb][4 * qb + e];
          acc[nb1][mb][4 * qa + e] = x1 * cs[e] - x2 * sn[e];
          acc[nb2][mb][4 * qb + e] = x1 * sn[e] + x2 * cs[e];
        }
      };
      rotate(0, 0, 1, 2);
      rotate(0, 1, 1, 3);
      rotate(0, 2, 2, 0);
      rotate(0, 3, 2, 1);
      rotate(1, 0, 2, 2);
      rotate(1, 1, 2, 3);
    }
    if (premul != 1.f) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nb][mb][v] *= premul;
    }
    // destination row of this token for this head
    char* dst;
    if (kind == 0) {
      dst = a.q_out + ((long)s * a.Hq + hh) * (D * 2);
    } else if (kind == 3) {
      dst = a.qx_out + ((long)s * a.Hqx + hh) * (D * 2);
    } else {
      char* const kvrow = (s < a.n_cache_rows) ? a.kv_out + (long)s * a.kv_stride_t
                                               : a.kv_tail + (long)(s - a.n_cache_rows) * a.kv_tail_stride_t;
      dst = kvrow + (long)hh * (2 * D * 2) + (kind == 2 ? D * 2 : 0);
    }
    dst += 16 * ge;
    // the half waves trade registers so that every lane owns eight consecutive features: 16-byte stores
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int bp = 0; bp < 2; ++bp) {
        unsigned ev[2], od[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          ev[e] = pack_bf16x2(acc[nb][mb][8 * bp + 2 * e], acc[nb][mb][8 * bp + 2 * e + 1]);
          od[e] = pack_bf16x2(acc[nb][mb][8 * bp + 4 + 2 * e], acc[nb][mb][8 * bp + 4 + 2 * e + 1]);
          half_swap(ev[e], od[e]);
        }
        if (row_ok) *(u32x4*)(dst + (32 * nb + 16 * bp) * 2) = u32x4{ev[0], ev[1], od[0], od[1]};
      }
  }
}

}  // namespace

hipError_t launch_qkv_gemm_prologue(const QkvGemmKernArgs& a_in, hipStream_t stream) {
  if (a_in.S <= 0) return hipSuccess;
  QkvGemmKernArgs a = a_in;
  a.n_row_tiles = (a.S + BM - 1) / BM;
  a.n_col_tiles = (a.Hq + 2 * a.Hkv + a.Hqx) / 2;
  const int lds = 4 * TILE + 1024;  // 129 KB of the CU's 160: above the default limit, asked for per launch (a host-side setting)
  hipError_t e = hipFuncSetAttribute((const void*)qkv_gemm_prologue_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return e;
  const int blocks = ((a.n_row_tiles + 7) / 8 + 7) / 8;  // blocks of 8 token tiles per XCD
  const unsigned grid = (unsigned)blocks * 8u * 8u * (unsigned)a.n_col_tiles;
  hipLaunchKernelGGL(qkv_gemm_prologue_kernel<2>, dim3(grid), dim3(512), lds, stream, a);
  return hipGetLastError();
}

}  // namespace magi
