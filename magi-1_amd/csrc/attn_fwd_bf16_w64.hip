// Range attention forward, bf16, 64 query rows per wavefront, for gfx950 (MI355X).
//
// Same mathematics and data path as attn_fwd_bf16.hip (S^T = K Q^T and O^T = V^T P^T on
// v_mfma_f32_32x32x16_bf16, K / V tiles of 64 keys double buffered in LDS by direct global->LDS loads, swizzled
// rows, transposing LDS reads for V^T), with one difference in the shape of a wave's work: a wave owns TWO
// blocks of 32 query rows (A = rows 0..31, B = rows 32..63 of its 64), so every K fragment and every V^T
// fragment read from LDS feeds two MFMAs instead of one.  That halves the LDS operand traffic per FLOP
// (0.5 KB per MFMA instead of 1 KB), which is what the 32-row kernels run out of: the transposing V^T reads
// alone need the full LDS bandwidth at the MFMA peak rate.
//
// The price is registers: Q 64 + O 128 + scores of one 32-key sub-tile 32 = 224 of the 256 a wave may hold at
// two waves per SIMD.  The key tile is therefore consumed in two 32-key halves (scores, softmax, PV for each),
// the probabilities overlay their score registers, and the operands come from LDS through ONE ring of four
// fragments that alternates between K and V^T fragments in the order the MFMAs consume them; the first V^T
// fragments of a half are on their way while its softmax runs.
//
// BOUNDED instantiation (MAGI_ATTN_BOUNDED_SCORES, needs pre-scaled q): the caller guarantees
// |q . k| <= score_bound (an exp2 exponent), small enough that 2^score neither overflows nor underflows in
// fp32 / bf16.  The softmax is shift invariant, so no running maximum is needed at all: p = 2^score, no row
// max, no rescale of O, no offset registers; the result is the same softmax.  QK-normed attention satisfies
// this by construction (|q| and |k| are fixed by the norm parameters).
#include "attn_common.h"

namespace magi {
namespace {

constexpr int ROW_BYTES = 256;  // D = 128 bf16
constexpr int BN = 64;          // keys per LDS tile
constexpr int TILE_BYTES = BN * ROW_BYTES;

// base ^ M computed where it is used.  The eight K and four V^T operand addresses of a lane differ by an XOR (the
// LDS swizzle), which no address-offset field can express; left to itself the compiler computes all twelve once
// and keeps them in registers across the tile loop, registers this kernel does not have.  The XOR is therefore
// written as inline assembly that also names a loop-variant scalar (`tie`, unused by the instruction) and a tag
// unique to the call site: the result can then be neither hoisted out of the tile loop nor shared between uses, and
// costs one v_xor per operand read.  (Not `asm volatile`: behind a volatile statement the compiler waits for ALL
// outstanding LDS reads instead of counting them.)
template <int M, int TAG>
__device__ __forceinline__ int swz(int base, int tie) {
  if constexpr (M == 0) return base;
  int r;
  asm("v_xor_b32 %0, %1, %2" : "=v"(r) : "n"(M), "v"(base), "s"(tie), "n"(TAG));
  return r;
}

// p in the lanes whose bit is set in the (wave-uniform) mask m, 0 elsewhere: v_cndmask reading the mask from a
// scalar register pair, so that masking the ragged end of a key range costs no vector registers
__device__ __forceinline__ float keep_lanes(float p, unsigned long long m) {
  float r;
  asm("v_cndmask_b32 %0, 0, %1, %2" : "=v"(r) : "v"(p), "s"(m));
  return r;
}

// WHATIF (tuning builds only, timing only: the results are wrong): parts of the bounded softmax left out, to measure
// what each costs.  1: no exponentials, 2: no row-sum additions.
template <int NW, int OCC, bool BOUNDED, int VPRE, int RD, bool PIPE = false, bool QNORM = false, int WHATIF = 0>
__global__ __launch_bounds__(64 * NW, OCC) void attn_fwd_bf16_w64_kernel(const AttnKernArgs a) {
  constexpr int BM = 64 * NW;
  constexpr int LW = 4;                 // waves that load tiles (the last LW of the workgroup)
  constexpr int LOADS = BN / (4 * LW);  // direct loads per loading wave per matrix per tile (4 rows each)
  static_assert(NW >= LW && NW % 4 == 0, "whole SIMD rounds of waves");
  // K and V double buffered in four separate LDS objects that are only named statically (an operand read then
  // never waits for the direct loads in flight to the other pair of slots)
  __shared__ __attribute__((aligned(1024))) unsigned char sK0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sK1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV1[TILE_BYTES];
  __shared__ int s_sel;

  const int tid = threadIdx.x;
  const WorkItem wi = locate_work(a, BM, tid, &s_sel);
  if (!wi.valid) return;
  const int qe = wi.qe, ks = wi.ks, ke = wi.ke;

  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, i = l & 31, g = l >> 5;
  const int row0 = wi.q0 + 64 * w;  // first row of this wave
  if (ke <= ks) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
      if (row0 + 32 * b + i < qe) store_empty_row(a, wi, row0 + 32 * b + i, g);
    return;
  }

  // ---- Q fragments (B operand of S^T = K Q^T): lane (i, g) holds Q[row][16kk + 8g .. +8] of both blocks ----
  bf16x8 qf[2][8];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int qr = min(row0 + 32 * b + i, qe - 1);
    const char* qp = a.q + (long)qr * a.qs_t + (long)wi.h * a.qs_h + g * 16;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[b][kk] = *(const bf16x8*)(qp + kk * 32);
  }
  if constexpr (QNORM) {
    // q holds the raw projection: per-(token, head) norm over the 128 features in fp32, times the softmax scale,
    // one rounding to bf16 (the cross-attention query norm, folded into this kernel's Q load).  A row's features
    // are spread over the lane pair (i, 0), (i, 1): 64 each, feature 16 kk + 8 g + e in fragment kk, element e.
    const float inv_d = 1.f / 128.f;
    float mean[2], rstd[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      float sum = 0.f;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += (float)qf[b][kk][e];
      sum += __shfl_xor(sum, 32);
      mean[b] = a.q_norm_kind == 0 ? sum * inv_d : 0.f;  // (RMS form: no centring)
      float sq = 0.f;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = (float)qf[b][kk][e] - mean[b];
          sq += d * d;
        }
      sq += __shfl_xor(sq, 32);
      rstd[b] = __builtin_amdgcn_rsqf(sq * inv_d + a.q_norm_eps) * a.scale_log2;
    }
    // (one fragment index at a time, so that the parameters of one fragment are all that is in registers)
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      __builtin_amdgcn_sched_barrier(0);
      const f32x4* gp = (const f32x4*)(a.q_norm_gamma + 16 * kk + 8 * g);
      const f32x4 g0 = gp[0], g1 = gp[1];
      f32x4 b0 = {0.f, 0.f, 0.f, 0.f}, b1 = b0;
      if (a.q_norm_beta) {
        const f32x4* bp = (const f32x4*)(a.q_norm_beta + 16 * kk + 8 * g);
        b0 = bp[0];
        b1 = bp[1];
      }
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float gm = (e < 4 ? g0[e & 3] : g1[e & 3]) + 1.f;
          const float bt = (e < 4 ? b0[e & 3] : b1[e & 3]) * a.scale_log2;
          qf[b][kk][e] = (__bf16)(((float)qf[b][kk][e] - mean[b]) * rstd[b] * gm + bt);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- K/V tile loader: loading wave wl fills rows 4*(wl + LW*j) .. +3; lane l sits at row +(l >> 4), slot l & 15 ----
  const int wl = w - (NW - LW);
  const long ks_t = a.ks_t, vs_t = a.vs_t;
  const int k_split = a.k_split;
  const long k2_delta = a.k2 ? (a.k2 - a.k) - (long)k_split * ks_t : 0;
  const long v2_delta = a.v2 ? (a.v2 - a.v) - (long)k_split * vs_t : 0;
  const char* const kcolp = a.k + (long)wi.kvh * a.ks_h;
  const char* const vcolp = a.v + (long)wi.kvh * a.vs_h;

  auto issue_mat = [&](int k0, unsigned char* tile_base, bool is_v) __attribute__((always_inline)) {
    if (NW > LW && wl < 0) return;  // (wave uniform) the other waves only consume
    unsigned char* dst = tile_base + wl * 1024;
    const long st = is_v ? vs_t : ks_t;
    const char* colp = is_v ? vcolp : kcolp;
    const long d2 = is_v ? v2_delta : k2_delta;
    // the lane geometry is re-derived from an opaque copy of the lane index at every call, so that nothing of it
    // occupies registers across the main loop
    int lane = l;
    asm volatile("" : "+v"(lane));
    const int lr = lane >> 4, sl = lane & 15;
    // logical 16-byte chunk that belongs at this lane's fixed LDS slot (K: c ^ (row & 15), V: c ^ ((row & 3) << 2))
    const int chunk = is_v ? (sl ^ (lr << 2)) : (sl ^ ((4 * (wl & 3) + lr) & 15));
    const bool interior = (k0 + BN <= ke) && (k0 + BN <= k_split || k0 >= k_split);
    if (interior) {
      // buffer-addressed direct loads: tile base in the resource descriptor, one 32-bit lane offset, the row
      // group of load j in the scalar offset
      const char* b = colp + (long)k0 * st + (k0 >= k_split ? d2 : 0);
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)b, 0, 0x7fffffff, 0x00020000);
      const unsigned voff = (unsigned)(4 * wl + lr) * (unsigned)st + (unsigned)(chunk * 16);
#pragma unroll
      for (int j = 0; j < LOADS; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, dst + j * LW * 1024), 16, voff,
                                                 (int)((unsigned)(4 * LW * j) * (unsigned)st), 0, 0);
    } else {
      // Ragged end of the range, or a tile that straddles the two key segments: per-lane rows, clamped to the last
      // valid key, each lane reading through the descriptor of the segment its row lives in.  Still buffer loads
      // (a global_load ... lds anywhere in the kernel counts as a possible FLAT access to LDS, after which the
      // compiler waits for ALL outstanding LDS reads in front of every MFMA instead of counting them).
      const char* b1 = colp + (long)k0 * st;  // row k0 of the first segment, of the second: (rows >= k_split only)
      const char* b2 = b1 + d2;
      const __amdgpu_buffer_rsrc_t rs1 = __builtin_amdgcn_make_buffer_rsrc((void*)b1, 0, 0x7fffffff, 0x00020000);
      const __amdgpu_buffer_rsrc_t rs2 = __builtin_amdgcn_make_buffer_rsrc((void*)b2, 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int j = 0; j < LOADS; ++j) {
        const int row = min(k0 + 4 * wl + lr + 4 * LW * j, ke - 1);
        const unsigned voff = (unsigned)(row - k0) * (unsigned)st + (unsigned)(chunk * 16);
        if (row < k_split)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs1, LDS_PTR(void, dst + j * LW * 1024), 16, voff, 0, 0, 0);
        else
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs2, LDS_PTR(void, dst + j * LW * 1024), 16, voff, 0, 0, 0);
      }
    }
  };

  // ---- per-lane LDS read bases ----
  // K as A operand: row = 32t + i, 16-byte chunk 2kk + g  ->  off = base_k ^ (kk << 5), + t * 32 rows
  const int base_k = i * ROW_BYTES + (((i & 15) ^ g) << 4);
  // V^T through the transposing read: 16-lane group q4 = l / 16 serves d block (q4 & 1), key group g;
  // inside it lane 4r + c points at row r, 8-byte column unit c.
  const int r4 = (l & 15) >> 2, c4 = l & 3, dblk = (l >> 4) & 1;
  const int base_v = (4 * g + r4) * ROW_BYTES + ((r4 << 6) | (dblk << 5) | (c4 << 3));

  f32x16 o_acc[2][4];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[b][mb][v] = 0.f;
  float m_run[2] = {-__builtin_inff(), -__builtin_inff()};  // running max of the raw scores (unused when BOUNDED)
  float l_run[2] = {0.f, 0.f};                               // this lane's share of the running sums
  const float c = a.scale_log2;
  const bool wave_on = row0 < qe;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  const int n_tiles = (ke - ks + BN - 1) / BN;

  // One 64-key tile for this wave.  The 32 operand fragments of a tile are consumed in this order:
  //   half t = 0, 1:  K(t, kk = 0..7)  [scores of 32 keys x 64 queries]   then   V^T(t, p = 0..7)  [PV of those keys]
  // each fragment feeding two MFMAs (block A, block B); fragment o is requested RD fragments ahead of its use.
  auto compute_tile = [&](const unsigned char* Kt, const unsigned char* Vt, int k0, auto ragged) __attribute__((always_inline)) {
    auto read_op = [&](auto oc) __attribute__((always_inline)) -> bf16x8 {
      constexpr int o = decltype(oc)::value;
      constexpr int t = o >> 4, j = o & 15;
      if constexpr (j < 8) {  // K rows 32t + i, features 16 j + 8 g .. +8
        return *LDS_PTR(const bf16x8, Kt + (swz<(j << 5), o>(base_k, k0) + t * 32 * ROW_BYTES));
      } else {      // V^T: 16-key slab s of half t, feature block mb
        constexpr int p = j - 8, s = 2 * t + (p >> 2), mb = p & 3;
        const int bv = swz<(mb << 6), o>(base_v, k0);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * s) * ROW_BYTES)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * s + 8) * ROW_BYTES)));
        const s16x8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, va);
      }
    };
    bf16x8 ring[RD];
    static_for<0, RD>([&](auto oc) __attribute__((always_inline)) { ring[decltype(oc)::value] = read_op(oc); });
    __builtin_amdgcn_sched_barrier(0);

    f32x16 sc[2];  // scores of the current half: [block][16 keys-per-lane]; later the packed probabilities
    static_for<0, 32>([&](auto oc) __attribute__((always_inline)) {
      constexpr int o = decltype(oc)::value;
      constexpr int t = o >> 4, j = o & 15;
      if constexpr (j == 8) {
        // ---- softmax of half t (32 keys x 64 queries: 16 + 16 values per lane, each lane one query per block) ----
        // Keys past the end of the range hold copies of the last valid row (the loader clamps), so their scores
        // are finite and the row maximum needs no mask; their probabilities are set to zero after the exp.
        const int kbase = k0 + 32 * t;
        auto softmax = [&](auto rc) __attribute__((always_inline)) {
          constexpr bool RAGGED = decltype(rc)::value;
          // register v of a lane holds key kbase + 8 (v / 4) + (v % 4) + 4 g (g = lane / 32): which of the two lane
          // halves keep their value is a scalar question per register
          const int left = ke - kbase;  // valid keys in this half (may be <= 0)
          auto prob = [&](float x, int v) __attribute__((always_inline)) -> float {
            const float p = (WHATIF & 1) ? x : __builtin_amdgcn_exp2f(x);
            if constexpr (RAGGED) {
              const int c0 = 8 * (v >> 2) + (v & 3);
              const unsigned long long m = (c0 < left ? 0x00000000ffffffffull : 0ull) | (c0 + 4 < left ? 0xffffffff00000000ull : 0ull);
              return keep_lanes(p, m);
            }
            return p;
          };
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            // Row sum of the probabilities in fp32, by plain additions.  (v_dot2c_f32_bf16 against (1, 1) would add a
            // packed pair in one instruction, but dot instructions do not execute beside an MFMA: each one holds
            // the matrix pipe up for about 16 cycles, measured, where exp2 / convert / add / fma run under it for
            // free.  Rounding to bf16 is unbiased, so the sum of the unrounded values is as good a denominator.)
            float psum = 0.f, psum2 = 0.f;
            if constexpr (BOUNDED) {
#pragma unroll
              for (int e = 0; e < 16; e += 2) {
                const float p0 = prob(sc[b][e], e), p1 = prob(sc[b][e + 1], e + 1);
                if constexpr (!(WHATIF & 2)) {
                  psum += p0;
                  psum2 += p1;
                }
                sc[b][8 * (e >> 3) + ((e & 7) >> 1)] = __builtin_bit_cast(float, pack_bf16x2(p0, p1));
              }
              l_run[b] += ((WHATIF & 2) ? 1.f : 0.f) + psum + psum2;
            } else {
              float mx = max3(sc[b][0], sc[b][1], sc[b][2]);
#pragma unroll
              for (int v = 3; v < 16; v += 2) mx = max3(mx, sc[b][v], sc[b][v + 1 < 16 ? v + 1 : v]);
              mx = half_swap_max(mx);
              const float m_new = fmaxf(m_run[b], mx);
              const float alpha = __builtin_amdgcn_exp2f((m_run[b] - m_new) * c);
              const float mc = m_new * c;
              m_run[b] = m_new;
#pragma unroll
              for (int e = 0; e < 16; e += 2) {
                const float p0 = prob(sc[b][e] * c - mc, e), p1 = prob(sc[b][e + 1] * c - mc, e + 1);
                psum += p0;
                psum2 += p1;
                sc[b][8 * (e >> 3) + ((e & 7) >> 1)] = __builtin_bit_cast(float, pack_bf16x2(p0, p1));
              }
              l_run[b] = l_run[b] * alpha + (psum + psum2);
              if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // some row of this block saw a new maximum
#pragma unroll
                for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                  for (int v = 0; v < 16; ++v) o_acc[b][mb][v] *= alpha;
              }
            }
          }
        };
        softmax(ragged);
        __builtin_amdgcn_sched_barrier(0);
        static_for<VPRE, RD>([&](auto pc) __attribute__((always_inline)) {
          constexpr int n = 16 * t + 8 + decltype(pc)::value;
          ring[n % RD] = read_op(std::integral_constant<int, n>{});
        });
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (j < 8) {
        // scores: S^T[key][q] += K[key][16 j ..] Q[q][16 j ..]
#pragma unroll
        for (int b = 0; b < 2; ++b)
          sc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[o % RD], qf[b][j], j == 0 ? zero16 : sc[b], 0, 0, 0);
      } else {
        // O^T[d][q] += V^T[d][key] P^T[key][q]; the packed probabilities of slab s sit in registers 8 s .. 8 s + 3
        constexpr int p = j - 8, s = p >> 2, mb = p & 3;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const f32x4 r = s ? __builtin_shufflevector(sc[b], sc[b], 8, 9, 10, 11) : __builtin_shufflevector(sc[b], sc[b], 0, 1, 2, 3);
          o_acc[b][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[o % RD], __builtin_bit_cast(bf16x8, r), o_acc[b][mb], 0, 0, 0);
        }
      }
      // refill the slot just consumed with the fragment RD ahead; of the first RD V^T fragments of a half only
      // VPRE are requested ahead of the softmax (they would occupy registers across it), the others right after it
      if constexpr (o + RD < 32) {
        constexpr int nj = (o + RD) & 15;
        if constexpr (!(nj >= 8 + VPRE && nj < 8 + RD)) ring[o % RD] = read_op(std::integral_constant<int, o + RD>{});
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  const int last = n_tiles - 1;
  if constexpr (PIPE) {
    // ---- software-pipelined main loop, ONE wave per SIMD (512 registers) ----
    // With a single wave on a SIMD nothing but the wave itself can fill the MFMA pipe while its own vector work
    // runs, so the three stages of consecutive tiles are interleaved instruction by instruction.  Step t issues,
    // in 64 slots of one MFMA each,
    //     slots  0..31   S(t+1) = K(t+1) Q^T        (16 K fragments x 2 row blocks)
    //     slots 32..63   O     += V(t-1)^T P(t-1)^T (16 V^T fragments x 2 row blocks)
    // and beside every MFMA one exp2, and every other slot one pack / one row-sum instruction, of softmax(t):
    // S(t) was finished by the MFMAs of step t-1 and P(t) is not needed before slot 32 of step t+1, so no
    // instruction of a slot waits for another one of the same slot.  Scores and probabilities alternate between
    // two register sets by the parity of t, the K / V tiles between two LDS slots each (K(t+1) and V(t-1) share
    // the parity t+1); the loop is unrolled by two so that registers and LDS slots are all named statically.
    // The pipelined loop takes a multiple of two tiles; the tiles in front of it (the last tile of the range,
    // which may be ragged, plus one more when the count is even) run the plain tile body above.
    static_assert(NW == 4 && OCC == 1 && BOUNDED, "pipelined loop: four waves, one per SIMD, bounded scores");
    constexpr int PRD = 6;  // operand fragments in flight between LDS and the MFMAs
    const int n_pipe = ((n_tiles - 1) / 2) * 2;
    const int n_peel = n_tiles - n_pipe;  // 1 or 2
    {
      // zero the V slots: the first pipelined step multiplies P(-1) = 0 with whatever the V slot of parity 1 holds,
      // which must be finite
      u32x4* z0 = (u32x4*)sV0;
      u32x4* z1 = (u32x4*)sV1;
#pragma unroll
      for (int r = 0; r < TILE_BYTES / (256 * 16); ++r) {
        z0[tid + 256 * r] = u32x4{0, 0, 0, 0};
        z1[tid + 256 * r] = u32x4{0, 0, 0, 0};
      }
      __syncthreads();
    }
    // peeled tiles: sequence s = 0 is tile `last`, s = 1 is tile 0; slot pair s & 1, chosen at run time
    issue_mat(ks + last * BN, sK0, false);
    issue_mat(ks + last * BN, sV0, true);
    for (int s = 0; s < n_peel; ++s) {
      wait_vmcnt<0>();
      __syncthreads();
      if (s + 1 < n_peel) {
        issue_mat(ks, sK1, false);
        issue_mat(ks, sV1, true);
      }
      if (wave_on) compute_tile(s ? sK1 : sK0, s ? sV1 : sV0, s ? ks : ks + last * BN, std::true_type{});
    }
    if (n_pipe > 0) {
      // pipelined tile t is tile n_peel - 1 + t of the range
      const int kp = ks + (n_peel - 1) * BN;
      f32x16 Sb[2][4];  // scores [parity][half * 2 + row block]
      u32x4 Pb[2][8];   // packed probabilities [parity][(half * 2 + slab) * 2 + row block]
      float psum[2] = {0.f, 0.f};
#pragma unroll
      for (int f = 0; f < 8; ++f) Pb[1][f] = u32x4{0, 0, 0, 0};
      __syncthreads();  // the peeled tiles have been read by everybody
      issue_mat(kp, sK0, false);
      issue_mat(kp + BN, sK1, false);

      // Q once more, as values born in accumulation registers (the score MFMAs read them there)
      u32x4 qa[2][8];
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
          const u32x4 t = __builtin_bit_cast(u32x4, qf[b][kk]);
          asm volatile("v_accvgpr_write_b32 %0, %4\n\tv_accvgpr_write_b32 %1, %5\n\tv_accvgpr_write_b32 %2, %6\n\tv_accvgpr_write_b32 %3, %7"
                       : "=a"(qa[b][kk][0]), "=a"(qa[b][kk][1]), "=a"(qa[b][kk][2]), "=a"(qa[b][kk][3])
                       : "v"(t[0]), "v"(t[1]), "v"(t[2]), "v"(t[3]));
        }
      // operand fragment o of a step: o < 16: K(half o / 8, features 16 (o % 8) ..) from Kt; else V^T(slab (o-16) / 4,
      // feature block (o-16) % 4) from Vt
      auto read_frag = [&](const unsigned char* Kt, const unsigned char* Vt, auto oc) __attribute__((always_inline)) -> bf16x8 {
        constexpr int o = decltype(oc)::value;
        if constexpr (o < 16) {
          constexpr int h = o >> 3, kk = o & 7;
          return *LDS_PTR(const bf16x8, Kt + ((base_k ^ (kk << 5)) + h * 32 * ROW_BYTES));
        } else {
          constexpr int p = o - 16, sg = p >> 2, mb = p & 3;
          const int bv = base_v ^ (mb << 6);
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * sg) * ROW_BYTES)));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * sg + 8) * ROW_BYTES)));
          const s16x8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          return __builtin_bit_cast(bf16x8, va);
        }
      };
      // the MFMA of slot sl: scores into Sn, or P V into the accumulators from Po
      auto mfma_slot = [&](auto slc, const bf16x8& frag, f32x16 (&Sn)[4], const u32x4 (&Po)[8]) __attribute__((always_inline)) {
        constexpr int sl = decltype(slc)::value;
        constexpr int o = sl >> 1, b = sl & 1;
        if constexpr (o < 16) {
          constexpr int h = o >> 3, kk = o & 7;
          // Score MFMAs through inline assembly, to choose their register files: at one wave per SIMD the
          // compiler gives every MFMA it selects itself an accumulator in the accumulation half of the register file
          // (right for O, which only MFMAs touch) and would then copy the scores, 64 registers per tile, to the
          // vector half for the softmax.  Here the scores are written to vector registers directly and Q is read
          // from accumulation registers.  The compiler does not see that these statements are MFMAs, which is safe
          // because a score register is next touched a whole pipeline step (32 MFMAs) later, and consecutive MFMAs
          // onto one accumulator are interlocked by the hardware.
          const u32x4 qv = qa[b][kk];
          if constexpr (kk == 0)
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(Sn[h * 2 + b]) : "v"(frag), "a"(qv));
          else
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(Sn[h * 2 + b]) : "v"(frag), "a"(qv));
        } else {
          constexpr int p = o - 16, sg = p >> 2, mb = p & 3;
          // (likewise: O in accumulation registers, V^T and P in vector registers)
          f32x16& acc = o_acc[b][mb];
          const u32x4 pv = Po[sg * 2 + b];
          asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(frag), "v"(pv));
        }
      };
      // softmax micro-operations of a step, numbered by the slot they ride in.  Element e = 0..63 of the lane:
      // score vector e / 16 (= half * 2 + row block), register e % 16; its exp2 runs in slot e, the pack of the
      // pair (e - 1, e) three slots after its second exp2, next to the additions of the two values to the row sum.
      auto pair_ops = [&](auto pc, auto kc, const float (&ex)[64], u32x4 (&Pn)[8]) __attribute__((always_inline)) {
        constexpr int pr = decltype(pc)::value;  // pair 0..31
        constexpr int k = decltype(kc)::value;   // 0: pack, 1: row sum
        constexpr int vi = pr >> 3, q = pr & 7, h = vi >> 1, b = vi & 1, slab = q >> 2;
        constexpr int f = (h * 2 + slab) * 2 + b;
        if constexpr (k == 0) Pn[f][q & 3] = pack_bf16x2(ex[2 * pr], ex[2 * pr + 1]);
        if constexpr (k == 1) psum[b] += ex[2 * pr];
        if constexpr (k == 2) psum[b] += ex[2 * pr + 1];
      };
      auto step = [&](int t, auto parc) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
        wait_vmcnt<0>();
        __syncthreads();  // K(t+1) and V(t-1) are in LDS for everybody; the slots of K(t) and V(t-2) are free
        if (t + 2 < n_pipe) issue_mat(kp + (t + 2) * BN, PAR ? sK1 : sK0, false);
        issue_mat(kp + t * BN, PAR ? sV1 : sV0, true);
        if (!wave_on) return;
        const unsigned char* Kt = PAR ? sK0 : sK1;  // K(t+1)
        const unsigned char* Vt = PAR ? sV0 : sV1;  // V(t-1)
        f32x16 (&Sc)[4] = Sb[PAR];
        f32x16 (&Sn)[4] = Sb[PAR ^ 1];
        u32x4 (&Pn)[8] = Pb[PAR];
        const u32x4 (&Po)[8] = Pb[PAR ^ 1];
        bf16x8 ring[PRD];
        float ex[64];  // exp2 of the scores, each alive for the few slots until its pair is packed
        static_for<0, PRD>([&](auto oc) __attribute__((always_inline)) { ring[decltype(oc)::value] = read_frag(Kt, Vt, oc); });
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, 64>([&](auto slc) __attribute__((always_inline)) {
          constexpr int sl = decltype(slc)::value;
          constexpr int o = sl >> 1;
          mfma_slot(slc, ring[o % PRD], Sn, Po);
          if constexpr ((sl & 1) && o + PRD < 32) ring[o % PRD] = read_frag(Kt, Vt, std::integral_constant<int, o + PRD>{});
          ex[sl] = __builtin_amdgcn_exp2f(Sc[sl >> 4][sl & 15]);
          if constexpr ((sl & 1) == 0 && sl >= 4) pair_ops(std::integral_constant<int, (sl - 4) / 2>{}, std::integral_constant<int, 0>{}, ex, Pn);
          if constexpr ((sl & 1) == 0 && sl >= 4) pair_ops(std::integral_constant<int, (sl - 4) / 2>{}, std::integral_constant<int, 1>{}, ex, Pn);
          if constexpr ((sl & 1) == 1 && sl >= 5) pair_ops(std::integral_constant<int, (sl - 5) / 2>{}, std::integral_constant<int, 2>{}, ex, Pn);
          __builtin_amdgcn_sched_barrier(0);
        });
        // pairs 30 and 31 finish after the last slot
        pair_ops(std::integral_constant<int, 30>{}, std::integral_constant<int, 0>{}, ex, Pn);
        pair_ops(std::integral_constant<int, 31>{}, std::integral_constant<int, 0>{}, ex, Pn);
        pair_ops(std::integral_constant<int, 30>{}, std::integral_constant<int, 1>{}, ex, Pn);
        pair_ops(std::integral_constant<int, 31>{}, std::integral_constant<int, 1>{}, ex, Pn);
        pair_ops(std::integral_constant<int, 30>{}, std::integral_constant<int, 2>{}, ex, Pn);
        pair_ops(std::integral_constant<int, 31>{}, std::integral_constant<int, 2>{}, ex, Pn);
        __builtin_amdgcn_sched_barrier(0);
      };
      // fill: S(0) = K(0) Q^T
      wait_vmcnt<0>();
      __syncthreads();
      if (wave_on) {
        bf16x8 ring[PRD];
        static_for<0, PRD>([&](auto oc) __attribute__((always_inline)) { ring[decltype(oc)::value] = read_frag(sK0, sV0, oc); });
        static_for<0, 32>([&](auto slc) __attribute__((always_inline)) {
          constexpr int sl = decltype(slc)::value;
          constexpr int o = sl >> 1;
          mfma_slot(slc, ring[o % PRD], Sb[0], Pb[1]);
          if constexpr ((sl & 1) && o + PRD < 16) ring[o % PRD] = read_frag(sK0, sV0, std::integral_constant<int, o + PRD>{});
          __builtin_amdgcn_sched_barrier(0);
        });
      }
      for (int t = 0; t < n_pipe; t += 2) {
        step(t, std::integral_constant<int, 0>{});
        step(t + 1, std::integral_constant<int, 1>{});
      }
      // drain: O += V(n_pipe-1)^T P(n_pipe-1)^T  (parity 1)
      wait_vmcnt<0>();
      __syncthreads();
      if (wave_on) {
        bf16x8 ring[PRD];
        static_for<0, PRD>([&](auto oc) __attribute__((always_inline)) {
          ring[decltype(oc)::value] = read_frag(sK1, sV1, std::integral_constant<int, 16 + decltype(oc)::value>{});
        });
        static_for<32, 64>([&](auto slc) __attribute__((always_inline)) {
          constexpr int sl = decltype(slc)::value;
          constexpr int o = sl >> 1;
          mfma_slot(slc, ring[(o - 16) % PRD], Sb[0], Pb[1]);
          if constexpr ((sl & 1) && o + PRD < 32) ring[(o - 16) % PRD] = read_frag(sK1, sV1, std::integral_constant<int, o + PRD>{});
          __builtin_amdgcn_sched_barrier(0);
        });
        l_run[0] += psum[0];
        l_run[1] += psum[1];
        // the epilogue reads the accumulators with vector instructions, and the compiler has not seen the MFMAs above:
        // let the last of them (8 passes of 4 cycles, then write-back) retire first
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
  // Tile order: the LAST tile of the key range first (it may hold the ragged end, so it runs the copy of the tile
  // body that masks the tail; the order of keys is immaterial to a softmax), then tiles 0 .. n_tiles-2 with the
  // mask-free body, two per loop iteration so that every LDS slot is named statically.  Tile `last` uses slot
  // pair 0, tile j slot pair (j + 1) & 1.
  const std::integral_constant<int, 0> slot0;
  const std::integral_constant<int, 1> slot1;
  issue_mat(ks + last * BN, sK0, false);
  issue_mat(ks + last * BN, sV0, true);
  // one tile: wait for it, request the next one (tile `nxt` of the range, if any) into the other slot pair, compute
  auto step = [&](int cur, int nxt, auto sc_, auto ragged) __attribute__((always_inline)) {
    constexpr int B = decltype(sc_)::value;
    wait_vmcnt<0>();
    __syncthreads();  // the tile landed in everybody's view; the other slot pair is free
    if (nxt < last) {
      issue_mat(ks + nxt * BN, B ? sK0 : sK1, false);
      issue_mat(ks + nxt * BN, B ? sV0 : sV1, true);
    }
    if (!wave_on) return;
    compute_tile(B ? sK1 : sK0, B ? sV1 : sV0, ks + cur * BN, ragged);
  };
  step(last, 0, slot0, std::true_type{});
  int j = 0;
  for (; j + 1 < last; j += 2) {
    step(j, j + 1, slot1, std::false_type{});
    step(j + 1, j + 2, slot0, std::false_type{});
  }
  if (j < last) step(j, j + 1, slot1, std::false_type{});

  }  // !PIPE

  if (!wave_on) return;
  // ---- epilogue: normalise and store ----
  // A lane holds four consecutive features per (mb, quad), its partner in the other half wave the next four: the
  // halves trade registers so that every lane owns eight consecutive features and stores 16 bytes at a time.
  int lane_e = l;
  asm volatile("" : "+v"(lane_e));
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const float l_tot = l_run[b] + __shfl_xor(l_run[b], 32);
    const float inv = 1.f / l_tot;
    const int q_row = row0 + 32 * b + (lane_e & 31);
    const bool row_ok = q_row < qe;
    char* const op = a.out + (long)q_row * a.os_t + wi.o_head + 16 * (lane_e >> 5);
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int bp = 0; bp < 2; ++bp) {
        unsigned ev[2], od[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          ev[e] = pack_bf16x2(o_acc[b][mb][8 * bp + 2 * e] * inv, o_acc[b][mb][8 * bp + 2 * e + 1] * inv);
          od[e] = pack_bf16x2(o_acc[b][mb][8 * bp + 4 + 2 * e] * inv, o_acc[b][mb][8 * bp + 4 + 2 * e + 1] * inv);
          half_swap(ev[e], od[e]);  // lower half: (own even, partner's even); upper half: (partner's odd, own odd)
        }
        if (row_ok) *(u32x4*)(op + (32 * mb + 16 * bp) * 2) = u32x4{ev[0], ev[1], od[0], od[1]};
      }
    if (row_ok && a.lse && (lane_e >> 5) == 0)
      a.lse[(long)wi.h * a.total_q + q_row] =
          ((BOUNDED ? 0.f : m_run[b] * c) + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  }
}

}  // namespace

hipError_t launch_attn_fwd_bf16_w64(const AttnKernArgs& a, hipStream_t stream) {
  const unsigned grid = a.per_xcd * 8u;
  [[maybe_unused]] const bool bounded = (a.flags & ATTN_BOUNDED) != 0;
#ifdef MAGI_TUNING  // (tuning builds can also run the 64-row kernels with the running maximum: slower, it spills)
#define MAGI_W64_LAUNCH(NW, OCC, VPRE, RD)                                                                              \
  do {                                                                                                                   \
    if (bounded)                                                                                                         \
      hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<NW, OCC, true, VPRE, RD>), dim3(grid), dim3(64 * NW), 0, stream, a);  \
    else                                                                                                                 \
      hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<NW, OCC, false, VPRE, RD>), dim3(grid), dim3(64 * NW), 0, stream, a); \
  } while (0)
#else
#define MAGI_W64_LAUNCH(NW, OCC, VPRE, RD) \
  hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<NW, OCC, true, VPRE, RD>), dim3(grid), dim3(64 * NW), 0, stream, a)
#endif
#ifdef MAGI_TUNING
  if (a.variant >= 101 && a.variant <= 103 && bounded) {  // MAGI_ATTN_VARIANT = 100 + WHATIF
    if (a.variant == 101) hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 2, true, 0, 4, false, false, 1>), dim3(grid), dim3(256), 0, stream, a);
    if (a.variant == 102) hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 2, true, 0, 4, false, false, 2>), dim3(grid), dim3(256), 0, stream, a);
    if (a.variant == 103) hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 2, true, 0, 4, false, false, 3>), dim3(grid), dim3(256), 0, stream, a);
  } else if (a.variant == 20)  // software-pipelined loop, one wave per SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 1, true, 0, 4, true>), dim3(grid), dim3(256), 0, stream, a);
  else if (a.block_m == 512 && a.variant == 12)
    MAGI_W64_LAUNCH(8, 1, 0, 2);
  else if (a.variant == 12)
    MAGI_W64_LAUNCH(4, 2, 0, 2);
  else
#endif
  if (a.q_norm_gamma)  // raw q, normalised while it is loaded (cross attention)
    hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 2, true, 0, 4, false, true>), dim3(grid), dim3(256), 0, stream, a);
  else if (a.block_m == 512)  // 8 waves, one workgroup per CU: every K / V tile fetched once for 512 rows
    MAGI_W64_LAUNCH(8, 1, 0, 4);
  else  // 4 waves, two workgroups per CU
    MAGI_W64_LAUNCH(4, 2, 0, 4);
#undef MAGI_W64_LAUNCH
  return hipGetLastError();
}

}  // namespace magi
