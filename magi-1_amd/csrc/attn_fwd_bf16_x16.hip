// Range attention forward, bf16, bounded scores, 64 query rows per wavefront on v_mfma_f32_16x16x32_bf16,
// for gfx950 (MI355X).
//
// Same algorithm, tile loop and LDS staging as attn_fwd_bf16_w64.hip (S^T = K Q^T and O^T = V^T P^T, p = 2^score
// without a running maximum, K / V tiles of 64 keys double buffered in LDS by direct global->LDS loads, transposing
// LDS reads for V^T), on the other bf16 MFMA shape.  Why: this part runs at its board power limit, and a
// 16x16x32 MFMA spends less energy per FLOP than a 32x32x16 one (it sums 32 products into each accumulator element
// instead of 16, so half as many fp32 accumulator reads and writes per FLOP): an MFMA-only loop on random operands
// holds ~14 % more FLOP/s at the limit with this shape, measured on the same box.
//
// Shape of a wave's work.  A wave owns 64 query rows as FOUR blocks of 16 (qb).  Lane l = (n = l % 16, g = l / 16):
//   S^T block (16 keys x 16 queries) = K[16 keys x 32 d] Q^T[32 d x 16 queries], accumulated over 4 d steps (kk):
//       A = K fragment : lane holds K[key n][d = 32 kk + 8 g .. +8]          (one ds_read_b128, 1 KB per wave)
//       B = Q fragment : lane holds Q[query n][d = 32 kk + 8 g .. +8]        (registers, 64 in all)
//       D             : lane holds S^T[key 4 g + r][query n], r = 0..3
//     every K fragment feeds the four query blocks: 4 MFMAs per 1 KB read from LDS, the same bytes per FLOP as the
//     32x32x16 kernel's two.
//   O^T block (16 d x 16 queries) += V^T[16 d x 32 keys] P^T[32 keys x 16 queries]:
//       B = P fragment : lane holds the probabilities of query n for 8 keys; the D layout above hands a lane keys
//                        4 g + r of each 16-key block, so the 32 keys of a step are two key blocks (kb = 0, 1) and
//                        operand element e is key 16 (e / 4) + 4 g + e % 4: two S^T accumulators, packed, no
//                        lane exchange
//       A = V^T fragment: lane holds V[those 8 keys][d = 16 db + n]: two transposing reads (ds_read_b64_tr_b16),
//                        one per key block; feeds the four query blocks
//       D             : lane holds O^T[d = 16 db + 4 g + r][query n]
// Registers: Q 64 + O 128 + the scores of one 32-key half tile 32 + a ring of four operand fragments 16.
//
// The epilogue goes through LDS (the tile slots are free by then): every wave writes its 64 x 128 normalised
// outputs as bf16 rows and reads them back 16 bytes per lane, so that 16 consecutive lanes store one whole 256-byte
// row: every global store instruction writes four complete rows.
#include "attn_common.h"

namespace magi {
namespace {

constexpr int ROW_BYTES = 256;  // D = 128 bf16
constexpr int BN = 64;          // keys per LDS tile
// A tile in LDS is 16 groups of four rows (what one wave-wide direct load fills: 64 lanes x 16 bytes).  The groups are
// spaced by a little more than their 1024 bytes, so that consecutive groups start in different banks and the operand
// reads need no address arithmetic beyond constant offsets (see the read bases below).
constexpr int K_GROUP = 1024 + 64, V_GROUP = 1024 + 128;
constexpr int K_TILE_BYTES = (BN / 4) * K_GROUP, V_TILE_BYTES = (BN / 4) * V_GROUP;

typedef float f32x4v __attribute__((ext_vector_type(4)));

// base ^ M computed where it is used (one v_xor per operand read instead of a register per address across the tile
// loop): inline assembly that also names a loop-variant scalar (`tie`, unused by the instruction) and a tag unique
// to the call site, so that the result is neither hoisted out of the loop nor shared.  Not `asm volatile`: behind a
// volatile statement the compiler waits for ALL outstanding LDS reads instead of counting them.
template <int M, int TAG>
__device__ __forceinline__ int swz(int base, int tie) {
  if constexpr (M == 0) return base;
  int r;
  asm("v_xor_b32 %0, %1, %2" : "=v"(r) : "n"(M), "v"(base), "s"(tie), "n"(TAG));
  return r;
}

// QMODE: what q holds.  0: q as the score MFMAs take it (pre-scaled by the caller).  1: the raw query projection:
// per-(token, head) norm in fp32 while it is loaded, times the softmax scale, one rounding to bf16.  2: unscaled
// bf16 q as the reference's callers pass it: multiplied by the softmax scale while it is loaded (a second rounding
// to bf16: 2^-9 relative per element, the size of the first).
// order in which the feature blocks of V^T are visited: 0, 4, 1, 5, 2, 6, 3, 7
constexpr int v_block(int i) { return (i >> 1) + 4 * (i & 1); }

constexpr int Q_AS_IS = 0, Q_NORM = 1, Q_SCALE = 2;

template <int QMODE>
__global__ __launch_bounds__(256, 2) void attn_fwd_bf16_x16_kernel(const AttnKernArgs a) {
  constexpr int NW = 4, BM = 64 * NW;
  constexpr int LOADS = BN / (4 * NW);  // direct loads per wave per matrix per tile (4 rows each)
  constexpr int RING = 4;               // operand fragments in flight between LDS and the MFMAs
  // K and V double buffered in four separate LDS objects that are only named statically (an operand read then
  // never waits for the direct loads in flight to the other pair of slots)
  __shared__ __attribute__((aligned(1024))) unsigned char sK0[K_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV0[V_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sK1[K_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV1[V_TILE_BYTES];
  __shared__ int s_sel[LOCATE_WORDS];

  if (gate_closed(a)) return;
  const int tid = threadIdx.x;
  const WorkItem wi = locate_work(a, BM, tid, s_sel);
  if (!wi.valid) return;
  const int qe = wi.qe, ks = wi.ks, ke = wi.ke;

  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, n = l & 15, g = l >> 4;
  const int row0 = wi.q0 + 64 * w;  // first row of this wave
  if (ke <= ks) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
      if (row0 + 32 * b + (l & 31) < qe) store_empty_row(a, wi, row0 + 32 * b + (l & 31), l >> 5);
    return;
  }

  // ---- K/V tile loader: wave w fills rows 4 * (w + 4 j) .. +3; lane l sits at row +(l >> 4), slot l & 15 ----
  const long ks_t = a.ks_t, vs_t = a.vs_t;
  const int k_split = a.k_split;
  const long k2_delta = a.k2 ? (a.k2 - a.k) - (long)k_split * ks_t : 0;
  const long v2_delta = a.v2 ? (a.v2 - a.v) - (long)k_split * vs_t : 0;
  const char* const kcolp = a.k + (long)wi.kvh * a.ks_h;
  const char* const vcolp = a.v + (long)wi.kvh * a.vs_h;

  auto issue_mat = [&](int k0, unsigned char* tile_base, bool is_v) __attribute__((always_inline)) {
    const int group = is_v ? V_GROUP : K_GROUP;
    unsigned char* dst = tile_base + w * group;
    const long st = is_v ? vs_t : ks_t;
    const char* colp = is_v ? vcolp : kcolp;
    const long d2 = is_v ? v2_delta : k2_delta;
    // the lane geometry is re-derived from an opaque copy of the lane index at every call, so that nothing of it
    // occupies registers across the main loop
    int lane = l;
    asm volatile("" : "+v"(lane));
    const int lr = lane >> 4, sl = lane & 15;
    // logical 16-byte chunk that belongs at this lane's fixed LDS slot.  Row r of a tile (row r & 3 = lr of its
    // group) keeps chunk c at
    //   K: c ^ (r & 3)         (ds_read_b128 down 16 rows: four groups 64 bytes apart x four chunks)
    //   V: c ^ ((r & 3) << 1)  (transposing reads of 32 bytes from each of 8 rows: two groups 128 bytes apart x
    //                           four 32-byte slots)
    const int chunk = is_v ? (sl ^ (lr << 1)) : (sl ^ lr);
    const bool interior = (k0 + BN <= ke) && (k0 + BN <= k_split || k0 >= k_split);
    if (interior) {
      // buffer-addressed direct loads: tile base in the resource descriptor, one 32-bit lane offset, the row
      // group of load j in the scalar offset
      const char* b = colp + (long)k0 * st + (k0 >= k_split ? d2 : 0);
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)b, 0, 0x7fffffff, 0x00020000);
      const unsigned voff = (unsigned)(4 * w + lr) * (unsigned)st + (unsigned)(chunk * 16);
#pragma unroll
      for (int j = 0; j < LOADS; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, dst + j * NW * group), 16, voff,
                                                 (int)((unsigned)(4 * NW * j) * (unsigned)st), 0, 0);
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
        const int row = min(k0 + 4 * w + lr + 4 * NW * j, ke - 1);
        const unsigned voff = (unsigned)(row - k0) * (unsigned)st + (unsigned)(chunk * 16);
        if (row < k_split)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs1, LDS_PTR(void, dst + j * NW * group), 16, voff, 0, 0, 0);
        else
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs2, LDS_PTR(void, dst + j * NW * group), 16, voff, 0, 0, 0);
      }
    }
  };

  // The first tile (the LAST one of the key range, see below) is requested before q is loaded and normalised, so that
  // the two latencies overlap: it matters where a workgroup sees few tiles (the text cross attention).
  const int n_tiles = (ke - ks + BN - 1) / BN;
  const int last = n_tiles - 1;
  issue_mat(ks + last * BN, sK0, false);
  issue_mat(ks + last * BN, sV0, true);

  // ---- Q fragments (B operand of S^T = K Q^T): lane (n, g) holds Q[row 16 qb + n][32 kk + 8 g .. +8] ----
  bf16x8 qf[4][4];
#pragma unroll
  for (int qb = 0; qb < 4; ++qb) {
    const int qr = min(row0 + 16 * qb + n, qe - 1);
    const char* qp = a.q + (long)qr * a.qs_t + (long)wi.h * a.qs_h + g * 16;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) qf[qb][kk] = *(const bf16x8*)(qp + kk * 64);
  }
  if constexpr (QMODE == Q_SCALE) {
    const float cs = a.scale_log2;
#pragma unroll
    for (int qb = 0; qb < 4; ++qb)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[qb][kk][e] = (__bf16)((float)qf[qb][kk][e] * cs);
  }
  if constexpr (QMODE == Q_NORM) {
    // q holds the raw projection: per-(token, head) norm over the 128 features in fp32, times the softmax scale,
    // one rounding to bf16.  A row's features are spread over the four lanes (n, 0..3): 32 each, feature
    // 32 kk + 8 g + e in fragment kk, element e.
    const float inv_d = 1.f / 128.f;
    float mean[4], rstd[4];
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
      float sum = 0.f;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += (float)qf[qb][kk][e];
      sum += __shfl_xor(sum, 16);
      sum += __shfl_xor(sum, 32);
      mean[qb] = a.q_norm_kind == 0 ? sum * inv_d : 0.f;  // (RMS form: no centring)
      float sq = 0.f;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = (float)qf[qb][kk][e] - mean[qb];
          sq += d * d;
        }
      sq += __shfl_xor(sq, 16);
      sq += __shfl_xor(sq, 32);
      rstd[qb] = __builtin_amdgcn_rsqf(sq * inv_d + a.q_norm_eps) * a.scale_log2;
    }
    // (one fragment index at a time, so that the parameters of one fragment are all that is in registers)
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      __builtin_amdgcn_sched_barrier(0);
      const f32x4* gp = (const f32x4*)(a.q_norm_gamma + 32 * kk + 8 * g);
      const f32x4 g0 = gp[0], g1 = gp[1];
      f32x4 b0 = {0.f, 0.f, 0.f, 0.f}, b1 = b0;
      if (a.q_norm_beta) {
        const f32x4* bp = (const f32x4*)(a.q_norm_beta + 32 * kk + 8 * g);
        b0 = bp[0];
        b1 = bp[1];
      }
#pragma unroll
      for (int qb = 0; qb < 4; ++qb)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float gm = (e < 4 ? g0[e & 3] : g1[e & 3]) + 1.f;
          const float bt = (e < 4 ? b0[e & 3] : b1[e & 3]) * a.scale_log2;
          qf[qb][kk][e] = (__bf16)(((float)qf[qb][kk][e] - mean[qb]) * rstd[qb] * gm + bt);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- per-lane LDS read bases ----
  // K as A operand: row 16 kb + n, 16-byte chunk 4 kk + g, kept at (4 kk + g) ^ (n & 3) = 4 kk + (g ^ (n & 3)) of row
  // n & 3 of group 4 kb + n / 4: everything but the lane's own part is a constant offset of the read.  The 16 lanes
  // of one g touch four groups (64 bytes apart in bank terms) x four chunks: all 64 banks once.
  const int base_k = (n >> 2) * K_GROUP + (n & 3) * ROW_BYTES + ((g ^ (n & 3)) << 4);
  // V^T through the transposing read: the 16-lane group g serves key rows 4 g + r4 (r4 = (l % 16) / 4) of a 16-key
  // block, i.e. row r4 of group g (+ 4 per key block); lane 4 r4 + c4 of the group points at the four features
  // 16 db + 4 c4 .. +3 of its row, and receives the four rows' values of feature 16 db + l % 16.  Those 32 bytes of
  // the row are 32-byte slot db, kept at db ^ r4 = 4 (db / 4) + ((db % 4) ^ r4): one v_xor per value of db % 4,
  // the rest constant offsets.  Half a wave touches two groups (128 bytes apart in bank terms) x four slots x 32 bytes.
  const int r4 = n >> 2, c4 = n & 3;
  const int base_v = g * V_GROUP + r4 * ROW_BYTES + (r4 << 5) + (c4 << 3);

  f32x4v o_acc[8][4];  // [d block][query block]; zeroed below, right ahead of the first tile
  float l_run[4] = {0.f, 0.f, 0.f, 0.f};  // this lane's share of the row sums, per query block
  const bool wave_on = row0 < qe;
  const f32x4v zero4 = {0.f, 0.f, 0.f, 0.f};

  // One 64-key tile for this wave.  The 32 operand fragments of a tile are consumed in this order:
  //   half t = 0, 1:  K(t, kb = 0..1, kk = 0..3)  [scores of 32 keys x 64 queries]   then   V^T(t, db = 0, 4, 1, 5,
  //   2, 6, 3, 7: the two of a pair share their address)
  // each fragment feeding four MFMAs (the query blocks); fragment o is requested RD fragments ahead of its use.
  auto compute_tile = [&](const unsigned char* Kt, const unsigned char* Vt, int k0, auto ragged) __attribute__((always_inline)) {
    auto read_op = [&](auto oc) __attribute__((always_inline)) -> bf16x8 {
      constexpr int o = decltype(oc)::value;
      constexpr int t = o >> 4, j = o & 15;
      if constexpr (j < 8) {  // K rows 32 t + 16 kb + n, features 32 kk + 8 g .. +8
        constexpr int kb = j >> 2, kk = j & 3;
        return *LDS_PTR(const bf16x8, Kt + (base_k + kk * 64 + (8 * t + 4 * kb) * K_GROUP));
      } else {  // V^T: feature block db, the two 16-key blocks of half t
        constexpr int db = v_block(j - 8);
        const int bv = swz<((db & 3) << 5), 16 * t + (db & 3)>(base_v, k0) + (db >> 2) * 128;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (8 * t) * V_GROUP)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (8 * t + 4) * V_GROUP)));
        const s16x8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, va);
      }
    };
    constexpr int RD = RING;
    bf16x8 ring[RD];
    static_for<0, RD>([&](auto oc) __attribute__((always_inline)) { ring[decltype(oc)::value] = read_op(oc); });
    __builtin_amdgcn_sched_barrier(0);

    f32x4v sc[2][4];  // scores of the current half: [key block][query block]
    u32x4 pf[4];      // their probabilities as the B operand of the PV MFMAs, per query block
    auto consume = [&](auto oc) __attribute__((always_inline)) {
      constexpr int o = decltype(oc)::value;
      constexpr int t = o >> 4, j = o & 15;
      // ---- softmax of half t (32 keys x 64 queries: 32 values per lane, one query per lane and query block), one
      // (key block, query block) piece at a time: four exponentials, their sum, two packed pairs of the P operand.
      // (Keys past the end of the range need nothing here: their scores start from a large negative value, see below.)
      auto soft = [&](auto kc, auto qc) __attribute__((always_inline)) {
        constexpr int kb = decltype(kc)::value, qb = decltype(qc)::value;
        // Row sums in fp32 by plain additions on the unrounded values (rounding to bf16 is unbiased, so this is as
        // good a denominator; dot instructions would hold the matrix pipe up)
        const float p0 = __builtin_amdgcn_exp2f(sc[kb][qb][0]), p1 = __builtin_amdgcn_exp2f(sc[kb][qb][1]);
        const float p2 = __builtin_amdgcn_exp2f(sc[kb][qb][2]), p3 = __builtin_amdgcn_exp2f(sc[kb][qb][3]);
        l_run[qb] += (p0 + p1) + (p2 + p3);
        pf[qb][2 * kb] = pack_bf16x2(p0, p1);
        pf[qb][2 * kb + 1] = pack_bf16x2(p2, p3);
      };
      if constexpr (j == 8) {
        static_for<0, 4>([&](auto qc) __attribute__((always_inline)) {
          soft(std::integral_constant<int, 0>{}, qc);
          soft(std::integral_constant<int, 1>{}, qc);
        });
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, RD>([&](auto pc) __attribute__((always_inline)) {
          constexpr int nf = 16 * t + 8 + decltype(pc)::value;
          ring[nf % RD] = read_op(std::integral_constant<int, nf>{});
        });
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (j < 8) {
        // scores: S^T[key][q] += K[key][32 kk ..] Q[q][32 kk ..]
        constexpr int kb = j >> 2, kk = j & 3;
        // The accumulators of a key block start from 0.  In the ragged copy of the body, keys past the end of the
        // range (whose LDS rows hold copies of the last valid key: the loader clamps) start from -1e4 instead: their
        // scores stay far below any real one (|score| <= 64), 2^score is exactly 0, and neither the row sums nor
        // the P operand see them.  Register r of the lanes of group g is key 16 kb + 4 g + r of the half.
        f32x4v c0 = zero4;
        if constexpr (decltype(ragged)::value && kk == 0) {
          const int left = ke - (k0 + 32 * t) - 16 * kb - 4 * (l >> 4);  // valid keys from this lane's first one on
#pragma unroll
          for (int r = 0; r < 4; ++r) c0[r] = r < left ? 0.f : -1.0e4f;
        }
#pragma unroll
        for (int qb = 0; qb < 4; ++qb)
          sc[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[o % RD], qf[qb][kk], kk == 0 ? c0 : sc[kb][qb], 0, 0, 0);
      } else {
        // O^T[d][q] += V^T[d][key] P^T[key][q]
        constexpr int db = v_block(j - 8);
#pragma unroll
        for (int qb = 0; qb < 4; ++qb)
          o_acc[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[o % RD], __builtin_bit_cast(bf16x8, pf[qb]), o_acc[db][qb], 0, 0, 0);
      }
      // refill the slot just consumed with the fragment RD ahead; the first RD V^T fragments of a half are requested
      // right after the softmax instead (they would occupy registers across it)
      if constexpr (o + RD < 32) {
        constexpr int nj = (o + RD) & 15;
        if constexpr (!(nj >= 8 && nj < 8 + RD)) ring[o % RD] = read_op(std::integral_constant<int, o + RD>{});
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    static_for<0, 16>(consume);
    // (the ragged tile: a second half without a valid key has nothing to add.  Short key ranges, the text cross
    // attention with its dozen tiles per workgroup, are where this is noticeable.)
    if (!decltype(ragged)::value || ke - k0 > 32) static_for<16, 32>(consume);
  };

  // Tile order: the LAST tile of the key range first (it may hold the ragged end, so it runs the copy of the tile
  // body that masks the tail; the order of keys is immaterial to a softmax), then tiles 0 .. n_tiles-2 with the
  // mask-free body, two per loop iteration so that every LDS slot is named statically.  Tile `last` uses slot
  // pair 0, tile j slot pair (j + 1) & 1.
  const std::integral_constant<int, 0> slot0;
  const std::integral_constant<int, 1> slot1;
  // The accumulators start from zeros the compiler cannot see through: left to fold them into the first tile's
  // MFMAs it allocates that tile's registers differently from the steady-state body and spills two accumulators
  // there, a round trip to scratch memory for every workgroup.  (Here, behind the q fragments, so that the 128
  // registers are not held while q is loaded and normalised: the statement below pins the finished q fragments
  // ahead of them, or the compiler sinks the norm arithmetic to its first use, behind the zeros.)
  asm volatile("" ::"v"(qf[0][0]), "v"(qf[0][1]), "v"(qf[0][2]), "v"(qf[0][3]), "v"(qf[1][0]), "v"(qf[1][1]), "v"(qf[1][2]),
               "v"(qf[1][3]), "v"(qf[2][0]), "v"(qf[2][1]), "v"(qf[2][2]), "v"(qf[2][3]), "v"(qf[3][0]), "v"(qf[3][1]),
               "v"(qf[3][2]), "v"(qf[3][3]));
#pragma unroll
  for (int db = 0; db < 8; ++db)
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
      o_acc[db][qb] = f32x4v{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+v"(o_acc[db][qb]));
    }
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

  // ---- epilogue: normalise, transpose through LDS, store whole rows ----
  __syncthreads();  // every wave is done with the tile slots: wave w takes slot w as its 64 x 256-byte staging area
  if (!wave_on) return;
  unsigned char* const stage = w == 0 ? sK0 : w == 1 ? sV0 : w == 2 ? sK1 : sV1;
  int lane_e = l;
  asm volatile("" : "+v"(lane_e));
  const int ne = lane_e & 15, ge = lane_e >> 4;
  float l_tot[4];
#pragma unroll
  for (int qb = 0; qb < 4; ++qb) {
    float s = l_run[qb];
    s += __shfl_xor(s, 16);
    s += __shfl_xor(s, 32);
    l_tot[qb] = s;
    const float inv = 1.f / s;
    // lane (ne, ge) holds O[row 16 qb + ne][d = 16 db + 4 ge + r]: 8 bytes of bf16 at byte 32 db + 8 ge of the row,
    // i.e. half (ge & 1) of 16-byte chunk 2 db + ge / 2, kept at chunk ^ (row & 15) = chunk ^ ne
    unsigned char* const rowp = stage + (16 * qb + ne) * ROW_BYTES + ((ge & 1) << 3);
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const u32x2 v = {pack_bf16x2(o_acc[db][qb][0] * inv, o_acc[db][qb][1] * inv),
                       pack_bf16x2(o_acc[db][qb][2] * inv, o_acc[db][qb][3] * inv)};
      *LDS_PTR(u32x2, rowp + (((2 * db + (ge >> 1)) ^ ne) << 4)) = v;
    }
    const int q_row = row0 + 16 * qb + ne;
    if (a.lse && ge == 0 && q_row < qe)
      a.lse[(long)wi.h * a.total_q + q_row] = __builtin_amdgcn_logf(s) * 0.6931471805599453f;
  }
  // (the staging area is this wave's own: its LDS operations complete in order, no workgroup barrier is needed)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // 16 lanes x 16 bytes = one row; the wave stores four rows per instruction
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int r = 4 * it + ge;
    const u32x4 v = *LDS_PTR(const u32x4, stage + r * ROW_BYTES + ((ne ^ (r & 15)) << 4));
    const int q_row = row0 + r;
    if (q_row < qe) *(u32x4*)(a.out + (long)q_row * a.os_t + wi.o_head + 16 * ne) = v;
  }
}

}  // namespace

hipError_t launch_attn_fwd_bf16_x16(const AttnKernArgs& a, hipStream_t stream) {
  const dim3 grid(a.per_xcd * 8u);
  if (a.q_norm_gamma)  // raw q, normalised while it is loaded (cross attention)
    hipLaunchKernelGGL(attn_fwd_bf16_x16_kernel<Q_NORM>, grid, dim3(256), 0, stream, a);
  else if (a.flags & ATTN_SCALE_Q)  // unscaled q, scaled while it is loaded (the reference-shaped callables)
    hipLaunchKernelGGL(attn_fwd_bf16_x16_kernel<Q_SCALE>, grid, dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL(attn_fwd_bf16_x16_kernel<Q_AS_IS>, grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace magi
