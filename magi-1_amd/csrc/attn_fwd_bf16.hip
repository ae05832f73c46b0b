// Range attention forward, bf16 in / bf16 out, fp32 online softmax, for gfx950 (MI355X).
//
// One workgroup = NW wavefronts = 32*NW query rows of one (range, q head); wave w owns rows
// 32w..32w+31.  Key/value rows stream through LDS in tiles of BN keys held in a ring of NSTAGE
// stages, filled by direct global->LDS loads (no register staging) issued NSTAGE-1 tiles ahead.
//
// The scores are computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: the
// accumulator layout then puts ONE query per lane column (lane % 32) and spreads the keys over
// the registers, so row max / row sum are plain per-lane reductions plus one exchange between
// the two half-waves, and the probabilities are already in the B-operand layout of the second
// product O^T = V^T P^T.  V^T is fetched from the row-major V tile with the transposing LDS
// read ds_read_b64_tr_b16.
//
// LDS tile layout: rows of 256 bytes; the 16-byte chunk c of row r lives at chunk
// c ^ (r & 15) for K (conflict-free ds_read_b128 down a column of rows) and at
// c ^ ((r & 3) << 2) for V (conflict-free transposing reads of 4-row groups).  A direct load
// places lane l's 16 bytes at base + 16*l, so the swizzle is applied on the global side: lane
// l fetches the logical chunk that belongs at its fixed LDS slot.
//
// A single wavefront cannot keep the MFMA pipe busy (in-order issue, ~5 cycles between its VALU
// instructions, LDS and MFMA latencies in series): throughput comes from several waves per SIMD
// in different phases.  Both instantiations that the library picks run 3 waves / SIMD (<= 168 VGPRs,
// shallow operand prefetch):
//   * 4 waves per workgroup, three workgroups per CU, 48 KB of LDS each (64-key tiles, K double
//     buffered, ONE V slot that is refilled under the score MFMAs and the softmax of the same tile,
//     two barriers per tile, slots named statically): small grids and short key ranges;
//   * 12 waves per workgroup (DB), ONE workgroup per CU, 64 KB of LDS (K and V double buffered in
//     four statically named slots, one barrier per tile, the tile loads issued by four of the
//     waves, one per SIMD): every K / V tile is fetched from L2 once
//     for 384 query rows instead of 128.  On grids of many rounds with long key ranges this is the
//     faster one, although it needs more cycles: the part is power limited, and the bytes it does
//     not move come back as clock.
// Both have a PRESC form that takes q already multiplied by softmax_scale * log2(e) (the prologue
// does that ahead of q's rounding to bf16) and accumulates the score MFMAs onto the negated running
// maximum, so the MFMA result is the exp2 argument and no per-score multiply-subtract remains.
// Operand reads from LDS are written a few MFMAs ahead of their use and held there with scheduling
// barriers (the instruction scheduler otherwise sinks them to one MFMA ahead); the epilogue trades
// registers between the half waves so that every lane stores 16 contiguous bytes.
//
// Work decomposition: blockIdx -> (kv head, range slot, q tile, q head within the GQA group),
// laid out so that the workgroups an XCD receives (blockIdx % 8) share a KV head and walk the
// same keys at about the same time (each XCD has its own L2).  Ranges are visited longest
// first.  Fully masked key tiles never exist: a rectangle is walked from k_start to k_end only.
#include "attn_common.h"

namespace magi {
namespace {

constexpr int ROW_BYTES = 256;  // D = 128 bf16

// VSINGLE: the 4-wave form (two K slots, one V slot); DB: the 12-wave form (K and V double buffered); exactly one of them
template <int NW, int BN, int NSTAGE, int OCC, bool VSINGLE, bool DB = false, bool PRESC = false>
__global__ __launch_bounds__(64 * NW, OCC) void attn_fwd_bf16_kernel(const AttnKernArgs a) {
  constexpr int BM = 32 * NW;
  constexpr int TILE_BYTES = BN * ROW_BYTES;
  constexpr int LW = NW > 8 ? 4 : NW;      // waves that load tiles (a 64-row tile is 16 loads of 4 rows); a multiple of 4
  constexpr int LOADS = BN / (4 * LW);     // direct loads per loading wave per matrix per tile (4 rows each)
  constexpr int WPS = NW * OCC / 4;        // waves per SIMD
  constexpr int TILE_LOADS = 2 * LOADS;    // ... per wave per tile
  constexpr int NT = BN / 32;              // 32-key score tiles per key tile
  constexpr int NS = BN / 16;              // 16-key slabs per key tile
  constexpr int DK = WPS >= 3 ? 4 : 8;     // K operands in flight
  constexpr int DV = WPS >= 3 ? 4 : 8;     // V operands in flight
  constexpr bool VEARLY = !VSINGLE && WPS < 3;  // first V operands fetched under the last score MFMAs (needs registers)
  constexpr bool VMID = DB && PRESC;           // ... in the middle of the softmax (V is in LDS by then only in the DB loop)
  static_assert(LOADS >= 1 && NSTAGE >= 2 && NSTAGE <= 4, "bad tile configuration");
  static_assert(!VSINGLE || NSTAGE == 2, "single-V mode: two K slots and one V slot");
  static_assert(!DB || (NSTAGE == 2 && !VSINGLE), "static double buffer: two K slots and two V slots");
  static_assert(DB != VSINGLE, "one of the two tile loops");
  __shared__ int s_sel[LOCATE_WORDS];

  if (gate_closed(a)) return;
  const int tid = threadIdx.x;
  // ---- which piece of work is this workgroup? ----
  const WorkItem wi = locate_work(a, BM, tid, s_sel);
  if (!wi.valid) return;
  const int h = wi.h, q0 = wi.q0, qe = wi.qe, ks = wi.ks, ke = wi.ke;
  const unsigned kvh = (unsigned)wi.kvh;
  const long o_head = wi.o_head;

  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, i = l & 31, g = l >> 5;
  const int q_row = q0 + 32 * w + i;
  const bool row_ok = q_row < qe;

  if (ke <= ks) {  // no keys: zeros, lse = -inf
    if (row_ok) store_empty_row(a, wi, q_row, g);
    return;
  }

  // ---- Q fragments (B operand of S^T = K Q^T): lane (i, g) holds Q[row i][16kk + 8g .. +8] ----
  bf16x8 qf[8];
  {
    const int qr = min(q_row, qe - 1);
    const char* qp = a.q + (long)qr * a.qs_t + (long)h * a.qs_h + g * 16;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[kk] = *(const bf16x8*)(qp + kk * 32);

  }

  // ---- K/V tile loader: wave w fills rows 4*(w + NW*j) .. +3; lane l sits at row +(l >> 4), slot l & 15 ----
  const int lrow = l >> 4, slot = l & 15;
  // the loading waves are the LAST LW of the workgroup (the youngest waves, which the arbiter serves last anyway:
  // 0.6 % faster on the 720p launch than the first LW); wl = index among them
  const int wl = w - (NW - LW);
  const int row_in_tile0 = 4 * wl + lrow;                 // + 4*LW*j
  const int kchunk = slot ^ ((4 * (wl & 3) + lrow) & 15);  // logical chunk that belongs in this K slot
  const int vchunk = slot ^ (lrow << 2);                  // ... in this V slot
  const long ks_t = a.ks_t, vs_t = a.vs_t;
  const int k_split = a.k_split;
  const long k2_delta = a.k2 ? (a.k2 - a.k) - (long)k_split * ks_t : 0;
  const long v2_delta = a.v2 ? (a.v2 - a.v) - (long)k_split * vs_t : 0;
  const char* const kcolp = a.k + (long)kvh * a.ks_h;
  const char* const vcolp = a.v + (long)kvh * a.vs_h;
  const unsigned kvoff = (unsigned)row_in_tile0 * (unsigned)ks_t + (unsigned)(kchunk * 16);
  const unsigned vvoff = (unsigned)row_in_tile0 * (unsigned)vs_t + (unsigned)(vchunk * 16);
  const bool small_strides = ks_t * (BN + 4) < (1l << 31) && vs_t * (BN + 4) < (1l << 31);

  // LOADS load instructions per wave per matrix per tile, always, so outstanding loads can be counted.
  auto issue_mat = [&](int k0, unsigned char* tile_base, bool is_v) {
    if (NW > LW && wl < 0) return;  // (wave uniform) the other waves only consume
    unsigned char* dst = tile_base + wl * 1024;
    const long st = is_v ? vs_t : ks_t;
    const char* colp = is_v ? vcolp : kcolp;
    const long d2 = is_v ? v2_delta : k2_delta;
    const bool interior = small_strides && (k0 + BN <= ke) && (k0 + BN <= k_split || k0 >= k_split);
    if (interior) {
      // Buffer-addressed direct loads: scalar base (the tile's first row) in the resource descriptor, one
      // loop-invariant 32-bit lane offset, the row group of load j in the scalar offset.  This form costs the
      // SIMD next to nothing to issue; the 64-bit-address-per-lane form of the same load stalls it for well
      // over a hundred cycles per instruction.
      const char* b = colp + (long)k0 * st + (k0 >= k_split ? d2 : 0);
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)b, 0, 0x7fffffff, 0x00020000);
      unsigned voff = is_v ? vvoff : kvoff;
      if constexpr (PRESC) {
        // (this instantiation has no registers to spare: the lane offset is re-derived from an opaque copy of
        // the lane index instead of living across the loop)
        int lane = l;
        asm volatile("" : "+v"(lane));
        const int lr = lane >> 4, sl = lane & 15;
        const int chunk = is_v ? (sl ^ (lr << 2)) : (sl ^ ((4 * (wl & 3) + lr) & 15));
        voff = (unsigned)(4 * wl + lr) * (unsigned)st + (unsigned)(chunk * 16);
      }
#pragma unroll
      for (int j = 0; j < LOADS; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, dst + j * LW * 1024), 16, voff,
                                                 (int)((unsigned)(4 * LW * j) * (unsigned)st), 0, 0);
    } else {  // ragged end of the range, or a tile that straddles the two key segments
      // (rare: the lane geometry is re-derived here from an opaque copy of the lane index, so that nothing of
      // it occupies registers across the main loop)
      int lane = l;
      asm volatile("" : "+v"(lane));
      const int lrow_s = lane >> 4, slot_s = lane & 15;
      const int row_in_tile0 = 4 * wl + lrow_s;
      const int chunk = is_v ? (slot_s ^ (lrow_s << 2)) : (slot_s ^ ((4 * (wl & 3) + lrow_s) & 15));
#pragma unroll
      for (int j = 0; j < LOADS; ++j) {
        const int row = min(k0 + row_in_tile0 + 4 * LW * j, ke - 1);
        const char* p = colp + (long)row * st + (row >= k_split ? d2 : 0) + chunk * 16;
        __builtin_amdgcn_global_load_lds(GLOBAL_PTR(p), LDS_PTR(void, dst + j * LW * 1024), 16, 0, 0);
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

  f32x16 o_acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[mb][v] = 0.f;
  // running max of the raw scores.  PRESC (q carries softmax_scale * log2(e), so the scores are exp2 exponents): the
  // score MFMAs accumulate onto neg_m = -(running max) in all 16 registers (a lane's registers all belong to one
  // query) and deliver exponent - max directly: no per-score multiply-subtract; the maximum starts at 0
  float m_run = PRESC ? 0.f : -__builtin_inff();
  f32x16 neg_m;
#pragma unroll
  for (int v = 0; v < 16; ++v) neg_m[v] = 0.f;
  bool first = true;
  float l_run = 0.f;                // this lane's share of the running sum
  const float c = a.scale_log2;
  const bool wave_on = (q0 + 32 * w) < qe;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  const int n_tiles = (ke - ks + BN - 1) / BN;
  // One key tile for this wave: scores, online softmax, PV.  Kt / Vt: the tile's K and V slots; before_pv runs
  // between the softmax and the first V operand read (the single-V mode publishes V(it) there).
  auto compute_tile = [&](const unsigned char* Kt, const unsigned char* Vt, int k0, auto before_pv) {
    // LDS operand fetchers
    auto read_k = [&](int idx) -> bf16x8 {  // idx = 8t + kk
      return *LDS_PTR(const bf16x8, Kt + ((base_k ^ ((idx & 7) << 5)) + (idx >> 3) * 32 * ROW_BYTES));
    };
    auto read_v = [&](int p) -> bf16x8 {  // p = mb * NS + slab
      const int mb = p / NS, s = p % NS;
      const int bv = base_v ^ (mb << 6);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * s) * ROW_BYTES)));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * s + 8) * ROW_BYTES)));
      const s16x8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, va);
    };

    // S^T[key][q] for BN keys x 32 queries.  K operands run DK reads ahead of the MFMAs that consume
    // them; the first DV V operands are fetched under the last MFMAs.
    constexpr int RK = NT * 8;
    constexpr int RV = NS * 4;
    f32x16 s_acc[NT];
    bf16x8 kbuf[DK], vbuf[DV];
#pragma unroll
    for (int idx = 0; idx < DK; ++idx) kbuf[idx] = read_k(idx);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int idx = 0; idx < RK; ++idx) {
      const int t = idx >> 3, kk = idx & 7;
      s_acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kbuf[idx % DK], qf[kk],
                                                         kk == 0 ? (PRESC ? neg_m : zero16) : s_acc[t], 0, 0, 0);
      if (idx + DK < RK)
        kbuf[idx % DK] = read_k(idx + DK);
      else if (VEARLY && idx + DK - RK < DV)
        vbuf[idx + DK - RK] = read_v(idx + DK - RK);
      if (DK == 8 && NT == 2 && idx == 7) __builtin_amdgcn_sched_barrier(0);
      // Keep every operand read where it is written, DK MFMAs ahead of its use: left alone, the scheduler moves
      // the reads down to one MFMA ahead (2.5 % on the 720p launch).  The pre-scaled instantiations have no
      // registers for the pinned K pipeline (it spills); they pin the V pipeline below only.
      if (!PRESC) __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (k0 + BN > ke) {  // ragged last tile: keys >= ke do not exist
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = k0 + 32 * t + 8 * (v >> 2) + 4 * g + (v & 3);
          if (key >= ke) s_acc[t][v] = -__builtin_inff();
        }
    }
    // online softmax: every value this lane holds belongs to query i
    float mx = max3(s_acc[0][0], s_acc[0][1], s_acc[0][2]);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = (t == 0 ? 3 : 0); v < 16; v += 2) mx = max3(mx, s_acc[t][v], s_acc[t][v + 1 < 16 ? v + 1 : v]);
    mx = half_swap_max(mx);
    // Row sum of the probabilities in fp32, by plain additions.  (v_dot2c_f32_bf16 against (1, 1) would add a packed
    // pair in one instruction, but dot instructions do not execute beside an MFMA: each one holds the matrix pipe up
    // for about 16 cycles, measured, where exp2 / convert / add / fma run under it for free.  Rounding to bf16 is
    // unbiased, so the sum of the unrounded values is as good a denominator.)
    float psum = 0.f, psum2 = 0.f;
    if constexpr (PRESC) {
      // s_acc holds exponent - m_run: a positive value is a new row maximum (rare after the first tiles)
      const bool raise = first || mx > 0.f;
      if (__builtin_amdgcn_ballot_w64(raise) != 0) {
        const float delta = raise ? mx : 0.f;
        const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-delta);
        l_run *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) neg_m[v] -= delta;  // (the running maximum is -neg_m)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) s_acc[t][v] -= delta;
        if (!first) {
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[mb][v] *= alpha;
        }
      }
      first = false;
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          f32x16& sv = s_acc[s >> 1];
          const int v0 = 8 * (s & 1) + e;
          // (this instantiation has no register left for the two exponentials to outlive their packing: it keeps
          // the one-instruction pair sum on the packed values)
          const unsigned pk = pack_bf16x2(__builtin_amdgcn_exp2f(sv[v0]), __builtin_amdgcn_exp2f(sv[v0 + 1]));
          psum = pair_sum(pk, psum);
          sv[8 * (s & 1) + (e >> 1)] = __builtin_bit_cast(float, pk);
          if (VMID && s == NS - 2 && e == 6) {
            // three of the four slabs are packed: their score registers are free, and the first V operands can
            // be on their way from LDS while the last slab is exponentiated (0.3-0.4 % on the 720p launch)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < DV; ++p) vbuf[p] = read_v(p);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      l_run += psum;
    } else {
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
    const float mc = m_new * c;
    m_run = m_new;
    // the packed probabilities of slab s overwrite the first four of the eight score registers they came from
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        f32x16& sv = s_acc[s >> 1];
        const int v0 = 8 * (s & 1) + e;
        const float p0 = __builtin_amdgcn_exp2f(sv[v0] * c - mc);
        const float p1 = __builtin_amdgcn_exp2f(sv[v0 + 1] * c - mc);
        psum += p0;
        psum2 += p1;
        sv[8 * (s & 1) + (e >> 1)] = __builtin_bit_cast(float, pack_bf16x2(p0, p1));
      }
    l_run = l_run * alpha + (psum + psum2);
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // some row of this wave saw a new maximum
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[mb][v] *= alpha;
    }
    }
    auto p_operand = [&](int s) -> bf16x8 {  // B operand of the PV MFMAs for slab s
      const f32x16& sv = s_acc[s >> 1];
      const f32x4 r = (s & 1) ? __builtin_shufflevector(sv, sv, 8, 9, 10, 11) : __builtin_shufflevector(sv, sv, 0, 1, 2, 3);
      return __builtin_bit_cast(bf16x8, r);
    };

    // O^T[d][q] += V^T[d][key] P^T[key][q]; V operands run DV reads ahead
    __builtin_amdgcn_sched_barrier(0);
    before_pv();
    if (!VEARLY && !VMID) {
#pragma unroll
      for (int p = 0; p < DV; ++p) vbuf[p] = read_v(p);
    }
#pragma unroll
    for (int p = 0; p < RV; ++p) {
      const int mb = p / NS, s = p % NS;
      o_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vbuf[p % DV], p_operand(s), o_acc[mb], 0, 0, 0);
      if (p + DV < RV) vbuf[p % DV] = read_v(p + DV);
      __builtin_amdgcn_sched_barrier(0);  // (as above: 0.4-0.9 %)
    }
  };
  if constexpr (DB) {
    // K and V double buffered in four separate LDS objects, the loop unrolled by two so that every slot is named
    // statically (an operand read then never waits for the direct loads in flight to the other pair of slots);
    // one barrier per tile, and the loads of tile it+1 have the whole of iteration it to land.
    __shared__ __attribute__((aligned(1024))) unsigned char dK0[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char dV0[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char dK1[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char dV1[TILE_BYTES];
    issue_mat(ks, dK0, false);
    issue_mat(ks, dV0, true);
    auto step = [&](int it, auto bc) {
      constexpr int B = decltype(bc)::value;
      const int k0 = ks + it * BN;
      wait_vmcnt<0>();
      __syncthreads();
      if (it + 1 < n_tiles) {
        issue_mat(k0 + BN, B ? dK0 : dK1, false);
        issue_mat(k0 + BN, B ? dV0 : dV1, true);
      }
      if (!wave_on) return;
      compute_tile(B ? dK1 : dK0, B ? dV1 : dV0, k0, []() {});
    };
    for (int it = 0; it < n_tiles; it += 2) {
      step(it, std::integral_constant<int, 0>{});
      if (it + 1 >= n_tiles) break;
      step(it + 1, std::integral_constant<int, 1>{});
    }
  } else if constexpr (VSINGLE) {
    // single-V mode (48 KB of LDS, three workgroups per CU) with statically named slots, the loop unrolled by two:
    // K(it) was requested one iteration ago; V(it) is requested now, into the one V slot that PV(it-1) has just
    // released, and lands under the score MFMAs and the softmax of this tile; a second barrier publishes it
    // before PV(it).
    __shared__ __attribute__((aligned(1024))) unsigned char vK0[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char vK1[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char vV[TILE_BYTES];
    issue_mat(ks, vK0, false);
    auto step = [&](int it, auto bc) {
      constexpr int B = decltype(bc)::value;
      const int k0 = ks + it * BN;
      wait_vmcnt<0>();
      __syncthreads();
      issue_mat(k0, vV, true);
      if (it + 1 < n_tiles) issue_mat(k0 + BN, B ? vK0 : vK1, false);
      compute_tile(B ? vK1 : vK0, vV, k0, [&]() {
        if (it + 1 < n_tiles)
          wait_vmcnt<LOADS>();  // V(it) landed; the K(it+1) loads issued after it may still be in flight
        else
          wait_vmcnt<0>();
        __syncthreads();
      });
    };
    for (int it = 0; it < n_tiles; it += 2) {
      step(it, std::integral_constant<int, 0>{});
      if (it + 1 >= n_tiles) break;
      step(it + 1, std::integral_constant<int, 1>{});
    }
  }

  if (!wave_on) return;
  // ---- epilogue: normalise and store ----
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.f / l_tot;
  // A lane holds four consecutive features per (mb, b), its partner in the other half wave the next four: the
  // halves trade the odd-b registers of the lower half for the even-b registers of the upper one, after which
  // every lane owns eight consecutive features and stores 16 bytes at a time.
  // (the row address is derived here from an opaque copy of the lane index, or the compiler computes it at the
  // top of the kernel and carries two more registers through the main loop, which the pre-scaled instantiations
  // do not have)
  int lane_e = l;
  asm volatile("" : "+v"(lane_e));
  char* const op = a.out + (long)(q0 + 32 * w + (lane_e & 31)) * a.os_t + o_head + 16 * (lane_e >> 5);
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int bp = 0; bp < 2; ++bp) {
      unsigned ev[2], od[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        ev[e] = pack_bf16x2(o_acc[mb][8 * bp + 2 * e] * inv, o_acc[mb][8 * bp + 2 * e + 1] * inv);
        od[e] = pack_bf16x2(o_acc[mb][8 * bp + 4 + 2 * e] * inv, o_acc[mb][8 * bp + 4 + 2 * e + 1] * inv);
        half_swap(ev[e], od[e]);  // lower half: (own even, partner's even); upper half: (partner's odd, own odd)
      }
      if (row_ok) *(u32x4*)(op + (32 * mb + 16 * bp) * 2) = u32x4{ev[0], ev[1], od[0], od[1]};
    }
  if (row_ok) {
    if (a.lse && g == 0)
      a.lse[(long)h * a.total_q + q_row] = ((PRESC ? -neg_m[0] : m_run * c) + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  }
}

}  // namespace

hipError_t launch_attn_fwd_bf16(const AttnKernArgs& a, hipStream_t stream) {
  const dim3 grid(a.per_xcd * 8u);
  const bool presc = (a.flags & 2) != 0;  // q pre-scaled: the scores are exp2 exponents (PRESC instantiations)
  if (a.block_m == 384 && presc)  // 12 waves, 384 query rows, one workgroup per CU = 3 waves / SIMD sharing every tile
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<12, 64, 2, 1, false, true, true>), grid, dim3(768), 0, stream, a);
  else if (a.block_m == 384)
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<12, 64, 2, 1, false, true>), grid, dim3(768), 0, stream, a);
  else if (presc)  // 4 waves, 64-key tiles, double-buffered K, single V slot, three workgroups per CU
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 3, true, false, true>), grid, dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 3, true>), grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace magi
