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
// Instantiations with 2 waves / SIMD (deep prefetch, K and V double buffered), with 32-key tiles,
// with 8-wave workgroups, and a software-pipelined loop (PIPE: score MFMAs of the next tile, softmax
// and PV MFMAs of the current one interleaved in one basic block, 2 waves / SIMD) are kept for
// comparison; on the 720p layer none is faster.
//
// Work decomposition: blockIdx -> (kv head, range slot, q tile, q head within the GQA group),
// laid out so that the workgroups an XCD receives (blockIdx % 8) share a KV head and walk the
// same keys at about the same time (each XCD has its own L2).  Ranges are visited longest
// first.  Fully masked key tiles never exist: a rectangle is walked from k_start to k_end only.
#include "attn_common.h"

namespace magi {
namespace {

constexpr int ROW_BYTES = 256;  // D = 128 bf16

template <int NW, int BN, int NSTAGE, int OCC, bool VSINGLE, bool PIPE = false, bool DB = false, bool PRESC = false>
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
  static_assert(!PIPE || (NSTAGE == 2 && BN == 64 && !VSINGLE), "pipelined loop: 64-key tiles, two K slots and two V slots");
  static_assert(!DB || (NSTAGE == 2 && !VSINGLE && !PIPE), "static double buffer: two K slots and two V slots");
  // ring of NSTAGE (K tile, V tile) pairs for the loops that index their slots at run time; the single-V, the
  // double-buffered and the pipelined loops declare their slots as separate objects and leave this one a stub
  __shared__ __attribute__((aligned(1024))) unsigned char smem[(PIPE || DB || VSINGLE) ? 1 : 2 * NSTAGE][(PIPE || DB || VSINGLE) ? 16 : TILE_BYTES];
  __shared__ int s_sel;

  const int tid = threadIdx.x;
  // ---- which piece of work is this workgroup? ----
  const WorkItem wi = locate_work(a, BM, tid, &s_sel);
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
  auto issue_tile = [&](int k0, int stage) {
    issue_mat(k0, &smem[2 * stage][0], false);
    issue_mat(k0, &smem[2 * stage + 1][0], true);
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
  if constexpr (PIPE) {
    // Software-pipelined loop.  Iteration `it` runs, in ONE basic block, the score MFMAs of tile it+1, the
    // exp2 / pack / row-sum work of tile it, the PV MFMAs of tile it and the row max of tile it+1, cut into
    // 32 chunks of one MFMA + its operand reads + a few VALU instructions each (scheduling barriers pin the
    // chunks), so that the VALU work issues in the shadow of the MFMAs of the same wave.  The lazy rescale of
    // O and the tail mask sit between iterations.  K(t) lives in K slot t & 1, V(t) in V slot t & 1; the loads
    // for K(it+2) and V(it+1) are issued at the top of iteration it and have the whole iteration to land.
    // The four slots are four separate LDS objects and the loop is unrolled by two so that every access names
    // its slot statically: the compiler then knows that the operand reads of an iteration never touch the
    // slots the in-flight direct loads write, and does not make the reads wait for those loads.
    __shared__ __attribute__((aligned(1024))) unsigned char sK0[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char sK1[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char sV0[TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char sV1[TILE_BYTES];
    auto read_k = [&](const unsigned char* Kt, int idx) -> bf16x8 {  // idx = 8t + kk
      return *LDS_PTR(const bf16x8, Kt + ((base_k ^ ((idx & 7) << 5)) + (idx >> 3) * 32 * ROW_BYTES));
    };
    auto read_v = [&](const unsigned char* Vt, int p) -> bf16x8 {  // p = 4 * slab + mb
      const int mb = p & 3, sl = p >> 2;
      const int bv = base_v ^ (mb << 6);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * sl) * ROW_BYTES)));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, Vt + (bv + (16 * sl + 8) * ROW_BYTES)));
      const s16x8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, va);
    };
    constexpr int PD = 4;  // operand reads in flight (2 .. 8 measure the same)
    f32x16 sA[2], sB[2];   // scores of even / odd tiles
    float m_new, alpha;

    // ---- prologue: K(0) -> scores of tile 0 and their row max ----
    issue_mat(ks, sK0, false);
    wait_vmcnt<0>();
    __syncthreads();
    if (n_tiles > 1) issue_mat(ks + BN, sK1, false);
    issue_mat(ks, sV0, true);
    {
      bf16x8 kbuf[PD];
#pragma unroll
      for (int idx = 0; idx < PD; ++idx) kbuf[idx] = read_k(sK0, idx);
#pragma unroll
      for (int idx = 0; idx < 16; ++idx) {
        const int t = idx >> 3, kk = idx & 7;
        sA[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kbuf[idx % PD], qf[kk], kk == 0 ? zero16 : sA[t], 0, 0, 0);
        if (idx + PD < 16) kbuf[idx % PD] = read_k(sK0, idx + PD);
      }
      // keys past the end of the range repeat the last valid row (the loader clamps), so the max needs no mask
      float mx = sA[0][0];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sA[t][v]);
      m_new = half_swap_max(mx);
      alpha = 0.f;
    }

    // between iterations (tile `it` of parity P): lazy rescale, tail mask, publish the next tiles
    auto top = [&](int it, auto pc, f32x16 (&s_cur)[2]) {
      constexpr int P = decltype(pc)::value;
      const int k0 = ks + it * BN;
      if (it > 0 && __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // some row of this wave saw a new maximum
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
          for (int v = 0; v < 16; ++v) o_acc[mb][v] *= alpha;
      }
      if (k0 + BN > ke) {  // ragged last tile: keys >= ke do not exist
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = k0 + 32 * t + 8 * (v >> 2) + 4 * g + (v & 3);
            if (key >= ke) s_cur[t][v] = -__builtin_inff();
          }
      }
      wait_vmcnt<0>();
      __syncthreads();  // K(it+1) and V(it) landed; K slot P and V slot P^1 are free
      if (it + 2 < n_tiles) issue_mat(k0 + 2 * BN, P ? sK1 : sK0, false);
      if (it + 1 < n_tiles) issue_mat(k0 + BN, P ? sV0 : sV1, true);
    };
    constexpr int SM_OPS = 96;

    // one pipelined iteration for a tile of parity P
    auto step = [&](int it, auto pc, f32x16 (&s_cur)[2], f32x16 (&s_nxt)[2]) {
      constexpr int P = decltype(pc)::value;
      top(it, pc, s_cur);
      if (!wave_on) return;
      const unsigned char* Kn = P ? sK0 : sK1;
      const unsigned char* Vt = P ? sV1 : sV0;
      const float mc = m_new * c;
      const float m_prev = m_new;  // running max including tile it

      float psum = 0.f;
      float mxa = 0.f, mxb = 0.f, m_nx = 0.f, al_nx = 1.f;
      // softmax micro-ops of tile it: group j = elements (2j, 2j+1) of the 32 this lane holds, 6 ops per group
      // (the packed probabilities of slab s overwrite the first four of the eight score registers they came
      // from, so P needs no registers of its own)
      auto sm_op = [&](auto nc) {
        constexpr int n = decltype(nc)::value;
        constexpr int j = n / 6, k = n % 6;
        constexpr int t = j >> 3, v0 = 2 * (j & 7);
        constexpr int pw = 8 * ((j >> 2) & 1) + (j & 3);  // register of s_cur[t] that receives packed pair j
        if constexpr (k == 0) s_cur[t][v0] = fmaf(s_cur[t][v0], c, -mc);
        if constexpr (k == 1) s_cur[t][v0 + 1] = fmaf(s_cur[t][v0 + 1], c, -mc);
        if constexpr (k == 2) s_cur[t][v0] = __builtin_amdgcn_exp2f(s_cur[t][v0]);
        if constexpr (k == 3) s_cur[t][v0 + 1] = __builtin_amdgcn_exp2f(s_cur[t][v0 + 1]);
        if constexpr (k == 4) s_cur[t][pw] = __builtin_bit_cast(float, pack_bf16x2(s_cur[t][v0], s_cur[t][v0 + 1]));
        if constexpr (k == 5) {
          const float packed = s_cur[t][pw];  // (a bit_cast applied to the vector element itself reads element 0)
          psum = pair_sum(__builtin_bit_cast(unsigned, packed), psum);
        }
      };
      auto p_operand = [&](int sl) -> bf16x8 {  // B operand of the PV MFMAs for slab sl
        const f32x16& sv = s_cur[sl >> 1];
        const f32x4 r = (sl & 1) ? __builtin_shufflevector(sv, sv, 8, 9, 10, 11) : __builtin_shufflevector(sv, sv, 0, 1, 2, 3);
        return __builtin_bit_cast(bf16x8, r);
      };
      // row-max micro-ops of tile it+1: 8 + 8 max3, then combine / running max / alpha
      auto mr_op = [&](auto nc) {
        constexpr int n = decltype(nc)::value;
        constexpr int q = n & 7;
        if constexpr (n < 16) {
          const f32x16& sv = s_nxt[n >> 3];
          float& m = (n < 8) ? mxa : mxb;
          if constexpr (q == 0) m = max3(sv[0], sv[1], sv[2]);
          else if constexpr (q < 7) m = max3(m, sv[2 * q + 1], sv[2 * q + 2]);
          else m = max3(m, sv[15], sv[15]);
        } else if constexpr (n == 16) {
          m_nx = half_swap_max(max3(mxa, mxb, mxb));
        } else if constexpr (n == 17) {
          m_nx = max3(m_prev, m_nx, m_nx);
        } else if constexpr (n == 18) {
          al_nx = __builtin_amdgcn_exp2f((m_prev - m_nx) * c);
        }
      };
      bf16x8 obuf[PD];  // operand ring: K operands during the score MFMAs, then V operands
#pragma unroll
      for (int idx = 0; idx < PD; ++idx) obuf[idx] = read_k(Kn, idx);
      // VALU work that does not wait for the operand reads
      static_for<0, 6>(sm_op);
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, 32>([&](auto chc) {
        constexpr int ch = decltype(chc)::value;
        if constexpr (ch < 16) {
          constexpr int t = ch >> 3, kk = ch & 7;
          s_nxt[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(obuf[ch % PD], qf[kk], kk == 0 ? zero16 : s_nxt[t], 0, 0, 0);
          if constexpr (ch + PD < 16)
            obuf[ch % PD] = read_k(Kn, ch + PD);
          else
            obuf[ch % PD] = read_v(Vt, ch + PD - 16);
        } else {
          constexpr int p = ch - 16;
          o_acc[p & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(obuf[ch % PD], p_operand(p >> 2), o_acc[p & 3], 0, 0, 0);
          if constexpr (p + PD < 16) obuf[ch % PD] = read_v(Vt, p + PD);
        }
        // softmax ops: all 96 done after chunk 25 (slab 3 is needed by chunk 28)
        constexpr int lo = 6 + (90 * ch) / 26, hi0 = 6 + (90 * (ch + 1)) / 26, hi = hi0 < SM_OPS ? hi0 : SM_OPS;
        static_for<(lo < hi ? lo : hi), hi>(sm_op);
        // row max of tile it+1: first half of the scores is complete after chunk 7, the second after chunk 15
        if constexpr (ch >= 10 && ch < 18) mr_op(std::integral_constant<int, ch - 10>{});
        if constexpr (ch >= 19 && ch < 27) mr_op(std::integral_constant<int, ch - 19 + 8>{});
        if constexpr (ch >= 28 && ch < 31) mr_op(std::integral_constant<int, ch - 28 + 16>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      l_run = l_run * alpha + psum;
      m_run = m_prev;
      m_new = m_nx;
      alpha = al_nx;
    };
    // The last tile runs the same step: its score MFMAs read a K slot that holds no new tile and produce
    // values nobody uses (one wasted product per workgroup instead of a second copy of the loop body).
    const std::integral_constant<int, 0> even;
    const std::integral_constant<int, 1> odd;
    for (int it = 0; it < n_tiles; it += 2) {
      step(it, even, sA, sB);
      if (it + 1 >= n_tiles) break;
      step(it + 1, odd, sB, sA);
    }
  } else {
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
  } else {
    // ring of NSTAGE (K tile, V tile) pairs, tiles requested NSTAGE-1 ahead, one barrier per tile
#pragma unroll
    for (int p = 0; p < NSTAGE - 1; ++p)
      if (p < n_tiles) issue_tile(ks + p * BN, p);
    int stage = 0;
    for (int it = 0; it < n_tiles; ++it) {
      const int k0 = ks + it * BN;
      // tile `it` must have landed; up to NSTAGE-2 younger tiles may still be in flight
      const int younger = min(NSTAGE - 2, n_tiles - 1 - it);
      if (NSTAGE >= 4 && younger == 2)
        wait_vmcnt<2 * TILE_LOADS>();
      else if (NSTAGE >= 3 && younger == 1)
        wait_vmcnt<TILE_LOADS>();
      else
        wait_vmcnt<0>();
      __syncthreads();  // everybody's share landed; the stage read in the previous iteration is free again
      if (it + NSTAGE - 1 < n_tiles) {
        int st = stage + NSTAGE - 1;
        if (st >= NSTAGE) st -= NSTAGE;
        issue_tile(k0 + (NSTAGE - 1) * BN, st);
      }
      const unsigned char* Kt = &smem[2 * stage][0];
      const unsigned char* Vt = &smem[2 * stage + 1][0];
      stage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
      if (!wave_on) continue;
      compute_tile(Kt, Vt, k0, []() {});
    }
  }  // !DB
  }  // !PIPE

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
  const unsigned grid = a.per_xcd * 8u;
  const bool presc = (a.flags & 2) != 0;  // q pre-scaled: the scores are exp2 exponents (PRESC instantiations)
#ifdef MAGI_TUNING
  // comparison instantiations, reachable in tuning builds only (MAGI_ATTN_BLOCK_M / MAGI_ATTN_VARIANT)
  if (a.block_m == 256 && a.variant == 3)  // software-pipelined loop, 8 waves, 256 query rows, 2 waves / SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<8, 64, 2, 2, false, true>), dim3(grid), dim3(512), 0, stream, a);
  else if (a.block_m == 256)  // 8 waves, 256 query rows, 2 waves / SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<8, 64, 2, 2, false>), dim3(grid), dim3(512), 0, stream, a);
  else if (a.block_m == 128 && a.variant == 1)  // 32-key tiles, 3-stage ring, 3 waves / SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 32, 3, 3, false>), dim3(grid), dim3(256), 0, stream, a);
  else if (a.block_m == 128 && a.variant == 2)  // 64-key tiles, double-buffered K and V, 2 waves / SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 2, false>), dim3(grid), dim3(256), 0, stream, a);
  else if (a.block_m == 128 && a.variant == 3)  // software-pipelined loop, 2 waves / SIMD
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 2, false, true>), dim3(grid), dim3(256), 0, stream, a);
  else if (a.block_m == 384 && a.variant == 7)  // pre-scaled q through the instantiation with the per-score multiply
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<12, 64, 2, 1, false, false, true>), dim3(grid), dim3(768), 0, stream, a);
  else if (a.variant == 7)
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 3, true>), dim3(grid), dim3(256), 0, stream, a);
  else
#endif
  if (a.block_m == 384 && presc)  // 12 waves, 384 query rows, one workgroup per CU = 3 waves / SIMD sharing every tile
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<12, 64, 2, 1, false, false, true, true>), dim3(grid), dim3(768), 0, stream, a);
  else if (a.block_m == 384)
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<12, 64, 2, 1, false, false, true>), dim3(grid), dim3(768), 0, stream, a);
  else if (presc)  // 4 waves, 64-key tiles, double-buffered K, single V slot, three workgroups per CU
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 3, true, false, false, true>), dim3(grid), dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL((attn_fwd_bf16_kernel<4, 64, 2, 3, true>), dim3(grid), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace magi
