// fp8 (OCP e4m3fn) range attention forward and the per-(chunk, head) quantiser, for gfx950.
//
// Same organisation as the bf16 kernel (S^T = K Q^T, one query per lane column, online softmax in
// fp32, O^T = V^T P^T), built on v_mfma_f32_32x32x64_f8f6f4, which runs at twice the bf16 rate:
//   * K / V tiles are 64 rows x 128 bytes; the transposing LDS read is ds_read_b64_tr_b8;
//   * P is quantised to e4m3 after scaling by 2^8 (P <= 1 so P * 256 <= 256 < 448), the factor is
//     folded into the exponent of exp2 and divided out with the row sum;
//   * Q, K, V carry one fp32 scale per (chunk of `scale_chunk_tokens` tokens, head).  The key axis
//     is walked in pieces that never cross a scale chunk (nor the boundary between the two key
//     segments), so inside a tile the K and V scales are wave-uniform scalars: the K scale joins
//     the softmax scale, the V scale (relative to the largest V scale of the range) joins the exp2
//     exponent, and the Q scale is a per-lane constant because a lane owns one query.
#include "attn_common.h"

namespace magi {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int BN = 64;
constexpr int ROW_BYTES = 128;  // D = 128 fp8
// A tile in LDS is eight groups of eight rows (what one wave-wide direct load fills: 64 lanes x 16 bytes), in key
// order.  The groups are spaced by a little more than their 1024 bytes and the MFMAs take the keys of a tile in an
// order that spreads every operand read over the groups (see the read bases below): consecutive groups start 16
// (K) or 32 (V) bytes further round the banks, so no swizzle is needed and every read address is the lane's base
// plus a constant.
constexpr int K_GROUP = 1024 + 16, V_GROUP = 1024 + 32;
constexpr int K_TILE_BYTES = (BN / 8) * K_GROUP, V_TILE_BYTES = (BN / 8) * V_GROUP;
constexpr int NW = 4;
constexpr int BM = 32 * NW;
constexpr int LOADS = 8 / NW;  // direct loads per wave per matrix per tile (8 rows each)
constexpr float P_SHIFT = 8.f;

// FASTP (with POW2): the probabilities come from a piecewise-linear exp2 built on the matrix pipe's scaling
// instead of the quarter-rate v_exp_f32: the score registers hold e4m3 codes (see the softmax below).
template <bool POW2, bool FASTP = false>
__global__ __launch_bounds__(64 * NW, 3) void attn_fwd_fp8_kernel(const AttnKernArgs a) {
  // Two (K tile, V tile) buffers as four separate objects that are only ever indexed statically: the compiler
  // then knows that a read of one buffer cannot alias the direct-to-LDS loads in flight to the other and does
  // not make it wait for them (with one array and a run-time buffer index every LDS read waited for vmcnt(0),
  // i.e. for the tile that had just been requested).
  __shared__ __attribute__((aligned(1024))) unsigned char sK0[K_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV0[V_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sK1[K_TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char sV1[V_TILE_BYTES];
  __shared__ int s_sel[LOCATE_WORDS];

  const int tid = threadIdx.x;
  const WorkItem wi = locate_work(a, BM, tid, s_sel);
  if (!wi.valid) return;
  const int h = wi.h, kvh = wi.kvh, q0 = wi.q0, qe = wi.qe, ks = wi.ks, ke = wi.ke;
  const long o_head = wi.o_head;

  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, i = l & 31, g = l >> 5;
  const int q_row = q0 + 32 * w + i;
  const bool row_ok = q_row < qe;

  if (ke <= ks) {
    if (row_ok) store_empty_row(a, wi, q_row, g);
    return;
  }

  // ---- Q fragments: lane (i, g) holds Q[row i][64kk + 32g .. +32] for kk = 0, 1 ----
  const int C = a.scale_chunk_tokens;
  const int qr = min(q_row, qe - 1);
  i32x8 qf[2];
  {
    const char* qp = a.q + (long)qr * a.qs_t + (long)h * a.qs_h + g * 32;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const i32x4 lo = *(const i32x4*)(qp + kk * 64);
      const i32x4 hi = *(const i32x4*)(qp + kk * 64 + 16);
      qf[kk] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }
  const float q_sc = a.q_scale[(long)(qr / C) * a.Hq + h];  // this lane's query scale

  // largest V scale of the key range (reference for the relative V scale folded into exp2)
  float v_max = 0.f;
  // (the side segment's chunks may have scale tables of their own: reached from the main tables by a constant
  // element offset from chunk scale_split_chunk on)
  for (int cidx = ks / C; cidx <= (ke - 1) / C; ++cidx)
    v_max = fmaxf(v_max, a.v_scale[(long)cidx * a.Hkv + kvh + (cidx < a.scale_split_chunk ? 0 : a.v2_scale_delta)]);
  const float log2_vmax = __builtin_amdgcn_logf(v_max);

  // ---- tile loader: wave w fills rows 8*(w + NW*j) .. +7; lane l sits at row +(l >> 3), slot l & 7 ----
  const int lrow = l >> 3, slot = l & 7;
  const int row_in_tile0 = 8 * w + lrow;
  const int kchunk = slot, vchunk = slot;  // rows are kept as they are in memory
  const long ks_t = a.ks_t, vs_t = a.vs_t;
  const int k_split = a.k_split;
  const long k2_delta = a.k2 ? (a.k2 - a.k) - (long)k_split * ks_t : 0;
  const long v2_delta = a.v2 ? (a.v2 - a.v) - (long)k_split * vs_t : 0;
  const char* const kcolp = a.k + (long)kvh * a.ks_h + kchunk * 16;
  const char* const vcolp = a.v + (long)kvh * a.vs_h + vchunk * 16;

  // The key range is walked in pieces [k0, pe) that stay inside one scale chunk and one key segment.
  auto piece_end = [&](int k0, int chunk) {  // chunk = k0 / C
    int pe = min(ke, (chunk + 1) * C);
    if (k0 < k_split) pe = min(pe, k_split);
    return pe;
  };
  const unsigned kvoff = (unsigned)row_in_tile0 * (unsigned)ks_t + (unsigned)(kchunk * 16);
  const unsigned vvoff = (unsigned)row_in_tile0 * (unsigned)vs_t + (unsigned)(vchunk * 16);
  const char* const kcol_u = a.k + (long)kvh * a.ks_h;  // wave-uniform column bases
  const char* const vcol_u = a.v + (long)kvh * a.vs_h;
  auto issue_tile = [&](int k0, int pe, auto BUFC) {
    constexpr int BUF = decltype(BUFC)::value;
    unsigned char* const dK = BUF ? sK1 : sK0;
    unsigned char* const dV = BUF ? sV1 : sV0;
    const bool second = k0 >= k_split;
    if (k0 + BN <= pe) {
      // full tile inside one piece: buffer-addressed direct loads (scalar base in the descriptor, one
      // loop-invariant 32-bit lane offset, the row group in the scalar offset) cost the SIMD next to nothing
      // to issue, unlike the same load with a 64-bit address per lane
      const __amdgpu_buffer_rsrc_t kr = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(kcol_u + (long)k0 * ks_t + (second ? k2_delta : 0)), 0, 0x7fffffff, 0x00020000);
      const __amdgpu_buffer_rsrc_t vr = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(vcol_u + (long)k0 * vs_t + (second ? v2_delta : 0)), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int j = 0; j < LOADS; ++j) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, LDS_PTR(void, dK + (w + j * NW) * K_GROUP), 16, kvoff,
                                                 (int)((unsigned)(8 * NW * j) * (unsigned)ks_t), 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, LDS_PTR(void, dV + (w + j * NW) * V_GROUP), 16, vvoff,
                                                 (int)((unsigned)(8 * NW * j) * (unsigned)vs_t), 0, 0);
      }
      return;
    }
    // ragged end of a piece: per-lane rows clamped to the piece's last key.  Still buffer loads: a global_load ... lds
    // anywhere in the kernel counts as a possible FLAT access to LDS, after which the compiler waits for ALL
    // outstanding LDS reads in front of every MFMA instead of counting them.
    const __amdgpu_buffer_rsrc_t kr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(kcol_u + (long)k0 * ks_t + (second ? k2_delta : 0)), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t vr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(vcol_u + (long)k0 * vs_t + (second ? v2_delta : 0)), 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      const int rel = min(row_in_tile0 + 8 * NW * j, pe - 1 - k0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, LDS_PTR(void, dK + (w + j * NW) * K_GROUP), 16,
                                               (unsigned)rel * (unsigned)ks_t + (unsigned)(kchunk * 16), 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, LDS_PTR(void, dV + (w + j * NW) * V_GROUP), 16,
                                               (unsigned)rel * (unsigned)vs_t + (unsigned)(vchunk * 16), 0, 0, 0);
    }
  };

  // ---- per-lane LDS read bases ----
  // Order of the keys of a tile.  Row i of the score MFMA of half t (t = 0, 1) is key 8 (i & 7) + 4 t + (i >> 3) of
  // the tile, i.e. row 4 t + (i >> 3) of group i & 7; register v of lane (query, g) of its result is row
  // i = 8 (v >> 2) + 4 g + (v & 3), i.e. key
  //     32 g + 8 (v & 3) + 4 t + (v >> 2)                                                             (*)
  // which is also the key that slot 16 t + v of this lane's 32 slots of the P and V^T operands stands for.
  // K (A operand): 32 bytes at byte 64 kk + 32 g of that row.  The 16 lanes one ds_read_b128 serves at a time
  // (i = 0 .. 15 or 16 .. 31, one g) touch eight groups (16 bytes apart in bank terms) x two rows 128 bytes apart: all
  // 64 banks once.
  const int base_k = (i & 7) * K_GROUP + (i >> 3) * ROW_BYTES + g * 32;
  // V^T via ds_read_b64_tr_b8: in a 16-lane group lane pair (2r', 2r'+1) supplies row r' of 8, lane gets d column
  // l & 15.  Read n2 delivers slots 16 t + 4 b + r for t = n2 >> 1, b = 2 (n2 & 1) + (r' >> 2), r = r' & 3: by (*) row
  // 4 t + b of group 4 g + r.  The 32 lanes one ds_read_b64 serves at a time touch four groups (32 bytes apart in bank
  // terms) x two rows x 32 bytes.
  const int lam = l & 15, rp = lam >> 1, dblk = (l >> 4) & 1;
  const int base_v = (4 * g + (rp & 3)) * V_GROUP + (rp >> 2) * ROW_BYTES + dblk * 16 + (l & 1) * 8;

  f32x16 o_acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[mb][v] = 0.f;
  // Running maximum in exp2-exponent units.  In the general mode it starts at -inf; in the power-of-two mode
  // the score MFMAs accumulate onto neg_m = shift - m in all 16 registers (a lane's registers all belong to one
  // query), so they deliver the exp2 exponent directly and a tile only pays for a correction when it raises a
  // row's maximum; there m starts at 0 and the first tile sets it.
  float m_run = POW2 ? 0.f : -__builtin_inff();
  float l_run = 0.f;
  // FASTP: the score MFMAs carry 3 more on their scale exponent and accumulate onto (7 + shift - m) * 8, so a
  // register holds 8 (e + 7) for the exponent e of its probability.  An e4m3 code c above 7 stands for
  // 2^(c / 8 - 7) * (1 + (c % 8) / 8), so that register, converted to an integer, IS the e4m3 code of exp2 with a linear
  // mantissa (at most 6.2 % above 2^e) on a grid of an eighth of an octave: one full-rate convert-and-insert per
  // score (v_cvt_pk_u8_f32; it saturates at 0, and the row maximum keeps the codes at or below 120 = 2^8).  The row
  // sum is taken from the same codes on the matrix pipe, so the average excess cancels in the normalisation.
  // (Measured and dropped: v_cvt_pknorm_u16_f32 on pairs of scores and one v_perm_b32 per four for their high bytes,
  // 3 instructions per 4 scores instead of 4, is 20 % slower: those two do not issue at the full rate.)
  constexpr float XS = FASTP ? 8.f : 1.f;   // units of the accumulator per exponent unit
  constexpr float XB = FASTP ? 56.f : 0.f;  // accumulator value of exponent 0
  constexpr int XE = FASTP ? 3 : 0;         // log2(XS), carried by the key scale's exponent
  f32x16 neg_m;
#pragma unroll
  for (int v = 0; v < 16; ++v) neg_m[v] = XB;
  float cur_shift = 0.f;
  int first = 1;  // (wave-uniform, kept as an integer so that it lives in a scalar register) no tile seen yet
  const int e_q = (__builtin_bit_cast(int, q_sc) >> 23) & 0xff;  // E8M0 code of the (power-of-two) query scale
  const bool wave_on = __builtin_amdgcn_readfirstlane(q0 + 32 * w) < __builtin_amdgcn_readfirstlane(qe);  // (a scalar condition)
  // Selector rows of the row-sum MFMA (16x16x128, half the time of a 32x32x64 one).  Read as the B operand of that
  // shape, the P registers of lane l are column l % 16, and of the 128 products of a column they are numbers
  // 16 (l / 16) .. + 15 (registers 0-3) and 64 + 16 (l / 16) .. + 15 (registers 4-7): queries j and j + 16 share column j
  // in alternating runs of 16.  An fp4 A operand holds products 32 (l / 16) .. + 31 of row l % 16 in four registers, the
  // first two covering a run of query j, the last two one of query j + 16.  Rows 0 and 8 of A are 1.0 (fp4 e2m1
  // 0b0010) on the runs of j, rows 4 and 12 on those of j + 16, all else 0, and register 0 of the result of lane l is
  // row 4 (l / 16) of column l % 16: the sum over all 64 keys of the query the lane holds.
  const int ones_lo = (l & 7) == 0 ? 0x22222222 : 0, ones_hi = (l & 7) == 4 ? 0x22222222 : 0;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float c_q = a.scale_log2 * q_sc;  // softmax scale * log2(e) * q scale

  // Per-piece quantities, refreshed by the first tile of a piece: the scale loads (vector memory loads, whose
  // wait would also wait for the tile just requested) and the divisions stay out of the steady-state loop.
  // They are wave uniform and live in scalar registers.
  int chunk = ks / C;
  bool new_piece = true;
  float c = 0.f, shift = 0.f, unshift = 0.f;
  int e_k = 0;
  int k0 = ks, pe = piece_end(ks, chunk);
  issue_tile(k0, pe, std::integral_constant<int, 0>{});
  auto tile_step = [&](auto BUFC) {
    constexpr int BUF = decltype(BUFC)::value;
    int k1 = k0 + BN, pe1 = pe, chunk1 = chunk;  // the tile after this one
    bool new_piece1 = false;
    if (k1 >= pe) {
      k1 = pe;
      chunk1 = chunk + (k1 == (chunk + 1) * C ? 1 : 0);
      pe1 = (k1 < ke) ? piece_end(k1, chunk1) : ke;
      new_piece1 = true;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (k1 < ke) issue_tile(k1, pe1, std::integral_constant<int, BUF ^ 1>{});
    if (wave_on) {
      const unsigned char* const Kt = BUF ? sK1 : sK0;
      const unsigned char* const Vt = BUF ? sV1 : sV0;
      if (new_piece) {
        auto uni = [](float x) {
          return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
        };
        const bool side = chunk >= a.scale_split_chunk;
        const float k_sc = uni(a.k_scale[(long)chunk * a.Hkv + kvh + (side ? a.k2_scale_delta : 0)]);
        const float v_sc = a.v_scale[(long)chunk * a.Hkv + kvh + (side ? a.v2_scale_delta : 0)];
        if constexpr (!POW2) c = c_q * k_sc;                             // per-lane score scale inside this piece
        shift = uni(P_SHIFT + __builtin_amdgcn_logf(v_sc) - log2_vmax);  // <= 8
        unshift = uni(__builtin_amdgcn_exp2f(-shift));
        e_k = max(((__builtin_bit_cast(int, k_sc) >> 23) & 0xff) + XE, 0);  // E8M0 code of a power-of-two key scale
      }

      auto read_k = [&](int t, int kk) -> i32x8 {
        const int o = base_k + kk * 64 + t * (4 * ROW_BYTES);
        const i32x4 lo = *LDS_PTR(const i32x4, Kt + o);
        const i32x4 hi = *LDS_PTR(const i32x4, Kt + (o + 16));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      };
      auto read_v = [&](int mb) -> i32x8 {
        const int o = base_v + mb * 32;
        i32x2 r[4];
#pragma unroll
        for (int n2 = 0; n2 < 4; ++n2)
          r[n2] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(i32x2, Vt + (o + (4 * (n2 >> 1) + 2 * (n2 & 1)) * ROW_BYTES)));
        return i32x8{r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
      };

      // three waves share a SIMD (<= 168 VGPRs): K operands are fetched two at a time, V operands two at a time,
      // the second pair under the first PV MFMAs
      i32x8 ka[2], va[2];
      f32x16 s_acc[2];
      i32x8 pb;
      ka[0] = read_k(0, 0);
      ka[1] = read_k(0, 1);
      if constexpr (POW2) {
        if (shift != cur_shift) {  // a new scale chunk (wave-uniform): re-base the accumulator offset
          const float ds = (shift - cur_shift) * XS;
#pragma unroll
          for (int v = 0; v < 16; ++v) neg_m[v] += ds;
          cur_shift = shift;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          s_acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka[0], qf[0], neg_m, 0, 0, 0, e_k, 0, e_q);  // (FASTP: e_k carries + 3)
          if (t == 0) ka[0] = read_k(1, 0);
          __builtin_amdgcn_sched_barrier(0);  // (keeps each operand read one MFMA ahead of its use, where it is written)
          s_acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka[1], qf[1], s_acc[t], 0, 0, 0, e_k, 0, e_q);
          if (t == 0) ka[1] = read_k(1, 1);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          s_acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka[0], qf[0], zero16, 0, 0, 0, 0, 0, 0);
          if (t == 0) ka[0] = read_k(1, 0);
          s_acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka[1], qf[1], s_acc[t], 0, 0, 0, 0, 0, 0);
          if (t == 0) ka[1] = read_k(1, 1);
        }
      }
      if (!POW2) {  // the power-of-two mode keeps 16 registers for neg_m and fetches V after the softmax instead
        va[0] = read_v(0);
        va[1] = read_v(1);
      }
      if (k0 + BN > pe) {  // ragged last tile of a piece
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = k0 + 32 * g + 8 * (v & 3) + 4 * t + (v >> 2);
            if (key >= pe) s_acc[t][v] = -__builtin_inff();
          }
      }
      // (starting from a constant: a maximum of two raw MFMA results first would cost a canonicalising v_max for each)
      float mx = -__builtin_inff();
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 16; v += 2) mx = max3(mx, s_acc[t][v], s_acc[t][v + 1]);
      mx = half_swap_max(mx);
      if constexpr (POW2) {
        // s_acc already holds exponent - m_run + shift; a value above `shift` is a new row maximum
        const float over = mx - (shift * XS + XB);
        const bool up = over > 0.f;
        int any_up;  // (scalar test of the lane mask; the compiler's own goes through two vector instructions)
        asm("s_cmp_lg_u64 %1, 0\n\ts_cselect_b32 %0, 1, 0" : "=s"(any_up) : "s"(__builtin_amdgcn_ballot_w64(up)) : "scc");
        if ((first | any_up) != 0) {
          const float delta = (first != 0 || up) ? over : 0.f;
          const float alpha = first != 0 ? 1.f : __builtin_amdgcn_exp2f(-delta * (1.f / XS));  // nothing to rescale on the first tile
          m_run += delta * (1.f / XS);
          l_run *= alpha;
#pragma unroll
          for (int v = 0; v < 16; ++v) neg_m[v] -= delta;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) s_acc[t][v] -= delta;
          if (first == 0) {
#pragma unroll
            for (int mb = 0; mb < 4; ++mb)
#pragma unroll
              for (int v = 0; v < 16; ++v) o_acc[mb][v] *= alpha;
          }
        }
        first = 0;
#pragma unroll
        for (int n = 0; n < 8; ++n) {  // dword n = slots 4n .. 4n+3 = s_acc[n >> 2][4 (n & 3) .. +3]
          const float x0 = s_acc[n >> 2][4 * (n & 3) + 0], x1 = s_acc[n >> 2][4 * (n & 3) + 1];
          const float x2 = s_acc[n >> 2][4 * (n & 3) + 2], x3 = s_acc[n >> 2][4 * (n & 3) + 3];
          if constexpr (FASTP) {  // (the conversion saturates at 0 for negative values and -inf: a probability of 0)
            unsigned u = __builtin_amdgcn_cvt_pk_u8_f32(x0, 0, 0u);
            u = __builtin_amdgcn_cvt_pk_u8_f32(x1, 1, u);
            u = __builtin_amdgcn_cvt_pk_u8_f32(x2, 2, u);
            pb[n] = (int)__builtin_amdgcn_cvt_pk_u8_f32(x3, 3, u);
          } else {
            const float p0 = __builtin_amdgcn_exp2f(x0), p1 = __builtin_amdgcn_exp2f(x1);
            const float p2 = __builtin_amdgcn_exp2f(x2), p3 = __builtin_amdgcn_exp2f(x3);
            // v_cvt_pk_fp8_f32 keeps the other half of its destination: start from p0's register (its high half is
            // overwritten by the second conversion) instead of a zeroed one
            int u = __builtin_bit_cast(int, p0);
            u = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, u, false);
            u = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, u, true);
            pb[n] = u;
          }
        }
      } else {
        const float m_new = fmaxf(m_run, mx * c);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        const float mc = m_new - shift;
        m_run = m_new;
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          const float p0 = __builtin_amdgcn_exp2f(s_acc[n >> 2][4 * (n & 3) + 0] * c - mc);
          const float p1 = __builtin_amdgcn_exp2f(s_acc[n >> 2][4 * (n & 3) + 1] * c - mc);
          const float p2 = __builtin_amdgcn_exp2f(s_acc[n >> 2][4 * (n & 3) + 2] * c - mc);
          const float p3 = __builtin_amdgcn_exp2f(s_acc[n >> 2][4 * (n & 3) + 3] * c - mc);
          int u = __builtin_bit_cast(int, p0);  // see the power-of-two branch
          u = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, u, false);
          u = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, u, true);
          pb[n] = u;
        }
        l_run *= alpha;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[mb][v] *= alpha;
        }
      }
      if (POW2) {
        va[0] = read_v(0);
        va[1] = read_v(1);
      }
      // Row sums on the matrix pipe: one more, half-length MFMA per tile (selector rows times P^T, see `ones_lo`; A in
      // fp4 so that it takes four registers) instead of 32 vector additions per lane.  The sum is over the
      // probabilities AS ROUNDED to e4m3, i.e. of exactly what the PV product uses, and both lanes of a query get the
      // full sum.  Issued ahead of the PV MFMAs and read after them.
      __builtin_amdgcn_sched_barrier(0);
      i32x8 ones;
#pragma unroll
      for (int n = 0; n < 8; ++n) ones[n] = n < 2 ? ones_lo : n < 4 ? ones_hi : 0;
      f32x4 rowsum = {0.f, 0.f, 0.f, 0.f};
      rowsum = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pb, rowsum, 4, 0, 0, 0, 0, 0);
      asm volatile("" : "+v"(rowsum));  // (an empty statement that holds the MFMA here: left alone it sinks to its use, and the wave waits there)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {  // two V operands in flight, in alternating registers
        o_acc[mb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va[mb & 1], pb, o_acc[mb], 0, 0, 0, 0, 0, 0);
        if (mb + 2 < 4) va[mb & 1] = read_v(mb + 2);
      }
      __builtin_amdgcn_sched_barrier(0);
      l_run += rowsum[0] * unshift;
    }
    k0 = k1;
    pe = pe1;
    chunk = chunk1;
    new_piece = new_piece1;
  };
  while (true) {  // unrolled by two: every LDS buffer index is a compile-time constant
    tile_step(std::integral_constant<int, 0>{});
    if (k0 >= ke) break;
    tile_step(std::integral_constant<int, 1>{});
    if (k0 >= ke) break;
  }

  if (!wave_on) return;
  const float l_tot = l_run;  // (the row-sum MFMA hands every lane the sum over all keys of its query)
  const float inv = v_max * __builtin_amdgcn_exp2f(-P_SHIFT) / l_tot;
  // A lane holds four consecutive features per (mb, b), its partner in the other half wave the next four: the
  // halves trade the odd-b registers of the lower half for the even-b registers of the upper one, after which
  // every lane owns eight consecutive features and stores 16 bytes at a time.  (The row address is derived from
  // an opaque copy of the lane index so that it is computed here and not carried through the main loop.)
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
      a.lse[(long)h * a.total_q + q_row] = (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
  }
}

// ------------------------------------------------------------------------------------------------
// Quantiser: absmax per (chunk, head) -> scale = max(absmax, tiny) / 448; y = e4m3(clamp(x / scale)).
// ------------------------------------------------------------------------------------------------
constexpr int QT = 256;

__global__ __launch_bounds__(QT) void fill_zero_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * QT + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// grid (slices, H, n_chunks); 16 lanes x 16 bytes per (token, head) row; result: max |x| bits in amax[c*H + h]
__global__ __launch_bounds__(QT) void absmax_kernel(const char* x, long xs_t, long xs_h, unsigned* amax, int T, int H,
                                                    int chunk_tokens) {
  __shared__ unsigned s_red[QT / 64];
  const int c = blockIdx.z, h = blockIdx.y;
  const int t_begin = c * chunk_tokens, t_end = min(T, t_begin + chunk_tokens);
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4;
  unsigned m = 0u;
  for (int t = t_begin + blockIdx.x * (QT / 16) + sub; t < t_end; t += gridDim.x * (QT / 16)) {
    const u32x4 v = *(const u32x4*)(x + (long)t * xs_t + (long)h * xs_h + lane16 * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      m = max(m, (v[j] << 16) & 0x7fffffffu);
      m = max(m, v[j] & 0x7fff0000u);
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o));
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int j = 1; j < QT / 64; ++j) m = max(m, s_red[j]);
    atomicMax(&amax[c * H + h], m);  // non-negative floats order like their bit patterns
  }
}

// absmax of a (chunk, head) group -> its scale
__device__ __forceinline__ float scale_of_absmax(float amax, float premul, int pow2) {
  float f = fmaxf(amax * fabsf(premul) / 448.f, 1e-12f);
  if (pow2) {  // round up to a power of two
    unsigned b = __builtin_bit_cast(unsigned, f);
    b = ((b >> 23) + ((b & 0x7fffffu) ? 1u : 0u)) << 23;
    f = __builtin_bit_cast(float, b);
  }
  return f;
}

__global__ __launch_bounds__(QT) void finalize_scales_kernel(float* scales, int n, float premul, int pow2) {
  const int i = blockIdx.x * QT + threadIdx.x;
  if (i >= n) return;
  scales[i] = scale_of_absmax(scales[i], premul, pow2);
}

// 16 bytes of bf16 (8 elements) -> 8 bytes of e4m3: y = sat(x * premul / sc)
__device__ __forceinline__ u32x2 quantize8(const u32x4 v, float premul, float sc) {
  float fv[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    fv[2 * j] = __builtin_bit_cast(float, v[j] << 16);
    fv[2 * j + 1] = __builtin_bit_cast(float, v[j] & 0xffff0000u);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) fv[j] = fminf(fmaxf(fv[j] * premul / sc, -448.f), 448.f);
  u32x2 o;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    int u = 0;
    u = __builtin_amdgcn_cvt_pk_fp8_f32(fv[4 * j], fv[4 * j + 1], u, false);
    u = __builtin_amdgcn_cvt_pk_fp8_f32(fv[4 * j + 2], fv[4 * j + 3], u, true);
    o[j] = (unsigned)u;
  }
  return o;
}

// one thread per 8 elements
__global__ __launch_bounds__(QT) void quantize_kernel(const char* x, long xs_t, long xs_h, char* y, const float* scales,
                                                      int T, int H, int chunk_tokens, float premul) {
  const long gid = (long)blockIdx.x * QT + threadIdx.x;
  const long row = gid >> 4;
  const int part = (int)(gid & 15);
  if (row >= (long)T * H) return;
  const int t = (int)(row / H), h = (int)(row % H);
  const float sc = scales[(long)(t / chunk_tokens) * H + h];
  const u32x4 v = *(const u32x4*)(x + (long)t * xs_t + (long)h * xs_h + part * 16);
  *(u32x2*)(y + row * 128 + part * 8) = quantize8(v, premul, sc);
}

// The whole job in one launch with no memory beyond the inputs and outputs: a workgroup takes the absmax of its
// (chunk, head) group (a video chunk of one head is 5.5 MB at the 720p shape), reduces it through LDS, and
// quantises with the resulting scale.  To fill the chip when there are few groups, gridDim.z workgroups share a
// group: each of them takes the absmax of the WHOLE group (a maximum does not depend on the order, so all arrive
// at the same scale; the repeated reads are served by the caches, HBM sees the group once) and quantises its own
// slice of the rows; slice 0 writes the scale.  Groups that start at or after token n_first go to the second
// destination.
constexpr int QT1 = 1024;
constexpr int QROWS = QT1 / 16;  // rows per pass of a workgroup
__global__ __launch_bounds__(QT1) void quantize_groups_kernel(const char* x, long xs_t, long xs_h, char* y, float* scales,
                                                              int T, int H, int chunk_tokens, float premul, int pow2,
                                                              int n_first, char* y2, float* scales2) {
  __shared__ unsigned s_red[QT1 / 64];
  const int h = blockIdx.x, c = blockIdx.y;
  const int t_begin = c * chunk_tokens, t_end = min(T, t_begin + chunk_tokens);
  const int lane16 = threadIdx.x & 15, sub = threadIdx.x >> 4;
  const char* const xcol = x + (long)h * xs_h + lane16 * 16;
  unsigned m = 0u;
  auto fold = [&](const u32x4 v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      m = max(m, (v[j] << 16) & 0x7fffffffu);
      m = max(m, v[j] & 0x7fff0000u);
    }
  };
  constexpr int UN = 8;  // loads in flight per lane
  int t = t_begin + sub;
  for (; t + (UN - 1) * QROWS < t_end; t += UN * QROWS) {
    u32x4 v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = *(const u32x4*)(xcol + (long)(t + u * QROWS) * xs_t);
#pragma unroll
    for (int u = 0; u < UN; ++u) fold(v[u]);
  }
  for (; t < t_end; t += QROWS) fold(*(const u32x4*)(xcol + (long)t * xs_t));
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o));
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = m;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < QT1 / 64; ++j) m = max(m, s_red[j]);  // non-negative floats order like their bit patterns
  const float sc = scale_of_absmax(__builtin_bit_cast(float, m), premul, pow2);
  const bool second = t_begin >= n_first;
  const int t_off = second ? n_first : 0;
  if (threadIdx.x == 0 && blockIdx.z == 0) (second ? scales2 : scales)[(long)(c - t_off / chunk_tokens) * H + h] = sc;
  // this workgroup's slice of the rows
  const int per = (t_end - t_begin + (int)gridDim.z - 1) / (int)gridDim.z;
  const int s_begin = t_begin + (int)blockIdx.z * per, s_end = min(t_end, s_begin + per);
  char* const ycol = (second ? y2 : y) + (long)h * 128 + lane16 * 8 - (long)t_off * H * 128;
  t = s_begin + sub;
  for (; t + (UN - 1) * QROWS < s_end; t += UN * QROWS) {
    u32x4 v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = *(const u32x4*)(xcol + (long)(t + u * QROWS) * xs_t);
#pragma unroll
    for (int u = 0; u < UN; ++u) *(u32x2*)(ycol + (long)(t + u * QROWS) * H * 128) = quantize8(v[u], premul, sc);
  }
  for (; t < s_end; t += QROWS)
    *(u32x2*)(ycol + (long)t * H * 128) = quantize8(*(const u32x4*)(xcol + (long)t * xs_t), premul, sc);
}

}  // namespace

hipError_t launch_attn_fwd_fp8(const AttnKernArgs& a, hipStream_t stream) {
  const unsigned grid = a.per_xcd * 8u;
  if ((a.flags & 1) && (a.flags & 4))
    hipLaunchKernelGGL((attn_fwd_fp8_kernel<true, true>), dim3(grid), dim3(64 * NW), 0, stream, a);
  else if (a.flags & 1)
    hipLaunchKernelGGL(attn_fwd_fp8_kernel<true>, dim3(grid), dim3(64 * NW), 0, stream, a);
  else
    hipLaunchKernelGGL(attn_fwd_fp8_kernel<false>, dim3(grid), dim3(64 * NW), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_quantize_fp8(const char* x, long x_stride_t, long x_stride_h, char* y, float* scales, int T, int H,
                               int chunk_tokens, float premul, int pow2_scales, int n_first, char* y2, float* scales2,
                               bool one_launch, int compute_units, hipStream_t stream, int* n_launches) {
  const int n_chunks = (T + chunk_tokens - 1) / chunk_tokens;
  const int n = n_chunks * H;
  *n_launches = 0;
  if (n <= 0) return hipSuccess;
  // Unless asked for, one launch only when a group is small enough for one workgroup's two passes and there are
  // enough groups to spread over the chip (a second destination is served by that kernel alone); both paths give
  // the same bytes.
  if (n_first < T || (min(chunk_tokens, T) <= 8192 && (n >= 64 || (long)T * H <= 65536))) one_launch = true;
  if (one_launch) {
    if (n_chunks > 65535) return hipErrorInvalidValue;
    // workgroups per group: towards one per CU over the launch (every workgroup reads its whole group for the absmax, so
    // a second one per CU doubles what a CU pulls through its caches: 162 instead of 105 us at the 720p shape), each
    // slice at least four passes long
    int share = (compute_units + n - 1) / n;
    share = max(1, min(share, min(16, min(chunk_tokens, T) / (4 * QROWS))));
    hipLaunchKernelGGL(quantize_groups_kernel, dim3(H, n_chunks, share), dim3(QT1), 0, stream, x, x_stride_t, x_stride_h, y,
                       scales, T, H, chunk_tokens, premul, pow2_scales, n_first, y2, scales2);
    *n_launches = 1;
    return hipGetLastError();
  }
  hipLaunchKernelGGL(fill_zero_kernel, dim3((n + QT - 1) / QT), dim3(QT), 0, stream, (unsigned*)scales, n);
  const int rows_per_pass = QT / 16;
  int slices = (min(chunk_tokens, T) + rows_per_pass * 8 - 1) / (rows_per_pass * 8);
  slices = max(1, min(slices, 256));
  hipLaunchKernelGGL(absmax_kernel, dim3(slices, H, n_chunks), dim3(QT), 0, stream, x, x_stride_t, x_stride_h,
                     (unsigned*)scales, T, H, chunk_tokens);
  hipLaunchKernelGGL(finalize_scales_kernel, dim3((n + QT - 1) / QT), dim3(QT), 0, stream, scales, n, premul, pow2_scales);
  const long threads = (long)T * H * 16;
  hipLaunchKernelGGL(quantize_kernel, dim3((unsigned)((threads + QT - 1) / QT)), dim3(QT), 0, stream, x, x_stride_t,
                     x_stride_h, y, scales, T, H, chunk_tokens, premul);
  *n_launches = 4;
  return hipGetLastError();
}

}  // namespace magi
