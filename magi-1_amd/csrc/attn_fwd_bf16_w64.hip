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
// The library's default bounded-score kernel is the 16x16x32 form of attn_fwd_bf16_x16.hip (less energy per FLOP on
// this power-limited part); this 32x32x16 form issues half as many MFMAs and serves the 512-row workgroups and
// callers that ask for it (MAGI_ATTN_BOUNDED_MFMA32).  q must carry the softmax scale (MAGI_ATTN_Q_PRESCALED).
//
// Every instantiation is for BOUNDED scores (magi_attn_args.score_bound): the caller guarantees
// |q . k| <= score_bound (an exp2 exponent, q carrying softmax_scale * log2(e) by the time the MFMAs see it),
// small enough that 2^score neither overflows nor underflows in fp32 / bf16.  The softmax is shift invariant, so
// no running maximum is needed at all: p = 2^score, no row max, no rescale of O, no offset registers; the result
// is the same softmax.  QK-normed attention satisfies this by construction (|q| and |k| are fixed by the norm
// parameters).  Callers without such a promise get the online-softmax kernel of attn_fwd_bf16.hip.
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

template <int NW, int OCC, int VPRE, int RD>
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
  __shared__ int s_sel[LOCATE_WORDS];

  const int tid = threadIdx.x;
  const WorkItem wi = locate_work(a, BM, tid, s_sel);
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
  float l_run[2] = {0.f, 0.f};                               // this lane's share of the running sums
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
        // are finite; their probabilities are set to zero after the exp.
        const int kbase = k0 + 32 * t;
        auto softmax = [&](auto rc) __attribute__((always_inline)) {
          constexpr bool RAGGED = decltype(rc)::value;
          // register v of a lane holds key kbase + 8 (v / 4) + (v % 4) + 4 g (g = lane / 32): which of the two lane
          // halves keep their value is a scalar question per register
          const int left = ke - kbase;  // valid keys in this half (may be <= 0)
          auto prob = [&](float x, int v) __attribute__((always_inline)) -> float {
            const float p = __builtin_amdgcn_exp2f(x);
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
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
              const float p0 = prob(sc[b][e], e), p1 = prob(sc[b][e + 1], e + 1);
              psum += p0;
              psum2 += p1;
              sc[b][8 * (e >> 3) + ((e & 7) >> 1)] = __builtin_bit_cast(float, pack_bf16x2(p0, p1));
            }
            l_run[b] += psum + psum2;
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
          __builtin_amdgcn_logf(l_tot) * 0.6931471805599453f;
  }
}

}  // namespace

hipError_t launch_attn_fwd_bf16_w64(const AttnKernArgs& a, hipStream_t stream) {
  const dim3 grid(a.per_xcd * 8u);
  if (a.block_m == 512)  // 8 waves, one workgroup per CU: every K / V tile fetched once for 512 rows
    hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<8, 1, 0, 4>), grid, dim3(512), 0, stream, a);
  else  // 4 waves, two workgroups per CU
    hipLaunchKernelGGL((attn_fwd_bf16_w64_kernel<4, 2, 0, 4>), grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace magi
