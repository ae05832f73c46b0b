// Device-side pieces shared by the range-attention kernels (gfx950): vector types, the mapping from a
// workgroup to its piece of work, and small helpers.  Every kernel that includes this file decomposes the
// launch the same way, so the host side (api.cpp) sizes one grid for all of them.
#pragma once
#include "kernels.h"
#include "wave_ops.h"

#include <type_traits>

namespace magi {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((T __attribute__((address_space(3)))*)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int MAX_SORT = 256;  // ranges are ranked by key span inside the kernel up to this many

__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
  f32x2 x = {a, b};
  bf16x2 r = __builtin_convertvector(x, bf16x2);
  return __builtin_bit_cast(unsigned, r);
}

// range i of a device-side range list (pairs or cumulative), clamped to [0, total]
__device__ __forceinline__ void load_range(const int* r, int mode, int i, int total, int& s, int& e) {
  if (mode == 0) {
    s = r[2 * i];
    e = r[2 * i + 1];
  } else {
    s = r[i];
    e = r[i + 1];
  }
  s = max(0, min(s, total));
  e = max(s, min(e, total));
}

// f(integral_constant<int, I>) for I = B .. E-1, unrolled at compile time
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

// s_waitcnt vmcnt(N), leaving the other counters alone
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}

// p0 + p1 + acc for a packed pair of bf16 values
__device__ __forceinline__ float pair_sum(unsigned pk, float acc) {
  const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk), one, acc, false);
}

// A launch behind a measured score bound: true when this kernel is not the one the bound selects (every thread of
// the grid sees the same two values, so the whole launch returns).  NaN lengths fail the comparison and select the
// online-softmax kernel.
__device__ __forceinline__ bool gate_closed(const AttnKernArgs& a) {
  if (!a.gate) return false;
  const float b = __builtin_sqrtf(a.gate[0] * a.gate[1]) * a.scale_log2 * 1.01f;
  const bool fits = b <= 64.0f;  // MAGI_SCORE_BOUND_MAX
  return fits != (a.gate_want != 0);
}

// What one workgroup works on: q rows [q0, min(q0 + BM, qe)) of head h against keys [ks, ke) of kv head kvh.
struct WorkItem {
  int h, kvh;
  int q0, qe, ks, ke;
  long o_head;  // byte offset of head h inside a row of `out`
  bool valid;   // false: nothing to do (grid padding, or the q tile lies beyond the range)
};

// blockIdx -> (kv head, range slot, q tile, q head within the GQA group), laid out so that the workgroups an
// XCD receives (blockIdx % 8) share a KV head and walk the same keys at about the same time (each XCD has its
// own L2).  Ranges are visited longest key span first (ties by index), ranked here from the device-side list.
// Every thread of the workgroup must call this (it contains a barrier); s_sel is LOCATE_WORDS ints of LDS.
constexpr int LOCATE_WORDS = 4;
__device__ __forceinline__ WorkItem locate_work(const AttnKernArgs& a, int BM, int tid, int* s_sel) {
  WorkItem wi;
  wi.valid = false;
  const unsigned id = blockIdx.x;
  const unsigned f = (id & 7u) * a.per_xcd + (id >> 3);
  if (f >= a.total_wgs) return wi;
  const unsigned per_range = (unsigned)a.tiles_per_range * (unsigned)a.G;
  const unsigned per_kvh = (unsigned)a.n_ranges * per_range;
  const unsigned kvh = f / per_kvh;
  unsigned rem = f - kvh * per_kvh;
  const unsigned rslot = rem / per_range;
  rem -= rslot * per_range;
  const unsigned tile = rem / (unsigned)a.G;
  const unsigned hg = rem - tile * (unsigned)a.G;
  wi.kvh = (int)kvh;
  wi.h = (int)(kvh * a.G + hg);
  wi.o_head = a.out_group > 0 ? (long)(wi.h / a.out_group) * a.os_g + (long)(wi.h % a.out_group) * a.os_h
                              : (long)wi.h * a.os_h;
  int qs;
  if (a.n_ranges <= MAX_SORT) {
    // thread t ranks range t; the one whose rank is this workgroup's slot publishes the range itself (its q rows were
    // requested together with the key ranges: one memory latency for everything)
    if (tid < a.n_ranges) {
      int s, e, q_s, q_e;
      load_range(a.k_ranges, a.ranges_mode, tid, a.total_k, s, e);
      load_range(a.q_ranges, a.ranges_mode, tid, a.total_q, q_s, q_e);
      const int my = e - s;
      int rank = 0;
      for (int j = 0; j < a.n_ranges; ++j) {
        int sj, ej;
        load_range(a.k_ranges, a.ranges_mode, j, a.total_k, sj, ej);
        const int lj = ej - sj;
        rank += (lj > my) || (lj == my && j < tid);
      }
      if (rank == (int)rslot) {
        s_sel[0] = q_s;
        s_sel[1] = q_e;
        s_sel[2] = s;
        s_sel[3] = e;
      }
    }
    __syncthreads();
    qs = __builtin_amdgcn_readfirstlane(s_sel[0]);
    wi.qe = __builtin_amdgcn_readfirstlane(s_sel[1]);
    wi.ks = __builtin_amdgcn_readfirstlane(s_sel[2]);
    wi.ke = __builtin_amdgcn_readfirstlane(s_sel[3]);
  } else {
    const int ridx = a.n_ranges - 1 - (int)rslot;
    load_range(a.q_ranges, a.ranges_mode, ridx, a.total_q, qs, wi.qe);
    load_range(a.k_ranges, a.ranges_mode, ridx, a.total_k, wi.ks, wi.ke);
  }
  wi.q0 = qs + (int)tile * BM;
  wi.valid = wi.q0 < wi.qe;
  return wi;
}

// A q row whose range has no keys: zeros, lse = -inf.  Lane (row, g) writes half g of the 256-byte row.
__device__ __forceinline__ void store_empty_row(const AttnKernArgs& a, const WorkItem& wi, int q_row, int g) {
  char* op = a.out + (long)q_row * a.os_t + wi.o_head + g * 128;
#pragma unroll
  for (int c = 0; c < 8; ++c) *(u32x4*)(op + c * 16) = u32x4{0, 0, 0, 0};
  if (a.lse && g == 0) a.lse[(long)wi.h * a.total_q + q_row] = -__builtin_inff();
}

}  // namespace
}  // namespace magi
