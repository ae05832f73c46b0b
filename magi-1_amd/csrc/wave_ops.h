// Small wavefront-level device helpers shared by the attention kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>

namespace magi {

// Wave-wide max of the two half-waves' values (lane i and lane i + 32 hold the same query).
// v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second; issued through
// inline assembly because the compiler builtin hands back its first result for both outputs (seen with ROCm
// 7.2).  The inputs must be VALU results (not MFMA results); the s_nop covers the VALU-write -> swap-read
// wait states that the compiler inserts for the builtin.
__device__ __forceinline__ float half_swap_max(float x) {
  float lo = x, hi = x;
  // (the maximum inside the statement: fmaxf would first quiet both operands, two more instructions)
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1\n\tv_max_f32 %0, %0, %1" : "+v"(lo), "+v"(hi));
  return lo;
}

// Exchange lanes 32..63 of `a` with lanes 0..31 of `b` (both must be VALU results, see above).
__device__ __forceinline__ void half_swap(unsigned& a, unsigned& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// max of three; written as nested fmaxf so that the compiler (which knows the wait states an MFMA result
// needs before a VALU instruction may read it; it does not check inline assembly for them) forms v_max3_f32
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

}  // namespace magi
