// Measurement only, no part of libmagi_attn.so: what a loop of nothing but MFMAs sustains on this GPU, built as its
// own small shared library (libmagi_probe.so) that the benchmark loads after its timed region.
//
// The MI355X peak figures (2.5 PFLOP/s bf16, 5.0 PFLOP/s fp8, dense) are 256 CUs x 4 SIMDs x FLOP per clock at
// 2.4 GHz.  Under its board power limit the part does not hold that clock on real data: how far an MFMA-only loop
// gets depends on the operand values (all-zero operands toggle nothing).  The rate measured here, on the box the
// benchmark runs on, is the ceiling for any kernel made of the same MFMAs; the attention kernels' rates are
// reported against it beside the nominal peak.
//
// One wave per SIMD (256 workgroups of 256 threads on 256 CUs), operands in registers, enough independent
// accumulators that no MFMA waits for another, launches of ~30 ms so that the power controller settles.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "magi_probe.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

constexpr int OPERAND_WORDS = 1 << 20;

// KIND 0: v_mfma_f32_32x32x16_bf16 (the attention kernels' MFMA), 64 per round over 8 accumulators
// KIND 1: v_mfma_f32_16x16x32_bf16, 128 per round over 16 accumulators (the same FLOPs per round)
// KIND 2: v_mfma_scale_f32_32x32x64_f8f6f4 on e4m3 operands (the fp8 kernel's MFMA), 32 per round over 8 accumulators
// KIND 3: v_mfma_scale_f32_16x16x128_f8f6f4 on e4m3 operands, 64 per round over 16 accumulators (the same FLOPs)
template <int KIND>
__global__ __launch_bounds__(256, 1) void mfma_only_kernel(const uint32_t* operands, float* sink, int rounds) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  unsigned ra[8][8], rb[8][8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int v = 0; v < 8; ++v) {
      ra[j][v] = operands ? operands[(t * 67 + j * 8 + v) & (OPERAND_WORDS - 1)] : 0u;
      rb[j][v] = operands ? operands[(t * 131 + j * 8 + v + 4) & (OPERAND_WORDS - 1)] : 0u;
    }
  float r = 0.f;
  if constexpr (KIND == 3) {
    f32x4 acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < rounds; ++it) {
      static_for<0, 64>([&](auto sc) __attribute__((always_inline)) {
        constexpr int s = decltype(sc)::value;
        acc[s & 15] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(*(i32x8*)ra[s & 7], *(i32x8*)rb[(s >> 3) & 7], acc[s & 15],
                                                                       0, 0, 0, 0, 0, 0);
      });
      if ((it & 63) == 63)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] *= 1e-3f;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) r += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  } else if constexpr (KIND == 1) {
    f32x4 acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < rounds; ++it) {
      static_for<0, 128>([&](auto sc) __attribute__((always_inline)) {
        constexpr int s = decltype(sc)::value;
        const bf16x8 a = __builtin_bit_cast(bf16x8, *(u32x4*)&ra[s & 7][4 * ((s >> 6) & 1)]);
        const bf16x8 b = __builtin_bit_cast(bf16x8, *(u32x4*)&rb[(s >> 3) & 7][4 * ((s >> 6) & 1)]);
        acc[s & 15] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[s & 15], 0, 0, 0);
      });
      if ((it & 63) == 63)  // keep the sums finite (an overflow to inf would change the data-dependent power)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] *= 1e-3f;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) r += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  } else {
    f32x16 acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
    for (int it = 0; it < rounds; ++it) {
      static_for<0, 64>([&](auto sc) __attribute__((always_inline)) {
        constexpr int s = decltype(sc)::value;
        if constexpr (KIND == 2) {
          if constexpr (s % 2 == 0)  // (a 32x32x64 fp8 MFMA does the work of two bf16 32x32x16 ones)
            acc[(s / 2) & 7] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(*(i32x8*)ra[s & 7], *(i32x8*)rb[(s >> 3) & 7],
                                                                              acc[(s / 2) & 7], 0, 0, 0, 0, 0, 0);
        } else {
          acc[s & 7] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, *(u32x4*)ra[s & 7]),
                                                               __builtin_bit_cast(bf16x8, *(u32x4*)rb[(s >> 3) & 7]), acc[s & 7], 0, 0, 0);
        }
      });
      if ((it & 63) == 63)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] *= 1e-3f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) r += acc[j][v];
  }
  sink[t] = r;
}

}  // namespace

extern "C" int magi_probe_mfma_only(int kind, const uint32_t* operands, float* sink, int rounds, int launches,
                                    void* stream, float* ms_per_launch, double* flop_per_launch) {
  if (kind < 0 || kind > 3 || !sink || rounds <= 0 || launches <= 0 || !ms_per_launch || !flop_per_launch) return -22;
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -5;
  const dim3 grid(MAGI_PROBE_WORKGROUPS), block(256);
  auto launch = [&]() {
    if (kind == 0) hipLaunchKernelGGL(mfma_only_kernel<0>, grid, block, 0, st, operands, sink, rounds);
    if (kind == 1) hipLaunchKernelGGL(mfma_only_kernel<1>, grid, block, 0, st, operands, sink, rounds);
    if (kind == 2) hipLaunchKernelGGL(mfma_only_kernel<2>, grid, block, 0, st, operands, sink, rounds);
    if (kind == 3) hipLaunchKernelGGL(mfma_only_kernel<3>, grid, block, 0, st, operands, sink, rounds);
  };
  launch();  // warm-up, also brings the board to its operating point
  (void)hipEventRecord(e0, st);
  for (int i = 0; i < launches; ++i) launch();
  (void)hipEventRecord(e1, st);
  hipError_t e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (e != hipSuccess || hipGetLastError() != hipSuccess) return -5;
  *ms_per_launch = ms / launches;
  // per round and wave: 64 x 32x32x16 = 128 x 16x16x32; 32 x 32x32x64 = 64 x 16x16x128 (fp8: twice the FLOPs)
  const double per_round = (kind >= 2 ? 2.0 : 1.0) * 64.0 * 2.0 * 32 * 32 * 16;
  *flop_per_launch = per_round * rounds * MAGI_PROBE_WORKGROUPS * 4.0;
  return 0;
}
