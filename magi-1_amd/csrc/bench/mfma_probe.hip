// Stand-alone measurements behind the design of the attention kernels (gfx950 / MI355X):
//   1. what an MFMA-only loop sustains at the board's power limit, on all-zero and on random operands
//      (bf16 32x32x16 and fp8 32x32x64): the ceiling any kernel made of these MFMAs lives under;
//   2. which vector instructions execute beside an MFMA of another accumulator for free and which hold the
//      matrix pipe up (one wave per SIMD, one companion kind per MFMA slot).
// Build: make -C magi-1_amd/csrc probe      Run: magi-1_amd/csrc/bench/mfma_probe
// No part of libmagi_attn.so; prints a table.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

enum Companion { NONE, EXP2, CVT_PK_BF16, DOT2_BF16, ADD, FMA, XOR, MAX3, LDS_B128, LDS_TR_B64, SOFTMAX_MIX };

// bf16: 64 MFMA slots per round over 8 accumulators; companion C rides in every slot.
template <int C, bool FP8>
__global__ __launch_bounds__(256, 1) void probe(const unsigned* seed, float* out, int iters, int zero) {
  __shared__ __attribute__((aligned(1024))) unsigned char lds[32768];
  const int t = blockIdx.x * blockDim.x + threadIdx.x, l = threadIdx.x & 63;
  for (int i = threadIdx.x; i < 32768 / 4; i += blockDim.x) ((unsigned*)lds)[i] = zero ? 0u : seed[(i * 13 + t) & 0xfffff];
  __syncthreads();
  f32x16 acc[8];
  for (int j = 0; j < 8; ++j)
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
  unsigned ra[8][8], rb[8][8];
  for (int j = 0; j < 8; ++j)
    for (int v = 0; v < 8; ++v) {
      ra[j][v] = zero ? 0u : seed[(t * 67 + j * 8 + v) & 0xfffff];
      rb[j][v] = zero ? 0u : seed[(t * 131 + j * 8 + v + 4) & 0xfffff];
    }
  float x[64];
  for (int j = 0; j < 64; ++j) x[j] = 0.001f * ((l + j) & 31);
  float sum = 0.f, mx = 0.f;
  unsigned pk[4] = {0, 0, 0, 0};
  bf16x8 frag[4];
  for (int j = 0; j < 4; ++j) frag[j] = __builtin_bit_cast(bf16x8, *(uint4*)ra[j]);
  for (int it = 0; it < iters; ++it) {
    static_for<0, 64>([&](auto sc) __attribute__((always_inline)) {
      constexpr int s = decltype(sc)::value;
      if constexpr (FP8) {
        if constexpr (s % 2 == 0)  // (a 32x32x64 fp8 MFMA lasts two bf16 slots)
          acc[(s / 2) & 7] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(*(i32x8*)ra[s & 7], *(i32x8*)rb[(s >> 3) & 7], acc[(s / 2) & 7], 0, 0, 0, 0, 0, 0);
      } else {
        const bf16x8 a = (C == LDS_B128 || C == LDS_TR_B64) ? frag[s & 3] : __builtin_bit_cast(bf16x8, *(uint4*)ra[s & 7]);
        acc[s & 7] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, __builtin_bit_cast(bf16x8, *(uint4*)rb[(s >> 3) & 7]), acc[s & 7], 0, 0, 0);
      }
      if constexpr (C == EXP2 || C == SOFTMAX_MIX) x[s] = __builtin_amdgcn_exp2f(x[s]);
      if constexpr (C == CVT_PK_BF16 || (C == SOFTMAX_MIX && s % 2 == 0)) {
        f32x2 p = {x[(s + 60) & 63], x[(s + 61) & 63]};
        pk[s & 3] = __builtin_bit_cast(unsigned, __builtin_convertvector(p, bf16x2));
      }
      if constexpr (C == DOT2_BF16) {
        const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
        sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk[s & 3]), one, sum, false);
      }
      if constexpr (C == ADD || C == SOFTMAX_MIX) sum += x[(s + 50) & 63];
      if constexpr (C == FMA) x[s] = __builtin_fmaf(x[s], 0.99f, 0.001f);
      if constexpr (C == XOR) pk[s & 3] ^= (unsigned)(s * 32 + 1);
      if constexpr (C == MAX3) mx = fmaxf(fmaxf(mx, x[(s + 40) & 63]), x[(s + 41) & 63]);
      if constexpr (C == LDS_B128 && s % 2 == 1)  // one 1 KB operand read per two MFMAs, as the 64-row kernels do
        frag[(s >> 1) & 3] = *(const bf16x8 __attribute__((address_space(3)))*)(lds + ((l * 16 + (s >> 1) * 1024) & 32767));
      if constexpr (C == LDS_TR_B64 && s % 2 == 1) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(lds + ((l * 8 + (s >> 1) * 1024) & 32767)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(lds + ((l * 8 + (s >> 1) * 1024 + 512) & 32767)));
        frag[(s >> 1) & 3] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if ((it & 63) == 63) {  // keep the values in range (overflow to inf would change the data-dependent power)
      for (int j = 0; j < 8; ++j)
        for (int v = 0; v < 16; ++v) acc[j][v] *= 1e-3f;
      for (int j = 0; j < 64; ++j) x[j] = 0.001f * ((l + j + it) & 31);
    }
  }
  float r = sum + mx + pk[0] + pk[1] + pk[2] + pk[3];
  for (int j = 0; j < 8; ++j)
    for (int v = 0; v < 16; ++v) r += acc[j][v];
  for (int j = 0; j < 64; ++j) r += x[j];
  out[t] = r + (float)frag[0][0];
}

template <int C, bool FP8>
double run(const char* name, const unsigned* seed, float* out, int zero, double base) {
  const int iters = FP8 ? 12000 : 24000, grid = 256;  // about 30 ms per launch: long enough to sit at the power limit
  float best = 1e30f;
  for (int rep = 0; rep < 4; ++rep) {
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL((probe<C, FP8>), dim3(grid), dim3(256), 0, 0, seed, out, iters, zero);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (rep > 0 && ms < best) best = ms;
  }
  const double flop = (FP8 ? 2.0 * 32 * 32 * 64 * 32 : 2.0 * 32 * 32 * 16 * 64) * iters * grid * 4.0;
  const double tf = flop / (best * 1e-3) / 1e12;
  printf("  %-58s %8.2f ms  %7.0f TFLOP/s", name, best, tf);
  if (base > 0) printf("   %5.1f %% of the MFMA-only rate", 100.0 * tf / base);
  printf("\n");
  return tf;
}

int main() {
  unsigned* seed;
  float* out;
  (void)hipMalloc(&seed, (1 << 20) * 4);
  (void)hipMalloc(&out, 256 * 256 * 4);
  unsigned* h = (unsigned*)malloc((1 << 20) * 4);
  srand(1);
  for (int i = 0; i < (1 << 20); ++i) {  // two bf16 values of random sign, exponent 120..127, random mantissa
    const unsigned lo = ((rand() & 1) << 15) | ((120 + rand() % 8) << 7) | (rand() & 127);
    const unsigned hi = ((rand() & 1) << 15) | ((120 + rand() % 8) << 7) | (rand() & 127);
    h[i] = lo | (hi << 16);  // (read as four e4m3 bytes by the fp8 runs: random codes as well)
  }
  (void)hipMemcpy(seed, h, (1 << 20) * 4, hipMemcpyHostToDevice);
  printf("MFMA-only loops, one wave per SIMD, 256 workgroups of 4 waves, ~30 ms launches (best of 3 after a warm-up)\n");
  run<NONE, false>("bf16 32x32x16, all-zero operands", seed, out, 1, 0);
  const double b = run<NONE, false>("bf16 32x32x16, random operands", seed, out, 0, 0);
  run<NONE, true>("fp8 32x32x64 (f8f6f4), all-zero operands", seed, out, 1, 0);
  const double f = run<NONE, true>("fp8 32x32x64 (f8f6f4), random operands", seed, out, 0, 0);
  printf("bf16 MFMA per slot plus one companion instruction kind per slot (random operands)\n");
  run<EXP2, false>("+ v_exp_f32", seed, out, 0, b);
  run<CVT_PK_BF16, false>("+ v_cvt_pk_bf16_f32", seed, out, 0, b);
  run<ADD, false>("+ v_add_f32", seed, out, 0, b);
  run<FMA, false>("+ v_fma_f32", seed, out, 0, b);
  run<XOR, false>("+ v_xor_b32", seed, out, 0, b);
  run<MAX3, false>("+ v_max3_f32", seed, out, 0, b);
  run<DOT2_BF16, false>("+ v_dot2c_f32_bf16", seed, out, 0, b);
  run<LDS_B128, false>("+ ds_read_b128 per two slots (1 KB operand)", seed, out, 0, b);
  run<LDS_TR_B64, false>("+ 2 ds_read_b64_tr_b16 per two slots (1 KB operand)", seed, out, 0, b);
  run<SOFTMAX_MIX, false>("+ exp2, add and half a convert (the softmax of the 64-row kernel)", seed, out, 0, b);
  printf("fp8 MFMA (two slots long) with the same companions per slot\n");
  run<EXP2, true>("+ 2 v_exp_f32 per MFMA", seed, out, 0, f);
  run<SOFTMAX_MIX, true>("+ 2 exp2, 2 add, 1 convert per MFMA", seed, out, 0, f);
  return 0;
}
