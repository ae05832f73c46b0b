// Measured score bound for callers that state none (MAGI_ATTN_AUTO_BOUND): one streaming pass over q and one over k
// leave the largest squared row length of each in two words of a caller-provided workspace.  By Cauchy-Schwarz
// |q . k| <= |q| |k| for every pair, so the attention kernels launched behind these passes can decide ON THE DEVICE,
// with no host synchronisation, whether the bounded-score kernel applies (it does for QK-normed attention at ordinary
// gains) or the online-softmax kernel has to run.  HBM bound, 256 bytes per (token, head) row.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace magi {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__global__ void gate_init_kernel(unsigned* ws) {
  if (threadIdx.x < 4) ws[threadIdx.x] = 0u;
}

// 16 lanes per row of 128 bf16 values (16 bytes each).  A workgroup of 256 threads owns ROWS_PER_WG consecutive rows
// and walks them 64 at a time, four rows in flight per 16-lane group (one contiguous piece per workgroup streams a
// third faster on this part than a grid-stride walk of the same tensor).  The maximum is taken on bit patterns: sums
// of squares are non-negative, so their patterns order like their values, infinity lies above every finite sum and a
// NaN above infinity (whatever its sign bit): a tensor with a NaN row reports a NaN length, which no bound test passes.
constexpr int ROWS_PER_WG = 1024;
__global__ __launch_bounds__(256) void row_norm_max_kernel(const char* __restrict__ x, long stride_t, long stride_h,
                                                           int T, int H, unsigned* __restrict__ out_bits) {
  __shared__ unsigned s_best[4];
  const int sub = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const long rows = (long)T * H;
  const long first = (long)blockIdx.x * ROWS_PER_WG;
  const long last = min(first + ROWS_PER_WG, rows);
  unsigned best = 0u;
  // (a row index past the end is clamped to the last row: a maximum does not mind seeing a row twice)
  for (long r = first + grp; r < last; r += 64) {
    bf16x8 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const long ru = min(r + 16 * u, rows - 1);
      const long t = ru / H;
      const int h = (int)(ru - t * H);
      v[u] = *(const bf16x8*)(x + t * stride_t + (long)h * stride_h + sub * 16);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s += (float)v[u][e] * (float)v[u][e];
      s += __shfl_xor(s, 1);
      s += __shfl_xor(s, 2);
      s += __shfl_xor(s, 4);
      s += __shfl_xor(s, 8);
      best = max(best, __float_as_uint(s));
    }
  }
  best = max(best, (unsigned)__shfl_xor((int)best, 16));
  best = max(best, (unsigned)__shfl_xor((int)best, 32));
  if ((threadIdx.x & 63) == 0) s_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    best = max(max(s_best[0], s_best[1]), max(s_best[2], s_best[3]));
    if (best != 0u) atomicMax(out_bits, best);
  }
}

}  // namespace

hipError_t launch_gate_init(unsigned* ws, hipStream_t stream) {
  hipLaunchKernelGGL(gate_init_kernel, dim3(1), dim3(64), 0, stream, ws);
  return hipGetLastError();
}

hipError_t launch_row_norm_max(const char* x, long stride_t, long stride_h, int T, int H, unsigned* out_bits,
                               hipStream_t stream) {
  const long rows = (long)T * H;
  if (rows <= 0) return hipSuccess;
  const long blocks = (rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
  if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(row_norm_max_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, stride_t, stride_h, T, H, out_bits);
  return hipGetLastError();
}

}  // namespace magi
