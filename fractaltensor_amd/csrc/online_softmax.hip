// Row softmax through an online (max, denominator) scan for gfx950, fp32.
//
// One workgroup per row.  Every thread folds its strided elements into a
// running pair with m' = max(m, x), d' = d*exp(m-m') + exp(x-m'); pairs are
// merged across the wave with DPP-free shuffles and across waves through LDS
// using d = d1*exp(m1-m) + d2*exp(m2-m); a second pass writes exp(x-m)/d.
#include "ftk_common.h"

namespace ftk {

__device__ __forceinline__ void md_merge(float& m, float& d, float m2, float d2) {
  const float mn = fmaxf(m, m2);
  // a pair that has seen nothing is (-inf, 0): keep exp(-inf - -inf) out of it
  const float a = (m == -INFINITY) ? 0.0f : d * __expf(m - mn);
  const float b = (m2 == -INFINITY) ? 0.0f : d2 * __expf(m2 - mn);
  m = mn;
  d = a + b;
}

__global__ __launch_bounds__(256) void online_softmax_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                             int cols) {
  __shared__ float sm[4], sd[4];
  const float* xr = x + (size_t)blockIdx.x * cols;
  float* yr = y + (size_t)blockIdx.x * cols;
  float m = -INFINITY, d = 0.0f;
  for (int c = threadIdx.x; c < cols; c += 256) md_merge(m, d, xr[c], 1.0f);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off);
    const float d2 = __shfl_xor(d, off);
    md_merge(m, d, m2, d2);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    sm[wave] = m;
    sd[wave] = d;
  }
  __syncthreads();
  m = sm[0];
  d = sd[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) md_merge(m, d, sm[w], sd[w]);
  const float inv = 1.0f / d;
  for (int c = threadIdx.x; c < cols; c += 256) yr[c] = __expf(xr[c] - m) * inv;
}

}  // namespace ftk

extern "C" int ftk_online_softmax_f32(const float* x, float* y, int rows, int cols, ftk_stream_t stream) {
  using namespace ftk;
  if (!x || !y) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_online_softmax_f32: x and y must be non-NULL");
  if (rows <= 0 || cols <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_online_softmax_f32: rows and cols must be positive");
  hipLaunchKernelGGL(online_softmax_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, x, y, cols);
  return check_launch("online_softmax_kernel");
}
