// Row softmax for gfx950, fp32, [rows, cols] row-major, through (max, denominator) pairs that are merged
// with d = d1*exp(m1-m) + d2*exp(m2-m), m = max(m1, m2).
//
// HBM-bound work: every element is read once and written once, so the kernels are built around wide, coalesced
// accesses and one exponential per element.
//   Rows of up to 8192 columns are held in registers by one wave (or by 16 or 32 lanes of it for rows of up to
//     64 or 128 columns, so that short rows do not leave lanes idle): each lane folds its elements into a pair
//     (local maximum first, then the sum of exp(x - max): one exponential per element), the pairs are merged
//     across the lanes with shuffles, and the lane scales the exponentials it already holds.  Lanes take 16-byte
//     pieces when the row length and the pointers allow it, single elements otherwise.
//   Longer rows go one per workgroup: every thread scans its strided pieces online -- the running pair is
//     rescaled only when a piece raises the maximum -- pairs are merged across the wave and, through LDS, across
//     the waves; a second pass over the row (which the first left in L2) writes exp(x - m) / d.
#include "ftk_common.h"

namespace ftk {

__device__ __forceinline__ void md_merge(float& m, float& d, float m2, float d2) {
  const float mn = fmaxf(m, m2);
  // a pair that has seen nothing is (-inf, 0): keep exp(-inf - -inf) out of it
  const float a = (m == -INFINITY) ? 0.0f : d * fast_exp(m - mn);
  const float b = (m2 == -INFINITY) ? 0.0f : d2 * fast_exp(m2 - mn);
  m = mn;
  d = a + b;
}

// One row per LPR lanes, K pieces per lane; a piece is a float4 (VEC) or a float.  Piece p of lane l is piece
// l + LPR*p of the row.
template <int LPR, int K, bool VEC>
__global__ __launch_bounds__(256) void softmax_rows_in_registers_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                        long long rows, int cols) {
  constexpr int W = VEC ? 4 : 1;
  constexpr int RPW = 64 / LPR;  // rows per wave
  const int lane = threadIdx.x & 63;
  const int sub = lane % LPR;
  const long long row = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / LPR;
  const bool live = row < rows;
  const float* xr = x + (size_t)(live ? row : 0) * cols;
  float v[K][W];
  float m = -INFINITY;
#pragma unroll
  for (int p = 0; p < K; ++p) {
    const int c = (sub + LPR * p) * W;
    if (live && c < cols) {
      if constexpr (VEC) {
        const float4 t = *reinterpret_cast<const float4*>(xr + c);
        v[p][0] = t.x; v[p][1] = t.y; v[p][2] = t.z; v[p][3] = t.w;
      } else {
        v[p][0] = xr[c];
      }
    } else {
#pragma unroll
      for (int e = 0; e < W; ++e) v[p][e] = -INFINITY;
    }
#pragma unroll
    for (int e = 0; e < W; ++e) m = fmaxf(m, v[p][e]);
  }
  // the lane's pair: one exponential per element, kept for the output
  float d = 0.0f;
#pragma unroll
  for (int p = 0; p < K; ++p)
#pragma unroll
    for (int e = 0; e < W; ++e) {
      v[p][e] = (v[p][e] == -INFINITY) ? 0.0f : fast_exp(v[p][e] - m);
      d += v[p][e];
    }
  // merge the pairs of the row's lanes; every lane ends with the row's pair
  float mr = m, dr = d;
#pragma unroll
  for (int off = LPR / 2; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(mr, off);
    const float d2 = __shfl_xor(dr, off);
    md_merge(mr, dr, m2, d2);
  }
  // exp(x - mr) / dr = exp(x - m) * exp(m - mr) / dr
  const float scale = (m == -INFINITY) ? 0.0f : fast_exp(m - mr) * __builtin_amdgcn_rcpf(dr);
  if (!live) return;
  float* yr = y + (size_t)row * cols;
#pragma unroll
  for (int p = 0; p < K; ++p) {
    const int c = (sub + LPR * p) * W;
    if (c < cols) {
      if constexpr (VEC) {
        // streaming stores: y is not read again, and lines left dirty in L2 hold up the end of the kernel
        __builtin_nontemporal_store(v4f{v[p][0] * scale, v[p][1] * scale, v[p][2] * scale, v[p][3] * scale}, reinterpret_cast<v4f*>(yr + c));
      } else {
        __builtin_nontemporal_store(v[p][0] * scale, yr + c);
      }
    }
  }
}

// One row per workgroup, any length.
template <bool VEC>
__global__ __launch_bounds__(1024) void softmax_long_rows_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                 int cols) {
  constexpr int W = VEC ? 4 : 1;
  __shared__ float sm[16], sd[16];
  const float* xr = x + (size_t)blockIdx.x * cols;
  float* yr = y + (size_t)blockIdx.x * cols;
  const int pieces = cols / W;
  float m = -INFINITY, d = 0.0f;
  for (int p = threadIdx.x; p < pieces; p += 1024) {
    float t[W];
    if constexpr (VEC) {
      const float4 q = *reinterpret_cast<const float4*>(xr + 4 * p);
      t[0] = q.x; t[1] = q.y; t[2] = q.z; t[3] = q.w;
    } else {
      t[0] = xr[p];
    }
    float pm = t[0];
#pragma unroll
    for (int e = 1; e < W; ++e) pm = fmaxf(pm, t[e]);
    if (pm > m) {  // a new maximum: bring the running sum to it
      d *= fast_exp(m - pm);  // exp(-inf) = 0 for the first piece
      m = pm;
    }
#pragma unroll
    for (int e = 0; e < W; ++e) d += fast_exp(t[e] - m);
  }
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
  for (int w = 1; w < 16; ++w) md_merge(m, d, sm[w], sd[w]);
  const float inv = __builtin_amdgcn_rcpf(d);
  for (int p = threadIdx.x; p < pieces; p += 1024) {
    if constexpr (VEC) {
      const float4 q = *reinterpret_cast<const float4*>(xr + 4 * p);
      __builtin_nontemporal_store(v4f{fast_exp(q.x - m) * inv, fast_exp(q.y - m) * inv, fast_exp(q.z - m) * inv, fast_exp(q.w - m) * inv},
                                  reinterpret_cast<v4f*>(yr + 4 * p));
    } else {
      __builtin_nontemporal_store(fast_exp(xr[p] - m) * inv, yr + p);
    }
  }
}

template <int LPR, int K, bool VEC>
static void launch_in_registers(const float* x, float* y, long long rows, int cols, hipStream_t s) {
  const long long rows_per_block = 4 * (64 / LPR);
  const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL((softmax_rows_in_registers_kernel<LPR, K, VEC>), dim3(blocks), dim3(256), 0, s, x, y, rows, cols);
}

template <bool VEC>
static bool launch_by_length(const float* x, float* y, long long rows, int cols, hipStream_t s) {
  const int pieces = (cols + (VEC ? 3 : 0)) / (VEC ? 4 : 1);  // per row
  if (pieces <= 16) launch_in_registers<16, 1, VEC>(x, y, rows, cols, s);
  else if (pieces <= 32) launch_in_registers<32, 1, VEC>(x, y, rows, cols, s);
  else if (pieces <= 64) launch_in_registers<64, 1, VEC>(x, y, rows, cols, s);
  else if (pieces <= 128) launch_in_registers<64, 2, VEC>(x, y, rows, cols, s);
  else if (pieces <= 256) launch_in_registers<64, 4, VEC>(x, y, rows, cols, s);
  else if (pieces <= 512) launch_in_registers<64, 8, VEC>(x, y, rows, cols, s);
  else if (pieces <= 1024) launch_in_registers<64, 16, VEC>(x, y, rows, cols, s);
  else if (pieces <= 2048) launch_in_registers<64, 32, VEC>(x, y, rows, cols, s);
  else return false;
  return true;
}

}  // namespace ftk

extern "C" int ftk_online_softmax_f32(const float* x, float* y, int rows, int cols, ftk_stream_t stream) {
  using namespace ftk;
  if (!x || !y) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_online_softmax_f32: x and y must be non-NULL");
  if (rows <= 0 || cols <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_online_softmax_f32: rows and cols must be positive");
  hipStream_t s = (hipStream_t)stream;
  const bool vec = cols % 4 == 0 && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 16 == 0;
  const bool done = vec ? launch_by_length<true>(x, y, rows, cols, s) : launch_by_length<false>(x, y, rows, cols, s);
  if (!done) {
    if (vec) hipLaunchKernelGGL(softmax_long_rows_kernel<true>, dim3(rows), dim3(1024), 0, s, x, y, cols);
    else hipLaunchKernelGGL(softmax_long_rows_kernel<false>, dim3(rows), dim3(1024), 0, s, x, y, cols);
  }
  return check_launch("online_softmax_kernel");
}
