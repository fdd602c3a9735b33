// Embedding lookup for gfx950: out[i, :] = table[ids[i], :].
//
// The step before the LSTM in the reference's RNN programs: every word of a
// batch indexes the rows of the embedding matrix.  A row is moved by as many
// lanes as it has 16-byte pieces (whole rows per wave when E is small), so
// every load and store is a full-width coalesced access; the table is small
// and re-read from L2, the output is written once: the kernel is bound by the
// HBM write of n*E*4 bytes.  Ids outside [0, V) are counted in *bad and their
// rows are zero-filled, so nothing is ever read out of bounds.
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

template <typename Id>
__global__ __launch_bounds__(256) void embedding_gather_kernel(const float* __restrict__ table, const Id* __restrict__ ids,
                                                               float* __restrict__ out, long long n, int V, int E4,
                                                               int* __restrict__ bad) {
  // one thread per (row, 16-byte piece); consecutive threads walk along a row, then to the next row
  const long long total = n * E4;
  for (long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x; p < total; p += (long long)gridDim.x * blockDim.x) {
    const long long row = p / E4;
    const int piece = (int)(p - row * E4);
    const long long id = (long long)ids[row];
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (id >= 0 && id < V) {
      v = *reinterpret_cast<const float4*>(table + (size_t)id * E4 * 4 + 4 * piece);
    } else if (piece == 0 && bad) {
      atomicAdd(bad, 1);
    }
    *reinterpret_cast<float4*>(out + (size_t)row * E4 * 4 + 4 * piece) = v;
  }
}

// Rows of 2^k pieces, k <= 8 (E = 4 .. 1024 in powers of two): a workgroup moves 256 >> k rows per round
// with shifts instead of divisions, ROUNDS rounds per workgroup, and the output bypasses the caches (it is
// written once and not read here).
template <typename Id, int ROUNDS>
__global__ __launch_bounds__(256) void embedding_gather_pow2_kernel(const float* __restrict__ table, const Id* __restrict__ ids,
                                                                    float* __restrict__ out, long long n, int V, int log2_e4,
                                                                    int* __restrict__ bad) {
  const int rows_per_round = 256 >> log2_e4;
  const int piece = threadIdx.x & ((1 << log2_e4) - 1);
  const long long row0 = ((long long)blockIdx.x * ROUNDS) * rows_per_round + (threadIdx.x >> log2_e4);
  long long id[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const long long row = row0 + (long long)r * rows_per_round;
    id[r] = row < n ? (long long)ids[row] : -1;
  }
  float4 v[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    v[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (id[r] >= 0 && id[r] < V) v[r] = *reinterpret_cast<const float4*>(table + (((size_t)id[r] << log2_e4) + piece) * 4);
  }
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const long long row = row0 + (long long)r * rows_per_round;
    if (row < n) {
      if ((id[r] < 0 || id[r] >= V) && piece == 0 && bad) atomicAdd(bad, 1);
      float* dst = out + (((size_t)row << log2_e4) + piece) * 4;
      __builtin_nontemporal_store(v[r].x, dst);
      __builtin_nontemporal_store(v[r].y, dst + 1);
      __builtin_nontemporal_store(v[r].z, dst + 2);
      __builtin_nontemporal_store(v[r].w, dst + 3);
    }
  }
}

}  // namespace ftk

extern "C" int ftk_embedding_gather_f32(const float* table, const void* ids, int ids_are_64bit, float* out,
                                        long long n, int V, int E, int* bad_ids, ftk_stream_t stream) {
  using namespace ftk;
  if (!table || !ids || !out) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_embedding_gather_f32: table, ids, out must be non-NULL");
  if (n <= 0 || V <= 0 || E <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_embedding_gather_f32: n, V, E must be positive");
  if (E % 4) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_embedding_gather_f32: E=%d must be a multiple of 4", E);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  const int E4 = E / 4;
  hipStream_t s = (hipStream_t)stream;
  if ((E4 & (E4 - 1)) == 0 && E4 <= 256) {
    int k = 0;
    while ((1 << k) < E4) ++k;
    constexpr int ROUNDS = 4;
    const long long rows_per_block = (long long)ROUNDS * (256 >> k);
    const long long blocks = (n + rows_per_block - 1) / rows_per_block;
    if (blocks <= 0x7fffffffLL) {
      if (ids_are_64bit)
        hipLaunchKernelGGL((embedding_gather_pow2_kernel<long long, ROUNDS>), dim3((unsigned)blocks), dim3(256), 0, s, table,
                           (const long long*)ids, out, n, V, k, bad_ids);
      else
        hipLaunchKernelGGL((embedding_gather_pow2_kernel<int, ROUNDS>), dim3((unsigned)blocks), dim3(256), 0, s, table,
                           (const int*)ids, out, n, V, k, bad_ids);
      return check_launch("embedding_gather_pow2_kernel");
    }
  }
  const long long pieces = n * E4;
  const long long want = (pieces + 255) / 256;
  const int grid = (int)std::min<long long>(want, (long long)dp->cus * 32);
  if (ids_are_64bit)
    hipLaunchKernelGGL(embedding_gather_kernel<long long>, dim3(grid), dim3(256), 0, s, table, (const long long*)ids, out, n, V, E4, bad_ids);
  else
    hipLaunchKernelGGL(embedding_gather_kernel<int>, dim3(grid), dim3(256), 0, s, table, (const int*)ids, out, n, V, E4, bad_ids);
  return check_launch("embedding_gather_kernel");
}
