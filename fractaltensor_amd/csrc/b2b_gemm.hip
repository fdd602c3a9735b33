// Back-to-back fp16 GEMM D = (A @ B) @ C for gfx950, fp32 accumulation on
// v_mfma_f32_32x32x16_f16, the intermediate A@B never leaving registers.
//
// Each wave owns 32 rows of A.  Both products are computed transposed so that
// a lane always owns one A row:
//   GEMM1  P^T[n, i] = sum_k Bs[n][k] * A[i][k]     MFMA A-operand = Bs rows (LDS),
//                                                   B-operand = A row fragments (registers)
//   GEMM2  D^T[p, i] = sum_n Cs[p][n] * P[i][n]     A-operand = Cs rows (LDS),
//                                                   B-operand = P^T accumulators, rounded to fp16
// The 32x32 accumulator of lane (i = lane%32, half = lane/32) holds P^T rows
// n = 8g + 4*half + r (g = reg/4, r = reg%4).  An MFMA B-operand wants 8
// consecutive k per lane, but the order of the contraction index is free as
// long as both operands agree, so GEMM2 step s of an n-tile simply contracts
// over n = {16s + 4*half + r} U {16s + 8 + 4*half + r}: the eight values the
// lane already holds, and two 8-byte LDS reads of Cs for the other operand.
// No shuffle, no LDS round trip for P.
//
// A workgroup (8 waves) stages one problem's B and C in LDS once and then
// walks row tiles of that problem; the grid is (workgroups per problem, P
// tiles of 128, G).  D tiles go through an LDS transpose so global stores are
// full 16-byte-per-lane row segments.
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

constexpr int B2B_WAVES = 8;
constexpr int B2B_THREADS = B2B_WAVES * 64;
constexpr int B2B_PTILE = 128;  // p columns per workgroup
constexpr int B2B_DLD = B2B_PTILE + 4;  // padded D staging row (halfs)

__device__ __forceinline__ uint4 ldg16(const void* p) { return *reinterpret_cast<const uint4*>(p); }

template <int KS>  // K = 16 * KS
__global__ __launch_bounds__(B2B_THREADS) void b2b_gemm_kernel(const _Float16* __restrict__ A,
                                                               const _Float16* __restrict__ Bm,
                                                               const _Float16* __restrict__ Cm,
                                                               _Float16* __restrict__ D, int M, int N, int P) {
  constexpr int K = 16 * KS;
  constexpr int BLD = K + 8;  // padded Bs row (halfs)
  const int CLD = N + 4;      // padded Cs row (halfs)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  _Float16* Bs = reinterpret_cast<_Float16*>(smem);  // [N][BLD]
  _Float16* Cs = Bs + N * BLD;                       // [PTILE][CLD]
  _Float16* Ds = Cs + B2B_PTILE * CLD;               // [waves][32][DLD]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  const int g = blockIdx.z;
  const int p0 = blockIdx.y * B2B_PTILE;
  const int np_tiles = min(B2B_PTILE, P - p0) / 32;  // p tiles handled here (1..4)

  const _Float16* Ag = A + (size_t)g * M * K;
  const _Float16* Bg = Bm + (size_t)g * N * K;
  const _Float16* Cg = Cm + (size_t)g * P * N;
  _Float16* Dg = D + (size_t)g * M * P;
  _Float16* Dw = Ds + wave * 32 * B2B_DLD;

  // ---- stage this problem's Bs[n][k] and Cs[p][n] once per workgroup
  for (int idx = tid; idx < N * (K / 8); idx += B2B_THREADS) {
    const int n = idx / (K / 8);
    const int k8 = idx - n * (K / 8);
    *reinterpret_cast<uint4*>(Bs + n * BLD + 8 * k8) = ldg16(Bg + (size_t)n * K + 8 * k8);
  }
  for (int idx = tid; idx < np_tiles * 32 * (N / 8); idx += B2B_THREADS) {
    const int p = idx / (N / 8);
    const int n8 = idx - p * (N / 8);
    const uint4 v = ldg16(Cg + (size_t)(p0 + p) * N + 8 * n8);
    // CLD is not a multiple of 8 halfs: write as two 8-byte pieces
    *reinterpret_cast<uint2*>(Cs + p * CLD + 8 * n8) = make_uint2(v.x, v.y);
    *reinterpret_cast<uint2*>(Cs + p * CLD + 8 * n8 + 4) = make_uint2(v.z, v.w);
  }
  __syncthreads();

  const int row_tiles = (M + 31) / 32;
  const int wave_stride = gridDim.x * B2B_WAVES;
  for (int tile = blockIdx.x * B2B_WAVES + wave; tile < row_tiles; tile += wave_stride) {
    const int row_c = min(tile * 32 + j, M - 1);
    // ---- A row fragments: step s contracts k in [8s, 8s+8) (lanes 0-31) and
    //      [K/2 + 8s, K/2 + 8s + 8) (lanes 32-63): 16*KS contiguous bytes per lane
    v8h afrag[KS];
    const _Float16* arow = Ag + (size_t)row_c * K + hh * (K / 2);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const uint4 v = ldg16(arow + 8 * s);
      afrag[s] = *reinterpret_cast<const v8h*>(&v);
    }

    v16f dacc[4];
#pragma unroll
    for (int pt = 0; pt < 4; ++pt)
#pragma unroll
      for (int r = 0; r < 16; ++r) dacc[pt][r] = 0.0f;

    for (int nt = 0; nt < N / 32; ++nt) {
      // GEMM1: P^T tile [32 n, 32 rows]
      v16f pacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) pacc[r] = 0.0f;
      const _Float16* brow = Bs + (nt * 32 + j) * BLD + hh * (K / 2);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const v8h bfrag = *reinterpret_cast<const v8h*>(brow + 8 * s);
        pacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag, afrag[s], pacc, 0, 0, 0);
      }
      // round to fp16: the two B-operands of GEMM2 for this n tile
      v8h pf[2];
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) pf[s][e] = (_Float16)pacc[8 * s + e];
      // GEMM2: D^T[p tile] += Cs[p][n] * P
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) {
        if (pt < np_tiles) {
          const _Float16* crow = Cs + (pt * 32 + j) * CLD + nt * 32 + 4 * hh;
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const v4h c0 = *reinterpret_cast<const v4h*>(crow + 16 * s);
            const v4h c1 = *reinterpret_cast<const v4h*>(crow + 16 * s + 8);
            const v8h cfrag = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
            dacc[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cfrag, pf[s], dacc[pt], 0, 0, 0);
          }
        }
      }
    }

    // ---- epilogue: D^T accumulators -> LDS [row][p] -> 16-byte row segments.
    // A wave reads back only what it wrote itself and LDS operations of one
    // wave complete in order, so no workgroup barrier is needed.
#pragma unroll
    for (int pt = 0; pt < 4; ++pt) {
      if (pt < np_tiles) {
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const v4h o = {(_Float16)dacc[pt][4 * gq + 0], (_Float16)dacc[pt][4 * gq + 1],
                         (_Float16)dacc[pt][4 * gq + 2], (_Float16)dacc[pt][4 * gq + 3]};
          *reinterpret_cast<v4h*>(Dw + j * B2B_DLD + pt * 32 + 8 * gq + 4 * hh) = o;
        }
      }
    }
    const int segs = np_tiles * 4;  // 16-byte segments per row
    for (int idx = lane; idx < 32 * segs; idx += 64) {
      const int r = idx / segs;
      const int sg = idx - r * segs;
      const int grow = tile * 32 + r;
      if (grow < M) {
        const uint2 lo = *reinterpret_cast<const uint2*>(Dw + r * B2B_DLD + 8 * sg);
        const uint2 hi = *reinterpret_cast<const uint2*>(Dw + r * B2B_DLD + 8 * sg + 4);
        *reinterpret_cast<uint4*>(Dg + (size_t)grow * P + p0 + 8 * sg) = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    }
  }
}

static size_t b2b_lds_bytes(int N, int K) {
  return (size_t)(N * (K + 8) + B2B_PTILE * (N + 4) + B2B_WAVES * 32 * B2B_DLD) * 2;
}

template <int KS>
static int launch_b2b(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int P, int cus,
                      int lds_max, hipStream_t s) {
  constexpr int K = 16 * KS;
  const size_t lds = b2b_lds_bytes(N, K);
  if ((int)lds > lds_max)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE,
                "ftk_b2b_gemm_f16: B and C tiles for N=%d K=%d need %zu bytes of LDS, the device has %d", N, K, lds,
                lds_max);
  const int ptiles = (P + B2B_PTILE - 1) / B2B_PTILE;
  const int row_tiles = (M + 31) / 32;
  // enough workgroups per problem to fill the chip once; each walks its share of the row tiles
  int per_problem = (cus + G * ptiles - 1) / (G * ptiles);
  per_problem = std::max(1, std::min(per_problem, (row_tiles + B2B_WAVES - 1) / B2B_WAVES));
  const void* fn = (const void*)b2b_gemm_kernel<KS>;
  FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(b2b_gemm_kernel<KS>, dim3(per_problem, ptiles, G), dim3(B2B_THREADS), lds, s,
                     (const _Float16*)A, (const _Float16*)B, (const _Float16*)C, (_Float16*)D, M, N, P);
  return check_launch("b2b_gemm_kernel");
}

}  // namespace ftk

extern "C" int ftk_b2b_gemm_f16(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int K,
                                int P, ftk_stream_t stream) {
  using namespace ftk;
  if (!A || !B || !C || !D) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_b2b_gemm_f16: A, B, C, D must be non-NULL");
  if (G <= 0 || M <= 0 || N <= 0 || K <= 0 || P <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_b2b_gemm_f16: G, M, N, K, P must be positive");
  if (N % 32 || P % 32) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: N=%d and P=%d must be multiples of 32", N, P);
  if (G > 65535) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: G=%d above 65535", G);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  switch (K) {
    case 32: return launch_b2b<2>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    case 64: return launch_b2b<4>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    case 96: return launch_b2b<6>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    case 128: return launch_b2b<8>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    default:
      return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: K=%d must be one of 32, 64, 96, 128", K);
  }
}
