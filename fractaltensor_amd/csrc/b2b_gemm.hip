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
// A workgroup stages one problem's B and C in LDS once and then walks row tiles
// of that problem, each wave 64 rows at a time (two 32-row tiles sharing every
// B and C fragment read).  A rows are fetched with fully coalesced 16-byte
// loads (64 lanes = 4 whole rows), parked in a wave-private LDS region and read
// back as fragments; the fetch for the wave's next 64 rows is issued before the
// current rows go to the matrix cores, so reads, MFMAs and the D stores of
// successive row groups overlap.  D tiles leave through the same wave-private
// region so global stores are full 16-byte-per-lane row segments.  The grid is
// one-dimensional and remapped so that the workgroups of one problem share an
// XCD (and with it the L2 copy of B and C).
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "ftk_common.h"

namespace ftk {

constexpr int B2B_PTILE = 128;  // p columns per workgroup

typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

__device__ __forceinline__ v4u ldg16(const void* p) { return *reinterpret_cast<const v4u*>(p); }

struct B2BGrid {
  int per_problem;  // workgroups sharing one (problem, p tile)
  int ptiles;
  int total;        // per_problem * ptiles * G
  int wave_region;  // halfs of wave-private LDS (A rows in, D rows out)
};

template <int KS, int PT>  // K = 16 * KS, 32 * PT columns of D per workgroup
__global__ __launch_bounds__(256) void b2b_gemm_kernel(const _Float16* __restrict__ A,
                                                       const _Float16* __restrict__ Bm,
                                                       const _Float16* __restrict__ Cm, _Float16* __restrict__ D,
                                                       int M, int N, int P, int p_base, B2BGrid gr) {
  constexpr int K = 16 * KS;
  constexpr int BLD = K + 8;  // padded Bs / A-staging row (halfs)
  constexpr int AN = 2 * KS;  // 16-byte A loads per lane for 64 rows (64 rows * K/8 chunks over 64 lanes)
  const int CLD = N + 4;      // padded Cs row (halfs)
  const int threads = blockDim.x;
  const int waves = threads >> 6;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;

  // consecutive logical ids land on one XCD (hardware deals workgroups round-robin over 8 XCDs)
  int id = blockIdx.x;
  if ((gr.total & 7) == 0) id = (blockIdx.x & 7) * (gr.total >> 3) + (blockIdx.x >> 3);
  const int part = id % gr.per_problem;
  const int pt_idx = (id / gr.per_problem) % gr.ptiles;
  const int g = id / (gr.per_problem * gr.ptiles);

  constexpr int pw = 32 * PT;             // p columns handled here
  constexpr int DLD = pw + 4;             // padded D staging row (halfs)
  const int p0 = p_base + pt_idx * pw;

  _Float16* Bs = reinterpret_cast<_Float16*>(smem);  // [N][BLD]
  _Float16* Cs = Bs + N * BLD;                       // [pw][CLD]
  _Float16* Wa = Cs + pw * CLD + wave * gr.wave_region;  // wave-private: A rows in, [32][BLD]
  _Float16* Ws = Wa + 32 * BLD;                          // wave-private: D rows out, [32][DLD]

  const _Float16* Ag = A + (size_t)g * M * K;
  const _Float16* Bg = Bm + (size_t)g * N * K;
  const _Float16* Cg = Cm + (size_t)g * P * N + (size_t)p0 * N;
  _Float16* Dg = D + (size_t)g * M * P + p0;

  const int row_pairs = (M + 63) / 64;  // units of 64 rows
  const int wave_stride = gr.per_problem * waves;
  int pair = part * waves + wave;

  // ---- coalesced fetch of 64 A rows: load u covers 16-byte chunks u*64 + lane of the row group
  constexpr int CPR = K / 8;  // 16-byte chunks per row
  v4u areg[AN];
  auto fetch_a = [&](int pr_) __attribute__((always_inline)) {
    static_for<AN>([&](auto uc) __attribute__((always_inline)) {
      constexpr int u = decltype(uc)::value;
      const int chunk = u * 64 + lane;
      const int row = min(pr_ * 64 + chunk / CPR, M - 1);
      areg[u] = ldg16(Ag + (size_t)row * K + 8 * (chunk % CPR));
    });
  };
  // park them in the wave's LDS region, then pull the MFMA fragments: step s
  // contracts k in [8s, 8s+8) (lanes 0-31) and [K/2 + 8s, K/2 + 8s + 8) (lanes 32-63)
  v8h afrag[2][KS];
  auto park_a = [&]() __attribute__((always_inline)) {
    // 32 rows at a time through the same region; LDS operations of a wave complete in order
    static_for<2>([&](auto rtc) __attribute__((always_inline)) {
      constexpr int rt = decltype(rtc)::value;
      static_for<AN / 2>([&](auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const int chunk = u * 64 + lane;  // chunk within this 32-row half
        *reinterpret_cast<v4u*>(Wa + (chunk / CPR) * BLD + 8 * (chunk % CPR)) = areg[rt * (AN / 2) + u];
      });
#pragma unroll
      for (int s = 0; s < KS; ++s)
        afrag[rt][s] = *reinterpret_cast<const v8h*>(Wa + j * BLD + hh * (K / 2) + 8 * s);
    });
  };
  if (pair < row_pairs) fetch_a(pair);

  // ---- stage this problem's Bs[n][k] and Cs[p][n].  Eight loads of each per
  // thread are issued before the first is consumed (the accumulators are not
  // live yet, so the registers are free): for N = K = 128 and 128 columns that
  // is all of B and C in one round trip to memory instead of four.
  {
    constexpr int SB = 8;
    const int nb = N * (K / 8);
    const int n8s = N / 8;
    const int ncq = pw * n8s;
    for (int base = 0; base < max(nb, ncq); base += SB * threads) {
      v4u vb[SB], vc[SB];
#pragma unroll
      for (int u = 0; u < SB; ++u) {
        const int idx = base + u * threads + tid;
        if (idx < nb) vb[u] = ldg16(Bg + (size_t)idx * 8);
      }
#pragma unroll
      for (int u = 0; u < SB; ++u) {
        const int idx = base + u * threads + tid;
        if (idx < ncq) vc[u] = ldg16(Cg + (size_t)idx * 8);
      }
#pragma unroll
      for (int u = 0; u < SB; ++u) {
        const int idx = base + u * threads + tid;
        if (idx < nb) {
          const int n = idx / (K / 8);
          const int k8 = idx - n * (K / 8);
          *reinterpret_cast<v4u*>(Bs + n * BLD + 8 * k8) = vb[u];
        }
      }
#pragma unroll
      for (int u = 0; u < SB; ++u) {
        const int idx = base + u * threads + tid;
        if (idx < ncq) {
          const int p = idx / n8s;
          const int n8 = idx - p * n8s;
          // CLD is not a multiple of 8 halfs: two 8-byte pieces
          *reinterpret_cast<v2u*>(Cs + p * CLD + 8 * n8) = v2u{vc[u][0], vc[u][1]};
          *reinterpret_cast<v2u*>(Cs + p * CLD + 8 * n8 + 4) = v2u{vc[u][2], vc[u][3]};
        }
      }
    }
  }
  __syncthreads();

  // Software pipeline per wave: the fragments of row group n+1 are parked and
  // the fetch of group n+2 issued between the arithmetic of group n and its D
  // stores, so every load and store has a whole arithmetic phase to complete.
  if (pair < row_pairs) {
    park_a();
    if (pair + wave_stride < row_pairs) fetch_a(pair + wave_stride);
  }
  for (; pair < row_pairs; pair += wave_stride) {
    v16f dacc[2][PT];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int pt = 0; pt < PT; ++pt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dacc[rt][pt][r] = 0.0f;

    for (int nt = 0; nt < N / 32; ++nt) {
      // GEMM1: P^T tiles [32 n, 32 rows] for both row tiles
      v16f pacc[2];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int r = 0; r < 16; ++r) pacc[rt][r] = 0.0f;
      const _Float16* brow = Bs + (nt * 32 + j) * BLD + hh * (K / 2);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const v8h bfrag = *reinterpret_cast<const v8h*>(brow + 8 * s);
        pacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag, afrag[0][s], pacc[0], 0, 0, 0);
        pacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag, afrag[1][s], pacc[1], 0, 0, 0);
      }
      // round to fp16: the B-operands of GEMM2 for this n tile
      v8h pf[2][2];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) pf[rt][s][e] = (_Float16)pacc[rt][8 * s + e];
      // GEMM2: D^T[p tile] += Cs[p][n] * P
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        const _Float16* crow = Cs + (pt * 32 + j) * CLD + nt * 32 + 4 * hh;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const v4h c0 = *reinterpret_cast<const v4h*>(crow + 16 * s);
          const v4h c1 = *reinterpret_cast<const v4h*>(crow + 16 * s + 8);
          const v8h cfrag = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
          dacc[0][pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cfrag, pf[0][s], dacc[0][pt], 0, 0, 0);
          dacc[1][pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cfrag, pf[1][s], dacc[1][pt], 0, 0, 0);
        }
      }
    }

    if (pair + wave_stride < row_pairs) {
      park_a();
      if (pair + 2 * wave_stride < row_pairs) fetch_a(pair + 2 * wave_stride);
    }

    // ---- epilogue: D^T accumulators -> wave-private LDS [row][p] -> 16-byte
    // row segments.  A wave reads back only what it wrote itself and LDS
    // operations of one wave complete in order, so no barrier is needed.
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const v4h o = {(_Float16)dacc[rt][pt][4 * gq + 0], (_Float16)dacc[rt][pt][4 * gq + 1],
                         (_Float16)dacc[rt][pt][4 * gq + 2], (_Float16)dacc[rt][pt][4 * gq + 3]};
          *reinterpret_cast<v4h*>(Ws + j * DLD + pt * 32 + 8 * gq + 4 * hh) = o;
        }
      }
      constexpr int segs = PT * 4;  // 16-byte segments per row
#pragma unroll
      for (int idx = lane; idx < 32 * segs; idx += 64) {
        const int r = idx / segs;
        const int sg = idx - r * segs;
        const int grow = pair * 64 + 32 * rt + r;
        if (grow < M) {
          const v2u lo = *reinterpret_cast<const v2u*>(Ws + r * DLD + 8 * sg);
          const v2u hi = *reinterpret_cast<const v2u*>(Ws + r * DLD + 8 * sg + 4);
          __builtin_nontemporal_store(v4u{lo[0], lo[1], hi[0], hi[1]}, reinterpret_cast<v4u*>(Dg + (size_t)grow * P + 8 * sg));
        }
      }
    }
  }
}

// Eight-wave form of the same computation for the common shapes (N = 32*NT up
// to 128, all of B and C resident).  Two waves share a SIMD and every wave
// walks 32-row units, so the work is ordered to fit 256 registers and to start
// on the first rows to arrive: GEMM1 of a unit runs to completion and leaves P
// as fp16 B-operands in registers, then GEMM2 runs over the D columns in groups
// of 64 with its own accumulators and stores each group as it finishes.  The
// kernel is bound by how fast a CU's memory pipeline takes the workgroup's
// loads (B, C and 512 rows of A are all requested up front, B and C first
// because everything waits for them); units are small so that compute on the
// rows that have landed overlaps the rest of the stream and little work is
// left when the last rows arrive, and two waves per SIMD cover each other's LDS
// round trips, conversions and D stores.  The wave-private LDS region is used
// twice per unit: A rows on the way in, D rows on the way out.
//
// ROWMAJOR: B is given as [K, N] and C as [N, P], row-major, the layout of an operator program's (a @ b) @ c.
// Both are staged as they are (rows padded by 64 bytes) and the weight-side MFMA operands, which want 8
// consecutive k (or n) per lane, are read with ds_read_b64_tr_b16: 16 lanes hand in a 4-row x 16-column block
// and lane i receives column i of the four rows, so nothing is transposed on the way in.
template <int KS, int PT, int NT, bool ROWMAJOR>
__global__ __launch_bounds__(512) void b2b_gemm8_kernel(const _Float16* __restrict__ A,
                                                        const _Float16* __restrict__ Bm,
                                                        const _Float16* __restrict__ Cm, _Float16* __restrict__ D,
                                                        int M, int P, int p_base, B2BGrid gr) {
  constexpr int K = 16 * KS;
  constexpr int N = 32 * NT;
  constexpr int BLD = K + 8;   // padded Bs / A-staging row (halfs)
  constexpr int CLD = N + 4;   // padded Cs row (halfs)
  constexpr int BRS = N + 32;       // ROWMAJOR: Bs[k][n] row (halfs), 64 bytes of padding
  constexpr int CRS = 32 * PT + 32;  // ROWMAJOR: Cs[n][p] row
  using lds_v4s = __attribute__((address_space(3))) v4s;
  constexpr int AN = KS;       // 16-byte A loads per lane for 32 rows
#ifndef FTK_B2B_LA
#define FTK_B2B_LA 4
#endif
  constexpr int LA = FTK_B2B_LA;  // LDS fragments requested ahead of the MFMA that uses them
  constexpr int pw = 32 * PT;  // p columns handled here
  constexpr int PG = (PT + 1) / 2;  // column groups of up to 64
  constexpr int DLD = 64 + 4;  // padded D staging row (halfs)
  constexpr int threads = 512;
  constexpr int waves = 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;

  int id = blockIdx.x;
  if ((gr.total & 7) == 0) id = (blockIdx.x & 7) * (gr.total >> 3) + (blockIdx.x >> 3);
  const int part = id % gr.per_problem;
  const int pt_idx = (id / gr.per_problem) % gr.ptiles;
  const int g = id / (gr.per_problem * gr.ptiles);
  const int p0 = p_base + pt_idx * pw;

  _Float16* Bs = reinterpret_cast<_Float16*>(smem);        // [N][BLD], ROWMAJOR: [K][BRS]
  _Float16* Cs = Bs + (ROWMAJOR ? K * BRS : N * BLD);      // [pw][CLD], ROWMAJOR: [N][CRS]
  _Float16* Wr = Cs + (ROWMAJOR ? N * CRS : pw * CLD) + wave * gr.wave_region;  // wave-private: [32][BLD] A rows, then [32][DLD] D rows

  const _Float16* Ag = A + (size_t)g * M * K;
  const _Float16* Bg = Bm + (size_t)g * N * K;
  const _Float16* Cg = Cm + (size_t)g * P * N + (ROWMAJOR ? (size_t)p0 : (size_t)p0 * N);
  _Float16* Dg = D + (size_t)g * M * P + p0;

  // consecutive units of a workgroup go to consecutive waves: wave w takes units w, w + 8, ... of the
  // workgroup's contiguous row range, so the rows that are requested first belong to different waves
  const int units = (M + 31) / 32;
  const int per_wg = (units + gr.per_problem - 1) / gr.per_problem;
  const int unit_end = min(units, (part + 1) * per_wg);
  int unit = part * per_wg + wave;

  constexpr int CPR = K / 8;  // 16-byte chunks per row
  v4u areg0[AN], areg1[AN];
  auto fetch_a = [&](int un, v4u (&ar)[AN]) __attribute__((always_inline)) {
    static_for<AN>([&](auto uc) __attribute__((always_inline)) {
      constexpr int u = decltype(uc)::value;
      const int chunk = u * 64 + lane;
      const int row = min(un * 32 + chunk / CPR, M - 1);
      ar[u] = ldg16(Ag + (size_t)row * K + 8 * (chunk % CPR));
    });
  };

  // ---- stage Bs[n][k] and Cs[p][n], all loads of a thread in flight together
  {
    constexpr int nb = N * (K / 8), ncq = pw * (N / 8);
    constexpr int UB = (nb + threads - 1) / threads, UC = (ncq + threads - 1) / threads;
    v4u vb[UB], vc[UC];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int idx = u * threads + tid;
      if (idx < nb) vb[u] = ldg16(Bg + (size_t)idx * 8);
    }
#pragma unroll
    for (int u = 0; u < UC; ++u) {
      const int idx = u * threads + tid;
      if (idx < ncq) {
        if constexpr (ROWMAJOR) vc[u] = ldg16(Cg + (size_t)(idx / (pw / 8)) * P + 8 * (idx % (pw / 8)));  // row n, 8 columns of the p tile
        else vc[u] = ldg16(Cg + (size_t)idx * 8);
      }
    }
    // The memory system shares its bandwidth among everything that is outstanding: whatever is requested together
    // lands together, at the end of the burst.  So the requests go out in two waves of requests: B and C (which
    // everything waits for) and both A units of the first four waves now; the A units of the other four waves
    // once B and C have landed.  The first four waves (one per SIMD) then compute while the rows of their SIMD
    // partners are still on the way.  (A barrier between the B / C requests and the first A requests, which
    // kept the order in the CU's memory pipeline strict, cost 1 us of issue time and gained nothing.)
    if (wave < waves / 2) {
      if (unit < unit_end) fetch_a(unit, areg0);
      if (unit + waves < unit_end) fetch_a(unit + waves, areg1);
    }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int idx = u * threads + tid;
      if (idx < nb) {
        if constexpr (ROWMAJOR) *reinterpret_cast<v4u*>(Bs + (idx / (N / 8)) * BRS + 8 * (idx % (N / 8))) = vb[u];
        else *reinterpret_cast<v4u*>(Bs + (idx / CPR) * BLD + 8 * (idx % CPR)) = vb[u];
      }
    }
#pragma unroll
    for (int u = 0; u < UC; ++u) {
      const int idx = u * threads + tid;
      if (idx < ncq) {
        if constexpr (ROWMAJOR) {
          *reinterpret_cast<v4u*>(Cs + (idx / (pw / 8)) * CRS + 8 * (idx % (pw / 8))) = vc[u];
        } else {
          const int p = idx / (N / 8), n8 = idx % (N / 8);
          // CLD is not a multiple of 8 halfs: two 8-byte pieces
          *reinterpret_cast<v2u*>(Cs + p * CLD + 8 * n8) = v2u{vc[u][0], vc[u][1]};
          *reinterpret_cast<v2u*>(Cs + p * CLD + 8 * n8 + 4) = v2u{vc[u][2], vc[u][3]};
        }
      }
    }
  }
  __syncthreads();
  if (wave >= waves / 2) {
    if (unit < unit_end) fetch_a(unit, areg0);
    if (unit + waves < unit_end) fetch_a(unit + waves, areg1);
  }

  // one 32-row unit whose A chunks are in ar; refills ar with the unit two further on
  auto do_unit = [&](int un, v4u (&ar)[AN]) __attribute__((always_inline)) {
    // ---- A rows: park in the wave's region and pull the MFMA fragments; step s contracts
    // k in [8s, 8s+8) (lanes 0-31) and [K/2 + 8s, K/2 + 8s + 8) (lanes 32-63)
    v8h afrag[KS];
    static_for<AN>([&](auto uc) __attribute__((always_inline)) {
      constexpr int u = decltype(uc)::value;
      const int chunk = u * 64 + lane;
      *reinterpret_cast<v4u*>(Wr + (chunk / CPR) * BLD + 8 * (chunk % CPR)) = ar[u];
    });
#pragma unroll
    for (int s = 0; s < KS; ++s) afrag[s] = *reinterpret_cast<const v8h*>(Wr + j * BLD + hh * (K / 2) + 8 * s);
    if (un + 2 * waves < unit_end) fetch_a(un + 2 * waves, ar);

    // ---- GEMM1 for every n tile: P^T tiles [32 n, 32 rows], rounded to fp16.  The n tiles advance
    // together (k step outermost), so consecutive MFMAs belong to different accumulators and none waits
    // for the one before it.
    v8h pf[NT][2];
    {
      v16f pacc[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) pacc[nt][r] = 0.0f;
      const _Float16* brow = Bs + j * BLD + hh * (K / 2);
      // ROWMAJOR: the lane's block of the transposing read: rows k = hh*K/2 + 8s + (a | a + 4), columns 4b.. of
      // the 16-column half th of the n tile
      const _Float16* btr = Bs + (hh * (K / 2) + ((lane & 15) >> 2)) * BRS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
      // The fragment of product i + LA is requested before product i is issued: a wave that is alone on its SIMD
      // (the first and the last unit of a workgroup's schedule) otherwise waits out the LDS latency before every MFMA.
      constexpr int NI = KS * NT;
      auto read_b = [&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int s = i / NT, nt = i % NT;
        if constexpr (ROWMAJOR) {
          const _Float16* p0 = btr + 8 * s * BRS + 32 * nt;
          const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
          const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 4 * BRS));
          const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          return __builtin_bit_cast(v8h, both);
        } else {
          return *reinterpret_cast<const v8h*>(brow + nt * 32 * BLD + 8 * s);
        }
      };
      v8h bf[NI];
      static_for<(LA < NI ? LA : NI)>([&](auto ic) __attribute__((always_inline)) { bf[decltype(ic)::value] = read_b(ic); });
      static_for<NI>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i + LA < NI) bf[i + LA] = read_b(std::integral_constant<int, i + LA>{});
        pacc[i % NT] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[i], afrag[i / NT], pacc[i % NT], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      });
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) pf[nt][s][e] = (_Float16)pacc[nt][8 * s + e];
    }

    // ---- GEMM2 and store, 64 columns of D at a time
    static_for<PG>([&](auto pgc) __attribute__((always_inline)) {
      constexpr int pg = decltype(pgc)::value;
      constexpr int PW = (PT - 2 * pg) >= 2 ? 2 : 1;  // p tiles in this group
      v16f dacc[PW];
#pragma unroll
      for (int q = 0; q < PW; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) dacc[q][r] = 0.0f;
      constexpr int NI = NT * PW * 2;
      auto read_c = [&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int nt = i / (PW * 2), q = (i / 2) % PW, s = i % 2;
        if constexpr (ROWMAJOR) {
          // rows n = 32 nt + 16 s + 4 hh + a (and + 8), columns of p tile 2 pg + q
          const _Float16* ctr = Cs + (nt * 32 + 4 * hh + ((lane & 15) >> 2)) * CRS + (2 * pg + q) * 32 +
                                16 * ((lane >> 4) & 1) + 4 * (lane & 3);
          const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(ctr + 16 * s * CRS));
          const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(ctr + (16 * s + 8) * CRS));
          const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          return __builtin_bit_cast(v8h, both);
        } else {
          const _Float16* crow = Cs + ((2 * pg + q) * 32 + j) * CLD + nt * 32 + 4 * hh;
          const v4h c0 = *reinterpret_cast<const v4h*>(crow + 16 * s);
          const v4h c1 = *reinterpret_cast<const v4h*>(crow + 16 * s + 8);
          return v8h{c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
        }
      };
      v8h cf[NI];
      static_for<(LA < NI ? LA : NI)>([&](auto ic) __attribute__((always_inline)) { cf[decltype(ic)::value] = read_c(ic); });
      static_for<NI>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int nt = i / (PW * 2), q = (i / 2) % PW, s = i % 2;
        if constexpr (i + LA < NI) cf[i + LA] = read_c(std::integral_constant<int, i + LA>{});
        dacc[q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cf[i], pf[nt][s], dacc[q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      });
      // D^T accumulators -> wave-private LDS [row][p] -> 16-byte row segments.
      // A wave reads back only what it wrote itself and LDS operations of one
      // wave complete in order, so no barrier is needed.
#pragma unroll
      for (int q = 0; q < PW; ++q)
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const v4h o = {(_Float16)dacc[q][4 * gq + 0], (_Float16)dacc[q][4 * gq + 1], (_Float16)dacc[q][4 * gq + 2],
                         (_Float16)dacc[q][4 * gq + 3]};
          *reinterpret_cast<v4h*>(Wr + j * DLD + q * 32 + 8 * gq + 4 * hh) = o;
        }
      constexpr int segs = PW * 4;  // 16-byte segments per row
#pragma unroll
      for (int idx = lane; idx < 32 * segs; idx += 64) {
        const int r = idx / segs;
        const int sg = idx - r * segs;
        const int grow = un * 32 + r;
        if (grow < M) {
          const v2u lo = *reinterpret_cast<const v2u*>(Wr + r * DLD + 8 * sg);
          const v2u hi = *reinterpret_cast<const v2u*>(Wr + r * DLD + 8 * sg + 4);
          // streaming store: D is not read again by this launch.  Lines left dirty in L2 are written back only when the
          // kernel ends, and the next launch in the stream waits for that: with plain stores 4.7 us of every call of
          // configuration 2 lay between the last workgroup's end and the next launch's start.
          __builtin_nontemporal_store(v4u{lo[0], lo[1], hi[0], hi[1]}, reinterpret_cast<v4u*>(Dg + (size_t)grow * P + 64 * pg + 8 * sg));
        }
      }
    });
  };
  for (; unit < unit_end; unit += 2 * waves) {
    do_unit(unit, areg0);
    if (unit + waves < unit_end) do_unit(unit + waves, areg1);
  }
}

template <int KS, int PT, int NT, bool ROWMAJOR = false>
static int launch_b2b8(const void* A, const void* B, const void* C, void* D, int G, int M, int P, int p_base,
                       int ptiles, int cus, int lds_max, bool* handled, hipStream_t s) {
  constexpr int K = 16 * KS, N = 32 * NT, pw = 32 * PT, waves = 8;
  B2BGrid gr;
  gr.ptiles = ptiles;
  gr.wave_region = std::max(32 * (K + 8), 32 * (64 + 4));
  const size_t lds = (size_t)((ROWMAJOR ? K * (N + 32) + N * (pw + 32) : N * (K + 8) + pw * (N + 4)) + waves * gr.wave_region) * 2;
  *handled = (int)lds <= lds_max;
  if (!*handled) return FTK_OK;
  const int row_units = (M + 31) / 32;
  const long long units = (long long)G * gr.ptiles;
  long long per = (cus + units - 1) / units;
  per = std::max(1LL, std::min(per, (long long)(row_units + waves - 1) / waves));
  gr.per_problem = (int)per;
  const long long total = units * per;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: grid too large");
  gr.total = (int)total;
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)b2b_gemm8_kernel<KS, PT, NT, ROWMAJOR>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_once.done(attr_bit);
  }
  hipLaunchKernelGGL((b2b_gemm8_kernel<KS, PT, NT, ROWMAJOR>), dim3(gr.total), dim3(waves * 64), lds, s, (const _Float16*)A,
                     (const _Float16*)B, (const _Float16*)C, (_Float16*)D, M, P, p_base, gr);
  return check_launch("b2b_gemm8_kernel");
}

// Wide-N form (N = 256 or 512, K and P 64 or 128), built for the shapes of the reference's own benchmark, [M, 64] x [64, 256 | 512] x [., 64]
// (benchmarks/fused_two_hgemms/fractaltensor/fused_two_hgemms.cu:152-175): one problem, few bytes (2 to 4.5 MB that
// stay in the caches), so what counts is the length of the dependency chain and how many cache lines a workgroup
// touches.  The WAVES waves of a workgroup split N: wave w forms the 32*NTW columns [n0, n0 + 32 NTW) of P for a
// 32-row unit (K/16 * NTW MFMAs), rounds them to fp16 and multiplies them with its rows of C (2 * NTW * PT MFMAs),
// which leaves a partial D tile per wave; the partials are summed in fp32 through LDS and the 32 x P tile leaves as
// whole rows.  A wave's operands of B and C do not depend on the unit: the workgroup brings B and then C through
// LDS once (coalesced 16-byte loads, every cache line once; a wave's strided fragment loads would touch 32 lines per
// instruction), every wave keeps its fragments in registers, and the workgroup then walks its units with the next
// unit's A rows on the way while the current one is computed.  The contraction order of both products is the one
// of the kernels above.
template <int KS, int PT, int NTW, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void b2b_wide_kernel(const _Float16* __restrict__ A,
                                                              const _Float16* __restrict__ Bm,
                                                              const _Float16* __restrict__ Cm, _Float16* __restrict__ D,
                                                              int M, int units, int per) {
  constexpr int K = 16 * KS;
  constexpr int N = 32 * NTW * WAVES;
  constexpr int P = 32 * PT;
  constexpr int threads = WAVES * 64;
  constexpr int BLD = K + 8;  // padded row of B and of the A units (halfs)
  constexpr int CLD = N + 4;  // padded row of C (halfs)
  constexpr int RLD = P + 4;  // padded row of a partial tile (floats)
  constexpr int CPR = K / 8;  // 16-byte chunks per row of A and B
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // first B, then C pass through the whole of it; afterwards [A units x 2][partial tiles]
  _Float16* const stage = reinterpret_cast<_Float16*>(smem);
  _Float16* const As = reinterpret_cast<_Float16*>(smem);                  // [2][32][BLD]
  float* const red = reinterpret_cast<float*>(smem + 2 * 32 * BLD * 2);    // [WAVES][32][RLD]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  const int g = blockIdx.x / per;
  const int part = blockIdx.x - g * per;
  const int n0 = wave * 32 * NTW;

  const _Float16* Ag = A + (size_t)g * M * K;
  const _Float16* Bg = Bm + (size_t)g * N * K;
  const _Float16* Cg = Cm + (size_t)g * P * N;
  _Float16* Dg = D + (size_t)g * M * P;

  // ---- B, C and the first A unit: every load requested before the first is used
  constexpr int nb = N * CPR, nc = P * (N / 8);
  constexpr int UB = (nb + threads - 1) / threads, UC = (nc + threads - 1) / threads;
  constexpr bool a_all = 32 * CPR <= threads;   // one chunk of an A unit per thread
  static_assert(a_all, "an A unit is fetched by one load per thread");
  v4u vb[UB], vc[UC], va;
  auto fetch_a = [&](int un) __attribute__((always_inline)) {
    if (tid < 32 * CPR) va = ldg16(Ag + (size_t)min(un * 32 + tid / CPR, M - 1) * K + 8 * (tid % CPR));
  };
  auto park_a = [&](int buf) __attribute__((always_inline)) {
    if (tid < 32 * CPR) *reinterpret_cast<v4u*>(As + buf * 32 * BLD + (tid / CPR) * BLD + 8 * (tid % CPR)) = va;
  };
#pragma unroll
  for (int u = 0; u < UB; ++u) {
    const int idx = u * threads + tid;
    if (idx < nb) vb[u] = ldg16(Bg + (size_t)idx * 8);
  }
#pragma unroll
  for (int u = 0; u < UC; ++u) {
    const int idx = u * threads + tid;
    if (idx < nc) vc[u] = ldg16(Cg + (size_t)idx * 8);
  }
  int unit = part;
  if (unit < units) fetch_a(unit);

  v8h bfrag[NTW][KS];
  v4h cfrag[PT][NTW][2][2];
#pragma unroll
  for (int u = 0; u < UB; ++u) {
    const int idx = u * threads + tid;
    if (idx < nb) *reinterpret_cast<v4u*>(stage + (idx / CPR) * BLD + 8 * (idx % CPR)) = vb[u];
  }
  __syncthreads();
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int s = 0; s < KS; ++s)
      bfrag[nt][s] = *reinterpret_cast<const v8h*>(stage + (n0 + 32 * nt + j) * BLD + hh * (K / 2) + 8 * s);
  __syncthreads();
#pragma unroll
  for (int u = 0; u < UC; ++u) {
    const int idx = u * threads + tid;
    if (idx < nc) {
      const int p = idx / (N / 8), n8 = idx % (N / 8);
      *reinterpret_cast<v2u*>(stage + p * CLD + 8 * n8) = v2u{vc[u][0], vc[u][1]};   // CLD is no multiple of 8 halfs
      *reinterpret_cast<v2u*>(stage + p * CLD + 8 * n8 + 4) = v2u{vc[u][2], vc[u][3]};
    }
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < PT; ++q)
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const _Float16* crow = stage + (32 * q + j) * CLD + n0 + 32 * nt + 16 * s + 4 * hh;
        cfrag[q][nt][s][0] = *reinterpret_cast<const v4h*>(crow);
        cfrag[q][nt][s][1] = *reinterpret_cast<const v4h*>(crow + 8);
      }
  __syncthreads();
  if (unit < units) park_a(0);
  __syncthreads();

  int buf = 0;
  for (; unit < units; unit += per) {
    const int next = unit + per;
    if (next < units) fetch_a(next);
    const int r0 = unit * 32;
    // GEMM1: the wave's columns of P for the unit's rows, rounded to fp16
    v8h pf[NTW][2];
    {
      const _Float16* arow = As + buf * 32 * BLD + j * BLD + hh * (K / 2);
      v8h afrag[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) afrag[s] = *reinterpret_cast<const v8h*>(arow + 8 * s);
      v16f pacc[NTW];
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) pacc[nt][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) pacc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag[nt][s], afrag[s], pacc[nt], 0, 0, 0);
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) pf[nt][s][e] = (_Float16)pacc[nt][8 * s + e];
    }
    // GEMM2 over the wave's n: a partial D^T tile per 32 columns of D, written to LDS [wave][row][p]
    // (the lane holds p = 32q + 8g + 4hh + r of row j)
    float* mine = red + (size_t)wave * 32 * RLD + j * RLD;
#pragma unroll
    for (int q = 0; q < PT; ++q) {
      v16f dacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) dacc[r] = 0.0f;
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const v4h c0 = cfrag[q][nt][s][0], c1 = cfrag[q][nt][s][1];
          const v8h c = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
          dacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(c, pf[nt][s], dacc, 0, 0, 0);
        }
#pragma unroll
      for (int gq = 0; gq < 4; ++gq)
        *reinterpret_cast<v4f*>(mine + 32 * q + 8 * gq + 4 * hh) = v4f{dacc[4 * gq], dacc[4 * gq + 1], dacc[4 * gq + 2], dacc[4 * gq + 3]};
    }
    __syncthreads();
    constexpr int QPR = P / 4;  // quadruples per row
    for (int idx = tid; idx < 32 * QPR; idx += threads) {
      const int r = idx / QPR, c4 = idx - r * QPR;
      v4f sum = *reinterpret_cast<const v4f*>(red + r * RLD + 4 * c4);
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        const v4f x = *reinterpret_cast<const v4f*>(red + (size_t)w * 32 * RLD + r * RLD + 4 * c4);
        sum[0] += x[0]; sum[1] += x[1]; sum[2] += x[2]; sum[3] += x[3];
      }
      if (r0 + r < M) {
        const v4h o = {(_Float16)sum[0], (_Float16)sum[1], (_Float16)sum[2], (_Float16)sum[3]};
        __builtin_nontemporal_store(o, reinterpret_cast<v4h*>(Dg + (size_t)(r0 + r) * P + 4 * c4));
      }
    }
    if (next < units) park_a(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
}

template <int KS, int PT, int NTW, int WAVES>
static int launch_b2b_wide(const void* A, const void* B, const void* C, void* D, int G, int M, int cus, int lds_max,
                           bool* handled, hipStream_t s) {
  constexpr int K = 16 * KS, N = 32 * NTW * WAVES, P = 32 * PT;
  const size_t loop_bytes = (size_t)2 * 32 * (K + 8) * 2 + (size_t)WAVES * 32 * (P + 4) * sizeof(float);
  const size_t stage_bytes = std::max((size_t)N * (K + 8) * 2, (size_t)P * (N + 4) * 2);
  const size_t lds = std::max(loop_bytes, stage_bytes);
  const long long units = (M + 31) / 32;
  // enough workgroups to fill the chip once; each walks its share of the units with B and C fragments in registers
  const long long per = std::max(1LL, std::min(units, (long long)cus / std::max(1, G)));
  *handled = (int)lds <= lds_max && per * G <= 0x7fffffffLL;
  if (!*handled) return FTK_OK;
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)b2b_wide_kernel<KS, PT, NTW, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_once.done(attr_bit);
  }
  hipLaunchKernelGGL((b2b_wide_kernel<KS, PT, NTW, WAVES>), dim3((unsigned)(per * G)), dim3(WAVES * 64), lds, s,
                     (const _Float16*)A, (const _Float16*)B, (const _Float16*)C, (_Float16*)D, M, (int)units, (int)per);
  return check_launch("b2b_wide_kernel");
}

static int b2b_wave_region(int K, int pw) { return 32 * (K + 8) + 32 * (pw + 4); }

static size_t b2b_lds_bytes(int N, int K, int pw, int waves) {
  return (size_t)(N * (K + 8) + pw * (N + 4) + waves * b2b_wave_region(K, pw)) * 2;
}

template <int KS, int PT>
static int launch_b2b_cols(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int P,
                           int p_base, int ptiles, int cus, int lds_max, hipStream_t s) {
  constexpr int K = 16 * KS;
  constexpr int pw = 32 * PT;
  int waves = 4;
  while (waves > 1 && (int)b2b_lds_bytes(N, K, pw, waves) > lds_max) waves >>= 1;
  const size_t lds = b2b_lds_bytes(N, K, pw, waves);
  if ((int)lds > lds_max)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE,
                "ftk_b2b_gemm_f16: B and C tiles for N=%d K=%d P=%d need %zu bytes of LDS, the device has %d", N, K, P,
                lds, lds_max);
  B2BGrid gr;
  gr.ptiles = ptiles;
  gr.wave_region = b2b_wave_region(K, pw);
  const int row_pairs = (M + 63) / 64;
  const long long units = (long long)G * gr.ptiles;
  // enough workgroups per (problem, p tile) to fill the chip once; each walks its share of the rows
  long long per = (cus + units - 1) / units;
  per = std::max(1LL, std::min(per, (long long)(row_pairs + waves - 1) / waves));
  gr.per_problem = (int)per;
  const long long total = units * per;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: grid too large");
  gr.total = (int)total;
  const void* fn = (const void*)b2b_gemm_kernel<KS, PT>;
  static DeviceMax attr_lds;
  int dev;
  if (attr_lds.below((int)lds, &dev)) {
    FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_lds.raise(dev, (int)lds);
  }
  hipLaunchKernelGGL((b2b_gemm_kernel<KS, PT>), dim3(gr.total), dim3(waves * 64), lds, s, (const _Float16*)A,
                     (const _Float16*)B, (const _Float16*)C, (_Float16*)D, M, N, P, p_base, gr);
  return check_launch("b2b_gemm_kernel");
}

// Columns of D go out in workgroup tiles of 128; a remainder of 32, 64 or 96
// columns is a second launch of the narrower instantiation.
template <int KS>
static int launch_b2b(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int P, int cus,
                      int lds_max, hipStream_t s) {
  const int full = P / B2B_PTILE;
  const int rem = (P % B2B_PTILE) / 32;
  int rc = FTK_OK;
  if (full > 0) {
    // the eight-wave kernel covers K in {64, 128} x N in {64, 128}; FTK_B2B_WAVES=4 forces the four-wave one
    bool handled = false;
    static const bool allow8 = !(getenv("FTK_B2B_WAVES") && atoi(getenv("FTK_B2B_WAVES")) == 4);
    if constexpr (KS == 4 || KS == 8) {
      if (allow8 && N == 128) rc = launch_b2b8<KS, 4, 4>(A, B, C, D, G, M, P, 0, full, cus, lds_max, &handled, s);
      if (allow8 && N == 64) rc = launch_b2b8<KS, 4, 2>(A, B, C, D, G, M, P, 0, full, cus, lds_max, &handled, s);
    }
    if (!handled) rc = launch_b2b_cols<KS, 4>(A, B, C, D, G, M, N, P, 0, full, cus, lds_max, s);
  }
  if (rc) return rc;
  const int pb = full * B2B_PTILE;
  switch (rem) {
    case 1: return launch_b2b_cols<KS, 1>(A, B, C, D, G, M, N, P, pb, 1, cus, lds_max, s);
    case 2: return launch_b2b_cols<KS, 2>(A, B, C, D, G, M, N, P, pb, 1, cus, lds_max, s);
    case 3: return launch_b2b_cols<KS, 3>(A, B, C, D, G, M, N, P, pb, 1, cus, lds_max, s);
    default: return FTK_OK;
  }
}


// General form for everything the kernels above are not built for: any K % 16 == 0 (they hold a whole A row
// as register fragments and B with all of its k in LDS, K <= 128), N up to kStreamMaxN, B and C of any size --
// the shapes of the reference's own test, [192, 704] x [704, 448] x [448, 832] (tests/test_b2b_gemm.cu:137-149),
// among them.  A workgroup owns 32 rows.  Its waves share out the 32-column tiles of P = A B: a tile is one
// accumulator, the k loop runs over the whole of K with both operands read as 16-byte pieces straight from global
// memory (every lane its own row: 32 rows x 32 bytes per product, each cache line serves four products), and the
// tile goes to LDS rounded to fp16, [row][n].  After a barrier the waves share out the 32-column tiles of D: the
// rows of P are the B operand out of LDS, the rows of C the A operand from global memory.  Same transposed
// products, same rounding of P and same lane ownership as above; built for coverage, not for speed.
constexpr int kStreamMaxN = 2048;

__global__ __launch_bounds__(256) void b2b_stream_kernel(const _Float16* __restrict__ A, const _Float16* __restrict__ Bm,
                                                         const _Float16* __restrict__ Cm, _Float16* __restrict__ D, int M,
                                                         int N, int K, int P, int row_blocks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  _Float16* const Ps = reinterpret_cast<_Float16*>(smem);  // [32][N + 8]
  const int PLD = N + 8;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  const int g = blockIdx.x / row_blocks;
  const int rb = blockIdx.x - g * row_blocks;
  const int row = min(rb * 32 + j, M - 1);  // rows past the end repeat the last one and are not stored
  const _Float16* arow = A + ((size_t)g * M + row) * K + 8 * hh;
  for (int nt = wave; nt < N / 32; nt += 4) {
    const _Float16* brow = Bm + ((size_t)g * N + nt * 32 + j) * K + 8 * hh;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll 4
    for (int k = 0; k < K; k += 16) {
      const v8h bf = *reinterpret_cast<const v8h*>(brow + k);
      const v8h af = *reinterpret_cast<const v8h*>(arow + k);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af, acc, 0, 0, 0);
    }
    // the lane holds, for row j, the columns nt * 32 + 8 q + 4 hh + r of P
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4h o = {(_Float16)acc[4 * q], (_Float16)acc[4 * q + 1], (_Float16)acc[4 * q + 2], (_Float16)acc[4 * q + 3]};
      *reinterpret_cast<v4h*>(Ps + j * PLD + nt * 32 + 8 * q + 4 * hh) = o;
    }
  }
  __syncthreads();
  const _Float16* prow = Ps + j * PLD + 8 * hh;
  const bool stored = rb * 32 + j < M;
  _Float16* drow = D + ((size_t)g * M + row) * P + 4 * hh;
  for (int pt = wave; pt < P / 32; pt += 4) {
    const _Float16* crow = Cm + ((size_t)g * P + pt * 32 + j) * N + 8 * hh;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll 4
    for (int n = 0; n < N; n += 16) {
      const v8h cf = *reinterpret_cast<const v8h*>(crow + n);
      const v8h pf = *reinterpret_cast<const v8h*>(prow + n);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(cf, pf, acc, 0, 0, 0);
    }
    if (stored) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4h o = {(_Float16)acc[4 * q], (_Float16)acc[4 * q + 1], (_Float16)acc[4 * q + 2], (_Float16)acc[4 * q + 3]};
        *reinterpret_cast<v4h*>(drow + pt * 32 + 8 * q) = o;
      }
    }
  }
}

// The fused kernels keep B (all of K) and a tile of C in LDS: K of 32, 64, 96 or 128, and B and C small enough to
// fit beside one wave's region.  Everything else goes to the general kernel.
static bool b2b_fits_fused(int N, int K, int P, int lds_max) {
  return (K == 32 || K == 64 || K == 96 || K == 128) && (int)b2b_lds_bytes(N, K, std::min(P, B2B_PTILE), 1) <= lds_max &&
         (P % B2B_PTILE == 0 || (int)b2b_lds_bytes(N, K, P % B2B_PTILE, 1) <= lds_max);
}

static bool b2b_fits_stream(int N, int lds_max) { return N <= kStreamMaxN && 32 * (N + 8) * 2 <= lds_max; }

static int launch_b2b_stream(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int K, int P,
                             int lds_max, hipStream_t s) {
  const size_t lds = (size_t)32 * (N + 8) * 2;
  if (!b2b_fits_stream(N, lds_max))
    return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: N=%d: 32 rows of the intermediate product need %zu bytes of LDS (N <= %d)",
                N, lds, kStreamMaxN);
  const long long row_blocks = (M + 31) / 32;
  const long long total = row_blocks * G;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: grid too large");
  static DeviceMax attr_lds;
  int dev;
  if (attr_lds.below((int)lds, &dev)) {
    FTK_HIP(hipFuncSetAttribute((const void*)b2b_stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_lds.raise(dev, (int)lds);
  }
  hipLaunchKernelGGL(b2b_stream_kernel, dim3((unsigned)total), dim3(256), lds, s, (const _Float16*)A, (const _Float16*)B,
                     (const _Float16*)C, (_Float16*)D, M, N, K, P, (int)row_blocks);
  return check_launch("b2b_stream_kernel");
}

}  // namespace ftk

extern "C" int ftk_b2b_gemm_f16_supported(int N, int K, int P) {
  using namespace ftk;
  if (N <= 0 || K <= 0 || P <= 0 || N % 32 || P % 32 || K % 16) return 0;
  const DeviceProps* dp = nullptr;
  if (device_props(&dp)) return 0;
  return (b2b_fits_fused(N, K, P, dp->lds_optin) || b2b_fits_stream(N, dp->lds_optin)) ? 1 : 0;
}

extern "C" int ftk_b2b_gemm_f16(const void* A, const void* B, const void* C, void* D, int G, int M, int N, int K,
                                int P, ftk_stream_t stream) {
  using namespace ftk;
  if (!A || !B || !C || !D) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_b2b_gemm_f16: A, B, C, D must be non-NULL");
  if (G <= 0 || M <= 0 || N <= 0 || K <= 0 || P <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_b2b_gemm_f16: G, M, N, K, P must be positive");
  if (N % 32 || P % 32) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: N=%d and P=%d must be multiples of 32", N, P);
  if (K % 16) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_b2b_gemm_f16: K=%d must be a multiple of 16", K);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const bool fast = b2b_fits_fused(N, K, P, dp->lds_optin);
  if (!fast) return launch_b2b_stream(A, B, C, D, G, M, N, K, P, dp->lds_optin, s);
  // wide N with few columns of D (the reference benchmark's shapes): N split over the waves of a workgroup.
  // FTK_B2B_WIDE=0 keeps them on the general kernel.
  static const bool allow_wide = !(getenv("FTK_B2B_WIDE") && atoi(getenv("FTK_B2B_WIDE")) == 0);
  if (allow_wide && (K == 64 || K == 128) && (P == 64 || P == 128) && (N == 256 || N == 512)) {
    bool handled = false;
    const int cus = dp->cus, lds = dp->lds_optin;
    const int sel = (K == 128) * 4 + (P == 128) * 2 + (N == 512);
    switch (sel) {
      case 0: rc = launch_b2b_wide<4, 2, 1, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 1: rc = launch_b2b_wide<4, 2, 2, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 2: rc = launch_b2b_wide<4, 4, 1, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 3: rc = launch_b2b_wide<4, 4, 2, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 4: rc = launch_b2b_wide<8, 2, 1, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 5: rc = launch_b2b_wide<8, 2, 2, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      case 6: rc = launch_b2b_wide<8, 4, 1, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
      default: rc = launch_b2b_wide<8, 4, 2, 8>(A, B, C, D, G, M, cus, lds, &handled, s); break;
    }
    if (rc || handled) return rc;
  }
  switch (K) {
    case 32: return launch_b2b<2>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    case 64: return launch_b2b<4>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    case 96: return launch_b2b<6>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
    default: return launch_b2b<8>(A, B, C, D, G, M, N, P, dp->cus, dp->lds_optin, s);
  }
}

extern "C" int ftk_b2b_gemm_rowmajor_f16(const void* A, const void* B, const void* C, void* D, int G, int M, int N,
                                         int K, int P, ftk_stream_t stream) {
  using namespace ftk;
  const char* who = "ftk_b2b_gemm_rowmajor_f16";
  if (!A || !B || !C || !D) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: A, B, C, D must be non-NULL", who);
  if (G <= 0 || M <= 0 || N <= 0 || K <= 0 || P <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "%s: G, M, N, K, P must be positive", who);
  if ((K != 64 && K != 128) || (N != 64 && N != 128) || P % 128)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: built for K and N in {64, 128} and P a multiple of 128, got K=%d N=%d P=%d", who,
                K, N, P);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  bool handled = false;
  const int full = P / B2B_PTILE;
  if (K == 64 && N == 64) rc = launch_b2b8<4, 4, 2, true>(A, B, C, D, G, M, P, 0, full, dp->cus, dp->lds_optin, &handled, s);
  else if (K == 64) rc = launch_b2b8<4, 4, 4, true>(A, B, C, D, G, M, P, 0, full, dp->cus, dp->lds_optin, &handled, s);
  else if (N == 64) rc = launch_b2b8<8, 4, 2, true>(A, B, C, D, G, M, P, 0, full, dp->cus, dp->lds_optin, &handled, s);
  else rc = launch_b2b8<8, 4, 4, true>(A, B, C, D, G, M, P, 0, full, dp->cus, dp->lds_optin, &handled, s);
  if (rc) return rc;
  if (!handled) return fail(FTK_ERR_DEVICE, "%s: the device's LDS does not hold the B and C tiles", who);
  return FTK_OK;
}
