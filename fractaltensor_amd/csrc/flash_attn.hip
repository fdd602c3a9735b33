// Non-causal flash attention for gfx950: fp16 Q/K/V/O, fp32 accumulation on
// v_mfma_f32_32x32x16_f16, online softmax (running max and sum) in registers.
//
// Both contractions are computed transposed so that a lane owns one query row:
//   S^T[key, q] = sum_d Ks[key][d] * Q[q][d]     MFMA A-operand = K rows (LDS),
//                                                B-operand = Q row fragments (registers)
//   O^T[d, q]  += sum_key Vt[d][key] * P[q][key]  A-operand = V^T rows (LDS),
//                                                B-operand = exp'd scores, fp16 (registers)
// The 32x32 accumulator of lane (q = lane%32, half = lane/32) holds, for that
// one query, keys 8g + 4*half + r (g = reg/4, r = reg%4) of a 32-key subtile.
// Row max / row sum are therefore a reduction over the lane's own registers
// plus one exchange with lane^32; the rescale factor of O^T is lane-local; and
// the exp'd scores already are a valid MFMA B-operand if the PV product
// contracts keys in the order the lane holds them (step s of a subtile takes
// keys {16s + 4*half + r} U {16s + 8 + 4*half + r}), which only changes which
// two 8-byte pieces of a V^T row the A-operand reads.  P never touches LDS.
//
// A workgroup is 4 waves; each wave owns 32*QT query rows, the workgroup
// streams K/V in 64-key tiles: K as stored ([key][d], padded rows), V
// transposed on the way into LDS ([d][key]) by 4x4 register transposes.  Tiles
// are double buffered with register prefetch of the next tile.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "ftk_common.h"

namespace ftk {

// Compile-time loop: the body sees its index as a constant expression, so
// register arrays indexed by it are promoted to registers even when the body
// sits under a runtime condition.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

constexpr int FA_KT = 64;          // keys per tile
constexpr int FA_VLD = FA_KT + 4;  // padded V^T row (halfs)
constexpr float FA_TAU = 8.0f;     // slack (in powers of two) before the running maximum is moved

template <int D, int QT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void flash_attn_kernel(const _Float16* __restrict__ Q,
                                                         const _Float16* __restrict__ K,
                                                         const _Float16* __restrict__ V,
                                                         _Float16* __restrict__ O, int Sq, int Skv,
                                                         float scale_log2e, int nqb) {
  constexpr int KLD = D + 8;   // padded K row (halfs)
  constexpr int DS = D / 16;   // k steps of S^T
  constexpr int DT = D / 32;   // d tiles of O^T
  constexpr int KSZ = FA_KT * KLD;
  constexpr int VSZ = D * FA_VLD;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  _Float16* Ks = reinterpret_cast<_Float16*>(smem);  // [2][64][KLD]
  _Float16* Vt = Ks + 2 * KSZ;                       // [2][D][VLD]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  // One-dimensional grid of nqb query blocks x (batch*heads).  The hardware
  // deals workgroups round-robin over the 8 XCDs; remap so that the query
  // blocks of one head run on one XCD and share its L2 copy of K and V.
  int id = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) id = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int bh = id / nqb;
  const int qb = id - bh * nqb;
  constexpr int NT = WAVES * 64;  // threads
  const int q_base = qb * (WAVES * 32 * QT) + wave * (32 * QT);

  const _Float16* Qg = Q + (size_t)bh * Sq * D;
  const _Float16* Kg = K + (size_t)bh * Skv * D;
  const _Float16* Vg = V + (size_t)bh * Skv * D;
  _Float16* Og = O + (size_t)bh * Sq * D;

  // ---- Q row fragments, resident for the whole kernel
  v8h qf[QT][DS];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int row = min(q_base + 32 * qt + j, Sq - 1);
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(Qg + (size_t)row * D + 16 * s + 8 * hh);
      qf[qt][s] = *reinterpret_cast<const v8h*>(&v);
    }
  }

  v16f oacc[QT][DT];
  float m_run[QT], l_run[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = -INFINITY;
    l_run[qt] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[qt][dt][r] = 0.0f;
  }

  // ---- staging assignments
  constexpr int KN = FA_KT * (D / 8) / NT;   // 16-byte K loads per thread per tile
  constexpr int VN = (FA_KT / 4) * (D / 4) / NT;  // 4x4 V blocks per thread per tile
  static_assert(KN >= 1 && VN >= 1, "tile too small for this many threads");
  v4u kreg[KN];
  v2u vreg[VN][4];

  auto load_tile = [&](int kt) __attribute__((always_inline)) {
    const int key0 = kt * FA_KT;
    static_for<KN>([&](auto nc) __attribute__((always_inline)) {
      constexpr int n = decltype(nc)::value;
      const int idx = tid + NT * n;
      const int key = min(key0 + idx / (D / 8), Skv - 1);
      const int c8 = idx % (D / 8);
      kreg[n] = *reinterpret_cast<const v4u*>(Kg + (size_t)key * D + 8 * c8);
    });
    static_for<VN * 4>([&](auto nc) __attribute__((always_inline)) {
      constexpr int n = decltype(nc)::value / 4;
      constexpr int nn = decltype(nc)::value % 4;
      const int u = tid + NT * n;
      const int dg = u % (D / 4);
      const int kq = u / (D / 4);
      const int key = min(key0 + 4 * kq + nn, Skv - 1);
      vreg[n][nn] = *reinterpret_cast<const v2u*>(Vg + (size_t)key * D + 4 * dg);
    });
  };
  auto store_tile = [&](int buf) __attribute__((always_inline)) {
    _Float16* ks = Ks + buf * KSZ;
    _Float16* vt = Vt + buf * VSZ;
    static_for<KN>([&](auto nc) __attribute__((always_inline)) {
      constexpr int n = decltype(nc)::value;
      const int idx = tid + NT * n;
      const int key = idx / (D / 8);
      const int c8 = idx % (D / 8);
      *reinterpret_cast<v4u*>(ks + key * KLD + 8 * c8) = kreg[n];
    });
    static_for<VN>([&](auto nc) __attribute__((always_inline)) {
      constexpr int n = decltype(nc)::value;
      const int u = tid + NT * n;
      const int dg = u % (D / 4);
      const int kq = u / (D / 4);
      const v2u r0 = vreg[n][0], r1 = vreg[n][1], r2 = vreg[n][2], r3 = vreg[n][3];
      // 4x4 transpose of halfs: row e of the result = element e of keys 0..3
      v2u c0, c1, c2, c3;
      c0.x = __builtin_amdgcn_perm(r1.x, r0.x, 0x05040100u);
      c0.y = __builtin_amdgcn_perm(r3.x, r2.x, 0x05040100u);
      c1.x = __builtin_amdgcn_perm(r1.x, r0.x, 0x07060302u);
      c1.y = __builtin_amdgcn_perm(r3.x, r2.x, 0x07060302u);
      c2.x = __builtin_amdgcn_perm(r1.y, r0.y, 0x05040100u);
      c2.y = __builtin_amdgcn_perm(r3.y, r2.y, 0x05040100u);
      c3.x = __builtin_amdgcn_perm(r1.y, r0.y, 0x07060302u);
      c3.y = __builtin_amdgcn_perm(r3.y, r2.y, 0x07060302u);
      _Float16* dst = vt + (4 * dg) * FA_VLD + 4 * kq;
      *reinterpret_cast<v2u*>(dst) = c0;
      *reinterpret_cast<v2u*>(dst + FA_VLD) = c1;
      *reinterpret_cast<v2u*>(dst + 2 * FA_VLD) = c2;
      *reinterpret_cast<v2u*>(dst + 3 * FA_VLD) = c3;
    });
  };

  const int ntiles = (Skv + FA_KT - 1) / FA_KT;
  const float tau_raw = FA_TAU / scale_log2e;
  load_tile(0);
  store_tile(0);
  __syncthreads();

  auto process_tile = [&](int kt, auto ragged_c) __attribute__((always_inline)) {
    constexpr bool ragged = decltype(ragged_c)::value;
    const int buf = kt & 1;
    if (kt + 1 < ntiles) load_tile(kt + 1);
    const _Float16* ks = Ks + buf * KSZ;
    const _Float16* vt = Vt + buf * VSZ;

    // ---- S^T = K Q^T for two 32-key subtiles
    v16f sacc[QT][2];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[qt][k2][r] = 0.0f;
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) {
      const _Float16* krow = ks + (32 * k2 + j) * KLD + 8 * hh;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const v8h kf = *reinterpret_cast<const v8h*>(krow + 16 * s);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          sacc[qt][k2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[qt][s], sacc[qt][k2], 0, 0, 0);
      }
    }

    // ---- online softmax, one query row per lane (two lanes share a row).
    // Scores stay in raw units; p = exp2(s*c - m_ref*c) with c = scale*log2(e)
    // is one fused multiply-add and one exponential per score.  m_ref is a
    // reference maximum that is only moved (and O, l rescaled) when the true
    // row maximum has run ahead of it by more than FA_TAU in exponent units:
    // any m_ref gives the same O = acc/l, p merely ranges up to 2^FA_TAU.
    v8h pf[QT][2][2];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      if constexpr (ragged) {
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kt * FA_KT + 32 * k2 + 8 * (r >> 2) + 4 * hh + (r & 3);
            if (key >= Skv) sacc[qt][k2][r] = -INFINITY;
          }
      }
      float mx = sacc[qt][0][0];
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[qt][k2][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const bool need = mx > m_run[qt] + tau_raw;
      if (__builtin_amdgcn_ballot_w64(need) != 0) {
        const float m_new = need ? mx : m_run[qt];
        const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_new) * scale_log2e);
        m_run[qt] = m_new;
        l_run[qt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[qt][dt][r] *= alpha;
      }
      const float mc = -m_run[qt] * scale_log2e;
      float psum = 0.0f;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qt][k2][8 * s + e], scale_log2e, mc));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qt][k2][8 * s + e + 1], scale_log2e, mc));
            const v2h pp = {(_Float16)p0, (_Float16)p1};
            pf[qt][k2][s][e] = pp[0];
            pf[qt][k2][s][e + 1] = pp[1];
            // row sum over the rounded values that enter the PV product, two per instruction
            psum = __builtin_amdgcn_fdot2(pp, v2h{(_Float16)1.0f, (_Float16)1.0f}, psum, false);
          }
      l_run[qt] += psum;  // this lane's half of the row sum
    }

    // ---- O^T += V^T P^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const _Float16* vrow = vt + (32 * dt + j) * FA_VLD + 4 * hh;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const v4h v0 = *reinterpret_cast<const v4h*>(vrow + 32 * k2 + 16 * s);
          const v4h v1 = *reinterpret_cast<const v4h*>(vrow + 32 * k2 + 16 * s + 8);
          const v8h vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
          for (int qt = 0; qt < QT; ++qt)
            oacc[qt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[qt][k2][s], oacc[qt][dt], 0, 0, 0);
        }
    }

    if (kt + 1 < ntiles) store_tile(buf ^ 1);
    __syncthreads();
  };

  const bool has_ragged = (Skv % FA_KT) != 0;
  const int nfull = has_ragged ? ntiles - 1 : ntiles;
  for (int kt = 0; kt < nfull; ++kt) process_tile(kt, std::false_type{});
  if (has_ragged) process_tile(ntiles - 1, std::true_type{});

  // ---- normalise and store: lane holds d = 32dt + 8g + 4*half + r of its row
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const float l = l_run[qt] + __shfl_xor(l_run[qt], 32);
    const float inv = 1.0f / l;
    const int row = q_base + 32 * qt + j;
    if (row < Sq) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4h o = {(_Float16)(oacc[qt][dt][4 * g + 0] * inv), (_Float16)(oacc[qt][dt][4 * g + 1] * inv),
                         (_Float16)(oacc[qt][dt][4 * g + 2] * inv), (_Float16)(oacc[qt][dt][4 * g + 3] * inv)};
          *reinterpret_cast<v4h*>(Og + (size_t)row * D + 32 * dt + 8 * g + 4 * hh) = o;
        }
    }
  }
}

template <int D, int QT, int WAVES>
static int launch_fa(const void* Q, const void* K, const void* V, void* O, int BH, int Sq, int Skv, float scale,
                     int lds_max, hipStream_t s) {
  const size_t lds = (size_t)2 * (FA_KT * (D + 8) + D * FA_VLD) * 2;
  if ((int)lds > lds_max) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: needs %zu bytes of LDS", lds);
  const void* fn = (const void*)flash_attn_kernel<D, QT, WAVES>;
  static bool attr_set = false;
  if (!attr_set) {
    FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  constexpr int ROWS = WAVES * 32 * QT;
  const int nqb = (Sq + ROWS - 1) / ROWS;
  const long long total = (long long)nqb * BH;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: grid too large");
  hipLaunchKernelGGL((flash_attn_kernel<D, QT, WAVES>), dim3((unsigned)total), dim3(WAVES * 64), lds, s,
                     (const _Float16*)Q, (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv,
                     scale * 1.4426950408889634f, nqb);
  return check_launch("flash_attn_kernel");
}

// Tuning hook: FTK_FA_VARIANT=1|2|3 pins the tiling variant (read once).
static int fa_variant_override() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("FTK_FA_VARIANT");
    v = e ? atoi(e) : 0;
    if (v < 0 || v > 3) v = 0;
  }
  return v;
}

}  // namespace ftk

extern "C" int ftk_flash_attn_f16(const void* Q, const void* K, const void* V, void* O, int B, int Hd, int Sq, int Skv,
                                  int D, float scale, ftk_stream_t stream) {
  using namespace ftk;
  if (!Q || !K || !V || !O) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_flash_attn_f16: Q, K, V, O must be non-NULL");
  if (B <= 0 || Hd <= 0 || Sq <= 0 || Skv <= 0 || D <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_flash_attn_f16: B, Hd, Sq, Skv, D must be positive");
  if (D != 64 && D != 128) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: D=%d must be 64 or 128", D);
  const long long bh = (long long)B * Hd;
  if (bh > (1LL << 24)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: B*Hd=%lld too large", bh);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  // Variant: 0 = choose by problem size, 1 = 4 waves x 32 rows, 2 = 4 waves x 64 rows, 3 = 8 waves x 32 rows.
  int variant = fa_variant_override();
  // measured on MI355X at B8 H16 S2048 D128: 8 waves x 32 rows (two waves per SIMD, softmax of one
  // overlapping the MFMAs of the other) beats 4 waves x 64 rows, which beats 4 waves x 32 rows
  if (variant == 0) {
    const bool big = (long long)((Sq + 255) / 256) * bh >= dp->cus;
    variant = big ? (D == 128 ? 3 : 2) : 1;
  }
  const int lds = dp->lds_optin;
  if (D == 128) {
    switch (variant) {
      case 1: return launch_fa<128, 1, 4>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
      case 3: return launch_fa<128, 1, 8>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
      default: return launch_fa<128, 2, 4>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
    }
  }
  switch (variant) {
    case 1: return launch_fa<64, 1, 4>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
    case 3:  // a 64-key tile of 64-wide heads has too little to stage for 8 waves
    default: return launch_fa<64, 2, 4>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
  }
}

