// Windowed (plus gathered) attention for gfx950, fp32: every token attends to the window centred on it and,
// optionally, to a list of further positions of its own,
//   out[t] = softmax(scale * q[t] . K[P(t)]^T) . V[P(t)],   P(t) = window(t) ++ extra[t].
// The window of token t holds positions t - half + k * dilation, k = 0 .. window-1, half = (window-1)*dilation/2,
// wrapped at the ends the way the frontend's shifted_slide wraps them: p >= S becomes p - S, p < 0 becomes
// p + S - 1 (one short of circular).
//
// HBM-bound work: Q, K and V are read once from memory (a token's window rows are its neighbours' rows, served by
// the caches) and the output is written once; the arithmetic is a handful of short dot products per token.  A
// token is held by LPT lanes of a wave, each with NP 16-byte pieces of the row; a score is a lane-local dot
// product folded across the token's lanes with shuffles, and the softmax runs online over the key list (running
// maximum, denominator and weighted sum of V rows), so nothing but the row pieces lives in registers.  What the
// kernel is short of is cache-to-CU bandwidth, not HBM: a token reads one row of K and one of V per key, so the
// window rows that a workgroup's consecutive tokens share are staged in LDS once, and all workgroups of a
// sequence run on one XCD so that its K and V pass through one L2 only.
#include "ftk_common.h"

namespace ftk {

// STAGE: the workgroup's tokens are consecutive, so their windows overlap: the TPB + 2*half rows of K and of V they
// cover are copied into LDS once and every window key is read from there (a token's own gathered rows still come
// from global memory).
template <int LPT, int NP, bool STAGE, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void windowed_attn_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                                            const float* __restrict__ V, const int* __restrict__ extra,
                                                            float* __restrict__ O, long long G, int S, int D,
                                                            int window, int dilation, int R, float scale) {
  constexpr int TPW = 64 / LPT;        // tokens per wave
  constexpr int TPB = WAVES * TPW;     // tokens per workgroup
  const int lane = threadIdx.x & 63;
  const int sub = lane % LPT;
  // Workgroup ids go round the eight XCDs, each with its own L2; a sequence's K and V rows are read by all of its
  // tokens, so all workgroups of a sequence run on one XCD: sequence g = 8 * (id / (8 * bps)) + id % 8.
  const int bps = (S + TPB - 1) / TPB;  // workgroups per sequence
  const long long round = blockIdx.x / (8LL * bps);
  const int in_round = (int)(blockIdx.x - round * 8LL * bps);
  const long long g_raw = round * 8 + in_round % 8;
  const long long g = g_raw < G ? g_raw : G - 1;
  const int D4 = D / 4;
  const float* Kg = K + (size_t)g * S * D;
  const float* Vg = V + (size_t)g * S * D;
  const int half = (window - 1) * dilation / 2;
  const int nkeys = window + R;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int t0 = (in_round / 8) * TPB;                         // first token of the workgroup
  const int tl = (threadIdx.x >> 6) * TPW + lane / LPT;        // this lane's token within it
  const int t_raw = t0 + tl;
  const bool live = g_raw < G && t_raw < S;
  const int t = t_raw < S ? t_raw : S - 1;
  const long long tok = g * S + t;

  const int rows = TPB + 2 * half;  // staged rows: positions t0 - half .. t0 + TPB - 1 + half, wrapped
  if (STAGE) {
    float4* Ks = reinterpret_cast<float4*>(lds);
    float4* Vs = Ks + (size_t)rows * D4;
    for (int idx = threadIdx.x; idx < rows * D4; idx += 64 * WAVES) {
      const int r = idx / D4, pc = idx - r * D4;
      int p = t0 - half + r;
      p = p < 0 ? p + S - 1 : (p >= S ? p - S : p);
      p = min(max(p, 0), S - 1);  // rows that only tokens past the end of the sequence would use
      Ks[idx] = *reinterpret_cast<const float4*>(Kg + (size_t)p * D + 4 * pc);
      Vs[idx] = *reinterpret_cast<const float4*>(Vg + (size_t)p * D + 4 * pc);
    }
    __syncthreads();
  }

  float4 q[NP];
#pragma unroll
  for (int n = 0; n < NP; ++n) {
    const int pc = sub + LPT * n;
    q[n] = pc < D4 ? *reinterpret_cast<const float4*>(Q + (size_t)tok * D + 4 * pc) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float4 acc[NP];
#pragma unroll
  for (int n = 0; n < NP; ++n) acc[n] = make_float4(0.f, 0.f, 0.f, 0.f);
  float m = -INFINITY, den = 0.0f;

  constexpr int KB = NP == 1 ? 4 : 2;  // keys per round: their rows are all requested before the first is used
  for (int k0 = 0; k0 < nkeys; k0 += KB) {
    float4 kk[KB][NP], v[KB][NP];
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int k = min(k0 + b, nkeys - 1);  // a key past the end repeats the last one and is given no weight
      if (STAGE && k < window) {  // the same branch for the whole wave
        const int row4 = (tl + k * dilation) * D4;
#pragma unroll
        for (int n = 0; n < NP; ++n) {
          const int pc = sub + LPT * n;
          const bool in = pc < D4;
          kk[b][n] = in ? reinterpret_cast<const float4*>(lds)[row4 + pc] : make_float4(0.f, 0.f, 0.f, 0.f);
          v[b][n] = in ? reinterpret_cast<const float4*>(lds)[rows * D4 + row4 + pc] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      } else {
        int p;
        if (k < window) {
          p = t - half + k * dilation;
          p = p < 0 ? p + S - 1 : (p >= S ? p - S : p);
        } else {
          p = extra[(size_t)tok * R + (k - window)];
          p = min(max(p, 0), S - 1);  // the caller validates; never read out of bounds
        }
        const float* kr = Kg + (size_t)p * D;
        const float* vr = Vg + (size_t)p * D;
#pragma unroll
        for (int n = 0; n < NP; ++n) {
          const int pc = sub + LPT * n;
          const bool in = pc < D4;
          kk[b][n] = in ? *reinterpret_cast<const float4*>(kr + 4 * pc) : make_float4(0.f, 0.f, 0.f, 0.f);
          v[b][n] = in ? *reinterpret_cast<const float4*>(vr + 4 * pc) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      float s = 0.0f;
#pragma unroll
      for (int n = 0; n < NP; ++n) s += q[n].x * kk[b][n].x + q[n].y * kk[b][n].y + q[n].z * kk[b][n].z + q[n].w * kk[b][n].w;
#pragma unroll
      for (int off = LPT / 2; off >= 1; off >>= 1) s += __shfl_xor(s, off);
      s = k0 + b < nkeys ? s * scale : -INFINITY;
      const float mn = fmaxf(m, s);
      const float keep = fast_exp(m - mn);  // exp(-inf) = 0 for the first key
      const float w = fast_exp(s - mn);     // and for a key past the end
      den = den * keep + w;
#pragma unroll
      for (int n = 0; n < NP; ++n) {
        acc[n].x = acc[n].x * keep + w * v[b][n].x;
        acc[n].y = acc[n].y * keep + w * v[b][n].y;
        acc[n].z = acc[n].z * keep + w * v[b][n].z;
        acc[n].w = acc[n].w * keep + w * v[b][n].w;
      }
      m = mn;
    }
  }
  if (!live) return;
  const float inv = __builtin_amdgcn_rcpf(den);
#pragma unroll
  for (int n = 0; n < NP; ++n) {
    const int pc = sub + LPT * n;
    if (pc < D4)
      __builtin_nontemporal_store(v4f{acc[n].x * inv, acc[n].y * inv, acc[n].z * inv, acc[n].w * inv},
                                  reinterpret_cast<v4f*>(O + (size_t)tok * D + 4 * pc));   // streaming store: written once, not read again
  }
}

template <int LPT, int NP, int WAVES>
static int launch_windowed_of(const float* Q, const float* K, const float* V, const int* extra, float* O, long long G, int S,
                              int D, int window, int dilation, int R, float scale, hipStream_t s) {
  const long long per_block = WAVES * (64 / LPT);
  const long long bps = (S + per_block - 1) / per_block;  // workgroups per sequence
  const long long blocks = (G + 7) / 8 * 8 * bps;          // whole rounds of eight sequences
  if (blocks > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_windowed_attn_f32: %lld workgroups", blocks);
  // stage the window rows in LDS where the tokens of a workgroup share enough of them: at least eight tokens, a
  // span that is not much longer than they are, and room for it
  const long long rows = per_block + (long long)(window - 1) * dilation / 2 * 2;
  const long long lds = 2 * rows * D * (long long)sizeof(float);
  if (per_block >= 8 && window > 1 && rows <= 4 * per_block && lds <= 64 * 1024) {
    hipLaunchKernelGGL((windowed_attn_kernel<LPT, NP, true, WAVES>), dim3((unsigned)blocks), dim3(64 * WAVES), (size_t)lds, s, Q, K, V,
                       extra, O, G, S, D, window, dilation, R, scale);
  } else {
    hipLaunchKernelGGL((windowed_attn_kernel<LPT, NP, false, WAVES>), dim3((unsigned)blocks), dim3(64 * WAVES), 0, s, Q, K, V, extra,
                       O, G, S, D, window, dilation, R, scale);
  }
  return FTK_OK;
}

// Four waves per workgroup: sixteen (four times the tokens behind one halo of staged rows) measured slower.
template <int LPT, int NP>
static int launch_windowed(const float* Q, const float* K, const float* V, const int* extra, float* O, long long G, int S,
                           int D, int window, int dilation, int R, float scale, hipStream_t s) {
  return launch_windowed_of<LPT, NP, 4>(Q, K, V, extra, O, G, S, D, window, dilation, R, scale, s);
}

}  // namespace ftk

extern "C" int ftk_windowed_attn_f32(const float* Q, const float* K, const float* V, const int* extra_idx, float* O, int G,
                                     int S, int D, int window, int dilation, int R, float scale, ftk_stream_t stream) {
  using namespace ftk;
  if (!Q || !K || !V || !O) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_windowed_attn_f32: Q, K, V and O must be non-NULL");
  if (G <= 0 || S <= 0 || D <= 0 || window <= 0 || dilation <= 0 || R < 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_windowed_attn_f32: G, S, D, window and dilation must be positive, R non-negative");
  if ((R > 0) != (extra_idx != nullptr))
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_windowed_attn_f32: extra_idx goes with R > 0");
  if (window % 2 == 0) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_windowed_attn_f32: the window size must be odd (got %d)", window);
  if (D % 4 != 0 || D > 1024) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_windowed_attn_f32: D must be a multiple of 4, at most 1024 (got %d)", D);
  if ((long long)(window - 1) * dilation / 2 >= S)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_windowed_attn_f32: half the window span (%lld) must be below S = %d",
                (long long)(window - 1) * dilation / 2, S);
  if ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(O)) % 16 != 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_windowed_attn_f32: Q, K, V and O must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int D4 = D / 4;
  int rc;
#define FTK_WA(LPT, NP) launch_windowed<LPT, NP>(Q, K, V, extra_idx, O, G, S, D, window, dilation, R, scale, s)
  if (D4 <= 4) rc = FTK_WA(4, 1);
  else if (D4 <= 8) rc = FTK_WA(8, 1);
  else if (D4 <= 16) rc = FTK_WA(16, 1);
  else if (D4 <= 32) rc = FTK_WA(32, 1);
  else if (D4 <= 64) rc = FTK_WA(64, 1);
  else if (D4 <= 128) rc = FTK_WA(64, 2);
  else rc = FTK_WA(64, 4);
#undef FTK_WA
  if (rc) return rc;
  return check_launch("windowed_attn_kernel");
}
