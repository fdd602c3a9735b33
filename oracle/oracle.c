/*
 * Plain-C restatement of the FractalTensor hot-path algorithms (CPU oracle).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is compiled into oracle/liboracle.so
 * and loaded by tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py.  The shipped library never links or calls it.
 *
 * Single-threaded, straightforward loops; every function cites the reference
 * file:line whose algorithm it follows.  The numpy module next to this file
 * states the same algorithms and the two are checked against each other and
 * against closed forms in tests/test_oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* round-to-nearest-even float -> half */
static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
  if (x < 0x33000001u) return (uint16_t)sign;              /* underflow -> 0 */
  int e = (int)(x >> 23) - 127;
  uint32_t m = (x & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
    m &= 0x7fffffu;
  }
  uint32_t half_m = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  uint32_t out = (hexp << 10) + half_m;
  if (rem > halfway || (rem == halfway && (out & 1u))) ++out;
  return (uint16_t)(sign | out);
}

float orc_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t orc_float_to_half(float f) { return float_to_half(f); }

/* ------------------------------------------------------------------ LSTM */

static float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

/*
 * One batched LSTM cell, fused gate GEMM g = [x,h_prev] @ WU + bias with
 * column blocks i|f|o|c~ ; c = f*c_prev + i*tanh(c~) ; h = o*tanh(c).
 * examples/stacked_rnn/stacked_rnn.py:13-36 in the batched form of
 * benchmarks/rnn/baselines/stacked_lstm/pt_model/rnn.py:94-108.
 * x [B,I], h_prev/c_prev [B,H] (NULL = zeros), WU [(I+H),4H], bias [4H]|NULL.
 * gates: caller scratch [B,4H].
 */
static void lstm_cell_f32(const float* x, const float* h_prev, const float* c_prev,
                          const float* WU, const float* bias, float* h, float* c,
                          float* gates, int B, int I, int H) {
  const int N = 4 * H;
  for (int b = 0; b < B; ++b) {
    float* g = gates + (size_t)b * N;
    if (bias)
      memcpy(g, bias, sizeof(float) * N);
    else
      memset(g, 0, sizeof(float) * N);
    for (int k = 0; k < I; ++k) {
      const float a = x[(size_t)b * I + k];
      const float* w = WU + (size_t)k * N;
      for (int n = 0; n < N; ++n) g[n] += a * w[n];
    }
    if (h_prev) {
      for (int k = 0; k < H; ++k) {
        const float a = h_prev[(size_t)b * H + k];
        const float* w = WU + (size_t)(I + k) * N;
        for (int n = 0; n < N; ++n) g[n] += a * w[n];
      }
    }
    for (int u = 0; u < H; ++u) {
      const float ig = sigmoidf_(g[u]);
      const float fg = sigmoidf_(g[H + u]);
      const float og = sigmoidf_(g[2 * H + u]);
      const float cand = tanhf(g[3 * H + u]);
      const float cp = c_prev ? c_prev[(size_t)b * H + u] : 0.0f;
      const float cn = fg * cp + ig * cand;
      c[(size_t)b * H + u] = cn;
      h[(size_t)b * H + u] = og * tanhf(cn);
    }
  }
}

int orc_lstm_cell_f32(const float* x, const float* h_prev, const float* c_prev,
                      const float* WU, const float* bias, float* h, float* c,
                      int B, int I, int H) {
  float* gates = (float*)malloc(sizeof(float) * (size_t)B * 4 * H);
  if (!gates) return -1;
  lstm_cell_f32(x, h_prev, c_prev, WU, bias, h, c, gates, B, I, H);
  free(gates);
  return 0;
}

/*
 * L stacked layers, layer-major; layer l reads layer l-1's hidden sequence
 * (examples/stacked_rnn/stacked_rnn.py:54-79).  dilations[l] (NULL = all 1)
 * selects the state from step t-d, zero state for t<d: the recurrence of
 * examples/dilated_rnn/dilated_rnn.py:16-27 through DilatedMap
 * (kaleido/frontend/operations/fractaltensor/functional/apply_to_each.py:83-177).
 * xs [T,B,H], WU [L,2H,4H], bias [L,4H]|NULL, hsss/csss [L,T,B,H].
 */
int orc_stacked_lstm_f32(const float* xs, const float* WU, const float* bias,
                         const int* dilations, float* hsss, float* csss, int L,
                         int T, int B, int H) {
  float* gates = (float*)malloc(sizeof(float) * (size_t)B * 4 * H);
  if (!gates) return -1;
  const size_t cell = (size_t)B * H;
  for (int l = 0; l < L; ++l) {
    const int d = dilations ? dilations[l] : 1;
    const float* w = WU + (size_t)l * 2 * H * 4 * H;
    const float* bl = bias ? bias + (size_t)l * 4 * H : NULL;
    for (int t = 0; t < T; ++t) {
      const float* x = (l == 0) ? xs + (size_t)t * cell
                                : hsss + ((size_t)(l - 1) * T + t) * cell;
      const float* hp = (t >= d) ? hsss + ((size_t)l * T + (t - d)) * cell : NULL;
      const float* cp = (t >= d) ? csss + ((size_t)l * T + (t - d)) * cell : NULL;
      lstm_cell_f32(x, hp, cp, w, bl, hsss + ((size_t)l * T + t) * cell,
                    csss + ((size_t)l * T + t) * cell, gates, B, H, H);
    }
  }
  free(gates);
  return 0;
}

/* ---------------------------------------------------------- B2B GEMM f16 */

/*
 * D = (A @ B) @ C for G independent problems, fp16 storage, fp32 accumulate.
 * Layouts of kaleido/core/operators/tests/b2b_gemm_test_utils.h:3-9: A [M,K]
 * row-major, B stored [N,K], C stored [P,N], D [M,P] row-major.  The
 * intermediate is rounded to fp16 when round_p != 0
 * (kaleido/core/device/kernels/cutlass_wmma.h:512-517).  D is returned in
 * fp32 (not rounded) so the caller can compare at either precision.
 */
int orc_b2b_gemm_f16(const uint16_t* A, const uint16_t* Bm, const uint16_t* Cm,
                     float* D, int G, int M, int N, int K, int P, int round_p) {
  float* Bf = (float*)malloc(sizeof(float) * (size_t)N * K);
  float* Cf = (float*)malloc(sizeof(float) * (size_t)P * N);
  float* a = (float*)malloc(sizeof(float) * (size_t)K);
  float* p = (float*)malloc(sizeof(float) * (size_t)N);
  if (!Bf || !Cf || !a || !p) return -1;
  for (int g = 0; g < G; ++g) {
    const uint16_t* Ag = A + (size_t)g * M * K;
    for (size_t i = 0; i < (size_t)N * K; ++i) Bf[i] = half_to_float(Bm[(size_t)g * N * K + i]);
    for (size_t i = 0; i < (size_t)P * N; ++i) Cf[i] = half_to_float(Cm[(size_t)g * P * N + i]);
    for (int m = 0; m < M; ++m) {
      for (int k = 0; k < K; ++k) a[k] = half_to_float(Ag[(size_t)m * K + k]);
      for (int n = 0; n < N; ++n) {
        const float* b = Bf + (size_t)n * K;
        float acc = 0.0f;
        for (int k = 0; k < K; ++k) acc += a[k] * b[k];
        p[n] = round_p ? half_to_float(float_to_half(acc)) : acc;
      }
      float* d = D + ((size_t)g * M + m) * P;
      for (int q = 0; q < P; ++q) {
        const float* c = Cf + (size_t)q * N;
        float acc = 0.0f;
        for (int n = 0; n < N; ++n) acc += p[n] * c[n];
        d[q] = acc;
      }
    }
  }
  free(Bf);
  free(Cf);
  free(a);
  free(p);
  return 0;
}

/* ------------------------------------------------------- flash attention */

/*
 * Blockwise non-causal attention with the running (m, l, o) state of
 * examples/flash_attention/flash_attention.py:14-60 (o kept normalised at
 * every block, exactly as attn_func does), initial state m=-inf, l=0, o=0 as
 * examples/flash_attention/README.md:35-42 requires, score scaled by `scale`.
 * Q [BH,Sq,D], K/V [BH,Skv,D] fp16; O [BH,Sq,D] fp32.
 */
int orc_flash_attn_f16(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                       float* O, int BH, int Sq, int Skv, int D, float scale,
                       int block_kv) {
  float* Kf = (float*)malloc(sizeof(float) * (size_t)Skv * D);
  float* Vf = (float*)malloc(sizeof(float) * (size_t)Skv * D);
  float* q = (float*)malloc(sizeof(float) * (size_t)D);
  float* w = (float*)malloc(sizeof(float) * (size_t)block_kv);
  float* ev = (float*)malloc(sizeof(float) * (size_t)D);
  if (!Kf || !Vf || !q || !w || !ev) return -1;
  for (int bh = 0; bh < BH; ++bh) {
    for (size_t i = 0; i < (size_t)Skv * D; ++i) {
      Kf[i] = half_to_float(K[(size_t)bh * Skv * D + i]);
      Vf[i] = half_to_float(V[(size_t)bh * Skv * D + i]);
    }
    for (int s = 0; s < Sq; ++s) {
      for (int d = 0; d < D; ++d) q[d] = half_to_float(Q[((size_t)bh * Sq + s) * D + d]);
      float* o = O + ((size_t)bh * Sq + s) * D;
      float prev_m = -INFINITY, prev_l = 0.0f;
      for (int d = 0; d < D; ++d) o[d] = 0.0f;
      for (int k0 = 0; k0 < Skv; k0 += block_kv) {
        const int nk = (Skv - k0 < block_kv) ? Skv - k0 : block_kv;
        float cur_m = -INFINITY;
        for (int j = 0; j < nk; ++j) {
          const float* kr = Kf + (size_t)(k0 + j) * D;
          float acc = 0.0f;
          for (int d = 0; d < D; ++d) acc += q[d] * kr[d];
          w[j] = acc * scale;
          if (w[j] > cur_m) cur_m = w[j];
        }
        float cur_l = 0.0f;
        for (int d = 0; d < D; ++d) ev[d] = 0.0f;
        for (int j = 0; j < nk; ++j) {
          const float e = expf(w[j] - cur_m);
          cur_l += e;
          const float* vr = Vf + (size_t)(k0 + j) * D;
          for (int d = 0; d < D; ++d) ev[d] += e * vr[d];
        }
        const float new_m = cur_m > prev_m ? cur_m : prev_m;
        const float r_prev = expf(prev_m - new_m);
        const float r_cur = expf(cur_m - new_m);
        const float new_l = r_prev * prev_l + r_cur * cur_l;
        for (int d = 0; d < D; ++d)
          o[d] = (o[d] * prev_l * r_prev + r_cur * ev[d]) / new_l;
        prev_m = new_m;
        prev_l = new_l;
      }
    }
  }
  free(Kf);
  free(Vf);
  free(q);
  free(w);
  free(ev);
  return 0;
}

/* -------------------------------------------------------- online softmax */

/*
 * Row softmax through a running (m, d) pair, y = exp(x-m)/d.  The running
 * update is the corrected form of kaleido/core/device/kernels/online_softmax.h
 * :121-128 (m' = max(m,x); d' = d*exp(m-m') + exp(x-m')); the final map is
 * :149-155 including its clamp of x-m at -64.
 */
int orc_online_softmax_f32(const float* x, float* y, int rows, int cols) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (size_t)r * cols;
    float* yr = y + (size_t)r * cols;
    float m = -INFINITY, d = 0.0f;
    for (int j = 0; j < cols; ++j) {
      const float mn = xr[j] > m ? xr[j] : m;
      d = d * expf(m - mn) + expf(xr[j] - mn);
      m = mn;
    }
    for (int j = 0; j < cols; ++j) {
      float v = xr[j] - m;
      if (v < -64.0f) v = -64.0f;
      yr[j] = expf(v) / d;
    }
  }
  return 0;
}
