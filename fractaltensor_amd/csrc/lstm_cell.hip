// Fused fp32 LSTM cell for gfx950: gate GEMM on v_mfma_f32_32x32x2_f32, bias,
// sigmoid/tanh and the state update in one launch, batched over a list of
// independent cells (one wavefront stage of a stacked or dilated LSTM).
//
// Tiling.  A workgroup (4 waves) owns 32 batch rows x 32 hidden units, i.e. the
// 128 gate columns {i,f,o,c~} x 32 units, so the state update never leaves the
// workgroup.  The GEMM is computed transposed, gates^T[col, row] =
// WU^T[col, k] * act^T[k, row]: the MFMA "A" operand is a weight value, the
// "B" operand an activation value, and the 32x32 accumulator of lane
// (row = lane%32, half = lane/32) holds, for that one batch row, gate
// g = reg/4 of unit 4*half + reg%4 of the wave's 8 units.  All four gates of a
// (row, unit) pair therefore sit in one lane and the epilogue is lane-local.
//
// The K loop (K = I + H, first the x rows of WU then the h rows) runs in
// chunks of 32 staged through LDS, double buffered with register prefetch.
// Within a chunk the k index is permuted so that one 16-byte LDS read feeds
// four MFMAs: step (q, c) uses k = 8q + c for lanes 0-31 and k = 8q + 4 + c
// for lanes 32-63.
#include <algorithm>
#include <vector>

#include "ftk_common.h"

namespace ftk {

constexpr int kMaxCellsPerLaunch = 40;

struct CellDesc {
  const float* x;       // [B, I]
  const float* h_prev;  // [B, H] or nullptr (zero state)
  const float* c_prev;  // [B, H] or nullptr
  const float* WU;      // [(I+H), 4H]
  const float* bias;    // [4H] or nullptr
  float* h;             // [B, H]
  float* c;             // [B, H]
};

struct CellList {
  int n;
  CellDesc cells[kMaxCellsPerLaunch];
};

constexpr int KC = 32;        // k chunk
constexpr int ACT_LD = KC + 4;  // padded row of the activation tile (floats)
constexpr int W_LD = 128 + 8;   // padded row of the weight tile (floats)

__global__ __launch_bounds__(256) void lstm_cell_kernel(CellList list, int B, int I, int H) {
  __shared__ __attribute__((aligned(16))) float act_s[2][32 * ACT_LD];
  __shared__ __attribute__((aligned(16))) float w_s[2][KC * W_LD];

  const CellDesc cd = list.cells[blockIdx.z];
  const int ub = blockIdx.x;  // block of 32 hidden units
  const int rb = blockIdx.y;  // block of 32 batch rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  const int N4 = 4 * H;

  const int nch_x = I / KC;
  const int nch = nch_x + (cd.h_prev ? H / KC : 0);

  // global -> register staging assignments
  const int a_row = tid >> 3;  // 0..31
  const int a_c4 = tid & 7;    // float4 within the 32-wide chunk
  const int a_row_g = min(rb * 32 + a_row, B - 1);

  float4 a_reg;
  float4 w_reg0, w_reg1, w_reg2, w_reg3;

  auto load_chunk = [&](int ch) __attribute__((always_inline)) {
    const float* src;
    int ld, k0;
    if (ch < nch_x) {
      src = cd.x; ld = I; k0 = ch * KC;
    } else {
      src = cd.h_prev; ld = H; k0 = (ch - nch_x) * KC;
    }
    a_reg = *reinterpret_cast<const float4*>(src + (size_t)a_row_g * ld + k0 + 4 * a_c4);
    const int kw0 = ch * KC;  // row of WU: x rows first, then h rows
    auto ldw = [&](int n) __attribute__((always_inline)) {
      const int idx = tid + 256 * n;
      const int k = idx >> 5;
      const int c4 = idx & 31;
      const int g = c4 >> 3;
      const int u4 = c4 & 7;
      return *reinterpret_cast<const float4*>(cd.WU + (size_t)(kw0 + k) * N4 + g * H + ub * 32 + 4 * u4);
    };
    w_reg0 = ldw(0); w_reg1 = ldw(1); w_reg2 = ldw(2); w_reg3 = ldw(3);
  };
  auto store_chunk = [&](int buf) __attribute__((always_inline)) {
    *reinterpret_cast<float4*>(&act_s[buf][a_row * ACT_LD + 4 * a_c4]) = a_reg;
    auto stw = [&](int n, const float4& v) __attribute__((always_inline)) {
      const int idx = tid + 256 * n;
      const int k = idx >> 5;
      const int c4 = idx & 31;
      const int g = c4 >> 3;
      const int u4 = c4 & 7;
      // LDS column order: wave-major, then gate, then unit within the wave
      const int col = 32 * (u4 >> 1) + 8 * g + 4 * (u4 & 1);
      *reinterpret_cast<float4*>(&w_s[buf][k * W_LD + col]) = v;
    };
    stw(0, w_reg0); stw(1, w_reg1); stw(2, w_reg2); stw(3, w_reg3);
  };

  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  load_chunk(0);
  store_chunk(0);
  __syncthreads();
  for (int ch = 0; ch < nch; ++ch) {
    const int buf = ch & 1;
    if (ch + 1 < nch) load_chunk(ch + 1);
    const float* arow = &act_s[buf][j * ACT_LD + 4 * hh];
    const float* wcol = &w_s[buf][(4 * hh) * W_LD + 32 * wave + j];
#pragma unroll
    for (int q = 0; q < KC / 8; ++q) {
      const float4 b = *reinterpret_cast<const float4*>(arow + 8 * q);
      const float a0 = wcol[(8 * q + 0) * W_LD];
      const float a1 = wcol[(8 * q + 1) * W_LD];
      const float a2 = wcol[(8 * q + 2) * W_LD];
      const float a3 = wcol[(8 * q + 3) * W_LD];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b.y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a2, b.z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a3, b.w, acc, 0, 0, 0);
    }
    if (ch + 1 < nch) store_chunk(buf ^ 1);
    __syncthreads();
  }

  // Epilogue: lane (row j, half hh) holds gates of units u0..u0+3 for its row.
  const int row_g = rb * 32 + j;
  const int u0 = ub * 32 + 8 * wave + 4 * hh;
  if (row_g < B) {
    float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
    if (cd.c_prev) cp = *reinterpret_cast<const float4*>(cd.c_prev + (size_t)row_g * H + u0);
    float bi[4] = {0, 0, 0, 0}, bf[4] = {0, 0, 0, 0}, bo[4] = {0, 0, 0, 0}, bg[4] = {0, 0, 0, 0};
    if (cd.bias) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        bi[r] = cd.bias[u0 + r];
        bf[r] = cd.bias[H + u0 + r];
        bo[r] = cd.bias[2 * H + u0 + r];
        bg[r] = cd.bias[3 * H + u0 + r];
      }
    }
    const float cpv[4] = {cp.x, cp.y, cp.z, cp.w};
    float hv[4], cv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float ig = sigmoid_f(acc[r] + bi[r]);
      const float fg = sigmoid_f(acc[4 + r] + bf[r]);
      const float og = sigmoid_f(acc[8 + r] + bo[r]);
      const float cand = tanh_f(acc[12 + r] + bg[r]);
      cv[r] = fg * cpv[r] + ig * cand;
      hv[r] = og * tanh_f(cv[r]);
    }
    *reinterpret_cast<float4*>(cd.c + (size_t)row_g * H + u0) = make_float4(cv[0], cv[1], cv[2], cv[3]);
    *reinterpret_cast<float4*>(cd.h + (size_t)row_g * H + u0) = make_float4(hv[0], hv[1], hv[2], hv[3]);
  }
}

// State update alone (unfused baseline): gates hold the pre-activations.
__global__ __launch_bounds__(256) void lstm_elementwise_kernel(const float* __restrict__ gates,
                                                               const float* __restrict__ bias,
                                                               const float* __restrict__ c_prev,
                                                               float* __restrict__ h, float* __restrict__ c,
                                                               int B, int H) {
  const int n4 = B * H / 4;
  for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < n4; idx += gridDim.x * blockDim.x) {
    const int e = idx * 4;
    const int b = e / H;
    const int u = e - b * H;
    const float* g = gates + (size_t)b * 4 * H + u;
    float4 gi = *reinterpret_cast<const float4*>(g);
    float4 gf = *reinterpret_cast<const float4*>(g + H);
    float4 go = *reinterpret_cast<const float4*>(g + 2 * H);
    float4 gc = *reinterpret_cast<const float4*>(g + 3 * H);
    if (bias) {
      const float4 b0 = *reinterpret_cast<const float4*>(bias + u);
      const float4 b1 = *reinterpret_cast<const float4*>(bias + H + u);
      const float4 b2 = *reinterpret_cast<const float4*>(bias + 2 * H + u);
      const float4 b3 = *reinterpret_cast<const float4*>(bias + 3 * H + u);
      gi.x += b0.x; gi.y += b0.y; gi.z += b0.z; gi.w += b0.w;
      gf.x += b1.x; gf.y += b1.y; gf.z += b1.z; gf.w += b1.w;
      go.x += b2.x; go.y += b2.y; go.z += b2.z; go.w += b2.w;
      gc.x += b3.x; gc.y += b3.y; gc.z += b3.z; gc.w += b3.w;
    }
    float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c_prev) cp = *reinterpret_cast<const float4*>(c_prev + e);
    float4 cn, hn;
    cn.x = sigmoid_f(gf.x) * cp.x + sigmoid_f(gi.x) * tanh_f(gc.x);
    cn.y = sigmoid_f(gf.y) * cp.y + sigmoid_f(gi.y) * tanh_f(gc.y);
    cn.z = sigmoid_f(gf.z) * cp.z + sigmoid_f(gi.z) * tanh_f(gc.z);
    cn.w = sigmoid_f(gf.w) * cp.w + sigmoid_f(gi.w) * tanh_f(gc.w);
    hn.x = sigmoid_f(go.x) * tanh_f(cn.x);
    hn.y = sigmoid_f(go.y) * tanh_f(cn.y);
    hn.z = sigmoid_f(go.z) * tanh_f(cn.z);
    hn.w = sigmoid_f(go.w) * tanh_f(cn.w);
    *reinterpret_cast<float4*>(c + e) = cn;
    *reinterpret_cast<float4*>(h + e) = hn;
  }
}

static int launch_cells(const CellList& list, int B, int I, int H, hipStream_t s) {
  dim3 grid(H / 32, (B + 31) / 32, list.n);
  hipLaunchKernelGGL(lstm_cell_kernel, grid, dim3(256), 0, s, list, B, I, H);
  return check_launch("lstm_cell_kernel");
}

// Host side of the per-stage schedule: stage(l,t) = 1 + max(stage(l-1,t),
// stage(l,t-d_l)); cells of equal stage are independent and go out as one
// batched launch.  For d = 1 the stages are the diagonals l + t.
int run_wavefront(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss, float* csss,
                  int L, int T, int B, int H, hipStream_t s) {
  std::vector<int> stage((size_t)L * T, 0);
  int max_stage = 0;
  for (int l = 0; l < L; ++l) {
    const int d = dil ? dil[l] : 1;
    for (int t = 0; t < T; ++t) {
      int st = 0;
      if (l > 0) st = std::max(st, stage[(size_t)(l - 1) * T + t] + 1);
      if (t >= d) st = std::max(st, stage[(size_t)l * T + t - d] + 1);
      stage[(size_t)l * T + t] = st;
      max_stage = std::max(max_stage, st);
    }
  }
  std::vector<std::vector<int>> by_stage(max_stage + 1);
  for (int l = 0; l < L; ++l)
    for (int t = 0; t < T; ++t) by_stage[stage[(size_t)l * T + t]].push_back(l * T + t);

  const size_t cell = (size_t)B * H;
  for (const auto& cells : by_stage) {
    size_t pos = 0;
    while (pos < cells.size()) {
      CellList list;
      list.n = 0;
      while (pos < cells.size() && list.n < kMaxCellsPerLaunch) {
        const int l = cells[pos] / T, t = cells[pos] % T;
        const int d = dil ? dil[l] : 1;
        CellDesc& cd = list.cells[list.n++];
        cd.x = (l == 0) ? xs + (size_t)t * cell : hsss + ((size_t)(l - 1) * T + t) * cell;
        cd.h_prev = (t >= d) ? hsss + ((size_t)l * T + t - d) * cell : nullptr;
        cd.c_prev = (t >= d) ? csss + ((size_t)l * T + t - d) * cell : nullptr;
        cd.WU = WU + (size_t)l * 2 * H * 4 * H;
        cd.bias = bias ? bias + (size_t)l * 4 * H : nullptr;
        cd.h = hsss + ((size_t)l * T + t) * cell;
        cd.c = csss + ((size_t)l * T + t) * cell;
        ++pos;
      }
      int rc = launch_cells(list, B, H, H, s);
      if (rc) return rc;
    }
  }
  return FTK_OK;
}

}  // namespace ftk

extern "C" {

int ftk_lstm_cell_f32(const float* x, const float* h_prev, const float* c_prev, const float* WU, const float* bias,
                      float* h, float* c, int B, int I, int H, ftk_stream_t stream) {
  if (!x || !WU || !h || !c) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f32: x, WU, h, c must be non-NULL");
  if ((h_prev == nullptr) != (c_prev == nullptr))
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f32: h_prev and c_prev must both be given or both be NULL");
  if (B <= 0 || I <= 0 || H <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f32: B, I, H must be positive");
  if (I % 32 || H % 32)
    return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_lstm_cell_f32: I=%d and H=%d must be multiples of 32", I, H);
  if ((B + 31) / 32 > 65535) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_lstm_cell_f32: B=%d too large", B);
  ftk::CellList list;
  list.n = 1;
  list.cells[0] = ftk::CellDesc{x, h_prev, c_prev, WU, bias, h, c};
  return ftk::launch_cells(list, B, I, H, (hipStream_t)stream);
}

int ftk_lstm_elementwise_f32(const float* gates, const float* bias, const float* c_prev, float* h, float* c, int B,
                             int H, ftk_stream_t stream) {
  if (!gates || !h || !c) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_elementwise_f32: gates, h, c must be non-NULL");
  if (B <= 0 || H <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_elementwise_f32: B, H must be positive");
  if (H % 4) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_lstm_elementwise_f32: H=%d must be a multiple of 4", H);
  const int n4 = B * H / 4;
  const int blocks = std::min((n4 + 255) / 256, 2048);
  hipLaunchKernelGGL(ftk::lstm_elementwise_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, gates, bias,
                     c_prev, h, c, B, H);
  return ftk::check_launch("lstm_elementwise_kernel");
}

int ftk_stacked_lstm_wavefront_f32(const float* xs, const float* WU, const float* bias, const int* dilations,
                                   float* hsss, float* csss, int L, int T, int B, int H, ftk_stream_t stream) {
  if (!xs || !WU || !hsss || !csss)
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_stacked_lstm_wavefront_f32: xs, WU, hsss, csss must be non-NULL");
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0)
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_stacked_lstm_wavefront_f32: L, T, B, H must be positive");
  if (H % 32) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_stacked_lstm_wavefront_f32: H=%d must be a multiple of 32", H);
  if (dilations)
    for (int l = 0; l < L; ++l)
      if (dilations[l] <= 0)
        return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_stacked_lstm_wavefront_f32: dilations[%d]=%d must be positive", l,
                         dilations[l]);
  return ftk::run_wavefront(xs, WU, bias, dilations, hsss, csss, L, T, B, H, (hipStream_t)stream);
}

}  // extern "C"
