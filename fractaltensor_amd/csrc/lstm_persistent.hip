// Persistent stacked / dilated LSTM for H = 256 on gfx950.
//
// One launch evaluates every (layer, time) cell.  The grid is one 256-thread
// workgroup per compute unit; a fixed group of workgroups owns each layer for
// the whole launch and keeps its slice of that layer's [W;U] (512 x 1024
// fp32) in registers: a workgroup holds 128 gate columns (32 hidden units x
// {i,f,o,c~}), each of its four waves 32 of them as 256 VGPRs per lane, the
// MFMA "A" operands of v_mfma_f32_32x32x2_f32.  Eight such column slices make
// a layer; with spare compute units a layer gets several row slices as well,
// each handling its own subset of the batch's row blocks.
//
// Work item = (t, row block).  For an item the workgroup stages the activation
// tile [rows, 512] = [x_t | h_{t-d}] in LDS, runs the K = 512 product against
// the resident weights, applies bias, sigmoid/tanh and the state update in
// registers (all four gates of a (row, unit) pair land in one lane, see
// lstm_cell.hip) and writes h, c.  Batch rows never interact, so dependencies
// are per row block: item (l, t, rb) needs h[l-1][t][rb] from the layer below
// and h[l][t-d][rb] from all eight column slices of its own layer.  Producers
// publish a row block with a release fence and an atomic increment of
// flags[l][t][rb]; consumers spin (bounded) until the count reaches 8.
// Layer l therefore trails layer l-1 by one item: the wavefront of the
// reference's region schedule, without launches, device syncs or scatter.
//
// All workgroups must be co-resident: the host launches cooperatively with
// one workgroup per compute unit (each uses the whole register file of its
// CU).  Every wait is bounded by spin_limit polls; on expiry the kernel
// records an error word and every workgroup drains.
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

int run_wavefront(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss, float* csss,
                  int L, int T, int B, int H, hipStream_t s);

constexpr int PH = 256;            // hidden size this kernel is specialised for
constexpr int PK = 2 * PH;         // K of the gate GEMM
constexpr int PN = 4 * PH;         // gate columns
constexpr int P_LD = PK + 4;       // padded activation row in LDS (floats)
constexpr int PC = 8;              // column slices per layer (32 units each)
constexpr int kMaxLayers = 64;

struct PersistArgs {
  const float* xs;
  const float* WU;
  const float* bias;
  float* hsss;
  float* csss;
  int* flags;   // [L][T][NRB] completion counts
  int* status;  // [0] = error word
  int L, T, B;
  int nrb;         // row blocks of 32*RT rows
  int pr;          // row slices per layer
  int groups;      // workgroups that take part (= L * PC * pr)
  int xcd_remap;   // 1: grid is a multiple of 8, map workgroups so a layer shares an XCD
  int spin_limit;
  int dil[kMaxLayers];
};

__device__ __forceinline__ bool wait_count(int* flag, int target, int* status, int spin_limit) {
  int n = 0;
  while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
    __builtin_amdgcn_s_sleep(1);
    if (++n >= spin_limit) {
      __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    if ((n & 1023) == 0 && __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return false;
  }
  return true;
}

template <int RT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void lstm_persistent_kernel(PersistArgs a) {
  extern __shared__ __attribute__((aligned(16))) float tile[];  // [32*RT][P_LD]
  __shared__ int ok_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  constexpr int ROWS = 32 * RT;

  int q = blockIdx.x;
  if (a.xcd_remap) q = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (q >= a.groups) return;
  const int per_layer = PC * a.pr;
  const int l = q / per_layer;
  const int within = q - l * per_layer;
  const int pc = within % PC;
  const int prs = within / PC;
  const int d = a.dil[l];
  const int T = a.T, B = a.B;
  const size_t cell = (size_t)B * PH;

  // Resident weights: lane (i = j, half hh) of wave w holds, for MFMA step
  // s = 4q + c, WU[l][k = 8q + 4hh + c][gate(i)*H + 32pc + 8w + i%8].
  const int col = (j >> 3) * PH + 32 * pc + 8 * wave + (j & 7);
  const float* wl = a.WU + (size_t)l * PK * PN + col;
  float wr[PK / 2];
#pragma unroll
  for (int s = 0; s < PK / 2; ++s) {
    const int k = 8 * (s >> 2) + 4 * hh + (s & 3);
    wr[s] = wl[(size_t)k * PN];
  }
  const int u0 = 32 * pc + 8 * wave + 4 * hh;  // first of this lane's 4 units
  float bi[4] = {0, 0, 0, 0}, bf[4] = {0, 0, 0, 0}, bo[4] = {0, 0, 0, 0}, bg[4] = {0, 0, 0, 0};
  if (a.bias) {
    const float* bl = a.bias + (size_t)l * PN;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      bi[r] = bl[u0 + r];
      bf[r] = bl[PH + u0 + r];
      bo[r] = bl[2 * PH + u0 + r];
      bg[r] = bl[3 * PH + u0 + r];
    }
  }

  const int ld_c4 = tid & 63;   // float4 column within a 256-float half row
  const int ld_r0 = tid >> 6;   // first row this thread stages

  for (int t = 0; t < T; ++t) {
    const bool has_prev = t >= d;
    const float* xsrc = (l == 0) ? a.xs + (size_t)t * cell : a.hsss + ((size_t)(l - 1) * T + t) * cell;
    const float* hsrc = has_prev ? a.hsss + ((size_t)l * T + (t - d)) * cell : nullptr;
    const float* csrc = has_prev ? a.csss + ((size_t)l * T + (t - d)) * cell : nullptr;
    float* hdst = a.hsss + ((size_t)l * T + t) * cell;
    float* cdst = a.csss + ((size_t)l * T + t) * cell;

    for (int rb = prs; rb < a.nrb; rb += a.pr) {
      // ---- wait for the producers of this item's inputs
      if (tid == 0) {
        bool ok = true;
        if (l > 0) ok = wait_count(a.flags + ((size_t)(l - 1) * T + t) * a.nrb + rb, PC, a.status, a.spin_limit);
        if (ok && has_prev) ok = wait_count(a.flags + ((size_t)l * T + (t - d)) * a.nrb + rb, PC, a.status, a.spin_limit);
        ok_s = ok ? 1 : 0;
      }
      __syncthreads();  // also: every wave is done reading the previous tile
      if (!ok_s) return;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

      // ---- stage [x | h_prev] rows into LDS
      const int row0 = rb * ROWS;
#pragma unroll 4
      for (int r = ld_r0; r < ROWS; r += 4) {
        const int rg = min(row0 + r, B - 1);
        const float4 xv = *reinterpret_cast<const float4*>(xsrc + (size_t)rg * PH + 4 * ld_c4);
        *reinterpret_cast<float4*>(&tile[r * P_LD + 4 * ld_c4]) = xv;
        if (has_prev) {
          const float4 hv = *reinterpret_cast<const float4*>(hsrc + (size_t)rg * PH + 4 * ld_c4);
          *reinterpret_cast<float4*>(&tile[r * P_LD + PH + 4 * ld_c4]) = hv;
        }
      }
      __syncthreads();

      // ---- gates^T = WU^T * act^T on the matrix cores
      v16f acc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rt][r] = 0.0f;

      const float* arow = &tile[j * P_LD + 4 * hh];
#pragma unroll
      for (int qq = 0; qq < PH / 8; ++qq) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const float4 b = *reinterpret_cast<const float4*>(arow + rt * 32 * P_LD + 8 * qq);
          acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b.x, acc[rt], 0, 0, 0);
          acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b.y, acc[rt], 0, 0, 0);
          acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 2], b.z, acc[rt], 0, 0, 0);
          acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 3], b.w, acc[rt], 0, 0, 0);
        }
      }
      if (has_prev) {
#pragma unroll
        for (int qq = PH / 8; qq < PK / 8; ++qq) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            const float4 b = *reinterpret_cast<const float4*>(arow + rt * 32 * P_LD + 8 * qq);
            acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b.x, acc[rt], 0, 0, 0);
            acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b.y, acc[rt], 0, 0, 0);
            acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 2], b.z, acc[rt], 0, 0, 0);
            acc[rt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 3], b.w, acc[rt], 0, 0, 0);
          }
        }
      }

      // ---- state update, lane-local
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int rg = row0 + 32 * rt + j;
        if (rg < B) {
          float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
          if (has_prev) cp = *reinterpret_cast<const float4*>(csrc + (size_t)rg * PH + u0);
          const float cpv[4] = {cp.x, cp.y, cp.z, cp.w};
          float hv[4], cv[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float ig = sigmoid_f(acc[rt][r] + bi[r]);
            const float fg = sigmoid_f(acc[rt][4 + r] + bf[r]);
            const float og = sigmoid_f(acc[rt][8 + r] + bo[r]);
            const float cand = tanh_f(acc[rt][12 + r] + bg[r]);
            cv[r] = fg * cpv[r] + ig * cand;
            hv[r] = og * tanh_f(cv[r]);
          }
          *reinterpret_cast<float4*>(cdst + (size_t)rg * PH + u0) = make_float4(cv[0], cv[1], cv[2], cv[3]);
          *reinterpret_cast<float4*>(hdst + (size_t)rg * PH + u0) = make_float4(hv[0], hv[1], hv[2], hv[3]);
        }
      }

      // ---- publish: every thread's stores first, then one count per workgroup
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      __syncthreads();
      if (tid == 0)
        __hip_atomic_fetch_add(a.flags + ((size_t)l * T + t) * a.nrb + rb, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

__global__ void fill_zero_kernel(int* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

// Rows per item: 64 halves the per-item synchronisation cost, 32 gives a finer
// pipeline (shorter fill) and double the items to spread over row slices.
static int pick_rt(int B) { return B >= 64 ? 2 : 1; }

static size_t flag_count(int L, int T, int B) {
  const int rt = pick_rt(B);
  const int nrb = (B + 32 * rt - 1) / (32 * rt);
  return (size_t)L * T * nrb;
}

static int run_persistent(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss,
                          float* csss, int L, int T, int B, void* ws, size_t ws_bytes, hipStream_t s,
                          bool* handled) {
  *handled = false;
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  const int slots = dp->cus;
  if (L > kMaxLayers || L * PC > slots) return FTK_OK;  // not enough compute units to pin every layer: fall back
  const int rt = pick_rt(B);
  const size_t lds = (size_t)32 * rt * P_LD * sizeof(float);
  if ((int)lds > dp->lds_optin) return FTK_OK;

  const size_t nflags = flag_count(L, T, B);
  const size_t need = (nflags + 64) * sizeof(int);
  if (!ws || ws_bytes < need)
    return fail(FTK_ERR_WORKSPACE, "stacked LSTM needs a %zu-byte workspace, got %zu", need, ws_bytes);

  PersistArgs a;
  a.xs = xs; a.WU = WU; a.bias = bias; a.hsss = hsss; a.csss = csss;
  a.status = reinterpret_cast<int*>(ws);
  a.flags = a.status + 64;
  a.L = L; a.T = T; a.B = B;
  a.nrb = (B + 32 * rt - 1) / (32 * rt);
  a.pr = std::max(1, std::min(slots / (L * PC), a.nrb));
  a.groups = L * PC * a.pr;
  a.spin_limit = 1 << 22;
  for (int l = 0; l < kMaxLayers; ++l) a.dil[l] = (l < L && dil) ? dil[l] : 1;
  int grid = a.groups;
  a.xcd_remap = 0;
  if (grid % 8 == 0) a.xcd_remap = 1;

  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, a.status, nflags + 64);
  rc = check_launch("fill_zero_kernel");
  if (rc) return rc;

  void* kargs[] = {&a};
  const void* fn = rt == 2 ? (const void*)lstm_persistent_kernel<2> : (const void*)lstm_persistent_kernel<1>;
  FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  FTK_HIP(hipLaunchCooperativeKernel(fn, dim3(grid), dim3(256), kargs, (unsigned)lds, s));
  *handled = true;
  return FTK_OK;
}

static int check_stack_args(const char* who, const float* xs, const float* WU, float* hsss, float* csss, int L, int T,
                            int B, int H, const int* dil) {
  if (!xs || !WU || !hsss || !csss) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: xs, WU, hsss, csss must be non-NULL", who);
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: L, T, B, H must be positive", who);
  if (H % 32) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: H=%d must be a multiple of 32", who, H);
  if (dil)
    for (int l = 0; l < L; ++l)
      if (dil[l] <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: dilations[%d]=%d must be positive", who, l, dil[l]);
  return FTK_OK;
}

static int run_stack(const char* who, const float* xs, const float* WU, const float* bias, const int* dil,
                     float* hsss, float* csss, int L, int T, int B, int H, void* ws, size_t ws_bytes,
                     hipStream_t s) {
  int rc = check_stack_args(who, xs, WU, hsss, csss, L, T, B, H, dil);
  if (rc) return rc;
  if (H == PH) {
    bool handled = false;
    rc = run_persistent(xs, WU, bias, dil, hsss, csss, L, T, B, ws, ws_bytes, s, &handled);
    if (rc || handled) return rc;
  }
  return run_wavefront(xs, WU, bias, dil, hsss, csss, L, T, B, H, s);
}

}  // namespace ftk

extern "C" {

size_t ftk_stacked_lstm_workspace_bytes(int L, int T, int B, int H) {
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0) return 0;
  return (ftk::flag_count(L, T, B) + 64) * sizeof(int);
}

int ftk_stacked_lstm_f32(const float* xs, const float* WU, const float* bias, float* hsss, float* csss, int L, int T,
                         int B, int H, void* workspace, size_t workspace_bytes, ftk_stream_t stream) {
  return ftk::run_stack("ftk_stacked_lstm_f32", xs, WU, bias, nullptr, hsss, csss, L, T, B, H, workspace,
                        workspace_bytes, (hipStream_t)stream);
}

int ftk_dilated_lstm_f32(const float* xs, const float* WU, const float* bias, const int* dilations, float* hsss,
                         float* csss, int L, int T, int B, int H, void* workspace, size_t workspace_bytes,
                         ftk_stream_t stream) {
  if (!dilations) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_dilated_lstm_f32: dilations is NULL");
  return ftk::run_stack("ftk_dilated_lstm_f32", xs, WU, bias, dilations, hsss, csss, L, T, B, H, workspace,
                        workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
