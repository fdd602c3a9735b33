// Persistent stacked / dilated LSTM for H = 256 on gfx950.
//
// One launch evaluates every (layer, time) cell.  The grid is one 256-thread
// workgroup per compute unit; a fixed group of workgroups owns each layer for
// the whole launch and keeps its slice of that layer's [W;U] (512 x 1024
// fp32) in registers: a workgroup holds 128 gate columns (32 hidden units x
// {i,f,o,c~}), each of its four waves 32 of them as 256 VGPRs per lane, the
// MFMA "A" operands of v_mfma_f32_32x32x2_f32.  Eight such column slices make
// a layer; with spare compute units a layer gets several row slices as well,
// each handling its own subset of the batch's 32-row blocks.
//
// Work item = (t, row block).  For an item the workgroup stages the activation
// tile [32, 512] = [x_t | h_{t-d}] in LDS, runs the K = 512 product against
// the resident weights, applies bias, sigmoid/tanh and the state update in
// registers (all four gates of a (row, unit) pair land in one lane, see
// lstm_cell.hip) and writes h, c.  Batch rows never interact, so dependencies
// are per row block: item (l, t, rb) needs h[l-1][t][rb] from the layer below
// and h[l][t-d][rb] from all eight column slices of its own layer.  Layer l
// therefore trails layer l-1 by an item or two: the wavefront of the
// reference's region schedule, without launches, device syncs or scatter.
//
// Hand-off between compute units (which may sit on different XCDs, whose L2
// caches are not coherent with each other) uses no cache-wide fences: h is
// written with agent-scope write-through stores and read with agent-scope
// loads, the producer waits for its stores to be acknowledged, then one thread
// per workgroup increments flags[l][t][rb]; consumers poll that count with
// agent-scope loads until it reaches 8.  c is only ever re-read by the
// workgroup that wrote it and goes through the cache normally.
//
// The activation tile is double buffered: while item n is on the matrix cores
// the next item's tile is already in flight into registers (if its producers
// are done; otherwise the wave waits for them after its own MFMAs).  One
// workgroup barrier per item.
//
// All workgroups must be co-resident: the host launches cooperatively with at
// most one workgroup per compute unit (each uses the whole register file of
// its CU).  Every wait is bounded by spin_limit polls; on expiry the kernel
// records an error word and every workgroup drains.
#include <stdlib.h>

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
  int serial;      // 1: some workgroup's next item depends on its current one (no prefetch)
  int spin_limit;
  int trace_q;            // logical workgroup whose item timeline is recorded, or -1
  long long* trace;       // [items][5] 100 MHz clock stamps of that workgroup
  int dil[kMaxLayers];
};

typedef unsigned long long u64;

__device__ __forceinline__ int flag_load(const int* flag) {
  return __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Bounded wait until *flag >= target.  Every lane polls the same word, so the
// result is wave-uniform.
__device__ __forceinline__ bool wait_count(const int* flag, int target, int* status, int spin_limit) {
  int n = 0;
  while (flag_load(flag) < target) {
    __builtin_amdgcn_s_sleep(1);
    if (++n >= spin_limit) {
      __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    if ((n & 1023) == 0 && flag_load(status) != 0) return false;
  }
  return true;
}

// 8-byte agent-scope accesses: they bypass whatever a non-coherent cache level
// may hold, with no ordering side effects of their own.
__device__ __forceinline__ u64 coherent_load8(const float* p) {
  return __hip_atomic_load(reinterpret_cast<const u64*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coherent_store8(float* p, float a, float b) {
  u64 v = (u64)__float_as_uint(a) | ((u64)__float_as_uint(b) << 32);
  __hip_atomic_store(reinterpret_cast<u64*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

constexpr int P_TILE = 32 * P_LD;  // floats per LDS buffer
constexpr int P_PF = 32;           // 8-byte prefetch registers per thread (8 rows x 512 floats per wave)

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void lstm_persistent_kernel(PersistArgs a) {
  extern __shared__ __attribute__((aligned(16))) float tile[];  // [2][32][P_LD]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;

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
  const int my_rbs = (a.nrb - prs + a.pr - 1) / a.pr;  // row blocks this workgroup walks per time step
  const int n_items = T * my_rbs;

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

  // Staging: wave w moves rows 8w..8w+7 of the tile; a row is 256 floats of x
  // and 256 of h_prev, 128 eight-byte pieces each; lane handles pieces
  // lane and lane+64 of either half.
  u64 pf[P_PF];
  bool alive = true;

  auto item_t = [&](int n) { return n / my_rbs; };
  auto item_rb = [&](int n) { return prs + a.pr * (n % my_rbs); };

  // inputs of item n complete?  (blocking: bounded spin; otherwise one poll)
  auto deps_ready = [&](int n, bool blocking) __attribute__((always_inline)) -> bool {
    const int t = item_t(n), rb = item_rb(n);
    bool ok = true;
    if (l > 0) {
      const int* f = a.flags + ((size_t)(l - 1) * T + t) * a.nrb + rb;
      ok = blocking ? wait_count(f, PC, a.status, a.spin_limit) : (flag_load(f) >= PC);
    }
    if (ok && t >= d) {
      const int* f = a.flags + ((size_t)l * T + (t - d)) * a.nrb + rb;
      ok = blocking ? wait_count(f, PC, a.status, a.spin_limit) : (flag_load(f) >= PC);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // data loads stay behind the flag reads
    return ok;
  };
  auto issue_loads = [&](int n) __attribute__((always_inline)) {
    const int t = item_t(n), rb = item_rb(n);
    const float* xsrc = (l == 0) ? a.xs + (size_t)t * cell : a.hsss + ((size_t)(l - 1) * T + t) * cell;
    const bool has_prev = t >= d;
    const float* hsrc = a.hsss + ((size_t)l * T + (has_prev ? t - d : 0)) * cell;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int rg = min(rb * 32 + 8 * wave + r, B - 1);
      pf[4 * r + 0] = coherent_load8(xsrc + (size_t)rg * PH + 2 * lane);
      pf[4 * r + 1] = coherent_load8(xsrc + (size_t)rg * PH + 128 + 2 * lane);
      if (has_prev) {
        pf[4 * r + 2] = coherent_load8(hsrc + (size_t)rg * PH + 2 * lane);
        pf[4 * r + 3] = coherent_load8(hsrc + (size_t)rg * PH + 128 + 2 * lane);
      }
    }
  };
  auto write_tile = [&](int n, int buf) __attribute__((always_inline)) {
    const bool has_prev = item_t(n) >= d;
    float* dst = tile + buf * P_TILE + (8 * wave) * P_LD + 2 * lane;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      *reinterpret_cast<u64*>(dst + r * P_LD) = pf[4 * r + 0];
      *reinterpret_cast<u64*>(dst + r * P_LD + 128) = pf[4 * r + 1];
      if (has_prev) {
        *reinterpret_cast<u64*>(dst + r * P_LD + 256) = pf[4 * r + 2];
        *reinterpret_cast<u64*>(dst + r * P_LD + 384) = pf[4 * r + 3];
      }
    }
  };

  // prologue: first tile
  alive = deps_ready(0, true);
  if (alive) issue_loads(0);
  if (alive) write_tile(0, 0);
  __syncthreads();

  const bool tracing = (q == a.trace_q) && tid == 0;
  for (int n = 0; n < n_items; ++n) {
    const int buf = n & 1;
    if (tracing) a.trace[5 * n + 0] = wall_clock64();
    const int t = item_t(n), rb = item_rb(n);
    const bool has_prev = t >= d;
    const bool more = n + 1 < n_items;
    float* hdst = a.hsss + ((size_t)l * T + t) * cell;
    float* cdst = a.csss + ((size_t)l * T + t) * cell;
    const int rg = rb * 32 + j;
    const int rgc = min(rg, B - 1);

    float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
    if (alive && has_prev)
      cp = *reinterpret_cast<const float4*>(a.csss + ((size_t)l * T + (t - d)) * cell + (size_t)rgc * PH + u0);

    // the next item's flags are requested now and looked at half way through
    // the item, so their round trip to memory is off the critical path
    int f_below = PC, f_own = PC;
    if (more && !a.serial) {
      const int t1 = item_t(n + 1), rb1 = item_rb(n + 1);
      if (l > 0) f_below = flag_load(a.flags + ((size_t)(l - 1) * T + t1) * a.nrb + rb1);
      if (t1 >= d) f_own = flag_load(a.flags + ((size_t)l * T + (t1 - d)) * a.nrb + rb1);
    }

    // ---- gates^T = WU^T * act^T on the matrix cores; two accumulators so
    // that consecutive MFMAs never wait on each other's result
    v16f acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
    const float* arow = tile + buf * P_TILE + j * P_LD + 4 * hh;
#pragma unroll
    for (int qq = 0; qq < PH / 8; ++qq) {
      const v4f b = *reinterpret_cast<const v4f*>(arow + 8 * qq);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b[0], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b[1], acc1, 0, 0, 0);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 2], b[2], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 3], b[3], acc1, 0, 0, 0);
    }
    if (tracing) a.trace[5 * n + 1] = wall_clock64();

    // Half way through the item, fetch the next tile: wait (bounded) for its
    // producers, then put its loads in flight behind the rest of the MFMAs.
    // Waiting here rather than at the end of the item makes each layer settle
    // about one and a half items behind the layer below, which is what lets
    // the loads overlap the arithmetic in steady state.
    if (alive && more && !a.serial) {
      if (f_below < PC || f_own < PC) alive = deps_ready(n + 1, true);
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      if (alive) issue_loads(n + 1);
    }

    if (has_prev) {
#pragma unroll
      for (int qq = PH / 8; qq < PK / 8; ++qq) {
        const v4f b = *reinterpret_cast<const v4f*>(arow + 8 * qq);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b[0], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b[1], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 2], b[2], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 3], b[3], acc1, 0, 0, 0);
      }
    }
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = acc0[r] + acc1[r];

    // ---- state update, lane-local; h leaves through write-through stores
    if (alive && rg < B) {
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
      *reinterpret_cast<float4*>(cdst + (size_t)rg * PH + u0) = make_float4(cv[0], cv[1], cv[2], cv[3]);
      coherent_store8(hdst + (size_t)rg * PH + u0, hv[0], hv[1]);
      coherent_store8(hdst + (size_t)rg * PH + u0 + 2, hv[2], hv[3]);
    }

    if (tracing) a.trace[5 * n + 2] = wall_clock64();
    if (!a.serial) {
      if (alive && more) write_tile(n + 1, buf ^ 1);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0);  // this wave's h stores are acknowledged
      if (tracing) a.trace[5 * n + 3] = wall_clock64();
      __syncthreads();
      if (tracing) a.trace[5 * n + 4] = wall_clock64();
      if (tid == 0 && alive)
        __hip_atomic_fetch_add(a.flags + ((size_t)l * T + t) * a.nrb + rb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      // the next item needs this one: publish first, then fetch
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (tid == 0 && alive)
        __hip_atomic_fetch_add(a.flags + ((size_t)l * T + t) * a.nrb + rb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (alive && more) {
        alive = deps_ready(n + 1, true);
        if (alive) issue_loads(n + 1);
        if (alive) write_tile(n + 1, buf ^ 1);
      }
      __syncthreads();
    }
  }
}

__global__ void fill_zero_kernel(int* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

static size_t flag_count(int L, int T, int B) {
  const int nrb = (B + 31) / 32;
  return (size_t)L * T * nrb;
}

// Workspace layout: [64 ints: status][flags][trace: T*nrb*5 stamps of 8 bytes].
static size_t trace_offset_bytes(int L, int T, int B) { return ((flag_count(L, T, B) + 64) * sizeof(int) + 15) / 16 * 16; }
static size_t workspace_need(int L, int T, int B) {
  return trace_offset_bytes(L, T, B) + (size_t)T * ((B + 31) / 32) * 5 * sizeof(long long);
}

// Tuning hook: FTK_LSTM_TRACE=<logical workgroup> records that workgroup's per-item timeline.
static int trace_workgroup() {
  static int v = -2;
  if (v == -2) {
    const char* e = getenv("FTK_LSTM_TRACE");
    v = e ? atoi(e) : -1;
  }
  return v;
}

static int run_persistent(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss,
                          float* csss, int L, int T, int B, void* ws, size_t ws_bytes, hipStream_t s,
                          bool* handled) {
  *handled = false;
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  const size_t lds = (size_t)2 * P_TILE * sizeof(float);
  if ((int)lds > dp->lds_optin) return FTK_OK;
  const void* fn = (const void*)lstm_persistent_kernel;
  static bool attr_set = false;
  if (!attr_set) {
    FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  int per_cu = 0;
  FTK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 256, lds));
  const int slots = per_cu * dp->cus;
  if (L > kMaxLayers || L * PC > slots) return FTK_OK;  // cannot pin every layer on its own compute units: fall back

  const size_t nflags = flag_count(L, T, B);
  const size_t need = workspace_need(L, T, B);
  if (!ws || ws_bytes < need)
    return fail(FTK_ERR_WORKSPACE, "stacked LSTM needs a %zu-byte workspace, got %zu", need, ws_bytes);

  PersistArgs a;
  a.xs = xs; a.WU = WU; a.bias = bias; a.hsss = hsss; a.csss = csss;
  a.status = reinterpret_cast<int*>(ws);
  a.flags = a.status + 64;
  a.L = L; a.T = T; a.B = B;
  a.nrb = (B + 31) / 32;
  // spare compute units become row slices, but a workgroup keeps at least two
  // row blocks when it can so that the next tile never depends on the current item
  a.pr = std::max(1, std::min(slots / (L * PC), std::max(1, a.nrb / 2)));
  a.groups = L * PC * a.pr;
  a.spin_limit = 1 << 22;
  a.trace_q = trace_workgroup();
  a.trace = reinterpret_cast<long long*>(reinterpret_cast<char*>(ws) + trace_offset_bytes(L, T, B));
  const int min_rbs = a.nrb / a.pr;
  a.serial = 0;
  for (int l = 0; l < kMaxLayers; ++l) {
    a.dil[l] = (l < L && dil) ? dil[l] : 1;
    if (l < L && (long long)a.dil[l] * min_rbs < 2) a.serial = 1;
  }
  const int grid = a.groups;
  a.xcd_remap = (grid % 8 == 0) ? 1 : 0;

  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, a.status, nflags + 64);
  rc = check_launch("fill_zero_kernel");
  if (rc) return rc;

  void* kargs[] = {&a};
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
  return ftk::workspace_need(L, T, B);
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
