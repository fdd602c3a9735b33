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
// loads, every producer wave waits for its own stores to be acknowledged and
// then increments flags[l][t][rb]; consumers poll that count with agent-scope
// loads until it reaches 32 (8 column slices x 4 waves).  c is only ever re-read by the
// workgroup that wrote it and goes through the cache normally.
//
// The activation tile is double buffered and the item loop is software
// pipelined: the loads of tile n+1 are issued half way through item n, and the
// activations / state update / stores of item n-1 run in the shadow of item
// n's first MFMAs.  One workgroup barrier per item.
//
// All workgroups must be co-resident: the host launches cooperatively with at
// most one workgroup per compute unit (each uses the whole register file of
// its CU).  Every wait is bounded by spin_limit polls; on expiry the kernel
// records an error word and every workgroup drains.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

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
  int trace_q;            // logical workgroup whose item timeline is recorded, or -1
  long long* trace;       // [items][8] 100 MHz clock stamps of that workgroup
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

// 16 bytes per lane from global memory straight into LDS at lds_base + 16*lane
// (lds_base must be wave-uniform), agent scope.
__device__ __forceinline__ void lds_dma16(const float* gsrc, float* lds_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                   (__attribute__((address_space(3))) void*)lds_base, 16, 0, /*sc1*/ 16);
}

constexpr int P_TILE = 32 * P_LD;  // floats per LDS buffer
constexpr int FLAG_TARGET = PC * 4;  // one count per wave of each of the 8 column slices
constexpr int TS = 8;              // trace stamps per item

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void lstm_persistent_kernel(PersistArgs a) {
  extern __shared__ __attribute__((aligned(16))) float tile[];  // [2][32][P_LD], then 256 floats of scrap

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;

  int q = blockIdx.x;
  if (a.xcd_remap) q = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (q >= a.groups) return;
  if (q == a.trace_q && tid == 0) reinterpret_cast<long long*>(a.status + 16)[0] = wall_clock64();
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

  bool alive = true;
  if (q == a.trace_q && tid == 0) {
    long long* st = reinterpret_cast<long long*>(a.status + 16);
    st[1] = wall_clock64();  // weights requested (st[0]: kernel entry)
    float sink = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < PK / 2; s2 += 32) sink += wr[s2];
    if (sink == 12345.678f) st[3] = 0;
    st[2] = wall_clock64();  // weights (a sample of them) have arrived
  }

  auto item_t = [&](int n) { return n / my_rbs; };
  auto item_rb = [&](int n) { return prs + a.pr * (n % my_rbs); };
  auto flag_of = [&](int ll, int t, int rb) { return a.flags + ((size_t)ll * T + t) * a.nrb + rb; };

  // inputs of item n complete?  Bounded spin on the two counters.
  auto wait_deps = [&](int n) __attribute__((always_inline)) -> bool {
    const int t = item_t(n), rb = item_rb(n);
    bool ok = true;
    if (l > 0) ok = wait_count(flag_of(l - 1, t, rb), FLAG_TARGET, a.status, a.spin_limit);
    if (ok && t >= d) ok = wait_count(flag_of(l, t - d, rb), FLAG_TARGET, a.status, a.spin_limit);
    // The data loads must stay behind the flag reads.  The hardware issues and
    // returns loads in order, so a compiler barrier is all it takes; a fence
    // instruction here would also wait for this wave's outstanding stores.
    asm volatile("" ::: "memory");
    return ok;
  };
  // request / test the two counters of item n without waiting
  struct Flags { int below, own; };
  auto request_flags = [&](int n) __attribute__((always_inline)) -> Flags {
    Flags f{FLAG_TARGET, FLAG_TARGET};
    const int t = item_t(n), rb = item_rb(n);
    if (l > 0) f.below = flag_load(flag_of(l - 1, t, rb));
    if (t >= d) f.own = flag_load(flag_of(l, t - d, rb));
    return f;
  };
  auto flags_ready = [](const Flags& f) { return f.below >= FLAG_TARGET && f.own >= FLAG_TARGET; };

  // Tile n into LDS buffer buf, global -> LDS directly: wave w moves rows
  // 8w..8w+7; one instruction carries half a row (256 floats = 64 lanes x 16
  // bytes, consecutive lanes to consecutive LDS addresses), agent-scope so it
  // sees what other compute units published.
  auto issue_tile = [&](int n, int buf) __attribute__((always_inline)) {
    const int t = item_t(n), rb = item_rb(n);
    const float* xsrc = (l == 0) ? a.xs + (size_t)t * cell : a.hsss + ((size_t)(l - 1) * T + t) * cell;
    const bool has_prev = t >= d;
    const float* hsrc = a.hsss + ((size_t)l * T + (has_prev ? t - d : 0)) * cell;
    float* dst = tile + buf * P_TILE + (8 * wave) * P_LD;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int rg = min(rb * 32 + 8 * wave + r, B - 1);
      lds_dma16(xsrc + (size_t)rg * PH + 4 * lane, dst + r * P_LD);
      if (has_prev) lds_dma16(hsrc + (size_t)rg * PH + 4 * lane, dst + r * P_LD + PH);
    }
    // The first layer's input rows come from memory nobody has touched; pull the rows of the item after
    // this one towards the cache now, so that their copy into LDS one item later is served from L2 like
    // the other layers' rows.  One 4-byte-per-lane copy touches all 64 cache lines of the wave's 8 rows;
    // it lands in a scrap area behind the tiles (a load into registers would need them reserved until
    // the data arrives).
    if (l == 0 && n + 1 < n_items) {
      const int t2 = item_t(n + 1), rb2 = item_rb(n + 1);
      const int rg = min(rb2 * 32 + 8 * wave + (lane >> 3), B - 1);
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(a.xs + (size_t)t2 * cell + (size_t)rg * PH + 32 * (lane & 7)),
          (__attribute__((address_space(3))) void*)(tile + 2 * P_TILE + 64 * wave), 4, 0, 0);
    }
  };
  // steps [q0, q1) of the K loop (steps 0..31: x rows of WU, 32..63: h rows)
  // into two accumulators so that consecutive MFMAs never wait on each other's
  // result; the LDS read for step q+1 is issued before the MFMAs of step q
  auto mfma_part = [&](int buf, auto q0c, auto q1c, v16f& acc0, v16f& acc1) __attribute__((always_inline)) {
    constexpr int q0 = decltype(q0c)::value;
    constexpr int q1 = decltype(q1c)::value;
    const float* arow = tile + buf * P_TILE + j * P_LD + 4 * hh;
    v4f b = *reinterpret_cast<const v4f*>(arow + 8 * q0);
#pragma unroll
    for (int qq = q0; qq < q1; ++qq) {
      v4f bn = b;
      if (qq + 1 < q1) bn = *reinterpret_cast<const v4f*>(arow + 8 * (qq + 1));
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b[0], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b[1], acc1, 0, 0, 0);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 2], b[2], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 3], b[3], acc1, 0, 0, 0);
      b = bn;
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int g4 = q0; g4 < q1; ++g4) {
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };
  // bias, activations and state update of an item: lane-local and branch-free.
  // piece m (0..15) of the computation: gate (m & 3) of unit (m >> 2); the last
  // gate of a unit finishes its c and h
  float eg_i = 0.f, eg_f = 0.f, eg_o = 0.f;
  auto epilogue_piece = [&](const v16f& acc, const float4& cp, float (&hv)[4], float (&cv)[4], auto mc) __attribute__((always_inline)) {
    constexpr int m = decltype(mc)::value;
    constexpr int r = m >> 2;
    const float cpv[4] = {cp.x, cp.y, cp.z, cp.w};
    if constexpr ((m & 3) == 0) eg_i = sigmoid_f(acc[r] + bi[r]);
    if constexpr ((m & 3) == 1) eg_f = sigmoid_f(acc[4 + r] + bf[r]);
    if constexpr ((m & 3) == 2) eg_o = sigmoid_f(acc[8 + r] + bo[r]);
    if constexpr ((m & 3) == 3) {
      const float cand = tanh_f(acc[12 + r] + bg[r]);
      cv[r] = eg_f * cpv[r] + eg_i * cand;
      hv[r] = eg_o * tanh_f(cv[r]);
    }
  };
  auto epilogue_math = [&](const v16f& acc, const float4& cp, float (&hv)[4], float (&cv)[4]) __attribute__((always_inline)) {
    static_for<16>([&](auto mc) __attribute__((always_inline)) { epilogue_piece(acc, cp, hv, cv, mc); });
  };
  // h leaves through write-through stores, c through the cache
  auto epilogue = [&](int n, const v16f& acc, const float4& cp) __attribute__((always_inline)) {
    float hv[4], cv[4];
    epilogue_math(acc, cp, hv, cv);
    const int t = item_t(n), rb = item_rb(n);
    const int rg = rb * 32 + j;
    if (alive && rg < B) {
      float* hdst = a.hsss + ((size_t)l * T + t) * cell + (size_t)rg * PH + u0;
      float* cdst = a.csss + ((size_t)l * T + t) * cell + (size_t)rg * PH + u0;
      *reinterpret_cast<float4*>(cdst) = make_float4(cv[0], cv[1], cv[2], cv[3]);
      coherent_store8(hdst, hv[0], hv[1]);
      coherent_store8(hdst + 2, hv[2], hv[3]);
    }
  };
  auto load_cprev = [&](int n) __attribute__((always_inline)) -> float4 {
    const int t = item_t(n), rb = item_rb(n);
    float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
    if (alive && t >= d) {
      const int rgc = min(rb * 32 + j, B - 1);
      cp = *reinterpret_cast<const float4*>(a.csss + ((size_t)l * T + (t - d)) * cell + (size_t)rgc * PH + u0);
    }
    return cp;
  };
  // every wave publishes its own part of an item: its stores acknowledged, then one count
  auto publish = [&](int n) __attribute__((always_inline)) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    if (lane == 0 && alive)
      __hip_atomic_fetch_add(flag_of(l, item_t(n), item_rb(n)), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  const bool tracing = (q == a.trace_q) && tid == 0;
  v16f acc0, acc1;

  // How far apart an item and the item that needs it are in this workgroup's
  // own sequence decides the schedule: distance 1 (one row block, dilation 1)
  // leaves nothing to overlap.
  const long long own_distance = (long long)d * my_rbs;
  const bool serial = own_distance < 2;

  if (serial) {
    for (int n = 0; n < n_items; ++n) {
      if (tracing) a.trace[TS * n + 0] = wall_clock64();
      if (alive) alive = wait_deps(n);
      if (alive) issue_tile(n, 0);
      const float4 cp = load_cprev(n);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
      mfma_part(0, std::integral_constant<int, 0>{}, std::integral_constant<int, PH / 8>{}, acc0, acc1);
      if (item_t(n) >= d) mfma_part(0, std::integral_constant<int, PH / 8>{}, std::integral_constant<int, PK / 8>{}, acc0, acc1);
      v16f acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = acc0[r] + acc1[r];
      epilogue(n, acc, cp);
      publish(n);
      __syncthreads();  // the tile is rewritten by the next item
      if (tracing) a.trace[TS * n + 7] = wall_clock64();
    }
    return;
  }

  // ---- pipelined schedule.  Per item n:
  //   the first half of the x half of the MFMAs;
  //   publish item n-1: its h and c went out at the end of item n-1, so by now
  //     they are acknowledged and the wait costs nothing -- and nothing newer
  //     is outstanding yet that the wait would also catch;
  //   request tile n+1 into the other LDS buffer if its producers are seen to
  //     be done (their counters were requested at the end of item n-1); if
  //     not, look again after the x half, and wait only after the h half;
  //   the rest of the x half, the h half;
  //   wait for tile n+1, one workgroup barrier;
  //   activations, state update and stores of item n.  (Vector instructions do
  //   not hide behind fp32 MFMAs on this machine, so nothing is gained by
  //   deferring them, and the sooner the stores go out the sooner the layer
  //   above can start: an item is visible to its consumers about 2 us after
  //   its last MFMA.  That hand-over time, 31 times in a row, is what the
  //   wavefront pays at the start and at the end of a 32-layer stack.)
  alive = wait_deps(0);
  if (alive) issue_tile(0, 0);
  Flags fl = (n_items > 1) ? request_flags(1) : Flags{FLAG_TARGET, FLAG_TARGET};
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  constexpr int QX = PH / 8;   // MFMA steps of the x half
  constexpr int QE = QX / 2;   // steps before the previous item is published (its stores take about 2 us to be acknowledged)
  for (int n = 0; n < n_items; ++n) {
    const int buf = n & 1;
    if (tracing) a.trace[TS * n + 0] = wall_clock64();
    const bool has_prev = item_t(n) >= d;
    const bool more = n + 1 < n_items;
    bool pending = alive && more;  // tile n+1 still to be requested
    int looks = 0;                 // looks taken before the request went out (for the trace)

    auto look = [&]() __attribute__((always_inline)) {
      if (pending) {
        ++looks;
        if (flags_ready(fl)) {
          asm volatile("" ::: "memory");
          issue_tile(n + 1, buf ^ 1);
          pending = false;
        } else {
          fl = request_flags(n + 1);
        }
      }
    };

    const float4 cp = load_cprev(n);
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
    mfma_part(buf, std::integral_constant<int, 0>{}, std::integral_constant<int, QE>{}, acc0, acc1);
    if (n > 0) publish(n - 1);
    look();
    if (tracing) a.trace[TS * n + 1] = wall_clock64();
    mfma_part(buf, std::integral_constant<int, QE>{}, std::integral_constant<int, QX>{}, acc0, acc1);
    if (tracing) a.trace[TS * n + 2] = wall_clock64();
    look();
    if (tracing) a.trace[TS * n + 3] = wall_clock64();
    if (has_prev) mfma_part(buf, std::integral_constant<int, QX>{}, std::integral_constant<int, PK / 8>{}, acc0, acc1);
    if (tracing) a.trace[TS * n + 4] = wall_clock64() | ((long long)(pending ? 7 : looks) << 60);
    // last resort: wait for the producers here
    if (pending) {
      alive = wait_deps(n + 1);
      if (alive) issue_tile(n + 1, buf ^ 1);
    }
    if (n + 2 < n_items) fl = request_flags(n + 2);
    if (tracing) a.trace[TS * n + 5] = wall_clock64();
    __builtin_amdgcn_s_waitcnt(0);  // tile n+1 has landed in LDS
    if (tracing) a.trace[TS * n + 6] = wall_clock64();
    __syncthreads();
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = acc0[r] + acc1[r];
    epilogue(n, acc, cp);
    if (tracing) a.trace[TS * n + 7] = wall_clock64();
  }
  publish(n_items - 1);
}

__global__ void fill_zero_kernel(int* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

static size_t flag_count(int L, int T, int B) {
  const int nrb = (B + 31) / 32;
  return (size_t)L * T * nrb;
}

// Workspace layout: [64 ints: status][flags][trace: T*nrb*8 stamps of 8 bytes].
static size_t trace_offset_bytes(int L, int T, int B) { return ((flag_count(L, T, B) + 64) * sizeof(int) + 15) / 16 * 16; }
static size_t workspace_need(int L, int T, int B) {
  return trace_offset_bytes(L, T, B) + (size_t)T * ((B + 31) / 32) * 8 * sizeof(long long);
}

// Profiling hook: FTK_LSTM_PLAIN_LAUNCH=1 launches without the cooperative
// co-residency check (counter collection tools that cannot follow cooperative
// launches).  The grid never exceeds one workgroup per compute unit, so on an
// otherwise idle device the workgroups are co-resident all the same; if they
// are not, the bounded waits end the launch with the error word set.
static bool plain_launch() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("FTK_LSTM_PLAIN_LAUNCH");
    v = (e && atoi(e) != 0) ? 1 : 0;
  }
  return v == 1;
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
  const size_t lds = (size_t)2 * P_TILE * sizeof(float) + 1024;  // two tiles + the prefetch scrap area
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
  for (int l = 0; l < kMaxLayers; ++l) a.dil[l] = (l < L && dil) ? dil[l] : 1;
  const int grid = a.groups;
  a.xcd_remap = (grid % 8 == 0) ? 1 : 0;

  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, a.status, nflags + 64);
  rc = check_launch("fill_zero_kernel");
  if (rc) return rc;

  void* kargs[] = {&a};
  if (plain_launch()) {
    hipLaunchKernelGGL(lstm_persistent_kernel, dim3(grid), dim3(256), lds, s, a);
    rc = check_launch("lstm_persistent_kernel");
    if (rc) return rc;
  } else {
    FTK_HIP(hipLaunchCooperativeKernel(fn, dim3(grid), dim3(256), kargs, (unsigned)lds, s));
  }
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
