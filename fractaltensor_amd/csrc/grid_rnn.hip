// Stacked grid RNN for gfx950, fp32: every position (d, i, j) of a depth x first-axis x second-axis grid holds two
// tanh cells that share one state,
//   s        = [ h_x(d, i-1, j) | h_y(d, i, j-1) ]                     (zeros outside the grid)
//   h_x(d,i,j) = tanh(x_in @ Wx[d] + s @ Ux[d] + bx[d]),   h_y(d,i,j) = tanh(y_in @ Wy[d] + s @ Uy[d] + by[d])
// with (x_in, y_in) = (h_x, h_y)(d-1, i, j) above the first block and the two input sequences in it.
//
// Schedule.  Position (d, i, j) needs (d-1, i, j), (d, i-1, j) and (d, i, j-1), so all positions of one
// anti-diagonal plane m = d + i + j are independent: one launch per plane, D + L1 + L2 - 2 launches, each batched
// over the plane's positions.  Nothing is gathered or scattered: a workgroup finds its position from its index
// and reads the three neighbours where they lie in the output array.
//
// Tiling.  A workgroup owns 32 batch rows x 32 hidden units of one position, for both directions, and splits the
// work into products of K = H, one per wave: x_in @ W, y_in @ W, state_x @ U[:H], state_y @ U[H:] when the two
// directions share their parameters (four waves; the state products are computed once and serve both), six
// products otherwise.  A product whose state lies outside the grid is skipped.  Each wave runs its product on
// v_mfma_f32_32x32x2_f32 straight from global memory -- no operand is used by a second wave of the workgroup, so
// LDS staging would only add barriers -- with the operands of the next two or three k chunks of 32 in registers.  Within a
// chunk the k index is permuted: step (q, e) uses k = 4q + e for lanes 0-31 and k = 16 + 4q + e for lanes 32-63.  The products are added through LDS before bias
// and tanh.  Given a workspace, the entry point first re-lays the parameters so that the sixteen weights a lane
// needs of a chunk come in four loads that each cover 1 KB of consecutive bytes.  The activations are loaded as whole
// 128-byte row segments and turned round through a wave-private LDS tile.
//
// Placement.  Workgroups are numbered position-major, unit block fastest, and ids go round the eight XCDs: with
// eight unit blocks (H = 256) an XCD only ever touches one 32-column slice of every block's parameters.  (Running
// the positions of block d on XCD d % 8 instead, so that an XCD touches the parameters of four blocks only, was
// measured and is slower: the planes' positions do not divide evenly over the blocks.)
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

struct GridArgs {
  const float* xs;   // [L1 or L2, B, H]
  const float* ys;   // [L2 or L1, B, H]
  const float* W[2];     // [D, H, H]   per direction
  const float* U[2];     // [D, 2H, H]
  const float* bias[2];  // [D, bias_rows, H] or nullptr
  float* hsss;           // [D, L1, L2, 2, B, H]
  int D, L1, L2, B, H;
  int bias_rows;  // 1: one row for the whole batch, B: a row per batch row
  int crossed;    // 0: x_in = xs[i], y_in = ys[j];  1: x_in = xs[j], y_in = ys[i]
  int m;          // the plane d + i + j of this launch
  const float* Wp[2];  // the same parameters re-laid per wave (pack kernel below), or nullptr
  const float* Up[2];
};

constexpr int GKC = 32;  // k chunk

// Number of positions with d + i + j = m, and the z-th of them in (d, i) order.
__host__ __device__ inline int plane_positions(int D, int L1, int L2, int m, int z, int* d_out, int* i_out) {
  int n = 0;
  const int dlo = m - (L1 - 1) - (L2 - 1) > 0 ? m - (L1 - 1) - (L2 - 1) : 0;
  const int dhi = m < D - 1 ? m : D - 1;
  for (int d = dlo; d <= dhi; ++d) {
    const int r = m - d;
    const int ilo = r - (L2 - 1) > 0 ? r - (L2 - 1) : 0;
    const int ihi = r < L1 - 1 ? r : L1 - 1;
    const int cnt = ihi - ilo + 1;
    if (cnt <= 0) continue;
    if (z >= n && z < n + cnt) {
      *d_out = d;
      *i_out = ilo + (z - n);
    }
    n += cnt;
  }
  return n;
}

struct ChunkRegs {
  float4 a[4];
  float b[16];
};

// One k chunk of a product.  Every load instruction is made to cover whole cache lines -- what a CU runs out of
// here is the rate at which its L1 takes lines, not bytes.  The activations come as row segments: load q brings
// rows 8q .. 8q+7 of the chunk, 128 consecutive bytes each (8 lines per load; loading what the MFMAs want of a
// lane, 16 values of one row, touches 32), lane l holding floats 4*(l%8)..+3 of row 8q + l/8 (row_off);
// mfma_chunk turns them round.  Weights: lane (jl, hh) needs column jl of the weight rows k = 16*hh .. 16*hh+15.
// PACKED: they are four 16-byte pieces of the re-laid copy, 1 KB apart (four loads instead of sixteen, each 1 KB of
// consecutive bytes across the wave; wcol points at the lane's first piece of chunk 0, chunks are 1024 floats
// apart); otherwise sixteen loads of one value each, where they lie.
template <bool PACKED>
__device__ __forceinline__ void load_chunk(ChunkRegs& r, const float* __restrict__ arow, const float* __restrict__ wcol,
                                           int H, int c, const int (&row_off)[4]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) r.a[q] = *reinterpret_cast<const float4*>(arow + row_off[q] + c * GKC);
  if constexpr (PACKED) {
    const float4* wp = reinterpret_cast<const float4*>(wcol + (size_t)c * 1024);
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const float4 t = wp[64 * e4];  // one load instruction of the wave covers 1 KB of consecutive bytes
      r.b[4 * e4] = t.x; r.b[4 * e4 + 1] = t.y; r.b[4 * e4 + 2] = t.z; r.b[4 * e4 + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e) r.b[e] = wcol[(size_t)(c * GKC + e) * H];
  }
}

// Re-lays M [D][rows][H] (rows a multiple of 32) as [D][H/32 unit blocks][rows/32 chunks][4][64 lanes][4]: element
// 4*e4 + t of lane (jl, hh) of chunk c of unit block ub is M[32c + 16hh + 4*e4 + t][32ub + jl] -- the order
// load_chunk reads, one 16-byte piece per lane and load, so that a load instruction covers 1 KB of consecutive bytes.
__global__ __launch_bounds__(256) void grid_pack_weights_kernel(const float* __restrict__ M, float* __restrict__ out,
                                                                long long total4, int rows, int H) {
  const int ctot = rows / GKC, nub = H / 32;
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total4; idx += (long long)gridDim.x * 256) {
    const int lane = (int)(idx & 63);
    const int e4 = (int)((idx >> 6) & 3);
    const long long rest = idx >> 8;
    const int c = (int)(rest % ctot);
    const int ub = (int)((rest / ctot) % nub);
    const long long d = rest / ((long long)ctot * nub);
    const int k = c * GKC + 16 * (lane >> 5) + 4 * e4;
    const float* src = M + ((size_t)d * rows + k) * H + ub * 32 + (lane & 31);
    reinterpret_cast<float4*>(out)[idx] = make_float4(src[0], src[H], src[2 * (size_t)H], src[3 * (size_t)H]);
  }
}

constexpr int kTurnLd = GKC + 4;  // padded row of a wave's 32 x 32 turn-round tile in LDS (floats)
typedef __attribute__((address_space(3))) float lds_float;

// r.a holds row segments; they go through the wave's own LDS tile and come back as the MFMAs want them (lane
// (jl, hh): row jl, k = 16*hh + 4q..+3).  LDS operations of one wave execute in order, so the tile needs no second
// buffer and no barrier.  The pointer carries its address space: through a generic pointer the compiler emits
// flat loads and stores, which made this twice as slow as not turning at all.
__device__ __forceinline__ void mfma_chunk(v16f& acc, const ChunkRegs& r, lds_float* turn) {
  float4 a[4];
  {
    const int lane = threadIdx.x & 63;
    typedef __attribute__((address_space(3))) v4f lds_v4f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4f t = {r.a[q].x, r.a[q].y, r.a[q].z, r.a[q].w};
      *reinterpret_cast<lds_v4f*>(turn + (8 * q + (lane >> 3)) * kTurnLd + 4 * (lane & 7)) = t;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4f t = *reinterpret_cast<lds_v4f*>(turn + (lane & 31) * kTurnLd + 16 * (lane >> 5) + 4 * q);
      a[q] = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q].x, r.b[4 * q + 0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q].y, r.b[4 * q + 1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q].z, r.b[4 * q + 2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q].w, r.b[4 * q + 3], acc, 0, 0, 0);
  }
}

// acc += act[32 rows, H] @ w[H, 32 cols] with NS chunks in flight.  The scheduling fences keep the refill of a
// register set behind the MFMAs that read it and ahead of the next set's MFMAs, so the wait the compiler puts
// before a set's MFMAs leaves the younger refills outstanding.  That only works where no load sits under a
// run-time condition (at a join the compiler must assume the path with the fewest younger loads and ends up
// waiting for all of them), hence the chunk count as a template argument for the usual hidden sizes (128, 256, 384, 512, 768, 1024); NCH = 0 is
// the form for any other count.  NS is 3 with the parameters where they lie (20 loads per chunk: a wave cannot
// have more than 63 outstanding) and 2 with the re-laid copy (8 loads per chunk; 3 to 6 sets measured slower,
// 1.21 to 1.53 ms against 1.17 ms for H = 256, as did one).
template <int NCH, bool PACKED, int NS>
__device__ __forceinline__ void product(v16f& acc, const float* __restrict__ arow, const float* __restrict__ wcol, int H,
                                        const int (&row_off)[4], lds_float* turn) {
  auto fence = [] { __builtin_amdgcn_sched_barrier(0); };
  if constexpr (NCH >= NS) {
    H = NCH * GKC;  // known at compile time: the weight rows' addresses become constant offsets
    ChunkRegs r[NS];
    static_for<NS>([&](auto s) { load_chunk<PACKED>(r[s], arow, wcol, H, s, row_off); fence(); });
    constexpr int MAIN = NCH / NS - 1;  // rounds all of whose refills exist
    for (int k = 0; k < MAIN; ++k) {
      static_for<NS>([&](auto s) {
        mfma_chunk(acc, r[s], turn); fence();
        load_chunk<PACKED>(r[s], arow, wcol, H, NS * (k + 1) + s, row_off); fence();
      });
    }
    constexpr int CE = NS * MAIN;  // the sets hold chunks CE .. CE+NS-1; fewer than NS more follow
    static_for<NS>([&](auto s) {
      mfma_chunk(acc, r[s], turn); fence();
      if constexpr (CE + NS + s < NCH) { load_chunk<PACKED>(r[s], arow, wcol, H, CE + NS + s, row_off); fence(); }
    });
    static_for<NS>([&](auto s) {
      if constexpr (CE + NS + s < NCH) { mfma_chunk(acc, r[s], turn); fence(); }
    });
  } else {
    ChunkRegs r0, r1;
    const int nch = H / GKC;
    for (int c = 0; c < nch; c += 2) {  // two chunks per round, the second one clamped (and then not used)
      load_chunk<PACKED>(r0, arow, wcol, H, c, row_off);
      load_chunk<PACKED>(r1, arow, wcol, H, min(c + 1, nch - 1), row_off);
      mfma_chunk(acc, r0, turn);
      if (c + 1 < nch) mfma_chunk(acc, r1, turn);
    }
  }
}

// Occupancy is held at two (shared parameters) or three (six products) waves per SIMD on purpose: with more
// workgroups in flight the weight slices they stream no longer fit the L2 together, and the whole forward is
// slower (measured: 1.44 / 1.49 / 1.56 ms at 2 / 3 / 4 waves for H = 256 with the parameters where they lie; with
// the re-laid copy 1.17 / 1.17 / 1.21 ms, and 9.8 / 11.2 / 11.3 ms for H = 1024).
template <bool SHARED, int NCH, bool PACKED>
__global__ __launch_bounds__(SHARED ? 256 : 384) __attribute__((amdgpu_waves_per_eu(SHARED ? 2 : 3, SHARED ? 2 : 3)))
void grid_rnn_plane_kernel(GridArgs a) {
  constexpr int JOBS = SHARED ? 4 : 6;
  __shared__ float red[JOBS][16][64];
  __shared__ __attribute__((aligned(16))) float turn_tiles[JOBS][32 * kTurnLd];

  const int H = a.H, B = a.B;
  const int nub = H / 32, nrb = (B + 31) / 32;
  const int per_pos = nub * nrb;
  const int item = blockIdx.x;
  int d = 0, i = 0;
  plane_positions(a.D, a.L1, a.L2, a.m, item / per_pos, &d, &i);
  const int j = a.m - d - i;
  const int ub = item % nub;          // block of 32 hidden units
  const int rb = (item / nub) % nrb;  // block of 32 batch rows

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;  // the product
  const int jl = lane & 31;
  const int hh = lane >> 5;

  const size_t BH = (size_t)B * H;
  auto pos = [&](int dd, int ii, int jj, int which) {
    return a.hsss + ((((size_t)dd * a.L1 + ii) * a.L2 + jj) * 2 + which) * BH;
  };
  const float* x_in = d > 0 ? pos(d - 1, i, j, 0) : a.xs + (size_t)(a.crossed ? j : i) * BH;
  const float* y_in = d > 0 ? pos(d - 1, i, j, 1) : a.ys + (size_t)(a.crossed ? i : j) * BH;
  const float* sx = i > 0 ? pos(d, i - 1, j, 0) : nullptr;
  const float* sy = j > 0 ? pos(d, i, j - 1, 1) : nullptr;

  // this wave's product: kind 0 input @ W, 1 state_x @ U[:H], 2 state_y @ U[H:]
  const int dir = SHARED ? 0 : (wave & 1);
  const int kind = SHARED ? (wave < 2 ? 0 : wave - 1) : (wave >> 1);
  const bool y_side = SHARED ? wave == 1 : dir == 1;
  const float* act = kind == 0 ? (y_side ? y_in : x_in) : kind == 1 ? sx : sy;
  const float* w;  // where this lane's weights of chunk 0 lie
  if (PACKED) {
    const int cps = H / GKC;                       // chunks per product
    const int ctot = kind == 0 ? cps : 2 * cps;    // chunks of the whole matrix: U holds both state products
    const float* base = kind == 0 ? a.Wp[dir] + (size_t)d * H * H : a.Up[dir] + (size_t)d * 2 * H * H;
    w = base + ((size_t)ub * ctot + (kind == 2 ? cps : 0)) * 1024 + lane * 4;
  } else {
    const float* Ud = a.U[dir] + (size_t)d * 2 * H * H;
    const float* base = kind == 0 ? a.W[dir] + (size_t)d * H * H : kind == 1 ? Ud : Ud + (size_t)H * H;
    w = base + (size_t)(16 * hh) * H + ub * 32 + jl;
  }

  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  if (act) {
    // load q of a chunk: row 8q + lane/8 of the row block, floats 4*(lane%8)..+3
    int row_off[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) row_off[q] = min(rb * 32 + 8 * q + (lane >> 3), B - 1) * H + 4 * (lane & 7);
    lds_float* turn = (lds_float*)&turn_tiles[wave][0];
    product<NCH, PACKED, PACKED ? 2 : 3>(acc, act, w, H, row_off, turn);
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) red[wave][r][lane] = acc[r];
  __syncthreads();
  if (wave >= 4) return;

  // wave (dir, rh) finishes registers 8*rh .. 8*rh+7 of direction dir: lane (jl, hh) holds column jl of rows
  // 8*(r/4) + 4*hh + r%4
  const int od = wave & 1;
  const int rh = wave >> 1;
  float* out = pos(d, i, j, od);
  const float* bias = a.bias[od] ? a.bias[od] + (size_t)d * a.bias_rows * H : nullptr;
  const int col = ub * 32 + jl;
#pragma unroll
  for (int rr = 0; rr < 8; ++rr) {
    const int r = 8 * rh + rr;
    float v;
    if (SHARED) v = red[od][r][lane] + red[2][r][lane] + red[3][r][lane];
    else v = red[od][r][lane] + red[2 + od][r][lane] + red[4 + od][r][lane];
    const int row = rb * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
    if (row < B) {
      const float bv = bias ? bias[(size_t)(a.bias_rows == 1 ? 0 : row) * H + col] : 0.0f;
      out[(size_t)row * H + col] = tanh_f(v + bv);
    }
  }
}

}  // namespace ftk

extern "C" size_t ftk_grid_rnn_workspace_bytes(int D, int H) {
  if (D <= 0 || H <= 0) return 0;
  return 2 * (size_t)D * 3 * H * H * sizeof(float);  // W and U of both directions, re-laid
}

extern "C" int ftk_grid_rnn_f32(const float* xs, const float* ys, const float* Wx, const float* Ux, const float* bx,
                                const float* Wy, const float* Uy, const float* by, float* hsss, int D, int L1, int L2,
                                int B, int H, int bias_rows, int crossed, void* workspace, size_t workspace_bytes,
                                ftk_stream_t stream) {
  using namespace ftk;
  if (!xs || !ys || !Wx || !Ux || !Wy || !Uy || !hsss)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_grid_rnn_f32: inputs, weights and the output must be non-NULL");
  if (D <= 0 || L1 <= 0 || L2 <= 0 || B <= 0 || H <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_grid_rnn_f32: D, L1, L2, B and H must be positive");
  if (H % 32 != 0) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_grid_rnn_f32: H must be a multiple of 32 (got %d)", H);
  if (bias_rows != 1 && bias_rows != B)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_grid_rnn_f32: bias_rows must be 1 or B (got %d)", bias_rows);
  if ((bx == nullptr) != (by == nullptr))
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_grid_rnn_f32: give both biases or neither");
  GridArgs a;
  a.xs = xs; a.ys = ys;
  a.W[0] = Wx; a.W[1] = Wy;
  a.U[0] = Ux; a.U[1] = Uy;
  a.bias[0] = bx; a.bias[1] = by;
  a.hsss = hsss;
  a.D = D; a.L1 = L1; a.L2 = L2; a.B = B; a.H = H;
  a.bias_rows = bias_rows;
  a.crossed = crossed ? 1 : 0;
  const bool shared = Wx == Wy && Ux == Uy;
  hipStream_t st = (hipStream_t)stream;
  // with room for it, the parameters are re-laid first so that a lane's weights of a chunk are contiguous
  const size_t per_dir = (size_t)D * 3 * H * H;
  const bool packed = workspace && workspace_bytes >= (shared ? 1 : 2) * per_dir * sizeof(float) &&
                      reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
  a.Wp[0] = a.Wp[1] = a.Up[0] = a.Up[1] = nullptr;
  if (packed) {
    float* ws = static_cast<float*>(workspace);
    for (int dir = 0; dir < (shared ? 1 : 2); ++dir) {
      float* wp = ws + dir * per_dir;
      float* up = wp + (size_t)D * H * H;
      const long long w4 = (long long)D * H * H / 4, u4 = 2 * w4;
      hipLaunchKernelGGL(grid_pack_weights_kernel, dim3((unsigned)std::min<long long>((w4 + 255) / 256, 65536)), dim3(256), 0, st,
                         dir ? Wy : Wx, wp, w4, H, H);
      hipLaunchKernelGGL(grid_pack_weights_kernel, dim3((unsigned)std::min<long long>((u4 + 255) / 256, 65536)), dim3(256), 0, st,
                         dir ? Uy : Ux, up, u4, 2 * H, H);
      a.Wp[dir] = wp;
      a.Up[dir] = up;
    }
    if (shared) { a.Wp[1] = a.Wp[0]; a.Up[1] = a.Up[0]; }
  }
  const int per_pos = (H / 32) * ((B + 31) / 32);
  for (int m = 0; m <= D + L1 + L2 - 3; ++m) {
    int d0 = 0, i0 = 0;
    const long long groups = (long long)plane_positions(D, L1, L2, m, -1, &d0, &i0) * per_pos;
    if (groups <= 0) continue;
    if (groups > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_grid_rnn_f32: a plane of %lld workgroups", groups);
    a.m = m;
    const dim3 g((unsigned)groups);
#define FTK_GRID_LAUNCH_P(NCH, P)                                                                         \
  do {                                                                                                  \
    if (shared) hipLaunchKernelGGL((grid_rnn_plane_kernel<true, NCH, P>), g, dim3(256), 0, st, a);      \
    else hipLaunchKernelGGL((grid_rnn_plane_kernel<false, NCH, P>), g, dim3(384), 0, st, a);            \
  } while (0)
#define FTK_GRID_LAUNCH(NCH)                \
  do {                                      \
    if (packed) FTK_GRID_LAUNCH_P(NCH, true); \
    else FTK_GRID_LAUNCH_P(NCH, false);     \
  } while (0)
    if (H == 256) FTK_GRID_LAUNCH(8);
    else if (H == 512) FTK_GRID_LAUNCH(16);
    else if (H == 1024) FTK_GRID_LAUNCH(32);
    else if (H == 128) FTK_GRID_LAUNCH(4);
    else if (H == 384) FTK_GRID_LAUNCH(12);
    else if (H == 768) FTK_GRID_LAUNCH(24);
    else FTK_GRID_LAUNCH(0);
#undef FTK_GRID_LAUNCH
#undef FTK_GRID_LAUNCH_P
  }
  return check_launch("grid_rnn_plane_kernel");
}
