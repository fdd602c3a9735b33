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
//
// lstm_cell_f16_kernel is the fp16-storage flavour for hidden sizes whose
// weights no longer fit on chip: the same transposed product on
// v_mfma_f32_32x32x16_f16, a workgroup of 4 waves owning 256 batch rows x 32
// hidden units so that every weight is fetched once per cell, and k chunks of
// 32 copied from global memory straight into a ring of three to five LDS stages
// (global_load_lds_dwordx4), two workgroups per compute unit.
#include <stdlib.h>

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

// ---------------------------------------------------------------- fp16 cell
struct CellDescH {
  const _Float16* x;       // [B, I]; split flavour: [B, 2I], a row = its two planes [value | remainder]
  const _Float16* h_prev;  // [B, H] or nullptr (zero state); split flavour: [B, 2H] planes
  const void* c_prev;      // [B, H] or nullptr; fp16, split flavour: fp32
  const _Float16* WU;      // [(I+H), 4H], or the packed layout
  const float* bias;       // [4H] or nullptr
  void* h;                 // [B, H]; fp16, split flavour: fp32
  void* c;                 // [B, H]
  // split flavour only
  const float* xratio;     // [B]: scale of the x rows relative to the h rows, or nullptr (x is an h of the layer below)
  const float* wscale;     // [4H]: what a gate sum of column n is multiplied by to undo the operand scales
  _Float16* h_planes;      // [B, 2H]: the two planes of h for the cells that read it
  int rows;                // leading batch rows this cell computes (a ragged batch at its step), 0 = all B
};

struct CellListH {
  int n;
  int packed;  // 1: WU of every cell is in the packed layout; 2, 3: packed split weights (three / two planes per chunk)
  int* small_states = nullptr;  // split flavour: set to 1 when four neighbouring units of a row are written whose largest non-zero |h| is below 2^-26 (may be nullptr)
  CellDescH cells[kMaxCellsPerLaunch];
};

// The split flavour writes h as fp16(h * 2^14) plus the fp16 of what that leaves, unscaled: below h * 2^14 = 2^-12
// (|h| < 2^-26, 1.5e-8) the two planes hold fewer than 13 bits of a value.  One such value among larger ones is exact
// enough for the sums it enters; what is reported is a lane's four neighbouring units all being that small (and not
// all zero): a row, or a layer, that has faded.
constexpr unsigned kSmallStateStreamedBits = (127u - 12u) << 23;
constexpr int HK = 32;                       // k chunk
constexpr int HROWS = 256;                   // batch rows per workgroup
constexpr int H_ACT_BYTES = HROWS * HK * 2;  // activation rows of a chunk: 64 bytes each
// per unit-block width UB (32 or 64 hidden units = 128 or 256 gate columns): bytes of a weight row, of a stage
constexpr int cell_row_bytes(int ub) { return ub * 4 * 2; }
constexpr int cell_stage_bytes(int ub) { return H_ACT_BYTES + HK * cell_row_bytes(ub); }
// s_waitcnt immediate that waits for vmcnt <= n only (n < 64: bits 3:0 and 15:14; expcnt and lgkmcnt left open)
constexpr int vmcnt_only(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

#ifndef CELL_STAGES8
#define CELL_STAGES8 3
#endif
// LDS stages: chunk ch in use, the next stages - 1 chunks on their way.  What is in flight is what hides the
// 1.5 - 2 us a copy takes under load: 32 KB per compute unit and chunk.
constexpr int cell_stages(int ub) { return ub == 64 ? CELL_STAGES8 : 3; }
constexpr size_t cell_lds_bytes(int ub) { return (size_t)cell_stage_bytes(ub) * cell_stages(ub); }  // 72 KB / 96 KB

typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte offset) straight into LDS at
// lds_addr + 16*lane (lds_addr wave-uniform).  Opaque to the compiler: the caller waits with s_waitcnt vmcnt.
__device__ __forceinline__ void cell_dma16(const void* gbase, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_addr), "v"(byte_off), "s"(gbase) : "memory", "m0");
}

// LDS layout of a stage.  Both tiles are stored row-major as in memory, without padding, and their 16-byte
// chunks are swapped around within a row so that fragment reads do not collide on banks:
//   activation row r (64 bytes, 4 chunks): chunk c sits in slot c ^ ((r >> 2) & 3); the 16 lanes that a
//     ds_read_b128 serves together (16 consecutive rows, one chunk index) then touch 16 different 16-byte
//     positions of the 256-byte bank line;
//   weight row k (256 bytes, 16 chunks; chunk 4*ug + q = gate q of the 8 units of unit group ug): chunk c sits
//     in slot c ^ ((k & 3) << 2); the transposing read ds_read_b64_tr_b16 takes 64 bytes from each of four
//     consecutive rows per pass, which land in four different 64-byte groups.
// A copy instruction fills 1 KB of consecutive slots, each lane choosing the global chunk its slot holds.
// A ring of stages: while chunk ch is used, the next chunks are on their way (cell_stages).
//
// WAVES = 4: a workgroup owns 32 hidden units (two waves side by side, two on top of each other), two
// workgroups share a compute unit.  WAVES = 8: 64 hidden units (four waves side by side; weight rows of 512
// bytes, 32 chunks, the same slot rule), one workgroup per compute unit: every activation row then enters
// half as many LDS tiles.  Either way a wave owns 128 rows x 2 unit groups and two waves share a SIMD, the
// one filling the gaps that the barriers and LDS latencies of the other leave.
//
// PACKED: the cell's WU points at weights laid out by lstm_pack_weights_f16_kernel, per unit block the very
// bytes of the LDS rows above, so a workgroup streams one contiguous run of rows; otherwise at the
// [(I+H), 4H] matrix, from which a workgroup picks four segments per row.
//
// SPLIT: fp32 data on fp16 MFMAs.  Every fp32 operand v of a group that shares a power-of-two scale s (an
// activation row, a weight column) is the sum of two fp16 numbers, top = fp16(v s) and rest = fp16(v s - top),
// to within 2^-22 |v s|, so a product is top*top + top*rest + rest*top up to a term of 2^-22 of it.  The three
// products go into the same fp32 accumulators as three k chunks in a row -- (top, top), (top, rest), (rest,
// top) -- of a contraction three times as long: x and h_prev arrive as rows [top | rest], the packed weights
// hold the rows of every chunk three times in that order (lstm_pack_split_weights_kernel).  The x rows carry
// their own scale and the h rows 2^14, so between the last x chunk and the first h chunk the sums are
// multiplied by the ratio; the epilogue undoes the h and column scales, computes in fp32, writes h and c in
// fp32 and the two planes of h for the cells that read it next.
//
// GEMM: the product alone, C = A @ Bm for row-major fp16 A [B, I] (cell.x), Bm [I, 4H] (cell.WU) and C [B, 4H]
// (cell.h): no state, no activation; the workgroup's 4*UB columns are the four runs UB*ub .. +UB of the four
// column quarters, stored as they come out of the accumulators.
template <bool PACKED, int WAVES, bool SPLIT, bool GEMM = false>
__global__ __launch_bounds__(WAVES * 64, 8 / WAVES) void lstm_cell_f16_kernel(CellListH list, int B, int I, int H) {
  static_assert(!SPLIT || PACKED, "the split flavour reads packed weights");
  static_assert(!GEMM || (!SPLIT && !PACKED), "the plain product reads Bm as it is");
  constexpr int REP = SPLIT ? 3 : 1;        // k chunks per chunk of the contraction
  constexpr int UB = 8 * WAVES;             // hidden units per workgroup
  constexpr int CW = WAVES / 2;             // waves side by side
  constexpr int ROWB = cell_row_bytes(UB);  // bytes of a weight row in LDS
  constexpr int H_STAGE = cell_stage_bytes(UB);
  constexpr int ACT_COPIES = 16 / WAVES;    // activation copies per wave and chunk (1 KB = 16 rows each)
  extern __shared__ __attribute__((aligned(1024))) unsigned char cell_smem[];
  using lds_v4s = __attribute__((address_space(3))) v4s;

  // Workgroups are dealt to the 8 XCDs round-robin by their linear index.  All workgroups of a cell are
  // placed on one XCD (cell = xcd + 8 m), neighbouring unit blocks first: the cell's activation rows are then
  // fetched into one L2 instead of eight, and the 64-byte weight segments of neighbouring unit blocks that
  // share a cache line are served by the same L2.
  const int nub = H / UB, nrb = (B + HROWS - 1) / HROWS;
  // (the plain product has few, large problems: its workgroups are simply numbered problem, row block, column block)
  const int slot = GEMM ? (int)blockIdx.x : (int)(blockIdx.x >> 3);
  const int cell = GEMM ? slot / (nub * nrb) : (int)(blockIdx.x & 7) + 8 * (slot / (nub * nrb));
  if (cell >= list.n) return;
  const CellDescH cd = list.cells[cell];
  const int Bc = cd.rows > 0 ? cd.rows : B;  // rows of this cell
  const int ub = slot % nub;          // block of UB hidden units
  const int rb = (slot / nub) % nrb;  // block of 256 batch rows
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wr = wave / CW;  // rows 128*wr .. +128 of the block
  const int wc = wave % CW;  // unit groups 2*wc, 2*wc+1 of the block's
  const int j = lane & 31;
  const int hh = lane >> 5;
  const unsigned lds0 = (unsigned)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)cell_smem);

  const int nch_x = REP * (I / HK);
  const int nch = nch_x + (cd.h_prev ? REP * (H / HK) : 0);
  if (rb * HROWS >= Bc) return;  // a row block past the live rows of this step
  const bool full = rb * HROWS + HROWS <= Bc;

  // ---- copies: per chunk a wave issues ACT_COPIES activation copies (16 rows each, row lane/4) and 2 weight
  // copies (1 KB = 4 or 2 weight rows each)
  const unsigned a_lane_chunk = (unsigned)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  constexpr int LPR = ROWB / 16;  // lanes per weight row
  // weight copy g = 2*wave + i covers k rows g*(64/LPR) + lane/LPR; the lane's slot lane%LPR holds chunk
  // slot ^ ((k & 3) << 2), chunk 4*ug + q = gate q of units 8*ug .. +8 of the block
  unsigned w_lane_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const unsigned krow = (unsigned)((2 * wave + i) * (64 / LPR) + lane / LPR);
    const unsigned chunk = ((unsigned)lane % LPR) ^ ((krow & 3) << 2);
    w_lane_off[i] = ((unsigned)(lane / LPR) * (unsigned)(4 * H) + (chunk & 3) * (unsigned)H + (chunk >> 2) * 8) * 2;
  }

  auto issue = [&](int ch, int stage) __attribute__((always_inline)) {
    const _Float16* src;
    int ld, k0;
    if constexpr (SPLIT) {
      const bool in_x = ch < nch_x;
      const int v = in_x ? ch : ch - nch_x;
      const int width = in_x ? I : H;
      src = in_x ? cd.x : cd.h_prev;
      ld = 2 * width;
      k0 = (v / 3) * HK + (v % 3 == 2 ? width : 0);  // third pass of a chunk: the remainder plane
    } else if (ch < nch_x) {
      src = cd.x; ld = I; k0 = ch * HK;
    } else {
      src = cd.h_prev; ld = H; k0 = (ch - nch_x) * HK;
    }
    const int row0 = wave * 16 * ACT_COPIES;  // first of the wave's rows within the block
    const unsigned act_lds = lds0 + (unsigned)(stage * H_STAGE + row0 * 64);
    if (full) {
      const char* base = reinterpret_cast<const char*>(src + (size_t)(rb * HROWS + row0) * ld + k0);
      const unsigned off = ((unsigned)lane >> 2) * (unsigned)(2 * ld) + a_lane_chunk;
#pragma unroll
      for (int i = 0; i < ACT_COPIES; ++i) cell_dma16(base + (size_t)i * 32 * ld, off, act_lds + 1024u * i);
    } else {  // rows past the end of the batch repeat the last row; they are never stored
      const char* base = reinterpret_cast<const char*>(src + k0);
#pragma unroll
      for (int i = 0; i < ACT_COPIES; ++i) {
        const int row = min(rb * HROWS + row0 + 16 * i + (lane >> 2), Bc - 1);
        cell_dma16(base, (unsigned)row * (unsigned)(2 * ld) + a_lane_chunk, act_lds + 1024u * i);
      }
    }
    const unsigned w_lds = lds0 + (unsigned)(stage * H_STAGE + H_ACT_BYTES + wave * 2048);
    if constexpr (PACKED) {
      const char* wbase = reinterpret_cast<const char*>(cd.WU) + ((size_t)ub * REP * (I + H) + ch * HK) * ROWB + wave * 2048;
#pragma unroll
      for (int i = 0; i < 2; ++i) cell_dma16(wbase + 1024 * i, 16u * lane, w_lds + 1024u * i);
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const char* wbase = reinterpret_cast<const char*>(
            cd.WU + (size_t)(ch * HK + (2 * wave + i) * (64 / LPR)) * 4 * H + ub * UB);
        cell_dma16(wbase, w_lane_off[i], w_lds + 1024u * i);
      }
    }
  };

  // ---- fragment addresses within a stage
  unsigned a_off[2], w_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_off[ks] = (unsigned)((128 * wr + j) * 64 + (((2 * ks + hh) ^ ((j >> 2) & 3)) * 16));
  {
    const int ta = (lane & 15) >> 2, tb = lane & 3, th = (lane >> 4) & 1;
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2)
      w_off[u2] = (unsigned)(H_ACT_BYTES + (8 * hh + ta) * ROWB +
                             (((4 * (2 * wc + u2) + 2 * th + (tb >> 1)) ^ (ta << 2)) * 16) + 8 * (tb & 1));
  }

  v16f acc[4][2];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][u2][r] = 0.0f;

  // split flavour: the sums of the x chunks are in the x rows' scale; this brings them to the h rows'
  auto rescale_x = [&]() __attribute__((always_inline)) {
    if (!cd.xratio) return;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const float ratio = cd.xratio[min(rb * HROWS + 128 * wr + 32 * rt + j, Bc - 1)];
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rt][u2][r] *= ratio;
    }
  };

  constexpr int S = cell_stages(UB);
  constexpr int CPC = ACT_COPIES + 2;  // copies per wave and chunk
#pragma unroll
  for (int c = 0; c < S - 1; ++c)
    if (c < nch) issue(c, c);
  int stage = 0;
  for (int ch = 0; ch < nch; ++ch) {
    // copies complete in order: chunk ch has landed when no more are outstanding than were issued after it
    static_assert(S >= 3 && S <= 6, "wait counts below");
    switch (min(S - 2, nch - 1 - ch)) {
      case 0: __builtin_amdgcn_s_waitcnt(vmcnt_only(0)); break;
      case 1: __builtin_amdgcn_s_waitcnt(vmcnt_only(CPC)); break;
      case 2: __builtin_amdgcn_s_waitcnt(vmcnt_only(2 * CPC)); break;
      case 3: __builtin_amdgcn_s_waitcnt(vmcnt_only(3 * CPC)); break;
      default: __builtin_amdgcn_s_waitcnt(vmcnt_only(4 * CPC)); break;
    }
    __syncthreads();  // chunk ch is complete, and every wave is done with the stage of chunk ch-1
    const unsigned char* sb = cell_smem + stage * H_STAGE;
    // all fragments of the chunk are requested up front, the copies of chunk ch + 2 issued while they travel
    v8h wf[2][2], af[2][4];
    auto read_frags = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2) {
        const unsigned char* p0 = sb + w_off[u2] + 16 * ROWB * ks;
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 4 * ROWB));
        const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        wf[ks][u2] = __builtin_bit_cast(v8h, both);
      }
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) af[ks][rt] = *reinterpret_cast<const v8h*>(sb + a_off[ks] + 2048 * rt);
    };
    read_frags(0);
    __builtin_amdgcn_sched_barrier(0);
    if (ch + S - 1 < nch) issue(ch + S - 1, stage == 0 ? S - 1 : stage - 1);
    __builtin_amdgcn_sched_barrier(0);
    read_frags(1);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (SPLIT) {
      if (ch == nch_x) rescale_x();
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int u2 = 0; u2 < 2; ++u2)
          acc[rt][u2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[ks][u2], af[ks][rt], acc[rt][u2], 0, 0, 0);
    stage = stage == S - 1 ? 0 : stage + 1;
  }
  if constexpr (SPLIT) {
    if (nch == nch_x) rescale_x();  // zero state: there was no h chunk to do it before
  }

  // Epilogue: lane (row j, half hh) holds the four gates of units 4*hh .. 4*hh+3 of each of its unit groups.
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int row_g = rb * HROWS + 128 * wr + 32 * rt + j;
    if (row_g >= Bc) continue;
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2) {
      const int u0 = ub * UB + 8 * (2 * wc + u2) + 4 * hh;
      if constexpr (GEMM) {
        _Float16* crow = reinterpret_cast<_Float16*>(cd.h) + (size_t)row_g * 4 * H + u0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v4h o = {(_Float16)acc[rt][u2][4 * q], (_Float16)acc[rt][u2][4 * q + 1], (_Float16)acc[rt][u2][4 * q + 2],
                         (_Float16)acc[rt][u2][4 * q + 3]};
          *reinterpret_cast<v4h*>(crow + (size_t)q * H) = o;
        }
        continue;
      }
      v4f cp = {0, 0, 0, 0};
      if (cd.c_prev) {
        if constexpr (SPLIT) {
          cp = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(cd.c_prev) + (size_t)row_g * H + u0);
        } else {
          const v4h c16 = *reinterpret_cast<const v4h*>(reinterpret_cast<const _Float16*>(cd.c_prev) + (size_t)row_g * H + u0);
          cp = v4f{(float)c16[0], (float)c16[1], (float)c16[2], (float)c16[3]};
        }
      }
      v4f bi = {0, 0, 0, 0}, bf = bi, bo = bi, bg = bi;
      if (cd.bias) {
        bi = *reinterpret_cast<const v4f*>(cd.bias + u0);
        bf = *reinterpret_cast<const v4f*>(cd.bias + H + u0);
        bo = *reinterpret_cast<const v4f*>(cd.bias + 2 * H + u0);
        bg = *reinterpret_cast<const v4f*>(cd.bias + 3 * H + u0);
      }
      v4f si = {1, 1, 1, 1}, sf = si, so = si, sg = si;
      if constexpr (SPLIT) {
        si = *reinterpret_cast<const v4f*>(cd.wscale + u0);
        sf = *reinterpret_cast<const v4f*>(cd.wscale + H + u0);
        so = *reinterpret_cast<const v4f*>(cd.wscale + 2 * H + u0);
        sg = *reinterpret_cast<const v4f*>(cd.wscale + 3 * H + u0);
      }
      v4f hn, cn;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float ig = sigmoid_f(acc[rt][u2][r] * si[r] + bi[r]);
        const float fg = sigmoid_f(acc[rt][u2][4 + r] * sf[r] + bf[r]);
        const float og = sigmoid_f(acc[rt][u2][8 + r] * so[r] + bo[r]);
        const float cand = tanh_f(acc[rt][u2][12 + r] * sg[r] + bg[r]);
        cn[r] = fg * cp[r] + ig * cand;
        hn[r] = og * tanh_f(cn[r]);
      }
      if constexpr (SPLIT) {
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(cd.c) + (size_t)row_g * H + u0) = cn;
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(cd.h) + (size_t)row_g * H + u0) = hn;
        v4h top, rest;
        unsigned largest = 0;   // of the lane's four neighbouring units
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float hs = hn[r] * 16384.0f;  // |h| < 1: 2^14 keeps the value plane below 2^14
          top[r] = (_Float16)hs;
          rest[r] = (_Float16)(hs - (float)top[r]);
          largest = max(largest, __float_as_uint(hs) & 0x7fffffffu);
        }
        if (largest - 1u < kSmallStateStreamedBits - 1u && list.small_states) *list.small_states = 1;   // same word, same value: one transaction per wave
        _Float16* hp = cd.h_planes + (size_t)row_g * 2 * H + u0;
        *reinterpret_cast<v4h*>(hp) = top;
        *reinterpret_cast<v4h*>(hp + H) = rest;
      } else {
        v4h hv, cv;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          cv[r] = (_Float16)cn[r];
          hv[r] = (_Float16)hn[r];
        }
        *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(cd.c) + (size_t)row_g * H + u0) = cv;
        *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(cd.h) + (size_t)row_g * H + u0) = hv;
      }
    }
  }
}

// ------------------------------------------------ split flavour, four tiles per chunk
// The split products of a chunk from one copy of each plane: a stage holds the four tiles [x value][x
// remainder][w value][w remainder] of a 32-row chunk (64 KB at 64 hidden units per workgroup), and the three
// products (w value, x value), (w remainder, x value), (w value, x remainder) are formed from them: two thirds of
// the copies and of the LDS fragment reads of the three-chunks-in-a-row form above.  Two stages (128 KB): the
// next chunk is copied while this one is used, 48 MFMAs per wave.  8 waves, the wave tiling and every LDS layout
// as in lstm_cell_f16_kernel<true, 8, true>; packed weights as [chunk][plane][32 rows][512 bytes] per unit block
// (lstm_pack_split_weights_kernel with planes = 2).
constexpr int S4_TILE = 16384;
constexpr int S4_STAGE = 4 * S4_TILE;
constexpr size_t kSplit4Lds = 2 * S4_STAGE;

__global__ __launch_bounds__(512, 1) void lstm_cell_split4_kernel(CellListH list, int B, int I, int H) {
  constexpr int UB = 64, ROWB = 512;
  extern __shared__ __attribute__((aligned(1024))) unsigned char cell_smem[];
  using lds_v4s = __attribute__((address_space(3))) v4s;

  const int nub = H / UB, nrb = (B + HROWS - 1) / HROWS;
  const int slot = blockIdx.x >> 3;
  const int cell = (blockIdx.x & 7) + 8 * (slot / (nub * nrb));  // all workgroups of a cell on one XCD
  if (cell >= list.n) return;
  const CellDescH cd = list.cells[cell];
  const int Bc = cd.rows > 0 ? cd.rows : B;  // rows of this cell
  const int ub = slot % nub;
  const int rb = (slot / nub) % nrb;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wr = wave >> 2;  // rows 128*wr .. +128 of the block
  const int wc = wave & 3;   // unit groups 2*wc, 2*wc+1 of the block's eight
  const int j = lane & 31;
  const int hh = lane >> 5;
  const unsigned lds0 = (unsigned)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)cell_smem);

  const int nch_x = I / HK;
  const int nch = nch_x + (cd.h_prev ? H / HK : 0);
  if (rb * HROWS >= Bc) return;  // a row block past the live rows of this step
  const bool full = rb * HROWS + HROWS <= Bc;

  // per chunk a wave issues 2 + 2 activation copies (rows 32*wave + 16 i + lane/4 of each plane) and 2 + 2
  // weight copies (1 KB = rows 4*wave + 2 i + lane/32 of each plane, already in LDS order)
  const unsigned a_lane_chunk = (unsigned)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  auto issue = [&](int ch, int stage) __attribute__((always_inline)) {
    const bool in_x = ch < nch_x;
    const int width = in_x ? I : H;
    const _Float16* src = (in_x ? cd.x : cd.h_prev) + (in_x ? ch : ch - nch_x) * HK;
    const int ld = 2 * width;
    const int row0 = wave * 32;
    const unsigned st = lds0 + (unsigned)(stage * S4_STAGE);
#pragma unroll
    for (int pl = 0; pl < 2; ++pl) {
      const unsigned act_lds = st + (unsigned)(pl * S4_TILE + row0 * 64);
      if (full) {
        const char* base = reinterpret_cast<const char*>(src + pl * width + (size_t)(rb * HROWS + row0) * ld);
        const unsigned off = ((unsigned)lane >> 2) * (unsigned)(2 * ld) + a_lane_chunk;
#pragma unroll
        for (int i = 0; i < 2; ++i) cell_dma16(base + (size_t)i * 32 * ld, off, act_lds + 1024u * i);
      } else {  // rows past the end of the batch repeat the last row; they are never stored
        const char* base = reinterpret_cast<const char*>(src + pl * width);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int row = min(rb * HROWS + row0 + 16 * i + (lane >> 2), Bc - 1);
          cell_dma16(base, (unsigned)row * (unsigned)(2 * ld) + a_lane_chunk, act_lds + 1024u * i);
        }
      }
    }
    const char* wbase = reinterpret_cast<const char*>(cd.WU) + ((size_t)ub * (I + H) + ch * HK) * 2 * ROWB + wave * 2048;
#pragma unroll
    for (int pl = 0; pl < 2; ++pl)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        cell_dma16(wbase + pl * S4_TILE + 1024 * i, 16u * lane, st + (unsigned)((2 + pl) * S4_TILE + wave * 2048 + 1024 * i));
  };

  unsigned a_off[2], w_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_off[ks] = (unsigned)((128 * wr + j) * 64 + (((2 * ks + hh) ^ ((j >> 2) & 3)) * 16));
  {
    const int ta = (lane & 15) >> 2, tb = lane & 3, th = (lane >> 4) & 1;
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2)
      w_off[u2] = (unsigned)(2 * S4_TILE + (8 * hh + ta) * ROWB +
                             (((4 * (2 * wc + u2) + 2 * th + (tb >> 1)) ^ (ta << 2)) * 16) + 8 * (tb & 1));
  }

  v16f acc[4][2];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][u2][r] = 0.0f;

  auto rescale_x = [&]() __attribute__((always_inline)) {
    if (!cd.xratio) return;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const float ratio = cd.xratio[min(rb * HROWS + 128 * wr + 32 * rt + j, Bc - 1)];
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rt][u2][r] *= ratio;
    }
  };

  issue(0, 0);
  for (int ch = 0; ch < nch; ++ch) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __syncthreads();  // chunk ch is complete, and every wave is done with the stage of chunk ch-1
    const unsigned char* sb = cell_smem + (ch & 1) * S4_STAGE;
    if (ch + 1 < nch) issue(ch + 1, (ch + 1) & 1);
    if (ch == nch_x) rescale_x();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      v8h wt[2], wre[2];
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2) {
#pragma unroll
        for (int pl = 0; pl < 2; ++pl) {
          const unsigned char* p0 = sb + w_off[u2] + pl * S4_TILE + 16 * ROWB * ks;
          const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
          const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 4 * ROWB));
          const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          (pl ? wre[u2] : wt[u2]) = __builtin_bit_cast(v8h, both);
        }
      }
      v8h at[4], ar[4];
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        at[rt] = *reinterpret_cast<const v8h*>(sb + a_off[ks] + 2048 * rt);
        ar[rt] = *reinterpret_cast<const v8h*>(sb + S4_TILE + a_off[ks] + 2048 * rt);
      }
      // product by product, so that the MFMAs that add into one accumulator are eight apart
#pragma unroll
      for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int u2 = 0; u2 < 2; ++u2) acc[rt][u2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wt[u2], at[rt], acc[rt][u2], 0, 0, 0);
#pragma unroll
      for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int u2 = 0; u2 < 2; ++u2) acc[rt][u2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wre[u2], at[rt], acc[rt][u2], 0, 0, 0);
#pragma unroll
      for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int u2 = 0; u2 < 2; ++u2) acc[rt][u2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wt[u2], ar[rt], acc[rt][u2], 0, 0, 0);
    }
  }
  if (nch == nch_x) rescale_x();  // zero state: there was no h chunk to do it before

#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int row_g = rb * HROWS + 128 * wr + 32 * rt + j;
    if (row_g >= Bc) continue;
#pragma unroll
    for (int u2 = 0; u2 < 2; ++u2) {
      const int u0 = ub * UB + 8 * (2 * wc + u2) + 4 * hh;
      v4f cp = {0, 0, 0, 0};
      if (cd.c_prev) cp = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(cd.c_prev) + (size_t)row_g * H + u0);
      v4f bi = {0, 0, 0, 0}, bf = bi, bo = bi, bg = bi;
      if (cd.bias) {
        bi = *reinterpret_cast<const v4f*>(cd.bias + u0);
        bf = *reinterpret_cast<const v4f*>(cd.bias + H + u0);
        bo = *reinterpret_cast<const v4f*>(cd.bias + 2 * H + u0);
        bg = *reinterpret_cast<const v4f*>(cd.bias + 3 * H + u0);
      }
      const v4f si = *reinterpret_cast<const v4f*>(cd.wscale + u0);
      const v4f sf = *reinterpret_cast<const v4f*>(cd.wscale + H + u0);
      const v4f so = *reinterpret_cast<const v4f*>(cd.wscale + 2 * H + u0);
      const v4f sg = *reinterpret_cast<const v4f*>(cd.wscale + 3 * H + u0);
      v4f hn, cn;
      v4h top, rest;
      unsigned largest = 0;   // of the lane's four neighbouring units
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float ig = sigmoid_f(acc[rt][u2][r] * si[r] + bi[r]);
        const float fg = sigmoid_f(acc[rt][u2][4 + r] * sf[r] + bf[r]);
        const float og = sigmoid_f(acc[rt][u2][8 + r] * so[r] + bo[r]);
        const float cand = tanh_f(acc[rt][u2][12 + r] * sg[r] + bg[r]);
        cn[r] = fg * cp[r] + ig * cand;
        hn[r] = og * tanh_f(cn[r]);
        const float hs = hn[r] * 16384.0f;
        top[r] = (_Float16)hs;
        rest[r] = (_Float16)(hs - (float)top[r]);
        largest = max(largest, __float_as_uint(hs) & 0x7fffffffu);
      }
      if (largest - 1u < kSmallStateStreamedBits - 1u && list.small_states) *list.small_states = 1;   // same word, same value: one transaction per wave
      *reinterpret_cast<v4f*>(reinterpret_cast<float*>(cd.c) + (size_t)row_g * H + u0) = cn;
      *reinterpret_cast<v4f*>(reinterpret_cast<float*>(cd.h) + (size_t)row_g * H + u0) = hn;
      _Float16* hp = cd.h_planes + (size_t)row_g * 2 * H + u0;
      *reinterpret_cast<v4h*>(hp) = top;
      *reinterpret_cast<v4h*>(hp + H) = rest;
    }
  }
}

static int launch_cells(const CellList& list, int B, int I, int H, hipStream_t s) {
  dim3 grid(H / 32, (B + 31) / 32, list.n);
  hipLaunchKernelGGL(lstm_cell_kernel, grid, dim3(256), 0, s, list, B, I, H);
  return check_launch("lstm_cell_kernel");
}

// WU [n_layers, K2, 4H] -> per layer and block ub of UB hidden units the [K2][4*UB] tile the cell kernel keeps
// in LDS: row k holds chunks of 8 columns, chunk 4*ug + q = gate q of units UB*ub + 8*ug .. +8, stored in slot
// chunk ^ ((k & 3) << 2).  One thread per 16-byte chunk.
__global__ __launch_bounds__(256) void lstm_pack_weights_f16_kernel(const _Float16* __restrict__ WU,
                                                                    _Float16* __restrict__ packed, size_t chunks,
                                                                    int K2, int H, int UB) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= chunks) return;
  const int per_row = H / 2;  // 4H / 8
  const int n8 = (int)(idx % per_row);
  const size_t lk = idx / per_row;
  const int k = (int)(lk % K2);
  const size_t l = lk / K2;
  const int col = 8 * n8;
  const int q = col / H, u = col % H;
  const int ub = u / UB, ug = (u % UB) >> 3;
  const int slot = (4 * ug + q) ^ ((k & 3) << 2);
  const v4u v = *reinterpret_cast<const v4u*>(WU + idx * 8);
  *reinterpret_cast<v4u*>(packed + ((l * (H / UB) + ub) * K2 + k) * (4 * UB) + 8 * slot) = v;
}

// Hidden units per workgroup of the streaming kernel at hidden size H.
static int cell_unit_block(int H) { return H % 64 == 0 ? 64 : 32; }

int pack_weights_f16(const void* WU, void* packed, int layers, int K2, int H, hipStream_t s) {
  const size_t chunks = (size_t)layers * K2 * (H / 2);
  hipLaunchKernelGGL(lstm_pack_weights_f16_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s,
                     (const _Float16*)WU, (_Float16*)packed, chunks, K2, H, cell_unit_block(H));
  return check_launch("lstm_pack_weights_f16_kernel");
}

template <bool PACKED, int WAVES, bool SPLIT, bool GEMM = false>
static int launch_cells_f16(const CellListH& list, int B, int I, int H, hipStream_t s) {
  static DeviceOnce attr_once;
  constexpr int UB = 8 * WAVES;
  const void* fn = (const void*)lstm_cell_f16_kernel<PACKED, WAVES, SPLIT, GEMM>;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)cell_lds_bytes(UB)));
    attr_once.done(attr_bit);
  }
  const int groups = (list.n + 7) / 8;  // cells per XCD
  dim3 grid((GEMM ? list.n : 8 * groups) * (H / UB) * ((B + HROWS - 1) / HROWS));
  hipLaunchKernelGGL((lstm_cell_f16_kernel<PACKED, WAVES, SPLIT, GEMM>), grid, dim3(WAVES * 64), cell_lds_bytes(UB), s, list,
                     B, I, H);
  return check_launch("lstm_cell_f16_kernel");
}

static int launch_cells(const CellListH& list, int B, int I, int H, hipStream_t s) {
  if (list.packed == 3) {  // split products, four tiles per chunk
    static DeviceOnce attr_once;
    unsigned attr_bit;
    if (attr_once.pending(&attr_bit)) {
      FTK_HIP(hipFuncSetAttribute((const void*)lstm_cell_split4_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kSplit4Lds));
      attr_once.done(attr_bit);
    }
    const int groups = (list.n + 7) / 8;
    dim3 grid(8 * groups * (H / 64) * ((B + HROWS - 1) / HROWS));
    hipLaunchKernelGGL(lstm_cell_split4_kernel, grid, dim3(512), kSplit4Lds, s, list, B, I, H);
    return check_launch("lstm_cell_split4_kernel");
  }
  if (list.packed == 2)  // split products, three chunks in a row
    return cell_unit_block(H) == 64 ? launch_cells_f16<true, 8, true>(list, B, I, H, s)
                                    : launch_cells_f16<true, 4, true>(list, B, I, H, s);
  if (cell_unit_block(H) == 64)
    return list.packed ? launch_cells_f16<true, 8, false>(list, B, I, H, s) : launch_cells_f16<false, 8, false>(list, B, I, H, s);
  return list.packed ? launch_cells_f16<true, 4, false>(list, B, I, H, s) : launch_cells_f16<false, 4, false>(list, B, I, H, s);
}

// Host side of the per-stage schedule: stage(l,t) = 1 + max(stage(l-1,t),
// stage(l,t-d_l)); cells of equal stage are independent and go out as one
// batched launch.  For d = 1 the stages are the diagonals l + t.
static void set_packed(CellList&, bool) {}
static void set_packed(CellListH& list, bool packed) { list.packed = packed; }

static std::vector<std::vector<int>> cells_by_stage(int L, int T, const int* dil) {
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
  return by_stage;
}

static void set_rows(CellDesc&, int) {}
static void set_rows(CellDescH& cd, int rows) { cd.rows = rows; }

template <typename Elem, typename List>
static int run_wavefront_of(const Elem* xs, const Elem* WU, const float* bias, const int* dil, Elem* hsss, Elem* csss,
                            int L, int T, int B, int H, hipStream_t s, bool packed = false, const int* active = nullptr) {
  const std::vector<std::vector<int>> by_stage = cells_by_stage(L, T, dil);

  const size_t cell = (size_t)B * H;
  for (const auto& cells : by_stage) {
    size_t pos = 0;
    while (pos < cells.size()) {
      List list;
      list.n = 0;
      set_packed(list, packed);
      while (pos < cells.size() && list.n < kMaxCellsPerLaunch) {
        const int l = cells[pos] / T, t = cells[pos] % T;
        const int d = dil ? dil[l] : 1;
        auto& cd = list.cells[list.n++];
        cd.x = (l == 0) ? xs + (size_t)t * cell : hsss + ((size_t)(l - 1) * T + t) * cell;
        cd.h_prev = (t >= d) ? hsss + ((size_t)l * T + t - d) * cell : nullptr;
        cd.c_prev = (t >= d) ? csss + ((size_t)l * T + t - d) * cell : nullptr;
        cd.WU = WU + (size_t)l * 2 * H * 4 * H;
        cd.bias = bias ? bias + (size_t)l * 4 * H : nullptr;
        cd.h = hsss + ((size_t)l * T + t) * cell;
        cd.c = csss + ((size_t)l * T + t) * cell;
        set_rows(cd, active ? active[t] : 0);
        if (active && active[t] == 0) --list.n;  // nothing lives at this step
        ++pos;
      }
      if (list.n == 0) continue;
      int rc = launch_cells(list, B, H, H, s);
      if (rc) return rc;
    }
  }
  return FTK_OK;
}

int run_wavefront(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss, float* csss,
                  int L, int T, int B, int H, hipStream_t s) {
  return run_wavefront_of<float, CellList>(xs, WU, bias, dil, hsss, csss, L, T, B, H, s);
}

// The same schedule over fp16 arrays (H a multiple of 32).  packed: a buffer of the size of WU, into which the
// weights are first re-laid per unit block, or nullptr to read WU as it is.
int run_wavefront_f16(const void* xs, const void* WU, const float* bias, const int* dil, const int* active, void* hsss,
                      void* csss, int L, int T, int B, int H, void* packed, hipStream_t s) {
  if (packed) {
    int rc = pack_weights_f16(WU, packed, L, 2 * H, H, s);
    if (rc) return rc;
  }
  return run_wavefront_of<_Float16, CellListH>((const _Float16*)xs, (const _Float16*)(packed ? packed : WU), bias, dil,
                                               (_Float16*)hsss, (_Float16*)csss, L, T, B, H, s, packed != nullptr, active);
}

// ------------------------------------------------- fp32 stack on split products
constexpr int kSplitTopExp = 14;  // a group's largest magnitude is scaled into [2^14, 2^15)

// The power of two that brings a group maximum m into [2^14, 2^15), and its biased exponent (clamped so that
// every scale and inverse scale derived from it is a normal fp32 number).
__device__ __forceinline__ float split_scale(float m, int* biased_exp) {
  const int eb = min(max((int)((__float_as_uint(m) >> 23) & 0xff), 40), 230);
  *biased_exp = eb;
  return __uint_as_float((unsigned)(127 + kSplitTopExp + 127 - eb) << 23);
}

// Rows of xs [rows, I] -> [rows, 2I] = [value plane | remainder plane] under the row's own scale, and the factor
// 2^(eb - 127) that turns sums of such a row's products into the h rows' 2^14 scale.  One wave per row.
__global__ __launch_bounds__(256) void lstm_split_rows_any_kernel(const float* __restrict__ xs, _Float16* __restrict__ xp,
                                                                  float* __restrict__ xratio, int rows, int I) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* src = xs + (size_t)row * I;
  float m = 0.0f;
  for (int k = 4 * lane; k < I; k += 256) {
    const float4 v = *reinterpret_cast<const float4*>(src + k);
    m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  int eb;
  const float scale = split_scale(m, &eb);
  _Float16* dst = xp + (size_t)row * 2 * I;
  for (int k = 4 * lane; k < I; k += 256) {
    const float4 v = *reinterpret_cast<const float4*>(src + k);
    const float vs[4] = {v.x * scale, v.y * scale, v.z * scale, v.w * scale};
    v4h top, rest;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      top[r] = (_Float16)vs[r];
      rest[r] = (_Float16)(vs[r] - (float)top[r]);
    }
    *reinterpret_cast<v4h*>(dst + k) = top;
    *reinterpret_cast<v4h*>(dst + I + k) = rest;
  }
  if (lane == 0) xratio[row] = __uint_as_float((unsigned)eb << 23);
}

// Per layer and weight column: the scale its values are split under (wmul) and what undoes it together with
// the h rows' 2^14 after the sums (wscale).  One thread per column; neighbouring threads read neighbouring columns.
__global__ __launch_bounds__(256) void lstm_col_scale_kernel(const float* __restrict__ WU, float* __restrict__ wmul,
                                                             float* __restrict__ wscale, int layers, int K2, int N4) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)layers * N4) return;
  const size_t l = idx / N4;
  const int n = (int)(idx % N4);
  const float* col = WU + l * K2 * N4 + n;
  float m = 0.0f;
  for (int k = 0; k < K2; ++k) m = fmaxf(m, fabsf(col[(size_t)k * N4]));
  int eb;
  wmul[idx] = split_scale(m, &eb);
  wscale[idx] = __uint_as_float((unsigned)(eb - 2 * kSplitTopExp) << 23);  // 2^-(14 + 14 + 127 - eb)
}

// WU [layers, 2H, 4H] fp32 -> the packed rows of the split flavour: per layer and block of UB hidden units a
// [6H][4*UB] fp16 tile in the kernel's LDS chunk order (see lstm_pack_weights_f16_kernel), where chunk c of 32 k
// rows of the x half (then of the h half) appears three times: value plane, remainder plane, value plane.
__global__ __launch_bounds__(256) void lstm_pack_split_weights_kernel(const float* __restrict__ WU,
                                                                      const float* __restrict__ wmul,
                                                                      _Float16* __restrict__ packed, size_t chunks, int H,
                                                                      int UB, int planes) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= chunks) return;
  const int per_row = H / 2;  // 4H / 8
  const int K2 = 2 * H;
  const int n8 = (int)(idx % per_row);
  const size_t lk = idx / per_row;
  const int k = (int)(lk % K2);
  const size_t l = lk / K2;
  const int col = 8 * n8;
  const int q = col / H, u = col % H;
  const int ub = u / UB, ug = (u % UB) >> 3;
  const int part = k / H, kk = k % H;
  const float* src = WU + idx * 8;
  const float* mul = wmul + l * 4 * H + col;
  v8h top, rest;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const float vs = src[r] * mul[r];
    top[r] = (_Float16)vs;
    rest[r] = (_Float16)(vs - (float)top[r]);
  }
  const int slot = (4 * ug + q) ^ ((kk & 3) << 2);
  // planes = 3: value, remainder, value again (three chunks in a row); planes = 2: value, remainder
  const size_t vrow0 = (size_t)part * planes * H + (size_t)(kk / 32) * (32 * planes) + (kk % 32);
  _Float16* base = packed + (l * (H / UB) + ub) * (size_t)(2 * planes * H) * (4 * UB) + 8 * slot;
  *reinterpret_cast<v8h*>(base + vrow0 * (4 * UB)) = top;
  *reinterpret_cast<v8h*>(base + (vrow0 + 32) * (4 * UB)) = rest;
  if (planes == 3) *reinterpret_cast<v8h*>(base + (vrow0 + 64) * (4 * UB)) = top;
}

static size_t round256s(size_t v) { return (v + 255) / 256 * 256; }

// Workspace of the split-product stack: [status block][wscale L*4H][wmul L*4H][xratio T*B] floats, then fp16
// [xp T*B*2H][hp L*T*B*2H][packed weights L*6H*4H], every part on a 256-byte boundary.
size_t split_stack_workspace_bytes(int L, int T, int B, int H) {
  size_t n = kStatusBytes + 2 * round256s((size_t)L * 4 * H * sizeof(float)) + round256s((size_t)T * B * sizeof(float));
  n += round256s((size_t)T * B * 2 * H * sizeof(_Float16)) + round256s((size_t)L * T * B * 2 * H * sizeof(_Float16));
  n += (size_t)L * 6 * H * 4 * H * sizeof(_Float16);
  return n;
}

// The fp32 stack through the split flavour of the streaming cell kernel (H a multiple of 32).
int run_wavefront_split(const float* xs, const float* WU, const float* bias, const int* dil, const int* active, float* hsss,
                        float* csss, int L, int T, int B, int H, void* ws, hipStream_t s) {
  char* p = reinterpret_cast<char*>(ws) + kStatusBytes;
  float* wscale = reinterpret_cast<float*>(p);
  p += round256s((size_t)L * 4 * H * sizeof(float));
  float* wmul = reinterpret_cast<float*>(p);
  p += round256s((size_t)L * 4 * H * sizeof(float));
  float* xratio = reinterpret_cast<float*>(p);
  p += round256s((size_t)T * B * sizeof(float));
  _Float16* xp = reinterpret_cast<_Float16*>(p);
  p += round256s((size_t)T * B * 2 * H * sizeof(_Float16));
  _Float16* hp = reinterpret_cast<_Float16*>(p);
  p += round256s((size_t)L * T * B * 2 * H * sizeof(_Float16));
  _Float16* wp = reinterpret_cast<_Float16*>(p);

  const int UB = cell_unit_block(H);
  // 64 hidden units per workgroup: every plane copied once per chunk (four tiles); else three chunks in a row
  const bool four_tiles = UB == 64 && !getenv("FTK_LSTM_SPLIT_ROWS3");
  const int planes = four_tiles ? 2 : 3;
  const size_t cols = (size_t)L * 4 * H;
  hipLaunchKernelGGL(lstm_col_scale_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, s, WU, wmul, wscale, L,
                     2 * H, 4 * H);
  int rc = check_launch("lstm_col_scale_kernel");
  if (rc) return rc;
  const size_t chunks = (size_t)L * 2 * H * (H / 2);
  hipLaunchKernelGGL(lstm_pack_split_weights_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, WU, wmul, wp,
                     chunks, H, UB, planes);
  rc = check_launch("lstm_pack_split_weights_kernel");
  if (rc) return rc;
  const int rows = T * B;
  hipLaunchKernelGGL(lstm_split_rows_any_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, xs, xp, xratio, rows, H);
  rc = check_launch("lstm_split_rows_any_kernel");
  if (rc) return rc;

  const size_t cell = (size_t)B * H;
  for (const auto& cells : cells_by_stage(L, T, dil)) {
    size_t pos = 0;
    while (pos < cells.size()) {
      CellListH list;
      list.n = 0;
      list.packed = four_tiles ? 3 : 2;
      list.small_states = reinterpret_cast<int*>(ws) + 1;
      while (pos < cells.size() && list.n < kMaxCellsPerLaunch) {
        const int l = cells[pos] / T, t = cells[pos] % T;
        const int d = dil ? dil[l] : 1;
        CellDescH& cd = list.cells[list.n++];
        cd.x = (l == 0) ? xp + (size_t)t * 2 * cell : hp + ((size_t)(l - 1) * T + t) * 2 * cell;
        cd.h_prev = (t >= d) ? hp + ((size_t)l * T + t - d) * 2 * cell : nullptr;
        cd.c_prev = (t >= d) ? csss + ((size_t)l * T + t - d) * cell : nullptr;
        cd.WU = wp + (size_t)l * 2 * planes * H * 4 * H;
        cd.bias = bias ? bias + (size_t)l * 4 * H : nullptr;
        cd.h = hsss + ((size_t)l * T + t) * cell;
        cd.c = csss + ((size_t)l * T + t) * cell;
        cd.xratio = (l == 0) ? xratio + (size_t)t * B : nullptr;
        cd.wscale = wscale + (size_t)l * 4 * H;
        cd.h_planes = hp + ((size_t)l * T + t) * 2 * cell;
        cd.rows = active ? active[t] : 0;
        if (active && active[t] == 0) --list.n;  // nothing lives at this step
        ++pos;
      }
      if (list.n == 0) continue;
      rc = launch_cells(list, B, H, H, s);
      if (rc) return rc;
    }
  }
  return FTK_OK;
}

}  // namespace ftk

namespace ftk {
// gemm_f16.hip: the product for shapes made of whole 256 x 256 tiles
bool gemm_f16_tiles_fit(int M, int N, int K);
int launch_gemm_f16_tiles(const void* A, const void* Bm, void* C, int G, int M, int N, int K, hipStream_t s);
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

int ftk_lstm_cell_f16(const void* x, const void* h_prev, const void* c_prev, const void* WU, const float* bias,
                      void* h, void* c, int B, int I, int H, ftk_stream_t stream) {
  if (!x || !WU || !h || !c) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f16: x, WU, h, c must be non-NULL");
  if ((h_prev == nullptr) != (c_prev == nullptr))
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f16: h_prev and c_prev must both be given or both be NULL");
  if (B <= 0 || I <= 0 || H <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_cell_f16: B, I, H must be positive");
  if (I % 32 || H % 32)
    return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_lstm_cell_f16: I=%d and H=%d must be multiples of 32", I, H);
  if ((long long)B * std::max(I, H) >= (1ll << 30))
    return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_lstm_cell_f16: B=%d too large", B);
  ftk::CellListH list;
  list.n = 1;
  list.packed = 0;
  list.cells[0] = ftk::CellDescH{(const _Float16*)x, (const _Float16*)h_prev, c_prev, (const _Float16*)WU, bias, h, c,
                                 nullptr, nullptr, nullptr, 0};
  return ftk::launch_cells(list, B, I, H, (hipStream_t)stream);
}

int ftk_lstm_layer_f32(const float* xs, const float* WU, const float* bias, const float* h0, const float* c0, float* hs,
                       float* cs, int T, int B, int I, int H, ftk_stream_t stream) {
  const char* who = "ftk_lstm_layer_f32";
  if (!xs || !WU || !hs || !cs) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: xs, WU, hs, cs must be non-NULL", who);
  if ((h0 == nullptr) != (c0 == nullptr))
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: h0 and c0 must both be given or both be NULL", who);
  if (T <= 0 || B <= 0 || I <= 0 || H <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: T, B, I, H must be positive", who);
  if (I % 32 || H % 32) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: I=%d and H=%d must be multiples of 32", who, I, H);
  if ((B + 31) / 32 > 65535) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: B=%d too large", who, B);
  const size_t cell = (size_t)B * H;
  for (int t = 0; t < T; ++t) {  // one fused-cell launch per step, stream-ordered
    ftk::CellList list;
    list.n = 1;
    list.cells[0] = ftk::CellDesc{xs + (size_t)t * B * I, t ? hs + (t - 1) * cell : h0, t ? cs + (t - 1) * cell : c0,
                                  WU,  bias, hs + t * cell, cs + t * cell};
    int rc = ftk::launch_cells(list, B, I, H, (hipStream_t)stream);
    if (rc) return rc;
  }
  return FTK_OK;
}

int ftk_lstm_layer_f16(const void* xs, const void* WU, const float* bias, const void* h0, const void* c0, void* hs,
                       void* cs, int T, int B, int I, int H, ftk_stream_t stream) {
  const char* who = "ftk_lstm_layer_f16";
  if (!xs || !WU || !hs || !cs) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: xs, WU, hs, cs must be non-NULL", who);
  if ((h0 == nullptr) != (c0 == nullptr))
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: h0 and c0 must both be given or both be NULL", who);
  if (T <= 0 || B <= 0 || I <= 0 || H <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: T, B, I, H must be positive", who);
  if (I % 32 || H % 32) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: I=%d and H=%d must be multiples of 32", who, I, H);
  if ((long long)B * std::max(I, H) >= (1ll << 30)) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: B=%d too large", who, B);
  const _Float16* x16 = (const _Float16*)xs;
  _Float16* h16 = (_Float16*)hs;
  _Float16* c16 = (_Float16*)cs;
  const size_t cell = (size_t)B * H;
  for (int t = 0; t < T; ++t) {
    ftk::CellListH list;
    list.n = 1;
    list.packed = 0;
    list.cells[0] = ftk::CellDescH{x16 + (size_t)t * B * I, t ? h16 + (t - 1) * cell : (const _Float16*)h0,
                                   t ? (const void*)(c16 + (t - 1) * cell) : c0, (const _Float16*)WU, bias, h16 + t * cell,
                                   c16 + t * cell, nullptr, nullptr, nullptr, 0};
    int rc = ftk::launch_cells(list, B, I, H, (hipStream_t)stream);
    if (rc) return rc;
  }
  return FTK_OK;
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

// G products C = A @ Bm through the streaming cell kernel's product: every problem is a "cell" with x = A,
// no state, WU = Bm seen as four column quarters.
static int gemm_f16(const char* who, const void* A, const void* Bm, void* C, int G, int M, int N, int K, hipStream_t s) {
  if (!A || !Bm || !C) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: A, B, C must be non-NULL", who);
  if (G <= 0 || M <= 0 || N <= 0 || K <= 0) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: G, M, N, K must be positive", who);
  if (N % 128 || K % 32) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: N=%d must be a multiple of 128 and K=%d of 32", who, N, K);
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bm) | reinterpret_cast<uintptr_t>(C)) % 16)
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "%s: A, B, C must be 16-byte aligned", who);   // rows are copied and stored 16 bytes at a time
  // N a multiple of 256: the kernel built for the product (gemm_f16.hip); otherwise the cell kernel without the cell
  if (ftk::gemm_f16_tiles_fit(M, N, K)) return ftk::launch_gemm_f16_tiles(A, Bm, C, G, M, N, K, s);
  if ((long long)M * std::max(K, N) >= (1ll << 30)) return ftk::fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: M=%d too large", who, M);
  const int Hq = N / 4;  // a column quarter
  const _Float16* a = (const _Float16*)A;
  const _Float16* b = (const _Float16*)Bm;
  _Float16* c = (_Float16*)C;
  for (int g0 = 0; g0 < G; g0 += ftk::kMaxCellsPerLaunch) {
    ftk::CellListH list;
    list.n = std::min(ftk::kMaxCellsPerLaunch, G - g0);
    list.packed = 0;
    for (int i = 0; i < list.n; ++i) {
      const size_t g = (size_t)(g0 + i);
      list.cells[i] = ftk::CellDescH{a + g * M * K, nullptr, nullptr, b + g * K * N, nullptr, c + g * M * N, nullptr,
                                     nullptr, nullptr, nullptr, 0};
    }
    const int rc = Hq % 64 == 0 ? ftk::launch_cells_f16<false, 8, false, true>(list, M, K, Hq, s)
                                : ftk::launch_cells_f16<false, 4, false, true>(list, M, K, Hq, s);
    if (rc) return rc;
  }
  return FTK_OK;
}

int ftk_gemm_f16(const void* A, const void* B, void* C, int M, int N, int K, ftk_stream_t stream) {
  return gemm_f16("ftk_gemm_f16", A, B, C, 1, M, N, K, (hipStream_t)stream);
}

int ftk_batched_gemm_f16(const void* A, const void* B, void* C, int G, int M, int N, int K, ftk_stream_t stream) {
  return gemm_f16("ftk_batched_gemm_f16", A, B, C, G, M, N, K, (hipStream_t)stream);
}

}  // extern "C"
