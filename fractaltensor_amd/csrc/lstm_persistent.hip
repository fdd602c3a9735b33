// Persistent stacked / dilated LSTM on gfx950.
//
// One launch evaluates every (layer, time) cell.  The grid is one 256-thread
// workgroup per compute unit; a fixed group of workgroups owns each layer for
// the whole launch and keeps its slice of that layer's [W;U] in registers: a
// workgroup holds 128 gate columns (32 hidden units x {i,f,o,c~}), each of its
// four waves 32 of them as up to 256 VGPRs per lane, the MFMA "A" operands.
// H/32 such column slices make a layer; with spare compute units a layer gets
// several row slices as well, each handling its own subset of the batch's
// 32-row blocks.  Four flavours share the code (see the constants below):
// fp32 data at H = 256 with fp32 MFMAs or with every fp32 product formed as
// three fp16 MFMAs of split operands, and fp16 data at H = 512 and H = 256.
//
// Work item = (t, row block).  For an item the workgroup stages the activation
// tile [32, x_t | h_{t-d}] in LDS, runs the product against the resident
// weights, applies bias, sigmoid/tanh and the state update in registers (all
// four gates of a (row, unit) pair land in one lane, see lstm_cell.hip) and
// writes h, c.  Batch rows never interact, so dependencies are per row block:
// item (l, t, rb) needs h[l-1][t][rb] from the layer below and h[l][t-d][rb]
// from all column slices of its own layer.  Layer l therefore trails layer
// l-1 by an item or two: the wavefront of the reference's region schedule,
// without launches, device syncs or scatter.
//
// Hand-off between compute units (which may sit on different XCDs, whose L2
// caches are not coherent with each other) uses no cache-wide fences: what
// other compute units read is written with agent-scope write-through stores
// and read with agent-scope copies, every producer wave waits for its own
// stores to be acknowledged and then sets its own byte of flags[l][t][rb]
// (byte 4 x column slice + wave, a plain write-through store); consumers read
// the flag with one load, lane i byte i, until every producer's byte is set.
// (A count that the producers incremented atomically was the first form: the
// consumers' loads then queued behind up to 32 read-modify-writes of the same
// word, and the layer right above a layer that never waits paid 0.4 us per
// item for it.)  c is only ever re-read by the workgroup that wrote it and
// goes through the cache normally.
//
// The activation tile is double buffered, global -> LDS copies are requested
// an item ahead, results leave through an LDS staging area as full cache
// lines, and the order of everything within an item follows from one fact
// (comment above the loop): loads and stores share a counter, so a load result
// is only known once nothing at all is outstanding.  Two barriers per item.
//
// All workgroups must be co-resident: the host launches cooperatively with at
// most one workgroup per compute unit (each uses the whole register file of
// its CU).  Every wait is bounded by spin_limit polls; on expiry the kernel
// records an error word and every workgroup drains.
#include <stdlib.h>

#include <algorithm>
#include <mutex>
#include <type_traits>

#include "ftk_common.h"


namespace ftk {

int run_wavefront(const float* xs, const float* WU, const float* bias, const int* dil, float* hsss, float* csss,
                  int L, int T, int B, int H, hipStream_t s);
int run_wavefront_f16(const void* xs, const void* WU, const float* bias, const int* dil, const int* active, void* hsss,
                      void* csss, int L, int T, int B, int H, void* packed, hipStream_t s);
size_t split_stack_workspace_bytes(int L, int T, int B, int H);
int run_wavefront_split(const float* xs, const float* WU, const float* bias, const int* dil, const int* active, float* hsss,
                        float* csss, int L, int T, int B, int H, void* ws, hipStream_t s);

constexpr int PH = 256;            // hidden size this kernel is specialised for
constexpr int PK = 2 * PH;         // K of the gate GEMM
constexpr int PN = 4 * PH;         // gate columns
constexpr int P_LD = PK + 4;       // padded activation row in LDS (floats)
constexpr int PC = 8;              // column slices per layer (32 units each)
constexpr int kMaxLayers = 64;
constexpr int kMaxBlocks = 64;     // 32-row blocks a ragged batch may have (B <= 2048)

// Split products.  v_mfma_f32_32x32x16_f16 moves sixteen k per 8 passes where
// v_mfma_f32_32x32x2_f32 moves two per 16, so a product of two fp32 numbers is
// cheaper as three fp16 products than as one fp32 product, if each number is
// first cut in two: v * 2^e = top + rest with top = fp16(v * 2^e) and
// rest = fp16(v * 2^e - top).  The cut is exact up to the rounding of rest: 22
// significant bits for values within 2^-17 of the largest magnitude that shares
// the scale 2^e (a weight column, an input row, or the fixed 2^14 of h in
// (-1, 1)), where fp32 keeps 24, and 2^-40 of that magnitude below (the
// remainder is then an fp16 subnormal) -- what a sum of products needs.
// top*top, top*rest and rest*top are accumulated in fp32, in one accumulator
// where nothing waits for the sum and in two chains where a layer waits for
// its own results; rest*rest, 2^-22 of the product, is dropped.
constexpr int kSplitTop = 14;          // a scale group's largest magnitude lands in [2^14, 2^15)
constexpr float kSplitAct = 16384.0f;  // 2^14: the scale of h
constexpr int kSplitCommon = 12;       // input rows whose largest magnitude is below 2^(16 - 12) take the scale 2^12
// h * 2^14 below 2^-12 (|h| < 2^-26, 1.5e-8): the remainder plane, an fp16 subnormal from 2^-3 down, resolves 2^-24,
// and value plus remainder keep fewer than 13 bits
constexpr unsigned kSmallStateBits = (127u - 12u) << 23;

struct PersistArgs {
  const float* xs;
  const float* WU;
  const float* bias;
  float* hsss;
  float* csss;
  // split-product mode: every activation as two fp16 planes (rounded value, scaled remainder), see below
  const _Float16* xsp;   // [T][B][2][H] planes of the input rows
  const float* xratio;   // [T][B] what an input row's products are multiplied by to match the hidden rows' scale
  _Float16* hsp;         // [L][T][B][2][H] planes of every h
  unsigned char* flags;   // [L][T][NRB][kFlagStride]: one byte per producer wave
  int* status;  // [0] = error word
  int L, T, B;
  int nrb;         // row blocks of 32*RT rows
  int pr_of[kMaxLayers];        // row slices of layer l (its workgroups: column slices x row slices)
  int first_q[kMaxLayers + 1];  // first logical workgroup of layer l; [L] = all
  int groups;      // workgroups that take part (= first_q[L])
  int xcd_remap;   // 1: grid is a multiple of 8, workgroups in order, grid / 8 per XCD; w > 1: units of w workgroups
                   // (a layer's column slices of one row slice), unit u on XCD u % 8
  int spin_limit;
  int trace_q;            // logical workgroup whose item timeline is recorded, or -1
  long long* trace;       // [items][8] 100 MHz clock stamps of that workgroup
  int dil[kMaxLayers];
  int paired;                // 1: workgroups of pipelined layers take two row blocks per item (split products)
  int ragged;                // 1: row block rb takes part in steps t < steps_of[rb] only
  int steps_of[kMaxBlocks];
};

typedef unsigned long long u64;
template <int V> using IC = std::integral_constant<int, V>;

__device__ __forceinline__ int flag_load(const int* flag) {
  return __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A flag is kFlagStride bytes, one per producer wave (up to 16 column slices x 4 waves); lane i looks at byte i.
// Every wait is bounded: when the polls run out the status word is set and the caller drains.
constexpr int kFlagStride = 64;
// (Lanes past the last producer look at the last producer's byte: with a branch around the load the compiler waits for
// the byte where the branches join, and a look that is meant to be on its way while the wave works costs a round trip.)
__device__ __forceinline__ int flag_bytes_load(const unsigned char* flag, int lane, int target) {
  return __hip_atomic_load(flag + min(lane, target - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool all_set(int v) { return __builtin_amdgcn_ballot_w64(v != 0) == ~0ull; }
__device__ __forceinline__ bool wait_bytes(const unsigned char* flag, int lane, int target, int* status, int spin_limit) {
  int n = 0;
  while (!all_set(flag_bytes_load(flag, lane, target))) {
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

__device__ __forceinline__ void coherent_store8h(_Float16* p, v4h v) {
  __hip_atomic_store(reinterpret_cast<u64*>(p), __builtin_bit_cast(u64, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte
// offset + OFF) straight into LDS at lds_addr + 16*lane (wave-uniform byte
// address in LDS).  COHERENT: agent scope; otherwise through the caches, for
// data no other compute unit writes while it may be cached here.  Written as
// assembly so that base, LDS address and offset stay in scalar registers and
// the immediate field: with one wave per SIMD nothing hides the address
// arithmetic the compiler otherwise spends on every copy.  The compiler does
// not count these copies as outstanding loads; callers wait with vmcnt(0).
// (The hardware adds the instruction's immediate offset to the LDS address as
// well as to the global one, hence the subtraction.)
template <int OFF, bool COHERENT>
__device__ __forceinline__ void lds_dma16(const void* gbase, unsigned byte_off, unsigned lds_addr) {
  lds_addr -= OFF;
  if constexpr (COHERENT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3 sc1"
                 :: "s"(lds_addr), "v"(byte_off), "s"(gbase), "n"(OFF) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
                 :: "s"(lds_addr), "v"(byte_off), "s"(gbase), "n"(OFF) : "memory", "m0");
}
// The same with the LDS address formed in the instruction stream, base + DELTA: a caller with many destinations at
// fixed distances keeps one scalar register instead of one per destination (sixteen of them per phase would be
// spilled into a vector register's lanes and read back one by one in front of every copy).
template <int OFF, bool COHERENT, int DELTA>
__device__ __forceinline__ void lds_dma16_at(const void* gbase, unsigned byte_off, unsigned lds_base) {
  if constexpr (COHERENT)
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3 sc1"
                 :: "s"(lds_base), "v"(byte_off), "s"(gbase), "n"(OFF), "n"(DELTA - OFF) : "memory", "m0", "scc");
  else
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
                 :: "s"(lds_base), "v"(byte_off), "s"(gbase), "n"(OFF), "n"(DELTA - OFF) : "memory", "m0", "scc");
}
// 4 bytes per lane, through the caches: used to touch cache lines ahead of time.
__device__ __forceinline__ void lds_dma4(const void* gbase, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_addr), "v"(byte_off), "s"(gbase) : "memory", "m0");
}

// Activation rows are read with agent-scope loads (true) or through the caches (false).  Through the caches
// measures the same, and is only safe while every writer of a cache line sits on the reader's side of a
// non-coherent L2: a partly written line that such a cache fills from memory keeps the other part stale.
constexpr bool kCoherentTiles = true;

constexpr int P_TILE = 32 * P_LD;  // floats per LDS buffer
// output staging in LDS, per buffer: c and h as [32][32] fp32 with 144-byte rows, the two fp16 planes as
// [32][32] with 80-byte rows
constexpr int kStageRow32 = 144, kStageRow16 = 80;
constexpr int kStageC = 0, kStageH = 32 * kStageRow32, kStageTop = 2 * 32 * kStageRow32, kStageRest = kStageTop + 32 * kStageRow16;
constexpr int kStageBytes = kStageRest + 32 * kStageRow16;
constexpr int kRatioOffset = 2 * P_TILE * (int)sizeof(float) + 1024 + 2 * kStageBytes;   // bytes; [2 tile buffers][64 floats]
constexpr int kVoteOffset = kRatioOffset + 2 * 64 * (int)sizeof(float);   // bytes; one int per wave (serial schedule)
constexpr int kGateTableOffset = kVoteOffset + 64;   // bytes; [4 waves][2 lane halves][16 x (factor, bias)] (paired schedule)
constexpr size_t kPersistLds = (size_t)kGateTableOffset + 8 * 32 * sizeof(float);  // tiles, prefetch scrap, staging, row ratios, votes, gate table
static_assert(kPersistLds <= 160 * 1024, "the workgroup's LDS");
// Kernel flavours.  kProductsF32 / kProductsSplit: fp32 data, H = 256, the two ways of forming the products.
// kHalfData: fp16 inputs, weights, h and c (what the reference's CuTe LSTM stores), one fp16 MFMA per product
// with fp32 accumulation, H = 512: a row of 512 fp16 takes the 1024 bytes a row of 256 fp32 takes, and a
// wave's 32 gate columns x 1024 k of fp16 weights the 256 VGPRs the other flavours' weights take, so tiles,
// copies and schedule are shared; a layer then has 16 column slices instead of 8.
// kHalfData256: the same at H = 256.  A row then is 512 bytes, so a 1 KB copy carries two batch rows and a tile
// row holds the pair: [x of row 2i | x of row 2i+1 | h of row 2i | h of row 2i+1]; B must be even.
constexpr int kProductsF32 = 0, kProductsSplit = 1, kHalfData = 2, kHalfData256 = 3;
constexpr int TS = 8;              // trace stamps per item

template <int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void lstm_persistent_kernel(PersistArgs a) {
  constexpr bool SPLIT = MODE == kProductsSplit;
  constexpr bool F16 = MODE == kHalfData || MODE == kHalfData256;
  constexpr bool PAIR = MODE == kHalfData256;      // two batch rows per tile row
  constexpr int HID = MODE == kHalfData ? 2 * PH : PH;  // hidden size
  constexpr int NPC = HID / 32;           // column slices per layer (32 units each)
  constexpr int NG = 4 * HID;             // gate columns
  constexpr int FLAG_TARGET = NPC * 4;    // producer waves per flag: four of each column slice
  extern __shared__ __attribute__((aligned(16))) float tile[];  // [2][32][P_LD], 256 floats of scrap, 2 staging buffers

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31;
  const int hh = lane >> 5;
  // the batch row (within a 32-row block) whose activations this lane feeds to the MFMAs and whose results it
  // gets back.  With two batch rows per tile row, lanes 0..15 take the first of each pair and lanes 16..31 the
  // second: the 16 lanes of one pass of a fragment read then touch 16 different tile rows (16 bytes apart in the
  // bank line), where lanes 2r / 2r+1 on one tile row, 512 bytes apart, hit the same banks.
  const int jb = MODE == kHalfData256 ? 2 * (j & 15) + (j >> 4) : j;

  int q = blockIdx.x;
  if (a.xcd_remap == 1) q = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (a.xcd_remap > 1) {   // the i-th unit of XCD x is unit 8 i + x of the launch; slots beyond the last unit stay empty
    const int slot = blockIdx.x >> 3, w = a.xcd_remap;
    q = ((slot / w) * 8 + (int)(blockIdx.x & 7)) * w + slot % w;
  }
  if (q >= a.groups) return;
  if (q == a.trace_q && tid == 0) reinterpret_cast<long long*>(a.status + 16)[0] = wall_clock64();
  int l = 0;
  while (l + 1 < a.L && q >= a.first_q[l + 1]) ++l;
  const int pr = a.pr_of[l];
  const int within = q - a.first_q[l];
  const int pc = within % NPC;
  const int prs = within / NPC;
  const int d = a.dil[l];
  const int T = a.T, B = a.B;
  const size_t cell = (size_t)B * (F16 ? HID / 2 : PH);  // floats (or pairs of fp16) per [B, H] slab of activations
  const int my_rbs = (a.nrb - prs + pr - 1) / pr;  // row blocks this workgroup walks per time step
  const int n_items = T * my_rbs;

  // Resident weights.  fp32 products: lane (i = j, half hh) of wave w holds, for
  // MFMA step s = 4q + c, WU[l][k = 8q + 4hh + c][gate(i)*H + 32pc + 8w + i%8].
  // Split products: for MFMA step s the lane holds rows k = 16s + 8hh .. +7 of
  // the same column, as the fp16 pair described above.
  // fp16 data: rows k = 16s + 8hh .. +7 of the column for MFMA step s, 64 steps.
  const int col = (j >> 3) * HID + 32 * pc + 8 * wave + (j & 7);
  const float* wl = a.WU + (size_t)l * PK * PN + col;
  // Split products, first layer: input rows are split on a scale of their own, and their products move to h's scale
  // by a per-row factor before the h products join them -- unless every row of this launch's input took the common
  // scale 2^kSplitCommon (lstm_split_rows_kernel says so in the status block's third word).  Then the factor is the
  // same power of two for all rows, the input half of this layer's weights takes it, exactly, and nothing is
  // rescaled per item.
  const bool x_has_common_scale = SPLIT && l == 0 && flag_load(a.status + 2) == 0;
  const float xfold = x_has_common_scale ? kSplitAct / (float)(1 << kSplitCommon) : 1.0f;
  const bool x_rescaled = SPLIT && l == 0 && !x_has_common_scale;
  float wr[MODE == kProductsF32 ? PK / 2 : 1];
  v8h whi[SPLIT ? PK / 16 : 1], wlo[SPLIT ? PK / 16 : 1];
  v8h wh[F16 ? 2 * HID / 16 : 1];
  float ginv[16];  // split products: what accumulator register r is multiplied by to undo the scales
  if constexpr (F16) {
    const _Float16* wl16 = reinterpret_cast<const _Float16*>(a.WU) + (size_t)l * (2 * HID) * NG + col;
#pragma unroll
    for (int s = 0; s < 2 * HID / 16; ++s) {
#pragma unroll
      for (int e = 0; e < 8; ++e) wh[s][e] = wl16[(size_t)(16 * s + 8 * hh + e) * NG];
      // 16-bit loads land in a register each before they are packed: keep few of them in flight
      if (s % 4 == 3) asm volatile("" ::: "memory");
    }
  } else if constexpr (!SPLIT) {
#pragma unroll
    for (int s = 0; s < PK / 2; ++s) {
      const int k = 8 * (s >> 2) + 4 * hh + (s & 3);
      wr[s] = wl[(size_t)k * PN];
    }
  } else {
    // the column's largest magnitude decides its power-of-two scale.  (First layer, every input row on the common
    // scale: the input rows of WU take the factor between that scale and h's, see x_has_common_scale.)
    float cmax = 0.f;
#pragma unroll
    for (int s = 0; s < PK / 16; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) cmax = fmaxf(cmax, fabsf(wl[(size_t)(16 * s + 8 * hh + e) * PN]) * (s < PK / 32 ? xfold : 1.0f));
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32));
    const int eb = min(max((int)((__float_as_uint(cmax) >> 23) & 0xff), 15), 254);
    const float wscale = __uint_as_float((unsigned)(127 + kSplitTop + 127 - eb) << 23);  // column max -> [2^14, 2^15)
    const float winv = __uint_as_float((unsigned)(eb - kSplitTop) << 23);
    asm volatile("" ::: "memory");  // the second pass loads again instead of keeping 256 values alive
#pragma unroll
    for (int s = 0; s < PK / 16; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float w = wl[(size_t)(16 * s + 8 * hh + e) * PN] * (s < PK / 32 ? xfold * wscale : wscale);
        const _Float16 top = (_Float16)w;
        whi[s][e] = top;
        wlo[s][e] = (_Float16)(w - (float)top);
      }
#pragma unroll
    for (int r = 0; r < 16; ++r) ginv[r] = __shfl(winv, (r & 3) + 8 * (r >> 2) + 4 * hh) * (1.0f / kSplitAct);
    // Seven eighths of the fragments move to the accumulation registers, by hand.  The matrix instructions read
    // their operands from either register file; the vector ALU, which everything else here goes through, only from
    // the architectural one, whose 256 registers the weights alone would fill.  Left to itself the compiler parks
    // fragments in accumulation registers too, but as spills: four moves back and a wait state in front of every
    // MFMA that uses one, in loops where the issue slots beside an MFMA are what is scarce.
    auto to_acc = [](v8h v) __attribute__((always_inline)) -> v8h {
      typedef unsigned v4u __attribute__((ext_vector_type(4)));
      const v4u u = __builtin_bit_cast(v4u, v);
      unsigned a0, a1, a2, a3;
      asm("v_accvgpr_write_b32 %0, %1" : "=a"(a0) : "v"(u[0]));
      asm("v_accvgpr_write_b32 %0, %1" : "=a"(a1) : "v"(u[1]));
      asm("v_accvgpr_write_b32 %0, %1" : "=a"(a2) : "v"(u[2]));
      asm("v_accvgpr_write_b32 %0, %1" : "=a"(a3) : "v"(u[3]));
      const v4u r = {a0, a1, a2, a3};
      return __builtin_bit_cast(v8h, r);
    };
#pragma unroll
    for (int s = 0; s < PK / 16; ++s) {
      whi[s] = to_acc(whi[s]);
      if (s % 4 != 3) wlo[s] = to_acc(wlo[s]);
    }
  }
  const int u0 = 32 * pc + 8 * wave + 4 * hh;  // first of this lane's 4 units
  // sigmoid(v) = 1 / (1 + 2^(-v log2 e)): the -log2 e of the gates i, f, o (accumulator register r holds gate r / 4
  // of unit r % 4) is folded into what the register is multiplied by anyway (split products) and into the bias, so
  // the argument of the exponential is one multiply-add away from the accumulators.  The candidate keeps scale 1:
  // tanh_f needs its argument as it is (it switches to a polynomial near zero, where the exponential form loses
  // relative accuracy; with inputs of 1e-3 the states are that small and the error would reach 1e-4 of them).
  constexpr float kLog2e = 1.4426950408889634f;
  float esc[SPLIT ? 16 : 1], ebias[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float k = (r >> 2) == 3 ? 1.0f : -kLog2e;
    if constexpr (SPLIT) esc[r] = ginv[r] * k;
    ebias[r] = 0.0f;
    if (a.bias) ebias[r] = a.bias[(size_t)l * NG + (r >> 2) * HID + u0 + (r & 3)] * k;
  }
  bool alive = true;
  if (q == a.trace_q && tid == 0) {
    long long* st = reinterpret_cast<long long*>(a.status + 16);
    st[1] = wall_clock64();  // weights requested (st[0]: kernel entry)
    float sink = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < 32; s2 += 2) sink += F16 ? (float)wh[F16 ? s2 : 0][0] : SPLIT ? (float)whi[SPLIT ? s2 : 0][0] : wr[MODE == kProductsF32 ? 16 * s2 : 0];
    if (sink == 12345.678f) st[3] = 0;
    st[2] = wall_clock64();  // weights (a sample of them) have arrived
  }

  auto item_t = [&](int n) { return n / my_rbs; };
  auto item_rb = [&](int n) { return prs + pr * (n % my_rbs); };
  // Ragged batches (rows sorted by length, so a row block simply stops after its longest row): an item
  // past its block's last step is walked through like any other, but requests, computes, stores and counts
  // nothing; nothing that is computed depends on it.
  auto live = [&](int n) { return !a.ragged || item_t(n) < a.steps_of[item_rb(n)]; };
  auto flag_of = [&](int ll, int t, int rb) { return a.flags + (((size_t)ll * T + t) * a.nrb + rb) * kFlagStride; };

  // inputs of item n complete?  Bounded spin on the two flags.
  auto wait_deps = [&](int n) __attribute__((always_inline)) -> bool {
    const int t = item_t(n), rb = item_rb(n);
    bool ok = true;
    if (!live(n)) return true;
    if (l > 0) ok = wait_bytes(flag_of(l - 1, t, rb), lane, FLAG_TARGET, a.status, a.spin_limit);
    if (ok && t >= d) ok = wait_bytes(flag_of(l, t - d, rb), lane, FLAG_TARGET, a.status, a.spin_limit);
    // The data loads must stay behind the flag reads.  The hardware issues and
    // returns loads in order, so a compiler barrier is all it takes; a fence
    // instruction here would also wait for this wave's outstanding stores.
    asm volatile("" ::: "memory");
    return ok;
  };
  // request / test the two flags of item n without waiting (what a lane holds is its byte of each)
  struct Flags { int below, own; };
  auto request_flags = [&](int n) __attribute__((always_inline)) -> Flags {
    Flags f{1, 1};
    const int t = item_t(n), rb = item_rb(n);
    if (!live(n)) return f;
    if (l > 0) f.below = flag_bytes_load(flag_of(l - 1, t, rb), lane, FLAG_TARGET);
    if (t >= d) f.own = flag_bytes_load(flag_of(l, t - d, rb), lane, FLAG_TARGET);
    return f;
  };
  auto flags_ready = [=](const Flags& f) { return all_set(f.below) && all_set(f.own); };

  // Where the activation rows come from.  The two fp16 planes of a row take the
  // 1024 bytes of its fp32 form, so the tile code is the same for both: in
  // split mode a tile row is [x top | x rest | h top | h rest], 256 fp16 each, with
  // fp16 data [x | h], 512 fp16 each (xsp / hsp then are the fp16 xs and hsss themselves).
  const float* xin = (SPLIT || F16) ? reinterpret_cast<const float*>(a.xsp) : a.xs;
  const float* hin = (SPLIT || F16) ? reinterpret_cast<const float*>(a.hsp) : a.hsss;

  // Tile n into LDS buffer buf, global -> LDS directly: wave w moves rows
  // 8w..8w+7; one instruction carries half a tile row (1024 bytes = 64 lanes x
  // 16, consecutive lanes to consecutive LDS addresses).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lane16 = 16u * lane;
  const unsigned lane_lines = 1024u * (lane >> 3) + 128u * (lane & 7);  // one lane per cache line of 8 rows
  const unsigned tile_lds = (unsigned)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)tile);
  // part: kWholeTile, or only its x columns / only its h columns (the serial schedule asks for them at different times)
  constexpr int kWholeTile = 0, kTileX = 1, kTileH = 2;
  auto issue_tile = [&](int n, int buf, int part = 0) __attribute__((always_inline)) {
    const int t = item_t(n), rb = item_rb(n);
    if (!live(n)) return;
    const bool has_prev = t >= d && part != kTileX;
    const bool with_x = part != kTileH;
    const char* xsrc = reinterpret_cast<const char*>((l == 0) ? xin + (size_t)t * cell : hin + ((size_t)(l - 1) * T + t) * cell);
    const char* hsrc = reinterpret_cast<const char*>(hin + ((size_t)l * T + (has_prev ? t - d : 0)) * cell);
    const int row0 = rb * 32 + 8 * wave_u;
    if constexpr (PAIR) {  // four tile rows of two batch rows each per wave
      const unsigned ldsp = tile_lds + 4u * (unsigned)(buf * P_TILE + 4 * wave_u * P_LD);
      if (row0 + 8 <= B) {
        const char* xb = xsrc + (size_t)row0 * 512;
        const char* hb = hsrc + (size_t)row0 * 512;
        if (with_x) {
          static_for<4>([&](auto rc) __attribute__((always_inline)) {
            constexpr int r = decltype(rc)::value;
            lds_dma16<r * 1024, kCoherentTiles>(xb, lane16, ldsp + 4u * r * P_LD);
          });
        }
        if (has_prev) {
          static_for<4>([&](auto rc) __attribute__((always_inline)) {
            constexpr int r = decltype(rc)::value;
            lds_dma16<r * 1024, kCoherentTiles>(hb, lane16, ldsp + 4u * r * P_LD + 1024u);
          });
        }
      } else {  // pairs past the end of the (even) batch repeat the last pair
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const size_t rg = (size_t)max(min(row0 + 2 * r, B - 2), 0);
          if (with_x) lds_dma16<0, kCoherentTiles>(xsrc + rg * 512, lane16, ldsp + 4u * r * P_LD);
          if (has_prev) lds_dma16<0, kCoherentTiles>(hsrc + rg * 512, lane16, ldsp + 4u * r * P_LD + 1024u);
        }
      }
      return;
    }
    const unsigned lds0 = tile_lds + 4u * (unsigned)(buf * P_TILE + 8 * wave_u * P_LD);
    // Split products, first layer: the 32 rows' ratios (see load_ratio) travel with the x columns, into LDS, instead of
    // being loaded into a register: a register load that late in an item is waited for behind the copies of the
    // tile after next, which nothing else waits for before the item's end.
    if constexpr (SPLIT) {
      if (x_rescaled && with_x && wave_u == 0)
        lds_dma4(a.xratio + (size_t)t * B, 4u * (unsigned)min(rb * 32 + (lane & 31), B - 1), tile_lds + (unsigned)kRatioOffset + 256u * (unsigned)buf);
    }
    if (row0 + 8 <= B) {
      const char* xb = xsrc + (size_t)row0 * 1024;
      if (with_x) {
        static_for<8>([&](auto rc) __attribute__((always_inline)) {
          constexpr int r = decltype(rc)::value;
          lds_dma16<(r & 3) * 1024, kCoherentTiles>(xb + (r >> 2) * 4096, lane16, lds0 + 4u * r * P_LD);
        });
      }
      if (has_prev) {
        const char* hb = hsrc + (size_t)row0 * 1024;
        static_for<8>([&](auto rc) __attribute__((always_inline)) {
          constexpr int r = decltype(rc)::value;
          lds_dma16<(r & 3) * 1024, kCoherentTiles>(hb + (r >> 2) * 4096, lane16, lds0 + 4u * r * P_LD + 1024u);
        });
      }
    } else {  // the batch ends inside these 8 rows: rows past the end repeat the last one
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const size_t rg = (size_t)min(row0 + r, B - 1);
        if (with_x) lds_dma16<0, kCoherentTiles>(xsrc + rg * 1024, lane16, lds0 + 4u * r * P_LD);
        if (has_prev) lds_dma16<0, kCoherentTiles>(hsrc + rg * 1024, lane16, lds0 + 4u * r * P_LD + 1024u);
      }
    }
    // The first layer's input rows come from memory nobody has touched; pull the rows of the item after
    // this one towards the cache now, so that their copy into LDS one item later is served from L2 like
    // the other layers' rows.  One 4-byte-per-lane copy touches all 64 cache lines of the wave's 8 rows;
    // it lands in a scrap area behind the tiles (a load into registers would need them reserved until
    // the data arrives).
    if (!PAIR && with_x && l == 0 && n + 1 < n_items && live(n + 1)) {
      const int t2 = item_t(n + 1), rb2 = item_rb(n + 1);
      const int row2 = rb2 * 32 + 8 * wave_u;
      if (row2 + 8 <= B)
        lds_dma4(reinterpret_cast<const char*>(xin + (size_t)t2 * cell) + (size_t)row2 * 1024, lane_lines,
                 tile_lds + 4u * (unsigned)(2 * P_TILE + 64 * wave_u));
    }
  };
  // steps [q0, q1) of the K loop (steps 0..31: x rows of WU, 32..63: h rows)
  // into two accumulators so that consecutive MFMAs never wait on each other's
  // result; the LDS read for step q+1 is issued before the MFMAs of step q
  // first_c (here and below): these are an item's first products, the accumulators start from zero -- as the
  // matrix instruction's constant addend, which costs nothing, where clearing 48 accumulator registers costs 48
  // vector instructions per item
  const v16f zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  auto mfma_part = [&](int buf, auto q0c, auto q1c, auto first_c, v16f& acc0, v16f& acc1) __attribute__((always_inline)) {
    constexpr int q0 = decltype(q0c)::value;
    constexpr int q1 = decltype(q1c)::value;
    constexpr bool first = decltype(first_c)::value;
    const float* arow = tile + buf * P_TILE + j * P_LD + 4 * hh;
    v4f b = *reinterpret_cast<const v4f*>(arow + 8 * q0);
#pragma unroll
    for (int qq = q0; qq < q1; ++qq) {
      v4f bn = b;
      if (qq + 1 < q1) bn = *reinterpret_cast<const v4f*>(arow + 8 * (qq + 1));
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 0], b[0], first && qq == q0 ? zero16 : acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wr[4 * qq + 1], b[1], first && qq == q0 ? zero16 : acc1, 0, 0, 0);
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
  // the same in split mode: steps 0..15 are the x rows, 16..31 the h rows; a
  // lane reads its 8 k of both planes and three MFMAs use them
  auto mfma_split = [&](int buf, auto q0c, auto q1c, auto first_c, v16f& am, v16f& ar) __attribute__((always_inline)) {
    constexpr int q0 = decltype(q0c)::value;
    constexpr int q1 = decltype(q1c)::value;
    constexpr bool first = decltype(first_c)::value;
    const _Float16* arow = reinterpret_cast<const _Float16*>(tile + buf * P_TILE + j * P_LD) + 8 * hh;
    auto top_of = [&](int qq) { return *reinterpret_cast<const v8h*>(arow + (qq >> 4) * (2 * PH) + 16 * (qq & 15)); };
    auto rest_of = [&](int qq) { return *reinterpret_cast<const v8h*>(arow + (qq >> 4) * (2 * PH) + PH + 16 * (qq & 15)); };
    v8h bt = top_of(q0), br = rest_of(q0);
#pragma unroll
    for (int qq = q0; qq < q1; ++qq) {
      v8h btn = bt, brn = br;
      if (qq + 1 < q1) { btn = top_of(qq + 1); brn = rest_of(qq + 1); }
      // top x top in one accumulator; top x rest and rest x top share the other (two chains:
      // where a layer waits for its own results, an MFMA that adds to the one before it would lengthen the wait)
      am = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi[qq], bt, first && qq == q0 ? zero16 : am, 0, 0, 0);
      ar = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi[qq], br, first && qq == q0 ? zero16 : ar, 0, 0, 0);
      ar = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo[qq], bt, ar, 0, 0, 0);
      bt = btn; br = brn;
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int g4 = q0; g4 < q1; ++g4) {
      __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  };
  // fp16 data: the first HID/16 steps are the x rows, the rest the h rows; one MFMA per step, two accumulation chains
  auto mfma_half = [&](int buf, auto q0c, auto q1c, auto first_c, v16f& a0, v16f& a1) __attribute__((always_inline)) {
    constexpr int q0 = decltype(q0c)::value;
    constexpr int q1 = decltype(q1c)::value;
    constexpr bool first = decltype(first_c)::value;
    constexpr int SH = HID / 16;  // steps per half
    const _Float16* arow = PAIR ? reinterpret_cast<const _Float16*>(tile + buf * P_TILE + (jb >> 1) * P_LD) + (jb & 1) * HID + 8 * hh
                                : reinterpret_cast<const _Float16*>(tile + buf * P_TILE + j * P_LD) + 8 * hh;
    auto frag = [&](int qq) { return *reinterpret_cast<const v8h*>(arow + (qq / SH) * 512 + 16 * (qq % SH)); };
    v8h b0 = frag(q0), b1 = frag(q0 + 1);
#pragma unroll
    for (int qq = q0; qq < q1; qq += 2) {
      v8h b0n = b0, b1n = b1;
      if (qq + 2 < q1) { b0n = frag(qq + 2); b1n = frag(qq + 3); }
      a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh[F16 ? qq : 0], b0, first && qq == q0 ? zero16 : a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh[F16 ? qq + 1 : 0], b1, first && qq == q0 ? zero16 : a1, 0, 0, 0);
      b0 = b0n; b1 = b1n;
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int g2 = q0; g2 < q1; g2 += 2) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  };
  // one interface for all: K steps of the x half [x0, x1) or of the h half, in
  // units of a sixteenth of a half
  v16f acc0, acc1;
  // an item without an x half to start the accumulators from zero does not exist: the x half always runs
  auto mfma_range = [&](int buf, auto half_c, auto s0c, auto s1c) __attribute__((always_inline)) {
    constexpr int hf = decltype(half_c)::value, s0 = decltype(s0c)::value, s1 = decltype(s1c)::value;
    constexpr std::integral_constant<bool, hf == 0 && s0 == 0> first{};
    if constexpr (F16)
      mfma_half(buf, std::integral_constant<int, (HID / 16) * hf + s0 * (HID / 256)>{},
                std::integral_constant<int, (HID / 16) * hf + s1 * (HID / 256)>{}, first, acc0, acc1);
    else if constexpr (SPLIT)
      mfma_split(buf, std::integral_constant<int, 16 * hf + s0>{}, std::integral_constant<int, 16 * hf + s1>{}, first, acc0, acc1);
    else
      mfma_part(buf, std::integral_constant<int, 32 * hf + 2 * s0>{}, std::integral_constant<int, 32 * hf + 2 * s1>{}, first, acc0, acc1);
  };
  // split mode, first layer: the x rows carry a scale of their own; before the h
  // products join the same accumulators the x products move to h's scale (a
  // power of two: exact)
  // the ratio of this lane's row in the tile that has landed in buffer buf
  auto load_ratio = [&](int buf) __attribute__((always_inline)) -> float {
    if constexpr (SPLIT) {
      if (x_rescaled) return reinterpret_cast<const float*>(reinterpret_cast<const unsigned char*>(tile) + kRatioOffset)[64 * buf + j];
    }
    return 1.0f;
  };
  auto rescale_x = [&](float ratio) __attribute__((always_inline)) {
    if constexpr (SPLIT) {
      if (x_rescaled) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc0[r] *= ratio; acc1[r] *= ratio; }
      }
    }
  };
  // the arguments of an item's 12 sigmoid exponentials and its 4 candidate sums (see esc / ebias)
  auto gate_sums = [&]() __attribute__((always_inline)) -> v16f {
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if constexpr (SPLIT) acc[r] = esc[r] * (acc0[r] + acc1[r]) + ebias[r];
      else acc[r] = ((r >> 2) == 3 ? 1.0f : -kLog2e) * (acc0[r] + acc1[r]) + ebias[r];
    }
    return acc;
  };
  // activations and state update of an item: lane-local and branch-free.
  // piece m (0..15) of the computation: gate (m & 3) of unit (m >> 2); the last
  // gate of a unit finishes its c and h
  float eg_i = 0.f, eg_f = 0.f, eg_o = 0.f;
  auto epilogue_piece = [&](const v16f& acc, const float4& cp, float (&hv)[4], float (&cv)[4], auto mc) __attribute__((always_inline)) {
    constexpr int m = decltype(mc)::value;
    constexpr int r = m >> 2;
    const float cpv[4] = {cp.x, cp.y, cp.z, cp.w};
    auto inv1p = [](float e) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(e)); };
    if constexpr ((m & 3) == 0) eg_i = inv1p(acc[r]);
    if constexpr ((m & 3) == 1) eg_f = inv1p(acc[4 + r]);
    if constexpr ((m & 3) == 2) eg_o = inv1p(acc[8 + r]);
    if constexpr ((m & 3) == 3) {
      const float cand = tanh_f(acc[12 + r]);
      cv[r] = eg_f * cpv[r] + eg_i * cand;
      hv[r] = eg_o * tanh_f(cv[r]);
    }
  };
  auto epilogue_math = [&](const v16f& acc, const float4& cp, float (&hv)[4], float (&cv)[4]) __attribute__((always_inline)) {
    static_for<16>([&](auto mc) __attribute__((always_inline)) { epilogue_piece(acc, cp, hv, cv, mc); });
  };
  // The lane that computes (row, 4 units) does not store them: 64 lanes would touch 32 rows, a sliver of a
  // cache line in each.  The results cross a staging area in LDS instead ([32 rows][this workgroup's 32
  // units] per output, rows padded against bank conflicts), and after a barrier wave w stores rows
  // 8w..8w+7: 128 contiguous bytes of c and h per row, 64 of each fp16 plane.
  unsigned char* const stage = reinterpret_cast<unsigned char*>(tile + 2 * P_TILE + 256);
  bool small_reported = false;   // this wave has set the status block's small-states word
  auto stage_results = [&](const float (&hv)[4], const float (&cv)[4], int sbuf) __attribute__((always_inline)) {
    unsigned char* sb = stage + sbuf * kStageBytes;
    const int c4 = 8 * wave + 4 * hh;
    if constexpr (F16) {  // h and c leave as fp16: the two 16-bit staging planes hold them
      const v4h h16 = {(_Float16)hv[0], (_Float16)hv[1], (_Float16)hv[2], (_Float16)hv[3]};
      const v4h c16 = {(_Float16)cv[0], (_Float16)cv[1], (_Float16)cv[2], (_Float16)cv[3]};
      *reinterpret_cast<v4h*>(sb + kStageTop + jb * kStageRow16 + 2 * c4) = h16;
      *reinterpret_cast<v4h*>(sb + kStageRest + jb * kStageRow16 + 2 * c4) = c16;
      return;
    }
    *reinterpret_cast<float4*>(sb + kStageC + j * kStageRow32 + 4 * c4) = make_float4(cv[0], cv[1], cv[2], cv[3]);
    *reinterpret_cast<float4*>(sb + kStageH + j * kStageRow32 + 4 * c4) = make_float4(hv[0], hv[1], hv[2], hv[3]);
    if constexpr (SPLIT) {
      v4h top, rest;
      unsigned largest = 0;  // bit pattern of the largest |h * 2^14| of the lane's four neighbouring units
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = hv[r] * kSplitAct;
        top[r] = (_Float16)v;
        rest[r] = (_Float16)(v - (float)top[r]);
        largest = max(largest, __float_as_uint(v) & 0x7fffffffu);
      }
      *reinterpret_cast<v4h*>(sb + kStageTop + j * kStageRow16 + 2 * c4) = top;
      *reinterpret_cast<v4h*>(sb + kStageRest + j * kStageRow16 + 2 * c4) = rest;
      // the planes have a fixed scale: below kSmallState the two of them hold fewer than 13 bits of a value.  One such
      // value beside larger ones is exact enough for the sums it enters (2^-38 in absolute terms); where four
      // neighbouring units of a row are all that small (and not all zero) the row or the layer has faded, and the cells
      // that read it see it less accurately than 1e-4 of ITS size (the fp32 h and c in hsss / csss are exact either
      // way).  The status block's second word tells the caller that this happened.
      // (once per wave: a store per item to one word from every compute unit of a faded layer queues up behind
      // itself, and the wait for an item's stores then waits for it)
      if (!small_reported && __builtin_amdgcn_ballot_w64(largest - 1u < kSmallStateBits - 1u) != 0) {
        small_reported = true;
        if (lane == 0) __hip_atomic_store(a.status + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  auto epilogue_to_lds = [&](const v16f& acc, const float4& cp, int sbuf) __attribute__((always_inline)) {
    float hv[4], cv[4];
    epilogue_math(acc, cp, hv, cv);
    stage_results(hv, cv, sbuf);
  };
  // What consumers on other compute units read leaves through write-through stores (fp32 products: h;
  // split products: the two planes), the rest through the cache.
  auto store_block = [&](int t, int rb, bool is_live, int sbuf) __attribute__((always_inline)) {
    const int rl = 8 * wave + (lane >> 3), cc = lane & 7;
    const int rg = rb * 32 + rl;
    if constexpr (F16) {
      if (alive && rg < B && is_live) {
        const unsigned char* sb = stage + sbuf * kStageBytes;
        const size_t at16 = (((size_t)l * T + t) * B + rg) * HID + 32 * pc + 4 * cc;
        coherent_store8h(a.hsp + at16, *reinterpret_cast<const v4h*>(sb + kStageTop + rl * kStageRow16 + 8 * cc));
        *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(a.csss) + at16) =
            *reinterpret_cast<const v4h*>(sb + kStageRest + rl * kStageRow16 + 8 * cc);
      }
      return;
    }
    if (alive && rg < B && is_live) {
      const unsigned char* sb = stage + sbuf * kStageBytes;
      const size_t at = ((size_t)l * T + t) * cell + (size_t)rg * PH + 32 * pc + 4 * cc;
      const float4 cv = *reinterpret_cast<const float4*>(sb + kStageC + rl * kStageRow32 + 16 * cc);
      const float4 hv = *reinterpret_cast<const float4*>(sb + kStageH + rl * kStageRow32 + 16 * cc);
      *reinterpret_cast<float4*>(a.csss + at) = cv;
      if constexpr (SPLIT) {
        *reinterpret_cast<float4*>(a.hsss + at) = hv;
        _Float16* pdst = a.hsp + (((size_t)l * T + t) * B + rg) * (2 * PH) + 32 * pc + 4 * cc;
        coherent_store8h(pdst, *reinterpret_cast<const v4h*>(sb + kStageTop + rl * kStageRow16 + 8 * cc));
        coherent_store8h(pdst + PH, *reinterpret_cast<const v4h*>(sb + kStageRest + rl * kStageRow16 + 8 * cc));
      } else {
        coherent_store8(a.hsss + at, hv.x, hv.y);
        coherent_store8(a.hsss + at + 2, hv.z, hv.w);
      }
    }
  };
  auto store_item = [&](int n, int sbuf) __attribute__((always_inline)) { store_block(item_t(n), item_rb(n), live(n), sbuf); };
  // workgroup barrier that waits for nothing by itself: what has to be complete before it is waited for
  // explicitly (__syncthreads would also wait for the acknowledgement of every store in flight)
  auto barrier = [&]() __attribute__((always_inline)) {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  auto load_cprev_of = [&](int t, int rb, bool is_live) __attribute__((always_inline)) -> float4 {
    float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
    if (alive && t >= d && is_live) {
      const int rgc = min(rb * 32 + jb, B - 1);
      if constexpr (F16) {
        const v4h c16 = *reinterpret_cast<const v4h*>(reinterpret_cast<const _Float16*>(a.csss) +
                                                      (((size_t)l * T + (t - d)) * B + rgc) * HID + u0);
        cp = make_float4((float)c16[0], (float)c16[1], (float)c16[2], (float)c16[3]);
      } else {
        cp = *reinterpret_cast<const float4*>(a.csss + ((size_t)l * T + (t - d)) * cell + (size_t)rgc * PH + u0);
      }
    }
    return cp;
  };
  auto load_cprev = [&](int n) __attribute__((always_inline)) -> float4 { return load_cprev_of(item_t(n), item_rb(n), live(n)); };
  // every wave publishes its own part of an item: its stores acknowledged, then its byte of the flag
  auto publish = [&](int n) __attribute__((always_inline)) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    if (lane == 0 && alive && live(n))
      __hip_atomic_store(flag_of(l, item_t(n), item_rb(n)) + 4 * pc + wave, (unsigned char)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  const bool tracing = (q == a.trace_q) && tid == 0;

  // How far apart an item and the item that needs it are in this workgroup's
  // own sequence decides the schedule: distance 1 (one row block, dilation 1)
  // leaves nothing to overlap.
  const long long own_distance = (long long)d * my_rbs;
  const bool serial = own_distance < 2;

  if (serial) {
    // Every item waits for the one before it, so what an item costs is the chain from one hand-over to the next:
    // the siblings' h arrives -> its rows are copied -> h half of the products -> activations -> stores -> their
    // acknowledgement -> this wave's byte of the flag.  Everything that does not depend on the previous item is
    // taken off that chain: the x columns of tile n+1 are requested with the h columns of tile n (when the layer
    // below has them already), and the x half of item n+1 is formed between the stores of item n and the wait
    // for their acknowledgement, which takes longer than those MFMAs.
    // Whether the layer below is ready is something every wave sees for itself, at its own moment: a wave that
    // finds it ready requests its rows of the next tile's x columns early, and must not multiply with them before
    // the other waves' rows are there as well.  So the waves vote through LDS, and the early x half happens only
    // when all four requested their rows before this item's first barrier.
    int* const votes = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(tile) + kVoteOffset);
    bool xdone = false;    // the x half of the current item is in the accumulators already
    bool xhere = false;    // the x columns of this wave's rows of the current item's tile are in LDS (or on their way)
    for (int n = 0; n < n_items; ++n) {
      const int buf = n & 1;
      if (tracing) a.trace[TS * n + 0] = wall_clock64();
      if (alive) alive = wait_deps(n);
      if (alive) issue_tile(n, buf, xhere ? kTileH : kWholeTile);
      // the x columns of the next item: its own layer's dependency is this item, but the x rows only need the layer below
      bool xnext = false;
      if (alive && n + 1 < n_items && live(n + 1)) {
        bool below_ready = l == 0;
        if (l > 0) below_ready = all_set(flag_bytes_load(flag_of(l - 1, item_t(n + 1), item_rb(n + 1)), lane, FLAG_TARGET));
        if (below_ready) {
          asm volatile("" ::: "memory");
          issue_tile(n + 1, buf ^ 1, kTileX);
          xnext = true;
        }
      }
      const float4 cp = load_cprev(n);
      if (lane == 0) votes[wave] = xnext ? 1 : 0;
      // This item needs its own tile, not the next one's x columns: those were requested behind it (eight copies,
      // four with two batch rows per tile row), the counter of outstanding copies runs in issue order, and the
      // rest is waited for in front of the barrier behind the activations.
      if (xnext && PAIR) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
      else if (xnext) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      barrier();
      const int4 vote = *reinterpret_cast<const int4*>(votes);
      const bool xall = (vote.x & vote.y & vote.z & vote.w) != 0;   // the whole of tile n+1's x columns has landed
      if (live(n)) {
        if (!xdone) {
          mfma_range(buf, IC<0>{}, IC<0>{}, IC<16>{});
          rescale_x(load_ratio(buf));
        }
        if (item_t(n) >= d) mfma_range(buf, IC<1>{}, IC<0>{}, IC<16>{});
        epilogue_to_lds(gate_sums(), cp, 0);
      }
      // the next item's x columns, requested above, are waited for here, by hand: the compiler does not count those
      // copies, so the barrier's own fence waits for none of them
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // results staged; the next item's x columns complete; the tile may be rewritten by the item after the next
      store_item(n, 0);
      xdone = false;
      if (xall) {           // while the stores are acknowledged
        mfma_range(buf ^ 1, IC<0>{}, IC<0>{}, IC<16>{});
        rescale_x(load_ratio(buf ^ 1));
        xdone = true;
      }
      xhere = xnext;
      publish(n);
      if (tracing) a.trace[TS * n + 7] = wall_clock64();
    }
    return;
  }

  // ---- paired schedule (split products, and fp16 data at H = 256): an item is TWO row blocks (a, b) of one time
  // step, 64 batch rows.
  // What an item costs beyond its MFMAs -- the looks at the producers' flags, the waits for the stores'
  // acknowledgement, the barriers -- is paid once per hand-over whatever the number of rows, and with two blocks in
  // flight the activations of one block run on the vector pipeline while the matrix pipeline forms the other block's
  // products.  LDS has no room for two 64-row tiles; the tile is kept as two half buffers instead, XA = the 64 rows'
  // x columns and HB = their h columns (1 KB per row each), and the copies into one half are dealt out, one per
  // contraction step, over the MFMAs that read the other half, where a copy instruction meets a memory pipeline that
  // is not busy and does not hold the wave at issue.  Per item p, with X / H the halves of the products and E the
  // activations (which also split h into its planes and leave everything in a staging area):
  //   Xa(p) with Eb(p-1) -> staging 1    | the own layer's flags for item p are on their way
  //   Xb(p)                              | this wave's rows of item p's h columns -> HB; near its end, a look at the
  //                                        layer below's flags for item p+1
  //   wait for everything outstanding (the stores of block a of item p-1 among it: that block is published)
  //   barrier 1: HB and staging 1 complete, XA free
  //   stores of block b of item p-1 from staging 1
  //   Ha(p)                              | block a's rows of item p+1's x columns -> XA, if the layer below was seen
  //                                        ready
  //   wait for those stores alone: block b of item p-1 is published (split products)
  //   Hb(p) with Ea(p) -> staging 0      | block b's rows, on the phase's first steps
  //   (a wave that could not request its x rows waits for the layer below and requests them now)
  //   wait for everything outstanding (fp16 data: block b of item p-1 is published here)
  //   barrier 2: XA and staging 0 complete, HB free
  //   stores of block a of item p from staging 0
  // A wave only ever waits for the copies it issued itself, and fragment reads of a half follow a barrier that every
  // wave reached after such a wait.  Flags stay per 32-row block, so layers on the other schedules hand over to this
  // one and back.  The h columns of item p need this layer's item p - (own distance >= 2), whose second block was
  // published before barrier 2 of item p-1.
  if constexpr (SPLIT || MODE == kHalfData256) {
    const int ppt = (my_rbs + 1) / 2;            // pair items per time step
    if (a.paired && my_rbs >= 2 && (long long)d * ppt >= 2) {
      // PLAIN: every item has both its blocks at every step (no ragged batch, an even number of row blocks), and no
      // input row carries a scale of its own: the tests for a block that is missing or past its rows' end then fold
      // away, at the item's top most of all, and so does the rescaling of the x products, whose mere presence behind a
      // branch makes the compiler move both accumulators of a block out of and back into the accumulation registers
      // at every item.  Only the
      // workgroup that leaves time stamps carries the code for them.
      auto paired_schedule = [&](auto plain_c, auto traced_c) __attribute__((always_inline)) {
      constexpr bool PLAIN = decltype(plain_c)::value;
      constexpr bool TRACED = decltype(traced_c)::value;   // this workgroup leaves time stamps
      // fp16 data at H = 256 walks the same schedule: a batch row is 512 bytes there, a tile row of a half buffer holds
      // two of them (a copy instruction carries 1 KB), a contraction step is one MFMA instead of three, and h and c
      // leave as fp16.
      constexpr bool P16 = MODE == kHalfData256;
      constexpr int RB = P16 ? 512 : 1024;       // bytes of a batch row in a layer's arrays
      constexpr int TR = P16 ? 16 : 32;          // tile rows of a row block in a half buffer
      constexpr int NC = TR / 4;                 // copies per wave and block half: one tile row each
      constexpr int HLD = 1040;                  // bytes per row of a half buffer: 16 more than the 1 KB it holds
      const int n_pairs = T * ppt;
      unsigned char* const xa = reinterpret_cast<unsigned char*>(tile);
      unsigned char* const hb = xa + 2 * TR * HLD;
      const unsigned xa_lds = tile_lds, hb_lds = tile_lds + 2u * TR * HLD;
      // The per-register factors and biases of the gate sums move to a table in LDS, one set per wave and lane half,
      // in the order the activations take them: with four accumulators per lane the registers are needed elsewhere.
      // (a unit's four entries: gate i, the candidate, gates f and o -- the first part of a unit's activations takes
      // the first two with one read)
      float2* const gtab = reinterpret_cast<float2*>(reinterpret_cast<unsigned char*>(tile) + kGateTableOffset) + 16 * (2 * wave + hh);
      if (j == 0) {
#pragma unroll
        for (int m = 0; m < 16; ++m) {
          constexpr int gate_of[4] = {0, 3, 1, 2};
          const int reg = 4 * gate_of[m & 3] + (m >> 2);
          float factor = (reg >> 2) == 3 ? 1.0f : -kLog2e;
          if constexpr (SPLIT) factor = esc[SPLIT ? reg : 0];
          gtab[m] = make_float2(factor, ebias[reg]);
        }
      }
      // what part m of the activations needs from the table
      auto gate_entry = [&](auto mc) __attribute__((always_inline)) -> float4 {
        constexpr int m = decltype(mc)::value;
        if constexpr ((m & 3) == 0) return *reinterpret_cast<const float4*>(gtab + m);
        else if constexpr ((m & 3) == 3) return make_float4(0.f, 0.f, 0.f, 0.f);
        else { const float2 e = gtab[m + 1]; return make_float4(e.x, e.y, 0.f, 0.f); }
      };
      // Every per-layer array here has 1 KB per batch row (256 fp32, or the two fp16 planes of 256), and a flag is
      // kFlagStride bytes.  With one wave per SIMD the scalar arithmetic of an item has nothing to hide behind, so
      // an item's addresses are not multiplied out of (layer, step, row) each time: an item carries the byte offset
      // of its time step in those arrays (tO) and in a layer's flags (tF), the next item's follow by addition, and
      // the layer's bases are formed once.  (tF fits 32 bits: a layer's flags are 1/512 the size of its h.)
      const size_t stepO = (size_t)B * RB, dO = (size_t)d * stepO;
      const unsigned stepF = (unsigned)a.nrb * kFlagStride, dF = (unsigned)d * stepF;
      const char* const xbase = reinterpret_cast<const char*>((l == 0) ? xin : hin + (size_t)(l - 1) * T * cell);
      const char* const hbase = reinterpret_cast<const char*>(hin + (size_t)l * T * cell);
      char* const pbase = reinterpret_cast<char*>(a.hsp) + (size_t)l * T * stepO;
      char* const cbase = reinterpret_cast<char*>(a.csss + (size_t)l * T * cell);
      char* const obase = reinterpret_cast<char*>(a.hsss + (size_t)l * T * cell);
      unsigned char* const fown = flag_of(l, 0, 0);
      unsigned char* const fbelow = flag_of(max(l - 1, 0), 0, 0);
      // an item: time step t, row blocks rb0 and rb1 = rb0 + pr; on0 / on1: the block exists and is live at t.  Rows
      // are sorted by length, so a live second block has a live first one.
      struct Pair { int t, i, rb0, rb1; size_t tO; unsigned tF; int on0, on1; };
      auto pair_at = [&](int t, int i, size_t tO, unsigned tF) __attribute__((always_inline)) -> Pair {
        Pair x;
        x.t = t; x.i = i; x.tO = tO; x.tF = tF;
        x.rb0 = prs + pr * (2 * i);
        x.rb1 = x.rb0 + pr;
        x.on0 = PLAIN || !a.ragged || t < a.steps_of[x.rb0];
        x.on1 = PLAIN || (2 * i + 1 < my_rbs && (!a.ragged || t < a.steps_of[min(x.rb1, kMaxBlocks - 1)]));
        return x;
      };
      auto pair_after = [&](const Pair& x) __attribute__((always_inline)) -> Pair {
        return x.i + 1 < ppt ? pair_at(x.t, x.i + 1, x.tO, x.tF) : pair_at(x.t + 1, 0, x.tO + stepO, x.tF + stepF);
      };
      // A wave's 8 rows of a row block: where the first of them lies in global memory (the rows are 1 KB apart) and
      // where it goes in LDS.  The batch is a multiple of 8 rows here, so the 8 rows are all inside it or all beyond
      // its end; those beyond are copied from the batch's last 8 rows instead (nobody stores what comes of them).
      struct Rows { bool on; const char* g; unsigned lds; };
      auto rows_of = [&](const char* src, int rb, unsigned half_lds, int sub, bool on) __attribute__((always_inline)) -> Rows {
        return Rows{on, src + (unsigned)min(rb * 32 + 8 * wave_u, B - 8) * (unsigned)RB, half_lds + (unsigned)((TR * sub + NC * wave_u) * HLD)};
      };
      auto copy_row = [&](const Rows& x, auto r_c) __attribute__((always_inline)) {
        constexpr int r = decltype(r_c)::value;
        lds_dma16_at<(r & 3) * 1024, kCoherentTiles, r * HLD>(x.g + (r >> 2) * 4096, lane16, x.lds);
      };
      auto copy_block = [&](const char* src, int rb, unsigned half_lds, int sub) __attribute__((always_inline)) {
        const Rows x = rows_of(src, rb, half_lds, sub, true);
        static_for<NC>([&](auto r_c) __attribute__((always_inline)) { copy_row(x, r_c); });
      };
      auto copy_ratios = [&](const Pair& x) __attribute__((always_inline)) {   // first layer: the rows' scale ratios travel with their x columns
        if (PLAIN || !x_rescaled || wave_u != 0) return;
        if (x.on0) lds_dma4(a.xratio + (size_t)x.t * B, 4u * (unsigned)min(x.rb0 * 32 + (lane & 31), B - 1), tile_lds + (unsigned)kRatioOffset);
        if (x.on1) lds_dma4(a.xratio + (size_t)x.t * B, 4u * (unsigned)min(x.rb1 * 32 + (lane & 31), B - 1), tile_lds + (unsigned)kRatioOffset + 256u);
      };
      // One look at an item's two flags of layer ll, step t: lanes 0..31 take the bytes of block a's 32 producer
      // waves, lanes 32..63 those of block b (of block a again when there is no block b).  The load is unconditional
      // and its address always valid, so that nothing makes the compiler wait for it where it is issued: the wave
      // asks, works, and reads the answer later.  Callers ignore the answer where there is no such dependency.
      static_assert(FLAG_TARGET == 32, "one half of the wave per row block");
      auto look = [&](const unsigned char* layer_flags, unsigned tF, const Pair& x) __attribute__((always_inline)) -> int {
        unsigned off = tF + (unsigned)x.rb0 * kFlagStride + (lane & 31);
        if (lane >= 32 && x.on1) off += (unsigned)(x.rb1 - x.rb0) * kFlagStride;
        return __hip_atomic_load(layer_flags + off, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto wait_pair = [&](const Pair& x, int ll, int t) __attribute__((always_inline)) -> bool {
        bool ok = true;
        if (x.on0) ok = wait_bytes(flag_of(ll, t, x.rb0), lane, FLAG_TARGET, a.status, a.spin_limit);
        if (ok && x.on1) ok = wait_bytes(flag_of(ll, t, x.rb1), lane, FLAG_TARGET, a.status, a.spin_limit);
        asm volatile("" ::: "memory");   // the copies stay behind the flag reads
        return ok;
      };
      auto wait_below = [&](const Pair& x) __attribute__((always_inline)) -> bool { return l == 0 || wait_pair(x, l - 1, x.t); };
      auto wait_own = [&](const Pair& x) __attribute__((always_inline)) -> bool { return x.t < d || wait_pair(x, l, x.t - d); };
      // a wave publishes its part of one row block of an item; its stores have been waited for
      auto publish_block = [&](unsigned tF, int rb, bool on) __attribute__((always_inline)) {
        if (lane == 0 && alive && on)
          __hip_atomic_store(fown + (tF + (unsigned)rb * kFlagStride + 4 * pc + wave), (unsigned char)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      // store_block / load_cprev_of on the offsets an item carries
      auto store_rows = [&](int t, size_t tO, int rb, bool is_live, int sbuf) __attribute__((always_inline)) {
        if constexpr (P16) { store_block(t, rb, is_live, sbuf); return; }
        const int rl = 8 * wave + (lane >> 3), cc = lane & 7;
        const int rg = rb * 32 + rl;
        if (alive && rg < B && is_live) {
          const unsigned char* sb = stage + sbuf * kStageBytes;
          const size_t at = tO + (((unsigned)rg << 10) + 16u * (unsigned)(8 * pc + cc));
          *reinterpret_cast<float4*>(cbase + at) = *reinterpret_cast<const float4*>(sb + kStageC + rl * kStageRow32 + 16 * cc);
          *reinterpret_cast<float4*>(obase + at) = *reinterpret_cast<const float4*>(sb + kStageH + rl * kStageRow32 + 16 * cc);
          _Float16* pdst = reinterpret_cast<_Float16*>(pbase + tO + (((unsigned)rg << 10) + 8u * (unsigned)(8 * pc + cc)));
          coherent_store8h(pdst, *reinterpret_cast<const v4h*>(sb + kStageTop + rl * kStageRow16 + 8 * cc));
          coherent_store8h(pdst + PH, *reinterpret_cast<const v4h*>(sb + kStageRest + rl * kStageRow16 + 8 * cc));
        }
      };
      auto cprev_rows = [&](int t, size_t tO_prev, int rb, bool has) __attribute__((always_inline)) -> float4 {
        float4 cp = make_float4(0.f, 0.f, 0.f, 0.f);
        if constexpr (P16) {
          // the four fp16 values as they are, in the first two components: converted where they are used.  A
          // conversion here would wait for the load, and with it for the block's stores that left just before.
          if (alive && has && t >= d) {
            const uint2 raw = *reinterpret_cast<const uint2*>(reinterpret_cast<const _Float16*>(a.csss) +
                                                              (((size_t)l * T + (t - d)) * B + min(rb * 32 + jb, B - 1)) * HID + u0);
            cp.x = __uint_as_float(raw.x);
            cp.y = __uint_as_float(raw.y);
          }
          return cp;
        }
        if (alive && has)
          cp = *reinterpret_cast<const float4*>(cbase + tO_prev + (((unsigned)min(rb * 32 + j, B - 1) << 10) + 4u * (unsigned)u0));
        return cp;
      };
      // Waits until this wave's stores of a block are acknowledged, and for nothing younger: the counter of
      // outstanding vector-memory operations runs in issue order, loads and stores alike, so the stores are done once
      // no more operations are outstanding than were issued behind them.  `loads` (0 or 1) and `copies` (0 or 8) are
      // what the caller knows was issued behind the stores; more than that only makes the wait longer.
      auto wait_stores_behind = [&](bool one_load, bool eight_copies) __attribute__((always_inline)) {
        if (eight_copies && P16) {   // (four copies carry a block half there)
          if (one_load) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        } else if (eight_copies) {
          if (one_load) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        } else {
          if (one_load) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
      };
      auto wait_all = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
      };
      // piece m (0..15) of a block's activations, straight from the two accumulators: unit m >> 2, part m & 3.  With
      // one wave per SIMD a chain of dependent vector instructions runs at its latency, not at the issue rate, so a
      // piece carries two chains that do not depend on each other: parts 0..2 hold a sigmoid (gates i, f, o) beside a
      // third of the candidate's tanh, part 3 the tanh of the new c, whose exponential and polynomial are independent.
      float tc_v = 0.f, tc_e = 0.f, tc_x2 = 0.f, tc_p = 0.f, tc_r = 0.f;   // the candidate's tanh between the parts
      // (one accumulator, em, holds a block's sums: all three products of the split mode, the one product of fp16 data;
      // er is not used by this schedule)
      auto pair_piece = [&](const v16f& em, const v16f& er, const float4& cp, float (&hv)[4], float (&cv)[4], const float4 sb, auto mc) __attribute__((always_inline)) {
        constexpr int m = decltype(mc)::value;
        constexpr int r = m >> 2, g = m & 3, reg = 4 * g + r;
        float cpv[4] = {cp.x, cp.y, cp.z, cp.w};
        if constexpr (P16 && g == 2) {   // c of the step before arrives as four fp16 in two words
          const v4h c16 = __builtin_bit_cast(v4h, make_uint2(__float_as_uint(cp.x), __float_as_uint(cp.y)));
          cpv[r] = (float)c16[r];
        }
        auto inv1p = [](float e) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(e)); };
        if constexpr (g < 3) {
          const float v = sb.x * em[reg] + sb.y;
          if constexpr (g == 0) {
            eg_i = inv1p(v);
            tc_v = sb.z * em[12 + r] + sb.w;
            tc_e = fast_exp(2.0f * tc_v);
            tc_x2 = tc_v * tc_v;
          }
          if constexpr (g == 1) {
            eg_f = inv1p(v);
            tc_p = -0.33333333333f + tc_x2 * (0.13333333333f + tc_x2 * (-0.05396825397f + tc_x2 * 0.02186948854f));
            tc_r = __builtin_amdgcn_rcpf(1.0f + tc_e);
          }
          if constexpr (g == 2) {
            eg_o = inv1p(v);
            const float big = 1.0f - 2.0f * tc_r;
            const float small = tc_v * (1.0f + tc_x2 * tc_p);
            const float cand = fabsf(tc_v) < 0.25f ? small : big;   // tanh_f, in three parts
            cv[r] = eg_f * cpv[r] + eg_i * cand;
          }
        } else {
          hv[r] = eg_o * tanh_f(cv[r]);
        }
      };
      auto activations_alone = [&](const v16f& em, const v16f& er, const float4& cp, int sbuf) __attribute__((always_inline)) {
        float hv[4], cv[4];
        static_for<16>([&](auto mc) __attribute__((always_inline)) { pair_piece(em, er, cp, hv, cv, gate_entry(mc), mc); });
        stage_results(hv, cv, sbuf);
      };
      // Copies dealt out over a phase's 16 steps.  NW = 16: one per step, rows 0..7 of group lo, then of group hi;
      // NW = 8: group lo only, every other step.
      struct Weave { Rows lo, hi; };
      // One half (HF 0: x columns, 1: h columns) of one row block's products: rows 32 SUB.. of half buffer hbuf, into
      // am / ar.  EPI: the activations of ANOTHER block, from em / er, cp, are dealt out over the steps as well and
      // end in staging buffer esbuf.  A step's fragments are requested a step ahead.
      auto block_products = [&](const unsigned char* hbuf, auto sub_c, auto hf_c, v16f& am, v16f& ar, auto nw_c, const Weave& w,
                                auto epi_c, const v16f& em, const v16f& er, const float4& ecp, int esbuf, auto&& late) __attribute__((always_inline)) {
        constexpr int SUB = decltype(sub_c)::value, hf = decltype(hf_c)::value, NW = decltype(nw_c)::value;
        constexpr bool EPI = decltype(epi_c)::value;
        // (fp16 data: batch row jb of the block is half jb & 1 of tile row jb >> 1, and has no second plane)
        const _Float16* row = P16 ? reinterpret_cast<const _Float16*>(hbuf + (TR * SUB + (jb >> 1)) * HLD + (jb & 1) * RB) + 8 * hh
                                  : reinterpret_cast<const _Float16*>(hbuf + (TR * SUB + j) * HLD) + 8 * hh;
        constexpr int RO = P16 ? 0 : PH;   // where a row's second plane starts (fp16 elements)
        float hv[4], cv[4];
        v8h bt = *reinterpret_cast<const v8h*>(row), br = *reinterpret_cast<const v8h*>(row + RO);
        v8h nt = *reinterpret_cast<const v8h*>(row + 16), nr = *reinterpret_cast<const v8h*>(row + RO + 16);
        float4 sb = make_float4(0.f, 0.f, 0.f, 0.f);
        if constexpr (EPI) sb = gate_entry(IC<0>{});
        static_for<16>([&](auto s_c) __attribute__((always_inline)) {
          constexpr int sidx = decltype(s_c)::value;
          constexpr int qq = 16 * hf + sidx;
          constexpr bool first = hf == 0 && sidx == 0;
          v8h n2t = nt, n2r = nr;
          float4 nsb = sb;
          if constexpr (sidx + 2 < 16) {
            n2t = *reinterpret_cast<const v8h*>(row + 16 * (sidx + 2));
            if constexpr (!P16) n2r = *reinterpret_cast<const v8h*>(row + RO + 16 * (sidx + 2));
          }
          if constexpr (sidx + 1 < 16) {
            if constexpr (EPI) nsb = gate_entry(IC<sidx + 1>{});
          }
          if constexpr (P16) {   // one product per step, all into one accumulator (see below)
            am = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh[P16 ? qq : 0], bt, first ? zero16 : am, 0, 0, 0);
          } else {
            // (all three into one accumulator: the remainder planes are unscaled, and beside the activations of another
            // block nothing waits for this sum, so a chain of MFMAs that add to one another costs nothing here and saves
            // the activations a second accumulator to read and fold in)
            am = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi[SPLIT ? qq : 0], bt, first ? zero16 : am, 0, 0, 0);
            am = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi[SPLIT ? qq : 0], br, am, 0, 0, 0);
            am = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo[SPLIT ? qq : 0], bt, am, 0, 0, 0);
          }
          if constexpr (EPI) {
            pair_piece(em, er, ecp, hv, cv, sb, s_c);
            // the piece's results are pinned to this step: left alone, the compiler moves every piece behind the last
            // step, next to the only place that reads them
            if constexpr ((sidx & 3) == 0) asm volatile("" : "+v"(eg_i), "+v"(tc_e), "+v"(tc_x2));
            if constexpr ((sidx & 3) == 1) asm volatile("" : "+v"(eg_f), "+v"(tc_p), "+v"(tc_r));
            if constexpr ((sidx & 3) == 2) asm volatile("" : "+v"(eg_o), "+v"(cv[sidx >> 2]));
            if constexpr ((sidx & 3) == 3) asm volatile("" : "+v"(hv[sidx >> 2]));
          }
          // the order within the step: next step's fragments (and the piece's table entry) first, then the MFMAs
          // with the piece's vector instructions between them
          if constexpr (P16) {
            __builtin_amdgcn_sched_group_barrier(0x100, EPI ? 2 : 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (EPI) __builtin_amdgcn_sched_group_barrier(0x002, 20, 0);
          } else {
            __builtin_amdgcn_sched_group_barrier(0x100, EPI ? 3 : 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (EPI) __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (EPI) __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          }
          if constexpr (sidx == 13) late();   // something the caller wants issued near the end of the phase
          // (a group is NC copies: NW == 16 puts group lo on the first steps of the phase's first half and group hi on
          // the first of its second half, NW == 8 group lo on the even steps)
          if constexpr (NW == 16 && (sidx & 7) < NC) {
            if (sidx < 8 ? w.lo.on : w.hi.on) copy_row(sidx < 8 ? w.lo : w.hi, IC<(sidx & 7)>{});
          } else if constexpr (NW == 8 && (sidx & 1) == 0 && (sidx >> 1) < NC) {
            if (w.lo.on) copy_row(w.lo, IC<(sidx >> 1)>{});
          }
          bt = nt; br = nr; nt = n2t; nr = n2r; sb = nsb;
        });
        if constexpr (EPI) stage_results(hv, cv, esbuf);
      };
      const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
      v16f am0, ar0, am1, ar1;
      auto nothing = []() {};

      // item 0 is a first step: no h columns
      Pair cur = pair_at(0, 0, 0, 0u), prev = cur;
      alive = wait_below(cur);
      if (alive) {
        copy_ratios(cur);
        if (cur.on0) copy_block(xbase, cur.rb0, xa_lds, 0);
        if (cur.on1) copy_block(xbase, cur.rb1, xa_lds, 1);
      }
      float4 cp0 = zero4, cp1 = zero4;
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      bool b_pending = false;    // block b of item p-1 waits for its activations (they run under Xa of item p)
      bool a_stored = false, b_stored = false;   // stores of item p-1's blocks are on their way, not yet published
      for (int p = 0; p < n_pairs; ++p) {
        if (TRACED && tracing) a.trace[TS * p + 0] = wall_clock64();
        const bool more = p + 1 < n_pairs;
        const Pair nxt = more ? pair_after(cur) : cur;
        const bool has_prev = cur.t >= d;
        const bool on0 = alive && cur.on0, on1 = alive && cur.on1;
        float ratio0 = 1.0f, ratio1 = 1.0f;
        if (!PLAIN && x_rescaled) {
          const float* rr = reinterpret_cast<const float*>(reinterpret_cast<const unsigned char*>(tile) + kRatioOffset);
          ratio0 = rr[j];
          ratio1 = rr[64 + j];
        }
        const int fo = look(fown, has_prev ? cur.tF - dF : cur.tF, cur);   // this layer's flags for the item's h columns
        // (the layer below's flags for the next item's x columns are looked at as late as their use allows: near the
        // end of Xb, for the test behind barrier 1.  How far a layer runs behind the one below is set by how early it
        // has to see those flags.)
        int fb = 0;
        auto look_below = [&]() __attribute__((always_inline)) { fb = look(fbelow, nxt.tF, nxt); };
        // ---- Xa with Eb of the item before; one block only: its h columns are woven here
        const char* hsrc = hbase + (has_prev ? cur.tO - dO : 0);
        Weave wh{rows_of(hsrc, cur.rb0, hb_lds, 0, false), rows_of(hsrc, cur.rb1, hb_lds, 1, false)};
        if (on0 && !on1 && has_prev) {
          if (!all_set(fo)) alive = wait_own(cur);
          asm volatile("" ::: "memory");
          wh.lo.on = alive;
        }
        if (on0) {
          if (b_pending) block_products(xa, IC<0>{}, IC<0>{}, am0, ar0, IC<8>{}, wh, std::true_type{}, am1, ar1, cp1, 1, nothing);
          else block_products(xa, IC<0>{}, IC<0>{}, am0, ar0, IC<8>{}, wh, std::false_type{}, am1, ar1, cp1, 1, nothing);
          if (!PLAIN && x_rescaled) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { am0[r] *= ratio0; ar0[r] *= ratio0; }
          }
        } else if (b_pending) {
          activations_alone(am1, ar1, cp1, 1);
        }
        b_pending = false;
        if (TRACED && tracing) a.trace[TS * p + 1] = wall_clock64();
        // ---- Xb | h columns of both blocks -> HB
        if (on1) {
          if (has_prev) {
            if (!all_set(fo)) alive = wait_own(cur);
            asm volatile("" ::: "memory");
            wh.lo.on = wh.hi.on = alive;
          }
          block_products(xa, IC<1>{}, IC<0>{}, am1, ar1, IC<16>{}, wh, std::false_type{}, am1, ar1, cp1, 1, look_below);
          if (!PLAIN && x_rescaled) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { am1[r] *= ratio1; ar1[r] *= ratio1; }
          }
        } else {
          look_below();
        }
        if (TRACED && tracing) a.trace[TS * p + 2] = wall_clock64();
        wait_all();
        if (a_stored) publish_block(prev.tF, prev.rb0, prev.on0);
        a_stored = false;
        barrier();   // 1: HB and staging 1 complete, XA free
        if (TRACED && tracing) a.trace[TS * p + 3] = wall_clock64();
        if (p > 0) { store_rows(prev.t, prev.tO, prev.rb1, prev.on1, 1); b_stored = true; }
        const bool cp1_loads = alive && cur.on1 && has_prev;
        cp1 = cprev_rows(cur.t, cur.tO - dO, cur.rb1, cur.on1 && has_prev);
        // ---- Ha, Hb with Ea | x columns of the next item -> XA
        const bool x_ok = more && alive && (l == 0 || all_set(fb));
        asm volatile("" ::: "memory");
        if (x_ok) copy_ratios(nxt);
        const char* xsrc = xbase + nxt.tO;
        Weave wx{rows_of(xsrc, nxt.rb0, xa_lds, 0, x_ok && nxt.on0), rows_of(xsrc, nxt.rb1, xa_lds, 1, x_ok && nxt.on1)};
        if (on0 && has_prev) {
          block_products(hb, IC<0>{}, IC<1>{}, am0, ar0, IC<8>{}, wx, std::false_type{}, am0, ar0, cp0, 0, nothing);
          // block b of the item before: its stores left before Ha.  Published here instead of behind barrier 2, the
          // layer above sees it a quarter of an item earlier, and runs that much closer.
          // (Not with fp16 data: Ha is a third as long there, the acknowledgement of the stores has not come back
          // when it ends, and the wait costs more than the earlier publication gains: 1.26 against 1.23 ms.)
          if (b_stored && !P16) {
            wait_stores_behind(cp1_loads, wx.lo.on);
            publish_block(prev.tF, prev.rb1, prev.on1);
            b_stored = false;
          }
          wx.lo = wx.hi;
          wx.hi.on = false;   // block b's rows on the first eight steps: they have landed when the phase ends
          if (TRACED && tracing) a.trace[TS * p + 4] = wall_clock64();
          if (on1) block_products(hb, IC<1>{}, IC<1>{}, am1, ar1, IC<16>{}, wx, std::true_type{}, am0, ar0, cp0, 0, nothing);
          else {
            if (wx.lo.on) copy_block(xsrc, nxt.rb1, xa_lds, 1);
            activations_alone(am0, ar0, cp0, 0);
          }
        } else {
          if (x_ok && nxt.on0) copy_block(xsrc, nxt.rb0, xa_lds, 0);
          if (x_ok && nxt.on1) copy_block(xsrc, nxt.rb1, xa_lds, 1);
          if (TRACED && tracing) a.trace[TS * p + 4] = wall_clock64();
          if (on0) activations_alone(am0, ar0, cp0, 0);
        }
        b_pending = on1;
        if (TRACED && tracing) a.trace[TS * p + 5] = wall_clock64();
        if (more && !x_ok) {   // the layer below was not ready at barrier 1
          if (alive) alive = wait_below(nxt);
          if (alive) {
            copy_ratios(nxt);
            if (nxt.on0) copy_block(xsrc, nxt.rb0, xa_lds, 0);
            if (nxt.on1) copy_block(xsrc, nxt.rb1, xa_lds, 1);
          }
        }
        wait_all();
        if (b_stored) publish_block(prev.tF, prev.rb1, prev.on1);
        b_stored = false;
        barrier();   // 2: XA and staging 0 complete, HB free
        if (TRACED && tracing) a.trace[TS * p + 6] = wall_clock64();
        store_rows(cur.t, cur.tO, cur.rb0, cur.on0, 0);
        a_stored = true;
        if (more) cp0 = cprev_rows(nxt.t, nxt.tO - dO, nxt.rb0, nxt.on0 && nxt.t >= d);
        if (TRACED && tracing) a.trace[TS * p + 7] = wall_clock64();
        prev = cur;
        cur = nxt;
      }
      // the last item's second block
      if (b_pending) activations_alone(am1, ar1, cp1, 1);
      wait_all();
      if (a_stored) publish_block(prev.tF, prev.rb0, prev.on0);
      barrier();
      store_rows(prev.t, prev.tO, prev.rb1, prev.on1, 1);
      wait_all();
      publish_block(prev.tF, prev.rb1, prev.on1);
      };
      if (a.ragged || my_rbs % 2 != 0 || x_rescaled) paired_schedule(std::false_type{}, std::true_type{});
      else if (q == a.trace_q) paired_schedule(std::true_type{}, std::true_type{});
      else paired_schedule(std::true_type{}, std::false_type{});
      return;
    }
  }

  // ---- pipelined schedule.  Per item n:
  //   the MFMAs;
  //   if tile n+1 has not been requested yet: a look at its producers' completion counts (asked for when
  //     the item began), and the request if they are complete.  The counts of tile n+2 are asked for;
  //   activations and state update, results into the LDS staging area;
  //   everything outstanding is waited for (tiles on their way, and the stores of item n-1, which left an
  //     item ago), item n-1 is counted as complete, barrier: item n's tile buffer is free;
  //   the stores of item n leave (first: the sooner they are acknowledged the sooner the item counts);
  //     the loads item n+1 needs are issued; if tile n+2's producers were complete, the tile is requested
  //     now, a whole item ahead;
  //   a wave that still has not been able to request its part of tile n+1 waits for the producers now --
  //     after counting item n itself, which is what the layer above is waiting for while the wavefront
  //     fills;
  //   barrier: tile n+1 is complete.
  // Loads and stores share one counter of outstanding operations, and completion is reported in issue
  // order: the result of a load is known to have arrived only once everything issued before it, stores
  // included, has completed, so a look at completion counts less than about 2 us after an item's stores
  // have left waits for their acknowledgement.  Hence the order above: what is asked for before the barrier costs no
  // wait of its own, and an item that finds its successor's tile already requested touches no load
  // result until its MFMAs are done.  With split
  // products an item's MFMAs take less than those 2 us, so the only look inside an item is the one after
  // them; with fp32 products there is time for a look after every quarter of a half, and the previous
  // item is counted half way through the x half.
  constexpr int kFirstLook = MODE == kProductsF32 ? 0 : 7;
  alive = wait_deps(0);
  if (alive) issue_tile(0, 0);
  float4 cp = load_cprev(0);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  bool counted = true;                 // nothing to count before item 0
  bool pending = alive && n_items > 1;  // tile n+1 still to be requested
  Flags fl{0, 0};
  for (int n = 0; n < n_items; ++n) {
    const int buf = n & 1;
    if (tracing) a.trace[TS * n + 0] = wall_clock64();
    const bool has_prev = item_t(n) >= d;
    const float ratio = load_ratio(buf);   // tile n has landed (the barrier that ended the item before)
    int looks = 0;  // looks taken inside the item (for the trace)
    if (pending) fl = request_flags(n + 1);

    auto look = [&](int point) __attribute__((always_inline)) {
      if (pending && point >= kFirstLook) {
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

    const bool on = live(n);
    if (on) {
      mfma_range(buf, IC<0>{}, IC<0>{}, IC<4>{});
      look(0);
      mfma_range(buf, IC<0>{}, IC<4>{}, IC<8>{});
      look(1);
      if (MODE == kProductsF32 && !counted) { publish(n - 1); counted = true; }
      mfma_range(buf, IC<0>{}, IC<8>{}, IC<12>{});
      look(2);
      mfma_range(buf, IC<0>{}, IC<12>{}, IC<16>{});
      look(3);
      rescale_x(ratio);
      if (tracing) a.trace[TS * n + 1] = wall_clock64();
      if (has_prev) {
        mfma_range(buf, IC<1>{}, IC<0>{}, IC<4>{});
        look(4);
        mfma_range(buf, IC<1>{}, IC<4>{}, IC<8>{});
        look(5);
        mfma_range(buf, IC<1>{}, IC<8>{}, IC<12>{});
        look(6);
        mfma_range(buf, IC<1>{}, IC<12>{}, IC<16>{});
      }
    }
    if (tracing) a.trace[TS * n + 2] = wall_clock64();
    look(7);
    // Split products: item n-1 is counted here, before the activations.  Its stores left an MFMA phase and a look
    // ago (about 2 us: acknowledged by now), and the layer above gets the count 1 us earlier than after the
    // activations.  The counts of tile n+2 are asked for after that, not before: the wait inside publish() would
    // otherwise sit out their latency too, which the activations hide.
    if (MODE == kProductsSplit && !counted) { publish(n - 1); counted = true; }
    bool pending2 = alive && n + 2 < n_items;  // tile n+2 still to be requested
    Flags fl2{0, 0};
    if (pending2) fl2 = request_flags(n + 2);
    if (tracing) a.trace[TS * n + 3] = wall_clock64() | ((long long)(pending ? 7 : min(looks, 6)) << 60);
    if (on) epilogue_to_lds(gate_sums(), cp, buf);
    if (tracing) a.trace[TS * n + 4] = wall_clock64();
    if (!counted) publish(n - 1);
    else __builtin_amdgcn_s_waitcnt(0);
    // the counts asked for after the MFMAs have arrived with everything else: one more chance before the slow path
    // (not with fp16 data: an item is short there, and the extra request of counts behind a failed look costs more
    // than the look gains: 1.96 -> 2.36 ms at H = 256)
    // A tile requested here leaves AFTER the wait above, and nothing later in the item waits for it (the copies are
    // opaque to the compiler, and a wave only ever waits for its own): the wave waits for them on the spot.
    if constexpr (!F16) {
      const bool was_pending = pending;
      look(8);
      if (was_pending && !pending) __builtin_amdgcn_s_waitcnt(0);   // only the copies are outstanding here: no store has left yet
    }
    barrier();
    if (tracing) a.trace[TS * n + 5] = wall_clock64();
    store_item(n, buf);
    counted = false;
    if (tracing) a.trace[TS * n + 6] = wall_clock64();
    if (n + 1 < n_items) cp = load_cprev(n + 1);
    if (pending2 && !pending && flags_ready(fl2)) {
      issue_tile(n + 2, buf);
      pending2 = false;
    }
    if (pending) {
      publish(n);
      counted = true;
      alive = wait_deps(n + 1);
      if (alive) issue_tile(n + 1, buf ^ 1);
      __builtin_amdgcn_s_waitcnt(0);
    }
    barrier();   // tile n+1 is complete: every wave that requested a part of it has waited for that part
    if (tracing) a.trace[TS * n + 7] = wall_clock64();
    pending = pending2 && alive;
    fl = fl2;
  }
  if (!counted) publish(n_items - 1);
}

__global__ void fill_zero_kernel(int* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

// Split mode, before the persistent kernel: every input row as its two fp16
// planes, with the row's own power-of-two scale.  One wave per row of 256.
// Input rows -> their two fp16 planes and the factor that takes their products to h's scale.  A row whose largest
// magnitude is zero or in [2^-15, 2^4 (1 - 2^-11)] takes the common scale 2^kSplitCommon: its largest element stays
// finite in fp16 and the planes keep 22 bits of it (its remainder is no fp16 subnormal), as with a scale of the row's own.  Any other row gets a scale of
// its own, and *own_scales says that there is one.
__global__ __launch_bounds__(256) void lstm_split_rows_kernel(const float* xs, _Float16* xsp, float* xratio, int* own_scales, int rows) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float4 v = *reinterpret_cast<const float4*>(xs + (size_t)row * PH + 4 * lane);
  float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  int eb = min(max((int)((__float_as_uint(m) >> 23) & 0xff), 15), 254);
  const bool common = m == 0.0f || (m >= 0x1p-15f && m <= 16.0f * (1.0f - 0x1p-11f));
  if (common) eb = 127 + kSplitTop - kSplitCommon;   // the exponent whose own scale is the common one
  else if (lane == 0) __hip_atomic_store(own_scales, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const float scale = __uint_as_float((unsigned)(127 + kSplitTop + 127 - eb) << 23);
  const float vs[4] = {v.x * scale, v.y * scale, v.z * scale, v.w * scale};
  v4h top, rest;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    top[r] = (_Float16)vs[r];
    rest[r] = (_Float16)(vs[r] - (float)top[r]);
  }
  _Float16* dst = xsp + (size_t)row * (2 * PH) + 4 * lane;
  *reinterpret_cast<v4h*>(dst) = top;
  *reinterpret_cast<v4h*>(dst + PH) = rest;
  // the row's products carry 2^(141 - eb), h's carry 2^14: the ratio is 2^(eb - 127)
  if (lane == 0) xratio[row] = __uint_as_float((unsigned)eb << 23);
}

static size_t flag_count(int L, int T, int B) {
  const int nrb = (B + 31) / 32;
  return (size_t)L * T * nrb * (kFlagStride / sizeof(int));
}

// Workspace layout: [64 ints: status][flags][trace: T*nrb*8 stamps of 8 bytes]
// and, for the split-product mode, [xratio: T*B floats][xsp: T*B rows][hsp: L*T*B rows]
// of 1024 bytes each, every part on a 256-byte boundary.
static size_t trace_offset_bytes(int L, int T, int B) { return ((flag_count(L, T, B) + 64) * sizeof(int) + 15) / 16 * 16; }
static size_t round256(size_t v) { return (v + 255) / 256 * 256; }
static size_t xratio_offset_bytes(int L, int T, int B) {
  return round256(trace_offset_bytes(L, T, B) + (size_t)T * ((B + 31) / 32) * 8 * sizeof(long long));
}
static size_t xsp_offset_bytes(int L, int T, int B) { return round256(xratio_offset_bytes(L, T, B) + (size_t)T * B * sizeof(float)); }
static size_t hsp_offset_bytes(int L, int T, int B) { return xsp_offset_bytes(L, T, B) + (size_t)T * B * 2 * PH * sizeof(_Float16); }
static size_t workspace_need(int L, int T, int B) {
  return hsp_offset_bytes(L, T, B) + (size_t)L * T * B * 2 * PH * sizeof(_Float16);
}

// Polls a bounded wait makes before it gives up (a poll is a round trip to memory, about 1 us: seconds in all).
constexpr int kDefaultSpinLimit = 1 << 22;

// 0: fp32 products (v_mfma_f32_32x32x2_f32); 1: split products.  FTK_LSTM_PRODUCTS=f32|f16x3
// sets the initial value, ftk_lstm_set_products() changes it.
static int g_products = -1;
static int products_mode() {
  if (g_products < 0) {
    const char* e = getenv("FTK_LSTM_PRODUCTS");
    g_products = (e && (e[0] == 'f' && e[1] == '3')) ? 0 : 1;
  }
  return g_products;
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

template <int MODE>
static int persistent_function(const void** fn, size_t lds) {
  static DeviceOnce attr_once;
  *fn = (const void*)lstm_persistent_kernel<MODE>;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute(*fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_once.done(attr_bit);
  }
  return FTK_OK;
}

// Co-resident workgroups the device offers the persistent kernel of a flavour (0 if it cannot run at all).
static int persistent_slots(int mode, const void** fn, int* slots) {
  *slots = 0;
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  const size_t lds = kPersistLds;
  if ((int)lds > dp->lds_optin) return FTK_OK;
  rc = mode == kHalfData ? persistent_function<kHalfData>(fn, lds)
       : mode == kHalfData256 ? persistent_function<kHalfData256>(fn, lds)
       : mode == kProductsSplit ? persistent_function<kProductsSplit>(fn, lds)
                                : persistent_function<kProductsF32>(fn, lds);
  if (rc) return rc;
  int per_cu = 0;
  FTK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, *fn, 256, lds));
  *slots = per_cu * dp->cus;
  return FTK_OK;
}

// mode kProductsF32 / kProductsSplit: fp32 xs, WU, hsss, csss, H = 256.  kHalfData: the same arrays in fp16, H = 512.
static int run_persistent(int mode, const void* xs, const void* WU, const float* bias, const int* dil, const int* active,
                          void* hsss, void* csss, int L, int T, int B, void* ws, size_t ws_bytes, hipStream_t s,
                          bool* handled, int spin_limit = 0, bool keep_status = false) {
  *handled = false;
  const void* fn = nullptr;
  int slots = 0;
  int rc = persistent_slots(mode, &fn, &slots);
  if (rc) return rc;
  const size_t lds = kPersistLds;
  const bool split = mode == kProductsSplit;
  const bool half = mode == kHalfData || mode == kHalfData256;
  const int npc = mode == kHalfData ? 16 : PC;  // column slices (workgroups) per layer
  if (L > kMaxLayers || L * npc > slots) return FTK_OK;  // cannot pin every layer on its own compute units: fall back

  const size_t nflags = flag_count(L, T, B);
  // only the split products read planes; the other flavours need the status block, the flags and the trace
  const size_t need = split ? workspace_need(L, T, B) : xratio_offset_bytes(L, T, B);
  if (!ws || ws_bytes < need)
    return fail(FTK_ERR_WORKSPACE, "stacked LSTM needs a %zu-byte workspace, got %zu", need, ws_bytes);

  PersistArgs a;
  a.xs = reinterpret_cast<const float*>(xs);
  a.WU = reinterpret_cast<const float*>(WU);
  a.bias = bias;
  a.hsss = reinterpret_cast<float*>(hsss);
  a.csss = reinterpret_cast<float*>(csss);
  a.status = reinterpret_cast<int*>(ws);
  a.flags = reinterpret_cast<unsigned char*>(a.status + 64);
  char* wsb = reinterpret_cast<char*>(ws);
  float* xratio = nullptr;
  _Float16* xsp = nullptr;
  if (half) {  // the kernel reads its tiles from the fp16 arrays themselves
    a.xratio = nullptr;
    a.xsp = reinterpret_cast<const _Float16*>(xs);
    a.hsp = reinterpret_cast<_Float16*>(hsss);
  } else if (!split) {  // fp32 products: tiles come from xs and hsss
    a.xratio = nullptr;
    a.xsp = nullptr;
    a.hsp = nullptr;
  } else {
    xratio = reinterpret_cast<float*>(wsb + xratio_offset_bytes(L, T, B));
    xsp = reinterpret_cast<_Float16*>(wsb + xsp_offset_bytes(L, T, B));
    a.xratio = xratio;
    a.xsp = xsp;
    a.hsp = reinterpret_cast<_Float16*>(wsb + hsp_offset_bytes(L, T, B));
  }
  a.L = L; a.T = T; a.B = B;
  a.nrb = (B + 31) / 32;
  // spare compute units become row slices, but a workgroup keeps at least two
  // row blocks when it can so that the next tile never depends on the current item
  const int pr = std::max(1, std::min(slots / (L * npc), std::max(1, a.nrb / 2)));
  int used = 0;
  for (int l = 0; l < L; ++l) {
    a.pr_of[l] = pr;
    used += npc * pr;
  }
  // A layer whose own chain is shorter than four items (dilation x row blocks per workgroup) cannot have the
  // next tile under way while it works on an item: each of its items then costs a whole hand-over.  Such a
  // layer gets one row block per workgroup where compute units are left, so that a time step costs it one
  // hand-over instead of one per row block it walks.
  for (int l = 0; l < L; ++l) {
    const int d = dil ? dil[l] : 1;
    const int my_rbs = (a.nrb + pr - 1) / pr;
    if (d * my_rbs < 4 && my_rbs > 1 && used - npc * pr + npc * a.nrb <= slots && !getenv("FTK_LSTM_UNIFORM_SLICES")) {
      used += npc * (a.nrb - pr);
      a.pr_of[l] = a.nrb;
    }
  }
  a.first_q[0] = 0;
  for (int l = 0; l < L; ++l) a.first_q[l + 1] = a.first_q[l] + npc * a.pr_of[l];
  for (int l = L; l < kMaxLayers; ++l) { a.pr_of[l] = 1; a.first_q[l + 1] = a.first_q[L]; }
  a.groups = a.first_q[L];
  a.spin_limit = spin_limit > 0 ? spin_limit : kDefaultSpinLimit;
  a.trace_q = trace_workgroup();
  a.trace = reinterpret_cast<long long*>(reinterpret_cast<char*>(ws) + trace_offset_bytes(L, T, B));
  for (int l = 0; l < kMaxLayers; ++l) a.dil[l] = (l < L && dil) ? dil[l] : 1;
  // ragged batch: how many steps each 32-row block takes part in (its first row is its longest).  Batches
  // with more blocks than the table holds are computed in full, which gives the same live rows.
  a.ragged = (active && a.nrb <= kMaxBlocks) ? 1 : 0;
  for (int rb = 0; rb < kMaxBlocks; ++rb) {
    int steps = T;
    if (a.ragged) {
      steps = 0;
      while (steps < T && active[steps] > 32 * rb) ++steps;
    }
    a.steps_of[rb] = steps;
  }
  int grid = a.groups;
  a.xcd_remap = (grid % 8 == 0) ? 1 : 0;
  // Placement.  A unit is the npc workgroups that share a layer's rows (its column slices): they exchange h at every
  // step, and a unit stays on one XCD.  Units go to the XCDs in turn, unit u to XCD u % 8, so that consecutive layers
  // of a deep stack sit on different XCDs: the
  // layers at the bottom of a stack never wait and set the pace of all the others, which wait a little in every
  // item, and an XCD that holds only layers of the first kind runs every phase about 8 % slower than one that holds
  // only layers of the second (the clock follows what the XCD does), so the pacing layers are better spread, each
  // beside layers that leave the XCD some slack.  The grid is rounded up to whole units per XCD; workgroups beyond the
  // last unit leave at once.  (FTK_LSTM_LAYER_BLOCKS=1: the older placement, workgroups in order, grid / 8 per XCD.)
  {
    const int units = a.groups / npc, per_xcd = ((units + 7) / 8) * npc;
    static const bool blocks = getenv("FTK_LSTM_LAYER_BLOCKS") && atoi(getenv("FTK_LSTM_LAYER_BLOCKS")) != 0;
    if (npc > 1 && 8 * per_xcd <= slots && !blocks) {
      a.xcd_remap = npc;
      grid = 8 * per_xcd;
    }
  }
  // FTK_LSTM_PAIRS=0: pipelined layers of the split-product kernel walk single row blocks (the older schedule)
  static const bool pairs_off = getenv("FTK_LSTM_PAIRS") && atoi(getenv("FTK_LSTM_PAIRS")) == 0;
  a.paired = ((split || mode == kHalfData256) && !pairs_off && B % 8 == 0) ? 1 : 0;

  // flags and status block start from zero; a later launch of a stack that runs as several keeps the error word
  // of the earlier ones (it then drains at its first long wait, and the call reports the time-out)
  // (and its word for small states, see ftk_stacked_lstm_small_states)
  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, a.status + (keep_status ? 2 : 0),
                     nflags + 64 - (keep_status ? 2 : 0));
  rc = check_launch("fill_zero_kernel");
  if (rc) return rc;

  if (split) {
    const int rows = T * B;
    hipLaunchKernelGGL(lstm_split_rows_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, a.xs, xsp, xratio, a.status + 2, rows);
    rc = check_launch("lstm_split_rows_kernel");
    if (rc) return rc;
  }

  void* kargs[] = {&a};
  if (plain_launch()) {
    if (mode == kHalfData) hipLaunchKernelGGL(lstm_persistent_kernel<kHalfData>, dim3(grid), dim3(256), lds, s, a);
    else if (mode == kHalfData256) hipLaunchKernelGGL(lstm_persistent_kernel<kHalfData256>, dim3(grid), dim3(256), lds, s, a);
    else if (split) hipLaunchKernelGGL(lstm_persistent_kernel<kProductsSplit>, dim3(grid), dim3(256), lds, s, a);
    else hipLaunchKernelGGL(lstm_persistent_kernel<kProductsF32>, dim3(grid), dim3(256), lds, s, a);
    rc = check_launch("lstm_persistent_kernel");
    if (rc) return rc;
  } else {
    FTK_HIP(hipLaunchCooperativeKernel(fn, dim3(grid), dim3(256), kargs, (unsigned)lds, s));
  }
  *handled = true;
  return FTK_OK;
}

// Scratch of the entry point that allocates nothing: the status block, the flags and the trace of one persistent
// launch with fp32 products.  Every device the library runs on holds its own copy until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress; device code and launches use the address that call
// returns, kept per device.
constexpr size_t kScratchBytes = 2u << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// The device address of `scratch` on the current device (looked up once per device, with that device current).
static int scratch_of_current_device(const char* who, void** out, bool lookup) {
  *out = nullptr;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(FTK_ERR_DEVICE, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  }
  if (dev < 0 || dev >= kMaxDevices) return fail(FTK_ERR_DEVICE, "%s: device id %d is outside [0, %d)", who, dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev] && lookup) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return fail(FTK_ERR_DEVICE, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
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
                     const int* active, float* hsss, float* csss, int L, int T, int B, int H, void* ws,
                     size_t ws_bytes, hipStream_t s, int products = FTK_LSTM_PRODUCTS_DEFAULT, int spin_limit = 0) {
  int rc = check_stack_args(who, xs, WU, hsss, csss, L, T, B, H, dil);
  if (rc) return rc;
  if (products == FTK_LSTM_PRODUCTS_DEFAULT) products = products_mode();
  if (products != FTK_LSTM_PRODUCTS_F32 && products != FTK_LSTM_PRODUCTS_F16X3)
    return fail(FTK_ERR_INVALID_ARGUMENT, "%s: products = %d is none of FTK_LSTM_PRODUCTS_DEFAULT, _F32, _F16X3", who, products);
  if (spin_limit < 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: spin_limit = %d is negative", who, spin_limit);
  if (active) {
    for (int t = 0; t < T; ++t) {
      if (active[t] < 0 || active[t] > B)
        return fail(FTK_ERR_INVALID_ARGUMENT, "%s: active_rows[%d]=%d is outside [0, B=%d]", who, t, active[t], B);
      if (t > 0 && active[t] > active[t - 1])
        return fail(FTK_ERR_INVALID_ARGUMENT, "%s: active_rows must be non-increasing (rows sorted by length), but [%d]=%d > [%d]=%d",
                    who, t, active[t], t - 1, active[t - 1]);
    }
  }
  if (H == PH) {
    // A stack deeper than the chip holds at eight workgroups a layer runs as consecutive persistent launches: a
    // launch reads the hidden sequence of the layer below it, complete by then, like the first reads xs.
    const int mode = products == FTK_LSTM_PRODUCTS_F16X3 ? kProductsSplit : kProductsF32;
    const void* fn = nullptr;
    int slots = 0;
    rc = persistent_slots(mode, &fn, &slots);
    if (rc) return rc;
    const int chunk = std::min(slots / PC, kMaxLayers);
    const size_t slab = (size_t)T * B * H;
    bool handled = chunk >= 1;
    for (int l0 = 0; handled && l0 < L; l0 += chunk) {
      const int lc = std::min(chunk, L - l0);
      rc = run_persistent(mode, l0 == 0 ? xs : hsss + (size_t)(l0 - 1) * slab, WU + (size_t)l0 * 2 * H * 4 * H,
                          bias ? bias + (size_t)l0 * 4 * H : nullptr, dil ? dil + l0 : nullptr, active,
                          hsss + (size_t)l0 * slab, csss + (size_t)l0 * slab, lc, T, B, ws, ws_bytes, s, &handled,
                          spin_limit, l0 > 0);
      if (rc) return rc;
      if (!handled && l0 > 0) return fail(FTK_ERR_DEVICE, "%s: the persistent kernel ran for the first %d layers only", who, l0);
    }
    if (handled) return FTK_OK;
  }
  // the launches below wait for nothing: their status word is zero
  if (ws && ws_bytes >= kStatusBytes) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, s, reinterpret_cast<int*>(ws), (size_t)(kStatusBytes / sizeof(int)));
    rc = check_launch("fill_zero_kernel");
    if (rc) return rc;
  }
  // Other hidden sizes: one launch per stage of independent cells.  With split products (the default) and the
  // workspace the size query asks for, through the fp16-MFMA streaming kernel; else on fp32 MFMAs.
  if (H != PH && products == FTK_LSTM_PRODUCTS_F16X3 && ws && ws_bytes >= split_stack_workspace_bytes(L, T, B, H) &&
      (long long)B * H < (1ll << 29))
    return run_wavefront_split(xs, WU, bias, dil, active, hsss, csss, L, T, B, H, ws, s);
  return run_wavefront(xs, WU, bias, dil, hsss, csss, L, T, B, H, s);
}

}  // namespace ftk

namespace ftk {

// The persistent kernel holds the fp16 weights of H = 512, and of H = 256 with two batch rows per tile row (even B).
static bool f16_fits_on_chip(int B, int H) { return H == 2 * PH || (H == PH && !(B & 1)); }

// Whether the fp16 stack goes through the streaming cell kernel, one launch per stage of cells.  Always where the
// weights do not fit on chip; at H = 512 also when the stack is deeper than the 16 layers that 256 compute units
// hold at once: the persistent kernel then runs twice and fills its wavefront twice (5.5 ms at L = 32, T = 64,
// B = 256), while the streamed cells find the 134 MB of weights in the last-level cache (3.75 ms).  A ragged
// batch stays with the persistent kernel, which skips the row blocks that have ended.
// FTK_LSTM_F16_STREAM=1 / =0 in the environment forces the one or the other where both can run.
static bool f16_streams(int L, int B, int H, bool ragged) {
  if (!f16_fits_on_chip(B, H)) return true;
  if (const char* e = getenv("FTK_LSTM_F16_STREAM")) return e[0] == '1';
  return H == 2 * PH && L > 16 && !ragged;
}

}  // namespace ftk

extern "C" {

size_t ftk_stacked_lstm_workspace_bytes(int L, int T, int B, int H) {
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0) return 0;
  if (H != ftk::PH && H % 32 == 0) return ftk::split_stack_workspace_bytes(L, T, B, H);  // planes, scales, re-laid weights
  return ftk::workspace_need(L, T, B);
}

size_t ftk_stacked_lstm_f16_workspace_bytes(int L, int T, int B, int H) {
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0) return 0;
  // the status block and the re-laid weights of the streaming kernel
  const size_t packed = ftk::kStatusBytes + (size_t)L * 2 * H * 4 * H * sizeof(_Float16);
  if (!ftk::f16_fits_on_chip(B, H)) return packed;
  // which of the two runs is decided per call (a ragged batch stays with the persistent kernel): room for either
  return std::max(ftk::xratio_offset_bytes(L, T, B), ftk::f16_streams(L, B, H, false) ? packed : (size_t)0);
}

int ftk_stacked_lstm_f16(const void* xs, const void* WU, const float* bias, const int* dilations,
                         const int* active_rows, void* hsss, void* csss, int L, int T, int B, int H, void* workspace,
                         size_t workspace_bytes, ftk_stream_t stream) {
  using namespace ftk;
  const char* who = "ftk_stacked_lstm_f16";
  if (!xs || !WU || !hsss || !csss) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: xs, WU, hsss, csss must be non-NULL", who);
  if (L <= 0 || T <= 0 || B <= 0 || H <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: L, T, B, H must be positive", who);
  if (H % 32) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: H=%d must be a multiple of 32", who, H);
  if ((long long)B * H >= (1ll << 30)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: B*H = %lld is too large", who, (long long)B * H);
  // the persistent kernel holds the weights of H = 512, and of H = 256 with two batch rows per tile row (even B)
  const bool on_chip = !f16_streams(L, B, H, active_rows != nullptr);
  const int mode = H == PH ? kHalfData256 : kHalfData;
  const int npc = H / 32;
  if (dilations)
    for (int l = 0; l < L; ++l)
      if (dilations[l] <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: dilations[%d]=%d must be positive", who, l, dilations[l]);
  if (active_rows)
    for (int t = 0; t < T; ++t) {
      if (active_rows[t] < 0 || active_rows[t] > B)
        return fail(FTK_ERR_INVALID_ARGUMENT, "%s: active_rows[%d]=%d is outside [0, B=%d]", who, t, active_rows[t], B);
      if (t > 0 && active_rows[t] > active_rows[t - 1])
        return fail(FTK_ERR_INVALID_ARGUMENT, "%s: active_rows must be non-increasing (rows sorted by length)", who);
    }
  // every other shape streams the weights, one launch per stage of independent cells (dead rows are computed too)
  // (the workspace takes the weights re-laid per unit block, so that a workgroup reads one contiguous run)
  if (!on_chip) {
    const size_t need = ftk_stacked_lstm_f16_workspace_bytes(L, T, B, H);
    if (!workspace || workspace_bytes < need)
      return fail(FTK_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace ? workspace_bytes : (size_t)0);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, reinterpret_cast<int*>(workspace),
                       (size_t)(kStatusBytes / sizeof(int)));  // nothing below waits: the status word is zero
    int rcz = check_launch("fill_zero_kernel");
    if (rcz) return rcz;
    return run_wavefront_f16(xs, WU, bias, dilations, active_rows, hsss, csss, L, T, B, H,
                             reinterpret_cast<char*>(workspace) + kStatusBytes, (hipStream_t)stream);
  }
  const void* fn = nullptr;
  int slots = 0;
  int rc = persistent_slots(mode, &fn, &slots);
  if (rc) return rc;
  const int chunk = std::min(slots / npc, kMaxLayers);  // layers whose weights fit on the chip at once
  if (chunk < 1) return fail(FTK_ERR_DEVICE, "%s: the device cannot hold one layer's weights in registers", who);
  // deeper stacks run as consecutive launches of `chunk` layers: a chunk reads the hidden sequence of the
  // layer below it, complete by then, like the first chunk reads xs
  const size_t slab = (size_t)T * B * H;  // elements of one layer's h (or c)
  const _Float16* x16 = reinterpret_cast<const _Float16*>(xs);
  const _Float16* w16 = reinterpret_cast<const _Float16*>(WU);
  _Float16* h16 = reinterpret_cast<_Float16*>(hsss);
  _Float16* c16 = reinterpret_cast<_Float16*>(csss);
  for (int l0 = 0; l0 < L; l0 += chunk) {
    const int lc = std::min(chunk, L - l0);
    bool handled = false;
    rc = run_persistent(mode, l0 == 0 ? x16 : h16 + (size_t)(l0 - 1) * slab, w16 + (size_t)l0 * 2 * H * 4 * H,
                        bias ? bias + (size_t)l0 * 4 * H : nullptr, dilations ? dilations + l0 : nullptr, active_rows,
                        h16 + (size_t)l0 * slab, c16 + (size_t)l0 * slab, lc, T, B, workspace, workspace_bytes,
                        (hipStream_t)stream, &handled, 0, l0 > 0);
    if (rc) return rc;
    if (!handled) return fail(FTK_ERR_DEVICE, "%s: the persistent kernel cannot run on this device", who);
  }
  return FTK_OK;
}

int ftk_stacked_lstm_opts_f32(const float* xs, const float* WU, const float* bias, const int* dilations,
                              const int* active_rows, float* hsss, float* csss, int L, int T, int B, int H,
                              const ftk_lstm_options* options, void* workspace, size_t workspace_bytes,
                              ftk_stream_t stream) {
  const int products = options ? options->products : FTK_LSTM_PRODUCTS_DEFAULT;
  const int spin_limit = options ? options->spin_limit : 0;
  return ftk::run_stack("ftk_stacked_lstm_opts_f32", xs, WU, bias, dilations, active_rows, hsss, csss, L, T, B, H,
                        workspace, workspace_bytes, (hipStream_t)stream, products, spin_limit);
}

int ftk_stacked_lstm_status(const void* workspace, ftk_stream_t stream) {
  using namespace ftk;
  if (!workspace) {  // the built-in scratch of ftk_stacked_lstm_noalloc_f32 on the current device
    void* ptr = nullptr;
    if (scratch_of_current_device("ftk_stacked_lstm_status", &ptr, false) != FTK_OK || !ptr)
      return fail(FTK_ERR_INVALID_ARGUMENT,
                  "ftk_stacked_lstm_status: workspace is NULL and ftk_stacked_lstm_noalloc_f32 has not run on the current device");
    workspace = ptr;
  }
  int word = 0;
  FTK_HIP(hipMemcpyAsync(&word, workspace, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream));
  FTK_HIP(hipStreamSynchronize((hipStream_t)stream));
  if (word != 0)
    return fail(FTK_ERR_TIMEOUT,
                "stacked LSTM: a bounded wait of the persistent launch ran out of polls (status word %d); the launch drained "
                "early and hsss / csss are incomplete", word);
  return FTK_OK;
}

int ftk_stacked_lstm_small_states(const void* workspace, ftk_stream_t stream) {
  using namespace ftk;
  if (!workspace) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_stacked_lstm_small_states: workspace is NULL");
  int word = 0;
  FTK_HIP(hipMemcpyAsync(&word, reinterpret_cast<const int*>(workspace) + 1, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream));
  FTK_HIP(hipStreamSynchronize((hipStream_t)stream));
  return word != 0 ? 1 : 0;
}

int ftk_stacked_lstm_noalloc_f32(const float* xs, const float* WU, const float* bias, const int* dilations, float* hsss,
                                 float* csss, int L, int T, int B, int H, ftk_stream_t stream) {
  using namespace ftk;
  const char* who = "ftk_stacked_lstm_noalloc_f32";
  int rc = check_stack_args(who, xs, WU, hsss, csss, L, T, B, H, dilations);
  if (rc) return rc;
  if (H != PH) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: H = %d; only H = %d runs without a caller workspace", who, H, PH);
  const size_t need = xratio_offset_bytes(L, T, B);
  if (need > kScratchBytes)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE,
                "%s: L = %d, T = %d, B = %d needs %zu bytes of flags and trace, the built-in scratch holds %zu; use "
                "ftk_stacked_lstm_opts_f32 with a workspace", who, L, T, B, need, kScratchBytes);
  void* ptr = nullptr;
  rc = scratch_of_current_device(who, &ptr, true);
  if (rc) return rc;
  bool handled = false;
  rc = run_persistent(kProductsF32, xs, WU, bias, dilations, nullptr, hsss, csss, L, T, B, ptr, kScratchBytes,
                      (hipStream_t)stream, &handled, 0);
  if (rc) return rc;
  if (!handled)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: %d layers do not fit the device's compute units in one persistent launch", who, L);
  return FTK_OK;
}

int ftk_lstm_set_products(int mode) {
  if (mode != FTK_LSTM_PRODUCTS_F32 && mode != FTK_LSTM_PRODUCTS_F16X3)
    return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_lstm_set_products: mode %d is neither FTK_LSTM_PRODUCTS_F32 nor FTK_LSTM_PRODUCTS_F16X3", mode);
  ftk::g_products = mode;
  return FTK_OK;
}

int ftk_lstm_get_products(void) { return ftk::products_mode(); }

int ftk_stacked_lstm_f32(const float* xs, const float* WU, const float* bias, float* hsss, float* csss, int L, int T,
                         int B, int H, void* workspace, size_t workspace_bytes, ftk_stream_t stream) {
  return ftk::run_stack("ftk_stacked_lstm_f32", xs, WU, bias, nullptr, nullptr, hsss, csss, L, T, B, H, workspace,
                        workspace_bytes, (hipStream_t)stream);
}

int ftk_dilated_lstm_f32(const float* xs, const float* WU, const float* bias, const int* dilations, float* hsss,
                         float* csss, int L, int T, int B, int H, void* workspace, size_t workspace_bytes,
                         ftk_stream_t stream) {
  if (!dilations) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_dilated_lstm_f32: dilations is NULL");
  return ftk::run_stack("ftk_dilated_lstm_f32", xs, WU, bias, dilations, nullptr, hsss, csss, L, T, B, H, workspace,
                        workspace_bytes, (hipStream_t)stream);
}

int ftk_stacked_lstm_ragged_f32(const float* xs, const float* WU, const float* bias, const int* dilations,
                                const int* active_rows, float* hsss, float* csss, int L, int T, int B, int H,
                                void* workspace, size_t workspace_bytes, ftk_stream_t stream) {
  if (!active_rows) return ftk::fail(FTK_ERR_INVALID_ARGUMENT, "ftk_stacked_lstm_ragged_f32: active_rows is NULL");
  return ftk::run_stack("ftk_stacked_lstm_ragged_f32", xs, WU, bias, dilations, active_rows, hsss, csss, L, T, B, H,
                        workspace, workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
