// Plain fp16 product C = A @ Bm for shapes made of whole 256 x 256 tiles: one wave per SIMD, each with a
// 128 x 128 piece of the workgroup's tile in its accumulators.
//
// The streaming cell kernel (lstm_cell.hip, GEMM flavour) gives a wave 128 x 64 outputs, so every 16 MFMAs read
// 12 KB of fragments from LDS, and its two waves per SIMD meet at the same barrier.  Here a wave owns 128 x 128:
// 32 MFMAs per 16 KB of fragments, a third less LDS traffic per product, and the whole register file (256
// accumulator registers + fragments of two k steps).  With one wave per SIMD nothing fills a gap, so the loop
// leaves none it can avoid: the fragments of a k step are read while the MFMAs of the step before run, across
// the chunk boundary as well -- the barrier sits in the MIDDLE of a chunk, between its two k steps, where the
// second step's fragments are already in registers (what the chunk occupied in LDS is then free for copies) and
// the first step's fragments of the next chunk can be read behind it.
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

template <int V> using GIC = std::integral_constant<int, V>;

constexpr int GT = 256;               // rows and columns of a workgroup's tile
constexpr int GK = 32;                // k chunk: what a Bm stage holds; an A buffer holds a pair of chunks
constexpr int GS = 4;                 // Bm stages
constexpr int GP = 3;                 // A buffers
constexpr int G_ROWB = GT * 2;           // a Bm row of a chunk in LDS
constexpr int G_ABUF = GT * 128;         // A rows of a pair of chunks: 128 bytes, a whole cache line, each (32 KB)
constexpr int G_BST = GK * G_ROWB;       // 16 KB
constexpr int G_B0 = GP * G_ABUF;        // where the Bm stages start
constexpr int G_LDS = G_B0 + GS * G_BST; // 160 KB
constexpr int gemm_vmcnt(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }   // s_waitcnt: vmcnt <= n, nothing else

typedef short g4s __attribute__((ext_vector_type(4)));
typedef short g8s __attribute__((ext_vector_type(8)));

// stage and buffer numbers: integral constants in the loop that is unrolled over them, ints elsewhere
template <int M, int V> __device__ __forceinline__ constexpr GIC<(V + 1) % M> next_of(GIC<V>) { return {}; }
template <int M> __device__ __forceinline__ int next_of(int v) { return v + 1 == M ? 0 : v + 1; }
template <int M, int V> __device__ __forceinline__ constexpr GIC<(V + M - 1) % M> prev_of(GIC<V>) { return {}; }
template <int M> __device__ __forceinline__ int prev_of(int v) { return v == 0 ? M - 1 : v - 1; }

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte offset) into LDS at lds_addr + 16 * lane.
// The compiler does not count it: the loop waits with s_waitcnt vmcnt itself.
__device__ __forceinline__ void gemm_dma16(const void* gbase, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_addr), "v"(byte_off), "s"(gbase) : "memory", "m0");
}

// LDS: three A buffers, then four Bm stages.  An A buffer holds the tile's 256 rows of a pair of chunks, 128 bytes
// = 8 slots of 16 each: row r keeps k slot c in slot c ^ ((r >> 1) & 7) (16 rows in a row of one k slot fall on 16
// different 16-byte bank groups).  A copy brings 8 rows' whole 128-byte lines; with 64-byte rows, a chunk at a time,
// every line of A went from L2 to the compute unit twice.  Bm row k of a chunk (512 bytes, 32 slots = columns
// 8c .. 8c+7 of the tile) keeps slot c in c ^ ((k & 3) << 2).  The MFMA takes the Bm fragment as its first operand and
// the A fragment as its second: lane (j, hh) then holds, of output tile (rt, nt), row 32 rt + j and columns
// 32 nt + 8 q + 4 hh .. + 3 (q = 0..3).
__global__ __launch_bounds__(256, 1) void gemm_f16_tile_kernel(const _Float16* __restrict__ A, const _Float16* __restrict__ Bm,
                                                                _Float16* __restrict__ C, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gemm_smem[];
  using lds_g4s = __attribute__((address_space(3))) g4s;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wr = wave >> 1, wc = wave & 1;
  const int j = lane & 31, hh = lane >> 5;
  // Which tile: workgroups go to the 8 XCDs round-robin by their linear index, and the 32 that an XCD runs together
  // should share operands in its L2.  XCD x takes the x-th eighth of the tiles in walking order, and the walk goes
  // down a band of 8 (4, 2, 1) row blocks before it moves one column block on: 32 tiles in a row of the walk are 8 row
  // blocks x 4 column blocks, 12 operand panels for 32 tiles.
  const int tiles_m = (M + GT - 1) / GT, tiles_n = N / GT, per = tiles_m * tiles_n;
  int v = (int)blockIdx.x;
  if ((gridDim.x & 7) == 0) v = (v & 7) * (int)(gridDim.x >> 3) + (v >> 3);
  const int prob = v / per, t = v % per;
  const int bh = (tiles_m & 7) == 0 ? 8 : (tiles_m & 3) == 0 ? 4 : (tiles_m & 1) == 0 ? 2 : 1;
  const int band = t / (bh * tiles_n), r = t % (bh * tiles_n);
  const int m0 = (band * bh + r % bh) * GT, n0 = (r / bh) * GT;
  A += (size_t)prob * M * K;
  Bm += (size_t)prob * K * N;
  C += (size_t)prob * M * N;
  const unsigned lds0 = (unsigned)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)gemm_smem);
  const int nch = K / GK, npairs = (nch + 1) >> 1;

  // copies: wave w brings A rows 64 w .. + 64 of a pair of chunks (copy i of 8: 8 rows, row lane / 8) and Bm rows
  // 8 w .. + 8 of a chunk (copy i of 4: 2 rows, row lane / 32)
  unsigned b_lane[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const unsigned kr = (unsigned)(2 * p + (lane >> 5));   // k row & 3
    b_lane[p] = ((unsigned)lane >> 5) * (unsigned)(2 * N) + ((((unsigned)lane & 31) ^ (kr << 2)) * 16);
  }
  // a copy's lane offsets from its operand's base; the bases move on by a pair and by a chunk.  (Rows past the end
  // of A repeat its last row; they are never stored.)
  const int a_row0 = min(m0 + 64 * wave, M - 1);
  unsigned a_voff[8], b_voff[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = min(m0 + 64 * wave + 8 * i + (lane >> 3), M - 1);
    a_voff[i] = (unsigned)(row - a_row0) * (unsigned)(2 * K) + (unsigned)(((lane & 7) ^ (4 * (i & 1) + (lane >> 4))) * 16);
    asm volatile("" : "+v"(a_voff[i]));   // kept in registers, not formed again at every copy
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    b_voff[i] = b_lane[i & 1] + (unsigned)i * (unsigned)(2 * 2 * N);
    asm volatile("" : "+v"(b_voff[i]));
  }
  // K an odd number of chunks: the last pair is half a pair, and the lanes of its copies whose k slot lies beyond K
  // take the slot 64 bytes in front of it (what they bring is never read)
  const unsigned a_back[2] = {(unsigned)(((lane >> 2) & 1) * 64), (unsigned)((((lane >> 2) & 1) ^ 1) * 64)};
  const char* a_next = reinterpret_cast<const char*>(A + (size_t)a_row0 * K);   // of the pair that is copied next
  const char* b_next = reinterpret_cast<const char*>(Bm + (size_t)(8 * wave) * N + n0);   // of the chunk ...
  int a_idx = 0, b_idx = 0;   // which pair, which chunk (used outside the unrolled loop only)
  const size_t b_chunk = (size_t)GK * N * 2;
  const unsigned lds_wave_a = lds0 + (unsigned)(wave * 8192);
  const unsigned lds_wave_b = lds0 + (unsigned)(G_B0 + wave * 4096);
  // Copy i (of 8) of the pair at a_next into A buffer ab / copy i (of 4) of the chunk at b_next into Bm stage bs: ints,
  // or GICs for numbers known to the compiler (the LDS address is then one scalar addition of a constant away).
  auto copy_a = [&](auto ab, auto i_c, bool half_pair) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    if constexpr (std::is_integral_v<decltype(ab)>) {
      gemm_dma16(a_next, a_voff[i] - (half_pair ? a_back[i & 1] : 0u), lds_wave_a + (unsigned)(ab * G_ABUF + i * 1024));
    } else {
      constexpr int AB = decltype(ab)::value;
      asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                   :: "s"(lds_wave_a), "n"(AB * G_ABUF + i * 1024), "v"(a_voff[i]), "s"(a_next) : "memory", "m0", "scc");
    }
  };
  auto copy_b = [&](auto bs, auto i_c) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    if constexpr (std::is_integral_v<decltype(bs)>) {
      gemm_dma16(b_next, b_voff[i], lds_wave_b + (unsigned)(bs * G_BST + i * 1024));
    } else {
      constexpr int BS = decltype(bs)::value;
      asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                   :: "s"(lds_wave_b), "n"(BS * G_BST + i * 1024), "v"(b_voff[i]), "s"(b_next) : "memory", "m0", "scc");
    }
  };
  // Outside the unrolled loop the bases stop at the last pair and the last chunk: what is requested beyond the end of
  // K is the last pair / chunk once more, into a buffer nothing reads any more, so that every wait below counts the
  // same number of copies whatever K.
  auto a_advance = [&]() __attribute__((always_inline)) {
    if (a_idx + 1 < npairs) { a_next += 128; ++a_idx; }
  };
  auto b_advance = [&]() __attribute__((always_inline)) {
    if (b_idx + 1 < nch) { b_next += b_chunk; ++b_idx; }
  };
  auto a_is_half = [&]() __attribute__((always_inline)) { return (nch & 1) != 0 && a_idx == npairs - 1; };

  // fragment addresses: A within buffers 0 and 1 (a read's immediate offset reaches 64 KB) and within buffer 2, per k
  // step of the pair; Bm within the four stages
  unsigned a_reg[2][4], b_reg[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    a_reg[0][ks] = (unsigned)((128 * wr + j) * 128 + (((2 * ks + hh) ^ ((j >> 1) & 7)) * 16));
    a_reg[1][ks] = a_reg[0][ks] + 2u * G_ABUF;
    asm volatile("" : "+v"(a_reg[0][ks]), "+v"(a_reg[1][ks]));
  }
  {
    const int ta = (lane & 15) >> 2, tb = lane & 3, th = (lane >> 4) & 1;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      b_reg[nt] = (unsigned)(G_B0 + (8 * hh + ta) * G_ROWB + (((4 * (4 * wc + nt) + 2 * th + (tb >> 1)) ^ (ta << 2)) * 16) +
                             8 * (tb & 1));
      asm volatile("" : "+v"(b_reg[nt]));
    }
  }

  v16f acc[4][4];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][nt][r] = 0.0f;

  // the two sets of fragments: one k step of 16 each (4 row tiles of A, 4 column tiles of Bm)
  v8h af0[4], bf0[4], af1[4], bf1[4];
  g4s blo[4];
  // read number n (0..11) of a k step's fragments, in the order in which the MFMAs want them: Bm tile 0 (two
  // halves), A tile 0, Bm tiles 1..3, A tiles 1..3.  The k step is KS4 (0..3) of the pair in A buffer ab, KS4 & 1
  // of the chunk in Bm stage bs.
  auto frag_read = [&](auto ab, auto bs, auto ks4_c, auto n_c, v8h (&af)[4], v8h (&bf)[4]) __attribute__((always_inline)) {
    constexpr int n = decltype(n_c)::value, KS4 = decltype(ks4_c)::value;
    constexpr int kind = n < 2 ? 0 : n == 2 ? 1 : n < 9 ? 0 : 1;            // 0: Bm half, 1: A
    constexpr int nt = (n < 2 || n >= 9) ? 0 : 1 + ((n - 3) >> 1), half = n < 2 ? n : (n - 3) & 1;   // for kind 0
    constexpr int rt = n == 2 ? 0 : n - 8;                                  // for kind 1
    if constexpr (kind == 1) {
      const unsigned char* pa;
      if constexpr (std::is_integral_v<decltype(ab)>) {
        pa = gemm_smem + ab * G_ABUF + a_reg[0][KS4];
      } else {
        constexpr int AB = decltype(ab)::value;
        pa = gemm_smem + a_reg[AB >> 1][KS4] + (AB & 1) * G_ABUF;
      }
      af[rt] = *reinterpret_cast<const v8h*>(pa + 4096 * rt);
    } else {
      const unsigned char* pb;
      if constexpr (std::is_integral_v<decltype(bs)>) pb = gemm_smem + bs * G_BST + b_reg[nt];
      else pb = gemm_smem + b_reg[nt] + decltype(bs)::value * G_BST;
      const g4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_g4s*)(pb + 16 * G_ROWB * (KS4 & 1) + 4 * G_ROWB * half));
      if constexpr (half == 0) {
        blo[nt] = v;
      } else {
        const g8s both = {blo[nt][0], blo[nt][1], blo[nt][2], blo[nt][3], v[0], v[1], v[2], v[3]};
        bf[nt] = __builtin_bit_cast(v8h, both);
      }
    }
  };

  // One k step: 16 MFMAs on (af, bf); under them the 12 fragment reads of the step after (A buffer nab, Bm stage
  // nbs, k step nks4) into (naf, nbf) and four of the wave's copies: SET 1 copies 0..3, SET 2 copies 4..7 of the pair
  // at a_next into A buffer cdst; SET 3 the chunk at b_next into Bm stage cdst (0: none).  MAIN: inside the unrolled
  // loop, where every pair and chunk asked for exists.
  auto k_step = [&](v8h (&af)[4], v8h (&bf)[4], auto nab, auto nbs, auto nks4, v8h (&naf)[4], v8h (&nbf)[4], auto set_c,
                    auto cdst, auto main_c) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool MAIN = decltype(main_c)::value;
    bool half_pair = false;
    if constexpr (!MAIN && (SET == 1 || SET == 2)) half_pair = a_is_half();
    static_for<16>([&](auto s_c) __attribute__((always_inline)) {
      constexpr int s = decltype(s_c)::value;
      constexpr int rt = s >> 2, nt = s & 3;
      if constexpr (s < 12) frag_read(nab, nbs, nks4, s_c, naf, nbf);
      acc[rt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[nt], af[rt], acc[rt][nt], 0, 0, 0);
      if constexpr (SET != 0 && s < 12 && s % 3 == 1) {   // steps 1 4 7 10
        if constexpr (SET == 3) copy_b(cdst, GIC<(s / 3)>{});
        else copy_a(cdst, GIC<(4 * (SET - 1) + s / 3)>{}, half_pair);
      }
      if constexpr (s < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    });
    if constexpr (SET == 2) {
      if constexpr (MAIN) a_next += 128;
      else a_advance();
    }
    if constexpr (SET == 3) {
      if constexpr (MAIN) b_next += b_chunk;
      else b_advance();
    }
    __builtin_amdgcn_sched_barrier(0);   // the step's last MFMAs stay in front of what follows
  };

  // ---- prologue.  The loop below requests, beside chunk c, the Bm rows of chunk c + 3 and then half of an A pair:
  // the second half of pair c/2 + 2 when c is even, the first half of pair (c + 5)/2 when it is odd.  The prologue
  // requests what chunks -3, -2, -1 would have, behind pair 0: Bm 0, pair 1's first half, Bm 1, its second half,
  // Bm 2, pair 2's first half.
  static_assert(GS == 4 && GP == 3, "the order of the copies and the wait counts");
  {
    bool hp = a_is_half();
    static_for<8>([&](auto i_c) __attribute__((always_inline)) { copy_a(0, i_c, hp); });
    a_advance();
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_b(0, i_c); });
    b_advance();
    hp = a_is_half();
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_a(1, i_c, hp); });
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_b(1, i_c); });
    b_advance();
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_a(1, GIC<4 + decltype(i_c)::value>{}, hp); });
    a_advance();
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_b(2, i_c); });
    b_advance();
    hp = a_is_half();
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy_a(2, i_c, hp); });
  }
  __builtin_amdgcn_s_waitcnt(gemm_vmcnt(20));   // pair 0 and Bm 0 landed: 20 copies were requested behind them
  __builtin_amdgcn_s_barrier();
  static_for<12>([&](auto n_c) __attribute__((always_inline)) { frag_read(0, 0, GIC<0>{}, n_c, af0, bf0); });

  // Chunk ch = the HALF-th of the pair in A buffer ab, in Bm stage bs.
  auto chunk = [&](auto half_c, auto ab, auto bs, auto main_c) __attribute__((always_inline)) {
    constexpr int HALF = decltype(half_c)::value;
    k_step(af0, bf0, ab, bs, GIC<(2 * HALF + 1)>{}, af1, bf1, GIC<3>{}, prev_of<GS>(bs), main_c);
    // Chunk ch + 1 landed: copies complete in the order of their issue, and behind its Bm rows (its A rows are older)
    // 16 copies were requested: half a pair, the Bm rows of chunk ch + 2, half a pair, those of chunk ch + 3.  And
    // this wave's reads of chunk ch are complete.
    __builtin_amdgcn_s_waitcnt(gemm_vmcnt(16) & 0xC07F);   // and lgkmcnt(0)
    __builtin_amdgcn_s_barrier();   // every wave has chunk ch in registers
    if constexpr (HALF == 0) {   // the second half of the pair after next, into the buffer in front of this one
      k_step(af1, bf1, ab, next_of<GS>(bs), GIC<2>{}, af0, bf0, GIC<2>{}, prev_of<GP>(ab), main_c);
    } else {                     // this buffer is free: the first half of the pair three on
      k_step(af1, bf1, next_of<GP>(ab), next_of<GS>(bs), GIC<0>{}, af0, bf0, GIC<1>{}, ab, main_c);
    }
  };
  int ch = 0;
  for (; ch + 18 < nch; ch += 12) {   // every copy these twelve chunks request lies inside K
    static_for<12>([&](auto c_c) __attribute__((always_inline)) {
      constexpr int c = decltype(c_c)::value;
      chunk(GIC<(c & 1)>{}, GIC<((c >> 1) % GP)>{}, GIC<(c % GS)>{}, std::true_type{});
    });
  }
  a_idx = min(ch / 2 + 2, npairs - 1);
  b_idx = min(ch + 3, nch - 1);
  int ab = 0, bs = 0;   // ch is a multiple of 12
  for (; ch < nch; ch += 2) {
    chunk(GIC<0>{}, ab, bs, std::false_type{});
    bs = next_of<GS>(bs);
    if (ch + 1 < nch) chunk(GIC<1>{}, ab, bs, std::false_type{});
    bs = next_of<GS>(bs);
    ab = next_of<GP>(ab);
  }
  __builtin_amdgcn_s_waitcnt(gemm_vmcnt(0));   // no copy into LDS outlives the workgroup

  // ---- epilogue.  Of a tile's row, lane (j, 0) holds columns 8 q .. + 3 and lane (j, 1) columns 8 q + 4 .. + 7 for
  // q = 0..3: the two lanes exchange the halves of an even and an odd q, so that lane (j, 0) stores the 8 columns of
  // the even q and lane (j, 1) those of the odd one, 16 bytes each.
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int row = m0 + 128 * wr + 32 * rt + j;
    _Float16* crow = C + (size_t)row * N + n0 + 128 * wc + 8 * hh;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int qp = 0; qp < 2; ++qp) {
        v2u ev, od;
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const v2h e = {(_Float16)acc[rt][nt][8 * qp + 2 * w], (_Float16)acc[rt][nt][8 * qp + 2 * w + 1]};
          const v2h o = {(_Float16)acc[rt][nt][8 * qp + 4 + 2 * w], (_Float16)acc[rt][nt][8 * qp + 4 + 2 * w + 1]};
          ev[w] = __builtin_bit_cast(unsigned, e);
          od[w] = __builtin_bit_cast(unsigned, o);
          // upper lanes' ev <-> lower lanes' od
          asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1\n\ts_nop 1" : "+v"(ev[w]), "+v"(od[w]));
        }
        const v4u o = {ev[0], ev[1], od[0], od[1]};
        if (row < M) *reinterpret_cast<v4u*>(crow + 32 * nt + 16 * qp) = o;
      }
  }
}

// true when the tile kernel takes the shape
bool gemm_f16_tiles_fit(int M, int N, int K) { return M > 0 && N % GT == 0 && K % GK == 0; }

int launch_gemm_f16_tiles(const void* A, const void* Bm, void* C, int G, int M, int N, int K, hipStream_t s) {
  static DeviceOnce attr_once;
  constexpr int lds = G_LDS;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)gemm_f16_tile_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    attr_once.done(attr_bit);
  }
  const long long tiles = (long long)G * ((M + GT - 1) / GT) * (N / GT);
  if (tiles >= (1ll << 31)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "gemm: too many tiles");
  hipLaunchKernelGGL(gemm_f16_tile_kernel, dim3((unsigned)tiles), dim3(256), lds, s, (const _Float16*)A, (const _Float16*)Bm,
                     (_Float16*)C, M, N, K);
  return check_launch("gemm_f16_tile_kernel");
}

}  // namespace ftk
