// Plain fp16 product C = A @ Bm for shapes made of whole 256 x 256 tiles: one wave per SIMD, each with a
// 128 x 128 piece of the workgroup's tile in its accumulators.
//
// The streaming cell kernel (lstm_cell.hip, GEMM flavour) gives a wave 128 x 64 outputs, so every 16 MFMAs read
// 12 KB of fragments from LDS, and its two waves per SIMD meet at the same barrier.  Here a wave owns 128 x 128:
// 32 MFMAs per 16 KB of fragments, a third less LDS traffic per product, and the whole register file (256
// accumulator registers + fragments of two k steps).  With one wave per SIMD nothing fills a gap, so the loop
// leaves none it can avoid: the fragments of a k step are read while the MFMAs of the step before run, across
// the chunk boundary as well -- the barrier sits in the MIDDLE of a chunk, between its two k steps, where the
// second step's fragments are already in registers (the chunk's stage is then free for the copy of chunk
// ch + 4: its A rows beside the second k step, its Bm rows beside the next chunk's first) and the first step's
// fragments of the next chunk can be read behind it.
#include <algorithm>

#include "ftk_common.h"

namespace ftk {

template <int V> using GIC = std::integral_constant<int, V>;

constexpr int GT = 256;               // rows and columns of a workgroup's tile
constexpr int GK = 32;                // k chunk
constexpr int GS = 4;                 // LDS stages
constexpr int G_A_BYTES = GT * GK * 2;   // A rows of a chunk: 64 bytes each
constexpr int G_ROWB = GT * 2;           // a Bm row of a chunk in LDS
constexpr int G_STAGE = G_A_BYTES + GK * G_ROWB;   // 32 KB
constexpr int G_COPIES = 8;           // copies per wave and chunk (4 of A rows, 4 of Bm rows, 1 KB each)
constexpr int gemm_vmcnt(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }   // s_waitcnt: vmcnt <= n, nothing else

typedef short g4s __attribute__((ext_vector_type(4)));
typedef short g8s __attribute__((ext_vector_type(8)));

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte offset) into LDS at lds_addr + 16 * lane.
// The compiler does not count it: the loop waits with s_waitcnt vmcnt itself.
__device__ __forceinline__ void gemm_dma16(const void* gbase, unsigned byte_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_addr), "v"(byte_off), "s"(gbase) : "memory", "m0");
}

// LDS layout of a stage, as in the cell kernel: A row r (64 bytes, 4 chunks of 16) keeps chunk c in slot
// c ^ ((r >> 2) & 3); Bm row k (512 bytes, 32 chunks = columns 8c .. 8c+7 of the tile) keeps chunk c in slot
// c ^ ((k & 3) << 2).  The MFMA takes the Bm fragment as its first operand and the A fragment as its second:
// lane (j, hh) then holds, of output tile (rt, nt), row 32 rt + j and columns 32 nt + 8 q + 4 hh .. + 3 (q = 0..3).
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
  const int nch = K / GK;

  // copies: wave w brings A rows 64 w .. + 64 (copy i: 16 rows, row lane / 4) and Bm rows 8 w .. + 8 (copy i: 2 rows,
  // row lane / 32) of a chunk
  unsigned b_lane[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const unsigned kr = (unsigned)(2 * p + (lane >> 5));   // k row & 3
    b_lane[p] = ((unsigned)lane >> 5) * (unsigned)(2 * N) + ((((unsigned)lane & 31) ^ (kr << 2)) * 16);
  }
  // a copy's lane offsets from its operand's base for the chunk; the two bases move on by a chunk per chunk copied.
  // (Rows past the end of A repeat its last row; they are never stored.)
  const int a_row0 = min(m0 + 64 * wave, M - 1);
  unsigned a_voff[4], b_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = min(m0 + 64 * wave + 16 * i + (lane >> 2), M - 1);
    a_voff[i] = (unsigned)(row - a_row0) * (unsigned)(2 * K) + (unsigned)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
    b_voff[i] = b_lane[i & 1] + (unsigned)i * (unsigned)(2 * 2 * N);
    asm volatile("" : "+v"(a_voff[i]), "+v"(b_voff[i]));   // kept in registers, not formed again at every copy
  }
  const char* a_next = reinterpret_cast<const char*>(A + (size_t)a_row0 * K);   // of the chunk that is copied next
  const char* b_next = reinterpret_cast<const char*>(Bm + (size_t)(8 * wave) * N + n0);
  const size_t b_chunk = (size_t)GK * N * 2;
  const unsigned lds_wave = lds0 + (unsigned)(wave * 4096);
  // copy i (0..3: A rows, 4..7: Bm rows) of that chunk into a stage: an int, or a GIC for a stage known to the compiler
  // (the LDS address is then one scalar addition of a constant away)
  auto copy = [&](auto stage, auto i_c) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    constexpr int within = i < 4 ? i * 1024 : G_A_BYTES + (i - 4) * 1024;
    const void* base = i < 4 ? a_next : b_next;
    const unsigned voff = i < 4 ? a_voff[i & 3] : b_voff[i & 3];
    if constexpr (std::is_integral_v<decltype(stage)>) {
      gemm_dma16(base, voff, lds_wave + (unsigned)(stage * G_STAGE + within));
    } else {
      constexpr int ST = decltype(stage)::value;
      asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                   :: "s"(lds_wave), "n"(ST * G_STAGE + within), "v"(voff), "s"(base) : "memory", "m0", "scc");
    }
  };

  // fragment addresses within a stage; and, for stages known to the compiler, within each pair of stages (a read's
  // immediate offset reaches 64 KB: two stages)
  unsigned a_off[2], b_off[4], a_pair[2][2], b_pair[2][4];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_off[ks] = (unsigned)((128 * wr + j) * 64 + (((2 * ks + hh) ^ ((j >> 2) & 3)) * 16));
  {
    const int ta = (lane & 15) >> 2, tb = lane & 3, th = (lane >> 4) & 1;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
      b_off[nt] = (unsigned)(G_A_BYTES + (8 * hh + ta) * G_ROWB + (((4 * (4 * wc + nt) + 2 * th + (tb >> 1)) ^ (ta << 2)) * 16) +
                             8 * (tb & 1));
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      a_pair[h][ks] = a_off[ks] + (unsigned)(2 * h * G_STAGE);
      asm volatile("" : "+v"(a_pair[h][ks]));
    }
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      b_pair[h][nt] = b_off[nt] + (unsigned)(2 * h * G_STAGE);
      asm volatile("" : "+v"(b_pair[h][nt]));
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
  // halves), A tile 0, Bm tiles 1..3, A tiles 1..3
  auto frag_read = [&](auto stage, int ks, auto n_c, v8h (&af)[4], v8h (&bf)[4]) __attribute__((always_inline)) {
    constexpr int n = decltype(n_c)::value;
    constexpr int kind = n < 2 ? 0 : n == 2 ? 1 : n < 9 ? 0 : 1;            // 0: Bm half, 1: A
    constexpr int nt = (n < 2 || n >= 9) ? 0 : 1 + ((n - 3) >> 1), half = n < 2 ? n : (n - 3) & 1;   // for kind 0
    constexpr int rt = n == 2 ? 0 : n - 8;                                  // for kind 1
    const unsigned char* pa;
    const unsigned char* pb;
    if constexpr (std::is_integral_v<decltype(stage)>) {
      pa = gemm_smem + stage * G_STAGE + a_off[ks];
      pb = gemm_smem + stage * G_STAGE + b_off[nt];
    } else {
      constexpr int ST = decltype(stage)::value;
      pa = gemm_smem + a_pair[ST >> 1][ks] + (ST & 1) * G_STAGE;
      pb = gemm_smem + b_pair[ST >> 1][nt] + (ST & 1) * G_STAGE;
    }
    if constexpr (kind == 1) {
      af[rt] = *reinterpret_cast<const v8h*>(pa + 2048 * rt);
    } else {
      const g4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_g4s*)(pb + 16 * G_ROWB * ks + 4 * G_ROWB * half));
      if constexpr (half == 0) {
        blo[nt] = v;
      } else {
        const g8s both = {blo[nt][0], blo[nt][1], blo[nt][2], blo[nt][3], v[0], v[1], v[2], v[3]};
        bf[nt] = __builtin_bit_cast(v8h, both);
      }
    }
  };

  // One k step: 16 MFMAs on (af, bf); under them the 12 fragment reads of the step after (stage nst, k step nks)
  // into (naf, nbf) and four of the wave's copies into stage cst: SET 1 the A rows of the chunk that a_next points at,
  // SET 2 the Bm rows of the chunk that b_next points at (0: none).
  auto k_step = [&](v8h (&af)[4], v8h (&bf)[4], auto nst, int nks, v8h (&naf)[4], v8h (&nbf)[4], auto set_c, auto cst)
                    __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    static_for<16>([&](auto s_c) __attribute__((always_inline)) {
      constexpr int s = decltype(s_c)::value;
      constexpr int rt = s >> 2, nt = s & 3;
      if constexpr (s < 12) frag_read(nst, nks, s_c, naf, nbf);
      acc[rt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[nt], af[rt], acc[rt][nt], 0, 0, 0);
      if constexpr (SET != 0 && s < 12 && s % 3 == 1) copy(cst, GIC<(4 * (SET - 1) + s / 3)>{});   // steps 1 4 7 10
      if constexpr (s < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    });
    if constexpr (SET == 1) a_next += GK * 2;
    if constexpr (SET == 2) b_next += b_chunk;
    __builtin_amdgcn_sched_barrier(0);   // the step's last MFMAs stay in front of what follows
  };

  // ---- prologue: the first stages on their way, chunk 0 landed, its first k step's fragments read.  A chunk's A rows
  // are copied half a chunk before its Bm rows (below): of chunk 3 only the A rows are requested here.
  const int ahead = min(GS - 1, nch);
  for (int c = 0; c < ahead; ++c) {
    static_for<G_COPIES>([&](auto i_c) __attribute__((always_inline)) { copy(c, i_c); });
    a_next += GK * 2;
    b_next += b_chunk;
  }
  if (nch >= GS) {
    static_for<4>([&](auto i_c) __attribute__((always_inline)) { copy(GS - 1, i_c); });
    a_next += GK * 2;
  }
  switch (ahead - 1) {   // copies issued behind chunk 0's
    case 0: __builtin_amdgcn_s_waitcnt(gemm_vmcnt(0)); break;
    case 1: __builtin_amdgcn_s_waitcnt(gemm_vmcnt(G_COPIES)); break;
    default:
      if (nch >= GS) __builtin_amdgcn_s_waitcnt(gemm_vmcnt(2 * G_COPIES + 4));
      else __builtin_amdgcn_s_waitcnt(gemm_vmcnt(2 * G_COPIES));
      break;
  }
  __builtin_amdgcn_s_barrier();
  static_for<12>([&](auto n_c) __attribute__((always_inline)) { frag_read(0, 0, n_c, af0, bf0); });

  // chunk ch, in stage `stage` (an int, or a GIC in the loop that is unrolled over the stages); pstage: the stage of
  // chunk ch - 1.  Beside the first k step the Bm rows of chunk ch + 3 go into pstage (BROWS), beside the second the
  // A rows of chunk ch + 4 into `stage` (AROWS): eight copies in one k step left the other with issue slots to spare.
  auto chunk = [&](int ch, auto pstage, auto stage, auto nstage, auto brows_c, auto arows_c) __attribute__((always_inline)) {
    constexpr bool BROWS = decltype(brows_c)::value, AROWS = decltype(arows_c)::value;
    k_step(af0, bf0, stage, 1, af1, bf1, GIC<(BROWS ? 2 : 0)>{}, pstage);
    // chunk ch + 1 landed (copies complete in the order of their issue: as many may be outstanding as were issued
    // behind it: the A rows of chunks ch + 2 and ch + 3 and the Bm rows of the same); this wave's reads of chunk ch complete
    if constexpr (BROWS) {
      __builtin_amdgcn_s_waitcnt(gemm_vmcnt((GS - 2) * G_COPIES) & 0xC07F);   // and lgkmcnt(0)
    } else {
      switch (min(GS - 2, nch - 2 - ch)) {
        case 2: __builtin_amdgcn_s_waitcnt(gemm_vmcnt(2 * G_COPIES) & 0xC07F); break;
        case 1: __builtin_amdgcn_s_waitcnt(gemm_vmcnt(G_COPIES) & 0xC07F); break;
        default: __builtin_amdgcn_s_waitcnt(gemm_vmcnt(0) & 0xC07F); break;
      }
    }
    __builtin_amdgcn_s_barrier();   // every wave has chunk ch in registers: its stage takes chunk ch + GS
    k_step(af1, bf1, nstage, 0, af0, bf0, GIC<(AROWS ? 1 : 0)>{}, stage);
  };
  static_assert(GS == 4, "the unrolled loop and the wait counts");
  int ch = 0;
  for (; ch + GS + 3 < nch; ch += 4) {
    chunk(ch, GIC<3>{}, GIC<0>{}, GIC<1>{}, std::true_type{}, std::true_type{});
    chunk(ch + 1, GIC<0>{}, GIC<1>{}, GIC<2>{}, std::true_type{}, std::true_type{});
    chunk(ch + 2, GIC<1>{}, GIC<2>{}, GIC<3>{}, std::true_type{}, std::true_type{});
    chunk(ch + 3, GIC<2>{}, GIC<3>{}, GIC<0>{}, std::true_type{}, std::true_type{});
  }
  int stage = 0;
  for (; ch + GS < nch; ++ch) {
    const int nstage = (stage + 1) & 3;
    chunk(ch, (stage + 3) & 3, stage, nstage, std::true_type{}, std::true_type{});
    stage = nstage;
  }
  if (ch + GS - 1 < nch) {   // the last chunk's Bm rows are still to be requested
    const int nstage = (stage + 1) & 3;
    chunk(ch, (stage + 3) & 3, stage, nstage, std::true_type{}, std::false_type{});
    stage = nstage;
    ++ch;
  }
  for (; ch < nch; ++ch) {
    const int nstage = (stage + 1) & 3;
    chunk(ch, (stage + 3) & 3, stage, nstage, std::false_type{}, std::false_type{});
    stage = nstage;
  }

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
  constexpr int lds = G_STAGE * GS;
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
