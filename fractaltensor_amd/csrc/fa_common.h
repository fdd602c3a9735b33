// What the attention kernels share: the global -> LDS copy, the exchange between the two halves of a wave, and the
// padded LDS layout of a 64-key tile.
#pragma once

#include "ftk_common.h"

namespace ftk {

constexpr int FA_KT = 64;          // keys per tile

typedef short v4s __attribute__((ext_vector_type(4)));

// 16 bytes per lane from global memory (wave-uniform base + per-lane byte
// offset) straight into LDS at lds_base + 16*lane (lds_base wave-uniform).
// Issued as opaque assembly on purpose: the compiler would otherwise wait for
// every outstanding copy before the next LDS read that it cannot prove
// disjoint, which serialises the prefetch.  The caller waits with vmcnt(0)
// before the barrier that publishes the tile.
__device__ __forceinline__ void lds_dma16(const void* gbase, unsigned byte_off, void* lds_base) {
  const unsigned lds_addr = (unsigned)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)lds_base);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_addr), "v"(byte_off), "s"(gbase)
      : "memory", "m0");
}

// max(x, x of lane^32) without a trip through LDS: v_permlane32_swap exchanges
// the upper half of the first register with the lower half of the second, so
// with both holding x, afterwards one holds the lower lanes' x in every lane
// and the other the upper lanes'.  (Written as assembly: the compiler folds
// the two results of its builtin into one.)
__device__ __forceinline__ float max_with_other_half(float x) {
  float y = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));
  return fmaxf(x, y);
}

// LDS layout of a 64-key tile: rows as in memory plus padding, chosen so that
// fragment reads are bank-conflict free with plain immediate offsets:
//   K rows are padded by 16 bytes: a fragment read (ds_read_b128, 16 lanes =
//     16 consecutive keys, same columns) then touches 16 different 16-byte
//     chunks of the 256-byte bank line;
//   V rows are padded by 64 bytes: one 32-lane pass of the transposing read
//     covers 4 keys x 64 bytes, which land in four different 64-byte groups
//     (by 128 bytes where 64 would make the stride a multiple of the bank line, D = 96).
template <int D>
struct FaLayout {
  static constexpr int KRS = 2 * D + 16;   // K row stride, bytes
  static constexpr int VRS = (2 * D + 64) % 256 ? 2 * D + 64 : 2 * D + 128;   // V row stride, bytes
  static constexpr int KTB = FA_KT * KRS;  // K tile, bytes (a multiple of 1024)
  static constexpr int VTB = FA_KT * VRS;
  static_assert(KTB % 1024 == 0 && VTB % 1024 == 0, "tiles must be whole 1 KB copies");
};

}  // namespace ftk
