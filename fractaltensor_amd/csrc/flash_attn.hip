// Non-causal flash attention for gfx950: fp16 Q/K/V/O, fp32 accumulation on
// v_mfma_f32_32x32x16_f16, online softmax (running max and sum) in registers.
//
// Both contractions are computed transposed so that a lane owns one query row:
//   S^T[key, q] = sum_d K[key][d] * Q[q][d]      MFMA A-operand = K rows (LDS),
//                                                B-operand = Q row fragments (registers)
//   O^T[d, q]  += sum_key V[key][d] * P[q][key]   A-operand = V columns (LDS, transposing read),
//                                                B-operand = exp'd scores, fp16 (registers)
// The 32x32 accumulator of lane (q = lane%32, half = lane/32) holds, for that
// one query, keys 8g + 4*half + r (g = reg/4, r = reg%4) of a 32-key half tile.
// Row max / row sum are therefore a reduction over the lane's own registers
// plus one exchange with lane^32; the rescale factor of O^T is lane-local; and
// the exp'd scores already are a valid MFMA B-operand if the PV product
// contracts keys in the order the lane holds them (step s of a half tile takes
// keys {16s + 4*half + r} U {16s + 8 + 4*half + r}).  P never touches LDS.
//
// K and V tiles of 64 keys go from global memory straight into LDS
// (global_load_lds_dwordx4, 1 KB per wave instruction), both row-major as in
// memory, so staging costs no registers, no vector instructions and no LDS
// stores.  Each lane picks the 16 global bytes that land in its fixed LDS
// slot, so the LDS rows can carry padding (FaLayout) that makes fragment reads
// bank-conflict free at plain immediate offsets: no address arithmetic in the
// loop.  The A-operand of the PV product is read with ds_read_b64_tr_b16,
// where 16 lanes hand in the addresses of a 4-key x 16-column block (lane
// 4a+b: key a, columns 4b..4b+3) and lane i receives column i of the four
// keys, so V needs no transposed copy.  K is triple buffered (the scores of
// tile kt+1 are started during tile kt), V double buffered; one barrier per
// tile publishes the copies.
//
// What the loop is built around, measured on MI355X with two waves per SIMD:
// vector instructions do not hide behind MFMAs the way loads do -- a handful
// per MFMA are free, every further one costs issue time -- and dot-product
// instructions (v_dot2*) run on the matrix pipeline and stall it outright.
// So the per-score work is cut to one exponential, half a pack and a quarter of a packed add:
// Q is pre-multiplied by scale*log2(e), the reference maximum is subtracted by
// the matrix unit itself (score accumulators start from -m_ref instead of 0),
// row sums are packed fp16 adds over the rounded exponentials, and the loop is software pipelined per 32-key half
// tile with the instruction order written out and fenced step by step.
//
// flash_attn_pp_kernel (enough query blocks for 8 waves) orders the same work differently: the two waves of a SIMD
// alternate between a phase of matrix instructions only and a phase of vector instructions only, in opposite phases,
// and the running maximum is moved only when a sum of exponentials says it must (see the comment at the kernel).
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "ftk_common.h"
#include "fa_common.h"

namespace ftk {

constexpr float FA_TAU = 8.0f;     // slack (in powers of two) before the running maximum is moved
constexpr float FA_PMAX = 32768.0f;  // phase-alternating kernel: a lane's sum of exponentials above this moves the reference
constexpr int FA_TRACE_TILES = 256;

// Built with -DFTK_DEBUG_TRACE only (make TRACE=1): timeline of one wave of workgroup 0 when FTK_FA_TRACE is set,
// six stamps per key tile, read back with ftk_debug_read_fa_trace.  The library as shipped has neither.
#ifdef FTK_DEBUG_TRACE
__device__ long long fa_trace_buf[FA_TRACE_TILES * 6];
#endif

// MINB: workgroups per CU the register budget must allow.
// RAG: Skv is no multiple of the key tile (the last tile's tail is masked); a template parameter so that the kernel
// for whole tiles carries none of the masking code (with both in one kernel the tail steps spilled 63 registers per
// lane to scratch, which every wave wrote once: 87 MB of extra HBM writes per launch at B8 H16 S2048).
// PART: the workgroup takes one contiguous range of the keys (part_keys of them, a multiple of the tile) and leaves
// its unnormalised accumulators, reference maximum and sum of exponentials in part_o / part_ml for attn_merge_kernel:
// small grids with many keys are split over the keys so that they fill the chip.
template <int D, int QT, int WAVES, int MINB, bool TRACE, bool RAG, bool PART = false>
__global__ __launch_bounds__(WAVES * 64, MINB) void flash_attn_kernel(const _Float16* __restrict__ Q,
                                                         const _Float16* __restrict__ K,
                                                         const _Float16* __restrict__ V,
                                                         _Float16* __restrict__ O, int Sq, int Skv_all,
                                                         float scale_log2e, int nqb,
                                                         long long* __restrict__ trace, int trace_wave,
                                                         int nparts = 1, int part_keys = 0,
                                                         float* __restrict__ part_o = nullptr,
                                                         float* __restrict__ part_ml = nullptr) {
  using L = FaLayout<D>;
  constexpr int DS = D / 16;  // k steps of S^T
  constexpr int DT = D / 32;  // d tiles of O^T
  constexpr int RB = 2 * D;   // bytes per K or V row in global memory
  constexpr int KRS = L::KRS, VRS = L::VRS, KTB = L::KTB, VTB = L::VTB;
  constexpr int KCP = (KTB / 1024 + WAVES - 1) / WAVES;  // 1 KB copies per wave per K tile (upper bound)
  constexpr int VCP = (VTB / 1024 + WAVES - 1) / WAVES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* const Kb = smem;            // [3][KTB]
  unsigned char* const Vb = smem + 3 * KTB;  // [2][VTB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // wave index as a scalar, so that LDS copy destinations are provably wave-uniform
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31;
  const int hh = lane >> 5;
  // One-dimensional grid of nqb query blocks x (batch*heads).  The hardware
  // deals workgroups round-robin over the 8 XCDs; remap so that the query
  // blocks of one head run on one XCD and share its L2 copy of K and V.
  int id = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) id = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  int part = 0;
  if constexpr (PART) {
    part = id % nparts;
    id /= nparts;
  }
  const int bh = id / nqb;
  const int qb = id - bh * nqb;
  const int q_base = qb * (WAVES * 32 * QT) + wave * (32 * QT);
  const int key_first = PART ? part * part_keys : 0;
  const int Skv = PART ? min(part_keys, Skv_all - key_first) : Skv_all;   // the keys this workgroup sees

  const _Float16* Qg = Q + (size_t)bh * Sq * D;
  const _Float16* Kg = K + ((size_t)bh * Skv_all + key_first) * D;
  const _Float16* Vg = V + ((size_t)bh * Skv_all + key_first) * D;
  _Float16* Og = O + (size_t)bh * Sq * D;

  // ---- Q row fragments, resident for the whole kernel, pre-multiplied by
  // scale*log2(e) (in fp32, rounded once to fp16): scores then come out of the
  // matrix unit in exponent units and need no scaling instruction per score.
  v8h qf[QT][DS];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int row = min(q_base + 32 * qt + j, Sq - 1);
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(Qg + (size_t)row * D + 16 * s + 8 * hh);
      const v8h q = *reinterpret_cast<const v8h*>(&v);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[qt][s][e] = (_Float16)((float)q[e] * scale_log2e);
    }
  }

  v16f oacc[QT][DT];
  float l_run[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    l_run[qt] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[qt][dt][r] = 0.0f;
  }

  constexpr bool has_ragged = RAG;
  // ---- copies: copy c of a tile fills LDS bytes [1024c, 1024c + 1024) of the
  // padded tile, lane l the 16 bytes at 1024c + 16l; slots in the padding
  // fetch the row's first chunk (never read).  Wave w issues copies w, w+WAVES, ...
  unsigned k_src[KCP], v_src[VCP];  // byte offset of this lane's chunk within the tile in global memory
#pragma unroll
  for (int i = 0; i < KCP; ++i) {
    const int x = 1024 * (wave + WAVES * i) + 16 * lane;
    const int row = min(x / KRS, FA_KT - 1), col = x % KRS;
    k_src[i] = row * RB + (col < RB ? col : 0);
  }
#pragma unroll
  for (int i = 0; i < VCP; ++i) {
    const int x = 1024 * (wave + WAVES * i) + 16 * lane;
    const int row = min(x / VRS, FA_KT - 1), col = x % VRS;
    v_src[i] = row * RB + (col < RB ? col : 0);
  }
  // copy i (of this wave's share) of K tile kt into the K buffer at dst; no-op past the wave's last copy
  auto copy_k = [&](unsigned char* dst, int kt, auto i_c) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    if constexpr (i < KCP) {
      if (wave + WAVES * i < KTB / 1024) {
        const int key0 = kt * FA_KT;
        unsigned off = k_src[i];
        if (has_ragged && key0 + FA_KT > Skv) {  // ragged last tile: rows past the end re-read the last key (their scores are masked)
          const unsigned last = (unsigned)(Skv - 1 - key0), row = off / RB;
          if (row > last) off -= (row - last) * RB;
        }
        lds_dma16(Kg + (size_t)key0 * D, off, dst + 1024 * (wave + WAVES * i));
      }
    }
  };
  auto copy_v = [&](unsigned char* dst, int kt, auto i_c) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    if constexpr (i < VCP) {
      if (wave + WAVES * i < VTB / 1024) {
        const int key0 = kt * FA_KT;
        unsigned off = v_src[i];
        if (has_ragged && key0 + FA_KT > Skv) {
          const unsigned last = (unsigned)(Skv - 1 - key0), row = off / RB;
          if (row > last) off -= (row - last) * RB;
        }
        lds_dma16(Vg + (size_t)key0 * D, off, dst + 1024 * (wave + WAVES * i));
      }
    }
  };
  auto copy_k_all = [&](unsigned char* dst, int kt) __attribute__((always_inline)) {
    static_for<KCP>([&](auto i_c) __attribute__((always_inline)) { copy_k(dst, kt, i_c); });
  };
  auto copy_v_all = [&](unsigned char* dst, int kt) __attribute__((always_inline)) {
    static_for<VCP>([&](auto i_c) __attribute__((always_inline)) { copy_v(dst, kt, i_c); });
  };
  auto stamp = [&](int kt, int slot) __attribute__((always_inline)) {
    if constexpr (TRACE) {
      if (blockIdx.x == 0 && tid == 64 * trace_wave && kt < FA_TRACE_TILES) trace[kt * 6 + slot] = wall_clock64();
    }
  };
  auto copies_landed = [&](int kt) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    stamp(kt, 5);
    __syncthreads();
  };

  // ---- fragment addresses: one lane-dependent base per tile kind, everything
  // else (half tile, contraction step, d tile) is an immediate offset.
  // K: lane (j, hh) reads row 32*k2 + j, bytes [32s + 16hh, +16)
  const int k_lane = j * KRS + 16 * hh;
  // V: lane hands in (key a = (lane&15)>>2, column chunk b = lane&3) of the 16-column block
  // dhalf = (lane>>4)&1 of d tile dt, keys 4*hh + a (+ constant) of the step
  const int v_lane = (4 * hh + ((lane & 15) >> 2)) * VRS + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);

  const int ntiles = (Skv + FA_KT - 1) / FA_KT;

  using lds_v4s = __attribute__((address_space(3))) v4s;
  typedef short v8s __attribute__((ext_vector_type(8)));
  // kbase / vbase: LDS address of the half tile plus the lane's base
  auto read_k = [&](const unsigned char* kbase, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const v8h*>(kbase + 32 * s);
  };
  // A-operand of the PV product for (step s, d tile dt) of one half tile
  auto read_v = [&](const unsigned char* vbase, int s, int dt) __attribute__((always_inline)) {
    const unsigned char* p0 = vbase + 16 * s * VRS + 64 * dt;
    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 8 * VRS));
    const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(v8h, both);
  };

  // Scores are kept relative to a per-row reference maximum m_ref, and the
  // subtraction is free: every score chain starts its accumulator from nref =
  // -m_ref (a 16-register vector, one query per lane) instead of zero, so the
  // matrix unit hands back s - m_ref and p = exp2(s - m_ref) is a single
  // exponential.  m_ref only moves (and O, l are rescaled) when a row maximum
  // has run ahead of it by more than FA_TAU: any m_ref gives the same O =
  // acc/l, p merely ranges up to 2^FA_TAU.  The move happens between half
  // tiles, after everything computed with the old reference has been
  // accumulated, and also shifts the one score vector already computed against
  // the old reference.  A fully masked half has maximum -inf, never moves the
  // reference and exponentiates to zeros.
  v16f nref[QT];
  auto move_reference = [&](const float (&mx)[QT], v16f (&sn)[QT]) __attribute__((always_inline)) {
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const bool need = mx[qt] > FA_TAU;
      if (__builtin_amdgcn_ballot_w64(need) != 0) {
        const float delta = need ? -mx[qt] : 0.0f;  // new scores = old scores + delta
        const float alpha = __builtin_amdgcn_exp2f(delta);
        l_run[qt] *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          nref[qt][r] += delta;
          sn[qt][r] += delta;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[qt][dt][r] *= alpha;
      }
    }
  };

  // p = exp2(score e) of a half tile; pairs are packed to fp16 in the order
  // the PV product contracts them.  The row sum is taken over the packed pairs
  // once the half is complete (block A): dot-product instructions would do it
  // in half the instructions again but run on the matrix pipeline and stall the MFMAs.
  float held[QT];
  auto exp_element = [&](const v16f (&sc)[QT], v8h (&pf)[QT][2], auto e_c) __attribute__((always_inline)) {
    constexpr int e = decltype(e_c)::value;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const float p = __builtin_amdgcn_exp2f(sc[qt][e]);
      if constexpr ((e & 1) == 0) {
        held[qt] = p;
      } else {
        const v2h pp = {(_Float16)held[qt], (_Float16)p};
        pf[qt][e / 8][(e % 8) - 1] = pp[0];
        pf[qt][e / 8][e % 8] = pp[1];
      }
    }
  };

  // The loop is software pipelined per 32-key half tile in two kinds of
  // blocks, written in the instruction order they should issue in and fenced
  // step by step so that the order survives.  Vector instructions do not hide
  // behind matrix instructions on this machine (each costs issue time), so the
  // blocks are built to need few of them:
  //   E: DS steps of { QT score MFMAs of the NEXT half | one fragment read
  //      three steps ahead | exponentiate a few scores of THIS half }
  //   A: 2*DT steps of { QT MFMAs of P V of THIS half | one fragment read |
  //      first the remaining exponentials, then row maxima of the NEXT half's
  //      scores }, then move the reference maximum if needed.
  // NE of the 16 scores a lane holds per query are exponentiated in E, the
  // rest in the first DT steps of A (they belong to the second contraction
  // step of P V, which starts at step DT).  Fragment reads run three steps
  // ahead throughout, across block boundaries: the last three steps of a block
  // read the first three fragments of the next one (kpre / vpre).
  constexpr int NE = 12;   // 8 to 16 measure the same
  constexpr int NS = 2 * DT;
  // fragments read ahead of the matrix instruction that uses them (4 to 6 measure the same); a head dimension of 32
  // has two-step blocks, so two
  constexpr int LA = DS < 3 ? DS : 3;
  static_assert(LA <= DS && LA <= NS, "the lookahead must fit in one block");
  v8h kpre[LA], vpre[LA];
  auto block_e = [&](const unsigned char* kbase, const unsigned char* vbase, const v16f (&sc)[QT], v8h (&pf)[QT][2],
                     v16f (&sn)[QT], auto next_c) __attribute__((always_inline)) {
    constexpr bool has_next = decltype(next_c)::value;
    v8h kf[DS];
#pragma unroll
    for (int i = 0; i < LA; ++i) kf[i] = kpre[i];
    __builtin_amdgcn_sched_barrier(0);
    static_for<DS>([&](auto s_c) __attribute__((always_inline)) {
      constexpr int s = decltype(s_c)::value;
      if constexpr (has_next) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          sn[qt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], qf[qt][s], s == 0 ? nref[qt] : sn[qt], 0, 0, 0);
        if constexpr (s + LA < DS) kf[s + LA] = read_k(kbase, s + LA);
      }
      if constexpr (s + LA >= DS) vpre[s + LA - DS] = read_v(vbase, (s + LA - DS) / DT, (s + LA - DS) % DT);
      // scores [s*NE/DS, (s+1)*NE/DS)
      static_for<((s + 1) * NE) / DS - (s * NE) / DS>([&](auto i_c) __attribute__((always_inline)) {
        exp_element(sc, pf, std::integral_constant<int, (s * NE) / DS + decltype(i_c)::value>{});
      });
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  // knext: base of the K half tile whose scores the following E block computes (ignored without one)
  auto block_a = [&](const unsigned char* vbase, const unsigned char* knext, const v16f (&sc)[QT], v8h (&pf)[QT][2],
                     v16f (&sn)[QT], int key_next, auto next_c, auto mask_c, auto prek_c) __attribute__((always_inline)) {
    constexpr bool has_next = decltype(next_c)::value;
    constexpr bool mask = decltype(mask_c)::value;
    constexpr bool prefetch_k = decltype(prek_c)::value;
    v8h vf[NS];
#pragma unroll
    for (int i = 0; i < LA; ++i) vf[i] = vpre[i];
    float mx[QT];
    __builtin_amdgcn_sched_barrier(0);
    static_for<NS>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      constexpr int s = i / DT, dt = i % DT;
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
        oacc[qt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i], pf[qt][s], oacc[qt][dt], 0, 0, 0);
      if constexpr (i + LA < NS) {
        vf[i + LA] = read_v(vbase, (i + LA) / DT, (i + LA) % DT);
      } else if constexpr (prefetch_k) {
        kpre[i + LA - NS] = read_k(knext, i + LA - NS);
      }
      if constexpr (i < DT) {
        // remaining scores [NE + i*(16-NE)/DT, NE + (i+1)*(16-NE)/DT)
        constexpr int R = 16 - NE;
        static_for<((i + 1) * R) / DT - (i * R) / DT>([&](auto j_c) __attribute__((always_inline)) {
          exp_element(sc, pf, std::integral_constant<int, NE + (i * R) / DT + decltype(j_c)::value>{});
        });
        if constexpr (i == DT - 1) {
          // this lane's half of the row sum: the packed pairs, i.e. the values P V multiplies with, summed as a tree
          // of packed fp16 adds (7 instructions and a final add for 16 fp32 adds; B8 H16 S2048 D = 64: 186 -> 177 us)
#pragma unroll
          for (int qt = 0; qt < QT; ++qt) {
            v2h t[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) t[k] = v2h{pf[qt][k >> 2][2 * (k & 3)], pf[qt][k >> 2][2 * (k & 3) + 1]};
#pragma unroll
            for (int w = 4; w >= 1; w >>= 1)
#pragma unroll
              for (int k = 0; k < w; ++k) t[k] = t[k] + t[k + w];
            l_run[qt] += (float)t[0][0] + (float)t[0][1];
          }
        }
      } else if constexpr (has_next) {
        // row maxima of the next half's scores [(i-DT)*16/DT, (i-DT+1)*16/DT)
        constexpr int e0 = ((i - DT) * 16) / DT, e1 = ((i - DT + 1) * 16) / DT;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
          if constexpr (mask) {
#pragma unroll
            for (int r = e0; r < e1; ++r)
              if (key_next + 8 * (r >> 2) + 4 * hh + (r & 3) >= Skv) sn[qt][r] = -INFINITY;
          }
          float m = i == DT ? sn[qt][e0] : mx[qt];
#pragma unroll
          for (int r = e0; r < e1; ++r) m = fmaxf(m, sn[qt][r]);
          mx[qt] = m;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (has_next) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) mx[qt] = max_with_other_half(mx[qt]);
      move_reference(mx, sn);
    }
  };

  // K buffers rotate through (current, next, free), V buffers alternate
  int kcur = 0, knext = KTB, kfree = 2 * KTB;
  int vcur = 0, vnext = VTB;

  // ---- prologue: tiles 0 (K, V) and 1 (K) into LDS; scores of tile 0's first
  // half from a zero start, their row maximum becomes the first reference
  v16f sa[QT], sb[QT];
  v8h pa[QT][2], pb[QT][2];
  copy_k_all(Kb, 0);
  copy_v_all(Vb, 0);
  if (ntiles > 1) copy_k_all(Kb + KTB, 1);
  copies_landed(FA_TRACE_TILES);
  {
    const unsigned char* kbase = Kb + k_lane;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sa[qt][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < DS; ++s)
        sa[qt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(read_k(kbase, s), qf[qt][s], sa[qt], 0, 0, 0);
      if (ntiles == 1 && has_ragged) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (8 * (r >> 2) + 4 * hh + (r & 3) >= Skv) sa[qt][r] = -INFINITY;
      }
      float m = sa[qt][0];
#pragma unroll
      for (int r = 1; r < 16; ++r) m = fmaxf(m, sa[qt][r]);
      m = max_with_other_half(m);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sa[qt][r] -= m;
        nref[qt][r] = -m;
      }
    }
#pragma unroll
    for (int i = 0; i < LA; ++i) kpre[i] = read_k(kbase + 32 * KRS, i);
  }

  // One step = one 64-key tile: E and A for its first half (scores of the
  // second half computed on the way), E and A for its second half (scores of
  // tile kt+1's first half, whose K tile was copied one step earlier).  The
  // copies of K(kt+2) and V(kt+1) go into buffers that every wave finished
  // with before the barrier that ended the previous step, and are awaited at
  // the barrier that ends this one.
  auto step = [&](int kt, auto next_c, auto mask_c) __attribute__((always_inline)) {
    stamp(kt, 0);
    // A wave is held at issue while its copy instructions queue up in the memory pipeline.  With two waves
    // per SIMD the two take turns: the first issues its copies when the step begins, the second after the
    // first half tile, so that one of them always has MFMAs to issue.
    const bool copy_first = WAVES < 8 || wave < WAVES / 2;
    if (copy_first) {
      if (kt + 2 < ntiles) copy_k_all(Kb + kfree, kt + 2);
      if (kt + 1 < ntiles) copy_v_all(Vb + vnext, kt + 1);
    }
    const unsigned char* v0 = Vb + vcur + v_lane;
    block_e(Kb + kcur + k_lane + 32 * KRS, v0, sa, pa, sb, std::true_type{});
    stamp(kt, 1);
    block_a(v0, Kb + knext + k_lane, sa, pa, sb, kt * FA_KT + 32, std::true_type{}, mask_c, next_c);
    if (!copy_first) {
      if (kt + 2 < ntiles) copy_k_all(Kb + kfree, kt + 2);
      if (kt + 1 < ntiles) copy_v_all(Vb + vnext, kt + 1);
    }
    stamp(kt, 2);
    block_e(Kb + knext + k_lane, v0 + 32 * VRS, sb, pb, sa, next_c);
    stamp(kt, 3);
    block_a(v0 + 32 * VRS, Kb + knext + k_lane + 32 * KRS, sb, pb, sa, (kt + 1) * FA_KT, next_c, mask_c, next_c);
    stamp(kt, 4);
    copies_landed(kt);
    int t = kcur;
    kcur = knext;
    knext = kfree;
    kfree = t;
    t = vcur;
    vcur = vnext;
    vnext = t;
  };

  // Only the two steps that touch the last tile pay for masking its ragged
  // tail; they are peeled so that the main loop body is one straight line.
  for (int kt = 0; kt + 2 < ntiles; ++kt) step(kt, std::true_type{}, std::false_type{});
  if constexpr (has_ragged) {
    if (ntiles > 1) step(ntiles - 2, std::true_type{}, std::true_type{});
    step(ntiles - 1, std::false_type{}, std::true_type{});
  } else {
    if (ntiles > 1) step(ntiles - 2, std::true_type{}, std::false_type{});
    step(ntiles - 1, std::false_type{}, std::false_type{});
  }

  // ---- normalise and store.  A lane holds d = 32dt + 8g + 4*half + r of its row: 8-byte pieces scattered over
  // the row, which as stores fill no cache line (the memory system then writes more than twice the bytes of O).
  // So the wave turns its 32 x D tile round through LDS, which nobody reads any more after the barrier that ended
  // the last step: every lane writes its pieces into the wave's own padded tile, then 2D/16 lanes per row read 16
  // bytes each and the wave stores whole rows, 1 KB of consecutive bytes per instruction.  LDS executes a wave's
  // instructions in order, so the wave needs no barrier between its writes and its reads.
  if constexpr (PART) {
    // a part's result: O^T unnormalised, relative to the part's reference maximum m (in exponent units), and the sum
    // of exponentials l relative to the same m: what the merge rule of an online softmax takes
    // (kaleido/core/device/kernels/online_softmax.h:27-30)
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const float l = l_run[qt] + __shfl_xor(l_run[qt], 32);
      const int row = q_base + 32 * qt + j;
      if (row < Sq) {
        const size_t at = ((size_t)bh * nparts + part) * Sq + row;
        if (hh == 0) {
          part_ml[2 * at] = -nref[qt][0];
          part_ml[2 * at + 1] = l;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            *reinterpret_cast<float4*>(part_o + at * D + 32 * dt + 8 * g + 4 * hh) =
                make_float4(oacc[qt][dt][4 * g], oacc[qt][dt][4 * g + 1], oacc[qt][dt][4 * g + 2], oacc[qt][dt][4 * g + 3]);
      }
    }
    return;
  }
  constexpr int ORS = 2 * D + 16;        // padded row: the 32 rows' 8-byte pieces spread over all banks
  constexpr int LPR = D / 8;             // 16-byte chunks per row
  unsigned char* const ot = smem + wave * (32 * ORS);
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const float l = l_run[qt] + __shfl_xor(l_run[qt], 32);
    const float inv = 1.0f / l;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v2h lo = {(_Float16)(oacc[qt][dt][4 * g] * inv), (_Float16)(oacc[qt][dt][4 * g + 1] * inv)};
        const v2h hi = {(_Float16)(oacc[qt][dt][4 * g + 2] * inv), (_Float16)(oacc[qt][dt][4 * g + 3] * inv)};
        *reinterpret_cast<v2u*>(ot + j * ORS + 2 * (32 * dt + 8 * g + 4 * hh)) =
            v2u{__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
      }
#pragma unroll
    for (int idx = lane; idx < 32 * LPR; idx += 64) {   // consecutive lanes: consecutive chunks of a row, then the next row
      const int r = idx / LPR, c = idx - r * LPR;
      const v4u piece = *reinterpret_cast<const v4u*>(ot + r * ORS + 16 * c);
      const int row = q_base + 32 * qt + r;
      // streaming store: O is not read again by this launch, and lines left dirty in L2 are written back only when
      // the kernel ends, which the next launch in the stream waits for
      if (row < Sq) __builtin_nontemporal_store(piece, reinterpret_cast<v4u*>(Og + (size_t)row * D + 8 * c));
    }
  }
}

#ifdef FTK_DEBUG_TRACE
// FTK_FA_TRACE=1+w turns the per-tile timeline of wave w of workgroup 0 on (read once).
static int fa_trace_wave() {
  const char* e = getenv("FTK_FA_TRACE");
  return e && atoi(e) > 0 ? atoi(e) - 1 : 0;
}
// Device address of the stamp buffer, or NULL when tracing is off.
static long long* fa_trace_ptr() {
  static int on = -1;
  static long long* ptr = nullptr;
  if (on < 0) {
    const char* e = getenv("FTK_FA_TRACE");
    on = (e && atoi(e) > 0) ? 1 : 0;
    if (on && hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(fa_trace_buf)) != hipSuccess) ptr = nullptr;
  }
  return on ? ptr : nullptr;
}
#endif

// The same product with the two waves of a SIMD kept in opposite phases (8 waves x 32 query rows; RAG: the key
// length is no multiple of the tile, the tail of the last tile is masked).  A wave alternates between a phase of matrix instructions only -- M(t): O^T += V(t)^T P(t)^T, then the
// scores of tile t+1 -- and a phase of vector instructions only -- S(t): row maximum, exponentials, row sum and
// packing of tile t's scores -- with a workgroup barrier after every phase.  Waves 4..7 run one phase behind waves
// 0..3 (they pass one barrier more before the loop, the others one more after it), and wave w + 4 shares its SIMD
// with wave w: while one of the two feeds the matrix pipe the other one's vector work and copy issue run beside it,
// instead of both waves interleaving the two kinds of work and stalling at the same places.  The raised priority of
// the wave in M lets its next MFMA go ahead of the other wave's vector instructions.
// Tiles: K(t+1) and V(t) are read during M(t), i.e. in two consecutive phase slots.  K has two buffers, V three:
// waves 0..3 request V(t+1) at the start of S(t), waves 4..7 request K(t+2) at the start of their S(t), and each
// waits for its own copies before the barrier that ends its following M phase, one slot before the first reader.
template <int D, bool TRACE, bool RAG>
__global__ __launch_bounds__(512, 1) void flash_attn_pp_kernel(const _Float16* __restrict__ Q,
                                                                const _Float16* __restrict__ K,
                                                                const _Float16* __restrict__ V,
                                                                _Float16* __restrict__ O, int Sq, int Skv,
                                                                float scale_log2e, int nqb,
                                                                long long* __restrict__ trace, int trace_wave) {
  using L = FaLayout<D>;
  constexpr int DS = D / 16, DT = D / 32, RB = 2 * D;
  constexpr int KRS = L::KRS, VRS = L::VRS, KTB = L::KTB, VTB = L::VTB;
  constexpr int CW = 4;                                   // waves that share the copies of a tile
  constexpr int KCP = (KTB / 1024 + CW - 1) / CW, VCP = (VTB / 1024 + CW - 1) / CW;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* const Kb = smem;            // [2][KTB]
  unsigned char* const Vb = smem + 2 * KTB;  // [3][VTB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int group = wave >> 2, cw = wave & 3;
  const int j = lane & 31, hh = lane >> 5;
  int id = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) id = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int bh = id / nqb;
  const int qb = id - bh * nqb;
  const int q_base = qb * 256 + wave * 32;
  const _Float16* Qg = Q + (size_t)bh * Sq * D;
  const _Float16* Kg = K + (size_t)bh * Skv * D;
  const _Float16* Vg = V + (size_t)bh * Skv * D;
  _Float16* Og = O + (size_t)bh * Sq * D;

  v8h qf[DS];
  {
    const int row = min(q_base + j, Sq - 1);
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(Qg + (size_t)row * D + 16 * s + 8 * hh);
      const v8h q = *reinterpret_cast<const v8h*>(&v);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[s][e] = (_Float16)((float)q[e] * scale_log2e);
    }
  }
  v16f oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
  float l_run = 0.0f;

  unsigned k_src[KCP], v_src[VCP];
#pragma unroll
  for (int i = 0; i < KCP; ++i) {
    const int x = 1024 * (cw + CW * i) + 16 * lane;
    const int row = min(x / KRS, FA_KT - 1), col = x % KRS;
    k_src[i] = row * RB + (col < RB ? col : 0);
  }
#pragma unroll
  for (int i = 0; i < VCP; ++i) {
    const int x = 1024 * (cw + CW * i) + 16 * lane;
    const int row = min(x / VRS, FA_KT - 1), col = x % VRS;
    v_src[i] = row * RB + (col < RB ? col : 0);
  }
  // RAG (Skv no multiple of the tile): rows of the last tile past the end re-read the last key; their scores are masked
  auto ragged_off = [&](unsigned off, int kt) __attribute__((always_inline)) {
    if constexpr (RAG) {
      const int key0 = kt * FA_KT;
      if (key0 + FA_KT > Skv) {
        const unsigned last = (unsigned)(Skv - 1 - key0), row = off / RB;
        if (row > last) off -= (row - last) * RB;
      }
    }
    return off;
  };
  auto copy_k_tile = [&](unsigned char* dst, int kt) __attribute__((always_inline)) {
    static_for<KCP>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if (cw + CW * i < KTB / 1024) lds_dma16(Kg + (size_t)kt * FA_KT * D, ragged_off(k_src[i], kt), dst + 1024 * (cw + CW * i));
    });
  };
  auto copy_v_tile = [&](unsigned char* dst, int kt) __attribute__((always_inline)) {
    static_for<VCP>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if (cw + CW * i < VTB / 1024) lds_dma16(Vg + (size_t)kt * FA_KT * D, ragged_off(v_src[i], kt), dst + 1024 * (cw + CW * i));
    });
  };
  // a barrier that waits for nothing of the wave's own: whoever wrote what the barrier publishes has waited before it
  auto phase_barrier = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  const int k_lane = j * KRS + 16 * hh;
  const int v_lane = (4 * hh + ((lane & 15) >> 2)) * VRS + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
  const int ntiles = (Skv + FA_KT - 1) / FA_KT;
  // scores of keys past the end of a ragged last tile: minus infinity, so they exponentiate to zero and no maximum sees them
  auto mask_tail = [&](v16f (&sv)[2], int kt) __attribute__((always_inline)) {
    if constexpr (RAG) {
      if ((kt + 1) * FA_KT > Skv) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (kt * FA_KT + 32 * h + 8 * (r >> 2) + 4 * hh + (r & 3) >= Skv) sv[h][r] = -INFINITY;
      }
    }
  };
  using lds_v4s = __attribute__((address_space(3))) v4s;
  typedef short v8s __attribute__((ext_vector_type(8)));
  auto read_k = [&](const unsigned char* kbase, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const v8h*>(kbase + 32 * s);
  };
  auto read_v = [&](const unsigned char* vbase, int s, int dt) __attribute__((always_inline)) {
    const unsigned char* p0 = vbase + 16 * s * VRS + 64 * dt;
    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 8 * VRS));
    const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(v8h, both);
  };

  // ---- prologue: K(0), V(0) (waves 0..3) and K(1) (waves 4..7) into LDS; scores of tile 0 from a zero start, their
  // row maximum becomes the first reference
  if (group == 0) {
    copy_k_tile(Kb, 0);
    copy_v_tile(Vb, 0);
  } else if (ntiles > 1) {
    copy_k_tile(Kb + KTB, 1);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();
  v16f sc[2], nref;   // scores of the tile's two 32-key halves, relative to the reference; minus the reference
  v8h pf[2][2];       // their exponentials as the B operands of P V
  {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[h][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < DS; ++s)
        sc[h] = __builtin_amdgcn_mfma_f32_32x32x16_f16(read_k(Kb + k_lane + h * 32 * KRS, s), qf[s], sc[h], 0, 0, 0);
    }
    mask_tail(sc, 0);
    float m = sc[0][0];
#pragma unroll
    for (int r = 1; r < 32; ++r) m = fmaxf(m, sc[r >> 4][r & 15]);
    m = max_with_other_half(m);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[0][r] -= m;
      sc[1][r] -= m;
      nref[r] = -m;
    }
  }

  constexpr int LA = 4;          // fragments read ahead of the matrix instruction that uses them (6, 8, 12: no faster)
  constexpr int NM = 2 * DS + 2 * 2 * DT;   // matrix instructions of an M phase: P V first, then the next tile's scores
  constexpr int NPV = 4 * DT;
  v8h vpre[LA];
  int vcur = 0, vnext = VTB, vfree = 2 * VTB;   // V(t), V(t+1), and the buffer V(t+2) will go to
  int kcur = 0, knext = KTB;                    // K(t), K(t+1)

  // exponentials of the tile's scores, packed as the B operands of P V; returns this lane's share of their sum.
  // The row sum adds the packed fp16 pairs, i.e. the values P V multiplies with, as a tree of packed adds: 15 vector
  // instructions and a final add where fp32 adds of the unrounded values take 32 (B8 H16 S2048: 258 -> 248 us).  What the
  // fp16 adds cost in accuracy does not show beside the rounding of O itself: rms error against float64 3.53e-4 instead
  // of 3.52e-4, the largest error unchanged.  A sum beyond fp16's range comes out infinite and moves the reference.
  auto exponentials = [&]() __attribute__((always_inline)) {
    v2h t[16];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        const float p0 = __builtin_amdgcn_exp2f(sc[h][e]), p1 = __builtin_amdgcn_exp2f(sc[h][e + 1]);
        const v2h pp = {(_Float16)p0, (_Float16)p1};
        pf[h][e / 8][e % 8] = pp[0];
        pf[h][e / 8][e % 8 + 1] = pp[1];
        t[8 * h + e / 2] = pp;
      }
#pragma unroll
    for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
      for (int i = 0; i < w; ++i) t[i] = t[i] + t[i + w];
    return (float)t[0][0] + (float)t[0][1];
  };
  // The reference maximum is not tracked tile by tile: the scores are exponentiated against the reference as it is,
  // and only when a lane's sum of exponentials says that one of them may not fit fp16 (or came out infinite) are the
  // row maxima taken, the reference moved up to them, O and the row sums rescaled, and the tile exponentiated again.
  // Any reference gives the same O = acc / l; with this one p ranges up to 2^15.  What the common path saves against a
  // maximum per tile is sixteen v_max3, the exchange with the other half-wave and their share of the issue slots that
  // the other wave's matrix instructions need.
  auto phase_s = [&](int t) __attribute__((always_inline)) {
    if (group == 0) {
      if (t + 1 < ntiles) copy_v_tile(Vb + vnext, t + 1);
    } else {
      if (t + 2 < ntiles) copy_k_tile(Kb + kcur, t + 2);   // K(t) was last read in the slot before this one
    }
    const unsigned char* v0 = Vb + vcur + v_lane;
#pragma unroll
    for (int i = 0; i < LA; ++i) vpre[i] = read_v(v0, i / DT, i % DT);
    mask_tail(sc, t);
    float psum = exponentials();
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(psum <= FA_PMAX)) != 0, 0)) {
      // v_max3 as assembly: fmaxf would first quieten each operand with a v_max of its own
      float m;
      asm("v_max3_f32 %0, %1, %2, %3" : "=v"(m) : "v"(sc[0][0]), "v"(sc[0][1]), "v"(sc[1][0]));
      asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[1][1]), "v"(sc[0][2]));
      asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[1][2]), "v"(sc[0][3]));
      asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[1][3]), "v"(sc[0][4]));
#pragma unroll
      for (int r = 4; r < 16; r += 2) {
        asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[1][r]), "v"(sc[1][r + 1]));
        if (r + 2 < 16) asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[0][r + 1]), "v"(sc[0][r + 2]));
      }
      asm("v_max3_f32 %0, %0, %1, %2" : "+v"(m) : "v"(sc[0][15]), "v"(sc[0][15]));
      m = max_with_other_half(m);   // both lanes of a row move by the same amount
      const float delta = m > 0.0f ? -m : 0.0f;
      const float alpha = __builtin_amdgcn_exp2f(delta);
      l_run *= alpha;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        nref[r] += delta;
        sc[0][r] += delta;
        sc[1][r] += delta;
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
      psum = exponentials();
    }
    l_run += psum;
  };

  auto phase_m = [&](auto next_c) __attribute__((always_inline)) {
    constexpr bool has_next = decltype(next_c)::value;
    constexpr int N = has_next ? NM : NPV;
    const unsigned char* v0 = Vb + vcur + v_lane;
    const unsigned char* k1 = Kb + knext + k_lane;
    v8h fr[NM];
#pragma unroll
    for (int i = 0; i < LA; ++i) fr[i] = vpre[i];
    __builtin_amdgcn_s_setprio(3);
    __builtin_amdgcn_sched_barrier(0);
    static_for<N>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if constexpr (i < NPV) {          // half h of the tile, contraction step s of the half, d tile dt
        constexpr int h = i / (2 * DT), s = (i % (2 * DT)) / DT, dt = i % DT;
        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[i], pf[h][s], oacc[dt], 0, 0, 0);
      } else {                          // the two halves' score chains take turns
        constexpr int ii = i - NPV, s = ii / 2, h = ii % 2;
        sc[h] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[i], qf[s], s == 0 ? nref : sc[h], 0, 0, 0);
      }
      if constexpr (i + LA < N) {
        constexpr int n = i + LA;
        if constexpr (n < NPV) {
          fr[n] = read_v(v0 + (n / (2 * DT)) * 32 * VRS, (n % (2 * DT)) / DT, n % DT);
        } else {
          fr[n] = read_k(k1 + ((n - NPV) % 2) * 32 * KRS, (n - NPV) / 2);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_setprio(0);
  };
  auto rotate = [&]() __attribute__((always_inline)) {
    int x = vcur;
    vcur = vnext;
    vnext = vfree;
    vfree = x;
    x = kcur;
    kcur = knext;
    knext = x;
  };

  auto stamp = [&](int kt, int slot) __attribute__((always_inline)) {
    if constexpr (TRACE) {
      if (blockIdx.x == 0 && tid == 64 * trace_wave && kt < FA_TRACE_TILES) trace[kt * 6 + slot] = wall_clock64();
    }
  };
  if (group == 1) phase_barrier();
  for (int t = 0; t + 1 < ntiles; ++t) {
    stamp(t, 0);
    phase_s(t);
    stamp(t, 1);
    phase_barrier();
    stamp(t, 2);
    phase_m(std::true_type{});
    stamp(t, 3);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the copies this wave requested in S(t)
    stamp(t, 4);
    phase_barrier();
    stamp(t, 5);
    rotate();
  }
  phase_s(ntiles - 1);
  phase_barrier();
  phase_m(std::false_type{});
  phase_barrier();
  if (group == 0) phase_barrier();

  // ---- normalise and store: the wave turns its 32 x D tile round through LDS (nobody reads tiles any more) and
  // stores whole rows, 1 KB of consecutive bytes per instruction
  constexpr int ORS = 2 * D + 16;
  constexpr int LPR = D / 8;
  unsigned char* const ot = smem + wave * (32 * ORS);
  const float l = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const v2h lo = {(_Float16)(oacc[dt][4 * g] * inv), (_Float16)(oacc[dt][4 * g + 1] * inv)};
      const v2h hi = {(_Float16)(oacc[dt][4 * g + 2] * inv), (_Float16)(oacc[dt][4 * g + 3] * inv)};
      *reinterpret_cast<v2u*>(ot + j * ORS + 2 * (32 * dt + 8 * g + 4 * hh)) =
          v2u{__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
    }
#pragma unroll
  for (int idx = lane; idx < 32 * LPR; idx += 64) {
    const int r = idx / LPR, c = idx - r * LPR;
    const v4u piece = *reinterpret_cast<const v4u*>(ot + r * ORS + 16 * c);
    const int row = q_base + r;
    if (row < Sq) __builtin_nontemporal_store(piece, reinterpret_cast<v4u*>(Og + (size_t)row * D + 8 * c));
  }
}

template <int D>
static int launch_fa_pp(const void* Q, const void* K, const void* V, void* O, int BH, int Sq, int Skv, float scale,
                        int lds_max, hipStream_t s) {
  const size_t tiles = (size_t)2 * FaLayout<D>::KTB + (size_t)3 * FaLayout<D>::VTB;
  const size_t lds = std::max(tiles, (size_t)8 * 32 * (2 * D + 16));   // the O tiles of the eight waves go where the K / V tiles were
  if ((int)lds > lds_max) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: needs %zu bytes of LDS", lds);
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_pp_kernel<D, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_pp_kernel<D, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
#ifdef FTK_DEBUG_TRACE
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_pp_kernel<D, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
#endif
    attr_once.done(attr_bit);
  }
  const int nqb = (Sq + 255) / 256;
  const long long total = (long long)nqb * BH;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: grid too large");
#ifdef FTK_DEBUG_TRACE
  if (long long* trace = fa_trace_ptr()) {
    hipLaunchKernelGGL((flash_attn_pp_kernel<D, true, true>), dim3((unsigned)total), dim3(512), lds, s, (const _Float16*)Q,
                       (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv, scale * 1.4426950408889634f, nqb,
                       trace, fa_trace_wave());
    return check_launch("flash_attn_pp_kernel");
  }
#endif
  if (Skv % FA_KT)
    hipLaunchKernelGGL((flash_attn_pp_kernel<D, false, true>), dim3((unsigned)total), dim3(512), lds, s, (const _Float16*)Q,
                       (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv, scale * 1.4426950408889634f, nqb,
                       (long long*)nullptr, 0);
  else
    hipLaunchKernelGGL((flash_attn_pp_kernel<D, false, false>), dim3((unsigned)total), dim3(512), lds, s, (const _Float16*)Q,
                       (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv, scale * 1.4426950408889634f, nqb,
                       (long long*)nullptr, 0);
  return check_launch("flash_attn_pp_kernel");
}


template <int D, int QT, int WAVES, int MINB>
static int launch_fa(const void* Q, const void* K, const void* V, void* O, int BH, int Sq, int Skv, float scale,
                     int lds_max, hipStream_t s) {
  const size_t lds = (size_t)3 * FaLayout<D>::KTB + (size_t)2 * FaLayout<D>::VTB;  // three K tiles, two V tiles
  if ((int)lds > lds_max) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: needs %zu bytes of LDS", lds);
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_kernel<D, QT, WAVES, MINB, false, false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_kernel<D, QT, WAVES, MINB, false, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
#ifdef FTK_DEBUG_TRACE
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_kernel<D, QT, WAVES, MINB, true, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
#endif
    attr_once.done(attr_bit);
  }
  constexpr int ROWS = WAVES * 32 * QT;
  const int nqb = (Sq + ROWS - 1) / ROWS;
  const long long total = (long long)nqb * BH;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: grid too large");
#ifdef FTK_DEBUG_TRACE
  if (long long* trace = fa_trace_ptr()) {
    hipLaunchKernelGGL((flash_attn_kernel<D, QT, WAVES, MINB, true, true>), dim3((unsigned)total), dim3(WAVES * 64), lds,
                       s, (const _Float16*)Q, (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv,
                       scale * 1.4426950408889634f, nqb, trace, fa_trace_wave());
    return check_launch("flash_attn_kernel");
  }
#endif
  if (Skv % FA_KT)
    hipLaunchKernelGGL((flash_attn_kernel<D, QT, WAVES, MINB, false, true>), dim3((unsigned)total), dim3(WAVES * 64), lds,
                       s, (const _Float16*)Q, (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv,
                       scale * 1.4426950408889634f, nqb, (long long*)nullptr, 0);
  else
    hipLaunchKernelGGL((flash_attn_kernel<D, QT, WAVES, MINB, false, false>), dim3((unsigned)total), dim3(WAVES * 64), lds,
                       s, (const _Float16*)Q, (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv,
                       scale * 1.4426950408889634f, nqb, (long long*)nullptr, 0);
  return check_launch("flash_attn_kernel");
}

// The parts of a row merged by the rule of an online softmax: m = max m_p, l = sum l_p 2^(m_p - m),
// O = sum O_p 2^(m_p - m) / l.  One thread per (row, four columns).
template <int D>
__global__ __launch_bounds__(256) void attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                        _Float16* __restrict__ O, int nparts, int Sq, long long rows) {
  constexpr int CPR = D / 4;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * CPR) return;
  const long long row = idx / CPR;
  const int c = (int)(idx - row * CPR);
  const long long bh = row / Sq;
  const int r = (int)(row - bh * Sq);
  float m = -INFINITY;
  for (int p = 0; p < nparts; ++p) m = fmaxf(m, part_ml[2 * ((bh * nparts + p) * Sq + r)]);
  float l = 0.0f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int p = 0; p < nparts; ++p) {
    const long long at = (bh * nparts + p) * Sq + r;
    const float w = __builtin_amdgcn_exp2f(part_ml[2 * at] - m);
    l += w * part_ml[2 * at + 1];
    const float4 o = *reinterpret_cast<const float4*>(part_o + at * D + 4 * c);
    acc.x += w * o.x; acc.y += w * o.y; acc.z += w * o.z; acc.w += w * o.w;
  }
  const float inv = 1.0f / l;
  const v4h out = {(_Float16)(acc.x * inv), (_Float16)(acc.y * inv), (_Float16)(acc.z * inv), (_Float16)(acc.w * inv)};
  *reinterpret_cast<v4h*>(O + row * D + 4 * c) = out;
}

// How many parts the keys are cut into (1: no split).  A grid of 128-row query blocks that fills less than half the
// chip, with enough keys that every part keeps at least four tiles.
static int fa_split_parts(long long bh, int Sq, int Skv, int cus, int* part_keys) {
  *part_keys = Skv;
  const long long blocks = (long long)((Sq + 127) / 128) * bh;
  if (blocks * 2 > cus || Skv < 2048) return 1;
  long long want = std::min<long long>(std::min<long long>(cus / blocks, 64), Skv / (4 * FA_KT));
  if (want < 2) return 1;
  const int keys = (int)(((Skv + want - 1) / want + FA_KT - 1) / FA_KT * FA_KT);
  *part_keys = keys;
  return (Skv + keys - 1) / keys;
}

static size_t fa_split_bytes(long long bh, int Sq, int D, int nparts) {
  return (size_t)nparts * bh * Sq * (D + 2) * sizeof(float);
}

template <int D>
static int launch_fa_split(const void* Q, const void* K, const void* V, void* O, int BH, int Sq, int Skv, float scale, int nparts,
                           int part_keys, float* ws, int lds_max, hipStream_t s) {
  constexpr int WAVES = 4;
  const size_t lds = (size_t)3 * FaLayout<D>::KTB + (size_t)2 * FaLayout<D>::VTB;
  if ((int)lds > lds_max) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_ws_f16: needs %zu bytes of LDS", lds);
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_kernel<D, 1, WAVES, 1, false, true, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_once.done(attr_bit);
  }
  const int nqb = (Sq + WAVES * 32 - 1) / (WAVES * 32);
  const long long total = (long long)nqb * BH * nparts;
  if (total > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_ws_f16: grid too large");
  float* part_o = ws;
  float* part_ml = ws + (size_t)nparts * BH * Sq * D;
  hipLaunchKernelGGL((flash_attn_kernel<D, 1, WAVES, 1, false, true, true>), dim3((unsigned)total), dim3(WAVES * 64), lds, s,
                     (const _Float16*)Q, (const _Float16*)K, (const _Float16*)V, (_Float16*)O, Sq, Skv, scale * 1.4426950408889634f, nqb,
                     (long long*)nullptr, 0, nparts, part_keys, part_o, part_ml);
  int rc = check_launch("flash_attn_kernel (key parts)");
  if (rc) return rc;
  const long long rows = (long long)BH * Sq;
  const long long threads = rows * (D / 4);
  hipLaunchKernelGGL(attn_merge_kernel<D>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, part_o, part_ml, (_Float16*)O, nparts, Sq, rows);
  return check_launch("attn_merge_kernel");
}

// Tuning hook: FTK_FA_VARIANT=1|3 pins the tiling variant (read once).
static int fa_variant_override() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("FTK_FA_VARIANT");
    v = e ? atoi(e) : 0;
    if (v != 1 && v != 3) v = 0;
  }
  return v;
}

}  // namespace ftk

#ifdef FTK_DEBUG_TRACE
// Copies the first n stamps of the last traced launch to host memory (synchronises the device).  Not part of
// include/ftk.h: a tuning build declares it itself.
extern "C" int ftk_debug_read_fa_trace(long long* host_dst, int n) {
  using namespace ftk;
  if (!host_dst || n <= 0 || n > FA_TRACE_TILES * 6)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_debug_read_fa_trace: need host_dst and 0 < n <= %d", FA_TRACE_TILES * 6);
  FTK_HIP(hipDeviceSynchronize());
  FTK_HIP(hipMemcpyFromSymbol(host_dst, HIP_SYMBOL(fa_trace_buf), sizeof(long long) * n));
  return FTK_OK;
}
#endif

extern "C" size_t ftk_flash_attn_f16_workspace_bytes(int B, int Hd, int Sq, int Skv, int D) {
  using namespace ftk;
  if (B <= 0 || Hd <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return 0;
  const DeviceProps* dp = nullptr;
  const int cus = device_props(&dp) == FTK_OK ? dp->cus : 256;   // without a device: the part this library is written for
  int keys = 0;
  const int nparts = fa_split_parts((long long)B * Hd, Sq, Skv, cus, &keys);
  return nparts > 1 ? fa_split_bytes((long long)B * Hd, Sq, D, nparts) : 0;
}

extern "C" int ftk_flash_attn_ws_f16(const void* Q, const void* K, const void* V, void* O, int B, int Hd, int Sq, int Skv, int D,
                                     float scale, void* workspace, size_t workspace_bytes, ftk_stream_t stream) {
  using namespace ftk;
  if (Q && K && V && O && B > 0 && Hd > 0 && Sq > 0 && Skv > 0 && (D == 32 || D == 64 || D == 96 || D == 128) && workspace &&
      (long long)B * Hd <= (1LL << 24)) {
    const DeviceProps* dp = nullptr;
    int rc = device_props(&dp);
    if (rc) return rc;
    int keys = 0;
    const long long bh = (long long)B * Hd;
    const int nparts = fa_split_parts(bh, Sq, Skv, dp->cus, &keys);
    if (nparts > 1 && workspace_bytes >= fa_split_bytes(bh, Sq, D, nparts) && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
      hipStream_t s = (hipStream_t)stream;
      float* ws = reinterpret_cast<float*>(workspace);
      switch (D) {
        case 32: return launch_fa_split<32>(Q, K, V, O, (int)bh, Sq, Skv, scale, nparts, keys, ws, dp->lds_optin, s);
        case 64: return launch_fa_split<64>(Q, K, V, O, (int)bh, Sq, Skv, scale, nparts, keys, ws, dp->lds_optin, s);
        case 96: return launch_fa_split<96>(Q, K, V, O, (int)bh, Sq, Skv, scale, nparts, keys, ws, dp->lds_optin, s);
        default: return launch_fa_split<128>(Q, K, V, O, (int)bh, Sq, Skv, scale, nparts, keys, ws, dp->lds_optin, s);
      }
    }
  }
  return ftk_flash_attn_f16(Q, K, V, O, B, Hd, Sq, Skv, D, scale, stream);   // argument checks and the unsplit kernels
}

extern "C" int ftk_flash_attn_f16(const void* Q, const void* K, const void* V, void* O, int B, int Hd, int Sq, int Skv,
                                  int D, float scale, ftk_stream_t stream) {
  using namespace ftk;
  if (!Q || !K || !V || !O) return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_flash_attn_f16: Q, K, V, O must be non-NULL");
  if (B <= 0 || Hd <= 0 || Sq <= 0 || Skv <= 0 || D <= 0)
    return fail(FTK_ERR_INVALID_ARGUMENT, "ftk_flash_attn_f16: B, Hd, Sq, Skv, D must be positive");
  if (D != 32 && D != 64 && D != 96 && D != 128)
    return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: D=%d must be 32, 64, 96 or 128", D);
  const long long bh = (long long)B * Hd;
  if (bh > (1LL << 24)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f16: B*Hd=%lld too large", bh);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  // Variant: 0 = choose by problem size, 1 = 4 waves x 32 query rows (interleaved kernel), 3 = 8 waves x 32 query rows.
  // Eight waves (two per SIMD; K / V tiles shared by 256 rows) whenever 256-row blocks fill the chip, and also on
  // smaller grids once there are 512 keys or more: measured on MI355X at B2 H12 S2048 D64 33 against 49 us, B1 H16 S2048
  // D128 44 against 50 us, B2 H8 S1024 D128 22.3 against 23.5 us (64 workgroups against 128), B4 H8 S1024 D32 14.6
  // against 16.7 us; with few keys a launch is its own latency (9.5-10 us either way) and the 128-row blocks, which
  // spread a short problem over more compute units, are kept (B1 H4 S300 D128: 10.7 against 12.2 us).
  int variant = fa_variant_override();
  if (variant == 0) variant = ((long long)((Sq + 255) / 256) * bh >= dp->cus || Skv >= 512) ? 3 : 1;
  const int lds = dp->lds_optin;
  // Grids with enough query blocks for eight waves take the kernel whose two waves per SIMD alternate between matrix
  // and vector phases (B8 H16 S2048: 248-254 us against 291-297 for the interleaved kernel at D = 128, 208 against
  // 234 at D = 96, 165 against 180 at D = 64, 98 against 114 at D = 32); the interleaved kernel keeps the 128-row
  // blocks of small grids.
  if (D == 128) {
    if (variant == 1) return launch_fa<128, 1, 4, 1>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
    return launch_fa_pp<128>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
  }
  if (D == 96) {
    if (variant == 1) return launch_fa<96, 1, 4, 1>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
    return launch_fa_pp<96>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
  }
  if (D == 64) {
    if (variant == 1) return launch_fa<64, 1, 4, 1>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
    return launch_fa_pp<64>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
  }
  // D = 32: the head dimension of the reference's example program (examples/flash_attention/flash_attention.py:96-110)
  if (variant == 1) return launch_fa<32, 1, 4, 1>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
  return launch_fa_pp<32>(Q, K, V, O, (int)bh, Sq, Skv, scale, lds, s);
}

