// Non-causal flash attention with fp32 Q, K, V and O on the fp16 matrix pipe of gfx950: every product of two
// fp32 numbers is formed as three fp16 products of split operands, accumulated in fp32.
//
// The reference's attention program computes in fp32 (examples/flash_attention/flash_attention.py:14-91 with
// kaleido.float32 blocks, flash_attention_utils.py:20-24).  fp32 MFMAs move two k per 16 passes where fp16
// MFMAs move sixteen per 8, so, as in the stacked LSTM, an fp32 product is cheaper as three fp16 ones:
//   v * 2^e = top + rest,  top = fp16(v * 2^e),  rest = fp16(v * 2^e - top),
// and top * top, top * rest and rest * top go into one fp32 accumulator; rest * rest, 2^-22 of a product, is
// dropped.  What shares a power-of-two scale 2^e (its largest magnitude lands in [2^14, 2^15)): a row of Q, all
// of K of one (batch, head), all of V of one (batch, head), and the fixed 2^7 for the softmax weights p in
// [0, 2^8).  The two planes hold an element to within 2^-40 of its group's largest magnitude (2^-29 where the
// matrix unit flushes an fp16 subnormal: the remainder of an element below 2^-17 of the largest is one), which is
// what a sum of products is accurate to anyway: 22 significant bits of its own are kept by every element within
// 2^-17 of the largest.
//
// Three launches besides a clear: the largest |K| and |V| per (batch, head); the split of K and V into planes
// [row][top D | rest D] in the workspace; the attention kernel, which splits its rows of Q (times scale * log2 e)
// itself, in registers.  A plane row is an fp16 row of 2 D
// elements, so tiles, copies and fragment reads are those of the fp16 kernel at twice the head dimension
// (fa_common.h), and the contractions are its transposed ones: S^T = K Q^T, O^T += V^T P^T, a lane owns one query
// row, the running maximum and sum are lane-local.  The reference that the weights are taken against follows the
// running maximum lazily: it moves only when a score exceeds it by more than 8 bits (kLazyBits), so weights reach
// 2^8 at most and O's accumulators (accumulation registers, which vector instructions reach only through moves)
// are rescaled once per row block on ordinary data rather than whenever one of a wave's 32 rows finds a new
// maximum (every other half tile).
#include <algorithm>
#include <type_traits>

#include "fa_common.h"

namespace ftk {

typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int kF32Top = 14;             // a scale group's largest magnitude lands in [2^14, 2^15)
constexpr float kF32PBits = 7.0f;        // 2^7: the scale of the softmax weights in their fp16 planes
constexpr float kLazyBits = 7.99f;      // how far a score may exceed the softmax reference: weights below 2^8, below 65504 in their plane
// s_waitcnt immediate: at most n vector memory operations outstanding (n < 64), the other counters left alone
constexpr int vmcnt_at_most(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// the power of two that brings a largest magnitude with these float bits into [2^14, 2^15), and its inverse
__device__ __forceinline__ void split_scale(unsigned max_bits, float* scale, float* inv) {
  const int eb = min(max((int)((max_bits >> 23) & 0xff), 15), 254 - kF32Top);
  *scale = __uint_as_float((unsigned)(127 + kF32Top + 127 - eb) << 23);
  *inv = __uint_as_float((unsigned)(eb - kF32Top) << 23);
}

__global__ void attn_f32_clear_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// largest |x| of every (batch, head) of K and V, as float bits (which order like the magnitudes): grid
// (chunks, BH, 2), per_bh a multiple of 4
__global__ __launch_bounds__(256) void attn_f32_absmax_kernel(const float* K, const float* V, unsigned* bits, size_t per_bh, int BH) {
  __shared__ unsigned wave_max[4];
  const float* x = (blockIdx.z ? V : K) + (size_t)blockIdx.y * per_bh;
  unsigned m = 0;
#pragma unroll 4
  for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < per_bh; i += (size_t)gridDim.x * 1024) {
    const float4 v = *reinterpret_cast<const float4*>(x + i);
    m = max(max(m, __float_as_uint(fabsf(v.x))), max(__float_as_uint(fabsf(v.y)), max(__float_as_uint(fabsf(v.z)), __float_as_uint(fabsf(v.w)))));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  // one atomic per workgroup: thousands of them on one word take longer than the reading
  if (threadIdx.x == 0) {
    m = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
    if (m) atomicMax(bits + blockIdx.z * BH + blockIdx.y, m);
  }
}

// One wave per row of D floats of K (blockIdx.y 0) or V (1): planes [top D | rest D] of the row under its (batch,
// head)'s scale.
template <int D>
__global__ __launch_bounds__(256) void attn_f32_split_kernel(const float* K, const float* V, _Float16* kplanes, _Float16* vplanes,
                                                            const unsigned* group_bits, int rows_per_bh, long long rows, int BH) {
  constexpr int PER = D / 32;   // floats per lane: 1, 2, 3 or 4
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* X = blockIdx.y ? V : K;
  _Float16* planes = blockIdx.y ? vplanes : kplanes;
  constexpr int LANES = D / PER > 64 ? 64 : D / PER;   // 32 lanes x PER floats cover a row
  float scale, inv;
  split_scale(group_bits[blockIdx.y * BH + row / rows_per_bh], &scale, &inv);
  if (lane < LANES) {
    _Float16* dst = planes + row * (2 * D) + lane * PER;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const float s = X[row * D + lane * PER + e] * scale;
      const _Float16 top = (_Float16)s;
      dst[e] = top;
      dst[D + e] = (_Float16)(s - (float)top);
    }
  }
}

// 4 waves x 32 query rows per workgroup, one workgroup per compute unit (the accumulators of O, both planes of Q
// and the scores take more than 256 registers at D = 128).  K and V tiles of 64 keys, both double buffered.  A wave
// works through the tiles in halves of 32 keys, and with one wave per SIMD the softmax of a half has no other
// wave's MFMAs to run beside: it is cut in two, the maxima under the P V MFMAs of the half before and the weights
// under the score MFMAs of the half after (the comments in the kernel give the order).
template <int D>
__global__ __launch_bounds__(256, 1) void flash_attn_f32_kernel(const float* __restrict__ Q, const _Float16* __restrict__ Kp,
                                                                const _Float16* __restrict__ Vp, float q_mul,
                                                                const unsigned* __restrict__ kv_bits, float* __restrict__ O,
                                                                int Sq, int Skv, int nqb, int BH) {
  using L = FaLayout<2 * D>;          // a plane row is an fp16 row of 2 D elements
  constexpr int DS = D / 16;          // k steps of S^T
  constexpr int DT = D / 32;          // d tiles of O^T
  constexpr int RB = 4 * D;           // bytes per plane row in global memory
  constexpr int KRS = L::KRS, VRS = L::VRS, KTB = L::KTB, VTB = L::VTB;
  constexpr int WAVES = 4;
  constexpr int KCP = (KTB / 1024 + WAVES - 1) / WAVES, VCP = (VTB / 1024 + WAVES - 1) / WAVES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* const Kb = smem;            // [2][KTB]
  unsigned char* const Vb = smem + 2 * KTB;  // [2][VTB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31;
  const int hh = lane >> 5;
  int id = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) id = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);   // a head's query blocks share an XCD
  const int bh = id / nqb;
  const int qb = id - bh * nqb;
  const int q_base = qb * (WAVES * 32) + wave * 32;

  const _Float16* Kg = Kp + (size_t)bh * Skv * (2 * D);
  const _Float16* Vg = Vp + (size_t)bh * Skv * (2 * D);
  float* Og = O + (size_t)bh * Sq * D;

  // The lane's query row: the fp32 row is read, multiplied by q_mul (scale * log2 e: a score leaves the matrix unit in
  // exponent units), brought under the row's own power-of-two scale and split into the two planes here, in registers
  // (a lane and its partner 32 lanes on hold the row's two halves of every 16 columns).
  const int qrow = min(q_base + j, Sq - 1);
  v8h qt[DS], qr[DS];
  float s_mul;
  {
    const float* qsrc = Q + ((size_t)bh * Sq + qrow) * D + 8 * hh;
    float4 x[DS][2];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      x[s][0] = *reinterpret_cast<const float4*>(qsrc + 16 * s);
      x[s][1] = *reinterpret_cast<const float4*>(qsrc + 16 * s + 4);
    }
    unsigned m = 0;
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        x[s][h].x *= q_mul; x[s][h].y *= q_mul; x[s][h].z *= q_mul; x[s][h].w *= q_mul;
        m = max(max(m, __float_as_uint(fabsf(x[s][h].x))), max(__float_as_uint(fabsf(x[s][h].y)),
                                                               max(__float_as_uint(fabsf(x[s][h].z)), __float_as_uint(fabsf(x[s][h].w)))));
      }
    m = max(m, (unsigned)__shfl_xor((int)m, 32));   // the row's largest magnitude, as float bits
    float q_scale, q_inv;
    split_scale(m, &q_scale, &q_inv);
#pragma unroll
    for (int s = 0; s < DS; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float v[4] = {x[s][h].x * q_scale, x[s][h].y * q_scale, x[s][h].z * q_scale, x[s][h].w * q_scale};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const _Float16 top = (_Float16)v[e];
          qt[s][4 * h + e] = top;
          qr[s][4 * h + e] = (_Float16)(v[e] - (float)top);
        }
      }
    float k_scale, k_inv;
    split_scale(kv_bits[bh], &k_scale, &k_inv);
    s_mul = q_inv * k_inv;   // what a score is multiplied by to undo the scales
  }
  float v_scale, v_inv;
  split_scale(kv_bits[BH + bh], &v_scale, &v_inv);

  v16f om[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) om[dt][r] = 0.0f;

  // copies: as in the fp16 kernel, copy c of a tile fills LDS bytes [1024 c, 1024 c + 1024) of the padded tile
  unsigned k_src[KCP], v_src[VCP];
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
  // (a whole tile takes the copies' offsets as they are; the last tile of a ragged row of keys clamps each)
  auto copy_rows = [&](auto n_c, auto bytes_c, const unsigned (&src)[decltype(n_c)::value], const _Float16* rows, int key0,
                       unsigned char* dst) __attribute__((always_inline)) {
    constexpr int N = decltype(n_c)::value, COPIES = decltype(bytes_c)::value / 1024;
    if (key0 + FA_KT <= Skv) {
      static_for<N>([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        if (WAVES * i + WAVES - 1 < COPIES || wave + WAVES * i < COPIES) lds_dma16(rows, src[i], dst + 1024 * (wave + WAVES * i));
      });
    } else {
      static_for<N>([&](auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        if (wave + WAVES * i < COPIES) {
          unsigned off = src[i];
          const unsigned last = (unsigned)(Skv - 1 - key0), row = off / RB;   // rows past the end re-read the last key; their scores are masked
          if (row > last) off -= (row - last) * RB;
          lds_dma16(rows, off, dst + 1024 * (wave + WAVES * i));
        }
      });
    }
  };
  auto copy_k = [&](int kt, int buf) __attribute__((always_inline)) {
    copy_rows(std::integral_constant<int, KCP>{}, std::integral_constant<int, KTB>{}, k_src, Kg + (size_t)kt * FA_KT * (2 * D), kt * FA_KT,
              Kb + buf * KTB);
  };
  auto copy_v = [&](int kt, int buf) __attribute__((always_inline)) {
    copy_rows(std::integral_constant<int, VCP>{}, std::integral_constant<int, VTB>{}, v_src, Vg + (size_t)kt * FA_KT * (2 * D), kt * FA_KT,
              Vb + buf * VTB);
  };
  // every wave issues at least this many copies of a K tile, of a V tile (wave 0 may issue one more)
  constexpr int KC_MIN = KTB / 1024 / WAVES, VC_MIN = VTB / 1024 / WAVES;

  const int k_lane = j * KRS + 16 * hh;
  const int v_lane = (4 * hh + ((lane & 15) >> 2)) * VRS + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
  using lds_v4s = __attribute__((address_space(3))) v4s;
  typedef short v8s __attribute__((ext_vector_type(8)));
  // A-operand of the P V product: step s (16 keys) and d tile dt of one half tile; plane 0 = values, 1 = remainders
  auto read_v = [&](const unsigned char* vbase, int s, int dt, int plane) __attribute__((always_inline)) {
    const unsigned char* p0 = vbase + 16 * s * VRS + 64 * dt + plane * (2 * D);
    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0));
    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(p0 + 8 * VRS));
    const v8s both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(v8h, both);
  };

  const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // One wave per SIMD has only its own vector instructions to put beside its MFMAs, so the softmax of a half is cut in
  // two and each part runs under the MFMAs of another product:
  //   the scores of half h                  beside  the weights of half h - 1 (exp2, the split into planes)
  //   the P V product of half h - 1         beside  the raw scores and the maximum of half h
  // and then the reference moves if it has to (rarely, see kLazyBits) and O is rescaled.
  //
  // State between the two: raw[], the scores of the half before in the matrix unit's units (times s_mul: exponent
  // units), and m_ref, the reference they are taken against; pt / pr, the weights whose product is still to come.
  float raw[16];
  float m_ref = -INFINITY, l_run = 0.0f;   // l_run: the sum of the weights, in their planes' scale
  v8h pt[2], pr[2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) { pt[s][e] = (_Float16)0.0f; pr[s][e] = (_Float16)0.0f; }
#pragma unroll
  for (int r = 0; r < 16; ++r) raw[r] = -INFINITY;   // in front of the first half: weights of zero

  // weights of pair k (two neighbouring scores) of the half before: p * 2^7 = exp2(raw * s_mul - m_ref + kF32PBits), its two planes
  float lsum = 0.0f;
  unsigned ptu[8], pru[8];
  auto weight_pair = [&](auto k_c, float bias) __attribute__((always_inline)) {
    constexpr int k = decltype(k_c)::value;
    const float s0 = __builtin_amdgcn_exp2f(fmaf(raw[2 * k], s_mul, bias)), s1 = __builtin_amdgcn_exp2f(fmaf(raw[2 * k + 1], s_mul, bias));
    lsum += s0 + s1;
    const v2f sv = {s0, s1};
    const v2h top = __builtin_convertvector(sv, v2h);
    unsigned tu = __builtin_bit_cast(unsigned, top), ru;
    // the remainders, s - top rounded to fp16: one mixed-precision fma each (the fp16 value read as fp32 times -1, plus
    // s; the difference is exact in fp32) instead of a conversion back, a subtraction and a conversion
    asm("v_fma_mixlo_f16 %0, %1, -1.0, %2 op_sel_hi:[1,0,0]\n\tv_fma_mixhi_f16 %0, %1, -1.0, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
        : "=&v"(ru) : "v"(tu), "v"(s0), "v"(s1));
    // pinned to its place: left alone, the compiler moves the arithmetic to where the weights are read, out from under the MFMAs
    asm volatile("" : "+v"(tu), "+v"(ru), "+v"(lsum));
    ptu[k] = tu;
    pru[k] = ru;
  };
  // the weights of key step h of the half (pairs 4 h .. 4 h + 3) as the P V product's fragments
  auto weights_done = [&](int h) __attribute__((always_inline)) {
    pt[h] = __builtin_bit_cast(v8h, v4u{ptu[4 * h], ptu[4 * h + 1], ptu[4 * h + 2], ptu[4 * h + 3]});
    pr[h] = __builtin_bit_cast(v8h, v4u{pru[4 * h], pru[4 * h + 1], pru[4 * h + 2], pru[4 * h + 3]});
  };
  // With an even number of d tiles the P V product uses the weights of the first key step (pairs 0..3) alone for its
  // first half: only those are formed beside the scores, pairs 4..7 beside the first half of the product itself, and
  // the maxima of the next scores beside its second half -- a wave that is alone on its SIMD hides some four vector
  // instructions per MFMA, so the vector work is dealt out as evenly as the order allows.
  constexpr bool kDefer = DT % 2 == 0;
  constexpr int kPairsBesideScores = kDefer ? 4 : 8;
  float bias = 0.0f;   // what a raw score times s_mul is offset by in the weights' exponent (set where a half's weights begin)

  // Fragments live across the two products: each requests the other's first ones before it ends, so that no product
  // begins by waiting for LDS (a read takes some hundreds of cycles under this load).
  v8h kf_t[4], kf_r[4];   // K fragments (values, remainders) of a k step, four sets in turn
  v8h vf_t[4], vf_r[4];   // V fragments of a (key step, d tile) group, two pairs of groups in turn
  auto read_k = [&](const unsigned char* kbase, int s, int set) __attribute__((always_inline)) {
    kf_t[set] = *reinterpret_cast<const v8h*>(kbase + 32 * s);
    kf_r[set] = *reinterpret_cast<const v8h*>(kbase + 2 * D + 32 * s);
  };
  auto read_group = [&](const unsigned char* pvbase, int g, int set) __attribute__((always_inline)) {
    vf_t[set] = read_v(pvbase, g / DT, g % DT, 0);
    vf_r[set] = read_v(pvbase, g / DT, g % DT, 1);
  };

  // The scores of 32 keys (one half of a tile): value x value and the two mixed products, all into am.  A step's
  // K fragments are requested three steps ahead; PRELOADED: those of steps 0 and 1 by the product before.
  // Beside the MFMAs: the weights of the half before, a share with every step; the copies of a whole tile that is
  // on its way (COPY 1: K of tile ckt, 2: V of tile ckt; 0: none), a share with every step and no branch among them;
  // and at the end the first V fragments of the product that follows (rows at pvbase).
  auto scores = [&](auto preloaded_c, auto copy_c, int ckt, int cbuf, const unsigned char* kbase, const unsigned char* pvbase,
                    v16f& am) __attribute__((always_inline)) {
    constexpr bool PRELOADED = decltype(preloaded_c)::value;
    constexpr int COPY = decltype(copy_c)::value;
    constexpr int NCOPY = COPY == 1 ? KCP : VCP;
    if constexpr (!PRELOADED) {
      read_k(kbase, 0, 0);
      read_k(kbase, 1, 1);
    }
    if constexpr (DS > 2) read_k(kbase, 2, 2);
    bias = m_ref > -INFINITY ? kF32PBits - m_ref : 0.0f;   // (no reference before the first half: every raw score is -inf)
    lsum = 0.0f;
    const _Float16* crows = (COPY == 1 ? Kg : Vg) + (size_t)ckt * FA_KT * (2 * D);
    unsigned char* cdst = COPY == 1 ? Kb + cbuf * KTB : Vb + cbuf * VTB;
    __builtin_amdgcn_sched_barrier(0);
    static_for<DS>([&](auto s_c) __attribute__((always_inline)) {
      constexpr int s = decltype(s_c)::value, b = s % 4;
      am = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf_t[b], qt[s], s == 0 ? zero16 : am, 0, 0, 0);
      if constexpr (s + 3 < DS) read_k(kbase, s + 3, (s + 3) % 4);
      if constexpr (s >= DS - 2) read_group(pvbase, s - (DS - 2), s - (DS - 2));
      am = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf_t[b], qr[s], am, 0, 0, 0);
      am = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf_r[b], qt[s], am, 0, 0, 0);
      static_for<kPairsBesideScores * (s + 1) / DS - kPairsBesideScores * s / DS>([&](auto j_c) __attribute__((always_inline)) {
        weight_pair(std::integral_constant<int, kPairsBesideScores * s / DS + decltype(j_c)::value>{}, bias);
      });
      // the order within the step: MFMA, the reads, and the vector instructions in three shares behind the three MFMAs
      // (the first share holds the two exp2, four issue slots each)
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, s >= DS - 2 ? 4 : 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (COPY != 0) {
        static_for<NCOPY * (s + 1) / DS - NCOPY * s / DS>([&](auto j_c) __attribute__((always_inline)) {
          constexpr int i = NCOPY * s / DS + decltype(j_c)::value, COPIES = (COPY == 1 ? KTB : VTB) / 1024;
          const unsigned src = COPY == 1 ? k_src[i % KCP] : v_src[i % VCP];
          if (WAVES * i + WAVES - 1 < COPIES || wave + WAVES * i < COPIES) lds_dma16(crows, src, cdst + 1024 * (wave + WAVES * i));
        });
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    weights_done(0);
    if constexpr (!kDefer) {
      weights_done(1);
      l_run += lsum;
    }
  };

  // The P V product of the half whose weights are in pt / pr (V rows at pvbase), and beside it (MAXIMA) the raw
  // scores and the maximum of the half whose products are in am; then the reference moves if a score exceeds it
  // by more than kLazyBits, and O and the sum are brought to the new one.  Groups (key step, d tile: 3 MFMAs) are
  // taken two at a time, in an order in which no MFMA adds to the result of the one before it; a pair's V fragments are
  // requested under the pair before.
  auto pv_and_maxima = [&](auto maxima_c, auto next_k_c, auto mask_c, const unsigned char* pvbase, const unsigned char* next_kbase,
                           const v16f& am, int key0) __attribute__((always_inline)) {
    // MAXIMA false: the product alone, behind the last half, all of whose weights are there; MASK: the half is ragged
    constexpr bool MAXIMA = decltype(maxima_c)::value, NEXT_K = decltype(next_k_c)::value, MASK = decltype(mask_c)::value;
    constexpr bool DEFER = kDefer && MAXIMA;
    constexpr int NG = 2 * DT, NM = 3 * NG;
    constexpr int M0 = DEFER ? NM / 2 : 0, MN = NM - M0;   // the slots that hold the maxima
    // (the first pair's fragments were requested by the scores before; NEXT_K: the last slots request the K fragments
    // of steps 0 and 1 of the scores that follow, rows at next_kbase)
    float mx = -INFINITY;
    [[maybe_unused]] const int lim = Skv - key0 - 4 * hh;   // score r belongs to a key past the end when 8 (r >> 2) + (r & 3) >= lim
    static_for<NM>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value, pair = i / 6, k = i % 6, g0 = 2 * pair, g1 = g0 + 1;
      constexpr int b0 = (pair & 1) * 2, b1 = b0 + 1, nb = ((pair + 1) & 1) * 2;
      constexpr int sk0 = g0 / DT, dt0 = g0 % DT, sk1 = g1 / DT, dt1 = g1 % DT;
      if constexpr ((k == 1 || k == 3) && g0 + 2 < NG) read_group(pvbase, g0 + 2 + (k == 3), nb + (k == 3));   // the next pair's fragments
      if constexpr (NEXT_K && g0 + 2 >= NG && (k == 1 || k == 3)) read_k(next_kbase, k == 3, k == 3);
      if constexpr (k == 0) om[dt0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_t[b0], pt[sk0], om[dt0], 0, 0, 0);
      if constexpr (k == 1) om[dt1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_t[b1], pt[sk1], om[dt1], 0, 0, 0);
      if constexpr (k == 2) om[dt0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_t[b0], pr[sk0], om[dt0], 0, 0, 0);
      if constexpr (k == 3) om[dt1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_t[b1], pr[sk1], om[dt1], 0, 0, 0);
      if constexpr (k == 4) om[dt0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_r[b0], pt[sk0], om[dt0], 0, 0, 0);
      if constexpr (k == 5) om[dt1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf_r[b1], pt[sk1], om[dt1], 0, 0, 0);
      if constexpr (DEFER && i < M0) {   // the weights of the second key step (pairs 4..7), wanted by this product's second half
        static_for<4 * (i + 1) / M0 - 4 * i / M0>([&](auto j_c) __attribute__((always_inline)) {
          weight_pair(std::integral_constant<int, 4 + 4 * i / M0 + decltype(j_c)::value>{}, bias);
        });
        if constexpr (i == M0 - 1) {
          weights_done(1);
          l_run += lsum;
        }
      }
      if constexpr (MAXIMA && i >= M0) {
#pragma unroll
        for (int r = 16 * (i - M0) / MN; r < 16 * (i - M0 + 1) / MN; ++r) {
          raw[r] = am[r];
          if constexpr (MASK) {
            if (8 * (r >> 2) + (r & 3) >= lim) raw[r] = -INFINITY;
          }
          mx = fmaxf(mx, raw[r]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (MAXIMA) {
      mx = max_with_other_half(mx) * s_mul;   // finite: the half holds at least one key; s_mul > 0
      if (__builtin_amdgcn_ballot_w64(mx > m_ref + kLazyBits) != 0) {   // a row of the wave moves its reference
        const bool moves = mx > m_ref + kLazyBits;
        const float m_new = moves ? mx : m_ref;
        const float alpha = moves ? __builtin_amdgcn_exp2f(m_ref - m_new) : 1.0f;   // 0 the first time (m_ref = -inf)
        m_ref = m_new;
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) om[dt][r] *= alpha;
      }
    }
  };

  // A tile's K rows are last read by the scores of its second half and its V rows one half later, beside the next
  // tile's first maxima: K of tile kt + 1 is requested beside the scores of tile kt's first half, V of tile kt + 1
  // beside those of its second half, behind the barrier in the middle of the tile.  Copies complete in the order of their issue, so each of the two barriers waits for the
  // older of the two requests only.
  const int ntiles = (Skv + FA_KT - 1) / FA_KT;
  copy_k(0, 0);
  copy_v(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();

  const unsigned char* pend_v = Vb + v_lane;   // the V rows of the half whose product is still to come (first: zero weights on tile 0)
  for (int kt = 0; kt < ntiles; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < ntiles;
    const bool whole_next = (kt + 2) * FA_KT <= Skv;   // a tile follows and all of its 64 keys exist
    {   // first half; beside its scores, K of tile kt + 1 is requested (K[buf ^ 1] was last read before the barrier that ended tile kt - 1)
      v16f am;
      const unsigned char* kbase = Kb + buf * KTB + k_lane;
      if (whole_next) {
        scores(std::false_type{}, std::integral_constant<int, 1>{}, kt + 1, buf ^ 1, kbase, pend_v, am);
      } else {
        if (more) copy_k(kt + 1, buf ^ 1);   // the last, ragged tile: each copy clamps its rows
        scores(std::false_type{}, std::integral_constant<int, 0>{}, 0, 0, kbase, pend_v, am);
      }
      if (kt * FA_KT + 32 <= Skv) pv_and_maxima(std::true_type{}, std::true_type{}, std::false_type{}, pend_v, kbase + 32 * KRS, am, kt * FA_KT);
      else pv_and_maxima(std::true_type{}, std::true_type{}, std::true_type{}, pend_v, kbase + 32 * KRS, am, kt * FA_KT);
      pend_v = Vb + buf * VTB + v_lane;
    }
    // V of tile kt has landed in every wave (asked for half a tile ago or more); V[buf ^ 1] has been read for the last time
    if (more) __builtin_amdgcn_s_waitcnt(vmcnt_at_most(KC_MIN));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (kt * FA_KT + 32 < Skv) {   // second half (a tile that is followed by another has one); beside its scores, V of tile kt + 1 is requested
      v16f am;
      const unsigned char* kbase = Kb + buf * KTB + k_lane + 32 * KRS;
      if (whole_next) {
        scores(std::true_type{}, std::integral_constant<int, 2>{}, kt + 1, buf ^ 1, kbase, pend_v, am);
      } else {
        if (more) copy_v(kt + 1, buf ^ 1);
        scores(std::true_type{}, std::integral_constant<int, 0>{}, 0, 0, kbase, pend_v, am);
      }
      if (kt * FA_KT + 64 <= Skv) pv_and_maxima(std::true_type{}, std::false_type{}, std::false_type{}, pend_v, nullptr, am, kt * FA_KT + 32);
      else pv_and_maxima(std::true_type{}, std::false_type{}, std::true_type{}, pend_v, nullptr, am, kt * FA_KT + 32);
      pend_v = Vb + buf * VTB + v_lane + 32 * VRS;
    }
    // K of tile kt + 1 has landed; K[buf] has been read for the last time
    if (more) __builtin_amdgcn_s_waitcnt(vmcnt_at_most(VC_MIN));
    __syncthreads();
  }
  {   // the last half's weights, then its product
    bias = kF32PBits - m_ref;
    lsum = 0.0f;
    static_for<8>([&](auto k_c) __attribute__((always_inline)) { weight_pair(k_c, bias); });
    weights_done(0);
    weights_done(1);
    l_run += lsum;
    read_group(pend_v, 0, 0);
    read_group(pend_v, 1, 1);
    const v16f none = zero16;
    pv_and_maxima(std::false_type{}, std::false_type{}, std::false_type{}, pend_v, nullptr, none, 0);
  }
  __syncthreads();   // LDS is reused below

  // ---- normalise and store: the wave turns its 32 x D tile round through the LDS nobody reads any more (the
  // barrier above ended the last tile), so that whole rows leave as consecutive bytes
  constexpr int ORS = 4 * D + 16;
  constexpr int LPR = D / 4;   // 16-byte chunks per row
  unsigned char* const ot = smem + wave * (32 * ORS);
  const float l = l_run + __shfl_xor(l_run, 32);
  const float fin = v_inv / l;   // l in the scale of the weights' planes, as O's accumulators
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float4 o;
      o.x = om[dt][4 * g + 0] * fin;
      o.y = om[dt][4 * g + 1] * fin;
      o.z = om[dt][4 * g + 2] * fin;
      o.w = om[dt][4 * g + 3] * fin;
      *reinterpret_cast<float4*>(ot + j * ORS + 4 * (32 * dt + 8 * g + 4 * hh)) = o;
    }
#pragma unroll
  for (int idx = lane; idx < 32 * LPR; idx += 64) {
    const int r = idx / LPR, c = idx - r * LPR;
    const v4u piece = *reinterpret_cast<const v4u*>(ot + r * ORS + 16 * c);
    const int row = q_base + r;
    if (row < Sq) __builtin_nontemporal_store(piece, reinterpret_cast<v4u*>(Og + (size_t)row * D + 4 * c));
  }
}

static size_t round256f(size_t v) { return (v + 255) / 256 * 256; }

struct F32Layout {
  size_t bits, kp, vp, total;
};
static F32Layout f32_layout(long long bh, int Skv, int D) {
  F32Layout w;
  w.bits = 0;
  w.kp = round256f((size_t)2 * bh * sizeof(unsigned));
  w.vp = w.kp + round256f((size_t)bh * Skv * 2 * D * sizeof(_Float16));
  w.total = w.vp + round256f((size_t)bh * Skv * 2 * D * sizeof(_Float16));
  return w;
}

template <int D>
static int launch_fa_f32(const float* Q, const float* K, const float* V, float* O, int BH, int Sq, int Skv, float scale, char* ws,
                         const F32Layout& w, int lds_max, hipStream_t s) {
  using L = FaLayout<2 * D>;
  const size_t lds = std::max((size_t)2 * (L::KTB + L::VTB), (size_t)4 * 32 * (4 * D + 16));
  if ((int)lds > lds_max) return fail(FTK_ERR_DEVICE, "ftk_flash_attn_f32: D=%d needs %zu bytes of LDS, the device offers %d", D, lds, lds_max);
  unsigned* bits = reinterpret_cast<unsigned*>(ws + w.bits);
  _Float16* kp = reinterpret_cast<_Float16*>(ws + w.kp);
  _Float16* vp = reinterpret_cast<_Float16*>(ws + w.vp);
  hipLaunchKernelGGL(attn_f32_clear_kernel, dim3((2 * BH + 255) / 256), dim3(256), 0, s, bits, 2 * BH);
  int rc = check_launch("attn_f32_clear_kernel");
  if (rc) return rc;
  const size_t per_bh = (size_t)Skv * D;
  const int chunks = (int)std::min<size_t>(std::max(1, 4096 / (2 * BH)), (per_bh + 4095) / 4096);   // some 4096 workgroups in all
  hipLaunchKernelGGL(attn_f32_absmax_kernel, dim3(chunks, BH, 2), dim3(256), 0, s, K, V, bits, per_bh, BH);
  rc = check_launch("attn_f32_absmax_kernel");
  if (rc) return rc;
  const long long krows = (long long)BH * Skv;
  hipLaunchKernelGGL(attn_f32_split_kernel<D>, dim3((unsigned)((krows + 3) / 4), 2), dim3(256), 0, s, K, V, kp, vp, (const unsigned*)bits, Skv, krows,
                     BH);
  rc = check_launch("attn_f32_split_kernel");
  if (rc) return rc;
  const int nqb = (Sq + 127) / 128;
  const long long blocks = (long long)nqb * BH;
  if (blocks > 0x7fffffffLL) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "ftk_flash_attn_f32: grid too large");
  static DeviceOnce attr_once;
  unsigned attr_bit;
  if (attr_once.pending(&attr_bit)) {
    FTK_HIP(hipFuncSetAttribute((const void*)flash_attn_f32_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_once.done(attr_bit);
  }
  hipLaunchKernelGGL(flash_attn_f32_kernel<D>, dim3((unsigned)blocks), dim3(256), lds, s, Q, kp, vp, scale * 1.4426950408889634f, bits, O, Sq, Skv, nqb, BH);
  return check_launch("flash_attn_f32_kernel");
}

}  // namespace ftk

extern "C" size_t ftk_flash_attn_f32_workspace_bytes(int B, int Hd, int Sq, int Skv, int D) {
  if (B <= 0 || Hd <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return 0;
  return ftk::f32_layout((long long)B * Hd, Skv, D).total;
}

extern "C" int ftk_flash_attn_f32(const float* Q, const float* K, const float* V, float* O, int B, int Hd, int Sq, int Skv, int D,
                                  float scale, void* workspace, size_t workspace_bytes, ftk_stream_t stream) {
  using namespace ftk;
  const char* who = "ftk_flash_attn_f32";
  if (!Q || !K || !V || !O) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: Q, K, V, O must be non-NULL", who);
  if (B <= 0 || Hd <= 0 || Sq <= 0 || Skv <= 0 || D <= 0) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: B, Hd, Sq, Skv, D must be positive", who);
  if (D != 32 && D != 64 && D != 96 && D != 128) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: D=%d must be 32, 64, 96 or 128", who, D);
  if ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(O)) % 16)
    return fail(FTK_ERR_INVALID_ARGUMENT, "%s: Q, K, V, O must be 16-byte aligned", who);   // rows are read and written 16 bytes at a time
  if (!(scale > 0.0f) || !(scale < INFINITY)) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: scale must be positive and finite", who);
  const long long bh = (long long)B * Hd;
  if (bh > (1LL << 16)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: B*Hd=%lld too large", who, bh);
  if ((long long)Skv * D >= (1LL << 31) || (long long)Sq * D >= (1LL << 31)) return fail(FTK_ERR_UNSUPPORTED_SHAPE, "%s: a head is too large", who);
  const F32Layout w = f32_layout(bh, Skv, D);
  if (!workspace || workspace_bytes < w.total)
    return fail(FTK_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, w.total, workspace ? workspace_bytes : (size_t)0);
  if (reinterpret_cast<uintptr_t>(workspace) % 256) return fail(FTK_ERR_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", who);
  const DeviceProps* dp = nullptr;
  int rc = device_props(&dp);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  switch (D) {
    case 32: return launch_fa_f32<32>(Q, K, V, O, (int)bh, Sq, Skv, scale, ws, w, dp->lds_optin, s);
    case 64: return launch_fa_f32<64>(Q, K, V, O, (int)bh, Sq, Skv, scale, ws, w, dp->lds_optin, s);
    case 96: return launch_fa_f32<96>(Q, K, V, O, (int)bh, Sq, Skv, scale, ws, w, dp->lds_optin, s);
    default: return launch_fa_f32<128>(Q, K, V, O, (int)bh, Sq, Skv, scale, ws, w, dp->lds_optin, s);
  }
}
