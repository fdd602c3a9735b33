// Measurement probe, not part of libftkernels.so: what the matrix pipes of this part deliver under load, which is
// what the fractions of the nominal fp16 MFMA peak in the benchmark lines have to be read against.
// v_mfma_f32_32x32x16_f16 from registers only, one wave per SIMD on every CU, ~2.5 ms per run: time and shader clocks
// per instruction with (a) the same constant in every lane, (b) random operands, (c) random operands that change from
// one instruction to the next.  The instruction takes 32 clocks in all three; the clock the part holds differs.
// Prints one line per case.  Build: make probes (fractaltensor_amd/csrc/Makefile); run: ./mfma_rate
#include <hip/hip_runtime.h>

#include <cstdio>

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      printf("hip error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      return 1;                                                                    \
    }                                                                              \
  } while (0)

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// DATA: 0 = every lane the same constant, 1 = random, one operand pair, 2 = random, 8 x 4 operands in turn
template <int DATA>
__global__ __launch_bounds__(256) void mfma_alone(float* out, long long* stats, int iters) {
  v16f acc[4];
  for (int a = 0; a < 4; ++a)
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;
  v8h x[8], y[4];
  unsigned h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  auto next = [&]() {
    h = h * 1664525u + 1013904223u;
    return ((h >> 8) & 0xffff) / 65536.0f - 0.5f;
  };
  for (int i = 0; i < 8; ++i)
    for (int e = 0; e < 8; ++e) {
      const float r = next();
      x[i][e] = (_Float16)(DATA == 0 ? 0.25f : DATA == 1 ? (i == 0 ? r : (float)x[0][e]) : r);
    }
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 8; ++e) {
      const float r = next();
      y[i][e] = (_Float16)(DATA == 0 ? 0.5f : DATA == 1 ? (i == 0 ? r : (float)y[0][e]) : r);
    }
  const long long c0 = __builtin_readcyclecounter();
  const long long t0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[(4 * r + a) & 7], y[(r + a) & 3], acc[a], 0, 0, 0);
  }
  const long long t1 = wall_clock64();
  const long long c1 = __builtin_readcyclecounter();
  float s = 0;
  for (int a = 0; a < 4; ++a)
    for (int r = 0; r < 16; ++r) s += acc[a][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    stats[0] = t1 - t0;   // 100 MHz ticks
    stats[1] = c1 - c0;   // shader clocks
  }
}

template <int DATA>
static int run_alone(const char* what, float* out, long long* stats) {
  const int iters = 4000;
  hipLaunchKernelGGL((mfma_alone<DATA>), dim3(256), dim3(256), 0, 0, out, stats, 10);
  CK(hipDeviceSynchronize());
  for (int rep = 0; rep < 3; ++rep) hipLaunchKernelGGL((mfma_alone<DATA>), dim3(256), dim3(256), 0, 0, out, stats, iters);
  CK(hipDeviceSynchronize());
  long long h[2];
  CK(hipMemcpy(h, stats, sizeof(h), hipMemcpyDeviceToHost));
  const double ns = h[0] * 10.0 / (iters * 32.0), ghz = (double)h[1] / (h[0] * 10.0);
  printf("mfma alone, %-42s %6.2f ns per MFMA  %5.1f clocks per MFMA  %.2f GHz  -> %4.0f TFLOP/s on 1024 SIMDs\n", what, ns,
         (double)h[1] / (iters * 32.0), ghz, 1024 * 32768.0 / ns / 1e3);
  fflush(stdout);
  return 0;
}

int main() {
  float* out;
  long long* stats;
  CK(hipMalloc(&out, 256 * 512 * sizeof(float)));
  CK(hipMalloc(&stats, 64));
  if (run_alone<0>("every lane the same constant", out, stats)) return 1;
  if (run_alone<1>("random operands, one pair", out, stats)) return 1;
  if (run_alone<2>("random operands, 8 x 4 in turn", out, stats)) return 1;
  CK(hipFree(out));
  CK(hipFree(stats));
  return 0;
}
