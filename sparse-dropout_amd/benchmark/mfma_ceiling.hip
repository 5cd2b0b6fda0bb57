// What the matrix cores sustain when nothing else happens: back-to-back v_mfma_f32_32x32x16_f16 and
// v_mfma_f32_16x16x32_f16 from registers, 4 or 8 waves per CU on all 256 CUs, on constant and on N(0,1)
// operands.  On random data the chip is power-limited (the clock drops), so this, not the 2.5 PFLOP/s of the
// data sheet, is the ceiling a GEMM kernel can approach on the benchmark's data; it is also what says which
// MFMA shape to build the kernels on.
//
//   hipcc --offload-arch=gfx950 -O3 -w -Xclang -target-feature -Xclang -packed-fp32-ops \
//         -o /tmp/mfma_ceiling sparse-dropout_amd/benchmark/mfma_ceiling.hip && /tmp/mfma_ceiling
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <vector>
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int WAVES, int SHAPE>
__global__ __launch_bounds__(WAVES*64) void mfma_rate(const f16x8* src, float* out, int iters) {
  f16x8 a[4], b[4];
  for (int i = 0; i < 4; ++i) { a[i] = src[(blockIdx.x * WAVES * 64 + threadIdx.x) * 8 + i]; b[i] = src[(blockIdx.x * WAVES * 64 + threadIdx.x) * 8 + 4 + i]; }
  float s = 0;
  if constexpr (SHAPE == 32) {
    f32x16 c[8] = {};
    for (int it = 0; it < iters; it += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 3], b[(j + u) & 3], c[j], 0, 0, 0);
    }
    for (int j = 0; j < 8; ++j) for (int i = 0; i < 16; ++i) s += c[j][i];
  } else {
    f32x4 c[32] = {};
    for (int it = 0; it < iters; it += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 32; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j & 3], b[((j >> 2) + u) & 3], c[j], 0, 0, 0);
    }
    for (int j = 0; j < 32; ++j) for (int i = 0; i < 4; ++i) s += c[j][i];
  }
  out[blockIdx.x * WAVES * 64 + threadIdx.x] = s;
}
static float gauss() { float u1 = (rand() + 1.0f) / (RAND_MAX + 2.0f), u2 = (float)rand() / RAND_MAX; return sqrtf(-2 * logf(u1)) * cosf(6.2831853f * u2); }
template <int W, int S> float run(const f16x8* d, float* o, int blocks, int iters) {
  hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
  mfma_rate<W, S><<<blocks, W * 64>>>(d, o, 100); hipDeviceSynchronize();
  hipEventRecord(e0); mfma_rate<W, S><<<blocks, W * 64>>>(d, o, iters); hipEventRecord(e1); hipEventSynchronize(e1);
  float ms; hipEventElapsedTime(&ms, e0, e1); return ms;
}
int main() {
  int blocks = 256; size_t n = (size_t)blocks * 512 * 8 * 8;
  std::vector<_Float16> h(n);
  _Float16* d; hipMalloc(&d, n * 2); float* o; hipMalloc(&o, blocks * 512 * 4);
  for (int mode = 0; mode < 3; ++mode) {
    for (size_t i = 0; i < n; ++i) { float g = gauss(); h[i] = (_Float16)(mode == 0 ? 1.0f : (mode == 1 ? g : ((i / 32) % 2 ? g * 0.011f : g))); }
    hipMemcpy(d, h.data(), n * 2, hipMemcpyHostToDevice);
    const char* nm = mode == 0 ? "all ones" : (mode == 1 ? "N(0,1) both" : "A N(0,1), B N(0,1)/90");
    for (int rep = 0; rep < 2; ++rep) {
      int it32 = 20000, it16 = 10000;  // same flops: 8 x 32768 x it32 == 32 x 16384 x it16
      float m;
      m = run<4, 32>((const f16x8*)d, o, blocks, it32); printf("%-22s 32x32x16 4 waves/CU: %.2f ms %.1f TFLOP/s\n", nm, m, (double)blocks * 4 * 8.0 * it32 * 32768 / m / 1e9);
      m = run<4, 16>((const f16x8*)d, o, blocks, it16); printf("%-22s 16x16x32 4 waves/CU: %.2f ms %.1f TFLOP/s\n", nm, m, (double)blocks * 4 * 32.0 * it16 * 16384 / m / 1e9);
      m = run<8, 32>((const f16x8*)d, o, blocks, it32); printf("%-22s 32x32x16 8 waves/CU: %.2f ms %.1f TFLOP/s\n", nm, m, (double)blocks * 8 * 8.0 * it32 * 32768 / m / 1e9);
      m = run<8, 16>((const f16x8*)d, o, blocks, it16); printf("%-22s 16x16x32 8 waves/CU: %.2f ms %.1f TFLOP/s\n", nm, m, (double)blocks * 8 * 32.0 * it16 * 16384 / m / 1e9);
      fflush(stdout);
    }
  }
  return 0;
}
