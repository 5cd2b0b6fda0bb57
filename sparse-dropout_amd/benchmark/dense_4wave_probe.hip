// How fast the dense product C = A . B^T (fp16, fp32 accumulation, 8192^3) runs with FOUR waves per workgroup, each
// owning 128 x 128 of a 256 x 256 tile, against the library's eight waves of 128 x 64: per 64-wide reduction step a
// workgroup then reads 128 KB of fragments back from LDS instead of 192 KB (plus the same 64 KB written by the tile
// loads), and each SIMD runs one instruction stream instead of two.  The 256 accumulator registers of a wave are
// pinned to the accumulation registers by writing the MFMAs as inline assembly; left to the compiler they are spread
// over both register files, moved around inside the loop and spilled.
// Everything else follows the library's kernels: global_load_lds_dwordx4 into two 64 KB stages, 128-byte tile rows
// with the 16-byte chunks XOR-swizzled by the row, one barrier per step in front of the step's last unit, fragments
// of the next unit read before the MFMAs of the current one.  The store is plain (no staging through LDS): the
// program prints the time with and without it.
//
//   hipcc --offload-arch=gfx950 -O3 -w -Xclang -target-feature -Xclang -packed-fp32-ops \
//         -o /tmp/dense_4wave_probe sparse-dropout_amd/benchmark/dense_4wave_probe.hip && /tmp/dense_4wave_probe
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef __attribute__((address_space(3))) void lds_void;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#ifndef LOAD_EVERY
#define LOAD_EVERY 1
#endif
constexpr int THREADS = 256, BM = 256, BN = 256, BK = 64, STAGE = (BM + BN) * BK * 2, B_OFF = BM * BK * 2;

__device__ inline void load16_to_lds(const char* base, uint32_t lane_off, uint32_t lds_dst) {
  const uint64_t b = (uint64_t)(uintptr_t)base;
  const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t a = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sb), "s"(a)
               : "memory");
}

// acc += a . b^T on a 16 x 16 tile over 32 reduction indices; acc lives in the accumulation registers
__device__ inline void mfma16(f32x4& acc, const u32x4& a, const u32x4& b) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// A [M, K], B [N, K], C [M, N], all row-major fp16; M, N multiples of 256, K of 64
__global__ __launch_bounds__(THREADS) void gemm4(const __half* A, const __half* B, __half* C, int M, int N, int K,
                                                 int store) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t smem_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_void*)smem);
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int rh = wave / 2, nh = wave % 2;  // the wave's 128 rows and 128 columns of the tile
  // consecutive workgroups go to consecutive XCDs: give each XCD an 8 x 4 patch of tiles (as the library does)
  const int tiles_m = M / BM, tiles_n = N / BN;
  int tm, tn;
  {
    const int bid = blockIdx.x, xcd = bid % 8, slot = bid / 8;
    const int patches_n = tiles_n / 4;
    const int patch = (slot / 32) * 8 + xcd, in = slot % 32;
    tm = (patch / patches_n) * 8 + in % 8;
    tn = (patch % patches_n) * 4 + in / 8;
  }
  const char* a_base = reinterpret_cast<const char*>(A + (size_t)tm * BM * K);
  const char* b_base = reinterpret_cast<const char*>(B + (size_t)tn * BN * K);
  const uint32_t ldk = (uint32_t)K * 2;
  // tile loads: one instruction = 8 rows x 128 bytes; group g of 8 rows has its chunks swizzled by (row >> 1) & 7 =
  // 4 * (g & 1) + (lane >> 4)
  uint32_t lane_off[2];
#pragma unroll
  for (int par = 0; par < 2; ++par)
    lane_off[par] = (uint32_t)(lane / 8) * ldk + (uint32_t)(((lane % 8) ^ (4 * par + (lane >> 4))) * 16);
  // load i (0-7: rows of A, 8-15: rows of B) of this wave's 16 for a step
  auto issue_load = [&](int step, int stage, int i) {
    const uint32_t st = smem_a + (uint32_t)(stage * STAGE);
    const int g = wave * 8 + (i & 7);  // rows 8g .. 8g + 7 of the operand's 256
    const char* base = i < 8 ? a_base : b_base;
    load16_to_lds(base + (size_t)(8 * g) * ldk + (size_t)step * (BK * 2), lane_off[i & 1],
                  st + (i < 8 ? 0 : B_OFF) + g * 1024);
  };
  auto issue_loads = [&](int step, int stage) {
#pragma unroll
    for (int i = 0; i < 16; ++i) issue_load(step, stage, i);
  };
  // fragment of rows (lane % 16) of a 16-row tile, reduction indices 32 * kk + 8 * (lane / 16) .. + 7
  int f_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) f_off[kk] = (lane % 16) * 128 + ((4 * kk + lane / 16) ^ ((lane >> 1) & 7)) * 16;

  f32x4 acc[2][4][8];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int n = 0; n < 8; ++n) acc[r][m][n] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 af[2][4], bf[2][8];
  auto read_a = [&](int buf, int stage, int rb, int kk) {
    const char* p = smem + stage * STAGE + (2 * rh + rb) * 8192 + f_off[kk];
#pragma unroll
    for (int m = 0; m < 4; ++m) af[buf][m] = *reinterpret_cast<const u32x4*>(p + m * 2048);
  };
  auto read_b = [&](int buf, int stage, int kk) {
    const char* p = smem + stage * STAGE + B_OFF + (2 * nh) * 8192 + f_off[kk];
#pragma unroll
    for (int n = 0; n < 8; ++n) bf[buf][n] = *reinterpret_cast<const u32x4*>(p + n * 2048);
  };
  // the MFMAs of one unit; `prefetch` (the fragment reads of the next unit) is issued behind the first of them, so
  // that the wait in front of the unit covers only what the unit itself needs; `between(i)` runs behind MFMA i
  auto mfmas = [&](int rb, int abuf, int bbuf, auto prefetch, auto between) {
    __builtin_amdgcn_sched_barrier(0);
    mfma16(acc[rb][0][0], af[abuf][0], bf[bbuf][0]);
    __builtin_amdgcn_sched_barrier(0);
    prefetch();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int n = 0; n < 8; ++n)
        if (m || n) {
          mfma16(acc[rb][m][n], af[abuf][m], bf[bbuf][n]);
          between(m * 8 + n);
        }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto nothing = [](int) {};

  const int nsteps = K / BK;
  issue_loads(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (nsteps > 1) issue_loads(1, 1);
  read_a(0, 0, 0, 0);
  read_b(0, 0, 0);
  for (int step = 0; step < nsteps; ++step) {
    const int stage = step & 1;
    // units (row block, kk): (0,0) (1,0) (0,1) (1,1); the W fragments of a kk serve both row blocks
    mfmas(0, 0, 0, [&] { read_a(1, stage, 1, 0); }, nothing);
    mfmas(1, 1, 0, [&] {
      read_a(0, stage, 0, 1);
      read_b(1, stage, 1);
    }, nothing);
    mfmas(0, 0, 1, [&] { read_a(1, stage, 1, 1); }, nothing);
    // every fragment of this stage is in registers (or on its way): publish the next stage, refill this one
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const bool more = step + 2 < nsteps;
    if (LOAD_EVERY == 0 && more) issue_loads(step + 2, stage);
    mfmas(1, 1, 1, [&] {
      if (step + 1 < nsteps) {
        read_a(0, stage ^ 1, 0, 0);
        read_b(0, stage ^ 1, 0);
      }
    }, [&](int i) {
      // the wave's 16 tile loads, one behind every LOAD_EVERY-th MFMA: a wave that stands at a load issues nothing
      // else, and this SIMD has no second wave to fill in
      if (LOAD_EVERY > 0 && more && i % LOAD_EVERY == 0 && i / LOAD_EVERY - 1 < 16 && i >= LOAD_EVERY)
        issue_load(step + 2, stage, i / LOAD_EVERY - 1);
    });
    if (LOAD_EVERY > 0 && more) {  // what the unit had no room for
#pragma unroll
      for (int i = 31 / LOAD_EVERY; i < 16; ++i) issue_load(step + 2, stage, i);
    }
  }
  // the MFMAs above are opaque to the compiler: let the last ones drain before the accumulators are read
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  if (!store) {
    // keep the accumulators alive without the store's time
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < 8; ++n) s += acc[r][m][n][0] + acc[r][m][n][1] + acc[r][m][n][2] + acc[r][m][n][3];
    if (s == 123.456f) C[0] = __float2half(s);
    return;
  }
  // register v of lane l is element (4 * (l / 16) + v, l % 16) of the 16 x 16 tile
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int n = 0; n < 8; ++n)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const size_t row = (size_t)tm * BM + (2 * rh + r) * 64 + m * 16 + 4 * (lane / 16) + v;
          const size_t col = (size_t)tn * BN + nh * 128 + n * 16 + lane % 16;
          C[row * N + col] = __float2half(acc[r][m][n][v]);
        }
}

int main() {
  const int M = 8192, N = 8192, K = 8192;
  std::vector<__half> ha((size_t)M * K), hb((size_t)N * K);
  uint32_t s = 12345u;
  auto rnd = [&]() {
    s = s * 1664525u + 1013904223u;
    return ((int)(s >> 9) % 2001 - 1000) * 1e-3f;
  };
  for (auto& v : ha) v = __float2half(rnd());
  for (auto& v : hb) v = __float2half(rnd() * 0.011f);
  __half *A, *B, *C;
  if (hipMalloc(&A, ha.size() * 2) != hipSuccess || hipMalloc(&B, hb.size() * 2) != hipSuccess ||
      hipMalloc(&C, (size_t)M * N * 2) != hipSuccess) {
    printf("hipMalloc failed\n");
    return 1;
  }
  hipMemcpy(A, ha.data(), ha.size() * 2, hipMemcpyHostToDevice);
  hipMemcpy(B, hb.data(), hb.size() * 2, hipMemcpyHostToDevice);
  hipMemset(C, 0, (size_t)M * N * 2);
  hipFuncSetAttribute((const void*)gemm4, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE);
  const int grid = (M / BM) * (N / BN);
  // correctness on a few elements
  gemm4<<<grid, THREADS, 2 * STAGE>>>(A, B, C, M, N, K, 1);
  if (hipDeviceSynchronize() != hipSuccess) {
    printf("kernel failed: %s\n", hipGetErrorString(hipGetLastError()));
    return 1;
  }
  double worst = 0;
  for (int t = 0; t < 64; ++t) {
    const int i = (t * 1237 + 5) % M, j = (t * 7919 + 11) % N;
    double ref = 0;
    for (int k = 0; k < K; ++k) ref += (double)__half2float(ha[(size_t)i * K + k]) * (double)__half2float(hb[(size_t)j * K + k]);
    __half got;
    hipMemcpy(&got, C + (size_t)i * N + j, 2, hipMemcpyDeviceToHost);
    const double err = fabs((double)__half2float(got) - ref) / (fabs(ref) + 1e-2);
    if (err > worst) worst = err;
  }
  printf("largest relative error over 64 sampled elements: %.2e\n", worst);
  for (int store = 0; store < 2; ++store) {
    for (int rep = 0; rep < 3; ++rep) {
      hipEvent_t e0, e1;
      hipEventCreate(&e0);
      hipEventCreate(&e1);
      for (int w = 0; w < 3; ++w) gemm4<<<grid, THREADS, 2 * STAGE>>>(A, B, C, M, N, K, store);
      hipDeviceSynchronize();
      const int iters = 20;
      hipEventRecord(e0);
      for (int it = 0; it < iters; ++it) gemm4<<<grid, THREADS, 2 * STAGE>>>(A, B, C, M, N, K, store);
      hipEventRecord(e1);
      hipEventSynchronize(e1);
      float ms;
      hipEventElapsedTime(&ms, e0, e1);
      const double us = ms * 1e3 / iters;
      printf("%-22s %8.1f us per launch  %7.1f TFLOP/s\n", store ? "with the plain store" : "without the store", us,
             2.0 * M * N * K / (us * 1e-6) / 1e12);
    }
  }
  return 0;
}
