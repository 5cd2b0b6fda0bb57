// What the global -> LDS path sustains when nothing else happens: every CU streams 64 KB steps into two LDS
// stages with global_load_lds_dwordx4, one step in flight behind a barrier per step - the load side of the GEMM
// kernels without their fragment reads and MFMAs - under four address patterns:
//   private   each workgroup walks its own contiguous region (every byte fetched once per pass; regions small
//             enough to stay in L2)
//   rows      each workgroup's step is 512 rows of 128 bytes, 16 KB apart: the tile rows of an 8192-wide fp16
//             operand, private to the workgroup
//   shared    the 32 workgroups of an XCD walk the tile rows of 8 + 4 operand panels the way the GEMM's 8 x 4
//             patch of 256 x 256 tiles does (each step's bytes wanted by 4 or 8 workgroups at the same time);
//             the panels are `positions` steps long and walked round and round: with 64 positions all panels
//             together are 192 MB (they stay in the 256 MB memory-side cache), with 128 they are 384 MB (the
//             L2 misses, a fifth of the requests, go to HBM as 128-byte reads 16 KB apart)
//   hbm       private regions far larger than the caches
//   staged    the shared pattern with the tiles going through registers instead: global_load_dwordx4 for the next
//             step at the top of a step, ds_write_b128 into the other stage behind the step's fragment reads
// It prints bytes into LDS per second over the chip; the GEMM kernels' own rate is to be read against these.
// A second kernel leaves out the barrier: every wave streams on its own with 8 to 16 loads in flight ("free"), which is
// what the path delivers when nothing synchronises - from L1 (a wave re-reads its own 8 KB), from L2 with the tile rows
// of the shared pattern (8 rows x 128 B per load, 16 KB apart), with the same panels packed tile by tile (each load
// 1 KB contiguous, a 32 KB tile one run: what a pre-packed operand layout would give), with rows of 256 B (4 per
// load), and into registers instead of LDS.
// A third kernel ("deep") is the first with smaller steps and more stages: NL x 8 KB per step, NST - 1 steps in flight,
// with and without fragment reads - whether keeping more steps in flight lifts the rate of a step that also reads.
//
//   hipcc --offload-arch=gfx950 -O3 -w -Xclang -target-feature -Xclang -packed-fp32-ops \
//         -o /tmp/lds_load_ceiling sparse-dropout_amd/benchmark/lds_load_ceiling.hip && /tmp/lds_load_ceiling
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef __attribute__((address_space(3))) void lds_void;
constexpr int STAGE = 65536, THREADS = 512, LOADS = 8;  // per wave and step: 8 loads of 1 KB

__device__ inline void load16_to_lds(const char* base, uint32_t lane_off, uint32_t lds_dst) {
  const uint64_t b = (uint64_t)(uintptr_t)base;
  const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t a = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sb), "s"(a)
               : "memory");
}

// mode 0: private contiguous; 1: private tile rows; 2: shared panels of an XCD patch
// reads: 1 KB ds_read_b128 per wave and step from the stage that has landed (the GEMM kernels read 24: 16 KB of X
// fragments and 8 KB of W fragments per wave)
// NL: loads per wave and step (8 = the dense step's 64 KB; 6 = the 48 KB of a step at p = 0.5: the W tile and two of
// the four X tiles)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int NL>
__global__ __launch_bounds__(THREADS) void stream(const char* src, size_t region, int steps, int mode, int reads,
                                                  int positions, int* sink) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t smem_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_void*)smem);
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int wg = blockIdx.x;
  const size_t ROW = 16384;  // bytes between tile rows
  // per-lane offset inside a 1 KB load: 8 rows x 128 B for the row patterns, 1 KB contiguous otherwise
  const uint32_t lane_off = mode == 0 ? lane * 16 : (uint32_t)((lane / 8) * ROW + (lane % 8) * 16);
  // panels of the shared pattern: workgroup (r, c) of the XCD's 8 x 4 patch reads row panel r and column panel c
  const int xcd = wg % 8, slot = wg / 8;  // consecutive workgroups go to consecutive XCDs
  const int pr = slot % 8, pc = slot / 8 % 4;
  auto issue = [&](int step, int stage) {
    const uint32_t st = smem_a + stage * STAGE + wave * (LOADS * 1024);
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const char* p;
      if (mode == 0) {
        p = src + (size_t)wg * region + ((size_t)step * STAGE + (wave * LOADS + i) * 1024) % region;
      } else if (mode == 1) {
        // 64 loads of 8 rows = 512 rows of this workgroup's own 512-row band; a step moves 128 bytes along the rows
        p = src + (size_t)wg * 512 * ROW + (size_t)(wave * LOADS + i) * 8 * ROW + (size_t)(step % positions) * 128;
      } else {
        // loads 0-31: 256 rows of row panel pr; loads 32-63: 256 rows of column panel pc (panels of 256 rows)
        const int l = wave * LOADS + i;
        const int panel = l < 32 ? pr : 8 + pc;
        p = src + ((size_t)xcd * 12 + panel) * 256 * ROW + (size_t)(l % 32) * 8 * ROW + (size_t)(step % positions) * 128;
      }
      load16_to_lds(p, lane_off, st + i * 1024);
    }
  };
  u32x4 x = {0, 0, 0, 0};
  if (mode == 3) {  // through registers
    u32x4 regs[NL];
    auto fetch = [&](int step) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int l = wave * LOADS + i;
        const int panel = l < 32 ? pr : 8 + pc;
        const char* p = src + ((size_t)xcd * 12 + panel) * 256 * ROW + (size_t)(l % 32) * 8 * ROW +
                        (size_t)(step % positions) * 128 + (size_t)((lane / 8) * ROW + (lane % 8) * 16);
        regs[i] = *reinterpret_cast<const u32x4*>(p);
      }
    };
    auto put = [&](int stage) {
#pragma unroll
      for (int i = 0; i < NL; ++i)
        *reinterpret_cast<u32x4*>(smem + stage * STAGE + (wave * LOADS + i) * 1024 + lane * 16) = regs[i];
    };
    fetch(0);
    put(0);
    __syncthreads();
    for (int step = 0; step < steps; ++step) {
      if (step + 1 < steps) fetch(step + 1);
      const char* st = smem + (step & 1) * STAGE + lane * 16;
      for (int i = 0; i < reads; ++i) x ^= *reinterpret_cast<const u32x4*>(st + ((wave * 24 + i) % 64) * 1024);
      if (step + 1 < steps) put((step + 1) & 1);
      __syncthreads();
    }
    if ((x.x ^ x.y ^ x.z ^ x.w) == 0x12345678u) sink[wg] = 1;
    return;
  }
  issue(0, 0);
  for (int step = 0; step < steps; ++step) {
    if (step + 1 < steps) {
      issue(step + 1, (step + 1) & 1);
      // the loads of this step have landed, the next NL fly
      if (NL == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    const char* st = smem + (step & 1) * STAGE + lane * 16;
    for (int i = 0; i < reads; ++i) x ^= *reinterpret_cast<const u32x4*>(st + ((wave * 24 + i) % 64) * 1024);
  }
  if ((x.x ^ x.y ^ x.z ^ x.w) == 0x12345678u) sink[wg] = 1;
  if (threadIdx.x == 0) sink[wg] = *reinterpret_cast<int*>(smem + (steps & 1) * 4);
}

// pattern 0: the wave's own 8 KB again and again (L1); 1: tile rows of the shared panels; 2: the panels packed tile by
// tile; 3: rows of 256 B.  Eight loads per iteration, then a wait that leaves the last eight in flight.
template <bool TO_LDS>
__global__ __launch_bounds__(THREADS) void free_run(const char* src, int iters, int pattern, int positions, int* sink) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t smem_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_void*)smem);
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int wg = blockIdx.x;
  const size_t ROW = 16384;
  uint32_t lane_off = lane * 16;
  if (pattern == 1) lane_off = (uint32_t)((lane / 8) * ROW + (lane % 8) * 16);
  if (pattern == 3) lane_off = (uint32_t)((lane / 16) * ROW + (lane % 16) * 16);
  const int xcd = wg % 8, slot = wg / 8;
  const int pr = slot % 8, pc = slot / 8 % 4;
  u32x4 x = {0, 0, 0, 0};
  u32x4 regs[8];
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int l = wave * 8 + i;  // the 64 loads of a 64 KB step
      const int panel = l < 32 ? pr : 8 + pc;
      const size_t pbase = ((size_t)xcd * 12 + panel) * 256 * ROW;
      const char* p;
      if (pattern == 0) p = src + ((size_t)wg * 8 + wave) * 8192 + i * 1024;
      else if (pattern == 1) p = src + pbase + (size_t)(l % 32) * 8 * ROW + (size_t)(it % positions) * 128;
      else if (pattern == 2) p = src + (((size_t)xcd * 12 + panel) * positions + (it % positions)) * 32768 + (size_t)(l % 32) * 1024;
      else p = src + pbase + (size_t)(l % 32) * 8 * ROW + (size_t)((it % positions) / 2) * 256 + (size_t)(it & 1) * 4 * ROW;
      if (TO_LDS) {
        load16_to_lds(p, lane_off, smem_a + (it & 1) * STAGE + l * 1024);
      } else {
        if (it > 0) x ^= regs[i];
        regs[i] = *reinterpret_cast<const u32x4*>(p + lane_off);
      }
    }
    if (TO_LDS) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (!TO_LDS)
    for (int i = 0; i < 8; ++i) x ^= regs[i];
  if ((x.x ^ x.y ^ x.z ^ x.w) == 0x12345678u) sink[wg] = 1;
  if (threadIdx.x == 0) sink[wg] = *reinterpret_cast<int*>(smem + 4);
}

// NL loads of 1 KB per wave and step (shared-panel pattern), NST stages: the loads of step s + NST - 1 go out right behind
// the barrier that publishes step s; `reads` as in the first kernel
template <int NL, int NST>
__global__ __launch_bounds__(THREADS) void deep(const char* src, int steps, int reads, int positions, int* sink) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int DSTAGE = NL * 8 * 1024;
  const uint32_t smem_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_void*)smem);
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int wg = blockIdx.x;
  const size_t ROW = 16384;
  const uint32_t lane_off = (uint32_t)((lane / 8) * ROW + (lane % 8) * 16);
  const int xcd = wg % 8, slot = wg / 8;
  const int pr = slot % 8, pc = slot / 8 % 4;
  auto issue = [&](int step, int stage) {
    const uint32_t st = smem_a + stage * DSTAGE + wave * (NL * 1024);
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int l = wave * 8 + i;
      const int panel = l < 32 ? pr : 8 + pc;
      const char* p = src + ((size_t)xcd * 12 + panel) * 256 * ROW + (size_t)(l % 32) * 8 * ROW + (size_t)(step % positions) * 128;
      load16_to_lds(p, lane_off, st + i * 1024);
    }
  };
  u32x4 x = {0, 0, 0, 0};
  for (int s = 0; s < NST - 1 && s < steps; ++s) issue(s, s);
  for (int step = 0; step < steps; ++step) {
    const int left = steps - 1 - step;
    const int ahead = left < NST - 2 ? left : NST - 2;  // younger steps that may still be in flight
    static_assert(NL == 4 || NL == 6, "the waits below");
    if (ahead == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (ahead == 1) { if (NL == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); }
    else if (ahead == 2) { if (NL == 6) asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); }
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    __syncthreads();
    if (step + NST - 1 < steps) issue(step + NST - 1, (step + NST - 1) % NST);
    const char* st = smem + (step % NST) * DSTAGE + lane * 16;
    for (int i = 0; i < reads; ++i) x ^= *reinterpret_cast<const u32x4*>(st + ((wave * 5 + i) % (NL * 8)) * 1024);
  }
  if ((x.x ^ x.y ^ x.z ^ x.w) == 0x12345678u) sink[wg] = 1;
  if (threadIdx.x == 0) sink[wg] = *reinterpret_cast<int*>(smem + 4);
}
template <int NL, int NST>
int run_deep(const char* d, int reads, int* sink) {
  constexpr int SMEM = NL * 8 * 1024 * NST;
  static_assert(SMEM <= 160 * 1024, "LDS of a CU");
  hipFuncSetAttribute((const void*)deep<NL, NST>, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
  const int wgs = 256, steps = 2048;
  for (int rep = 0; rep < 2; ++rep) {
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    deep<NL, NST><<<wgs, THREADS, SMEM>>>(d, 64, reads, 128, sink);
    hipDeviceSynchronize();
    hipEventRecord(e0);
    deep<NL, NST><<<wgs, THREADS, SMEM>>>(d, steps, reads, 128, sink);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    if (hipGetLastError() != hipSuccess) { printf("launch failed\n"); return 1; }
    const double tb = (double)wgs * steps * (NL * 8 * 1024) / (ms * 1e-3) / 1e12;
    printf("deep: %d KB step, %d in flight, %2d KB reads / wave  %8.3f ms  %6.2f TB/s into LDS  (%.0f clocks per step at 2.4 GHz)\n",
           NL * 8, NST - 1, reads, ms, tb, ms * 1e-3 / steps * 2.4e9);
  }
  return 0;
}

int main() {
  const int wgs = 256, steps = 2048;
  const size_t bytes = (size_t)8 << 30;
  char* d;
  if (hipMalloc(&d, bytes) != hipSuccess) { printf("hipMalloc failed\n"); return 1; }
  hipMemset(d, 1, bytes);
  int* sink; hipMalloc(&sink, wgs * 4);
  hipFuncSetAttribute((const void*)stream<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE);
  hipFuncSetAttribute((const void*)stream<6>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE);
  struct { const char* name; int mode; size_t region; int reads; int positions; int nl = 8; } cases[] = {
      {"private, 64 KB regions (L2)", 0, (size_t)64 << 10, 0, 128},
      {"private, 512 KB regions", 0, (size_t)512 << 10, 0, 128},
      {"hbm: private, 16 MB regions", 0, (size_t)16 << 20, 0, 128},
      {"rows: private tile rows", 1, 0, 0, 128},
      {"shared, 192 MB of panels", 2, 0, 0, 64},
      {"shared, 192 MB + 24 KB LDS reads / wave", 2, 0, 24, 64},
      {"shared, 384 MB of panels", 2, 0, 0, 128},
      {"shared, 384 MB + 24 KB LDS reads / wave", 2, 0, 24, 128},
      {"p=.5 step: 48 KB loads + 14 KB reads / wave", 2, 0, 14, 128, 6},
      {"staged, 384 MB of panels", 3, 0, 0, 128},
      {"staged, 384 MB + 24 KB LDS reads / wave", 3, 0, 24, 128},
      {"staged, p=.5 step: 48 KB + 14 KB reads / wave", 3, 0, 14, 128, 6},
      // the fragment volume of four waves of 128 x 128 (32 KB each) spread over this kernel's eight
      {"shared, 384 MB + 16 KB LDS reads / wave", 2, 0, 16, 128},
      {"p=.5 step: 48 KB loads + 10 KB reads / wave", 2, 0, 10, 128, 6},
  };
  for (auto& c : cases) {
    for (int rep = 0; rep < 2; ++rep) {
      hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
      auto launch = [&](int n) {
        if (c.nl == 8) stream<8><<<wgs, THREADS, 2 * STAGE>>>(d, c.region, n, c.mode, c.reads, c.positions, sink);
        else stream<6><<<wgs, THREADS, 2 * STAGE>>>(d, c.region, n, c.mode, c.reads, c.positions, sink);
      };
      launch(64);
      hipDeviceSynchronize();
      hipEventRecord(e0);
      launch(steps);
      hipEventRecord(e1); hipEventSynchronize(e1);
      float ms; hipEventElapsedTime(&ms, e0, e1);
      if (hipGetLastError() != hipSuccess) { printf("launch failed\n"); return 1; }
      const double tb = (double)wgs * steps * (c.nl * THREADS / 64 * 1024) / (ms * 1e-3) / 1e12;
      printf("%-40s %8.3f ms  %6.2f TB/s into LDS  (%.1f B/clk/CU at 2.4 GHz)\n", c.name, ms, tb, tb * 1e12 / 256 / 2.4e9);
    }
  }
  if (run_deep<6, 2>(d, 0, sink) || run_deep<6, 2>(d, 14, sink) || run_deep<6, 3>(d, 0, sink) || run_deep<6, 3>(d, 14, sink) ||
      run_deep<4, 2>(d, 0, sink) || run_deep<4, 2>(d, 12, sink) || run_deep<4, 3>(d, 0, sink) || run_deep<4, 3>(d, 12, sink) ||
      run_deep<4, 5>(d, 0, sink) || run_deep<4, 5>(d, 12, sink))
    return 1;
  hipFuncSetAttribute((const void*)free_run<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE);
  hipFuncSetAttribute((const void*)free_run<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * STAGE);
  struct { const char* name; int pattern; bool to_lds; } free_cases[] = {
      {"free: own 8 KB per wave (L1)", 0, true},
      {"free: own 8 KB per wave (L1) -> registers", 0, false},
      {"free: shared panels, 8 rows x 128 B per load", 1, true},
      {"free: shared panels, 8 x 128 B -> registers", 1, false},
      {"free: shared panels packed, 1 KB per load", 2, true},
      {"free: shared panels, 4 rows x 256 B per load", 3, true},
  };
  for (auto& c : free_cases) {
    for (int rep = 0; rep < 2; ++rep) {
      hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
      auto launch = [&](int n) {
        if (c.to_lds) free_run<true><<<wgs, THREADS, 2 * STAGE>>>(d, n, c.pattern, 64, sink);
        else free_run<false><<<wgs, THREADS, 2 * STAGE>>>(d, n, c.pattern, 64, sink);
      };
      launch(64);
      hipDeviceSynchronize();
      hipEventRecord(e0);
      launch(steps);
      hipEventRecord(e1); hipEventSynchronize(e1);
      float ms; hipEventElapsedTime(&ms, e0, e1);
      if (hipGetLastError() != hipSuccess) { printf("launch failed\n"); return 1; }
      const double tb = (double)wgs * steps * STAGE / (ms * 1e-3) / 1e12;
      printf("%-48s %8.3f ms  %6.2f TB/s          (%.1f B/clk/CU at 2.4 GHz)\n", c.name, ms, tb, tb * 1e12 / 256 / 2.4e9);
    }
  }
  return 0;
}
