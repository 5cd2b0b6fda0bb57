// Specialised gfx950 kernels for 64x64 mask blocks and tile-aligned shapes.
//
// ---- DSD, both operands reduction-contiguous (the forward Y = s*(keep.X).W^T, and dense) -------
// A workgroup owns 4 consecutive row blocks of X (256 rows) x 256 columns of Y.  Row blocks keep
// different K blocks, so the workgroup walks the UNION of their kept lists: per step it brings in
// one 256x64 tile of W (shared by everybody) and the 64x64 X tiles of just the row blocks that keep
// this K block, and issues MFMAs only for those.  The 8 waves are (column slice ns = wave%4) x
// (row-block pair rh = wave/4): a wave multiplies its 64-column slice of the W tile (held in
// registers for the step) with each kept X tile of its pair.  Waves w and w+4 land on the same SIMD,
// so every SIMD sees exactly (#kept row blocks) x 64x64x64 of MFMA work per step whatever the mask
// looks like: dropped blocks cost neither loads nor MFMAs and no wave idles behind a barrier.
//
// Global->LDS goes through global_load_lds_dwordx4 (no VGPR staging), two stages, one barrier per
// step.  A tile row is 128 B (64 halfs) and its 16-byte chunks are XOR-swizzled with (row>>1)&7,
// which makes the MFMA fragment reads (ds_read_b128, 32 rows x one chunk per half-wave) hit all
// 64 LDS banks; the swizzle is applied on the global side (which chunk a lane fetches), because the
// LDS side of a direct load is fixed at lane*16.
#include "common.h"

namespace sd {
namespace {

constexpr int R = 4;          // row blocks per workgroup
constexpr int BS = 64;        // mask block = tile edge along M and K
constexpr int BN = 256;       // output columns per workgroup
constexpr int THREADS = 512;  // 8 waves
constexpr int TILE = BS * BS * 2;              // bytes of one 64 x 64 tile (rows of 128 B)
constexpr int STAGE = (BN / BS) * TILE + R * TILE;  // W tile (32 KB) + up to 4 X tiles (32 KB)
constexpr int A_OFF = (BN / BS) * TILE;
constexpr int MAX_STEPS = 1024;
constexpr int SMEM_STEPS = 2 * STAGE;                  // uint16 kb[MAX_STEPS]
constexpr int SMEM_FLAGS = SMEM_STEPS + 2 * MAX_STEPS;  // uint8 flags[MAX_STEPS]
constexpr int SMEM_SCRATCH = SMEM_FLAGS + MAX_STEPS;    // uint32 per K block while merging
constexpr int SMEM_BYTES = SMEM_SCRATCH + 4 * MAX_STEPS + 16;

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;

// one wave-wide 1 KB direct load: lane i's 16 bytes land at lds_dst + 16*i
__device__ inline void load16_to_lds(const void* g, char* lds_dst) {
  __builtin_amdgcn_global_load_lds((glb_void*)g, (lds_void*)lds_dst, 16, 0, 0);
}

// Maps the launch index to an output tile so that the workgroups resident on one XCD (the hardware
// deals consecutive workgroup ids round-robin over the 8 XCDs, each with its own L2) cover a compact
// patch of the tile grid: each XCD gets a contiguous run of the tile order, and the order walks
// GROUP_M tile rows at a time (column by column inside a group).
__device__ inline void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8, GROUP_M = 4;
  const int total = tiles_m * tiles_n;
  const int per = total / XCDS, rem = total % XCDS;
  const int x = bid % XCDS, i = bid / XCDS;
  const int lin = x * per + (x < rem ? x : rem) + i;
  const int group = lin / (GROUP_M * tiles_n);
  const int first_m = group * GROUP_M;
  const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = lin - group * GROUP_M * tiles_n;
  tm = first_m + in_group % gm;
  tn = in_group / gm;
}

template <typename T>
__global__ __launch_bounds__(THREADS) void dsd_nt_kernel(GemmArgs g, int tiles_m, int tiles_n,
                                                         int Mb, int Kb) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  uint16_t* step_kb = reinterpret_cast<uint16_t*>(smem + SMEM_STEPS);
  uint8_t* step_fl = reinterpret_cast<uint8_t*>(smem + SMEM_FLAGS);
  uint32_t* scratch = reinterpret_cast<uint32_t*>(smem + SMEM_SCRATCH);
  int* nsteps_p = reinterpret_cast<int*>(smem + SMEM_SCRATCH + 4 * MAX_STEPS);

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int ns = wave % 4;  // 64-column slice
  const int rh = wave / 4;  // row-block pair
  const int rb0 = tm * R;   // first row block
  const int64_t n0 = (int64_t)tn * BN;

  // ---- union of the kept lists of the 4 row blocks: (K block, 4-bit keep flags) per step -------
  for (int i = tid; i < Kb; i += THREADS) scratch[i] = 0;
  __syncthreads();
  if (g.row_ptr) {
    for (int r = 0; r < R; ++r) {
      if (rb0 + r >= Mb) break;
      const int beg = g.row_ptr[rb0 + r], end = g.row_ptr[rb0 + r + 1];
      for (int i = beg + tid; i < end; i += THREADS) atomicOr(&scratch[g.col_idx[i]], 1u << r);
    }
  } else {
    const uint32_t all = (rb0 + R <= Mb) ? 0xfu : ((1u << (Mb - rb0)) - 1u);
    for (int i = tid; i < Kb; i += THREADS) scratch[i] = all;
  }
  __syncthreads();
  if (wave == 0) {
    int base = 0;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int k0 = 0; k0 < Kb; k0 += 64) {
      const int k = k0 + lane;
      const uint32_t f = (k < Kb) ? scratch[k] : 0u;
      const uint64_t bal = __ballot(f != 0);
      if (f) {
        const int pos = base + __popcll(bal & lt);
        step_kb[pos] = (uint16_t)k;
        step_fl[pos] = (uint8_t)f;
      }
      base += __popcll(bal);
    }
    if (lane == 0) *nsteps_p = base;
  }
  __syncthreads();
  const int nsteps = *nsteps_p;

  // ---- per-lane constants ---------------------------------------------------------------------
  // loads: a wave-wide load covers 8 tile rows; lane -> (row lane/8, physical chunk lane%8)
  const int ld_row = lane / 8;
  const int ld_pch = lane % 8;
  // fragment reads: lane -> tile row lane%32 (+32*tile), logical chunk 2*ks + lane/32
  const int fr_row = lane % 32;
  const int fr_sw = (lane >> 1) & 7;
  int koff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) koff[ks] = ((2 * ks + lane / 32) ^ fr_sw) * 16;

  const uint16_t* a_base = g.a.ptr + (int64_t)rb0 * BS * g.a.sr;
  const uint16_t* b_base = g.b.ptr + n0 * g.b.sr;

  auto issue_loads = [&](int step, int stage) {
    const int kb = step_kb[step];
    const uint32_t fl = step_fl[step];
    char* st = smem + stage * STAGE;
    // W tile: 32 row-octets, 4 per wave
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int oct = wave * 4 + j;
      const int row = oct * 8 + ld_row;
      const int ch = ld_pch ^ ((row >> 1) & 7);
      load16_to_lds(b_base + (int64_t)row * g.b.sr + kb * BS + ch * 8, st + oct * 1024);
    }
    // X tiles of the row blocks that keep this K block: 8 row-octets each, one per wave
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (fl & (1u << r)) {
        const int row = wave * 8 + ld_row;
        const int ch = ld_pch ^ ((row >> 1) & 7);
        load16_to_lds(a_base + (int64_t)(r * BS + row) * g.a.sr + kb * BS + ch * 8,
                      st + A_OFF + r * TILE + wave * 1024);
      }
    }
  };

  f32x16 acc[2][2][2];  // [row block of the pair][m tile][n tile]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][b][c][v] = 0.f;

  if (nsteps > 0) issue_loads(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int step = 0; step < nsteps; ++step) {
    const int stage = step & 1;
    if (step + 1 < nsteps) issue_loads(step + 1, stage ^ 1);
    const uint32_t mine = (step_fl[step] >> (2 * rh)) & 3u;
    if (mine) {
      const char* st = smem + stage * STAGE;
      u32x4 bf[2][4];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
          bf[nt][ks] = *reinterpret_cast<const u32x4*>(st + (ns * 64 + nt * 32 + fr_row) * 128 + koff[ks]);
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        if (mine & (1u << rr)) {
          const char* at = st + A_OFF + (2 * rh + rr) * TILE;
          u32x4 af[2][4];
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
              af[mt][ks] = *reinterpret_cast<const u32x4*>(at + (mt * 32 + fr_row) * 128 + koff[ks]);
#pragma unroll
          for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
              for (int nt = 0; nt < 2; ++nt)
                acc[rr][mt][nt] = T::mfma32(af[mt][ks], bf[nt][ks], acc[rr][mt][nt]);
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  // ---- epilogue: scale, round once, store (row-major C) -----------------------------------------
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int rb = rb0 + 2 * rh + rr;
    if (rb >= Mb) continue;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = mt * 32 + 8 * (v / 4) + 4 * (lane / 32) + (v % 4);
          const int64_t m = (int64_t)rb * BS + row;
          const int64_t n = n0 + ns * 64 + nt * 32 + (lane % 32);
          g.c[m * g.c_sr + n] = T::from_float(acc[rr][mt][nt][v] * g.scale);
        }
  }
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

template <typename T>
int launch_dsd_nt(const GemmArgs& g, hipStream_t stream) {
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dsd_nt_kernel<T>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
    if (e != hipSuccess) return fail(SD_ERR_RUNTIME, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    configured = true;
  }
  const int Mb = (int)(g.M / BS), Kb = (int)(g.K / BS);
  const int tiles_m = (Mb + R - 1) / R, tiles_n = (int)(g.N / BN);
  hipLaunchKernelGGL(dsd_nt_kernel<T>, dim3((unsigned)(tiles_m * tiles_n)), dim3(THREADS), SMEM_BYTES,
                     stream, g, tiles_m, tiles_n, Mb, Kb);
  return check_launch("dsd_nt_kernel");
}

}  // namespace

int launch_fast(const GemmArgs& g, int mode, int dtype, hipStream_t stream) {
  if (mode == kSdd) return SD_ERR_UNSUPPORTED;
  if (mode == kDsd && g.bs != BS) return SD_ERR_UNSUPPORTED;
  // both operands reduction-contiguous, C row-major, everything tile-aligned and 16-byte aligned
  const bool layout_ok = g.a.sc == 1 && g.b.sc == 1 && g.c_sc == 1;
  const bool shape_ok = g.M > 0 && g.M % BS == 0 && g.N > 0 && g.N % BN == 0 && g.K > 0 &&
                        g.K % BS == 0 && g.K / BS <= MAX_STEPS;
  const bool align_ok = aligned16(g.a.ptr) && aligned16(g.b.ptr) && g.a.sr % 8 == 0 && g.b.sr % 8 == 0;
  const int64_t tiles = ((g.M / BS + R - 1) / R) * (g.N / BN);
  if (!(layout_ok && shape_ok && align_ok) || tiles > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  return dtype == SD_BF16 ? launch_dsd_nt<BF16>(g, stream) : launch_dsd_nt<F16>(g, stream);
}

}  // namespace sd
