// Shape-generic MFMA GEMM for the three SparseDrop products (dense, DSD, SDD).
//
// Handles everything the specialised kernels do not: any M, N, K (edge tiles predicated), any
// row-/column-major combination of A, B and C, any block size that is a multiple of 64.
// Workgroup = 256 threads = 4 waves in a 2x2 grid, tile 64 (M) x 128 (N) x 32 (K); each wave owns
// 32x64 of the output as two 32x32 fp32 accumulators fed by v_mfma_f32_32x32x16_{f16,bf16}.
// Operand tiles are staged in LDS as [row][k] whatever the global layout is (operands whose
// reduction index is strided are transposed on the way in), and the next tile's global loads are
// issued into registers before the current tile's MFMAs so their latency overlaps the math.
//
//   DSD (matmul_dsd.cuh:47-66 in the reference): the K loop walks the CSR list of the row block the
//        tile lies in, so dropped blocks cost neither loads nor MFMAs.
//   SDD (matmul_sdd.cuh:44-65): a wave whose 32x64 piece lies in a dropped output block skips its
//        MFMAs and stores zeros; a workgroup with nothing kept skips the K loop altogether.
//   Split-K: when the output has too few tiles to fill the chip and the reduction is long (the weight
//        gradient of a tall activation matrix: dW[N,K] summed over M = 131072 rows for the conv
//        configuration), blockIdx.y splits the reduction (for DSD: the row block's kept list); partial
//        tiles go to an fp32 workspace and a second kernel sums, scales, rounds once and stores.
#include "common.h"

namespace sd {
namespace {

constexpr int BM = 64, BN = 128, BK = 32;
constexpr int LDS_LD = BK + 8;  // halfs per LDS row: 80 B keeps 16-byte alignment and staggers banks
constexpr int THREADS = 256;

// One 8-element piece of an operand tile, held in registers between the global load and the LDS store.
struct Chunk {
  u32x4 v;
};

// Loads tile rows [r0, r0+ROWS) x k [k0, k0+BK) of `m` (rows limited to `rmax`, k to `kmax`) into
// registers.  kcontig: 8 consecutive k per chunk; otherwise 8 consecutive rows per chunk.
template <int ROWS>
__device__ inline void load_tile(const Mat& m, bool kcontig, bool vec_ok, int64_t r0, int64_t rmax,
                                 int64_t k0, int64_t kmax, Chunk (&regs)[ROWS * BK / 8 / THREADS]) {
  constexpr int NCH = ROWS * BK / 8 / THREADS;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = t + i * THREADS;
    int64_t r, k;
    int64_t step;  // element stride between the 8 items of the chunk
    int64_t lim;   // how many of the 8 are inside the matrix
    if (kcontig) {
      r = r0 + c / (BK / 8);
      k = k0 + (c % (BK / 8)) * 8;
      step = m.sc;
      lim = (r < rmax) ? (kmax - k) : 0;
    } else {
      k = k0 + c / (ROWS / 8);
      r = r0 + (c % (ROWS / 8)) * 8;
      step = m.sr;
      lim = (k < kmax) ? (rmax - r) : 0;
    }
    const uint16_t* p = m.ptr + r * m.sr + k * m.sc;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (lim >= 8 && vec_ok) {
      v = *reinterpret_cast<const u32x4*>(p);
    } else if (lim > 0) {
      uint16_t e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = (j < lim) ? p[j * step] : (uint16_t)0;
      v.x = e[0] | ((uint32_t)e[1] << 16);
      v.y = e[2] | ((uint32_t)e[3] << 16);
      v.z = e[4] | ((uint32_t)e[5] << 16);
      v.w = e[6] | ((uint32_t)e[7] << 16);
    }
    regs[i].v = v;
  }
}

template <int ROWS>
__device__ inline void store_tile(uint16_t* lds, bool kcontig,
                                  const Chunk (&regs)[ROWS * BK / 8 / THREADS]) {
  constexpr int NCH = ROWS * BK / 8 / THREADS;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = t + i * THREADS;
    if (kcontig) {
      const int r = c / (BK / 8), k = (c % (BK / 8)) * 8;
      *reinterpret_cast<u32x4*>(lds + r * LDS_LD + k) = regs[i].v;
    } else {
      const int k = c / (ROWS / 8), r = (c % (ROWS / 8)) * 8;
      const u32x4 v = regs[i].v;
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 8; ++j)
        lds[(r + j) * LDS_LD + k] = (uint16_t)(w[j / 2] >> ((j & 1) * 16));
    }
  }
}

// Walks the k offsets (multiples of BK) a tile has to visit.
struct KWalk {
  // dense / SDD: [0, K);  DSD: kept blocks of one row of the list
  const int32_t* idx;
  int32_t pos, end;
  int64_t bs, K;
  int64_t k, kend;
  bool listed;
  uint32_t quads;  // keep bits of the four 32 x 32 quadrants of the block being walked (0xf unless listed so)
  int half;        // which 32-wide half of that block the last next() returned
  // split s of S takes an equal share of the BK-steps (dense) or of the list entries (listed)
  __device__ inline void init_dense(int64_t K_, int s, int S) {
    listed = false;
    quads = 0xfu;
    half = 0;
    K = K_;
    const int64_t steps = (K_ + BK - 1) / BK;
    k = steps * s / S * BK;
    kend = steps * (s + 1) / S * BK;
    if (kend > K_) kend = K_;
  }
  __device__ inline void init_list(const int32_t* col_idx, int32_t beg, int32_t end_, int64_t bs_,
                                   int64_t K_, int s, int S) {
    listed = true;
    idx = col_idx;
    const int64_t len = end_ - beg;
    pos = beg + (int32_t)(len * s / S);
    end = beg + (int32_t)(len * (s + 1) / S);
    bs = bs_;
    K = K_;
    k = 0;
    kend = 0;
    quads = 0xfu;
    half = 0;
  }
  // next k offset or -1
  __device__ inline int64_t next() {
    if (k >= kend) {
      if (!listed || pos >= end) return -1;
      const int32_t e = idx[pos++];
      const int64_t blk = entry_block(e);
      quads = entry_quads(e);
      k = blk * bs;
      kend = k + bs < K ? k + bs : K;
      if (k >= kend) return -1;
    }
    const int64_t r = k;
    half = listed ? (int)(((k % bs) / BK) & 1) : 0;  // BK = 32: the half of a 64-block (only read for such lists)
    k += BK;
    return r;
  }
};

// quadrant keep bits of block `want` if it occurs in the ascending list idx[beg, end) (0xf for a list without
// such bits), else 0
__device__ inline uint32_t list_lookup(const int32_t* idx, int32_t beg, int32_t end, int32_t want) {
  while (beg < end) {
    const int32_t mid = (beg + end) >> 1;
    const int32_t v = entry_block(idx[mid]);
    if (v == want) return entry_quads(idx[mid]);
    if (v < want) beg = mid + 1; else end = mid;
  }
  return 0u;
}

template <typename T, int MODE, bool TRANS_OUT, bool SPLIT>
__global__ __launch_bounds__(THREADS) void gemm_generic_kernel(GemmArgs g, int tiles_n, bool a_kc,
                                                               bool b_kc, bool a_vec, bool b_vec) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[BM * LDS_LD];
  __shared__ __attribute__((aligned(16))) uint16_t sB[BN * LDS_LD];

  const int tile_m = blockIdx.x / tiles_n;
  const int tile_n = blockIdx.x % tiles_n;
  const int64_t m0 = (int64_t)tile_m * BM;
  const int64_t n0 = (int64_t)tile_n * BN;
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int wm = wave / 2, wn = wave % 2;  // wave's 32x64 piece

  KWalk walk;
  uint32_t sdd_quads = 0x3u;  // SDD: which 32-column halves of the wave's piece are kept
  bool wave_kept = true;
  bool any_kept = true;
  if (MODE == kDsd) {
    const int64_t rb = m0 / g.bs;
    walk.init_list(g.col_idx, g.row_ptr[rb], g.row_ptr[rb + 1], g.bs, g.K, SPLIT ? blockIdx.y : 0,
                   SPLIT ? gridDim.y : 1);
  } else {
    walk.init_dense(g.K, SPLIT ? blockIdx.y : 0, SPLIT ? gridDim.y : 1);
    if (MODE == kSdd) {
      const int64_t rb = m0 / g.bs;
      const int32_t beg = g.row_ptr[rb], end = g.row_ptr[rb + 1];
      const uint32_t q0 = list_lookup(g.col_idx, beg, end, (int32_t)(n0 / g.bs));
      const uint32_t q1 = (n0 + 64 < g.N) ? list_lookup(g.col_idx, beg, end, (int32_t)((n0 + 64) / g.bs)) : 0u;
      // with quadrant bits (block size 32, g.bs == 64 == the wave grid): the wave's 32 x 64 piece is row half wm of
      // one 64-block, its two 32-column halves are quadrants (wm, 0) and (wm, 1)
      sdd_quads = ((wn ? q1 : q0) >> (2 * wm)) & 0x3u;
      if (!g.quads) sdd_quads = (wn ? q1 : q0) ? 0x3u : 0u;
      wave_kept = sdd_quads != 0u;
      any_kept = (q0 | q1) != 0u;
    }
  }

  f32x16 acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  if (any_kept) {
    Chunk ra[BM * BK / 8 / THREADS], rb[BN * BK / 8 / THREADS];
    int64_t k0 = walk.next();
    if (k0 >= 0) {
      load_tile<BM>(g.a, a_kc, a_vec, m0, g.M, k0, g.K, ra);
      load_tile<BN>(g.b, b_kc, b_vec, n0, g.N, k0, g.K, rb);
    }
    while (k0 >= 0) {
      // DSD with quadrant bits: the wave's 32 rows are row half wm of the 64-block, this step its 32-wide half
      const bool step_kept = !(MODE == kDsd && g.quads) || ((walk.quads >> (2 * wm + walk.half)) & 1u);
      store_tile<BM>(sA, a_kc, ra);
      store_tile<BN>(sB, b_kc, rb);
      __syncthreads();
      k0 = walk.next();
      if (k0 >= 0) {
        load_tile<BM>(g.a, a_kc, a_vec, m0, g.M, k0, g.K, ra);
        load_tile<BN>(g.b, b_kc, b_vec, n0, g.N, k0, g.K, rb);
      }
      if (wave_kept && step_kept) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
          const int kk = ks * 16 + (lane / 32) * 8;
          const u32x4 fa =
              *reinterpret_cast<const u32x4*>(sA + (wm * 32 + lane % 32) * LDS_LD + kk);
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const u32x4 fb = *reinterpret_cast<const u32x4*>(
                sB + (wn * 64 + j * 32 + lane % 32) * LDS_LD + kk);
            acc[j] = TRANS_OUT ? T::mfma32(fb, fa, acc[j]) : T::mfma32(fa, fb, acc[j]);
          }
        }
      }
      __syncthreads();
    }
  }

  // epilogue: scale in fp32, round once, predicated store (or the raw fp32 partial tile when the
  // reduction is split).
  // MFMA result layout: register v of lane l is element (row 8*(v/4) + 4*(l/32) + v%4, col l%32)
  // of D = (first operand rows) x (second operand rows).
  if (MODE == kSdd && g.kept_only && !wave_kept) return;  // the caller never reads dropped tiles
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int reg_i = 8 * (v / 4) + 4 * (lane / 32) + (v % 4);
      const int lane_i = lane % 32;
      const int64_t m = m0 + wm * 32 + (TRANS_OUT ? lane_i : reg_i);
      const int64_t n = n0 + wn * 64 + j * 32 + (TRANS_OUT ? reg_i : lane_i);
      if (m < g.M && n < g.N) {
        if (MODE == kSdd && !((sdd_quads >> j) & 1u)) acc[j][v] = 0.f;  // a dropped 32-column quadrant of a kept block
        if (SPLIT) {
          // workspace layout follows C's contiguous index so that lanes stay coalesced
          const int64_t e = TRANS_OUT ? n * g.M + m : m * g.N + n;
          g.ws[(int64_t)blockIdx.y * g.M * g.N + e] = acc[j][v];
        } else {
          store_result<T, MODE == kSdd>(g, m, n, acc[j][v] * g.scale);
        }
      }
    }
  }
}

// C = scale * sum over splits of the fp32 partial tiles.  A workgroup owns 256 consecutive elements of C's
// contiguous order (the workspace is laid out the same way): lane l of every wave takes elements 4l .. 4l+3 as
// one 16-byte load per split, the four waves share out the splits and their partial sums meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs g, int splits, bool trans) {
  __shared__ float part[3][256];
  const int64_t total = g.M * g.N;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int64_t e0 = (int64_t)blockIdx.x * 256 + lane * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (e0 + 3 < total && total % 4 == 0) {
    const float* src = g.ws + e0;
    int s = wave;
#pragma unroll 4
    for (; s < splits; s += 4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(src + (int64_t)s * total);
      acc[0] += v[0];
      acc[1] += v[1];
      acc[2] += v[2];
      acc[3] += v[3];
    }
  } else {
    for (int s = wave; s < splits; s += 4)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (e0 + v < total) acc[v] += g.ws[(int64_t)s * total + e0 + v];
  }
  if (wave > 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) part[wave - 1][lane * 4 + v] = acc[v];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int64_t e = e0 + v;
    if (e >= total) break;
    const float sum = ((acc[v] + part[0][lane * 4 + v]) + part[1][lane * 4 + v]) + part[2][lane * 4 + v];
    const int64_t m = trans ? e % g.M : e / g.N;
    const int64_t n = trans ? e / g.M : e % g.N;
    store_result<T, false>(g, m, n, sum * g.scale);  // only DSD and dense products split their reduction
  }
}

template <typename T, int MODE>
int launch_t(const GemmArgs& g, hipStream_t stream) {
  const int64_t tiles_m = ceil_div(g.M, BM), tiles_n = ceil_div(g.N, BN);
  if (tiles_m * tiles_n > 0x7fffffffLL) return fail(SD_ERR_UNSUPPORTED, "too many output tiles");
  const bool a_kc = g.a.sc == 1, b_kc = g.b.sc == 1;
  // 16-byte loads need an aligned base and a leading dimension that keeps every chunk aligned
  auto vec_ok = [](const Mat& m) {
    const int64_t ld = (m.sc == 1) ? m.sr : m.sc;
    return (reinterpret_cast<uintptr_t>(m.ptr) % 16 == 0) && (ld % 8 == 0);
  };
  const bool a_vec = vec_ok(g.a), b_vec = vec_ok(g.b);
  const bool trans_out = (g.c_sr == 1 && g.c_sc != 1);
  int splits = (MODE == kSdd) ? 1 : generic_splits(g.M, g.N, g.K, g.bs, MODE);
  if (splits > 1 && (g.ws == nullptr || g.ws_bytes < (int64_t)splits * g.M * g.N * 4)) splits = 1;
  dim3 block(THREADS);
  if (splits > 1) {
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)splits);
    if (trans_out)
      hipLaunchKernelGGL((gemm_generic_kernel<T, MODE, true, true>), grid, block, 0, stream, g,
                         (int)tiles_n, a_kc, b_kc, a_vec, b_vec);
    else
      hipLaunchKernelGGL((gemm_generic_kernel<T, MODE, false, true>), grid, block, 0, stream, g,
                         (int)tiles_n, a_kc, b_kc, a_vec, b_vec);
    if (int rc = check_launch("gemm_generic (split)")) return rc;
    return launch_splitk_reduce(g, splits, trans_out, T::id, stream);
  }
  dim3 grid((unsigned)(tiles_m * tiles_n));
  if (trans_out)
    hipLaunchKernelGGL((gemm_generic_kernel<T, MODE, true, false>), grid, block, 0, stream, g,
                       (int)tiles_n, a_kc, b_kc, a_vec, b_vec);
  else
    hipLaunchKernelGGL((gemm_generic_kernel<T, MODE, false, false>), grid, block, 0, stream, g,
                       (int)tiles_n, a_kc, b_kc, a_vec, b_vec);
  note_kernel("generic");
  return check_launch("gemm_generic");
}

template <typename T>
int launch_mode(const GemmArgs& g, int mode, hipStream_t stream) {
  switch (mode) {
    case kDense: return launch_t<T, kDense>(g, stream);
    case kDsd: return launch_t<T, kDsd>(g, stream);
    case kSdd: return launch_t<T, kSdd>(g, stream);
  }
  return fail(SD_ERR_INVALID, "bad mode %d", mode);
}

}  // namespace

int launch_splitk_reduce(const GemmArgs& g, int splits, bool trans_out, int dtype, hipStream_t stream) {
  const dim3 grid((unsigned)ceil_div(g.M * g.N, 256));
  if (dtype == SD_BF16)
    hipLaunchKernelGGL(splitk_reduce_kernel<BF16>, grid, dim3(256), 0, stream, g, splits, trans_out);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<F16>, grid, dim3(256), 0, stream, g, splits, trans_out);
  return check_launch("splitk_reduce");
}

// Split the reduction when the output tiles alone cannot fill the 256 CUs and each tile has a long
// reduction: aim for about two workgroups per CU, keep at least 8 K-steps (two 64-blocks) per split.
int generic_splits(int64_t M, int64_t N, int64_t K, int64_t bs, int mode) {
  if (mode == kSdd || M <= 0 || N <= 0) return 1;
  const int64_t tiles = ceil_div(M, BM) * ceil_div(N, BN);
  if (tiles >= 192 || K < 2048) return 1;
  const int64_t units = (mode == kDsd && bs > 0) ? ceil_div(K, bs) : ceil_div(K, 64);
  int64_t want = ceil_div(512, tiles);
  if (want > units / 2) want = units / 2;
  if (want > 128) want = 128;
  // the product must stay a sane workspace: 256 MiB at most
  while (want > 1 && want * M * N * 4 > (256LL << 20)) --want;
  return want < 2 ? 1 : (int)want;
}

int launch_generic(const GemmArgs& g, int mode, int dtype, hipStream_t stream) {
  if (g.M == 0 || g.N == 0) return SD_OK;
  return dtype == SD_BF16 ? launch_mode<BF16>(g, mode, stream) : launch_mode<F16>(g, mode, stream);
}

}  // namespace sd
