// Input gradient of the (block-dropout) convolution in one launch, without the gradient of the patch
// matrix ever reaching memory:
//
//   dx[n, c, h, w] = scale * sum over taps (r, s) of keep[m / 64, k / 64] * (dY . W)[m, k]
//   with m = (n, (h + pad_h - r * dil_h) / stride_h, (w + pad_w - s * dil_w) / stride_w) the output position the
//   tap reads from (taps whose quotients are not whole or fall outside the output contribute nothing), k = (c, r, s)
//
// i.e. the SDD product dY . W restricted to kept 64 x 64 tiles followed by col2im (the adjoint of the
// F.unfold gather of flash_dropout/functional/im2col_conv2d.py:17-20).
//
// A workgroup owns HB = 2 * (64 / Q) * stride_h input rows of one image, all channels.  The output rows whose taps
// reach them lie in at most four consecutive 64-position row blocks of dY; each of the eight waves keeps 32
// rows of them (all of the reduction, K_out <= 256) in registers as MFMA operands for the whole kernel, so
// that (for K_out <= 128) two workgroups fit a CU and one folds while the other multiplies.  Then, for every 64-column block of the patch
// matrix in turn: the W tile of the block arrives by direct loads (double buffered), every wave multiplies
// one 32-row half of one dY tile with it (MFMA, fp32) if the mask keeps that tile and writes the scaled
// result, rounded once as the two-kernel route rounds it, to an LDS staging area; after a barrier each
// thread, owner of a fixed (input row, w) and of a few of the block's channels, adds up the taps of its
// elements that fall in this block from the staging area.  A channel's R*S columns span at most two
// consecutive blocks, so its sums are carried in a small fp32 ring in LDS and written out once, when its last
// column has been seen.  Every sum has one owner and a fixed order: the result is deterministic.
#include <atomic>

#include "common.h"

namespace sd {
namespace {

constexpr int BS = 64;
constexpr int TILE = BS * BS * 2;
constexpr int THREADS = 512;
constexpr int NB = 4;           // row blocks of dY per workgroup
constexpr int KS_LIMIT = 4;     // 64-wide reduction steps at most: K_out <= 256
// A staged tile is kept column by column: [64 columns][64 positions + 4].  A lane's four accumulator registers of
// one group are four consecutive positions of one column, i.e. one 8-byte store (the 136-byte column pitch puts the 32
// columns of a store on all 64 banks once), and the fold's lanes, which run along w, read consecutive halfs.
constexpr int STAGE_LD = 68;
// LDS of an instance for K_out <= 64 * KS_MAX: two W tiles (one per buffer) of KS_MAX * 8 KB, the staging area, the ring
template <int KS_MAX>
struct DxLds {
  static constexpr int OFF_STAGE = 2 * KS_MAX * TILE;
  static constexpr int OFF_ACC = OFF_STAGE + NB * BS * STAGE_LD * 2;
  // K_out <= 128: half a CU's LDS, so that two workgroups share a CU; beyond, all of it (a few bytes are static)
  static constexpr int DYN_LDS_MAX = (KS_MAX <= 2 ? 81920 : 163840) - 256;
  static constexpr int ACC_MAX = DYN_LDS_MAX - OFF_ACC;  // bytes left for the ring of open channel sums
};

typedef __attribute__((address_space(3))) void lds_void;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// wave-wide 1 KB direct global->LDS load (lane i's 16 bytes land at lds_dst + 16*i); issued as assembly so
// that the compiler keeps counting LDS reads precisely, waited for with an explicit vmcnt(0)
__device__ inline void load16_to_lds(const void* g, char* lds_dst) {
  const uint32_t a = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void*)lds_dst);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(a) : "memory");
}
__device__ inline u32x2 lds_read_tr(const char* p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
  return __builtin_bit_cast(u32x2, v);
}

struct DxArgs {
  const uint16_t* dy;  // [N*P*Q, K_out], row-major
  int64_t dy_ld;
  const uint16_t* w;   // [K_out, C*R*S], row-major
  int64_t w_ld;
  uint16_t* dx;        // [N, C, H, W] by element strides
  int64_t sn, sc, sh, sw;
  const uint8_t* mask;  // [N*P*Q/64, ceil(C*R*S/64)] bytes, non-zero = dropped; null = keep everything
  int64_t msr, msc;
  int C, H, W, P, Q, R, S, pad_h, pad_w;
  int sth, stw, dlh, dlw;  // strides and dilations
  int rpb_shift;        // log2(64 / Q): output rows per row block
  int HB, bands;        // input rows per workgroup, workgroups per image
  int blocks_per_img;   // P * Q / 64
  int K, Kb, KS;        // C*R*S, its 64-blocks, K_out / 64
  int ring_n;           // channels whose sums can be open at once: those of one block column plus the carried ones
  float scale;
};

// RT, ST: the kernel size at compile time (the tap loops unroll and the per-tap address terms become per-thread
// constants), or 0, 0 for any size.
template <typename T, int RT, int ST, int KS_MAX>
__global__ __launch_bounds__(THREADS) void conv_dx_kernel(DxArgs g) {
  constexpr int OFF_STAGE = DxLds<KS_MAX>::OFF_STAGE, OFF_ACC = DxLds<KS_MAX>::OFF_ACC;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* wt = smem;
  uint16_t* stage = reinterpret_cast<uint16_t*>(smem + OFF_STAGE);
  float* ring = reinterpret_cast<float*>(smem + OFF_ACC);

  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int img = blockIdx.x / g.bands, band = blockIdx.x - img * g.bands;
  const int h0 = band * g.HB;
  const int RS = RT > 0 ? RT * ST : g.R * g.S;
  const int rpb = 1 << g.rpb_shift;
  // output rows the taps of input rows [h0, h0 + HB) read: p = (h + pad_h - r * dil) / stride where that divides;
  // the first of them is the quotient rounded up (also below zero)
  const int t_lo = h0 + g.pad_h - (g.R - 1) * g.dlh;
  const int p_lo = t_lo >= 0 ? (t_lo + g.sth - 1) / g.sth : -((-t_lo) / g.sth);
  const int pb0 = p_lo >> g.rpb_shift;  // arithmetic shift: floor, also below zero
  const int pbn = g.P >> g.rpb_shift;   // row blocks per image

  // ---- keep flags of the four row blocks: bit j = block column j kept ----------------------------------
  __shared__ uint64_t keep[NB];  // in LDS: indexed by run-time row blocks below
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int pb = pb0 + b;
    const bool valid = pb >= 0 && pb < pbn;
    bool k = valid && lane < g.Kb;
    if (k && g.mask) k = g.mask[((int64_t)img * g.blocks_per_img + pb) * g.msr + lane * g.msc] == 0;
    const uint64_t bits = __ballot(k);
    if (tid == 0) keep[b] = bits;
  }
  __syncthreads();

  // ---- this wave's 32 rows of dY as MFMA fragments (lane: row lane % 32, 8 reduction indices per 16), the
  //      first W tile, the ring ----------------------------------------------------------------------------
  const int t_blk = wave >> 1, half = wave & 1;  // this wave's dY row block and its 32-row half
  const int ld_row = wave * 8 + lane / 8, ld_pch = lane % 8;
  u32x4 af[KS_MAX][4];
#pragma unroll
  for (int ks = 0; ks < KS_MAX; ++ks)
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) af[ks][kk] = u32x4{0u, 0u, 0u, 0u};
  if (keep[t_blk] != 0) {  // inside the image and something kept
    const int64_t m = ((int64_t)img * g.blocks_per_img + pb0 + t_blk) * BS + half * 32 + lane % 32;
    const uint16_t* src = g.dy + m * g.dy_ld + (lane / 32) * 8;
#pragma unroll
    for (int ks = 0; ks < KS_MAX; ++ks)
      if (ks < g.KS) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) af[ks][kk] = *reinterpret_cast<const u32x4*>(src + ks * BS + kk * 16);
      }
  }
  // W tile of block column j, reduction step ks: rows = reduction index, 64 columns = 128 bytes each
  auto load_w = [&](int j, int buf) {
    int chunk = ld_pch ^ (((ld_row >> 1) & 1) << 2);
    if (j * BS + chunk * 8 >= g.K) chunk = 0;  // past the last column: never gathered, only kept readable
    for (int ks = 0; ks < g.KS; ++ks)
      load16_to_lds(g.w + (int64_t)(ks * BS + ld_row) * g.w_ld + j * BS + chunk * 8,
                    wt + (buf * KS_MAX + ks) * TILE + wave * 1024);
  };
  load_w(0, 0);
  const int hw_n = g.HB * g.W;  // elements per channel in the band
  for (int i = tid; i < g.ring_n * hw_n; i += THREADS) ring[i] = 0.f;

  // ---- per-lane fragment offsets (the tile layouts of the GEMM kernels) ----------------------------------
  int b_off[4];
  {
    const int b4 = lane / 16, e = (lane % 16) / 4, j4 = lane % 4;
    const int row = 8 * (b4 / 2) + e;
    const int b_ch = (2 * (b4 % 2) + j4 / 2) ^ (((e >> 1) & 1) << 2);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      b_off[kk] = (16 * kk + row) * 128 + b_ch * 16 + (j4 % 2) * 8;  // ^ 64 for the second 32 columns
    }
  }
  // ---- this thread's fixed (input row, w) and channel phase for the gather ------------------------------
  const int groups = THREADS / hw_n;            // channels handled per pass over the block's channels (>= 1)
  const int cgrp = tid / hw_n;                  // >= groups: idle in the gather
  const int hw = tid - cgrp * hw_n;
  const int hl = hw / g.W, wq = hw - hl * g.W;
  const int h = h0 + hl;

  // known kernel size: per tap row the staged row it reads and the keep word of its row block, per tap column
  // the position inside that row (-1: the tap falls outside the output)
  constexpr int RN = RT > 0 ? RT : 1, SN = ST > 0 ? ST : 1;
  [[maybe_unused]] uint64_t tap_keep[RN];
  [[maybe_unused]] int tap_row[RN], tap_col[SN];
  if constexpr (RT > 0) {
#pragma unroll
    for (int rr = 0; rr < RT; ++rr) {
      const int t = h + g.pad_h - rr * g.dlh;
      const int p = t >= 0 ? t / g.sth : 0;
      const bool ok = t >= 0 && p * g.sth == t && p < g.P && h < g.H;
      const int b = ok ? (p >> g.rpb_shift) - pb0 : 0;
      tap_keep[rr] = ok ? keep[b] : 0ull;
      tap_row[rr] = b * BS * STAGE_LD + (p - (pb0 + b) * rpb) * g.Q;
    }
#pragma unroll
    for (int ss = 0; ss < ST; ++ss) {
      const int u = wq + g.pad_w - ss * g.dlw;
      const int q = u >= 0 ? u / g.stw : 0;
      tap_col[ss] = (u >= 0 && q * g.stw == u && q < g.Q) ? q : -1;
    }
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int j = 0; j < g.Kb; ++j) {
    if (j + 1 < g.Kb) load_w(j + 1, (j + 1) & 1);
    // ---- kept tiles of this block column: MFMA, scale, round, stage ------------------------------------
    if ((keep[t_blk] >> j) & 1ull) {
      f32x16 acc[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS_MAX; ++ks) {
        if (ks >= g.KS) break;
        const char* bt = wt + ((j & 1) * KS_MAX + ks) * TILE;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) {
            const char* p = bt + (b_off[kk] ^ (nt * 64));
            const u32x2 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * 128);
            acc[nt] = T::mfma32(af[ks][kk], u32x4{lo.x, lo.y, hi.x, hi.y}, acc[nt]);
          }
        }
      }
      // accumulator register v of lane l is position 8*(v/4) + 4*(l/32) + v%4 of the wave's 32, column l%32
      uint16_t* st = stage + t_blk * BS * STAGE_LD + half * 32 + 4 * (lane / 32);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const uint32_t lo = (uint32_t)T::from_float(acc[nt][4 * q4] * g.scale) |
                              ((uint32_t)T::from_float(acc[nt][4 * q4 + 1] * g.scale) << 16);
          const uint32_t hi = (uint32_t)T::from_float(acc[nt][4 * q4 + 2] * g.scale) |
                              ((uint32_t)T::from_float(acc[nt][4 * q4 + 3] * g.scale) << 16);
          *reinterpret_cast<u32x2*>(st + (nt * 32 + lane % 32) * STAGE_LD + 8 * q4) = u32x2{lo, hi};
        }
    }
    // the next W tile has had the products to arrive; so have the stores of the previous block's sums
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // ---- the taps of this block column, summed into the owners' ring entries ----------------------------
    {
      const int k_lo = j * BS, k_hi = (k_lo + BS < g.K ? k_lo + BS : g.K) - 1;
      const int c_lo = k_lo / RS, c_hi = k_hi / RS;
      if (cgrp < groups && h < g.H) {
        int slot = (c_lo + cgrp) % g.ring_n;
        for (int c = c_lo + cgrp; c <= c_hi; c += groups) {
          float sum = 0.f;
          int k = c * RS - k_lo;  // column of tap (0, 0) inside the block (may be negative)
          if constexpr (RT > 0) {
#pragma unroll
            for (int rr = 0; rr < RT; ++rr) {
              const bool row_ok = (tap_keep[rr] >> j) & 1ull;
#pragma unroll
              for (int ss = 0; ss < ST; ++ss, ++k)
                if (row_ok && tap_col[ss] >= 0 && (unsigned)k < (unsigned)BS)
                  sum += T::to_float(stage[tap_row[rr] + tap_col[ss] + k * STAGE_LD]);
            }
          } else {
            for (int rr = 0; rr < g.R; ++rr) {
              const int t = h + g.pad_h - rr * g.dlh;
              const int p = t >= 0 ? t / g.sth : 0;
              const int b = (p >> g.rpb_shift) - pb0;
              const bool row_ok = t >= 0 && p * g.sth == t && p < g.P && ((keep[b & (NB - 1)] >> j) & 1ull);
              const uint16_t* srow = stage + (b & (NB - 1)) * BS * STAGE_LD + (p - (pb0 + b) * rpb) * g.Q;
              for (int ss = 0; ss < g.S; ++ss, ++k) {
                const int u = wq + g.pad_w - ss * g.dlw;
                const int q = u >= 0 ? u / g.stw : 0;
                if (row_ok && k >= 0 && k < BS && u >= 0 && q * g.stw == u && q < g.Q)
                  sum += T::to_float(srow[q + k * STAGE_LD]);
              }
            }
          }
          float* r = ring + (slot * hw_n + hw);
          slot += groups;
          if (slot >= g.ring_n) slot -= g.ring_n;
          const float total = *r + sum;
          if (c * RS + RS - 1 <= k_hi) {  // the channel's last column is in this block: done
            g.dx[(int64_t)img * g.sn + (int64_t)c * g.sc + (int64_t)h * g.sh + (int64_t)wq * g.sw] = T::from_float(total);
            *r = 0.f;
          } else {
            *r = total;
          }
        }
      }
    }
    __syncthreads();  // the staging area and this block's W buffer are free again
  }
}

template <typename T, int RT, int ST, int KS_MAX>
int launch_t(const DxArgs& g, int64_t wgs, hipStream_t stream) {
  const int smem = DxLds<KS_MAX>::OFF_ACC + g.ring_n * g.HB * g.W * 4;
  if (smem > DxLds<KS_MAX>::DYN_LDS_MAX) return SD_ERR_UNSUPPORTED;  // the ring of open channel sums does not fit
  static std::atomic<bool> configured[16] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
    return fail(SD_ERR_RUNTIME, "hipGetDevice failed or device index out of range");
  if (!configured[dev].load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_dx_kernel<T, RT, ST, KS_MAX>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, DxLds<KS_MAX>::DYN_LDS_MAX);
    if (e != hipSuccess) return fail(SD_ERR_RUNTIME, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    configured[dev].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL((conv_dx_kernel<T, RT, ST, KS_MAX>), dim3((unsigned)wgs), dim3(THREADS), smem, stream, g);
  note_kernel("conv_dx:fused");
  return check_launch("conv_dx_kernel");
}

}  // namespace

// Returns SD_ERR_UNSUPPORTED (no message, nothing launched) for geometries the kernel does not take.
int launch_conv_dx(const void* dy, int64_t dy_ld, const void* w, int64_t w_ld, void* dx, int64_t sn, int64_t sc,
                   int64_t sh, int64_t sw, const uint8_t* mask, int64_t msr, int64_t msc, int64_t n, int64_t c,
                   int64_t h, int64_t wd, int64_t k_out, int64_t r, int64_t s, int64_t pad_h, int64_t pad_w,
                   int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w, float scale, int dtype,
                   hipStream_t stream) {
  if (stride_h < 1 || stride_w < 1 || dil_h < 1 || dil_w < 1 || stride_h > 8 || stride_w > 8 || dil_h > 8 || dil_w > 8)
    return SD_ERR_UNSUPPORTED;
  const int64_t P = (h + 2 * pad_h - dil_h * (r - 1) - 1) / stride_h + 1;
  const int64_t Q = (wd + 2 * pad_w - dil_w * (s - 1) - 1) / stride_w + 1;
  if (P <= 0 || Q <= 0 || Q > BS || BS % Q != 0 || (P * Q) % BS != 0) return SD_ERR_UNSUPPORTED;
  if (k_out % BS != 0 || k_out > BS * KS_LIMIT) return SD_ERR_UNSUPPORTED;
  const int64_t K = c * r * s, Kb = (K + BS - 1) / BS;
  if (Kb > 64 || K % 8 != 0 || r * s > BS) return SD_ERR_UNSUPPORTED;  // keep flags are one 64-bit word per row block
  const int64_t rpb = BS / Q;
  // a channel's columns span at most two blocks; the ring holds every channel a block column can touch
  const int64_t ring_n = (BS + r * s - 1) / (r * s) + 2;
  const int64_t ring_max = k_out > 2 * BS ? DxLds<4>::ACC_MAX : DxLds<2>::ACC_MAX;
  // a band of HB input rows per workgroup: the input rows under two row blocks of output, fewer if a band's elements
  // of one channel outnumber the threads or the ring of open channel sums would not fit
  // and the output rows one band's taps read must fit the four row blocks the waves hold: at most
  // (HB - 1 + (R - 1) * dil) / stride + 1 of them, the first up to rpb - 1 rows into its block
  auto rows_fit = [&](int64_t hb) { return (rpb - 1) + (hb - 1 + (r - 1) * dil_h) / stride_h + 1 <= NB * rpb; };
  int64_t HB = 2 * rpb * stride_h;
  while (HB > 1 && (HB * wd > THREADS || ring_n * HB * wd * 4 > ring_max || !rows_fit(HB))) HB /= 2;
  if (!rows_fit(HB)) return SD_ERR_UNSUPPORTED;
  const int64_t hw_n = HB * wd;
  if (hw_n > THREADS) return SD_ERR_UNSUPPORTED;
  const bool align_ok = reinterpret_cast<uintptr_t>(dy) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                        dy_ld % 8 == 0 && w_ld % 8 == 0 && dy_ld >= k_out && w_ld >= K;
  if (!align_ok) return SD_ERR_UNSUPPORTED;
  const int64_t bands = (h + HB - 1) / HB;
  const int64_t wgs = n * bands;
  if (wgs > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  DxArgs g;
  g.dy = static_cast<const uint16_t*>(dy);
  g.dy_ld = dy_ld;
  g.w = static_cast<const uint16_t*>(w);
  g.w_ld = w_ld;
  g.dx = static_cast<uint16_t*>(dx);
  g.sn = sn;
  g.sc = sc;
  g.sh = sh;
  g.sw = sw;
  g.mask = mask;
  g.msr = msr;
  g.msc = msc;
  g.C = (int)c;
  g.H = (int)h;
  g.W = (int)wd;
  g.P = (int)P;
  g.Q = (int)Q;
  g.R = (int)r;
  g.S = (int)s;
  g.pad_h = (int)pad_h;
  g.pad_w = (int)pad_w;
  g.sth = (int)stride_h;
  g.stw = (int)stride_w;
  g.dlh = (int)dil_h;
  g.dlw = (int)dil_w;
  g.rpb_shift = 0;
  while ((1 << g.rpb_shift) < rpb) ++g.rpb_shift;
  g.HB = (int)HB;
  g.bands = (int)bands;
  g.blocks_per_img = (int)(P * Q / BS);
  g.K = (int)K;
  g.Kb = (int)Kb;
  g.KS = (int)(k_out / BS);
  g.scale = scale;
  g.ring_n = (int)ring_n;
  const bool bf = dtype == SD_BF16, wide = k_out > 2 * BS;
  if (r == 3 && s == 3) {
    if (wide) return bf ? launch_t<BF16, 3, 3, 4>(g, wgs, stream) : launch_t<F16, 3, 3, 4>(g, wgs, stream);
    return bf ? launch_t<BF16, 3, 3, 2>(g, wgs, stream) : launch_t<F16, 3, 3, 2>(g, wgs, stream);
  }
  if (wide) return bf ? launch_t<BF16, 0, 0, 4>(g, wgs, stream) : launch_t<F16, 0, 0, 4>(g, wgs, stream);
  return bf ? launch_t<BF16, 0, 0, 2>(g, wgs, stream) : launch_t<F16, 0, 0, 2>(g, wgs, stream);
}

}  // namespace sd
