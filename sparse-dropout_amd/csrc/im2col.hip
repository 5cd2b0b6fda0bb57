// im2col gather (and its adjoint) feeding the SparseDrop GEMMs for conv.
//
// cols[(n*P+p)*Q+q, c*R*S + r*S + s] = x[n, c, p*sh + r*dh - ph, q*sw + s*dw - pw]   (0 outside)
// — the F.unfold column order of flash_dropout/functional/im2col_conv2d.py:17-20.
//
// HBM-bound byte shuffling: the patch matrix is R*S times the input, so the kernel is built around
// its writes.  A workgroup owns 64 consecutive rows (n,p,q) and walks 64-column tiles; lanes run along
// q while reading (consecutive pixels of an image row), the 64x64 tile is turned in LDS, and lanes run
// along the column index while writing, so both sides are coalesced.  With a kept-block list only
// kept blocks are produced: dropped blocks are never read by the DSD kernels, so they are not written.
#include "common.h"

namespace sd {
namespace {

struct ConvGeom {
  int n, c, h, w, r, s, p, q;
  int pad_h, pad_w, str_h, str_w, dil_h, dil_w;
  int64_t xs_n, xs_c, xs_h, xs_w;  // element strides of the image tensor
};

constexpr int TILE = 64;
constexpr int TLD = TILE + 2;  // 33 words per LDS row: conflict-free turned reads

__global__ __launch_bounds__(256) void im2col_kernel(const uint16_t* __restrict__ x,
                                                     uint16_t* __restrict__ cols, int64_t ld,
                                                     ConvGeom g, const int32_t* row_ptr,
                                                     const int32_t* col_idx, int bs) {
  __shared__ uint16_t tile[TILE * TLD];
  const int t = threadIdx.x;
  const int64_t rows = (int64_t)g.n * g.p * g.q;
  const int ncols = g.c * g.r * g.s;
  const int64_t r0 = (int64_t)blockIdx.x * TILE;

  // this thread's row while gathering (fixed: 256 % 64 == 0)
  const int64_t grow = r0 + (t % TILE);
  const bool row_ok = grow < rows;
  int n_i = 0, h_base = 0, w_base = 0;
  if (row_ok) {
    const int pq = (int)(grow % ((int64_t)g.p * g.q));
    n_i = (int)(grow / ((int64_t)g.p * g.q));
    h_base = (pq / g.q) * g.str_h - g.pad_h;
    w_base = (pq % g.q) * g.str_w - g.pad_w;
  }
  const uint16_t* xn = x + (int64_t)n_i * g.xs_n;

  const int sub_per_block = bs / TILE;  // 64-column tiles per mask block
  const int ntiles = (ncols + TILE - 1) / TILE;
  int32_t pos = 0, end = 0;
  if (row_ptr) {
    const int64_t rb = r0 / bs;
    pos = row_ptr[rb];
    end = row_ptr[rb + 1];
  }
  int sub = 0, ct = -1;
  for (;;) {
    // next column tile: all of them, or the tiles of the kept blocks of this row block
    if (row_ptr) {
      if (pos >= end) break;
      ct = col_idx[pos] * sub_per_block + sub;
      if (++sub == sub_per_block) { sub = 0; ++pos; }
      if (ct >= ntiles) continue;
    } else {
      if (++ct >= ntiles) break;
    }
    const int c0 = ct * TILE;
    // gather: lanes along rows (q fastest)
#pragma unroll 4
    for (int i = 0; i < TILE * TILE / 256; ++i) {
      const int col_l = t / TILE + i * (256 / TILE);
      const int col = c0 + col_l;
      uint16_t v = 0;
      if (row_ok && col < ncols) {
        const int ci = col / (g.r * g.s);
        const int rs = col % (g.r * g.s);
        const int hh = h_base + (rs / g.s) * g.dil_h;
        const int ww = w_base + (rs % g.s) * g.dil_w;
        if (hh >= 0 && hh < g.h && ww >= 0 && ww < g.w)
          v = xn[(int64_t)ci * g.xs_c + (int64_t)hh * g.xs_h + (int64_t)ww * g.xs_w];
      }
      tile[col_l * TLD + (t % TILE)] = v;
    }
    __syncthreads();
    // write: lanes along columns
#pragma unroll 4
    for (int i = 0; i < TILE * TILE / 256; ++i) {
      const int row_l = t / TILE + i * (256 / TILE);
      const int col_l = t % TILE;
      const int64_t row = r0 + row_l;
      if (row < rows && c0 + col_l < ncols) cols[row * ld + c0 + col_l] = tile[col_l * TLD + row_l];
    }
    __syncthreads();
  }
}

// Adjoint: one thread per image element sums the (at most R*S) patch-matrix entries that were
// gathered from it; fp32 accumulation, one rounding.  Lanes run along w.
template <typename T>
__global__ __launch_bounds__(256) void col2im_kernel(const uint16_t* __restrict__ cols, int64_t ld,
                                                     uint16_t* __restrict__ dx, ConvGeom g,
                                                     const uint8_t* mask, int64_t msr, int64_t msc,
                                                     int bs) {
  const int64_t total = (int64_t)g.n * g.c * g.h * g.w;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int wi = (int)(e % g.w);
  const int hi = (int)((e / g.w) % g.h);
  const int ci = (int)((e / ((int64_t)g.w * g.h)) % g.c);
  const int ni = (int)(e / ((int64_t)g.w * g.h * g.c));
  float acc = 0.f;
  for (int rr = 0; rr < g.r; ++rr) {
    const int pu = hi + g.pad_h - rr * g.dil_h;
    if (pu < 0 || pu % g.str_h) continue;
    const int pp = pu / g.str_h;
    if (pp >= g.p) continue;
    for (int ss = 0; ss < g.s; ++ss) {
      const int qu = wi + g.pad_w - ss * g.dil_w;
      if (qu < 0 || qu % g.str_w) continue;
      const int qq = qu / g.str_w;
      if (qq >= g.q) continue;
      const int64_t row = ((int64_t)ni * g.p + pp) * g.q + qq;
      const int col = (ci * g.r + rr) * g.s + ss;
      if (mask && mask[(row / bs) * msr + (col / bs) * msc]) continue;
      acc += T::to_float(cols[row * ld + col]);
    }
  }
  dx[(int64_t)ni * g.xs_n + (int64_t)ci * g.xs_c + (int64_t)hi * g.xs_h + (int64_t)wi * g.xs_w] =
      T::from_float(acc);
}

}  // namespace

static int make_geom(ConvGeom& g, int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s,
                     int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h,
                     int64_t dil_w, int64_t sn, int64_t sc, int64_t sh, int64_t sw) {
  SD_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && r > 0 && s > 0, "conv: sizes must be positive");
  SD_REQUIRE(stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0 && pad_h >= 0 && pad_w >= 0,
             "conv: stride/dilation must be positive and padding non-negative");
  const int64_t p = (h + 2 * pad_h - dil_h * (r - 1) - 1) / stride_h + 1;
  const int64_t q = (w + 2 * pad_w - dil_w * (s - 1) - 1) / stride_w + 1;
  SD_REQUIRE(h + 2 * pad_h - dil_h * (r - 1) - 1 >= 0 && w + 2 * pad_w - dil_w * (s - 1) - 1 >= 0,
             "conv: kernel does not fit the padded image");
  SD_REQUIRE(n < (1 << 30) && c * r * s < (1 << 30) && h < (1 << 30) && w < (1 << 30) &&
                 p * q < (1LL << 31),
             "conv: extent too large");
  g = ConvGeom{(int)n, (int)c, (int)h, (int)w, (int)r, (int)s, (int)p, (int)q,
               (int)pad_h, (int)pad_w, (int)stride_h, (int)stride_w, (int)dil_h, (int)dil_w,
               sn, sc, sh, sw};
  return SD_OK;
}

int im2col(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t sw, void* cols, int64_t ld,
           int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
           int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
           const int32_t* row_ptr, const int32_t* col_idx, int64_t bs, hipStream_t stream) {
  ConvGeom g;
  if (int rc = make_geom(g, n, c, h, w, r, s, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, sn, sc,
                         sh, sw))
    return rc;
  SD_REQUIRE(x && cols, "im2col: null pointer");
  SD_REQUIRE(ld >= c * r * s, "im2col: cols_ld %lld < C*R*S %lld", (long long)ld, (long long)(c * r * s));
  SD_REQUIRE((row_ptr == nullptr) == (col_idx == nullptr), "im2col: pass both list arrays or neither");
  if (row_ptr) SD_REQUIRE(bs > 0 && bs % TILE == 0, "im2col: block_size must be a multiple of 64");
  const int64_t rows = n * g.p * g.q;
  const int64_t blocks = ceil_div(rows, TILE);
  SD_REQUIRE(blocks <= 0x7fffffffLL, "im2col: too many rows");
  hipLaunchKernelGGL(im2col_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                     (const uint16_t*)x, (uint16_t*)cols, ld, g, row_ptr, col_idx,
                     row_ptr ? (int)bs : TILE);
  return check_launch("im2col");
}

int col2im(const void* cols, int64_t ld, void* dx, int64_t sn, int64_t sc, int64_t sh, int64_t sw,
           int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
           int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
           const uint8_t* mask, int64_t msr, int64_t msc, int64_t bs, int dtype, hipStream_t stream) {
  ConvGeom g;
  if (int rc = make_geom(g, n, c, h, w, r, s, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, sn, sc,
                         sh, sw))
    return rc;
  SD_REQUIRE(dx && cols, "col2im: null pointer");
  SD_REQUIRE(ld >= c * r * s, "col2im: cols_ld %lld < C*R*S %lld", (long long)ld, (long long)(c * r * s));
  if (mask) SD_REQUIRE(bs > 0, "col2im: block_size must be positive with a mask");
  const int64_t total = n * c * h * w;
  const int64_t blocks = ceil_div(total, 256);
  SD_REQUIRE(blocks <= 0x7fffffffLL, "col2im: image too large");
  if (dtype == SD_BF16)
    hipLaunchKernelGGL(col2im_kernel<BF16>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1);
  else
    hipLaunchKernelGGL(col2im_kernel<F16>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1);
  return check_launch("col2im");
}

}  // namespace sd
