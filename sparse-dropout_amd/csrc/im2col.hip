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
constexpr int TLD = TILE + 2;  // 33 words per LDS row: both the 2-byte column writes and the 4-byte row reads are conflict-free

__global__ __launch_bounds__(256) void im2col_kernel(const uint16_t* __restrict__ x,
                                                     uint16_t* __restrict__ cols, int64_t ld,
                                                     ConvGeom g, const int32_t* row_ptr,
                                                     const int32_t* col_idx, int bs) {
  __shared__ __attribute__((aligned(4))) uint16_t tile[TILE * TLD];  // [row][col]
  const int t = threadIdx.x;
  const int lane = t % 64;
  const int wave = __builtin_amdgcn_readfirstlane(t / 64);
  const int64_t rows = (int64_t)g.n * g.p * g.q;
  const int ncols = g.c * g.r * g.s;
  const int64_t r0 = (int64_t)blockIdx.x * TILE;

  // gather phase: lane = row of the tile, so a wave reads consecutive pixels of an image row
  const int64_t grow = r0 + lane;
  const bool row_ok = grow < rows;
  int h_base = 0, w_base = 0;
  const uint16_t* xrow = x;
  if (row_ok) {
    const int pq = (int)(grow % ((int64_t)g.p * g.q));
    const int n_i = (int)(grow / ((int64_t)g.p * g.q));
    h_base = (pq / g.q) * g.str_h - g.pad_h;
    w_base = (pq % g.q) * g.str_w - g.pad_w;
    xrow = x + (int64_t)n_i * g.xs_n + (int64_t)h_base * g.xs_h + (int64_t)w_base * g.xs_w;
  }
  // write phase: 32 lanes x 4 bytes cover the 128 bytes of one tile row; needs even, 4-byte aligned columns
  const bool pair_ok = (ld % 2 == 0) && (reinterpret_cast<uintptr_t>(cols) % 4 == 0);

  const int sub_per_block = bs / TILE;  // 64-column tiles per mask block
  const int ntiles = (ncols + TILE - 1) / TILE;
  const int rs_n = g.r * g.s;
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
    // gather: wave w takes columns w, w+4, ...; the column's (c, r, s) is wave-uniform
#pragma unroll 4
    for (int i = 0; i < TILE / 4; ++i) {
      const int col_l = wave + 4 * i;
      const int col = c0 + col_l;
      uint16_t v = 0;
      if (col < ncols) {
        const int ci = col / rs_n;
        const int rs = col - ci * rs_n;
        const int dh = (rs / g.s) * g.dil_h;
        const int dw = (rs % g.s) * g.dil_w;
        const int hh = h_base + dh, ww = w_base + dw;
        if (row_ok && hh >= 0 && hh < g.h && ww >= 0 && ww < g.w)
          v = xrow[(int64_t)ci * g.xs_c + (int64_t)dh * g.xs_h + (int64_t)dw * g.xs_w];
      }
      tile[lane * TLD + col_l] = v;
    }
    __syncthreads();
    // write: 4 bytes per lane, a full 128-byte line per half wave
    if (pair_ok) {
#pragma unroll 4
      for (int i = 0; i < TILE * TILE / 2 / 256; ++i) {
        const int row_l = t / 32 + i * 8;
        const int cp = (t % 32) * 2;
        const int64_t row = r0 + row_l;
        if (row < rows) {
          const uint32_t two = *reinterpret_cast<const uint32_t*>(&tile[row_l * TLD + cp]);
          uint16_t* dst = cols + row * ld + c0 + cp;
          if (c0 + cp + 1 < ncols) *reinterpret_cast<uint32_t*>(dst) = two;
          else if (c0 + cp < ncols) *dst = (uint16_t)two;
        }
      }
    } else {
#pragma unroll 4
      for (int i = 0; i < TILE * TILE / 256; ++i) {
        const int row_l = t / TILE + i * (256 / TILE);
        const int col_l = t % TILE;
        const int64_t row = r0 + row_l;
        if (row < rows && c0 + col_l < ncols) cols[row * ld + c0 + col_l] = tile[row_l * TLD + col_l];
      }
    }
    __syncthreads();
  }
}

// Patch-staged variant for the common case that the 64 rows of a workgroup lie in one image
// ((P*Q) % 64 == 0): per 64-column tile the (at most 64/(R*S) + 2) input channels it touches are copied
// once into LDS as a zero-padded patch [channel][input row][padded input column]; every output element
// is then an LDS read with no bounds check, and a thread assembles 8 consecutive columns of one row
// into a single 16-byte store.  Global reads drop to the unique bytes, global writes are full lines.
constexpr int PATCH_MAX_BYTES = 48 * 1024;

__global__ __launch_bounds__(256) void im2col_patch_kernel(const uint16_t* __restrict__ x,
                                                           uint16_t* __restrict__ cols, int64_t ld,
                                                           ConvGeom g, const int32_t* row_ptr,
                                                           const int32_t* col_idx, int bs, int hp,
                                                           int wp, int max_ch) {
  extern __shared__ __attribute__((aligned(16))) uint16_t patch[];  // [max_ch][hp][wp]
  __shared__ int col_off[TILE];  // patch offset of each column of the tile (0 past the last column: never stored)
  const int t = threadIdx.x;
  const int ncols = g.c * g.r * g.s;
  const int rs_n = g.r * g.s;
  const int pq = g.p * g.q;
  const int64_t r0 = (int64_t)blockIdx.x * TILE;
  const int n_i = (int)(r0 / pq);
  const int pq0 = (int)(r0 % pq);
  const int p_lo = pq0 / g.q;
  const int h_lo = p_lo * g.str_h - g.pad_h;  // input row of patch row 0
  const uint16_t* xn = x + (int64_t)n_i * g.xs_n;

  // per-thread output rows (two per tile): patch offset of their top-left tap
  int row_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row_l = t / 8 + 32 * i;
    const int pql = pq0 + row_l;
    row_off[i] = ((pql / g.q - p_lo) * g.str_h) * wp + (pql % g.q) * g.str_w;
  }

  const int sub_per_block = bs / TILE;
  const int ntiles = (ncols + TILE - 1) / TILE;
  int32_t pos = 0, end = 0;
  if (row_ptr) {
    const int64_t rb = r0 / bs;
    pos = row_ptr[rb];
    end = row_ptr[rb + 1];
  }
  int sub = 0, ct = -1;
  for (;;) {
    if (row_ptr) {
      if (pos >= end) break;
      ct = col_idx[pos] * sub_per_block + sub;
      if (++sub == sub_per_block) { sub = 0; ++pos; }
      if (ct >= ntiles) continue;
    } else {
      if (++ct >= ntiles) break;
    }
    const int c0 = ct * TILE;
    const int ch_lo = c0 / rs_n;
    const int last = (c0 + TILE - 1 < ncols ? c0 + TILE - 1 : ncols - 1);
    const int nch = last / rs_n - ch_lo + 1;
    // stage the patch: lanes along the padded input column
    const int per_ch = hp * wp;
    for (int e = t; e < nch * per_ch; e += 256) {
      const int ci = e / per_ch, rem = e - ci * per_ch;
      const int hh = h_lo + rem / wp, ww = rem % wp - g.pad_w;
      uint16_t v = 0;
      if (hh >= 0 && hh < g.h && ww >= 0 && ww < g.w)
        v = xn[(int64_t)(ch_lo + ci) * g.xs_c + (int64_t)hh * g.xs_h + (int64_t)ww * g.xs_w];
      patch[e] = v;
    }
    if (t < TILE) {
      const int col = c0 + t;
      int off = 0;
      if (col < ncols) {
        const int ci = col / rs_n, rs = col - ci * rs_n;
        off = ((ci - ch_lo) * hp + (rs / g.s) * g.dil_h) * wp + (rs % g.s) * g.dil_w;
      }
      col_off[t] = off;
    }
    __syncthreads();
    const int ch8 = (t % 8) * 8;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row_l = t / 8 + 32 * i;
      uint16_t e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int off = col_off[ch8 + j];
        e[j] = patch[off + row_off[i]];
      }
      uint16_t* dst = cols + (r0 + row_l) * ld + c0 + ch8;
      if (c0 + ch8 + 8 <= ncols) {
        u32x4 v;
        v.x = e[0] | ((uint32_t)e[1] << 16);
        v.y = e[2] | ((uint32_t)e[3] << 16);
        v.z = e[4] | ((uint32_t)e[5] << 16);
        v.w = e[6] | ((uint32_t)e[7] << 16);
        *reinterpret_cast<u32x4*>(dst) = v;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (c0 + ch8 + j < ncols) dst[j] = e[j];
      }
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

// Tiled adjoint for aligned patch matrices.  A workgroup owns one image, a band of `hb` input rows and a
// group of 8 channels.  Everything of the patch matrix that feeds those outputs — the 8*R*S columns of
// the channel group, for every output row p that touches the band and every q — is copied to LDS first
// with 16-byte loads (R*S consecutive lanes cover one contiguous row segment; dropped blocks are filled
// with zeros instead of being read), then each thread sums the taps of its outputs out of LDS.  Global
// reads are whole segments instead of one 2-byte element per lane and cache line.
constexpr int C2I_CG = 8;
constexpr int C2I_MAX_LDS = 60 * 1024;  // below the 64 KB a kernel gets without asking

template <typename T>
__global__ __launch_bounds__(256) void col2im_tile_kernel(const uint16_t* __restrict__ cols, int64_t ld,
                                                          uint16_t* __restrict__ dx, ConvGeom g,
                                                          const uint8_t* mask, int64_t msr, int64_t msc,
                                                          int bs, int hb, int np_max, int bands) {
  extern __shared__ __attribute__((aligned(16))) uint16_t seg[];  // [p][q][8*R*S + 2]
  const int t = threadIdx.x;
  const int rs_n = g.r * g.s;
  const int seg_h = C2I_CG * rs_n + 2;  // halfs per (p, q) segment; the 2 spare halfs spread the banks
  int b = blockIdx.x;
  const int band = b % bands;
  b /= bands;
  const int cgs = g.c / C2I_CG;
  const int c0 = (b % cgs) * C2I_CG;
  const int n_i = b / cgs;
  const int h0 = band * hb;
  const int h1 = (h0 + hb < g.h ? h0 + hb : g.h);  // band = input rows [h0, h1)
  // output rows p with a tap inside the band: p*str_h - pad_h + r*dil_h in [h0, h1) for some r
  int p_lo = h0 + g.pad_h - (g.r - 1) * g.dil_h;
  p_lo = p_lo <= 0 ? 0 : (p_lo + g.str_h - 1) / g.str_h;
  int p_hi = (h1 - 1 + g.pad_h) / g.str_h;
  if (p_hi > g.p - 1) p_hi = g.p - 1;
  const int np = p_hi - p_lo + 1;  // <= np_max (may be <= 0 for a band no output row reaches)

  // ---- stage: R*S 16-byte chunks per (p, q) --------------------------------------------------------
  const int chunks = (np > 0 ? np : 0) * g.q * rs_n;
  const int64_t row0 = ((int64_t)n_i * g.p + p_lo) * g.q;
  const int col0 = c0 * rs_n;
  for (int ch = t; ch < chunks; ch += 256) {
    const int row_l = ch / rs_n, k = ch - row_l * rs_n;
    const int64_t row = row0 + row_l;
    const int col = col0 + k * 8;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (!mask || !mask[(row / bs) * msr + (col / bs) * msc])
      v = *reinterpret_cast<const u32x4*>(cols + row * ld + col);
    uint32_t* dst = reinterpret_cast<uint32_t*>(seg + row_l * seg_h + k * 8);
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
  }
  __syncthreads();

  // ---- sum the taps ----------------------------------------------------------------------------------
  const bool c_fast = g.xs_c == 1;  // channels-last image: lanes along c, else along w
  const int outs = C2I_CG * (h1 - h0) * g.w;
  uint16_t* dxn = dx + (int64_t)n_i * g.xs_n;
  for (int o = t; o < outs; o += 256) {
    int c_l, hi, wi;
    if (c_fast) {
      c_l = o % C2I_CG;
      wi = (o / C2I_CG) % g.w;
      hi = h0 + o / (C2I_CG * g.w);
    } else {
      wi = o % g.w;
      hi = h0 + (o / g.w) % (h1 - h0);
      c_l = o / (g.w * (h1 - h0));
    }
    float acc = 0.f;
    for (int rr = 0; rr < g.r; ++rr) {
      const int pu = hi + g.pad_h - rr * g.dil_h;
      if (pu < 0) break;  // pu only decreases with rr
      int pp = pu;
      if (g.str_h != 1) {
        pp = pu / g.str_h;
        if (pp * g.str_h != pu) continue;
      }
      if (pp >= g.p) continue;
      const uint16_t* prow = seg + (pp - p_lo) * g.q * seg_h + (c_l * g.r + rr) * g.s;
      for (int ss = 0; ss < g.s; ++ss) {
        const int qu = wi + g.pad_w - ss * g.dil_w;
        if (qu < 0) break;
        int qq = qu;
        if (g.str_w != 1) {
          qq = qu / g.str_w;
          if (qq * g.str_w != qu) continue;
        }
        if (qq >= g.q) continue;
        acc += T::to_float(prow[qq * seg_h + ss]);
      }
    }
    dxn[(int64_t)(c0 + c_l) * g.xs_c + (int64_t)hi * g.xs_h + (int64_t)wi * g.xs_w] = T::from_float(acc);
  }
}

// The same for unit stride and dilation (the usual 3x3 / 5x5 layer), where output (h, w) takes tap
// (r, s) from patch row (h + pad_h - r, w + pad_w - s): the staged window gets a zero halo, rows and
// columns outside the patch matrix included, so the tap loop has no bounds checks and walks LDS with
// constant strides.  A thread owns one (channel, w) column of the band and runs down its rows.
template <typename T>
__global__ __launch_bounds__(256) void col2im_unit_kernel(const uint16_t* __restrict__ cols, int64_t ld,
                                                          uint16_t* __restrict__ dx, ConvGeom g,
                                                          const uint8_t* mask, int64_t msr, int64_t msc,
                                                          int bs, int hb, int bands) {
  extern __shared__ __attribute__((aligned(16))) uint16_t seg[];  // [hb + R - 1][W + S - 1][8*R*S + 2]
  const int t = threadIdx.x;
  const int rs_n = g.r * g.s;
  const int seg_h = C2I_CG * rs_n + 2;
  const int bs_shift = (bs & (bs - 1)) == 0 ? 31 - __builtin_clz((unsigned)bs) : -1;
  int b = blockIdx.x;
  const int band = b % bands;
  b /= bands;
  const int cgs = g.c / C2I_CG;
  const int c0 = (b % cgs) * C2I_CG;
  const int n_i = b / cgs;
  const int h0 = band * hb;
  const int h1 = (h0 + hb < g.h ? h0 + hb : g.h);
  const int pe = (h1 - h0) + g.r - 1, qe = g.w + g.s - 1;     // staged window
  const int p_first = h0 + g.pad_h - (g.r - 1), q_first = g.pad_w - (g.s - 1);  // its top-left (p, q)

  // ---- stage: R*S 16-byte chunks per window position, zeros outside the matrix and for dropped blocks
  const int chunks = pe * qe * rs_n;
  const int col0 = c0 * rs_n;
  // the few mask entries the window can touch are copied to LDS first, so that the staging loop does not
  // chain a global mask read in front of every data load
  __shared__ uint8_t mtab[256];
  int64_t rb_lo = 0;
  int cb_lo = 0, cb_n = 1;
  bool mask_in_lds = false;
  if (mask) {
    const int pp_lo = p_first > 0 ? p_first : 0;
    const int pp_hi = p_first + pe - 1 < g.p - 1 ? p_first + pe - 1 : g.p - 1;
    rb_lo = (((int64_t)n_i * g.p + pp_lo) * g.q) / bs;
    const int64_t rb_hi = (((int64_t)n_i * g.p + pp_hi) * g.q + g.q - 1) / bs;
    cb_lo = col0 / bs;
    cb_n = (col0 + C2I_CG * rs_n - 1) / bs - cb_lo + 1;
    const int64_t rb_n = pp_hi >= pp_lo ? rb_hi - rb_lo + 1 : 0;
    mask_in_lds = rb_n * cb_n <= 256;
    if (mask_in_lds) {
      if (t < rb_n * cb_n) mtab[t] = mask[(rb_lo + t / cb_n) * msr + (cb_lo + t % cb_n) * msc];
      __syncthreads();
    }
  }
  for (int ch0 = t; ch0 < chunks; ch0 += 4 * 256) {
    u32x4 v[4];
    const uint16_t* src[4];  // null: zeros
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // four independent mask reads, then four independent loads, per lane
      const int ch = ch0 + i * 256;
      src[i] = nullptr;
      uint8_t dropped = 0;
      if (ch < chunks) {
        const int pos = ch / rs_n, k = ch - pos * rs_n;
        const int pp = p_first + pos / qe, qq = q_first + pos % qe;
        if (pp >= 0 && pp < g.p && qq >= 0 && qq < g.q) {
          const int64_t row = ((int64_t)n_i * g.p + pp) * g.q + qq;
          const int col = col0 + k * 8;
          src[i] = cols + row * ld + col;
          if (mask) {
            // block sizes are powers of two in practice: a shift instead of a 64-bit division per chunk
            const int64_t rb = bs_shift >= 0 ? row >> bs_shift : row / bs;
            const int cb = bs_shift >= 0 ? col >> bs_shift : col / bs;
            dropped = mask_in_lds ? mtab[(rb - rb_lo) * cb_n + (cb - cb_lo)] : mask[rb * msr + cb * msc];
          }
        }
      }
      if (dropped) src[i] = nullptr;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = u32x4{0u, 0u, 0u, 0u};
      if (src[i]) v[i] = *reinterpret_cast<const u32x4*>(src[i]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = ch0 + i * 256;
      if (ch < chunks) {
        const int pos = ch / rs_n, k = ch - pos * rs_n;
        uint32_t* dst = reinterpret_cast<uint32_t*>(seg + pos * seg_h + k * 8);
        dst[0] = v[i].x;
        dst[1] = v[i].y;
        dst[2] = v[i].z;
        dst[3] = v[i].w;
      }
    }
  }
  __syncthreads();

  // ---- sum the taps: window position of tap (r, s) of output (h, w) is (h - h0 + R-1-r, w + S-1-s) ---
  const bool c_fast = g.xs_c == 1;
  const int pairs = C2I_CG * g.w;
  const int row_h = qe * seg_h;  // halfs per window row
  uint16_t* dxn = dx + (int64_t)n_i * g.xs_n;
  for (int pr = t; pr < pairs; pr += 256) {
    const int c_l = c_fast ? pr % C2I_CG : pr / g.w;
    const int wi = c_fast ? pr / C2I_CG : pr % g.w;
    // tap (0, 0) of the band's first row
    const uint16_t* base = seg + (g.r - 1) * row_h + (wi + g.s - 1) * seg_h + c_l * rs_n;
    uint16_t* out = dxn + (int64_t)(c0 + c_l) * g.xs_c + (int64_t)h0 * g.xs_h + (int64_t)wi * g.xs_w;
    for (int hl = 0; hl < h1 - h0; ++hl) {
      float acc = 0.f;
      const uint16_t* tap_r = base + hl * row_h;
      for (int rr = 0; rr < g.r; ++rr) {
        const uint16_t* tap = tap_r;
        for (int ss = 0; ss < g.s; ++ss) {
          acc += T::to_float(*tap);
          tap -= seg_h - 1;  // one window column to the left, next s
        }
        tap_r -= row_h - g.s;  // one window row up, next r
      }
      out[(int64_t)hl * g.xs_h] = T::from_float(acc);
    }
  }
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
  // patch-staged kernel: workgroup rows inside one image, 16-byte aligned stores, patch fits in LDS
  const int64_t pq = (int64_t)g.p * g.q;
  const int rows_p = (int)((TILE + g.q - 2) / g.q + 1);  // output rows p a 64-row group can touch
  const int hp = (rows_p - 1) * g.str_h + (g.r - 1) * g.dil_h + 1;
  const int wp = (g.q - 1) * g.str_w + (g.s - 1) * g.dil_w + 1;
  const int max_ch = (int)((TILE + r * s - 2) / (r * s) + 1);
  const int64_t patch_bytes = (int64_t)max_ch * hp * wp * 2;
  if (pq % TILE == 0 && ld % 8 == 0 && reinterpret_cast<uintptr_t>(cols) % 16 == 0 &&
      patch_bytes <= PATCH_MAX_BYTES) {
    hipLaunchKernelGGL(im2col_patch_kernel, dim3((unsigned)blocks), dim3(256), (size_t)patch_bytes, stream,
                       (const uint16_t*)x, (uint16_t*)cols, ld, g, row_ptr, col_idx,
                       row_ptr ? (int)bs : TILE, hp, wp, max_ch);
    return check_launch("im2col_patch");
  }
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
  // tiled kernel: 16-byte loads of 8-channel column groups need aligned rows and whole groups
  if (c % C2I_CG == 0 && ld % 8 == 0 && reinterpret_cast<uintptr_t>(cols) % 16 == 0 &&
      (!mask || bs % 8 == 0)) {
    const int seg_bytes = (C2I_CG * g.r * g.s + 2) * 2;
    const bool unit = g.str_h == 1 && g.str_w == 1 && g.dil_h == 1 && g.dil_w == 1;
    for (int band_rows = 8; band_rows >= 1; band_rows /= 2) {  // the tallest band whose staging fits
      const int hb = band_rows < g.h ? band_rows : g.h;
      if (unit) {
        const int64_t lds = (int64_t)(hb + g.r - 1) * (g.w + g.s - 1) * seg_bytes;
        const int64_t bands = ceil_div(g.h, hb);
        const int64_t wgs = n * (c / C2I_CG) * bands;
        if (lds > C2I_MAX_LDS || wgs > 0x7fffffffLL) continue;
        if (dtype == SD_BF16)
          hipLaunchKernelGGL(col2im_unit_kernel<BF16>, dim3((unsigned)wgs), dim3(256), (size_t)lds, stream,
                             (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1,
                             hb, (int)bands);
        else
          hipLaunchKernelGGL(col2im_unit_kernel<F16>, dim3((unsigned)wgs), dim3(256), (size_t)lds, stream,
                             (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1,
                             hb, (int)bands);
        return check_launch("col2im_unit");
      }
      const int np_max = (hb - 1 + (g.r - 1) * g.dil_h) / g.str_h + 1;
      const int64_t lds = (int64_t)np_max * g.q * seg_bytes;
      const int64_t bands = ceil_div(g.h, hb);
      const int64_t wgs = n * (c / C2I_CG) * bands;
      if (lds > C2I_MAX_LDS || wgs > 0x7fffffffLL) continue;
      if (dtype == SD_BF16)
        hipLaunchKernelGGL(col2im_tile_kernel<BF16>, dim3((unsigned)wgs), dim3(256), (size_t)lds, stream,
                           (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1, hb,
                           np_max, (int)bands);
      else
        hipLaunchKernelGGL(col2im_tile_kernel<F16>, dim3((unsigned)wgs), dim3(256), (size_t)lds, stream,
                           (const uint16_t*)cols, ld, (uint16_t*)dx, g, mask, msr, msc, mask ? (int)bs : 1, hb,
                           np_max, (int)bands);
      return check_launch("col2im_tile");
    }
  }
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
