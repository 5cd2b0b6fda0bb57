// Shared device/host helpers for the SparseDrop gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "sparsedrop.h"

namespace sd {

// ---- error plumbing -------------------------------------------------------------------------
char* last_error_buf();  // thread-local, 512 bytes (api.hip)

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}

// Records which kernel (and workgroup shape) the calling thread's last launch used: sd_last_kernel_detail().
char* kernel_detail_buf();  // thread-local, 96 bytes (api.hip)
inline void note_kernel(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(kernel_detail_buf(), 96, fmt, ap);
  va_end(ap);
}

#define SD_REQUIRE(cond, ...)                                  \
  do {                                                         \
    if (!(cond)) return ::sd::fail(SD_ERR_INVALID, __VA_ARGS__); \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SD_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
  return SD_OK;
}

// ---- vector types ---------------------------------------------------------------------------
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

struct F16 {
  using vec8 = f16x8;
  static constexpr int id = SD_F16;
  __device__ static inline uint16_t from_float(float x) {
    _Float16 h = (_Float16)x;
    return __builtin_bit_cast(uint16_t, h);
  }
  __device__ static inline float to_float(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
  // D(32x32) += A(32x16) * B(16x32); lane l supplies row/col l%32, k = 8*(l/32)..+7 of its operand.
  __device__ static inline f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  __device__ static inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

struct BF16 {
  using vec8 = bf16x8;
  static constexpr int id = SD_BF16;
  __device__ static inline uint16_t from_float(float x) {
    __bf16 h = (__bf16)x;
    return __builtin_bit_cast(uint16_t, h);
  }
  __device__ static inline float to_float(uint16_t v) {
    return __builtin_bit_cast(float, (uint32_t)v << 16);
  }
  __device__ static inline f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  __device__ static inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- operand descriptors --------------------------------------------------------------------
// A matrix operand as the kernels see it: base pointer plus element strides along its row index
// and along its second index.
struct Mat {
  const uint16_t* ptr;
  int64_t sr;  // stride of the row index
  int64_t sc;  // stride of the column index
};

struct GemmArgs {
  Mat a;         // [M, K]
  Mat b;         // [N, K]
  uint16_t* c;   // [M, N]
  int64_t c_sr, c_sc;
  int64_t M, N, K;
  int64_t bs;     // mask block size (0 for dense)
  bool quads;     // the lists are on the 64 grid of a block-size-32 mask: bits 28-31 of an entry say which of its four
                  // 32 x 32 quadrants are kept (bit 2a + b: row half a, column half b); 0 in those bits = all four
  float scale;
  const int32_t* row_ptr;  // CSR of the mask (DSD: over A; SDD: over C); null for dense
  const int32_t* col_idx;
  float* ws;         // optional split-K workspace (fp32 partial tiles), may be null
  int64_t ws_bytes;
  bool kept_only;    // SDD: dropped tiles of C are left untouched instead of being zeroed
  float keep_hint;   // SDD: the caller's estimate of the kept fraction of blocks (picks the workgroup shape); < 0 = unknown
  // fused epilogue (0 = none): DSD / dense: C = act(v), and v itself to `aux` when that is given (the pre-activation
  // the backward needs); SDD: C = v * act'(aux[m, n]) (aux: the pre-activation, or for ReLU the activated tensor).
  // v is the scaled fp32 accumulator; aux is addressed like C but with its own strides.
  int act;
  uint16_t* aux;
  int64_t aux_sr, aux_sc;
};

// Geometry of a convolution whose patch matrix the DSD kernel gathers itself (implicit GEMM):
// x[n][c][h][w] with unit w stride, row block = 64 / Q whole output rows of one image.
struct ImplicitConv {
  const uint16_t* x;
  int64_t sn, sc, sh;  // element strides of x
  int C, H, W, Q;      // channels, input height and width, output width
  int RS, S;           // taps per channel, kernel width
  int pad_h, pad_w;
  int sth, stw, dlh, dlw;  // strides and dilations
  int rpb;             // output rows per 64-row block (64 / Q)
  int blocks_per_img;  // P * Q / 64
  int PR;              // input rows the output rows of a workgroup's 4 row blocks (units == 4: of one block) touch:
                       // (output rows - 1) * stride + (R - 1) * dilation + 1
  int units;           // forward: 1 = the 4 row blocks share one run of input rows, 4 = each has its own (P*Q % 256 != 0)
  int PW;              // halfs per row of the LDS copy: 8 zeros, then the W of the image
  int patch_stride;    // weight gradient: halfs between the two alternating copies (set by the launcher)
  int K;               // C * R * S
  // ceil(2^32 / d) for the divisors the kernel needs (0 for d = 1): x / d == umulhi(x, m) while x * d < 2^32
  uint32_t m_spc, m_spr, m_RS, m_S, m_Q;  // d = PR * W / 8, W / 8, R * S, S, Q
};

enum Mode { kDense = 0, kDsd = 1, kSdd = 2 };

// list entry -> block index / quadrant keep bits
__device__ inline int32_t entry_block(int32_t e) { return (int32_t)((uint32_t)e & 0x0fffffffu); }
__device__ inline uint32_t entry_quads(int32_t e) {
  const uint32_t q = (uint32_t)e >> 28;
  return q ? q : 0xfu;
}

// ---- fused epilogues --------------------------------------------------------------------------
// GELU is the exact (erf) form, torch.nn.GELU's default: gelu(x) = x * Phi(x), gelu'(x) = Phi(x) + x * phi(x).
// Phi comes from the rational approximation of erf in Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7, far
// under the resolution of the fp16 / bf16 results): one exponential, one reciprocal and a degree-5 polynomial, a
// third of the instructions of erff, which matters because the epilogue of a GEMM has nothing to hide them behind.
// *pdf receives exp(-x^2 / 2), which the derivative needs as well.
__device__ inline float normal_cdf(float x, float* pdf) {
  const float z = fabsf(x) * 0.70710678118654752f;
  const float e = __expf(-z * z);
  const float t = __builtin_amdgcn_rcpf(1.f + 0.3275911f * z);
  const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
  const float tail = 0.5f * poly * e;  // Phi(-|x|)
  *pdf = e;
  return x >= 0.f ? 1.f - tail : tail;
}
__device__ inline float act_apply(int act, float x) {
  if (act == SD_ACT_RELU) return x > 0.f ? x : 0.f;
  if (act == SD_ACT_GELU) {
    float e;
    return x * normal_cdf(x, &e);
  }
  return x;
}
__device__ inline float act_derivative(int act, float x) {
  if (act == SD_ACT_RELU) return x > 0.f ? 1.f : 0.f;
  if (act == SD_ACT_GELU) {
    float e;
    const float cdf = normal_cdf(x, &e);
    return cdf + x * 0.39894228040143268f * e;
  }
  return 1.f;
}
// Stores element (m, n) of the result: v is the scaled fp32 accumulator.  SDD multiplies by the derivative of the
// activation at aux[m, n]; the others apply the activation and, if asked, also keep v.
template <typename T, bool SDD>
__device__ inline void store_result(const GemmArgs& g, int64_t m, int64_t n, float v) {
  if (g.act != SD_ACT_NONE) {
    if (SDD) {
      if (v != 0.f) v *= act_derivative(g.act, T::to_float(g.aux[m * g.aux_sr + n * g.aux_sc]));  // dropped tiles stay exact zeros
    } else {
      if (g.aux) g.aux[m * g.aux_sr + n * g.aux_sc] = T::from_float(v);
      v = act_apply(g.act, v);
    }
  }
  g.c[m * g.c_sr + n * g.c_sc] = T::from_float(v);
}

// One wave's [ROWS][COLS] tile of unscaled fp32 accumulators, staged in the wave's own LDS region (pitch COLS + 4
// floats) with COLS running along C's contiguous index, goes out in full 16-byte pieces: a lane takes 8 consecutive
// elements of one row, scales them, applies the fused epilogue, rounds once and stores them (128-byte lines are
// written whole by 8 neighbouring lanes).  s0 / c0: where the tile starts along C's strided / contiguous index
// (c0 a multiple of 8); along_n: the contiguous index is n (row-major C).  part: fp32 partial sums of a split
// reduction go to `part` (C's element order, unscaled) instead.
template <typename T, bool SDD, int ROWS, int COLS>
__device__ inline void store_staged_tile(const GemmArgs& g, const float* stg, int lane, bool along_n, int64_t s0,
                                         int64_t c0, float* part) {
  constexpr int PITCH = COLS + 4, LPR = COLS / 8, RPP = 64 / LPR;  // lanes per row, rows per pass
  const int64_t s_ext = along_n ? g.M : g.N, c_ext = along_n ? g.N : g.M;
  const int64_t ld = along_n ? g.c_sr : g.c_sc, unit = along_n ? g.c_sc : g.c_sr;
  bool vec = unit == 1 && ld % 8 == 0 && reinterpret_cast<uintptr_t>(g.c) % 16 == 0;
  const bool has_aux = g.act != SD_ACT_NONE && g.aux != nullptr;
  const int64_t ald = along_n ? g.aux_sr : g.aux_sc, aunit = along_n ? g.aux_sc : g.aux_sr;
  if (has_aux) vec = vec && aunit == 1 && ald % 8 == 0 && reinterpret_cast<uintptr_t>(g.aux) % 16 == 0;
#pragma unroll
  for (int pass = 0; pass < ROWS / RPP; ++pass) {
    const int row = pass * RPP + lane / LPR, ch = lane % LPR;
    const int64_t si = s0 + row, ci = c0 + ch * 8;
    if (si >= s_ext || ci >= c_ext) continue;
    const f32x4 lo = *reinterpret_cast<const f32x4*>(stg + row * PITCH + ch * 8);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(stg + row * PITCH + ch * 8 + 4);
    float r[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    const int valid = c_ext - ci < 8 ? (int)(c_ext - ci) : 8;
    if (part) {
      float* dst = part + si * c_ext + ci;
      if (valid == 8 && c_ext % 4 == 0) {
        *reinterpret_cast<f32x4*>(dst) = lo;
        *reinterpret_cast<f32x4*>(dst + 4) = hi;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (i < valid) dst[i] = r[i];
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] *= g.scale;
    if (!(vec && valid == 8)) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i < valid) store_result<T, SDD>(g, along_n ? si : ci + i, along_n ? ci + i : si, r[i]);
      continue;
    }
    auto pack = [&](const float (&v)[8]) {
      return u32x4{(uint32_t)T::from_float(v[0]) | ((uint32_t)T::from_float(v[1]) << 16),
                   (uint32_t)T::from_float(v[2]) | ((uint32_t)T::from_float(v[3]) << 16),
                   (uint32_t)T::from_float(v[4]) | ((uint32_t)T::from_float(v[5]) << 16),
                   (uint32_t)T::from_float(v[6]) | ((uint32_t)T::from_float(v[7]) << 16)};
    };
    if (g.act != SD_ACT_NONE) {
      if (SDD) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(g.aux + si * ald + ci);
        const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint16_t h = (uint16_t)(i & 1 ? w[i / 2] >> 16 : w[i / 2] & 0xffffu);
          if (r[i] != 0.f) r[i] *= act_derivative(g.act, T::to_float(h));  // dropped tiles stay exact zeros
        }
      } else {
        if (has_aux) *reinterpret_cast<u32x4*>(g.aux + si * ald + ci) = pack(r);
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = act_apply(g.act, r[i]);
      }
    }
    *reinterpret_cast<u32x4*>(g.c + si * ld + ci) = pack(r);
  }
}

// launchers (one per translation unit)
int launch_generic(const GemmArgs& g, int mode, int dtype, hipStream_t stream);
// number of reduction splits the generic kernel would like for this problem (1 = none); it needs
// splits * M * N * 4 bytes of workspace for that
int generic_splits(int64_t M, int64_t N, int64_t K, int64_t bs, int mode);
// reduction splits the fast DSD kernel would like (1 = none); same scratch rule
int fast_splits(int64_t M, int64_t N, int64_t K);
// C = scale * sum of `splits` fp32 partials [splits][M*N] laid out in C's element order
int launch_splitk_reduce(const GemmArgs& g, int splits, bool trans_out, int dtype, hipStream_t stream);
// returns SD_ERR_UNSUPPORTED (without setting an error message) when the fast path does not apply
int launch_fast(const GemmArgs& g, int mode, int dtype, hipStream_t stream);
// dX (SDD) and dW (DSD, reduction-strided operands, column-major C) of one layer in a single launch;
// SD_ERR_UNSUPPORTED with nothing launched when the pair does not qualify
int launch_backward_pair(const GemmArgs& gx, const GemmArgs& gw, int dtype, hipStream_t stream);
// The forward product on its specialised kernel and the kept lists of its mask (stored: mask / msr / msc; drawn when
// mask is null: seed / offset or the device-resident state, p, stored to mask_out) in a single launch; arguments as
// for build_lists / random_lists.  SD_ERR_UNSUPPORTED with nothing launched when the pair does not qualify.
int forward_with_lists(const GemmArgs& g, const uint8_t* mask, int64_t msr, int64_t msc, uint64_t seed, uint64_t offset,
                       uint64_t* state, float p, int64_t stored_mb, int64_t stored_kb, uint8_t* mask_out, int64_t split,
                       int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                       int dtype, hipStream_t stream);
struct MaskSrc;
int launch_forward_with_lists(const GemmArgs& g, const MaskSrc& src, int64_t mb, int64_t kb, int32_t* row_ptr,
                              int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, uint8_t* mask_out,
                              int64_t mask_rows, int dtype, hipStream_t stream);
// forward of the block-dropout convolution without the patch matrix: g.a is unused, g.b the [K_out, C*R*S]
// weight matrix, g.c the [N*P*Q, K_out] output, the lists over the patch matrix's block grid.  Returns
// SD_ERR_UNSUPPORTED (without an error message) for geometries it does not take.
int launch_conv_implicit(const GemmArgs& g, const ImplicitConv& cg, int64_t P, int64_t stride_h, int64_t stride_w,
                         int64_t dil_h, int64_t dil_w, int64_t R, int64_t x_sw, int dtype, hipStream_t stream);
// weight gradient of the same convolution without the patch matrix: g.M = C*R*S, g.N = K_out, g.K = N*P*Q, g.b =
// dY^T, g.c column-major, the lists those of the transposed mask; cg.PR = rows one 64-position block touches.
int launch_conv_implicit_dw(const GemmArgs& g, ImplicitConv cg, int64_t P, int64_t stride_h, int64_t stride_w,
                            int64_t dil_h, int64_t dil_w, int64_t R, int64_t x_sw, int dtype, hipStream_t stream);
// reduction splits that launch would like for a [M x N] result over a reduction of K (1 = none)
int conv_dw_splits(int64_t M, int64_t N, int64_t K);
// input gradient of the stride-1 convolution straight from dY and the weights (kept 64 x 64 tiles of the patch
// matrix's gradient are formed and folded in LDS); SD_ERR_UNSUPPORTED without a message for what it does not take
int launch_conv_dx(const void* dy, int64_t dy_ld, const void* w, int64_t w_ld, void* dx, int64_t sn, int64_t sc,
                   int64_t sh, int64_t sw, const uint8_t* mask, int64_t msr, int64_t msc, int64_t n, int64_t c,
                   int64_t h, int64_t wd, int64_t k_out, int64_t r, int64_t s, int64_t pad_h, int64_t pad_w,
                   int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w, float scale, int dtype,
                   hipStream_t stream);
// which workgroup shape the DSD kernel runs in: chosen from the shape, or forced (tuning and tests);
// returns the previous policy, -1 for an unknown one
enum { kTileAuto = 0, kTileBig = 1, kTileMid = 2 };
int set_tile_policy(int policy);

}  // namespace sd
