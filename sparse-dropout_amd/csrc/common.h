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
  float scale;
  const int32_t* row_ptr;  // CSR of the mask (DSD: over A; SDD: over C); null for dense
  const int32_t* col_idx;
  float* ws;         // optional split-K workspace (fp32 partial tiles), may be null
  int64_t ws_bytes;
  bool kept_only;    // SDD: dropped tiles of C are left untouched instead of being zeroed
  float keep_hint;   // SDD: the caller's estimate of the kept fraction of blocks (picks the workgroup shape); < 0 = unknown
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
