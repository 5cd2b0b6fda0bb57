// extern "C" surface of libsparsedrop: argument validation and dispatch.  No kernels here.
#include "common.h"
#include "tile_map.h"

#include <cstdlib>
#include <cstring>

namespace sd {

char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

char* kernel_detail_buf() {
  static thread_local char buf[96] = {0};
  return buf;
}

int build_lists(const uint8_t* mask, int64_t msr, int64_t msc, int64_t stored_mb, int64_t stored_kb, int64_t split,
                int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                int32_t* row_idx, hipStream_t stream);
int random_lists(uint64_t seed, uint64_t offset, uint64_t* state, float p, int64_t stored_mb, int64_t stored_kb,
                 uint8_t* mask_out, int64_t split, int64_t mb, int64_t kb, int32_t* row_ptr,
                 int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, hipStream_t stream);
int increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                    int64_t* table, int64_t* row_indices, int64_t* row_widths, hipStream_t stream);
int im2col(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t sw, void* cols, int64_t ld,
           int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
           int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
           const int32_t* row_ptr, const int32_t* col_idx, int64_t bs, hipStream_t stream);
int col2im(const void* cols, int64_t ld, void* dx, int64_t sn, int64_t sc, int64_t sh, int64_t sw,
           int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
           int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
           const uint8_t* mask, int64_t msr, int64_t msc, int64_t bs, int dtype, hipStream_t stream);

namespace {

constexpr int64_t kMaxDim = 1LL << 31;

int check_mat(const char* name, const void* p, int64_t sr, int64_t sc, int64_t rows, int64_t cols) {
  SD_REQUIRE(p != nullptr || rows == 0 || cols == 0, "%s: null pointer", name);
  SD_REQUIRE(sr == 1 || sc == 1, "%s must be row or column major (strides %lld, %lld)", name,
             (long long)sr, (long long)sc);
  SD_REQUIRE(sr >= 1 && sc >= 1, "%s: strides must be positive", name);
  // the non-unit stride must span the contiguous extent, or rows overlap
  if (sc == 1 && rows > 1) SD_REQUIRE(sr >= cols, "%s: row stride %lld < %lld columns", name, (long long)sr, (long long)cols);
  if (sr == 1 && sc != 1 && cols > 1) SD_REQUIRE(sc >= rows, "%s: column stride %lld < %lld rows", name, (long long)sc, (long long)rows);
  return SD_OK;
}

int check_common(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                 void* C, int64_t csr, int64_t csc, int64_t M, int64_t N, int64_t K, int dtype) {
  SD_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative dimension");
  SD_REQUIRE(M < kMaxDim && N < kMaxDim && K < kMaxDim, "dimension too large");
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  if (int rc = check_mat("A", A, asr, asc, M, K)) return rc;
  if (int rc = check_mat("B", B, bsr, bsc, N, K)) return rc;
  if (int rc = check_mat("C", C, csr, csc, M, N)) return rc;
  return SD_OK;
}

int check_sparse(int64_t bs, float scale) {
  SD_REQUIRE(bs > 0, "block_size must be positive");
  if (bs % 32 != 0)
    return fail(SD_ERR_UNSUPPORTED, "block_size %lld: only multiples of 32 are supported", (long long)bs);
  SD_REQUIRE(scale == scale, "scale is NaN");
  return SD_OK;
}

thread_local const char* last_kernel = "";

bool generic_forced() {
  static const bool force_generic = [] {
    const char* e = std::getenv("SPARSEDROP_FORCE_GENERIC");
    return e && e[0] == '1';
  }();
  return force_generic;
}

// SPARSEDROP_SEPARATE_BACKWARD=1: sd_dropout_matmul_backward launches its two products one after the other even where
// they qualify for the single launch (for comparing the two)
bool separate_backward_forced() {
  static const bool forced = [] {
    const char* e = std::getenv("SPARSEDROP_SEPARATE_BACKWARD");
    return e && e[0] == '1';
  }();
  return forced;
}

int run(const GemmArgs& g, int mode, int dtype, hipStream_t stream) {
  if (!generic_forced()) {
    const int rc = launch_fast(g, mode, dtype, stream);
    if (rc != SD_ERR_UNSUPPORTED) {
      last_kernel = "specialised";
      return rc;
    }
  }
  last_kernel = "generic";
  return launch_generic(g, mode, dtype, stream);
}

GemmArgs make_args(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                   void* C, int64_t csr, int64_t csc, int64_t M, int64_t N, int64_t K, int64_t bs,
                   float scale, const int32_t* row_ptr, const int32_t* col_idx, void* ws = nullptr,
                   int64_t ws_bytes = 0) {
  GemmArgs g;
  g.a = Mat{(const uint16_t*)A, asr, asc};
  g.b = Mat{(const uint16_t*)B, bsr, bsc};
  g.c = (uint16_t*)C;
  g.c_sr = csr;
  g.c_sc = csc;
  g.M = M;
  g.N = N;
  g.K = K;
  // an odd multiple of 32 (the *_lists calls pass 32 for all of them): the lists are on the 64 grid and carry the
  // keep bits of each entry's four 32-blocks
  g.quads = bs % 64 == 32;
  g.bs = g.quads ? 64 : bs;
  g.scale = scale;
  g.row_ptr = row_ptr;
  g.col_idx = col_idx;
  // split-K scratch is optional: unusable pointers just mean "no split"
  const bool ws_ok = ws != nullptr && ws_bytes > 0 && reinterpret_cast<uintptr_t>(ws) % 16 == 0;
  g.ws = ws_ok ? static_cast<float*>(ws) : nullptr;
  g.ws_bytes = ws_ok ? ws_bytes : 0;
  g.kept_only = false;
  g.keep_hint = -1.f;
  g.act = SD_ACT_NONE;
  g.aux = nullptr;
  g.aux_sr = g.aux_sc = 0;
  return g;
}

}  // namespace
}  // namespace sd

using namespace sd;

// Geometry of an implicit-GEMM launch whose LDS copy of the input covers `blocks` 64-position row blocks.
static ImplicitConv conv_geometry(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t c, int64_t h, int64_t w,
                                  int64_t P, int64_t Q, int64_t r, int64_t s, int64_t pad_h, int64_t pad_w,
                                  int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w, int64_t blocks) {
  ImplicitConv cg;
  cg.x = static_cast<const uint16_t*>(x);
  cg.sn = sn;
  cg.sc = sc;
  cg.sh = sh;
  cg.C = (int)c;
  cg.H = (int)h;
  cg.W = (int)w;
  cg.Q = (int)Q;
  cg.RS = (int)(r * s);
  cg.S = (int)s;
  cg.pad_h = (int)pad_h;
  cg.pad_w = (int)pad_w;
  cg.rpb = (int)(64 / Q);
  cg.blocks_per_img = (int)(P * Q / 64);
  cg.sth = (int)stride_h;
  cg.stw = (int)stride_w;
  cg.dlh = (int)dil_h;
  cg.dlw = (int)dil_w;
  cg.PR = (int)((blocks * (64 / Q) - 1) * stride_h + (r - 1) * dil_h + 1);
  cg.PW = (int)(w + 8);
  cg.patch_stride = 0;
  cg.units = 1;
  cg.K = (int)(c * r * s);
  auto magic = [](int64_t d) { return d <= 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d); };
  cg.m_spc = magic(cg.PR * (w / 8));
  cg.m_spr = magic(w / 8);
  cg.m_RS = magic(r * s);
  cg.m_S = magic(s);
  cg.m_Q = magic(Q);
  return cg;
}

extern "C" {

int sd_version(void) { return 110; }

// build.py writes the hash of the sources this library was compiled from into build/source_hash.inc
#if __has_include("source_hash.inc")
#include "source_hash.inc"
#else
#define SD_SOURCE_HASH "unknown"
#endif
const char* sd_source_hash(void) { return SD_SOURCE_HASH; }

const char* sd_last_error(void) { return last_error_buf(); }

const char* sd_last_kernel(void) { return last_kernel; }

const char* sd_last_kernel_detail(void) { return kernel_detail_buf(); }

int sd_tile_of_block(int kind, int64_t block, int64_t tiles_m, int64_t tiles_n, int32_t* tile_m, int32_t* tile_n) {
  SD_REQUIRE(kind == 0 || kind == 1, "tile_of_block: kind must be 0 (DSD order) or 1 (SDD order)");
  SD_REQUIRE(tile_m && tile_n, "tile_of_block: null output");
  SD_REQUIRE(tiles_m > 0 && tiles_n > 0 && tiles_m * tiles_n < kMaxDim, "tile_of_block: bad grid");
  SD_REQUIRE(block >= 0 && block < tiles_m * tiles_n, "tile_of_block: block outside the grid");
  int tm = 0, tn = 0;
  if (kind == 0)
    tile_of_block<DSD_GROUP_M>((int)block, (int)tiles_m, (int)tiles_n, tm, tn);
  else
    tile_of_block<SDD_GROUP_M>((int)block, (int)tiles_m, (int)tiles_n, tm, tn);
  *tile_m = tm;
  *tile_n = tn;
  return SD_OK;
}

int sd_set_tile_policy(int policy) { return sd::set_tile_policy(policy); }

int64_t sd_workspace_bytes(int64_t mb, int64_t kb) {
  if (mb < 0 || kb < 0) return 0;
  // row_ptr[mb+1] then col_idx[mb*kb], the first padded to a 16-byte boundary
  const int64_t ptr_bytes = ((mb + 1) * 4 + 15) / 16 * 16;
  return ptr_bytes + mb * kb * 4;
}

static int check_list_grid(int64_t mb, int64_t kb, int64_t split, int64_t out_mb, int64_t out_kb,
                           const int32_t* row_ptr, const int32_t* col_idx, const int32_t* col_ptr,
                           const int32_t* row_idx) {
  SD_REQUIRE(mb > 0 && kb > 0, "build_lists: mask must be non-empty (got %lld x %lld)", (long long)mb, (long long)kb);
  SD_REQUIRE(split > -(1 << 16) && split < (1 << 16), "build_lists: split out of range (got %lld)", (long long)split);
  if (split <= 0) {
    // a mask at block size 32 * sub listed on the 64 grid: its 32-blocks merged two by two.  The grid must end inside
    // the mask's last row / column of entries (for sub == 1 that fixes it)
    const int64_t sub = split ? -split : 1;
    SD_REQUIRE(2 * out_mb > (mb - 1) * sub && out_mb <= (mb * sub + 1) / 2 && 2 * out_kb > (kb - 1) * sub &&
                   out_kb <= (kb * sub + 1) / 2,
               "build_lists: a %lld x %lld grid of 64-blocks does not match a %lld x %lld mask at block size %lld",
               (long long)out_mb, (long long)out_kb, (long long)mb, (long long)kb, (long long)(32 * sub));
    SD_REQUIRE(out_kb < (1 << 28), "build_lists: merged lists keep four bits of every entry for the quadrants");
  } else {
    // the listed grid is the mask repeated split x split, cropped inside its last row / column of entries
    SD_REQUIRE(out_mb > (mb - 1) * split && out_mb <= mb * split && out_kb > (kb - 1) * split && out_kb <= kb * split,
               "build_lists: a %lld x %lld grid does not match a %lld x %lld mask split by %lld", (long long)out_mb,
               (long long)out_kb, (long long)mb, (long long)kb, (long long)split);
  }
  SD_REQUIRE(out_mb * out_kb < kMaxDim, "build_lists: mask too large for 32-bit lists");
  SD_REQUIRE((row_ptr == nullptr) == (col_idx == nullptr), "build_lists: pass both CSR arrays or neither");
  SD_REQUIRE((col_ptr == nullptr) == (row_idx == nullptr), "build_lists: pass both CSC arrays or neither");
  SD_REQUIRE(row_ptr || col_ptr, "build_lists: nothing to build");
  return SD_OK;
}

int sd_build_lists_split(const uint8_t* mask, int64_t mb, int64_t kb, int64_t msr, int64_t msc,
                         int64_t split, int64_t out_mb, int64_t out_kb, int32_t* row_ptr,
                         int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, void* stream) {
  SD_REQUIRE(mask != nullptr, "build_lists: null mask");
  if (int rc = check_list_grid(mb, kb, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx)) return rc;
  SD_REQUIRE(msr >= 1 && msc >= 1 && (msr == 1 || msc == 1), "build_lists: mask must be row or column major");
  return build_lists(mask, msr, msc, mb, kb, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx,
                     (hipStream_t)stream);
}

int sd_build_lists(const uint8_t* mask, int64_t mb, int64_t kb, int64_t msr, int64_t msc,
                   int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                   void* stream) {
  return sd_build_lists_split(mask, mb, kb, msr, msc, 1, mb, kb, row_ptr, col_idx, col_ptr, row_idx, stream);
}

int sd_random_lists(uint64_t seed, uint64_t offset, float p, int64_t mb, int64_t kb, uint8_t* mask_out,
                    int64_t split, int64_t out_mb, int64_t out_kb, int32_t* row_ptr, int32_t* col_idx,
                    int32_t* col_ptr, int32_t* row_idx, void* stream) {
  SD_REQUIRE(p >= 0.f && p < 1.f, "random_lists: p must be in [0, 1) (got %g)", (double)p);
  SD_REQUIRE(mask_out != nullptr, "random_lists: null mask_out");
  if (int rc = check_list_grid(mb, kb, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx)) return rc;
  return random_lists(seed, offset, nullptr, p, mb, kb, mask_out, split, out_mb, out_kb, row_ptr, col_idx, col_ptr,
                      row_idx, (hipStream_t)stream);
}

int sd_random_lists_state(uint64_t* state, float p, int64_t mb, int64_t kb, uint8_t* mask_out, int64_t split,
                          int64_t out_mb, int64_t out_kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                          int32_t* row_idx, void* stream) {
  SD_REQUIRE(state != nullptr && reinterpret_cast<uintptr_t>(state) % 8 == 0, "random_lists: state must be an aligned device pointer");
  SD_REQUIRE(p >= 0.f && p < 1.f, "random_lists: p must be in [0, 1) (got %g)", (double)p);
  SD_REQUIRE(mask_out != nullptr, "random_lists: null mask_out");
  if (int rc = check_list_grid(mb, kb, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx)) return rc;
  return random_lists(0, 0, state, p, mb, kb, mask_out, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx,
                      (hipStream_t)stream);
}

int sd_increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                       int64_t* table, int64_t* row_indices, int64_t* row_widths, void* stream) {
  SD_REQUIRE(row_ptr && col_idx && table && row_indices && row_widths, "increment_table: null pointer");
  SD_REQUIRE(mb > 0 && block_k > 0, "increment_table: mb and block_k must be positive");
  return increment_table(row_ptr, col_idx, mb, block_k, table, row_indices, row_widths, (hipStream_t)stream);
}

int64_t sd_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t block_size, int sparse) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int splits = generic_splits(M, N, K, sparse ? block_size : 0, sparse ? kDsd : kDense);
  if (!sparse || block_size == 64) {
    const int fs = fast_splits(M, N, K);
    if (fs > splits) splits = fs;
  }
  return splits > 1 ? (int64_t)splits * M * N * 4 : 0;
}

int sd_gemm(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc, void* C,
            int64_t csr, int64_t csc, int64_t M, int64_t N, int64_t K, int dtype, void* workspace,
            int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, 0, 1.0f, nullptr, nullptr,
                         workspace, workspace_bytes);
  return run(g, kDense, dtype, (hipStream_t)stream);
}

int sd_gemm_dsd_lists(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                      void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                      int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype,
                      void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_dsd: null list");
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx,
                         workspace, workspace_bytes);
  return run(g, kDsd, dtype, (hipStream_t)stream);
}

int sd_gemm_sdd_lists(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                      void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                      int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_sdd: null list");
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx);
  return run(g, kSdd, dtype, (hipStream_t)stream);
}

int sd_gemm_sdd_lists_ex(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                         void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                         int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype, int kept_only,
                         float keep_hint, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_sdd: null list");
  SD_REQUIRE(!(keep_hint > 1.f), "gemm_sdd: keep_hint must be a fraction in [0, 1], or negative for unknown");
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx);
  g.kept_only = kept_only != 0;
  g.keep_hint = keep_hint == keep_hint ? keep_hint : -1.f;
  return run(g, kSdd, dtype, (hipStream_t)stream);
}

static int check_act(int act, const void* aux, int64_t xsr, int64_t xsc, int64_t M, int64_t N, bool aux_required) {
  SD_REQUIRE(act == SD_ACT_NONE || act == SD_ACT_RELU || act == SD_ACT_GELU, "act must be SD_ACT_NONE, SD_ACT_RELU or SD_ACT_GELU (got %d)", act);
  if (act == SD_ACT_NONE) return SD_OK;
  SD_REQUIRE(!aux_required || aux != nullptr, "the activation gradient needs the tensor it is evaluated at");
  if (aux) return check_mat("aux", aux, xsr, xsc, M, N);
  return SD_OK;
}

int sd_gemm_act(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc, void* C,
                int64_t csr, int64_t csc, int64_t M, int64_t N, int64_t K, int dtype, int act, void* pre_out,
                int64_t pre_stride_r, int64_t pre_stride_c, void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_act(act, pre_out, pre_stride_r, pre_stride_c, M, N, false)) return rc;
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, 0, 1.0f, nullptr, nullptr,
                         workspace, workspace_bytes);
  g.act = act;
  g.aux = act != SD_ACT_NONE ? static_cast<uint16_t*>(pre_out) : nullptr;
  g.aux_sr = pre_stride_r;
  g.aux_sc = pre_stride_c;
  // Row-major A with a reduction-strided B (a weight given as a transposed view) is the operand layout of the input
  // gradient: the specialised kernel that takes it multiplies by an activation's derivative in its store, it does
  // not apply one.  With an activation that layout runs on the generic kernel, whose store applies it.
  if (act != SD_ACT_NONE && asc == 1 && bsr == 1 && bsc != 1 && csc == 1) {
    last_kernel = "generic";
    return launch_generic(g, kDense, dtype, (hipStream_t)stream);
  }
  return run(g, kDense, dtype, (hipStream_t)stream);
}

int sd_gemm_dsd_lists_act(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                          void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                          int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype, int act, void* pre_out,
                          int64_t pre_stride_r, int64_t pre_stride_c, void* workspace, int64_t workspace_bytes,
                          void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_dsd: null list");
  if (int rc = check_act(act, pre_out, pre_stride_r, pre_stride_c, M, N, false)) return rc;
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx,
                         workspace, workspace_bytes);
  g.act = act;
  g.aux = act != SD_ACT_NONE ? static_cast<uint16_t*>(pre_out) : nullptr;
  g.aux_sr = pre_stride_r;
  g.aux_sc = pre_stride_c;
  return run(g, kDsd, dtype, (hipStream_t)stream);
}

int sd_gemm_sdd_lists_actgrad(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                              void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                              int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype, int act,
                              const void* act_at, int64_t at_stride_r, int64_t at_stride_c, float keep_hint,
                              void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_sdd: null list");
  SD_REQUIRE(!(keep_hint > 1.f), "gemm_sdd: keep_hint must be a fraction in [0, 1], or negative for unknown");
  if (int rc = check_act(act, act_at, at_stride_r, at_stride_c, M, N, true)) return rc;
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx);
  g.keep_hint = keep_hint == keep_hint ? keep_hint : -1.f;
  g.act = act;
  g.aux = act != SD_ACT_NONE ? const_cast<uint16_t*>(static_cast<const uint16_t*>(act_at)) : nullptr;
  g.aux_sr = at_stride_r;
  g.aux_sc = at_stride_c;
  return run(g, kSdd, dtype, (hipStream_t)stream);
}

int sd_gemm_sdd_lists_kept(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc,
                           void* C, int64_t csr, int64_t csc, const int32_t* row_ptr, const int32_t* col_idx,
                           int64_t M, int64_t N, int64_t K, int64_t bs, float scale, int dtype, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  SD_REQUIRE(row_ptr && col_idx, "gemm_sdd: null list");
  GemmArgs g = make_args(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, bs, scale, row_ptr, col_idx);
  g.kept_only = true;
  return run(g, kSdd, dtype, (hipStream_t)stream);
}

// Builds the CSR list of a [rows x cols] operand's mask at the head of the workspace.  When the block
// size is a larger multiple of 64 and the workspace holds the finer list, the mask is listed at 64
// granularity (each entry repeated) so that the 64-block kernels apply; *bs and *used report the choice.
static int lists_in_workspace(const uint8_t* mask, int64_t msr, int64_t msc, int64_t rows, int64_t cols,
                              int64_t* bs, void* workspace, int64_t workspace_bytes, int32_t** row_ptr,
                              int32_t** col_idx, int64_t* used, void* stream) {
  SD_REQUIRE(mask != nullptr, "null mask");
  const int64_t mb = ceil_div(rows, *bs), kb = ceil_div(cols, *bs);
  SD_REQUIRE(mb > 0 && kb > 0, "empty mask");
  int64_t split = 1, out_mb = mb, out_kb = kb;
  if (*bs % 64 == 32) {  // listed on the 64 grid with quadrant bits; the *_lists calls are told so by block size 32
    split = -(*bs / 32);
    out_mb = ceil_div(rows, 64);
    out_kb = ceil_div(cols, 64);
    *bs = 32;
  } else if (*bs > 64 && *bs % 64 == 0 && ceil_div(rows, 64) * ceil_div(cols, 64) < kMaxDim &&
             workspace_bytes >= sd_workspace_bytes(ceil_div(rows, 64), ceil_div(cols, 64))) {
    split = *bs / 64;
    out_mb = ceil_div(rows, 64);
    out_kb = ceil_div(cols, 64);
    *bs = 64;
  }
  const int64_t need = sd_workspace_bytes(out_mb, out_kb);
  SD_REQUIRE(workspace != nullptr && workspace_bytes >= need, "workspace too small: need %lld bytes, got %lld",
             (long long)need, (long long)workspace_bytes);
  SD_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, "workspace must be 16-byte aligned");
  *row_ptr = (int32_t*)workspace;
  *col_idx = (int32_t*)((char*)workspace + ((out_mb + 1) * 4 + 15) / 16 * 16);
  *used = (need + 15) / 16 * 16;
  return sd_build_lists_split(mask, mb, kb, msr, msc, split, out_mb, out_kb, *row_ptr, *col_idx, nullptr,
                              nullptr, stream);
}

int sd_gemm_dsd(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc, void* C,
                int64_t csr, int64_t csc, const uint8_t* mask, int64_t msr, int64_t msc, int64_t M,
                int64_t N, int64_t K, int64_t bs, float scale, int dtype, void* workspace,
                int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  if (M == 0 || N == 0) return SD_OK;
  SD_REQUIRE(K > 0, "gemm_dsd: K must be positive");
  int32_t *row_ptr, *col_idx;
  int64_t used;
  if (int rc = lists_in_workspace(mask, msr, msc, M, K, &bs, workspace, workspace_bytes, &row_ptr, &col_idx,
                                  &used, stream))
    return rc;
  // whatever the caller provided beyond the lists serves as split-K scratch
  return sd_gemm_dsd_lists(A, asr, asc, B, bsr, bsc, C, csr, csc, row_ptr, col_idx, M, N, K, bs, scale,
                           dtype, workspace_bytes > used ? (char*)workspace + used : nullptr,
                           workspace_bytes > used ? workspace_bytes - used : 0, stream);
}

int sd_gemm_sdd(const void* A, int64_t asr, int64_t asc, const void* B, int64_t bsr, int64_t bsc, void* C,
                int64_t csr, int64_t csc, const uint8_t* mask, int64_t msr, int64_t msc, int64_t M,
                int64_t N, int64_t K, int64_t bs, float scale, int dtype, void* workspace,
                int64_t workspace_bytes, void* stream) {
  if (int rc = check_common(A, asr, asc, B, bsr, bsc, C, csr, csc, M, N, K, dtype)) return rc;
  if (int rc = check_sparse(bs, scale)) return rc;
  if (M == 0 || N == 0) return SD_OK;
  int32_t *row_ptr, *col_idx;
  int64_t used;
  if (int rc = lists_in_workspace(mask, msr, msc, M, N, &bs, workspace, workspace_bytes, &row_ptr, &col_idx,
                                  &used, stream))
    return rc;
  return sd_gemm_sdd_lists(A, asr, asc, B, bsr, bsc, C, csr, csc, row_ptr, col_idx, M, N, K, bs, scale,
                           dtype, stream);
}

// granularity of the lists the fused calls build and take: 64 for block sizes that are multiples of 64
static int64_t list_granule(int64_t bs) { return bs % 32 == 0 ? 64 : bs; }
// what tells the *_lists calls that the lists carry quadrant bits: block size 32, whatever odd multiple of 32 the mask has
static int64_t lists_block_size(int64_t bs) { return bs % 64 == 32 ? 32 : list_granule(bs); }
// the `split` argument of the list builders for a mask at this block size
static int64_t list_split(int64_t bs) { return bs % 64 == 32 ? -(bs / 32) : bs / list_granule(bs); }

int sd_dropout_matmul_forward(const void* X, int64_t xsr, int64_t xsc, const void* W, int64_t wsr, int64_t wsc,
                              void* Y, int64_t ysr, int64_t ysc, const uint8_t* mask, int64_t msr, int64_t msc,
                              uint64_t* rng_state, uint64_t seed, uint64_t offset, double p, uint8_t* mask_out,
                              int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, int64_t M,
                              int64_t N, int64_t K, int64_t bs, int dtype, void* workspace, int64_t workspace_bytes,
                              void* stream) {
  return sd_dropout_matmul_forward_act(X, xsr, xsc, W, wsr, wsc, Y, ysr, ysc, mask, msr, msc, rng_state, seed, offset, p,
                                       mask_out, row_ptr, col_idx, col_ptr, row_idx, M, N, K, bs, dtype, SD_ACT_NONE,
                                       nullptr, 0, 0, workspace, workspace_bytes, stream);
}

// SPARSEDROP_SEPARATE_FORWARD=1: the lists and the product of the fused forward always in two launches (for measuring)
static bool separate_forward_forced() {
  static const bool forced = [] {
    const char* e = std::getenv("SPARSEDROP_SEPARATE_FORWARD");
    return e && e[0] == '1';
  }();
  return forced;
}

int sd_dropout_matmul_forward_act(const void* X, int64_t xsr, int64_t xsc, const void* W, int64_t wsr, int64_t wsc,
                                  void* Y, int64_t ysr, int64_t ysc, const uint8_t* mask, int64_t msr, int64_t msc,
                                  uint64_t* rng_state, uint64_t seed, uint64_t offset, double p, uint8_t* mask_out,
                                  int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, int64_t M,
                                  int64_t N, int64_t K, int64_t bs, int dtype, int act, void* pre_out,
                                  int64_t pre_stride_r, int64_t pre_stride_c, void* workspace, int64_t workspace_bytes,
                                  void* stream) {
  if (int rc = check_common(X, xsr, xsc, W, wsr, wsc, Y, ysr, ysc, M, N, K, dtype)) return rc;
  SD_REQUIRE(p >= 0.f && p < 1.f, "dropout_matmul_forward: p must be in [0, 1) (got %g)", (double)p);
  if (int rc = check_sparse(bs, 1.f)) return rc;
  SD_REQUIRE(M > 0 && K > 0, "dropout_matmul_forward: empty operand");
  SD_REQUIRE(row_ptr && col_idx, "dropout_matmul_forward: the CSR list arrays are required");
  if (int rc = check_act(act, pre_out, pre_stride_r, pre_stride_c, M, N, false)) return rc;
  const int64_t g = list_granule(bs), split = list_split(bs);  // negative for odd multiples of 32: merged two by two
  const int64_t mb = ceil_div(M, bs), kb = ceil_div(K, bs), out_mb = ceil_div(M, g), out_kb = ceil_div(K, g);
  const float scale = (float)(1.0 / (1.0 - p));  // in double, as the reference's Python evaluates it
  // what the list calls below would check, up front: the single launch takes the same arguments
  if (int rc = check_list_grid(mb, kb, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx)) return rc;
  if (mask) {
    SD_REQUIRE(msr >= 1 && msc >= 1 && (msr == 1 || msc == 1), "build_lists: mask must be row or column major");
  } else {
    SD_REQUIRE(mask_out != nullptr, "random_lists: null mask_out");
    SD_REQUIRE(rng_state == nullptr || reinterpret_cast<uintptr_t>(rng_state) % 8 == 0,
               "random_lists: state must be an aligned device pointer");
  }
  auto with_act = [&](GemmArgs a) {
    a.act = act;
    a.aux = act != SD_ACT_NONE ? static_cast<uint16_t*>(pre_out) : nullptr;
    a.aux_sr = pre_stride_r;
    a.aux_sc = pre_stride_c;
    return a;
  };
  if (N > 0 && !generic_forced() && !separate_forward_forced()) {
    // lists and product in one launch where the pair qualifies (small products, where a launch is a large part)
    const GemmArgs a = with_act(make_args(X, xsr, xsc, W, wsr, wsc, Y, ysr, ysc, M, N, K, lists_block_size(bs), scale,
                                          row_ptr, col_idx, workspace, workspace_bytes));
    const int rc = forward_with_lists(a, mask, msr, msc, seed, offset, rng_state, (float)p, mb, kb, mask_out, split, out_mb,
                                      out_kb, row_ptr, col_idx, col_ptr, row_idx, dtype, (hipStream_t)stream);
    if (rc != SD_ERR_UNSUPPORTED) {
      last_kernel = "specialised";
      return rc;
    }
  }
  if (mask) {
    if (int rc = sd_build_lists_split(mask, mb, kb, msr, msc, split, out_mb, out_kb, row_ptr, col_idx, col_ptr, row_idx,
                                      stream))
      return rc;
  } else if (rng_state) {
    if (int rc = sd_random_lists_state(rng_state, (float)p, mb, kb, mask_out, split, out_mb, out_kb, row_ptr, col_idx, col_ptr,
                                       row_idx, stream))
      return rc;
  } else {
    if (int rc = sd_random_lists(seed, offset, (float)p, mb, kb, mask_out, split, out_mb, out_kb, row_ptr, col_idx, col_ptr,
                                 row_idx, stream))
      return rc;
  }
  if (N == 0) return SD_OK;
  return sd_gemm_dsd_lists_act(X, xsr, xsc, W, wsr, wsc, Y, ysr, ysc, row_ptr, col_idx, M, N, K, lists_block_size(bs),
                               scale, dtype, act, pre_out, pre_stride_r, pre_stride_c, workspace, workspace_bytes,
                               stream);
}

int sd_dropout_matmul_backward(const void* dY, int64_t gsr, int64_t gsc, const void* W, int64_t wsr, int64_t wsc,
                               const void* X, int64_t xsr, int64_t xsc, void* dX, int64_t dxsr, int64_t dxsc,
                               void* dW, int64_t dwsr, int64_t dwsc, const int32_t* row_ptr, const int32_t* col_idx,
                               const int32_t* col_ptr, const int32_t* row_idx, int64_t M, int64_t N, int64_t K,
                               int64_t bs, double p, int dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  return sd_dropout_matmul_backward_act(dY, gsr, gsc, W, wsr, wsc, X, xsr, xsc, dX, dxsr, dxsc, dW, dwsr, dwsc, row_ptr,
                                        col_idx, col_ptr, row_idx, M, N, K, bs, p, dtype, SD_ACT_NONE, nullptr, 0, 0,
                                        workspace, workspace_bytes, stream);
}

int sd_dropout_matmul_backward_act(const void* dY, int64_t gsr, int64_t gsc, const void* W, int64_t wsr, int64_t wsc,
                                   const void* X, int64_t xsr, int64_t xsc, void* dX, int64_t dxsr, int64_t dxsc,
                                   void* dW, int64_t dwsr, int64_t dwsc, const int32_t* row_ptr,
                                   const int32_t* col_idx, const int32_t* col_ptr, const int32_t* row_idx, int64_t M,
                                   int64_t N, int64_t K, int64_t bs, double p, int dtype, int act, const void* act_at,
                                   int64_t at_stride_r, int64_t at_stride_c, void* workspace, int64_t workspace_bytes,
                                   void* stream) {
  SD_REQUIRE(p >= 0.f && p < 1.f, "dropout_matmul_backward: p must be in [0, 1) (got %g)", (double)p);
  if (dX) {
    if (int rc = check_act(act, act_at, at_stride_r, at_stride_c, M, K, true)) return rc;
  }
  if (int rc = check_sparse(bs, 1.f)) return rc;
  SD_REQUIRE(dX || dW, "dropout_matmul_backward: nothing to compute");
  const int64_t g = lists_block_size(bs);  // 32: lists on the 64 grid with quadrant bits
  const float scale = (float)(1.0 / (1.0 - p));  // in double, as the reference's Python evaluates it
  if (dX && dW && row_ptr && col_idx && col_ptr && row_idx && !generic_forced() && !separate_backward_forced()) {
    // both gradients in one launch where the pair qualifies (same operands and checks as the two calls below)
    if (int rc = check_common(dY, gsr, gsc, W, wsc, wsr, dX, dxsr, dxsc, M, K, N, dtype)) return rc;
    if (int rc = check_common(X, xsc, xsr, dY, gsc, gsr, dW, dwsc, dwsr, K, N, M, dtype)) return rc;
    GemmArgs gx = make_args(dY, gsr, gsc, W, wsc, wsr, dX, dxsr, dxsc, M, K, N, g, scale, row_ptr, col_idx);
    gx.keep_hint = (float)(1.0 - p);
    gx.act = act;
    gx.aux = act != SD_ACT_NONE ? const_cast<uint16_t*>(static_cast<const uint16_t*>(act_at)) : nullptr;
    gx.aux_sr = at_stride_r;
    gx.aux_sc = at_stride_c;
    GemmArgs gw = make_args(X, xsc, xsr, dY, gsc, gsr, dW, dwsc, dwsr, K, N, M, g, scale, col_ptr, row_idx, workspace,
                            workspace_bytes);
    const int rc = launch_backward_pair(gx, gw, dtype, (hipStream_t)stream);
    if (rc != SD_ERR_UNSUPPORTED) {
      last_kernel = "specialised";
      return rc;
    }
  }
  if (dX) {
    // dX[M,K] = scale * (dY[M,N] . W[N,K]) where kept: A = dY, B = W^T as the [K, N] view of W
    SD_REQUIRE(row_ptr && col_idx, "dropout_matmul_backward: dX needs the CSR lists");
    if (int rc = sd_gemm_sdd_lists_actgrad(dY, gsr, gsc, W, wsc, wsr, dX, dxsr, dxsc, row_ptr, col_idx, M, K, N, g,
                                           scale, dtype, act, act_at, at_stride_r, at_stride_c, (float)(1.0 - p), stream))
      return rc;
  }
  if (dW) {
    // dW^T[K,N] = scale * X^T[K,M] (kept blocks) . dY[M,N]: A = X^T, B = dY^T, C = dW^T, lists of the transposed mask
    SD_REQUIRE(col_ptr && row_idx, "dropout_matmul_backward: dW needs the CSC lists");
    if (int rc = sd_gemm_dsd_lists(X, xsc, xsr, dY, gsc, gsr, dW, dwsc, dwsr, col_ptr, row_idx, K, N, M, g, scale, dtype,
                                   workspace, workspace_bytes, stream))
      return rc;
  }
  return SD_OK;
}

int sd_im2col(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t sw, void* cols, int64_t ld,
              int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
              int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
              const int32_t* row_ptr, const int32_t* col_idx, int64_t bs, int dtype, void* stream) {
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  return im2col(x, sn, sc, sh, sw, cols, ld, n, c, h, w, r, s, pad_h, pad_w, stride_h, stride_w, dil_h,
                dil_w, row_ptr, col_idx, bs, (hipStream_t)stream);
}

int sd_col2im(const void* cols, int64_t ld, void* dx, int64_t sn, int64_t sc, int64_t sh, int64_t sw,
              int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s, int64_t pad_h,
              int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
              const uint8_t* mask, int64_t msr, int64_t msc, int64_t bs, int dtype, void* stream) {
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  return col2im(cols, ld, dx, sn, sc, sh, sw, n, c, h, w, r, s, pad_h, pad_w, stride_h, stride_w, dil_h,
                dil_w, mask, msr, msc, bs, dtype, (hipStream_t)stream);
}

int sd_conv2d_dsd_lists(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t sw, const void* weight,
                        int64_t wld, void* y, int64_t yld, int64_t n, int64_t c, int64_t h, int64_t w,
                        int64_t k_out, int64_t r, int64_t s, int64_t pad_h, int64_t pad_w, int64_t stride_h,
                        int64_t stride_w, int64_t dil_h, int64_t dil_w, const int32_t* row_ptr,
                        const int32_t* col_idx, int64_t bs, float scale, int dtype, void* stream) {
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  SD_REQUIRE(x && weight && y, "null pointer argument");
  SD_REQUIRE((row_ptr == nullptr) == (col_idx == nullptr), "row_ptr and col_idx must both be given or both be null");
  SD_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && k_out > 0 && r > 0 && s > 0, "sizes must be positive");
  SD_REQUIRE(stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0 && pad_h >= 0 && pad_w >= 0,
             "strides and dilations must be positive, paddings non-negative");
  if (row_ptr) {
    if (int rc = check_sparse(bs, scale)) return rc;
  } else {
    SD_REQUIRE(scale == scale, "scale is NaN");
    bs = 64;
  }
  const int64_t P = (h + 2 * pad_h - dil_h * (r - 1) - 1) / stride_h + 1;
  const int64_t Q = (w + 2 * pad_w - dil_w * (s - 1) - 1) / stride_w + 1;
  SD_REQUIRE(P > 0 && Q > 0, "the kernel does not fit the padded input");
  SD_REQUIRE(wld >= c * r * s && yld >= k_out, "leading dimensions too small");
  if (bs != 64 || Q > 64 || 64 % Q != 0 || c * r * s > (1 << 16) || h > (1 << 20) || w > (1 << 12) || r > 64 || s > 64 ||
      stride_h > 8 || stride_w > 8 || dil_h > 8 || dil_w > 8)
    return SD_ERR_UNSUPPORTED;
  // a workgroup's 256 output positions: 4 * 64 / Q consecutive rows of one image where P * Q allows, else four
  // separate 64-position blocks
  const bool one_run = (P * Q) % 256 == 0;
  ImplicitConv cg = conv_geometry(x, sn, sc, sh, c, h, w, P, Q, r, s, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w,
                                  /*blocks=*/one_run ? 4 : 1);
  cg.units = one_run ? 1 : 4;
  GemmArgs g = make_args(nullptr, 0, 0, weight, wld, 1, y, yld, 1, n * P * Q, k_out, c * r * s, bs, scale, row_ptr,
                         col_idx);
  const int rc = launch_conv_implicit(g, cg, P, stride_h, stride_w, dil_h, dil_w, r, sw, dtype, (hipStream_t)stream);
  if (rc == SD_OK) last_kernel = "specialised";
  return rc;
}

int sd_conv2d_dx(const void* dy, int64_t dy_ld, const void* weight, int64_t weight_ld, void* dx, int64_t sn,
                 int64_t sc, int64_t sh, int64_t sw, const uint8_t* mask, int64_t msr, int64_t msc, int64_t n,
                 int64_t c, int64_t h, int64_t w, int64_t k_out, int64_t r, int64_t s, int64_t pad_h, int64_t pad_w,
                 int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w, int64_t bs, float scale, int dtype,
                 void* stream) {
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  SD_REQUIRE(dy && weight && dx, "null pointer argument");
  SD_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && k_out > 0 && r > 0 && s > 0, "sizes must be positive");
  SD_REQUIRE(stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0 && pad_h >= 0 && pad_w >= 0,
             "strides and dilations must be positive, paddings non-negative");
  SD_REQUIRE(scale == scale, "scale is NaN");
  if (mask != nullptr && bs != 64) return SD_ERR_UNSUPPORTED;
  if (h > (1 << 20) || w > (1 << 12) || c * r * s > (1 << 16)) return SD_ERR_UNSUPPORTED;
  const int rc = launch_conv_dx(dy, dy_ld, weight, weight_ld, dx, sn, sc, sh, sw, mask, msr, msc, n, c, h, w, k_out, r,
                                s, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, scale, dtype, (hipStream_t)stream);
  if (rc == SD_OK) last_kernel = "specialised";
  return rc;
}

int64_t sd_conv2d_dw_workspace_bytes(int64_t n, int64_t c, int64_t k_out, int64_t r, int64_t s, int64_t p, int64_t q) {
  if (n <= 0 || c <= 0 || k_out <= 0 || r <= 0 || s <= 0 || p <= 0 || q <= 0) return 0;
  const int64_t rows = c * r * s;
  const int splits = conv_dw_splits(rows, k_out, n * p * q);
  return splits > 1 ? (int64_t)splits * rows * k_out * 4 : 0;
}

int sd_conv2d_dw_lists(const void* x, int64_t sn, int64_t sc, int64_t sh, int64_t sw, const void* dy, int64_t dyld,
                       void* dw, int64_t dwld, int64_t n, int64_t c, int64_t h, int64_t w, int64_t k_out, int64_t r,
                       int64_t s, int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h,
                       int64_t dil_w, const int32_t* col_ptr, const int32_t* row_idx, int64_t bs, float scale,
                       int dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  SD_REQUIRE(dtype == SD_F16 || dtype == SD_BF16, "dtype must be SD_F16 or SD_BF16 (got %d)", dtype);
  SD_REQUIRE(x && dy && dw, "null pointer argument");
  SD_REQUIRE((col_ptr == nullptr) == (row_idx == nullptr), "col_ptr and row_idx must both be given or both be null");
  SD_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && k_out > 0 && r > 0 && s > 0, "sizes must be positive");
  SD_REQUIRE(stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0 && pad_h >= 0 && pad_w >= 0,
             "strides and dilations must be positive, paddings non-negative");
  if (col_ptr) {
    if (int rc = check_sparse(bs, scale)) return rc;
  } else {
    SD_REQUIRE(scale == scale, "scale is NaN");
    bs = 64;
  }
  const int64_t P = (h + 2 * pad_h - dil_h * (r - 1) - 1) / stride_h + 1;
  const int64_t Q = (w + 2 * pad_w - dil_w * (s - 1) - 1) / stride_w + 1;
  SD_REQUIRE(P > 0 && Q > 0, "the kernel does not fit the padded input");
  SD_REQUIRE(dyld >= k_out && dwld >= c * r * s, "leading dimensions too small");
  if (bs != 64 || Q > 64 || 64 % Q != 0 || c * r * s > (1 << 16) || h > (1 << 20) || w > (1 << 12) || r > 64 || s > 64 ||
      stride_h > 8 || stride_w > 8 || dil_h > 8 || dil_w > 8)
    return SD_ERR_UNSUPPORTED;
  ImplicitConv cg = conv_geometry(x, sn, sc, sh, c, h, w, P, Q, r, s, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w,
                                  /*blocks=*/1);
  GemmArgs g = make_args(nullptr, 1, c * r * s, dy, 1, dyld, dw, 1, dwld, c * r * s, k_out, n * P * Q, bs, scale,
                         col_ptr, row_idx, workspace, workspace_bytes);
  const int rc = launch_conv_implicit_dw(g, cg, P, stride_h, stride_w, dil_h, dil_w, r, sw, dtype, (hipStream_t)stream);
  if (rc == SD_OK) last_kernel = "specialised";
  return rc;
}

}  // extern "C"
