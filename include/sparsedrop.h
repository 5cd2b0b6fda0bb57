/*
 * libsparsedrop — C ABI of the MI355X (gfx950) SparseDrop kernels.
 *
 * Block-wise dropout fused into the following matmul: one Bernoulli per block_size x block_size
 * tile of the activation matrix X[M,K]; dropped tiles are never loaded or multiplied.
 *
 *     Y  = s * (keep (.) X) * W^T        "DSD"  (dense = sparse x dense)      s = 1/(1-p)
 *     dX = s * (dY * W) (.) keep         "SDD"  (sparse = dense x dense)
 *     dW = s * dY^T * (keep (.) X)       "DSD"  on transposed operands
 *
 * This header replaces, entry point for entry point, the pybind11 module "gemm" of the reference
 * (flash_dropout/cuda/src/gemm_binding.cu:137-141) and the Python shim that loads it
 * (flash_dropout/cuda/binding_gemm.py:26-47).  Everything is plain pointers and sizes:
 * no torch types cross this boundary.
 *
 * Conventions (all entry points)
 *   - Every pointer is a DEVICE pointer on the current HIP device, unless stated otherwise.
 *   - A matrix is (ptr, stride_r, stride_c) in ELEMENTS; like the reference's check_operand
 *     (gemm_binding.cu:18-22) one of the two strides must be 1 (row- or column-major).  The
 *     reference derives this from the tensor strides (gemm_binding.cu:90-92); here the caller
 *     passes the strides themselves.
 *   - "B" operands are [N, K]: out-features x reduction, as in the reference (gemm_binding.cu:56-69).
 *   - mask is one byte per block, non-zero = DROPPED (flash_dropout/functional/utils.py:15),
 *     with its own two strides in bytes.
 *   - dtype: SD_F16 or SD_BF16 for A, B and C; accumulation is always fp32 and the scale is applied
 *     to the fp32 accumulator before the single rounding at the store (gemm.cuh:55-66).
 *   - stream is a hipStream_t passed as void* (NULL = the null stream).  All work is enqueued on it
 *     and the call returns without synchronising.  The reference launches on the legacy default
 *     stream (matmul_dsd.cuh:105); callers pass torch's current stream instead.
 *   - Return value: SD_OK, or an error code with the reason in sd_last_error() (thread-local).
 *     Shapes and strides are always validated on the host (the reference only has assert()s,
 *     matmul_dsd.cuh:79-95).  The library allocates no device memory; workspaces are the caller's.
 *   - Supported block sizes: multiples of 32.  M, N, K are arbitrary (edge tiles are predicated);
 *     the mask has ceil(M/block_size) x ceil(K/block_size) entries.  The kernels work on 64 x 64 tiles: a multiple
 *     of 64 is listed with every mask entry repeated, and an odd multiple of 32 (32, 96, 160, ...) on the grid of its
 *     32-blocks merged two by two, a list entry remembering which of its 32 x 32 quadrants are kept (the report's
 *     block splitting, report.pdf
 *     section 3.3, in both directions; the reference's Triton path takes any block size divisible by its tile,
 *     flash_dropout/triton/utils.py:6-19, its CUDA path only 128, matmul_dsd.cuh:92-93).
 */
#ifndef SPARSEDROP_H_
#define SPARSEDROP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum sd_status {
  SD_OK = 0,
  SD_ERR_INVALID = 1,     /* bad shape / stride / pointer / argument */
  SD_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for */
  SD_ERR_RUNTIME = 3      /* HIP launch or runtime failure */
};

enum sd_dtype { SD_F16 = 0, SD_BF16 = 1 };

/* activations the GEMM epilogues can apply; GELU is the exact (erf) form, torch.nn.GELU's default */
enum sd_act { SD_ACT_NONE = 0, SD_ACT_RELU = 1, SD_ACT_GELU = 2 };

/* Library version (major*10000 + minor*100 + patch). No reference counterpart. */
int sd_version(void);

/* Message of the last failing call on this thread ("" if none).  Replaces the TORCH_CHECK
 * exceptions of gemm_binding.cu:18-22,87-89. */
const char* sd_last_error(void);

/* Which GEMM kernel family the calling thread's last sd_gemm* call ran on: "specialised" (the tiled
 * kernels for 64-blocks and aligned operands) or "generic" (any shape and layout, several times slower
 * per FLOP); "" before the first call.  For tests and for callers who want to know whether a shape is on
 * the fast path.  No counterpart in the reference. */
const char* sd_last_kernel(void);

/* What that call ran on, in more detail: kernel family, workgroup shape and reduction splits, e.g. "dsd:big splits=1",
 * "dsd:mid:strided:ragged splits=4", "sdd:mid", "sdd:small" (shapes: 256 x 256 / 128 x 128 output tiles for DSD, 4 / 2 / 2
 * row blocks by column groups of up to 6 / 4 / 2 blocks for SDD), "generic", "conv_fwd:implicit:rows-per-step", "conv_dw:implicit
 * splits=85", "conv_dx:fused".  The conv entry points that return SD_ERR_UNSUPPORTED leave it unchanged (the caller's
 * explicit route then shows its own GEMM here).  Diagnostic text, not a stable format. */
const char* sd_last_kernel_detail(void);

/* Hash of the source files the library was built from (written by csrc/build.py); the Python loader compares it
 * with the tree next to it and refuses a stale library.  No counterpart in the reference. */
const char* sd_source_hash(void);

/* The workgroup-to-tile map of the specialised kernels, evaluated on the host: launch index `block` of a
 * tiles_m x tiles_n grid -> (tile_m, tile_n); kind 0 = DSD / dense order, 1 = SDD order.  The hardware deals
 * consecutive workgroup ids round-robin to the 8 XCDs; the map gives each XCD a compact patch of the grid.  It
 * must be a bijection onto the grid, which tests check through this entry point; the reference's counterpart is
 * threadblock_swizzle (flash_dropout/cuda/src/gemm.cuh:84-97). */
int sd_tile_of_block(int kind, int64_t block, int64_t tiles_m, int64_t tiles_n, int32_t* tile_m, int32_t* tile_n);

/* Workgroup shape of the specialised DSD / dense kernels: SD_TILE_AUTO picks from the shape (256 x 256
 * output tiles when there are more than 128 of them, 128 x 128 otherwise; the SDD kernel's group shape follows the
 * same rule), the other two
 * force one shape for every later call of the process (SD_TILE_BIG also makes sd_conv2d_dsd_lists keep one
 * LDS copy of all channels' input rows instead of a copy per step where both fit).  Returns the previous setting, -1 for an unknown
 * value.  A tuning and test hook, process-global and not thread-safe against concurrent GEMM calls (a call that
 * races with it runs with either shape); not for production use.  Results do not depend on it beyond fp32 summation order.  No
 * counterpart in the reference (its tile is a compile-time GemmConfig, gemm_configs/gemm_config.cuh:19-100). */
#define SD_TILE_AUTO 0
#define SD_TILE_BIG 1
#define SD_TILE_MID 2
int sd_set_tile_policy(int policy);

/* ---------------------------------------------------------------------------------------------
 * (a) block-mask -> compacted kept-block lists
 *
 * Replaces the torch ops of flash_dropout/functional/utils.py:57-60 (row widths, cumsum, nonzero)
 * and torch.nonzero(~mask) of flash_dropout/functional/blockwise_dropout_matmul_triton.py:48,
 * without the device->host synchronisation those imply.
 *
 *   CSR: row_ptr[mb+1], col_idx[capacity mb*kb]; kept column blocks of row r, ascending, are
 *        col_idx[row_ptr[r] .. row_ptr[r+1]).  col_idx[0..nnz) equals nonzero(~mask)[:,1].
 *   CSC: col_ptr[kb+1], row_idx[capacity mb*kb]; kept row blocks of column c, ascending.
 * Either pair may be NULL (both NULL is an error).  Entries past nnz are left untouched.
 * ------------------------------------------------------------------------------------------- */
int sd_build_lists(const uint8_t* mask, int64_t mb, int64_t kb, int64_t mask_stride_r,
                   int64_t mask_stride_c, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                   int32_t* row_idx, void* stream);

/* Block splitting.  split == 0: the mask is at block size 32, HALF the 64 the lists are over: out_mb = ceil(mb / 2),
 * out_kb = ceil(kb / 2), a list entry is kept when any of the (up to) four mask entries it covers is, and bits 28-31 of
 * the entry say which: bit 2a + b = mask entry (2i + a, 2j + b) kept (row_idx, the list by columns, stores them as the
 * list of the transposed mask needs them: halves swapped).  The *_lists entry points take such lists when called with
 * block_size 32: the 64 x 64 tile of a kept entry is computed and its dropped quadrants contribute / come out as zeros.
 * split == -k (k = 3, 5, ...; -1 is the same as 0): the mask is at block size 32 * k; its entries are repeated k x k
 * times onto the grid of 32-blocks and that grid is merged two by two as above.  out_mb x out_kb is the grid of
 * 64-blocks of the masked matrix, ceil(M / 64) x ceil(K / 64): it must end inside the mask's last row and column of
 * entries, (mb - 1) * k < 2 * out_mb and out_mb <= ceil(mb * k / 2).  A 32-block past the end of the matrix but inside
 * the mask's last entry counts as kept when that entry is (nothing of it is ever loaded or stored).
 * split >= 1: the same lists for the mask with every entry repeated split x split times, cropped
 * to out_mb x out_kb ((mb-1)*split < out_mb <= mb*split, likewise out_kb); capacities out_mb*out_kb.
 * A mask drawn at block size 64*split over an [M,K] operand is listed with out_mb = ceil(M/64),
 * out_kb = ceil(K/64) and then drives the 64-block kernels (block_size 64 in the *_lists calls), which
 * compute the same product: the repeated mask expands to the same element mask
 * (flash_dropout/functional/naive.py:18-23 zeroes whole block_size x block_size tiles).  The reference
 * fixes block_size = 128 = its tile (matmul_dsd.cuh:92-93) and has no counterpart. */
int sd_build_lists_split(const uint8_t* mask, int64_t mb, int64_t kb, int64_t mask_stride_r,
                         int64_t mask_stride_c, int64_t split, int64_t out_mb, int64_t out_kb,
                         int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                         void* stream);

/* Draws the mask on the device and lists it in the same launch: replaces
 * blockwise_dropout_mask, flash_dropout/functional/utils.py:11-16 (torch.rand(mb, kb) < p, True =
 * dropped) followed by the compaction above.  Entry e = i*kb + j is dropped iff
 * (w >> 8) * 2^-24 < p (compared in fp32), w = word e%4 of Philox4x32-10 with counter
 * (lo32(e/4), hi32(e/4), lo32(offset), hi32(offset)) and key (lo32(seed), hi32(seed)): a pure function
 * of (seed, offset, e), not torch's generator stream.  mask_out receives the mb x kb mask as row-major
 * bytes (the autograd context and parity tests keep it); split / out_mb / out_kb as above (split 0 included). */
int sd_random_lists(uint64_t seed, uint64_t offset, float p, int64_t mb, int64_t kb, uint8_t* mask_out,
                    int64_t split, int64_t out_mb, int64_t out_kb, int32_t* row_ptr, int32_t* col_idx,
                    int32_t* col_ptr, int32_t* row_idx, void* stream);

/* The same draw keyed by device memory: state is a device pointer to four uint64 {seed, offset, 0, 0}; the
 * kernels read seed and offset from there and add 1 to the offset once every workgroup has read them (the
 * third word counts workgroups while a call runs and is zero again when it ends; the fourth is unused), all
 * on `stream`, without a memset and for masks of up to 2^18 entries without an extra launch.
 * Nothing about the draw is baked into the launch arguments, so a captured HIP graph that contains this
 * call draws a new mask at every replay (with sd_random_lists the seed is a launch argument and a replay
 * would repeat the mask).  The reference has no counterpart: its mask comes from torch.rand on torch's
 * generator (flash_dropout/functional/utils.py:15), which torch itself makes graph-safe the same way. */
int sd_random_lists_state(uint64_t* state, float p, int64_t mb, int64_t kb, uint8_t* mask_out, int64_t split,
                          int64_t out_mb, int64_t out_kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                          int32_t* row_idx, void* stream);

/* Pointer-increment table of flash_dropout/functional/utils.py:19-69 from a CSR list:
 * table[i] = col_idx[i]*block_k for the first kept block of a row, else (col_idx[i]-col_idx[i-1])*block_k;
 * row_indices[r] = row_ptr[r]; row_widths[r] = row_ptr[r+1]-row_ptr[r].
 * table has capacity >= nnz (mb*kb is always enough). */
int sd_increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                       int64_t* table, int64_t* row_indices, int64_t* row_widths, void* stream);

/* Bytes of workspace the mask-taking GEMM entry points need for an mb x kb mask.  For a block size that
 * is a larger multiple of 64, a workspace sized for the 64-granular grid instead
 * (sd_workspace_bytes(ceil(rows/64), ceil(cols/64)) of the masked matrix) makes them split the mask and
 * run the 64-block kernels; the smaller size is accepted and runs the generic kernel. */
int64_t sd_workspace_bytes(int64_t mb, int64_t kb);

/* Optional split-K scratch.  When the output has too few tiles to fill the GPU and the reduction is long
 * (the weight gradient of a tall activation matrix), sd_gemm and the DSD entry points split the reduction
 * over several workgroups and need fp32 scratch for the partial tiles: this returns how many bytes
 * (0 = no split wanted) for C[M,N] with reduction length K; sparse = 0 for sd_gemm, 1 for DSD.
 * Passing less (or NULL) is always allowed and only costs speed.  The mask-taking sd_gemm_dsd takes it
 * appended to its list workspace: workspace_bytes >= round16(sd_workspace_bytes) + this.
 * No counterpart in the reference (its kernels never split the reduction). */
int64_t sd_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t block_size, int sparse);

/* ---------------------------------------------------------------------------------------------
 * dense C[M,N] = A[M,K] * B[N,K]^T            replaces gemm()      gemm_binding.cu:47-54
 * ------------------------------------------------------------------------------------------- */
int sd_gemm(const void* A, int64_t a_stride_r, int64_t a_stride_c,
            const void* B, int64_t b_stride_r, int64_t b_stride_c,
            void* C, int64_t c_stride_r, int64_t c_stride_c,
            int64_t M, int64_t N, int64_t K, int dtype,
            void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (b)/(d) DSD: C[M,N] = scale * sum over kept K-blocks of A's row-block of A_blk * B_blk^T
 *         mask is [ceil(M/bs), ceil(K/bs)] over A.            replaces gemm_dsd()  gemm_binding.cu:82-94
 * (c)     SDD: C tile = scale * A * B^T where kept, exactly 0 where dropped
 *         mask is [ceil(M/bs), ceil(N/bs)] over C.            replaces gemm_sdd()  gemm_binding.cu:122-135
 *
 * The *_lists forms take the CSR list of the same mask (built once by sd_build_lists and shared by
 * forward and backward); the mask forms build it into `workspace` (>= sd_workspace_bytes) on `stream`
 * first.  For the weight gradient call sd_gemm_dsd*(X^T, dY^T, mask^T) exactly as
 * flash_dropout/functional/blockwise_dropout_matmul_cuda.py:49-51 does — with the CSC list of the
 * forward mask as the CSR list of mask^T — and pass C strides (1, ldc) to get dW[N,K] row-major
 * directly instead of a transposed view.
 * ------------------------------------------------------------------------------------------- */
int sd_gemm_dsd(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                const void* B, int64_t b_stride_r, int64_t b_stride_c,
                void* C, int64_t c_stride_r, int64_t c_stride_c,
                const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                void* workspace, int64_t workspace_bytes, void* stream);

int sd_gemm_sdd(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                const void* B, int64_t b_stride_r, int64_t b_stride_c,
                void* C, int64_t c_stride_r, int64_t c_stride_c,
                const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                void* workspace, int64_t workspace_bytes, void* stream);

/* sd_gemm_dsd without a workspace argument and without any allocation: the kept-block list is built into an
 * array in device memory that is part of the library image (SD_NOALLOC_SCRATCH_BYTES; every GPU the library is
 * used on holds its own copy until the process ends).  No counterpart in the reference; it is for callers that
 * cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, results and errors as sd_gemm_dsd otherwise, except that the reduction is never
 * split over workgroups (there is no scratch for partial tiles).  Limits: round16(sd_workspace_bytes(grid)) of
 * the 64-granular block grid must fit the array, i.e. about 2^18 mask blocks (a 32768 x 32768 operand at block
 * size 64); larger operands return SD_ERR_INVALID and launch nothing.  Nothing in the array has to start at
 * zero (the list builder writes every entry the product reads), but all calls on one GPU share it: calls that
 * overlap on one GPU (two streams, two host threads) race on the list and must be serialised by the caller.
 * First use: the first call on a device looks the array's address up and raises the LDS limit of the kernels it
 * launches (runtime calls that are not stream operations), so a caller that captures a graph makes one call with the
 * same shapes and block size on that device BEFORE the capture begins; every later call, captured or not, issues
 * nothing but kernel launches on `stream`. */
#define SD_NOALLOC_SCRATCH_BYTES 1114112 /* 16-byte padded row_ptr of up to 16383 row blocks + 2^18 int32 */
int64_t sd_noalloc_scratch_bytes(void);
int sd_gemm_dsd_noalloc(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                        const void* B, int64_t b_stride_r, int64_t b_stride_c,
                        void* C, int64_t c_stride_r, int64_t c_stride_c,
                        const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                        int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                        void* stream);

int sd_gemm_dsd_lists(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                      const void* B, int64_t b_stride_r, int64_t b_stride_c,
                      void* C, int64_t c_stride_r, int64_t c_stride_c,
                      const int32_t* row_ptr, const int32_t* col_idx,
                      int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                      void* workspace, int64_t workspace_bytes, void* stream);

int sd_gemm_sdd_lists(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                      const void* B, int64_t b_stride_r, int64_t b_stride_c,
                      void* C, int64_t c_stride_r, int64_t c_stride_c,
                      const int32_t* row_ptr, const int32_t* col_idx,
                      int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                      void* stream);

/* sd_gemm_sdd_lists with its options spelled out.  kept_only != 0: as sd_gemm_sdd_lists_kept below.  keep_hint: the
 * caller's estimate of the fraction of blocks kept (1 - p), or negative for unknown; the lists live on the device,
 * so this is all the host has to choose the workgroup shape by (it counts the workgroups the large shape would
 * have; unknown counts as everything kept).  It never changes results.  `scale` plays no part in that choice. */
int sd_gemm_sdd_lists_ex(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                         const void* B, int64_t b_stride_r, int64_t b_stride_c,
                         void* C, int64_t c_stride_r, int64_t c_stride_c,
                         const int32_t* row_ptr, const int32_t* col_idx,
                         int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                         int kept_only, float keep_hint, void* stream);

/* The two products with the activation that sits between dropout-linear layers fused into their stores (the
 * reference's models interleave exactly these: eval/mlp/model.py:21-28 DropoutMM, ReLU, DropoutMM, ...;
 * eval/llm/model.py:58-60 Linear, GELU, DropoutMM; its kernels have no epilogue, gemm.cuh:55-66):
 *   sd_gemm_dsd_lists_act:      C = act(v), v = scale * sum over kept blocks, applied to the fp32 accumulator before
 *                               the one rounding; pre_out (NULL, or a matrix of C's shape with its own strides)
 *                               receives v itself, which the GELU backward needs.
 *   sd_gemm_sdd_lists_actgrad:  C = v * act'(act_at[m, n]) where kept, exactly 0 where dropped: the input gradient
 *                               of a layer whose input was act(act_at), i.e. the gradient with respect to the
 *                               previous layer's pre-activation.  For ReLU act_at may be the activated tensor itself
 *                               (same sign).  act_at has C's shape and its own strides.
 * act = SD_ACT_NONE makes them sd_gemm_dsd_lists / sd_gemm_sdd_lists_ex. */
int sd_gemm_dsd_lists_act(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                          const void* B, int64_t b_stride_r, int64_t b_stride_c,
                          void* C, int64_t c_stride_r, int64_t c_stride_c,
                          const int32_t* row_ptr, const int32_t* col_idx,
                          int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                          int act, void* pre_out, int64_t pre_stride_r, int64_t pre_stride_c,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* The dense product with the same fused store, C = act(A . B^T) (and the pre-activation to pre_out when given): a
 * layer without dropout inside a stack that fuses its activations (the reference's first layer, eval/mlp/model.py:
 * 31-33, has p = 0).  B must have a contiguous reduction index when act != SD_ACT_NONE. */
int sd_gemm_act(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                const void* B, int64_t b_stride_r, int64_t b_stride_c,
                void* C, int64_t c_stride_r, int64_t c_stride_c,
                int64_t M, int64_t N, int64_t K, int dtype, int act,
                void* pre_out, int64_t pre_stride_r, int64_t pre_stride_c,
                void* workspace, int64_t workspace_bytes, void* stream);

int sd_gemm_sdd_lists_actgrad(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                              const void* B, int64_t b_stride_r, int64_t b_stride_c,
                              void* C, int64_t c_stride_r, int64_t c_stride_c,
                              const int32_t* row_ptr, const int32_t* col_idx,
                              int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                              int act, const void* act_at, int64_t at_stride_r, int64_t at_stride_c,
                              float keep_hint, void* stream);

/* sd_gemm_sdd_lists for a consumer that reads kept tiles only (sd_col2im with the same mask does): the
 * dropped tiles of C are left untouched instead of being written as zeros, which for half of a large C
 * dropped is a third of the call's memory traffic.  The reference always writes them
 * (matmul_sdd.cuh:44-65); no counterpart there. */
int sd_gemm_sdd_lists_kept(const void* A, int64_t a_stride_r, int64_t a_stride_c,
                           const void* B, int64_t b_stride_r, int64_t b_stride_c,
                           void* C, int64_t c_stride_r, int64_t c_stride_c,
                           const int32_t* row_ptr, const int32_t* col_idx,
                           int64_t M, int64_t N, int64_t K, int64_t block_size, float scale, int dtype,
                           void* stream);

/* ---------------------------------------------------------------------------------------------
 * The reference's autograd function in two calls (one launch path each instead of two), for small layers whose
 * step time is the host's launch path.
 *
 * sd_dropout_matmul_forward = BlockwiseDropoutMatmulCUDA.forward,
 * flash_dropout/functional/blockwise_dropout_matmul_cuda.py:10-32: the block mask (given: `mask`, [ceil(M/bs),
 * ceil(K/bs)] bytes with strides, non-zero = dropped; or drawn with probability p: from the device-resident state
 * `rng_state` as sd_random_lists_state does, or, when that is NULL too, from (seed, offset) as sd_random_lists does;
 * a drawn mask is stored to mask_out), its kept-block lists, and Y = (keep . X) / (1 - p) . W^T.  The lists are left
 * in the caller's arrays for the backward call; they are built at the granularity the kernels run at:
 * g = 64 when block_size is a multiple of 64 (else block_size), i.e. row_ptr[ceil(M/g) + 1], col_idx[ceil(M/g) *
 * ceil(K/g)], col_ptr[ceil(K/g) + 1], row_idx[same capacity]; the CSC pair may be NULL when no weight gradient
 * will be asked for.  workspace: optional split-reduction scratch (sd_splitk_workspace_bytes(M, N, K, g, 1)).
 *
 * sd_dropout_matmul_backward = BlockwiseDropoutMatmulCUDA.backward, same file :36-53: dX = (dY . W) . keep / (1 - p)
 * (written in full, zeros where dropped) and dW = dY^T . (keep . X) / (1 - p), each skipped when its pointer is NULL.
 * dW is written through its own strides: pass a row-major [N, K] tensor to get what the reference returns as a
 * transposed view.  workspace: optional split-reduction scratch for dW (sd_splitk_workspace_bytes(K, N, M, g, 1)).
 *
 * p is a double in these calls: the products are scaled by (float)(1 / (1 - p)) evaluated in double precision, which
 * is the number the reference's Python passes to its kernels (blockwise_dropout_matmul_cuda.py:29), and the draw
 * compares against (float)p as sd_random_lists does.
 * ------------------------------------------------------------------------------------------- */
int sd_dropout_matmul_forward(const void* X, int64_t x_stride_r, int64_t x_stride_c,
                              const void* W, int64_t w_stride_r, int64_t w_stride_c,
                              void* Y, int64_t y_stride_r, int64_t y_stride_c,
                              const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                              uint64_t* rng_state, uint64_t seed, uint64_t offset, double p, uint8_t* mask_out,
                              int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                              int64_t M, int64_t N, int64_t K, int64_t block_size, int dtype,
                              void* workspace, int64_t workspace_bytes, void* stream);

int sd_dropout_matmul_backward(const void* dY, int64_t dy_stride_r, int64_t dy_stride_c,
                               const void* W, int64_t w_stride_r, int64_t w_stride_c,
                               const void* X, int64_t x_stride_r, int64_t x_stride_c,
                               void* dX, int64_t dx_stride_r, int64_t dx_stride_c,
                               void* dW, int64_t dw_stride_r, int64_t dw_stride_c,
                               const int32_t* row_ptr, const int32_t* col_idx,
                               const int32_t* col_ptr, const int32_t* row_idx,
                               int64_t M, int64_t N, int64_t K, int64_t block_size, double p, int dtype,
                               void* workspace, int64_t workspace_bytes, void* stream);

/* The same with the derivative of an activation multiplied into dX (sd_gemm_sdd_lists_actgrad's epilogue):
 * dX = (dY . W) . keep / (1 - p) * act'(act_at[m, k]), for a layer whose input is act(previous layer's output);
 * act = SD_ACT_NONE is the plain call.  No counterpart in the reference, whose layers run the activation gradient as a
 * kernel of its own.
 * Where both gradients are asked for and neither product would fill the chip by itself (at most 512 workgroups each,
 * both on the same workgroup shape), the two run as ONE launch - the weight gradient's workgroups follow the input
 * gradient's in the same grid - so small layers pay for one launch and run the two side by side.
 * SPARSEDROP_SEPARATE_BACKWARD=1 in the environment keeps them apart (for comparing). */
int sd_dropout_matmul_backward_act(const void* dY, int64_t dy_stride_r, int64_t dy_stride_c,
                                   const void* W, int64_t w_stride_r, int64_t w_stride_c,
                                   const void* X, int64_t x_stride_r, int64_t x_stride_c,
                                   void* dX, int64_t dx_stride_r, int64_t dx_stride_c,
                                   void* dW, int64_t dw_stride_r, int64_t dw_stride_c,
                                   const int32_t* row_ptr, const int32_t* col_idx,
                                   const int32_t* col_ptr, const int32_t* row_idx,
                                   int64_t M, int64_t N, int64_t K, int64_t block_size, double p, int dtype,
                                   int act, const void* act_at, int64_t at_stride_r, int64_t at_stride_c,
                                   void* workspace, int64_t workspace_bytes, void* stream);

/* sd_dropout_matmul_forward with an activation in the product's store (sd_gemm_dsd_lists_act's epilogue):
 * Y = act((keep . X) / (1 - p) . W^T), the value before the activation to pre_out when that is given; act = SD_ACT_NONE
 * is the plain call.  No counterpart in the reference, whose layers run the activation as a kernel of its own.
 * Where the product is small (at most 512 workgroups) and its mask has at most 2^18 entries on the 64 grid, the mask
 * draw, both lists and the product run as ONE launch: the product's workgroups evaluate the keep bits of their own
 * row blocks from the mask source, other workgroups of the same grid write the lists the backward reads.
 * SPARSEDROP_SEPARATE_FORWARD=1 in the environment keeps the list build a launch of its own (for comparing). */
int sd_dropout_matmul_forward_act(const void* X, int64_t x_stride_r, int64_t x_stride_c,
                                  const void* W, int64_t w_stride_r, int64_t w_stride_c,
                                  void* Y, int64_t y_stride_r, int64_t y_stride_c,
                                  const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                                  uint64_t* rng_state, uint64_t seed, uint64_t offset, double p, uint8_t* mask_out,
                                  int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                                  int64_t M, int64_t N, int64_t K, int64_t block_size, int dtype,
                                  int act, void* pre_out, int64_t pre_stride_r, int64_t pre_stride_c,
                                  void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (e) im2col gather feeding the same GEMMs for conv.
 *
 * cols[(n*P+p)*Q+q, c*R*S + r*S + s] = x[n, c, p*stride_h + r*dil_h - pad_h, q*stride_w + s*dil_w - pad_w]
 * (zero outside the image): the matrix F.unfold(...).permute(0,2,1) of
 * flash_dropout/functional/im2col_conv2d.py:17-20, materialised row-major [N*P*Q, C*R*S] (ld = cols_ld).
 * x is addressed by four element strides, so NCHW and channels-last both work (the reference's dead
 * kernel, flash_dropout/cuda/src/im2col.cuh:21-72, was channels-last only with (r,s,c) columns).
 * With a CSR list (row_ptr/col_idx over the [ceil(NPQ/bs), ceil(CRS/bs)] block mask) only kept blocks
 * are written; dropped blocks are left untouched (the DSD kernels never read them).  NULL lists = all.
 *
 * sd_col2im is the adjoint (dx[n,c,h,w] = sum of every cols entry that im2col filled from that pixel;
 * dx is fully overwritten): the backward of the gather.  With a mask (one byte per block of cols,
 * non-zero = dropped, strides in bytes) dropped blocks are not read and count as zero; NULL = read all.
 * ------------------------------------------------------------------------------------------- */
int sd_im2col(const void* x, int64_t x_stride_n, int64_t x_stride_c, int64_t x_stride_h,
              int64_t x_stride_w, void* cols, int64_t cols_ld,
              int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s,
              int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w,
              int64_t dil_h, int64_t dil_w,
              const int32_t* row_ptr, const int32_t* col_idx, int64_t block_size,
              int dtype, void* stream);

int sd_col2im(const void* cols, int64_t cols_ld, void* dx, int64_t dx_stride_n,
              int64_t dx_stride_c, int64_t dx_stride_h, int64_t dx_stride_w,
              int64_t n, int64_t c, int64_t h, int64_t w, int64_t r, int64_t s,
              int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w,
              int64_t dil_h, int64_t dil_w,
              const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c, int64_t block_size,
              int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Implicit-GEMM forward of the block-dropout convolution: the product sd_im2col + sd_gemm_dsd_lists
 * compute, y[(n*P+p)*Q+q, k] = scale * sum over the kept blocks (row_ptr/col_idx, block_size 64, over the
 * [N*P*Q / 64, ceil(C*R*S / 64)] grid of the patch matrix) of cols[m, j] * weight[k, j], without the patch
 * matrix ever existing in memory: each workgroup keeps the input rows its 256 output positions touch in LDS
 * and builds the kept 64 x 64 patch tiles from them.  weight is the [k_out, C*R*S] matrix (the kernel
 * viewed as in flash_dropout/functional/im2col_conv2d.py:21-24), y is [N*P*Q, k_out] row-major with
 * leading dimension y_ld.  This is what report.pdf section 5.3 proposes as future work; the reference has
 * no counterpart (its conv variants are stubs, layers/dropout_conv.py:86-99).
 *
 * Taken: strides and dilations up to 8, unit w stride of x, W a multiple of 8, Q a divisor of 64, P*Q a multiple of
 * 64, C*R*S a multiple of 8 and at most 65536, pad_w <= 8 and (S - 1) * dil_w - pad_w <= 8, and one of two LDS budgets:
 * the input rows that the <= 64 / (R*S) + 2 channels of one 64-column step touch within 24 KB (any number of
 * channels; not 1 x 1 kernels with many channels), or the input rows of 256 output positions of ALL channels plus
 * a column table within about 55 KB (C * (256/Q + R - 1) * (W + 8) * 2 + ceil(C*R*S/64) * 128; needs P*Q a
 * multiple of 256).
 * Anything else returns SD_ERR_UNSUPPORTED with nothing launched: use sd_im2col + sd_gemm_dsd_lists.
 * NULL lists = every block kept: the dense convolution (block_size is then ignored, scale still applied).
 * ------------------------------------------------------------------------------------------- */
int sd_conv2d_dsd_lists(const void* x, int64_t x_stride_n, int64_t x_stride_c, int64_t x_stride_h,
                        int64_t x_stride_w, const void* weight, int64_t weight_ld,
                        void* y, int64_t y_ld,
                        int64_t n, int64_t c, int64_t h, int64_t w, int64_t k_out, int64_t r, int64_t s,
                        int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w,
                        int64_t dil_h, int64_t dil_w,
                        const int32_t* row_ptr, const int32_t* col_idx, int64_t block_size, float scale,
                        int dtype, void* stream);

/* Weight gradient of the same convolution, also without the patch matrix:
 * dw[k, j] = scale * sum over the kept blocks of dy[m, k] * cols[m, j], i.e. sd_im2col + sd_gemm_dsd_lists on the
 * transposed operands.  dy is [N*P*Q, k_out] row-major (leading dimension dy_ld), dw [k_out, C*R*S] row-major
 * (dw_ld); col_ptr / row_idx are the CSC lists of the patch matrix's mask (kept row blocks per column block; NULL,
 * NULL = dense).  The reduction runs over output positions: every step copies the input rows of its 64 positions
 * (the channels of the workgroup's 256 columns only) into LDS and builds the kept tiles from them; it is split over
 * workgroups when `workspace` (sd_conv2d_dw_workspace_bytes bytes, 16-byte aligned; may be NULL) allows.
 * Taken: strides and dilations up to 8, unit w stride of x, W a multiple of 8, Q a divisor of 64, P*Q a multiple of 64,
 * C*R*S and k_out multiples of 8, one step's copy <= 24 KB.  Anything else returns SD_ERR_UNSUPPORTED with
 * nothing launched.  No counterpart in the reference. */
/* Input gradient of the same convolution in one launch: sd_gemm_sdd_lists_kept + sd_col2im without the gradient
 * of the patch matrix in memory.  dy is [N*P*Q, k_out] row-major, weight [k_out, C*R*S] row-major, dx [N, C, H, W]
 * addressed by element strides, fully overwritten.  mask: one byte per 64 x 64 block of the patch
 * matrix (non-zero = dropped, strides in bytes), NULL = dense.  A workgroup keeps the dY rows of the output rows
 * that reach its band of input rows in registers, forms the kept tiles of dY . W per 64-column block and folds them
 * (deterministically: every dx element has one owner and a fixed summation order).  Taken: strides and dilations up to 8,
 * block_size 64, k_out a multiple of 64 up to 256, Q a divisor of 64, P*Q a multiple of 64, C*R*S a multiple of 8 and at most 4096,
 * R*S <= 64, kernels whose taps from one input row reach at most three 64-position row blocks; anything else returns SD_ERR_UNSUPPORTED
 * with nothing launched.  No counterpart in the reference. */
int sd_conv2d_dx(const void* dy, int64_t dy_ld, const void* weight, int64_t weight_ld,
                 void* dx, int64_t dx_stride_n, int64_t dx_stride_c, int64_t dx_stride_h, int64_t dx_stride_w,
                 const uint8_t* mask, int64_t mask_stride_r, int64_t mask_stride_c,
                 int64_t n, int64_t c, int64_t h, int64_t w, int64_t k_out, int64_t r, int64_t s,
                 int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w, int64_t dil_h, int64_t dil_w,
                 int64_t block_size, float scale, int dtype, void* stream);

int64_t sd_conv2d_dw_workspace_bytes(int64_t n, int64_t c, int64_t k_out, int64_t r, int64_t s, int64_t p, int64_t q);
int sd_conv2d_dw_lists(const void* x, int64_t x_stride_n, int64_t x_stride_c, int64_t x_stride_h,
                       int64_t x_stride_w, const void* dy, int64_t dy_ld, void* dw, int64_t dw_ld,
                       int64_t n, int64_t c, int64_t h, int64_t w, int64_t k_out, int64_t r, int64_t s,
                       int64_t pad_h, int64_t pad_w, int64_t stride_h, int64_t stride_w,
                       int64_t dil_h, int64_t dil_w,
                       const int32_t* col_ptr, const int32_t* row_idx, int64_t block_size, float scale,
                       int dtype, void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPARSEDROP_H_ */
