// Block mask -> compacted kept-block lists (CSR over row blocks, CSC over column blocks).
//
// Integer/byte work, bound by launch latency and a few KB of HBM traffic.  The lists come out in
// ascending order — the order of nonzero(~mask)
// (flash_dropout/functional/blockwise_dropout_matmul_triton.py:48) — without atomics and without
// a device->host synchronisation.  Masks of up to 2^18 entries are listed by one launch (a flat
// stream compaction, see build_lists_flat); larger ones by count / scan / fill launches in which one
// wave owns one row (or column) of the mask, 64 entries per step, __ballot + popcount giving each kept
// block its slot.  The mask is either stored (bool bytes, any of the two majornesses) or drawn on the
// fly from a counter-based generator, and may be listed at a finer granularity than it was drawn.
#include "common.h"
#include "mask_source.h"

namespace sd {
namespace {

// Number of kept entries of one line; whole wave cooperates.
__device__ inline int wave_count_kept(const ListJob& job, int64_t line, int lane) {
  int total = 0;
  for (int64_t base = 0; base < job.len; base += kWave) {
    const int64_t i = base + lane;
    const bool kept = (i < job.len) && job.kept(line, i);
    total += __popcll(__ballot(kept));
  }
  return total;
}

// Writes the indices of the kept entries of the line, ascending, to out[0 .. count).
__device__ inline void wave_fill_kept(const ListJob& job, int64_t line, int lane, int32_t* out) {
  int written = 0;
  const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t base = 0; base < job.len; base += kWave) {
    const int64_t i = base + lane;
    const bool kept = (i < job.len) && job.kept(line, i);
    const uint64_t bal = __ballot(kept);
    if (kept) out[written + __popcll(bal & lt)] = job.entry(line, i);
    written += __popcll(bal);
  }
}

// In-place inclusive scan of ptr[1 .. n] by one thread block (ptr[0] is set to 0).
template <int THREADS>
__device__ inline void block_scan_inplace(int32_t* ptr, int64_t n, int32_t* lds /*THREADS*/) {
  const int t = threadIdx.x;
  int32_t carry = 0;
  if (t == 0) ptr[0] = 0;
  for (int64_t base = 0; base < n; base += THREADS) {
    int64_t i = base + t;
    int32_t v = (i < n) ? ptr[1 + i] : 0;
    lds[t] = v;
    __syncthreads();
    for (int off = 1; off < THREADS; off <<= 1) {
      int32_t add = (t >= off) ? lds[t - off] : 0;
      __syncthreads();
      lds[t] += add;
      __syncthreads();
    }
    if (i < n) ptr[1 + i] = lds[t] + carry;
    carry += lds[THREADS - 1];
    __syncthreads();
  }
}

// The single-launch builder (flat_lists_block) as a launch of its own.
constexpr int kFlatThreads = 1024;

__global__ __launch_bounds__(kFlatThreads) void build_lists_flat(FlatJobs f) {
  __shared__ int32_t lds[kFlatThreads / kWave];
  flat_lists_block<kFlatThreads>(f, (int)blockIdx.x, lds);
  report_in(const_cast<uint64_t*>(f.job0.src.state), gridDim.x);
}

// The same for the multi-launch form, after every kernel of a draw has read the state.
__global__ void advance_state_kernel(uint64_t* state) { state[1] += 1; }

__global__ __launch_bounds__(256) void mask_store_kernel(MaskSrc src, int64_t mb, uint8_t* out) {
  src.resolve();
  write_mask(src, mb, out, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}

// Three-launch form for large masks: grid-wide count, one block per list scans, grid-wide fill.
__global__ __launch_bounds__(256) void lists_count(ListJob job0, ListJob job1) {
  const int lane = threadIdx.x % kWave;
  const int64_t w = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t n0 = job0.ptr ? job0.nlines : 0;
  ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
  job.src.resolve();
  int c = wave_count_kept(job, line, lane);
  if (lane == 0) job.ptr[1 + line] = c;
}

__global__ __launch_bounds__(1024) void lists_scan(ListJob job0, ListJob job1) {
  __shared__ int32_t lds[1024];
  const ListJob job = (blockIdx.x == 0) ? job0 : job1;
  if (job.ptr == nullptr) return;
  block_scan_inplace<1024>(job.ptr, job.nlines, lds);
}

__global__ __launch_bounds__(256) void lists_fill(ListJob job0, ListJob job1) {
  const int lane = threadIdx.x % kWave;
  const int64_t w = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t n0 = job0.ptr ? job0.nlines : 0;
  ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
  job.src.resolve();
  wave_fill_kept(job, line, lane, job.idx + job.ptr[line]);
}

// table / row_indices / row_widths of the reference's mask_to_increment_table
// (flash_dropout/functional/utils.py:57-67) from the CSR list; one wave per row.
__global__ __launch_bounds__(256) void increment_table_kernel(const int32_t* row_ptr,
                                                              const int32_t* col_idx, int64_t mb,
                                                              int64_t block_k, int64_t* table,
                                                              int64_t* row_indices,
                                                              int64_t* row_widths) {
  const int lane = threadIdx.x % kWave;
  const int64_t nwaves = (int64_t)gridDim.x * (256 / kWave);
  for (int64_t r = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave; r < mb; r += nwaves) {
    const int32_t beg = row_ptr[r], end = row_ptr[r + 1];
    if (lane == 0) {
      row_indices[r] = beg;
      row_widths[r] = end - beg;
    }
    for (int32_t i = beg + lane; i < end; i += kWave) {
      int64_t cur = col_idx[i];
      int64_t prev = (i == beg) ? 0 : col_idx[i - 1];
      table[i] = (cur - prev) * block_k;
    }
  }
}

}  // namespace

// *advanced: whether the launch also moved a device-resident generator state on
static int launch_lists(const MaskSrc& src, int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx,
                        int32_t* col_ptr, int32_t* row_idx, uint8_t* mask_out, int64_t mask_rows,
                        hipStream_t stream, bool* advanced = nullptr) {
  ListJob csr{src, 0, mb, kb, row_ptr, col_idx};
  ListJob csc{src, 1, kb, mb, col_ptr, row_idx};
  if (mb * kb <= kFlatMaxEntries) {
    const FlatJobs f = flat_jobs(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, mask_out, mask_rows, kFlatThreads);
    hipLaunchKernelGGL(build_lists_flat, dim3(f.blocks()), dim3(kFlatThreads), 0, stream, f);
    if (advanced) *advanced = src.state != nullptr;
    return check_launch("build_lists_flat");
  }
  if (mask_out) {
    const int64_t total = mask_rows * src.kb;
    const unsigned blocks = (unsigned)(ceil_div(total, 256) < 4096 ? ceil_div(total, 256) : 4096);
    hipLaunchKernelGGL(mask_store_kernel, dim3(blocks), dim3(256), 0, stream, src, mask_rows, mask_out);
  }
  const int64_t waves = (row_ptr ? mb : 0) + (col_ptr ? kb : 0);
  const unsigned blocks = (unsigned)ceil_div(waves, 4);
  hipLaunchKernelGGL(lists_count, dim3(blocks), dim3(256), 0, stream, csr, csc);
  hipLaunchKernelGGL(lists_scan, dim3(2), dim3(1024), 0, stream, csr, csc);
  hipLaunchKernelGGL(lists_fill, dim3(blocks), dim3(256), 0, stream, csr, csc);
  return check_launch("build_lists");
}

// Lists over an mb x kb grid in which every stored mask entry covers split x split grid entries; split <= 0: the
// grid is of 64-blocks and the stored mask (stored_mb x stored_kb entries) is at block size 32 * |split| (0 counts as
// -1): its 32-blocks are merged two by two, the four keep bits of an entry kept beside it.
int build_lists(const uint8_t* mask, int64_t msr, int64_t msc, int64_t stored_mb, int64_t stored_kb, int64_t split,
                int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{mask, msr, msc, (int32_t)(split > 0 ? split : (split < 0 ? -split : 1)), split > 0 ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
              0, 0, 0, 0, 0.f, nullptr};
  return launch_lists(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, nullptr, 0, stream);
}

// Same with the mask drawn on the device; it is also stored to mask_out ([stored_mb, stored_kb] bytes).
int random_lists(uint64_t seed, uint64_t offset, uint64_t* state, float p, int64_t stored_mb, int64_t stored_kb,
                 uint8_t* mask_out, int64_t split, int64_t mb, int64_t kb, int32_t* row_ptr,
                 int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{nullptr, 0, 0, (int32_t)(split > 0 ? split : (split < 0 ? -split : 1)), split > 0 ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
              (uint32_t)seed, (uint32_t)(seed >> 32), (uint32_t)offset, (uint32_t)(offset >> 32), p, state};
  bool advanced = false;
  if (int rc = launch_lists(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, mask_out, stored_mb, stream, &advanced))
    return rc;
  if (state && !advanced) {
    hipLaunchKernelGGL(advance_state_kernel, dim3(1), dim3(1), 0, stream, state);
    return check_launch("advance_state");
  }
  return SD_OK;
}

int forward_with_lists(const GemmArgs& g, const uint8_t* mask, int64_t msr, int64_t msc, uint64_t seed, uint64_t offset,
                       uint64_t* state, float p, int64_t stored_mb, int64_t stored_kb, uint8_t* mask_out, int64_t split,
                       int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                       int dtype, hipStream_t stream) {
  MaskSrc src{mask, msr, msc, (int32_t)(split > 0 ? split : (split < 0 ? -split : 1)), split > 0 ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
              0, 0, 0, 0, 0.f, nullptr};
  if (mask == nullptr) {
    src = MaskSrc{nullptr, 0, 0, (int32_t)(split > 0 ? split : (split < 0 ? -split : 1)), split > 0 ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
                  (uint32_t)seed, (uint32_t)(seed >> 32), (uint32_t)offset, (uint32_t)(offset >> 32), p, state};
  }
  return launch_forward_with_lists(g, src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, mask ? nullptr : mask_out,
                                   stored_mb, dtype, stream);
}

int increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                    int64_t* table, int64_t* row_indices, int64_t* row_widths, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(mb, 4) < 4096 ? ceil_div(mb, 4) : 4096);
  hipLaunchKernelGGL(increment_table_kernel, dim3(blocks), dim3(256), 0, stream, row_ptr, col_idx,
                     mb, block_k, table, row_indices, row_widths);
  return check_launch("increment_table");
}

}  // namespace sd
