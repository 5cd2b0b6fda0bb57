// Block mask -> compacted kept-block lists (CSR over row blocks, CSC over column blocks).
//
// Integer/byte work, bound by launch latency and a few KB of HBM traffic: one wave owns one row
// (or column) of the mask, 64 mask bytes per step; __ballot + popcount give each kept block its
// slot, so the lists come out in ascending order — the order of nonzero(~mask)
// (flash_dropout/functional/blockwise_dropout_matmul_triton.py:48) — without atomics and without
// a device->host synchronisation.
#include "common.h"

namespace sd {
namespace {

constexpr int kWave = 64;

// Number of kept (zero) bytes among line[0 .. n) with element stride `st`; whole wave cooperates.
__device__ inline int wave_count_kept(const uint8_t* line, int64_t n, int64_t st, int lane) {
  int total = 0;
  for (int64_t base = 0; base < n; base += kWave) {
    int64_t i = base + lane;
    bool kept = (i < n) && (line[i * st] == 0);
    total += __popcll(__ballot(kept));
  }
  return total;
}

// Writes the indices of kept bytes of the line, ascending, to out[0 .. count).
__device__ inline void wave_fill_kept(const uint8_t* line, int64_t n, int64_t st, int lane,
                                      int32_t* out) {
  int written = 0;
  const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t base = 0; base < n; base += kWave) {
    int64_t i = base + lane;
    bool kept = (i < n) && (line[i * st] == 0);
    uint64_t bal = __ballot(kept);
    if (kept) out[written + __popcll(bal & lt)] = (int32_t)i;
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

struct ListJob {
  const uint8_t* mask;
  int64_t nlines;   // number of rows (CSR) / columns (CSC)
  int64_t len;      // entries per line
  int64_t st_line;  // byte stride between lines
  int64_t st_elem;  // byte stride along a line
  int32_t* ptr;     // [nlines + 1]
  int32_t* idx;     // [capacity nlines * len]
};

// One thread block does count -> scan -> fill for one list.  Block 0 takes job0, block 1 job1.
// All traffic of a job stays inside its block, so __syncthreads() (which also orders the block's
// global writes for the block's own later reads) is the only synchronisation needed.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void build_lists_fused(ListJob job0, ListJob job1) {
  __shared__ int32_t lds[THREADS];
  const ListJob job = (blockIdx.x == 0) ? job0 : job1;
  if (job.ptr == nullptr) return;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  constexpr int kWaves = THREADS / kWave;
  for (int64_t line = wave; line < job.nlines; line += kWaves) {
    int c = wave_count_kept(job.mask + line * job.st_line, job.len, job.st_elem, lane);
    if (lane == 0) job.ptr[1 + line] = c;
  }
  __syncthreads();
  block_scan_inplace<THREADS>(job.ptr, job.nlines, lds);
  __syncthreads();
  for (int64_t line = wave; line < job.nlines; line += kWaves) {
    wave_fill_kept(job.mask + line * job.st_line, job.len, job.st_elem, lane,
                   job.idx + job.ptr[line]);
  }
}

// Three-launch form for large masks: grid-wide count, one block per list scans, grid-wide fill.
__global__ __launch_bounds__(256) void lists_count(ListJob job0, ListJob job1) {
  const int lane = threadIdx.x % kWave;
  const int64_t w = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t n0 = job0.ptr ? job0.nlines : 0;
  const ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
  int c = wave_count_kept(job.mask + line * job.st_line, job.len, job.st_elem, lane);
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
  const ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
  wave_fill_kept(job.mask + line * job.st_line, job.len, job.st_elem, lane, job.idx + job.ptr[line]);
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

int build_lists(const uint8_t* mask, int64_t mb, int64_t kb, int64_t msr, int64_t msc,
                int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx,
                hipStream_t stream) {
  ListJob csr{mask, mb, kb, msr, msc, row_ptr, col_idx};
  ListJob csc{mask, kb, mb, msc, msr, col_ptr, row_idx};
  if (mb * kb <= (1 << 18)) {
    hipLaunchKernelGGL(build_lists_fused<1024>, dim3(2), dim3(1024), 0, stream, csr, csc);
    return check_launch("build_lists_fused");
  }
  const int64_t waves = (row_ptr ? mb : 0) + (col_ptr ? kb : 0);
  const unsigned blocks = (unsigned)ceil_div(waves, 4);
  hipLaunchKernelGGL(lists_count, dim3(blocks), dim3(256), 0, stream, csr, csc);
  hipLaunchKernelGGL(lists_scan, dim3(2), dim3(1024), 0, stream, csr, csc);
  hipLaunchKernelGGL(lists_fill, dim3(blocks), dim3(256), 0, stream, csr, csc);
  return check_launch("build_lists");
}

int increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                    int64_t* table, int64_t* row_indices, int64_t* row_widths, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(mb, 4) < 4096 ? ceil_div(mb, 4) : 4096);
  hipLaunchKernelGGL(increment_table_kernel, dim3(blocks), dim3(256), 0, stream, row_ptr, col_idx,
                     mb, block_k, table, row_indices, row_widths);
  return check_launch("increment_table");
}

}  // namespace sd
