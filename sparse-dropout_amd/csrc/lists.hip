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

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): 10 rounds of
// two 32x32->64 multiplies, key bumped by the Weyl constants between rounds.
struct Philox {
  uint32_t k0, k1;
  __host__ __device__ static inline void round(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
    c[1] = (uint32_t)p1;
    c[3] = (uint32_t)p0;
    c[0] = n0;
    c[2] = n2;
  }
  __host__ __device__ inline void operator()(uint32_t (&c)[4]) const {
    uint32_t a = k0, b = k1;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
      round(c, a, b);
      a += 0x9E3779B9u;
      b += 0xBB67AE85u;
    }
  }
};

// Where "is block (i, j) dropped" comes from: a stored bool mask, or a Bernoulli(p) draw that is a pure
// function of (seed, offset, entry index), so every reader recomputes the same value and no pass over
// a stored mask is needed.  Each stored / drawn entry covers split x split entries of the listed grid
// (a logical block size that is a multiple of the 64 the kernels work in).
struct MaskSrc {
  const uint8_t* mask;  // null: drawn
  int64_t st_row, st_col;
  int32_t split;
  int32_t kb;  // entries per row of the stored / drawn mask
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  float p;
  __device__ inline bool dropped_entry(int32_t si, int32_t sj) const {
    if (mask) return mask[si * st_row + sj * st_col] != 0;
    const uint64_t e = (uint64_t)si * (uint32_t)kb + (uint32_t)sj;
    uint32_t c[4] = {(uint32_t)(e >> 2), (uint32_t)(e >> 34), off_lo, off_hi};
    Philox{seed_lo, seed_hi}(c);
    // 24 random bits -> [0, 1) in steps of 2^-24, exact in fp32; True (dropped) with probability p
    return (float)(c[e & 3] >> 8) * 0x1p-24f < p;
  }
  __device__ inline bool dropped(int32_t i, int32_t j) const {
    return split == 1 ? dropped_entry(i, j) : dropped_entry(i / split, j / split);
  }
};

struct ListJob {
  MaskSrc src;
  int32_t by_col;  // lines are columns of the grid (CSC) instead of rows (CSR)
  int64_t nlines;  // number of rows (CSR) / columns (CSC)
  int64_t len;     // entries per line
  int32_t* ptr;    // [nlines + 1]
  int32_t* idx;    // [capacity nlines * len]
  __device__ inline bool kept(int64_t line, int64_t e) const {
    return by_col ? !src.dropped((int32_t)e, (int32_t)line) : !src.dropped((int32_t)line, (int32_t)e);
  }
};

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

// Stores a drawn mask as row-major bytes (1 = dropped) for the caller to keep.
__device__ inline void write_mask(const MaskSrc& src, int64_t mb, uint8_t* out, int64_t first,
                                  int64_t stride) {
  const int64_t total = mb * src.kb;
  for (int64_t e = first; e < total; e += stride)
    out[e] = src.dropped_entry((int32_t)(e / src.kb), (int32_t)(e % src.kb)) ? 1 : 0;
}

// One thread block does count -> scan -> fill for one list.  Block 0 takes job0, block 1 job1, block 2
// (launched only for a drawn mask) stores the mask.  All traffic of a job stays inside its block, so
// __syncthreads() (which also orders the block's global writes for the block's own later reads) is
// the only synchronisation needed.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void build_lists_fused(ListJob job0, ListJob job1,
                                                             uint8_t* mask_out, int64_t mask_rows) {
  __shared__ int32_t lds[THREADS];
  if (blockIdx.x == 2) {
    write_mask(job0.src, mask_rows, mask_out, threadIdx.x, THREADS);
    return;
  }
  const ListJob job = (blockIdx.x == 0) ? job0 : job1;
  if (job.ptr == nullptr) return;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  constexpr int kWaves = THREADS / kWave;
  for (int64_t line = wave; line < job.nlines; line += kWaves) {
    int c = wave_count_kept(job, line, lane);
    if (lane == 0) job.ptr[1 + line] = c;
  }
  __syncthreads();
  block_scan_inplace<THREADS>(job.ptr, job.nlines, lds);
  __syncthreads();
  for (int64_t line = wave; line < job.nlines; line += kWaves) {
    wave_fill_kept(job, line, lane, job.idx + job.ptr[line]);
  }
}

__global__ __launch_bounds__(256) void mask_store_kernel(MaskSrc src, int64_t mb, uint8_t* out) {
  write_mask(src, mb, out, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}

// Three-launch form for large masks: grid-wide count, one block per list scans, grid-wide fill.
__global__ __launch_bounds__(256) void lists_count(ListJob job0, ListJob job1) {
  const int lane = threadIdx.x % kWave;
  const int64_t w = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t n0 = job0.ptr ? job0.nlines : 0;
  const ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
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
  const ListJob job = (w < n0) ? job0 : job1;
  const int64_t line = (w < n0) ? w : w - n0;
  if (job.ptr == nullptr || line >= job.nlines) return;
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

static int launch_lists(const MaskSrc& src, int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx,
                        int32_t* col_ptr, int32_t* row_idx, uint8_t* mask_out, int64_t mask_rows,
                        hipStream_t stream) {
  ListJob csr{src, 0, mb, kb, row_ptr, col_idx};
  ListJob csc{src, 1, kb, mb, col_ptr, row_idx};
  if (mb * kb <= (1 << 18)) {
    hipLaunchKernelGGL(build_lists_fused<1024>, dim3(mask_out ? 3 : 2), dim3(1024), 0, stream, csr, csc,
                       mask_out, mask_rows);
    return check_launch("build_lists_fused");
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

// Lists over an mb x kb grid in which every stored mask entry covers split x split grid entries.
int build_lists(const uint8_t* mask, int64_t msr, int64_t msc, int64_t stored_kb, int64_t split,
                int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{mask, msr, msc, (int32_t)split, (int32_t)stored_kb, 0, 0, 0, 0, 0.f};
  return launch_lists(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, nullptr, 0, stream);
}

// Same with the mask drawn on the device; it is also stored to mask_out ([stored_mb, stored_kb] bytes).
int random_lists(uint64_t seed, uint64_t offset, float p, int64_t stored_mb, int64_t stored_kb,
                 uint8_t* mask_out, int64_t split, int64_t mb, int64_t kb, int32_t* row_ptr,
                 int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{nullptr, 0, 0, (int32_t)split, (int32_t)stored_kb, (uint32_t)seed, (uint32_t)(seed >> 32),
              (uint32_t)offset, (uint32_t)(offset >> 32), p};
  return launch_lists(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, mask_out, stored_mb, stream);
}

int increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                    int64_t* table, int64_t* row_indices, int64_t* row_widths, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(mb, 4) < 4096 ? ceil_div(mb, 4) : 4096);
  hipLaunchKernelGGL(increment_table_kernel, dim3(blocks), dim3(256), 0, stream, row_ptr, col_idx,
                     mb, block_k, table, row_indices, row_widths);
  return check_launch("increment_table");
}

}  // namespace sd
