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
// (a logical block size that is a multiple of the 64 the kernels work in), or, with merge == 2, a quarter of
// one: a mask at block size 32 is listed on the 64 grid, an entry being kept when any of its four 32-blocks
// is, with those four keep bits stored in the top bits of its list entry (quad_bits).
struct MaskSrc {
  const uint8_t* mask;  // null: drawn
  int64_t st_row, st_col;
  int32_t split;
  int32_t merge;  // 1, or 2: four stored / drawn entries per listed entry
  int32_t mb;     // rows of the stored / drawn mask (only read when merge == 2)
  int32_t kb;  // entries per row of the stored / drawn mask
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  float p;
  const uint64_t* state;  // device-resident {seed, offset} that overrides the four words above, or null
  // Kernels call this once on their copy: a draw keyed by device memory lets a captured graph draw a
  // fresh mask at every replay (the host bumps nothing; a one-thread kernel advances the offset).
  __device__ inline void resolve() {
    if (state) {
      const uint64_t sd = state[0], off = state[1];
      seed_lo = (uint32_t)sd;
      seed_hi = (uint32_t)(sd >> 32);
      off_lo = (uint32_t)off;
      off_hi = (uint32_t)(off >> 32);
    }
  }
  __device__ inline bool dropped_entry(int32_t si, int32_t sj) const {
    if (mask) return mask[si * st_row + sj * st_col] != 0;
    const uint64_t e = (uint64_t)si * (uint32_t)kb + (uint32_t)sj;
    uint32_t c[4] = {(uint32_t)(e >> 2), (uint32_t)(e >> 34), off_lo, off_hi};
    Philox{seed_lo, seed_hi}(c);
    // 24 random bits -> [0, 1) in steps of 2^-24, exact in fp32; True (dropped) with probability p
    return (float)(c[e & 3] >> 8) * 0x1p-24f < p;
  }
  // One generator call yields the draws of four consecutive entries: bit v = entry 4 * grp + v is dropped.
  __device__ inline uint32_t dropped4(uint64_t grp) const {
    uint32_t c[4] = {(uint32_t)grp, (uint32_t)(grp >> 32), off_lo, off_hi};
    Philox{seed_lo, seed_hi}(c);
    uint32_t bits = 0;
#pragma unroll
    for (int v = 0; v < 4; ++v) bits |= ((float)(c[v] >> 8) * 0x1p-24f < p ? 1u : 0u) << v;
    return bits;
  }
  // merge == 2: keep bits of the four 32-blocks of listed entry (i, j); bit 2a + b = block (2i + a, 2j + b)
  __device__ inline uint32_t kept_quads(int32_t i, int32_t j) const {
    uint32_t q = 0;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int32_t si = 2 * i + a, sj = 2 * j + b;
        if (si < mb && sj < kb && !dropped_entry(si, sj)) q |= 1u << (2 * a + b);
      }
    return q;
  }
  __device__ inline bool dropped(int32_t i, int32_t j) const {
    if (merge == 2) return kept_quads(i, j) == 0;
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
  // what goes into idx for kept entry e of `line`: e itself, with merge == 2 the four keep bits of its
  // 32-blocks in bits 28-31 (bit 2a + b: row half a, column half b of the LIST's own orientation, i.e.
  // transposed for a list by columns, which is the row list of the transposed mask)
  __device__ inline int32_t entry(int64_t line, int64_t e) const {
    if (src.merge != 2) return (int32_t)e;
    uint32_t q = by_col ? src.kept_quads((int32_t)e, (int32_t)line) : src.kept_quads((int32_t)line, (int32_t)e);
    if (by_col) q = (q & 0x9u) | ((q & 0x2u) << 1) | ((q & 0x4u) >> 1);
    return (int32_t)((uint32_t)e | (q << 28));
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

// Stores a drawn mask as row-major bytes (1 = dropped) for the caller to keep.
__device__ inline void write_mask(const MaskSrc& src, int64_t mb, uint8_t* out, int64_t first,
                                  int64_t stride) {
  const int64_t total = mb * src.kb;
  if (src.mask == nullptr) {  // drawn: four entries per generator call
    for (int64_t grp = first; grp * 4 < total; grp += stride) {
      const uint32_t bits = src.dropped4((uint64_t)grp);
      for (int v = 0; v < 4 && grp * 4 + v < total; ++v) out[grp * 4 + v] = (bits >> v) & 1u;
    }
    return;
  }
  for (int64_t e = first; e < total; e += stride)
    out[e] = src.dropped_entry((int32_t)(e / src.kb), (int32_t)(e % src.kb)) ? 1 : 0;
}

// ---- single-launch builder for masks of up to 2^18 entries ------------------------------------------
// A list is a stream compaction of the mask read in line-major order ("flat" index f = line * len + e):
// idx gets e of every kept entry, ptr[line] the number of kept entries before the line.  A block owns
// kFlatChunk consecutive flat entries.  Blocks do not talk to each other: each first counts the kept
// entries in front of its chunk itself (one sweep over at most 2^18 mask bytes, or draws), which replaces
// the grid-wide scan and keeps the whole build in one launch with every load independent of the others.
constexpr int kFlatThreads = 1024;
constexpr int kFlatPer = 4;  // consecutive entries per thread
constexpr int kFlatChunk = kFlatThreads * kFlatPer;

// Exclusive prefix of v over the block (thread order) and the block total; lds holds one int per wave.
__device__ inline int block_exclusive_scan(int v, int32_t* lds, int& total) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  int incl = v;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += up;
  }
  __syncthreads();  // lds may still be read from a previous call
  if (lane == kWave - 1) lds[wave] = incl;
  __syncthreads();
  int before = 0, sum = 0;
  for (int w = 0; w < kFlatThreads / kWave; ++w) {
    const int t = lds[w];
    if (w < wave) before += t;
    sum += t;
  }
  total = sum;
  return before + incl - v;
}

// `advance` (the device-resident generator state of a draw keyed by it, else null): the block that finishes
// last moves the state on to the next draw.  Every block has read the state by the time it reports in
// (state[2] counts arrivals and is left at zero), so no block can see the new offset.
__global__ __launch_bounds__(kFlatThreads) void build_lists_flat(ListJob job0, ListJob job1, int blocks0,
                                                                int blocks1, uint8_t* mask_out,
                                                                int64_t mask_rows, uint64_t* advance) {
  __shared__ int32_t lds[kFlatThreads / kWave];
  const int tid = threadIdx.x;
  int b = blockIdx.x;
  auto report_in = [&]() {
    if (advance == nullptr) return;
    __syncthreads();
    if (tid == 0) {
      unsigned* arrivals = reinterpret_cast<unsigned*>(advance + 2);
      if (atomicAdd(arrivals, 1u) == gridDim.x - 1) {
        *arrivals = 0u;
        advance[1] += 1;
      }
    }
  };
  if (b >= blocks0 + blocks1) {  // launched only for a drawn mask: store it for the caller
    const int nb = gridDim.x - blocks0 - blocks1;
    job0.src.resolve();
    write_mask(job0.src, mask_rows, mask_out, (int64_t)(b - blocks0 - blocks1) * kFlatThreads + tid,
               (int64_t)nb * kFlatThreads);
    report_in();
    return;
  }
  const bool second = b >= blocks0;
  ListJob job = second ? job1 : job0;
  job.src.resolve();
  if (second) b -= blocks0;
  const int len = (int)job.len;
  const int total_entries = (int)(job.nlines * job.len);
  const int f0 = b * kFlatChunk;

  // kept entries in front of this block's chunk
  // a mask drawn at the listed granularity: entry index = row-major position, four entries share a generator call
  const bool drawn4 = job.src.mask == nullptr && job.src.split == 1 && job.src.merge == 1 && job.src.kb == (job.by_col ? (int)job.nlines : len);
  int cnt = 0;
  if (drawn4 && !job.by_col) {
    for (int grp = tid; grp * 4 < f0; grp += kFlatThreads) cnt += __popc(~job.src.dropped4((uint64_t)grp) & 0xFu);
  } else if (drawn4) {
    // lines are columns: in front of (col0, row0) lies every entry of an earlier column and the rows above in col0
    const int kb = job.src.kb;
    const int col0 = f0 / len, row0 = f0 - col0 * len;
    for (int grp = tid; grp * 4 < total_entries; grp += kFlatThreads) {
      uint32_t kept = ~job.src.dropped4((uint64_t)grp) & 0xFu;
      int row = (grp * 4) / kb, col = grp * 4 - row * kb;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const bool front = grp * 4 + v < total_entries && (col < col0 || (col == col0 && row < row0));
        if (!front) kept &= ~(1u << v);
        if (++col == kb) { col = 0; ++row; }
      }
      cnt += __popc(kept);
    }
  } else {
    for (int f = tid; f < f0; f += kFlatThreads) {
      const int line = f / len;
      cnt += job.kept(line, f - line * len) ? 1 : 0;
    }
  }
  int base;
  block_exclusive_scan(cnt, lds, base);

  // this thread's entries
  const int mine = f0 + tid * kFlatPer;
  int line = mine / len, e = mine - line * len;
  uint32_t bits = 0;
  if (drawn4 && !job.by_col) {  // mine is a multiple of four: one generator call
    if (mine < total_entries) {
      bits = ~job.src.dropped4((uint64_t)(mine / 4)) & 0xFu;
      if (mine + 4 > total_entries) bits &= (1u << (total_entries - mine)) - 1u;
    }
  } else {
    int l = line, x = e;
#pragma unroll
    for (int v = 0; v < kFlatPer; ++v) {
      if (mine + v < total_entries && job.kept(l, x)) bits |= 1u << v;
      if (++x == len) { x = 0; ++l; }
    }
  }
  int chunk_total;
  int pos = base + block_exclusive_scan(__popc(bits), lds, chunk_total);
#pragma unroll
  for (int v = 0; v < kFlatPer; ++v) {
    if (mine + v < total_entries) {
      if (e == 0) job.ptr[line] = pos;
      if (bits & (1u << v)) job.idx[pos++] = job.entry(line, e);
    }
    if (++e == len) { e = 0; ++line; }
  }
  if (tid == 0 && f0 + kFlatChunk >= total_entries) job.ptr[job.nlines] = base + chunk_total;
  report_in();
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
  if (mb * kb <= (1 << 18)) {
    const int per_list = (int)ceil_div(mb * kb, kFlatChunk);
    const int blocks0 = row_ptr ? per_list : 0, blocks1 = col_ptr ? per_list : 0;
    const int blocks_mask = mask_out ? (int)ceil_div(mask_rows * src.kb, kFlatChunk) : 0;
    hipLaunchKernelGGL(build_lists_flat, dim3(blocks0 + blocks1 + blocks_mask), dim3(kFlatThreads), 0, stream,
                       csr, csc, blocks0, blocks1, mask_out, mask_rows, const_cast<uint64_t*>(src.state));
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

// Lists over an mb x kb grid in which every stored mask entry covers split x split grid entries; split == 0: the
// stored mask is at half the granularity (stored_mb x stored_kb entries) and is merged two by two.
int build_lists(const uint8_t* mask, int64_t msr, int64_t msc, int64_t stored_mb, int64_t stored_kb, int64_t split,
                int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx, int32_t* col_ptr,
                int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{mask, msr, msc, (int32_t)(split ? split : 1), split ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
              0, 0, 0, 0, 0.f, nullptr};
  return launch_lists(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, nullptr, 0, stream);
}

// Same with the mask drawn on the device; it is also stored to mask_out ([stored_mb, stored_kb] bytes).
int random_lists(uint64_t seed, uint64_t offset, uint64_t* state, float p, int64_t stored_mb, int64_t stored_kb,
                 uint8_t* mask_out, int64_t split, int64_t mb, int64_t kb, int32_t* row_ptr,
                 int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, hipStream_t stream) {
  MaskSrc src{nullptr, 0, 0, (int32_t)(split ? split : 1), split ? 1 : 2, (int32_t)stored_mb, (int32_t)stored_kb,
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

int increment_table(const int32_t* row_ptr, const int32_t* col_idx, int64_t mb, int64_t block_k,
                    int64_t* table, int64_t* row_indices, int64_t* row_widths, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(mb, 4) < 4096 ? ceil_div(mb, 4) : 4096);
  hipLaunchKernelGGL(increment_table_kernel, dim3(blocks), dim3(256), 0, stream, row_ptr, col_idx,
                     mb, block_k, table, row_indices, row_widths);
  return check_launch("increment_table");
}

}  // namespace sd
