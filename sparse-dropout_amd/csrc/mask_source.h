// Where a block mask comes from (stored bytes or a counter-based draw) and the single-launch list builder over it,
// as device code that more than one kernel uses: the list builder's own launch, and the forward product that builds
// the lists of its mask in the same launch.
#pragma once
#include "common.h"

namespace sd {

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
// (a logical block size that is a multiple of the 64 the kernels work in), or, with merge == 2, the listed grid is
// twice as coarse as a grid of 32-blocks of which every stored entry covers split x split: a mask at block size
// 32 * split (32, 96, 160, ...) is listed on the 64 grid, an entry being kept when any of its four 32-blocks is, with
// those four keep bits stored in the top bits of its list entry (quad_bits).
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
        // 32-blocks (2i + a, 2j + b); a stored entry covers split x split of them (block size 32 * split)
        const int32_t si = (2 * i + a) / split, sj = (2 * j + b) / split;
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
// THREADS * kFlatPer consecutive flat entries.  Blocks do not talk to each other: each first counts the kept
// entries in front of its chunk itself (one sweep over at most 2^18 mask bytes, or draws), which replaces
// the grid-wide scan and keeps the whole build in one launch with every load independent of the others.
constexpr int kFlatPer = 4;  // consecutive entries per thread
constexpr int64_t kFlatMaxEntries = 1 << 18;

// The blocks of one such build: blocks0 for the list by rows, blocks1 for the list by columns, blocks_mask that
// store a drawn mask for the caller (all three may be zero).
struct FlatJobs {
  ListJob job0, job1;
  int32_t blocks0, blocks1, blocks_mask;
  uint8_t* mask_out;
  int64_t mask_rows;
  __host__ __device__ inline int blocks() const { return blocks0 + blocks1 + blocks_mask; }
};

// The build of the lists the pointers ask for, by blocks of `threads` threads.
inline FlatJobs flat_jobs(const MaskSrc& src, int64_t mb, int64_t kb, int32_t* row_ptr, int32_t* col_idx,
                          int32_t* col_ptr, int32_t* row_idx, uint8_t* mask_out, int64_t mask_rows, int threads) {
  FlatJobs f;
  f.job0 = ListJob{src, 0, mb, kb, row_ptr, col_idx};
  f.job1 = ListJob{src, 1, kb, mb, col_ptr, row_idx};
  const int64_t chunk = (int64_t)threads * kFlatPer;
  const int per_list = (int)ceil_div(mb * kb, chunk);
  f.blocks0 = row_ptr ? per_list : 0;
  f.blocks1 = col_ptr ? per_list : 0;
  f.blocks_mask = mask_out ? (int)ceil_div(mask_rows * src.kb, chunk) : 0;
  f.mask_out = mask_out;
  f.mask_rows = mask_rows;
  return f;
}

// Exclusive prefix of v over the block (thread order) and the block total; lds holds one int per wave.
template <int THREADS>
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
  for (int w = 0; w < THREADS / kWave; ++w) {
    const int t = lds[w];
    if (w < wave) before += t;
    sum += t;
  }
  total = sum;
  return before + incl - v;
}

// A draw keyed by a device-resident generator state: the block that finishes last moves the state on to the next
// draw.  Every block of the launch calls this once, after it has read the state (state[2] counts arrivals and is
// left at zero), so no block can see the new offset.  `advance` null: nothing to do.
__device__ inline void report_in(uint64_t* advance, unsigned blocks_in_launch) {
  if (advance == nullptr) return;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned* arrivals = reinterpret_cast<unsigned*>(advance + 2);
    if (atomicAdd(arrivals, 1u) == blocks_in_launch - 1) {
      *arrivals = 0u;
      advance[1] += 1;
    }
  }
}

// Block b (of f.blocks()) of the build, by a block of THREADS threads; lds: THREADS / 64 ints.
template <int THREADS>
__device__ inline void flat_lists_block(const FlatJobs& f, int b, int32_t* lds) {
  constexpr int kFlatChunk = THREADS * kFlatPer;
  const int tid = threadIdx.x;
  if (b >= f.blocks0 + f.blocks1) {  // store the drawn mask for the caller
    MaskSrc src = f.job0.src;
    src.resolve();
    write_mask(src, f.mask_rows, f.mask_out, (int64_t)(b - f.blocks0 - f.blocks1) * THREADS + tid,
               (int64_t)f.blocks_mask * THREADS);
    return;
  }
  const bool second = b >= f.blocks0;
  ListJob job = second ? f.job1 : f.job0;
  job.src.resolve();
  if (second) b -= f.blocks0;
  const int len = (int)job.len;
  const int total_entries = (int)(job.nlines * job.len);
  const int f0 = b * kFlatChunk;

  // kept entries in front of this block's chunk
  // a mask drawn at the listed granularity: entry index = row-major position, four entries share a generator call
  const bool drawn4 = job.src.mask == nullptr && job.src.split == 1 && job.src.merge == 1 && job.src.kb == (job.by_col ? (int)job.nlines : len);
  int cnt = 0;
  if (drawn4 && !job.by_col) {
    for (int grp = tid; grp * 4 < f0; grp += THREADS) cnt += __popc(~job.src.dropped4((uint64_t)grp) & 0xFu);
  } else if (drawn4) {
    // lines are columns: in front of (col0, row0) lies every entry of an earlier column and the rows above in col0
    const int kb = job.src.kb;
    const int col0 = f0 / len, row0 = f0 - col0 * len;
    for (int grp = tid; grp * 4 < total_entries; grp += THREADS) {
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
    for (int f = tid; f < f0; f += THREADS) {
      const int line = f / len;
      cnt += job.kept(line, f - line * len) ? 1 : 0;
    }
  }
  int base;
  block_exclusive_scan<THREADS>(cnt, lds, base);

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
  int pos = base + block_exclusive_scan<THREADS>(__popc(bits), lds, chunk_total);
#pragma unroll
  for (int v = 0; v < kFlatPer; ++v) {
    if (mine + v < total_entries) {
      if (e == 0) job.ptr[line] = pos;
      if (bits & (1u << v)) job.idx[pos++] = job.entry(line, e);
    }
    if (++e == len) { e = 0; ++line; }
  }
  if (tid == 0 && f0 + kFlatChunk >= total_entries) job.ptr[job.nlines] = base + chunk_total;
}

}  // namespace sd
