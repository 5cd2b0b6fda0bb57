// Specialised gfx950 kernels for 64x64 mask blocks and tile-aligned shapes.
//
// ---- DSD, both operands reduction-contiguous (the forward Y = s*(keep.X).W^T, and dense) -------
// A workgroup owns 4 consecutive row blocks of X (256 rows) x 256 columns of Y.  Row blocks keep
// different K blocks, so the workgroup walks the UNION of their kept lists: per step it brings in
// one 256x64 tile of W (shared by everybody) and the 64x64 X tiles of just the row blocks that keep
// this K block, and issues MFMAs only for those.  The 8 waves are (column slice ns = wave%4) x
// (row-block pair rh = wave/4): a wave multiplies its 64-column slice of the W tile (held in
// registers for the step) with each kept X tile of its pair, in v_mfma_f32_16x16x32 tiles (measured on
// N(0,1) operands, where the clock is power-limited, that instruction sustains about 17 % more FLOP/s than
// v_mfma_f32_32x32x16).  Waves w and w+4 land on the same SIMD,
// so every SIMD sees exactly (#kept row blocks) x 64x64x64 of MFMA work per step whatever the mask
// looks like: dropped blocks cost neither loads nor MFMAs and no wave idles behind a barrier.
//
// Global->LDS goes through global_load_lds_dwordx4 (no VGPR staging), two stages.  Two step loops:
//  * aligned operands on the 256 x 256 shape (what the large products run on): the two waves of a SIMD work in
//    opposite phases - one reads fragments and issues loads while the other issues nothing but MFMAs - with a
//    barrier per phase; see "the step loop of the 256 x 256 shape" in dsd_body.  A wave that stands at a load or a
//    fragment read (the texture path takes a 1 KB load every 25 clocks or so) issues no MFMA behind it, so with both
//    waves of a SIMD in the same phase the parts of a step add up instead of overlapping.
//  * ragged operands, masks of block size 32 and the 128 x 128 shape: one barrier per step, in front of the MFMAs of
//    the step's last (row block, half of the K block) unit, when every fragment of the current stage is in
//    registers; the loads of the step after next and the fragment reads of the next step's first unit are issued
//    behind it and run under those MFMAs.
// Staging the tiles through registers (global_load_dwordx4 + ds_write_b128) moves them no faster; dealing loads and
// reads out between the MFMAs of one wave loses.
// A tile row is 128 B (64 halfs) and its 16-byte chunks are XOR-swizzled with (row>>1)&7,
// which makes the MFMA fragment reads (ds_read_b128, 16 rows x one chunk per 16-lane group) hit all
// 64 LDS banks; the swizzle is applied on the global side (which chunk a lane fetches), because the
// LDS side of a direct load is fixed at lane*16.
//
// ---- DSD, both operands reduction-strided (the weight gradient dW = s*dY^T.(keep.X)) ------------
// Same walk with the roles renamed: the "row blocks" are K blocks of X (rows of X^T), the list is the
// CSC list (kept row blocks of X per K block), the reduction runs over M.  Tiles arrive in memory
// order [reduction][64 or 256 contiguous columns] and the MFMA fragments (8 consecutive reduction
// elements of one column per lane) are formed by ds_read_b64_tr_b16, two per fragment.  That read
// takes, per 16-lane group, 4 reduction rows x 32 bytes; the chunk swizzles below put those on
// distinct banks.
//
// Either instance writes C in either majorness: for a column-major C (the row-major dW[N,K] seen as
// the [K,N] product's transpose) the two MFMA operands are swapped, so that lanes run along C's rows,
// its contiguous index.
//
// ---- SDD (the input gradient dX = s*(dY.W) (.) keep) ----------------------------------------------
// Only kept output tiles are computed; the reduction (over N) is dense.  dY tiles are reduction-contiguous
// (swizzled as in the forward), W tiles reduction-strided (read with ds_read_b64_tr_b16 as in dW).  See
// sdd_group_kernel for how tiles are grouped into workgroups; dropped tiles are written as zeros.
#include <atomic>
#include <cstdlib>
#include <type_traits>

#include "common.h"
#include "mask_source.h"
#include "tile_map.h"

namespace sd {
namespace {

constexpr int R = 4;          // row blocks per workgroup
constexpr int BS = 64;        // mask block = tile edge along M and K
constexpr int BN = 256;       // output columns per workgroup
constexpr int THREADS = 512;  // 8 waves
constexpr int TILE = BS * BS * 2;              // bytes of one 64 x 64 tile (rows of 128 B)
constexpr int MAX_STEPS = 1024;
// step table: one uint32 per step of the union walk, reduction block | keep bits << 16 (four bits per row block
// of the workgroup: which 32 x 32 quadrants of its tile are kept; all four unless the mask has block size 32),
// followed by STEP_PAD zero entries so that look-ahead reads past the end are harmless
constexpr int STEP_PAD = 4;
// Shape of a DSD workgroup: RH groups of RW row blocks x NS column slices of NT * 32 columns; wave
// (rh, ns) multiplies its slice of the W tile with the kept X tiles of its RW row blocks.  Waves (rh, ns)
// with equal ns share a SIMD, so a SIMD's MFMA work per step depends on how many row blocks keep the K
// block, not on which.
//   DsdBig  256 rows x 256 columns, 8 waves of 2 row blocks x 64 columns: the least operand traffic per
//           MFMA; what large products run on
//   DsdMid  128 rows x 128 columns, 8 waves of 1 row block x 32 columns: four times as many workgroups, for
//           products whose 256 x 256 tiles would leave most of the 256 CUs without one; two workgroups fit
//           a CU (72 KB of LDS, under 128 VGPRs).  More LDS fragment traffic per MFMA (1.5 KB against
//           0.75 KB), which is why the big shape wins as soon as it can fill the chip
template <int RH_, int NS_, int NT_, int RW_ = 2, int NST_ = 2>
struct DsdShape {
  static constexpr int RH = RH_, NS = NS_, NT = NT_, RW = RW_;  // RW: row blocks a wave owns (2 or 1)
  static constexpr int NST = NST_;           // stages of LDS (steps whose tiles are resident or on their way)
  static constexpr int R = RW * RH;          // row blocks per workgroup
  static constexpr int NW = RH * NS;         // waves
  static constexpr int THREADS = 64 * NW;
  static constexpr int BN = NS * NT * 32;    // output columns per workgroup
  static constexpr int B_TILE = BN * BS * 2; // bytes of the W tile of one step
  static constexpr int A_OFF = B_TILE;       // X tiles follow it
  static constexpr int STAGE = B_TILE + R * TILE;
  static constexpr int BL = B_TILE / 1024 / NW;  // wave-wide 1 KB loads per wave for the W tile
  static constexpr int AL = TILE / 1024 / NW;    // ... for one X tile
  static constexpr int SMEM_STEPS = NST * STAGE;
  static constexpr int SMEM_SCRATCH = SMEM_STEPS + 4 * (MAX_STEPS + STEP_PAD);  // uint32 per K block while merging
  static constexpr int SMEM_BYTES = SMEM_SCRATCH + 4 * MAX_STEPS + 16;
  static_assert(BL >= 1 && AL >= 1 && BL * NW * 1024 == B_TILE && AL * NW * 1024 == TILE, "loads must divide evenly");
};
using DsdBig = DsdShape<2, 4, 2>;  // (8 waves of 1 row block x 128 columns, DsdShape<4, 2, 4, 1>, measured 2-4 % slower)
using DsdMid = DsdShape<2, 4, 1, 1>;
// The same on aligned operands with four stages: a step of this shape is 16 MFMAs per wave, far shorter than a load's
// way through L2 and memory, so three steps are kept in flight instead of one (one workgroup per CU: 136 KB of LDS)
using DsdMidDeep = DsdShape<2, 4, 1, 1, 4>;
// 256 rows x 128 columns, 8 waves: the shape of the implicit-GEMM convolution, whose input patch has to
// fit in LDS next to the stages
using DsdConv = DsdShape<2, 4, 1>;
constexpr int CONV_PATCH_MAX = 163840 - DsdConv::SMEM_BYTES - 16;  // bytes left for patch + column table
constexpr int CONV_T_PATCH_MAX = 24 * 1024;  // weight gradient: bytes of one step's copy of its input rows
__device__ inline int step_block(uint32_t e) { return (int)(e & 0xffffu); }
__device__ inline uint32_t step_flags(uint32_t e) { return e >> 16; }
__device__ inline uint32_t row_quads(uint32_t flags, int r) { return (flags >> (4 * r)) & 0xfu; }  // of row block r
__device__ inline uint32_t uniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane(v); }

typedef __attribute__((address_space(3))) void lds_void;

// One wave-wide 1 KB direct global->LDS load: lane i's 16 bytes land at lds_dst + 16*i (lds_dst is
// wave-uniform and goes through M0).  Issued as inline assembly on purpose: when the compiler sees a
// direct-to-LDS load in flight it stops counting LDS reads precisely (every wait becomes
// lgkmcnt(0), and transpose reads get a vmcnt(0) in front), which serialises the fragment reads with
// the MFMAs.  Written this way the loads are invisible to its counters; the kernels wait for them
// themselves with s_waitcnt vmcnt(0) before the barrier that publishes a stage.
// lds_dst is the destination's LDS byte address (lds_address() of a pointer, plus wave-uniform offsets): kept as
// an integer in scalar registers, so no pointer conversion is made per load.
__device__ inline uint32_t lds_address(const void* p) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_void*)p);
}
__device__ inline void load16_to_lds(const void* g, uint32_t lds_dst) {
  const uint32_t a = uniform(lds_dst);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(a) : "memory");
}
// The same with the address split into a wave-uniform 64-bit base (SGPRs) and a 32-bit per-lane byte
// offset: half the VGPR reads per load and no 64-bit VALU add to form the lane addresses.
__device__ inline void load16_to_lds(const char* base, uint32_t lane_off, uint32_t lds_dst) {
  const uint64_t b = (uint64_t)(uintptr_t)base;
  const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t a = uniform(lds_dst);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sb), "s"(a)
               : "memory");
}

// Waits until at most n of the wave's loads are outstanding (they return in order: everything issued before the last
// n has landed).  n is wave-uniform and only known at run time, the instruction takes an immediate.
__device__ inline void wait_loads_all_but(int n) {
  if (n >= 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  else if (n == 11) asm volatile("s_waitcnt vmcnt(11)" ::: "memory");
  else if (n == 10) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
  else if (n == 9) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
  else if (n == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (n == 7) asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
  else if (n == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (n == 5) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  else if (n == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (n == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
  else if (n == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else if (n == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// 4 reduction-consecutive halfs of one column, gathered from 4 LDS rows (see the file comment)
__device__ inline u32x2 lds_read_tr(const char* p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
  return __builtin_bit_cast(u32x2, v);
}

// Chunk swizzles of tiles kept in memory order [reduction row][columns] (read with ds_read_b64_tr_b16).  One
// transposing read takes, per 16-lane group, 4 consecutive reduction rows x 32 bytes, and the groups of a wave
// are 8 reduction rows apart.  A 64-column tile has rows of 128 B: rows r and r+2 would share banks, so bit 2 of
// the 16-byte chunk index follows bit 1 of the row; rows 8 apart would too, so bit 1 follows bit 3 of the row.
// Rows of a 256- or 128-column tile are a multiple of 256 B apart: chunk bits 2-3 follow the row's low two bits.
__device__ inline int swz_x(int row) { return (((row >> 1) & 1) << 2) ^ (((row >> 3) & 1) << 1); }
__device__ inline int swz_w(int row) { return ((row & 3) << 2) ^ (((row >> 3) & 1) << 1); }

// TRANS = false: A[row][red], B[col][red] with the reduction index contiguous (forward / dense)
// TRANS = true : A and B are given as transposed views, the reduction index is the strided one (dW)
// In both cases "Mb" counts the row blocks of A (of X^T for dW) and "Kb" the reduction blocks.
// CM = C is column-major: the MFMA operands are swapped so that lanes run along C's rows
// RAGGED = some of M, N, K is not a multiple of 64; a separate instance so that the aligned case carries
// none of the edge handling
// IMPLICIT = A is the patch matrix of a convolution, never materialised: the workgroup copies the input rows
// its 256 output positions touch (all channels) into LDS once, and per step builds the kept 64 x 64 tiles of
// the patch matrix from that copy, in the layout the fragment reads expect, instead of loading them.  A
// table in LDS maps a patch-matrix column (c, r, s) to its offset in the copy; whether
// a tap falls outside the image never has to be asked: the copy carries a halo of zeros.
// IMPLICIT = 2: the same with a copy per step that holds only the channels of the step's 64 columns (any number
// of input channels fits); the reduction-strided instance (the weight gradient) always works that way.
// bid: the workgroup's index in the launch order of this product; the reduction is split nsplit ways and this
// workgroup takes part `split` (the kernels below pass their block indices; the fused backward launch its own)
// ms: where the mask comes from when the kept lists do not exist yet (the forward launch that also builds them);
// the keep bits of the workgroup's row blocks are then evaluated from it directly, g.row_ptr is not read
template <typename T, bool TRANS, bool CM, bool RAGGED, typename S, int IMPLICIT = 0>
__device__ __forceinline__ void dsd_body(const GemmArgs& g, int tiles_m, int tiles_n, int Mb, int Kb_all,
                                         const ImplicitConv& cg, const int bid, const int nsplit, const int split,
                                         const MaskSrc* ms = nullptr) {
  static_assert(!IMPLICIT || (S::R == 4 && S::THREADS == 512), "the gather assumes 512 threads x 4 row blocks");
  static_assert(S::R <= 4, "a step's keep bits are four per row block in 16 bits");
  constexpr int R = S::R, BN = S::BN, THREADS = S::THREADS, NT = S::NT, STAGE = S::STAGE, A_OFF = S::A_OFF;
  constexpr int BL = S::BL, AL = S::AL, RW = S::RW;
  constexpr bool STEP_COPIES = IMPLICIT != 0 && (TRANS || IMPLICIT == 2);  // input rows copied per step
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t smem_a = lds_address(smem);
  uint32_t* step_e = reinterpret_cast<uint32_t*>(smem + S::SMEM_STEPS);
  uint32_t* scratch = reinterpret_cast<uint32_t*>(smem + S::SMEM_SCRATCH);
  int* nsteps_p = reinterpret_cast<int*>(smem + S::SMEM_SCRATCH + 4 * MAX_STEPS);

  int tm, tn;
  tile_of_block<DSD_GROUP_M>(bid, tiles_m, tiles_n, tm, tn);
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int wave_u = (int)uniform((uint32_t)wave);  // the same in a scalar register, for load addresses
  const int ns = wave % S::NS;  // column slice
  const int rh = wave / S::NS;  // row-block pair
  const int rb0 = tm * R;   // first row block
  const int64_t n0 = (int64_t)tn * BN;
  const int nvalid = (int)((g.N - n0) < BN ? (g.N - n0) : BN);  // columns of this tile inside C
  // split reduction: part `split` takes the reduction blocks [kb_lo, kb_lo + Kb) and leaves an fp32 partial
  const int kb_lo = (int)((int64_t)Kb_all * split / nsplit);
  const int Kb = (int)((int64_t)Kb_all * (split + 1) / nsplit) - kb_lo;

  // ---- union of the kept lists of the 4 row blocks: (K block, 4-bit keep flags) per step -------
  for (int i = tid; i < Kb; i += THREADS) scratch[i] = 0;
  __syncthreads();
  if (ms) {
    const int rows = (rb0 + R <= Mb) ? R : Mb - rb0;
    for (int i = tid; i < rows * Kb; i += THREADS) {
      const int r = i / Kb, k = i - r * Kb;
      const uint32_t q = ms->merge == 2 ? ms->kept_quads(rb0 + r, kb_lo + k) : (ms->dropped(rb0 + r, kb_lo + k) ? 0u : 0xfu);
      if (q) atomicOr(&scratch[k], q << (4 * r));
    }
  } else if (g.row_ptr) {
    for (int r = 0; r < R; ++r) {
      if (rb0 + r >= Mb) break;
      const int beg = g.row_ptr[rb0 + r], end = g.row_ptr[rb0 + r + 1];
      for (int i = beg + tid; i < end; i += THREADS) {
        const int32_t e = g.col_idx[i];
        const int k = entry_block(e) - kb_lo;
        if (k >= 0 && k < Kb) atomicOr(&scratch[k], (IMPLICIT ? 0xfu : entry_quads(e)) << (4 * r));
      }
    }
  } else {
    const int rows = (rb0 + R <= Mb) ? R : Mb - rb0;
    const uint32_t all = rows >= 4 ? 0xffffu : ((1u << (4 * rows)) - 1u);
    for (int i = tid; i < Kb; i += THREADS) scratch[i] = all;
  }
  __syncthreads();
  if (wave == 0) {
    int base = 0;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int k0 = 0; k0 < Kb; k0 += 64) {
      const int k = k0 + lane;
      const uint32_t f = (k < Kb) ? scratch[k] : 0u;
      const uint64_t bal = __ballot(f != 0);
      if (f) {
        const int pos = base + __popcll(bal & lt);
        step_e[pos] = (uint32_t)(kb_lo + k) | (f << 16);
      }
      base += __popcll(bal);
    }
    if (lane < STEP_PAD) step_e[base + lane] = 0u;
    if (lane == 0) *nsteps_p = base;
  }
  __syncthreads();
  const int nsteps = *nsteps_p;

  // ---- implicit GEMM: input rows -> LDS with a zero halo, column table -------------------------------
  // Patch layout: [channel][input row][8 zero halfs | W image halfs]; the zero group in front of a row is
  // the left halo of that row and the right halo of the row before it, rows outside the image are zeros,
  // so a tap never needs a bounds test: element (m, k) of the patch matrix is
  // patch[base(m) + ktab[k]] with base(m) = (output row of m inside the workgroup) * PW + 8 + q - pad_w
  // and ktab[k] = ((c * PR + r) * PW + s) for column k = (c, r, s), both kept as byte offsets.
  uint16_t* patch = reinterpret_cast<uint16_t*>(smem + ((S::SMEM_BYTES + 15) & ~15));
  uint16_t* ktab = nullptr;
  uint32_t gat_base[4];  // byte offset of (this thread's tile row, tap 0) in the patch, per row block
  const int gat_row = tid / 8, gat_pc = tid % 8;  // the tile row and physical 16-byte chunk this thread builds
  [[maybe_unused]] auto div = [](int x, uint32_t magic) { return magic ? (int)__umulhi((uint32_t)x, magic) : x; };
  if constexpr (IMPLICIT == 1 && !TRANS) {
    const int img = rb0 / cg.blocks_per_img;
    const int p0 = (rb0 - img * cg.blocks_per_img) * cg.rpb;  // first output row of the workgroup
    const int h0 = p0 * cg.sth - cg.pad_h;                     // input row of patch row 0
    const int spr = cg.W / 8, spc = cg.PR * spr;               // 16-byte segments per row, per channel
    const int total = cg.C * spc;
    const int rows = cg.C * cg.PR;
    ktab = patch + rows * cg.PW + 8;
    const uint16_t* ximg = cg.x + (int64_t)img * cg.sn;
    constexpr int MAXSEG = (CONV_PATCH_MAX / 16 + THREADS - 1) / THREADS;
    u32x4 v[MAXSEG];
    int dst[MAXSEG];
#pragma unroll
    for (int j = 0; j < MAXSEG; ++j) {  // all loads first, so that their latencies overlap
      const int seg = tid + j * THREADS;
      const int c = div(seg, cg.m_spc), rem = seg - c * spc;
      const int row = div(rem, cg.m_spr), w8 = rem - row * spr;
      const int h = h0 + row;
      dst[j] = seg < total ? (c * cg.PR + row) * cg.PW + 8 + w8 * 8 : -1;
      v[j] = u32x4{0u, 0u, 0u, 0u};
      if (seg < total && h >= 0 && h < cg.H)
        v[j] = *reinterpret_cast<const u32x4*>(ximg + c * cg.sc + h * cg.sh + w8 * 8);
    }
    for (int m = tid; m <= rows; m += THREADS)  // the halo groups, one more after the last row
      *reinterpret_cast<u32x4*>(patch + m * cg.PW) = u32x4{0u, 0u, 0u, 0u};
    for (int k = tid; k < Kb_all * BS; k += THREADS) {
      const int c = div(k, cg.m_RS), tap = k - c * cg.RS;
      const int rr = div(tap, cg.m_S), ss = tap - rr * cg.S;
      // columns past the last one read anything readable: their fragments are zeroed before the MFMAs
      ktab[k] = k < cg.K ? (uint16_t)(((c * cg.PR + rr * cg.dlh) * cg.PW + ss * cg.dlw) * 2) : (uint16_t)0;
    }
    const int prow = div(gat_row, cg.m_Q), q = gat_row - prow * cg.Q;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      gat_base[r] = (uint32_t)(((r * cg.rpb + prow) * cg.sth * cg.PW + 8 + q * cg.stw - cg.pad_w) * 2);
#pragma unroll
    for (int j = 0; j < MAXSEG; ++j)
      if (dst[j] >= 0) *reinterpret_cast<u32x4*>(patch + dst[j]) = v[j];
    __syncthreads();
  }
  // Weight gradient (reduction-strided instance): the reduction runs over output positions, so every step
  // has its own 64 positions (rpb output rows of one image) and its own copy of the input rows they touch --
  // only the channels of the workgroup's 256 patch-matrix columns, PR = rpb + R - 1 rows each.  Two copies
  // alternate: the one for step s+2 is fetched into registers at the top of step s and written to LDS at
  // its end, the tiles of step s+1 are built from the other while step s computes.  The tile a row block
  // keeps is [64 positions][its 64 columns], rows of 128 bytes, in the swizzle of the transposing reads.
  // The forward's per-step form (IMPLICIT == 2) does the same with the 256 positions of the workgroup fixed and
  // the channels moving: a step's copy holds the <= 64 / (R*S) + 2 channels its 64 columns touch.
  constexpr int TSEG = STEP_COPIES ? (CONV_T_PATCH_MAX / 16 + THREADS - 1) / THREADS : 1;
  [[maybe_unused]] u32x4 tp_v[TSEG];      // a step's input rows on their way to LDS
  [[maybe_unused]] int tp_dst[TSEG];      // where this thread's segments go in a copy (halfs), -1 = none
  [[maybe_unused]] int64_t tp_src[TSEG];  // and where they come from, relative to (image, input row h0)
  [[maybe_unused]] int tp_row[TSEG];      // their row in the copy (forward: their input row in the image)
  [[maybe_unused]] int tp_c[TSEG];        // forward: their channel, counted from the step's first
  [[maybe_unused]] uint16_t* patch1 = nullptr;
  [[maybe_unused]] const uint16_t* tcopy = patch;  // the copy the next step's tiles are built from
  if constexpr (IMPLICIT == 2 && !TRANS) {
    // cg.units == 1: the four row blocks are 4 * rpb consecutive output rows of one image and share one run of
    // PR = 4 * rpb + R - 1 input rows per channel; cg.units == 4 (P * Q not a multiple of 256, e.g. 8 x 8 images):
    // every row block has its own PR = rpb + R - 1 rows per channel, possibly from another image.
    const int nch = (BS + cg.RS - 2) / cg.RS + 1;  // channels 64 consecutive columns can touch
    const int spr = cg.W / 8, spc = cg.PR * spr;
    const int per_unit = nch * spc, total = cg.units * per_unit, rows = cg.units * nch * cg.PR;
    patch1 = patch + cg.patch_stride;
    ktab = patch1 + cg.patch_stride;
#pragma unroll
    for (int j = 0; j < TSEG; ++j) {
      const int seg = tid + j * THREADS;
      const int u = (seg >= per_unit ? 1 : 0) + (seg >= 2 * per_unit ? 1 : 0) + (seg >= 3 * per_unit ? 1 : 0);
      const int su = seg - u * per_unit;
      const int c = div(su, cg.m_spc), rem = su - c * spc;
      const int row = div(rem, cg.m_spr), w8 = rem - row * spr;
      const int rb = rb0 + u;
      const int img = rb / cg.blocks_per_img;
      const int h = (rb - img * cg.blocks_per_img) * cg.rpb * cg.sth - cg.pad_h + row;  // input row of the segment
      tp_dst[j] = (seg < total && rb < Mb) ? ((u * nch + c) * cg.PR + row) * cg.PW + 8 + w8 * 8 : -1;
      tp_src[j] = (int64_t)img * cg.sn + (int64_t)c * cg.sc + (int64_t)h * cg.sh + w8 * 8;
      tp_row[j] = h;
      tp_c[j] = c;
    }
    for (int m = tid; m <= rows; m += THREADS) {  // the halo groups of both copies; the steps never write them
      *reinterpret_cast<u32x4*>(patch + m * cg.PW) = u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(patch1 + m * cg.PW) = u32x4{0u, 0u, 0u, 0u};
    }
    for (int k = tid; k < Kb_all * BS; k += THREADS) {
      const int c = div(k, cg.m_RS), tap = k - c * cg.RS;
      const int rr = div(tap, cg.m_S), ss = tap - rr * cg.S;
      const int c_lo = div(k & ~(BS - 1), cg.m_RS);  // first channel of the column's block = of its step's copy
      ktab[k] = k < cg.K ? (uint16_t)((((c - c_lo) * cg.PR + rr * cg.dlh) * cg.PW + ss * cg.dlw) * 2) : (uint16_t)0;
    }
    const int prow = div(gat_row, cg.m_Q), q = gat_row - prow * cg.Q;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int first_row = cg.units == 1 ? r * cg.rpb * cg.sth : r * nch * cg.PR;  // of row block r in a copy
      gat_base[r] = (uint32_t)(((first_row + prow * cg.sth) * cg.PW + 8 + q * cg.stw - cg.pad_w) * 2);
    }
  }
  if constexpr (IMPLICIT && TRANS) {
    const int k_lo = rb0 * BS;
    const int k_hi = k_lo + R * BS < cg.K ? k_lo + R * BS : cg.K;
    const int c_lo = div(k_lo, cg.m_RS), nch = div(k_hi - 1, cg.m_RS) - c_lo + 1;
    const int spr = cg.W / 8, spc = cg.PR * spr;
    const int total = nch * spc, rows = nch * cg.PR;
    patch1 = patch + cg.patch_stride;
    ktab = patch1 + cg.patch_stride;
#pragma unroll
    for (int j = 0; j < TSEG; ++j) {
      const int seg = tid + j * THREADS;
      const int c = div(seg, cg.m_spc), rem = seg - c * spc;
      const int row = div(rem, cg.m_spr), w8 = rem - row * spr;
      tp_dst[j] = seg < total ? (c * cg.PR + row) * cg.PW + 8 + w8 * 8 : -1;
      tp_src[j] = (int64_t)(c_lo + c) * cg.sc + (int64_t)row * cg.sh + w8 * 8;
      tp_row[j] = row;
    }
    for (int m = tid; m <= rows; m += THREADS) {  // the halo groups of both copies; the steps never write them
      *reinterpret_cast<u32x4*>(patch + m * cg.PW) = u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(patch1 + m * cg.PW) = u32x4{0u, 0u, 0u, 0u};
    }
    for (int kl = tid; kl < R * BS; kl += THREADS) {
      const int k = k_lo + kl;
      const int c = div(k, cg.m_RS), tap = k - c * cg.RS;
      const int rr = div(tap, cg.m_S), ss = tap - rr * cg.S;
      // columns past the last one belong to rows of the result that are not stored
      ktab[kl] = k < cg.K ? (uint16_t)((((c - c_lo) * cg.PR + rr * cg.dlh) * cg.PW + ss * cg.dlw) * 2) : (uint16_t)0;
    }
    const int prow = div(gat_row, cg.m_Q), q = gat_row - prow * cg.Q;
    gat_base[0] = (uint32_t)((prow * cg.sth * cg.PW + 8 + q * cg.stw - cg.pad_w) * 2);
  }
  // fetches the input rows of the step with table word `entry` (its reduction block is a block of 64 positions)
  [[maybe_unused]] auto tpatch_load = [&](uint32_t entry) {
    if constexpr (!TRANS) {  // forward: the step's reduction block is a block of 64 columns, i.e. a run of channels
      const int c_lo = div(step_block(entry) * BS, cg.m_RS);
      const uint16_t* src = cg.x + (int64_t)c_lo * cg.sc;
#pragma unroll
      for (int j = 0; j < TSEG; ++j) {
        tp_v[j] = u32x4{0u, 0u, 0u, 0u};
        if (tp_dst[j] >= 0 && tp_row[j] >= 0 && tp_row[j] < cg.H && c_lo + tp_c[j] < cg.C)
          tp_v[j] = *reinterpret_cast<const u32x4*>(src + tp_src[j]);
      }
      return;
    }
    const int mb = step_block(entry);
    const int img = mb / cg.blocks_per_img;
    const int h0 = (mb - img * cg.blocks_per_img) * cg.rpb * cg.sth - cg.pad_h;
    const uint16_t* src = cg.x + (int64_t)img * cg.sn + (int64_t)h0 * cg.sh;
#pragma unroll
    for (int j = 0; j < TSEG; ++j) {
      const int h = h0 + tp_row[j];
      tp_v[j] = u32x4{0u, 0u, 0u, 0u};
      if (tp_dst[j] >= 0 && h >= 0 && h < cg.H) tp_v[j] = *reinterpret_cast<const u32x4*>(src + tp_src[j]);
    }
  };
  [[maybe_unused]] auto tpatch_store = [&](uint16_t* copy) {
#pragma unroll
    for (int j = 0; j < TSEG; ++j)
      if (tp_dst[j] >= 0) *reinterpret_cast<u32x4*>(copy + tp_dst[j]) = tp_v[j];
  };
  // this thread's 16 bytes of the tile [64 positions][64 columns of row block r] from a step's copy
  [[maybe_unused]] auto gather_tile_t = [&](int r, const uint16_t* copy, char* tile) {
    const int lc = gat_pc ^ swz_x(gat_row);  // logical chunk: columns r*64 + lc*8 .. +7 of the workgroup
    const u16x8 off = *reinterpret_cast<const u16x8*>(ktab + r * BS + lc * 8);
    const char* pb = reinterpret_cast<const char*>(copy) + gat_base[0];
    uint32_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = *reinterpret_cast<const uint16_t*>(pb + off[e]);
    *reinterpret_cast<u32x4*>(tile + gat_row * 128 + gat_pc * 16) =
        u32x4{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
  };
  // builds this thread's 16 bytes of the patch-matrix tile (row block r of the workgroup, reduction block kb)
  auto gather_tile = [&](int r, int kb, char* tile) {
    const int lc = gat_pc ^ ((gat_row >> 1) & 7);  // logical chunk: columns kb*64 + lc*8 .. +7
    const u16x8 off = *reinterpret_cast<const u16x8*>(ktab + kb * BS + lc * 8);
    const char* pb = reinterpret_cast<const char*>(IMPLICIT == 2 ? tcopy : patch) + gat_base[r];
    uint32_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = *reinterpret_cast<const uint16_t*>(pb + off[e]);
    *reinterpret_cast<u32x4*>(tile + gat_row * 128 + gat_pc * 16) =
        u32x4{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
  };

  // ---- per-lane constants ---------------------------------------------------------------------
  // fragment reads for v_mfma_f32_16x16x32: lane l supplies row (column of C) l%16 of its operand and the 8
  // reduction elements 8*(l/16) .. +7 of a 32-wide reduction step kk
  int a_off[2], b_off[2];  // byte offsets inside an X tile / the W tile, per reduction step; 16-row tile 0
  if (!TRANS) {
    // rows of 128 B; lane -> tile row lane%16 (+16*tile), logical 16 B chunk 4*kk + lane/16,
    // physical chunk = logical ^ ((row>>1)&7): 16 consecutive lanes hit all 64 banks once
    const int fr_row = lane % 16;
    const int fr_sw = (lane >> 1) & 7;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int ko = ((4 * kk + lane / 16) ^ fr_sw) * 16;
      a_off[kk] = fr_row * 128 + ko;
      b_off[kk] = (ns * 32 * NT + fr_row) * 128 + ko;
    }
  } else {
    // rows are reduction indices.  16-lane group b = lane/16, lane = 16b + 4e + j reads 8 bytes of
    // row (8*b + e) [+32*kk, +4 for the second half], columns 4j .. +3 [+16*tile].
    const int b4 = lane / 16, e = (lane % 16) / 4, j = lane % 4;
    const int row = 8 * b4 + e;
    // X tile rows are 128 B (8 chunks), W tile rows 2*BN bytes (32 or 16 chunks); see swz_x / swz_w
    const int a_ch = (j / 2) ^ swz_x(row);
    const int b_ch = (ns * 4 * NT + j / 2) ^ swz_w(row);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      a_off[kk] = (32 * kk + row) * 128 + a_ch * 16 + (j % 2) * 8;
      b_off[kk] = (32 * kk + row) * (2 * BN) + b_ch * 16 + (j % 2) * 8;
    }
  }

  // global -> LDS: every wave-wide load fills 1 KB of LDS in lane order.  Per-lane byte offsets are
  // fixed for the whole kernel; per step only a wave-uniform base moves.
  uint32_t b_lane[BL], a_lane[AL];
  bool b_valid[BL];  // the lane's 16 bytes of the W tile lie inside the matrix (a tile may overhang N)
  // Ragged edges (all in units of 8 elements, the 16 bytes of one lane's load).  A 64-block that overhangs
  // the matrix along the strided index of its operand is fetched with the overhanging rows redirected to
  // its last valid row; one that overhangs along the contiguous index with the overhanging 16-byte chunks
  // redirected to its first chunk.  Either way every load stays inside the matrix and lands in the LDS slot
  // of the element it stands in for.  What stands in along M (or N) only ever reaches accumulator rows
  // (columns) that are not stored; what stands in along the reduction is zeroed in the fragments before
  // it reaches an MFMA.
  const int m_valid = (int)(g.M % BS), k_valid = (int)(g.K % BS);
  const int r_tail = (RAGGED && m_valid) ? Mb - 1 - rb0 : -1;   // patch row block that is ragged
  const int kb_tail = (RAGGED && k_valid) ? Kb_all - 1 : -1;    // reduction block that is ragged
  // what to add (mod 2^32) to a lane's offset for a block ragged along M / along the reduction: the row and
  // the chunk term of an offset are redirected independently, so the two corrections add up
  uint32_t a_delta_m[AL], a_delta_k[AL], b_delta_k[BL];
  const char* a_tile0;  // first X tile of the patch at reduction block 0
  const char* b_tile0;  // W tile at reduction block 0
  int64_t red_stride;   // bytes between consecutive reduction blocks
  uint32_t a_rstride;   // bytes between consecutive row blocks of the patch
  if (!TRANS) {
    // 8 tile rows per load; lane -> (row lane/8, physical chunk lane%8)
    const int ld_row = lane / 8, ld_pch = lane % 8;
    // element offset of the lane's chunk; the swizzle (the LDS slot) stays that of `row`
    auto chunk_at = [&](int row, int64_t ld, int rows_valid, bool clamp_row, bool clamp_k) {
      const int rc = (clamp_row && row >= rows_valid) ? rows_valid - 1 : row;
      int c = ld_pch ^ ((row >> 1) & 7);
      if (clamp_k && c * 8 >= k_valid) c = 0;
      return (uint32_t)(rc * ld + c * 8) * 2u;
    };
#pragma unroll
    for (int jj = 0; jj < BL; ++jj) {
      const int row = (wave * BL + jj) * 8 + ld_row;
      b_lane[jj] = chunk_at(row, g.b.sr, 0, false, false);
      b_delta_k[jj] = chunk_at(row, g.b.sr, 0, false, kb_tail >= 0) - b_lane[jj];
      b_valid[jj] = row < nvalid;
    }
#pragma unroll
    for (int i = 0; i < AL; ++i) {
      const int row = (wave * AL + i) * 8 + ld_row;
      a_lane[i] = chunk_at(row, g.a.sr, 0, false, false);
      a_delta_m[i] = chunk_at(row, g.a.sr, m_valid, r_tail >= 0, false) - a_lane[i];
      a_delta_k[i] = chunk_at(row, g.a.sr, 0, false, kb_tail >= 0) - a_lane[i];
    }
    a_tile0 = reinterpret_cast<const char*>(g.a.ptr + (int64_t)rb0 * BS * g.a.sr);
    b_tile0 = reinterpret_cast<const char*>(g.b.ptr + n0 * g.b.sr);
    red_stride = BS * 2;
    a_rstride = (uint32_t)(BS * g.a.sr) * 2u;
  } else {
    // W tile: reduction rows of 2*BN bytes, 2 or 4 of them per load; X tiles: 8 reduction rows of 128 B per load
    constexpr int CPR = BN / 8;  // 16-byte chunks per W tile row
#pragma unroll
    for (int jj = 0; jj < BL; ++jj) {
      const int row = (wave * BL + jj) * (64 / CPR) + lane / CPR;
      const int col = ((lane % CPR) ^ swz_w(row)) * 8;
      b_lane[jj] = (uint32_t)(row * g.b.sc + col) * 2u;
      b_valid[jj] = col < nvalid;
      const int rc = (kb_tail >= 0 && row >= k_valid) ? k_valid - 1 : row;
      b_delta_k[jj] = (uint32_t)(rc * g.b.sc + col) * 2u - b_lane[jj];
    }
    auto chunk_at = [&](int row, bool clamp_m, bool clamp_k) {
      const int rc = (clamp_k && row >= k_valid) ? k_valid - 1 : row;
      int c = (lane % 8) ^ swz_x(row);
      if (clamp_m && c * 8 >= m_valid) c = 0;
      return (uint32_t)(rc * g.a.sc + c * 8) * 2u;
    };
#pragma unroll
    for (int i = 0; i < AL; ++i) {
      const int row = (wave * AL + i) * 8 + lane / 8;
      a_lane[i] = chunk_at(row, false, false);
      a_delta_m[i] = chunk_at(row, r_tail >= 0, false) - a_lane[i];
      a_delta_k[i] = chunk_at(row, false, kb_tail >= 0) - a_lane[i];
    }
    a_tile0 = reinterpret_cast<const char*>(g.a.ptr + (int64_t)rb0 * BS);
    b_tile0 = reinterpret_cast<const char*>(g.b.ptr + n0);
    red_stride = (int64_t)BS * g.a.sc * 2;  // == BS * g.b.sc * 2 only if the leading dimensions agree
    a_rstride = BS * 2;
  }
  const int64_t b_red_stride = TRANS ? (int64_t)BS * g.b.sc * 2 : (int64_t)BS * 2;

  // with_w: the W tile too; rowsel: bit r = the X tile of row block r may be loaded (if the step keeps it)
  auto issue_loads = [&](uint32_t entry, int stage, bool with_w = true, uint32_t rowsel = 0xfu) {  // entry: wave-uniform step table word
    const int kb = step_block(entry);
    const uint32_t fl = step_flags(entry);
    [[maybe_unused]] char* st = smem + stage * STAGE;
    const uint32_t st_a = smem_a + (uint32_t)(stage * STAGE);
    const char* bp = b_tile0 + kb * b_red_stride;
    const char* ap = a_tile0 + kb * red_stride;
    const bool red_tail = RAGGED && kb == kb_tail;  // wave-uniform
#pragma unroll
    for (int jj = 0; jj < BL; ++jj)
      if (with_w && b_valid[jj]) {
        uint32_t off = b_lane[jj];
        if (RAGGED) off += red_tail ? b_delta_k[jj] : 0u;
        load16_to_lds(bp, off, st_a + (uint32_t)((wave_u * BL + jj) * 1024));
      }
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (row_quads(fl, r) && ((rowsel >> r) & 1u)) {
        if constexpr (IMPLICIT && !TRANS) {
          gather_tile(r, kb, st + A_OFF + r * TILE);
          continue;
        }
        if constexpr (IMPLICIT && TRANS) {
          gather_tile_t(r, tcopy, st + A_OFF + r * TILE);
          continue;
        }
#pragma unroll
        for (int i = 0; i < AL; ++i) {
          uint32_t off = a_lane[i];
          if (RAGGED) off += (r == r_tail ? a_delta_m[i] : 0u) + (red_tail ? a_delta_k[i] : 0u);
          load16_to_lds(ap + r * a_rstride, off, st_a + (uint32_t)(A_OFF + r * TILE + (wave_u * AL + i) * 1024));
        }
      }
  };
  // zeroes the elements of a fragment whose reduction index (32*kk + 8*(lane/16) + 0..7 inside the
  // block) is not below k_valid
  auto mask_fragment = [&](u32x4& f, int kk) {
    const int n = k_valid - (32 * kk + 8 * (lane / 16));  // valid elements among the lane's 8
    f.x &= n >= 2 ? ~0u : (n == 1 ? 0xffffu : 0u);
    f.y &= n >= 4 ? ~0u : (n == 3 ? 0xffffu : 0u);
    f.z &= n >= 6 ? ~0u : (n == 5 ? 0xffffu : 0u);
    f.w &= n >= 8 ? ~0u : (n == 7 ? 0xffffu : 0u);
  };

  constexpr int NT16 = 2 * NT;  // 16-column MFMA tiles of the wave's column slice
  f32x4 acc[RW][4][NT16];  // [row block of the wave][16-row tile][16-column tile]
#pragma unroll
  for (int a = 0; a < RW; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int c = 0; c < NT16; ++c)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[a][b][c][v] = 0.f;

  // fragment reads for one 32-wide reduction step kk: the four 16-row tiles of an X tile / the 16-column
  // tiles of the W slice
  auto read_a = [&](const char* at, int kk, u32x4 (&dst)[4]) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      if (!TRANS) {
        dst[mt] = *reinterpret_cast<const u32x4*>(at + a_off[kk] + mt * 16 * 128);
      } else {
        // the 16-column tile sits in bits 1-2 of the chunk index, i.e. 32 bytes, under the XOR swizzle
        const char* p = at + (a_off[kk] ^ (mt * 32));
        const u32x2 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * 128);
        dst[mt] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
    }
  };
  auto read_b = [&](const char* st, int kk, u32x4 (&dst)[NT16][2]) {
#pragma unroll
    for (int nt = 0; nt < NT16; ++nt) {
      if (!TRANS) {
        dst[nt][kk] = *reinterpret_cast<const u32x4*>(st + b_off[kk] + nt * 16 * 128);
      } else {
        const char* p = st + (b_off[kk] ^ (nt * 32));
        const u32x2 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * 2 * BN);
        dst[nt][kk] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
    }
  };

  // One step of MFMA work for this wave, specialised on which of its two row blocks keep the K block
  // (MINE = 1, 2 or 3).  The work is a chain of units (row block, kk); the LDS reads of unit u+1 are
  // issued before the MFMAs of unit u so that their latency hides behind 4 * NT16 MFMAs.  The W
  // fragments are read during the first row block's units and stay in registers for the second.
  // quads: the keep bits of the wave's row blocks (four each); a quadrant that is not kept is zeroed in the X
  // fragments, in the ragged-edge instance only (masks of block size 32 run on it)
  auto compute = [&](auto mine_c, const char* st, bool mid_loads, uint32_t mid_entry, int mid_stage,
                     bool red_tail, uint32_t quads) {
    constexpr int MINE = decltype(mine_c)::value;
    constexpr int NR = (MINE == 3) ? 2 : 1;
    constexpr int R0 = (MINE == 2) ? 1 : 0;
    u32x4 bf[NT16][2];
    const char* at0 = st + A_OFF + (RW * rh + R0) * TILE;
    u32x4 af[2][4];
    read_b(st, 0, bf);
    read_a(at0, 0, af[0]);
#pragma unroll
    for (int u = 0; u < NR * 2; ++u) {
      const int rr = R0 + u / 2, kk = u % 2;
      if (u + 1 < NR * 2) {
        const int kk1 = (u + 1) % 2;
        if (u + 1 < 2) read_b(st, kk1, bf);
        read_a(at0 + ((u + 1) / 2) * TILE, kk1, af[(u + 1) & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (RAGGED && g.quads) {  // a mask of block size 32: zero the 32 x 32 quadrants of the tile that are dropped
        const uint32_t q = row_quads(quads, rr);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          if (!((q >> (2 * (mt / 2) + kk)) & 1u)) af[u & 1][mt] = u32x4{0u, 0u, 0u, 0u};
      }
      if (RAGGED && red_tail) {  // ragged reduction block: nothing past the end may reach the MFMAs
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) mask_fragment(af[u & 1][mt], kk);
        if (u < 2) {
#pragma unroll
          for (int nt = 0; nt < NT16; ++nt) mask_fragment(bf[nt][kk], kk);
        }
      }
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT16; ++nt)
          acc[rr][mt][nt] = T::mfma16(af[u & 1][mt], bf[nt][kk], acc[rr][mt][nt]);  // measured 2-3 % faster than (bf, af)
      __builtin_amdgcn_sched_barrier(0);
      if (u == NR - 1 && mid_loads) issue_loads(mid_entry, mid_stage);
    }
  };

  // Table words are read two steps ahead into a VGPR and made uniform a step later, when the read has
  // long returned: a read-and-wait at the top of a step would put an LDS round trip in front of its MFMAs.
  const bool late = __builtin_amdgcn_readfirstlane(rh) != 0;
  uint32_t e_cur = uniform(step_e[0]), e_next = uniform(step_e[1]);

  // ---- the step loop of the 256 x 256 shape on aligned operands: the two waves of a SIMD in opposite phases -------
  // Waves w and w + 4 (the two row-block pairs of one column slice) share a SIMD.  A step of a wave is a MEMORY phase -
  // the wave's share of the coming tiles is put on its way, then every fragment of the step is read into registers -
  // followed by a COMPUTE phase that issues nothing but MFMAs.  A barrier ends each phase, and the second group of
  // four waves starts one phase later than the first: whenever one wave of a SIMD stands at a fragment read or a load,
  // the other one feeds the matrix cores.  (With both waves in the same phase the parts of a step add up, because a
  // wave that stands at a memory instruction issues no MFMA behind it: 8192^3 dense forward 0.95 -> 0.82 ms.)
  // Who loads what follows from who reads what first.  Group 0 (row blocks 0-1) reads the W tile of step c in phase
  // 2c, group 1 (row blocks 2-3) in phase 2c + 1; X tiles are read by their own group only.  So, reading step c,
  //   group 0 loads W(c+1) into the other stage          (last read in phase 2c - 1, needed in phase 2c + 2),
  //   group 1 loads X[2-3](c+1) into the other stage     (last read in phase 2c - 1, needed in phase 2c + 3)
  //           and X[0-1](c+2) into the stage it reads    (last read in phase 2c,     needed in phase 2c + 4),
  // and each wave waits for its own loads at the end of the compute phase that follows: every load has a whole
  // phase to land, and with everything kept the two groups issue the same number (8 per wave).
  // Measured against this arrangement and slower: loads behind or between the fragment reads; loads issued by
  // the computing wave, between its MFMAs (+27 % on the dense product: a load holds its wave for 50-60 clocks) or
  // behind them (+12 % dense, nothing gained at p = 0.5).  Every instruction of the memory phase costs its wave four
  // clocks or more, so the loads are kept to one branch per group and six instructions each: the same loads issued
  // from a per-load choice between the groups' code (a few branches and a dozen scalar instructions more per load)
  // cost 20 % of the kernel; the same loads as buffer loads with a scalar offset (three instructions each) gain nothing.
  constexpr bool PINGPONG = IMPLICIT == 0 && !RAGGED && RW == 2 && S::RH == 2 && S::NS == 4 && NT == 2;
  if constexpr (PINGPONG) {
    const int rh_u = __builtin_amdgcn_readfirstlane(rh);
    const bool grp1 = rh_u != 0;
    const int wg = wave_u & 3;  // the wave inside its group
    // per-lane byte offsets of the wave's direct loads (group 0: W tile, group 1: X tiles).  A load fills 1 KB of LDS in
    // lane order; which chunk of which tile row a lane fetches depends on the load's index only through the swizzle bits
    // that index reaches, so a few variants serve all loads and the rest of the address is wave-uniform.
    constexpr int NV = TRANS ? 4 : 2;
    uint32_t ld_off[NV];
    if (!TRANS) {
      // 8 tile rows of 128 B per load; lane -> (row lane/8, physical chunk lane%8); bit 2 of the swizzle is the load's parity
      const int lr = lane / 8, pch = lane % 8;
      const int64_t ld = grp1 ? g.a.sr : g.b.sr;
#pragma unroll
      for (int v = 0; v < NV; ++v) ld_off[v] = (uint32_t)(lr * ld + ((pch ^ (((lr >> 1) & 3) | (v << 2))) * 8)) * 2u;
    } else if (!grp1) {
      // W tile rows are reduction rows of 2*BN bytes, two per load: row = 2i + lane/32; swz_w needs row&3 and bit 3
      const int lr = lane / 32, pch = lane % 32;
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        int c = pch ^ swz_w(2 * (v & 1) + lr + 8 * (v >> 1));
        if (c * 8 >= nvalid) c = 0;  // past N: fetch something readable, those columns are never stored
        ld_off[v] = (uint32_t)(lr * g.b.sc + c * 8) * 2u;
      }
    } else {
      // X tile rows are reduction rows of 128 B, eight per load: row = 8i + lane/8; swz_x needs bit 1 and bit 3
      const int lr = lane / 8, pch = lane % 8;
#pragma unroll
      for (int v = 0; v < NV; ++v) ld_off[v] = (uint32_t)(lr * g.a.sc + ((pch ^ swz_x(lr + 8 * (v & 1))) * 8)) * 2u;
    }
    const int64_t w_step = (TRANS ? 2 * g.b.sc : 8 * g.b.sr) * 2;  // bytes between the rows of consecutive W loads
    const int64_t x_step = (TRANS ? 8 * g.a.sc : 8 * g.a.sr) * 2;  // ... X loads
    const char* b_wave0 = b_tile0 + wg * 8 * w_step;
    const char* a_wave0 = a_tile0 + wg * 2 * x_step;
    auto load_w = [&](uint32_t entry, int stage) {  // the W tile of a step: 32 loads, 8 per wave of group 0
      const char* bp = b_wave0 + step_block(entry) * b_red_stride;
      const uint32_t dst = smem_a + (uint32_t)(stage * STAGE + wg * 8 * 1024);
      // tile rows are columns of C: a wave's 64 are all inside the matrix or all past N (N is a multiple of 64).  One test
      // for all eight loads: a test per load puts every load behind two taken branches (3 % of the kernel).
      if (!TRANS && wg * 64 >= nvalid) return;
#pragma unroll
      for (int jj = 0; jj < 8; ++jj)
        load16_to_lds(bp + jj * w_step, ld_off[TRANS ? ((jj & 1) | (((jj >> 2) & 1) << 1)) : (jj & 1)], dst + (uint32_t)(jj * 1024));
    };
    auto load_x = [&](uint32_t entry, int stage, int r0) {  // the kept X tiles of row blocks r0, r0 + 1: 2 loads per wave and tile
      const uint32_t fl = step_flags(entry);
      const char* ap = a_wave0 + step_block(entry) * red_stride;
      const uint32_t dst = smem_a + (uint32_t)(stage * STAGE + A_OFF + wg * 2 * 1024);
#pragma unroll
      for (int rr = 0; rr < 2; ++rr)
        if (row_quads(fl, r0 + rr)) {
#pragma unroll
          for (int j = 0; j < 2; ++j)
            load16_to_lds(ap + (r0 + rr) * a_rstride + j * x_step, ld_off[j], dst + (uint32_t)((r0 + rr) * TILE + j * 1024));
        }
    };
    u32x4 af[2][2][4];  // [row block of the wave][kk][16-row tile]
    u32x4 bf[NT16][2];
    if (nsteps > 0) {
      uint32_t e0 = uniform(step_e[0]), e1 = uniform(step_e[1]), e2 = uniform(step_e[2]);
      issue_loads(e0, 0);
      if (nsteps > 1) issue_loads(e1, 1, false, 0x3u);  // X[0-1](1): nobody's memory phase comes early enough for it
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (grp1) __syncthreads();  // phase 0 belongs to group 0
      for (int step = 0; step < nsteps; ++step) {
        const int stage = step & 1;
        const uint32_t e3 = step_e[step + 3];  // a VGPR until the end of the step
        // which of the wave's two row blocks keep this K block: wave-uniform, in a scalar register (2-3 % against
        // per-lane conditions)
        // (a mask of block size 32 keeps or drops each 32 x 32 quadrant of a tile: four bits per row block)
        const uint32_t q_rows[2] = {row_quads(step_flags(e0), 2 * rh_u), row_quads(step_flags(e0), 2 * rh_u + 1)};
        const uint32_t m = (q_rows[0] ? 1u : 0u) | (q_rows[1] ? 2u : 0u);
        // ---- memory phase.  The loads go first (they then have the rest of this phase and the whole compute phase to
        // land: 3 % faster than behind the reads), in one branch per group; the reads stay in code common to both
        // groups (under a branch per group the compiler keeps two sets of fragment registers and spills).
        const char* st = smem + stage * STAGE;
        if (!grp1) {
          if (step + 1 < nsteps) load_w(e1, stage ^ 1);
        } else {
          if (step + 1 < nsteps) load_x(e1, stage ^ 1, 2);
          if (step + 2 < nsteps) load_x(e2, stage, 0);
        }
        if (m) {
          read_b(st, 0, bf);
          read_b(st, 1, bf);
        }
        if (m & 1u) {
          read_a(st + A_OFF + (2 * rh) * TILE, 0, af[0][0]);
          read_a(st + A_OFF + (2 * rh) * TILE, 1, af[0][1]);
        }
        if (m & 2u) {
          read_a(st + A_OFF + (2 * rh + 1) * TILE, 0, af[1][0]);
          read_a(st + A_OFF + (2 * rh + 1) * TILE, 1, af[1][1]);
        }
        __syncthreads();
        // ---- compute phase
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          const uint32_t q = q_rows[rr];
          {
            // some quadrants of the X tile are dropped: quadrant (row half h, reduction half kk) feeds the MFMAs of the
            // 16-row tiles 2h, 2h + 1 at depth kk and nothing else, so dropping it is leaving those eight out
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
              for (int h = 0; h < 2; ++h)
                if ((q >> (2 * h + kk)) & 1u) {
#pragma unroll
                  for (int mt = 2 * h; mt < 2 * h + 2; ++mt)
#pragma unroll
                    for (int nt = 0; nt < NT16; ++nt) acc[rr][mt][nt] = T::mfma16(af[rr][kk][mt], bf[nt][kk], acc[rr][mt][nt]);
                }
          }
        }
        __builtin_amdgcn_s_setprio(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads have landed
        if (!(grp1 && step + 1 == nsteps)) __syncthreads();  // (group 1's last compute phase is nobody's memory phase)
        e0 = e1;
        e1 = e2;
        e2 = uniform(e3);
      }
    }
  } else if constexpr (IMPLICIT == 0 && !RAGGED && S::NST > 2) {
    // ---- the step loop of the 128 x 128 shape on aligned operands: three steps in flight ---------------------------
    // A step here is 12 fragment reads and 16 MFMAs per wave; with one step in flight every step waits out a whole
    // load latency (measured: 2200 clocks a step, whatever the drop rate).  So the tiles of steps s + 1 .. s + 3 are on
    // their way while step s computes: four stages, one barrier per step (it publishes step s and frees the stage of
    // step s - 1, into which the loads of step s + 3 go right behind it).  A wave waits for its own loads of step s
    // only: loads return in order, so it allows as many outstanding as it issued for the two steps after - a number
    // that depends on which X tiles those steps keep, hence the choice among waits below.
    static_assert(RW == 1 && S::NST == 4, "one row block per wave, four stages");
    constexpr int NST = S::NST;
    const int rh_u = (int)uniform((uint32_t)rh);
    const bool w_any = TRANS || wave_u * BL * 8 < nvalid;  // this wave's rows of the W tile are columns inside C
    // (reduction-strided W tile: lanes whose columns lie past N fetch column 0 of their row instead - readable, and
    // those columns are never stored)
    uint32_t b_ld[BL];
#pragma unroll
    for (int jj = 0; jj < BL; ++jj) {
      b_ld[jj] = b_lane[jj];
      if constexpr (TRANS) {
        constexpr int CPR = BN / 8;
        const int row = (wave * BL + jj) * (64 / CPR) + lane / CPR;
        if (!b_valid[jj]) b_ld[jj] = (uint32_t)(row * g.b.sc) * 2u;
      }
    }
    auto loads_of = [&](uint32_t e) {  // load instructions this wave issues for a step
      const uint32_t fl = step_flags(e);
      int n = w_any ? BL : 0;
#pragma unroll
      for (int r = 0; r < R; ++r) n += row_quads(fl, r) ? AL : 0;
      return n;
    };
    auto issue = [&](uint32_t e, int stage) {
      const int kb = step_block(e);
      const uint32_t fl = step_flags(e);
      const uint32_t st_a = smem_a + (uint32_t)(stage * STAGE);
      const char* bp = b_tile0 + kb * b_red_stride;
      const char* ap = a_tile0 + kb * red_stride;
      if (w_any) {
#pragma unroll
        for (int jj = 0; jj < BL; ++jj) load16_to_lds(bp, b_ld[jj], st_a + (uint32_t)((wave_u * BL + jj) * 1024));
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (row_quads(fl, r)) {
#pragma unroll
          for (int i = 0; i < AL; ++i)
            load16_to_lds(ap + r * a_rstride, a_lane[i], st_a + (uint32_t)(A_OFF + r * TILE + (wave_u * AL + i) * 1024));
        }
    };
    if (nsteps > 0) {
      uint32_t e0 = uniform(step_e[0]), e1 = uniform(step_e[1]), e2 = uniform(step_e[2]), e3 = uniform(step_e[3]);
      issue(e0, 0);
      int c1 = 0, c2 = 0;
      if (nsteps > 1) {
        issue(e1, 1);
        c1 = (int)uniform((uint32_t)loads_of(e1));
      }
      if (nsteps > 2) {
        issue(e2, 2);
        c2 = (int)uniform((uint32_t)loads_of(e2));
      }
      u32x4 bf[NT16][2];
      u32x4 af[2][4];
      for (int step = 0; step < nsteps; ++step) {
        const uint32_t e4 = step_e[step + 4];  // a VGPR until the end of the step
        wait_loads_all_but(c1 + c2);
        __syncthreads();
        int c3 = 0;
        if (step + 3 < nsteps) {
          issue(e3, (step + 3) % NST);
          c3 = (int)uniform((uint32_t)loads_of(e3));
        }
        if (row_quads(step_flags(e0), rh_u)) {
          const char* st = smem + (step % NST) * STAGE;
          const char* at = st + A_OFF + rh * TILE;
          read_b(st, 0, bf);
          read_a(at, 0, af[0]);
          read_b(st, 1, bf);
          read_a(at, 1, af[1]);
#pragma unroll
          for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
              for (int nt = 0; nt < NT16; ++nt) acc[0][mt][nt] = T::mfma16(af[kk][mt], bf[nt][kk], acc[0][mt][nt]);
        }
        e0 = e1;
        e1 = e2;
        e2 = e3;
        e3 = uniform(e4);
        c1 = c2;
        c2 = c3;
      }
      __syncthreads();  // the epilogue reuses the stages
    }
  } else if constexpr (IMPLICIT == 0) {
    // The products that read their operands from memory run the units of all steps as one chain: the barrier
    // that publishes the next stage stands in front of the MFMAs of a step's LAST unit, not behind them.  By
    // then the wave holds every fragment it needs from the current stage in registers (the barrier's own wait
    // for outstanding LDS reads sees to that), so the one barrier also frees the current stage, and the wave
    // issues, behind it, the loads of the step after next into that stage and the fragment reads of the next
    // step's first unit - both run under the last unit's MFMAs instead of in front of the next step's first.
    u32x4 bf[NT16][2];
    u32x4 af[2][4];
    auto wave_quads = [&](uint32_t e) { return (step_flags(e) >> (4 * RW * rh)) & ((1u << (4 * RW)) - 1u); };
    auto wave_mine = [&](uint32_t q) { return ((q & 0xfu) ? 1u : 0u) | ((RW == 2 && (q >> 4)) ? 2u : 0u); };
    // fragments of the first unit of the step with table word e, whose tiles are in `stage`
    auto first_reads = [&](uint32_t e, int stage) {
      const uint32_t m = wave_mine(wave_quads(e));
      if (m != 0u) {
        const char* st = smem + stage * STAGE;
        read_b(st, 0, bf);
        read_a(st + A_OFF + (RW * rh + (m == 2u ? 1 : 0)) * TILE, 0, af[0]);
      }
    };
    // the step boundary, see above; e_nn: table word of the step after next (only read when there is one)
    auto boundary = [&](int step, int stage, uint32_t e_nx, uint32_t e_nn, bool defer_loads = false) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads for the next step have landed
      __syncthreads();
      if (step + 2 < nsteps && !defer_loads) issue_loads(uniform(e_nn), stage);
      if (step + 1 < nsteps) first_reads(e_nx, stage ^ 1);
    };
    auto units = [&](auto mine_c, int step, int stage, uint32_t e_nx, uint32_t e_nn, bool red_tail,
                     uint32_t quads) {
      constexpr int MINE = decltype(mine_c)::value;
      constexpr int NR = (MINE == 3) ? 2 : 1;
      constexpr int R0 = (MINE == 2) ? 1 : 0;
      constexpr bool DEFER = MINE == 3;
      const char* st = smem + stage * STAGE;
      const char* at0 = st + A_OFF + (RW * rh + R0) * TILE;
#pragma unroll
      for (int u = 0; u < NR * 2; ++u) {
        const int rr = R0 + u / 2, kk = u % 2;
        if (u + 1 < NR * 2) {
          const int kk1 = (u + 1) % 2;
          if (u + 1 < 2) read_b(st, kk1, bf);
          read_a(at0 + ((u + 1) / 2) * TILE, kk1, af[(u + 1) & 1]);
        } else {
          boundary(step, stage, e_nx, e_nn, DEFER && late);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (RAGGED && g.quads) {  // a mask of block size 32: zero the dropped 32 x 32 quadrants of the tile
          const uint32_t q = row_quads(quads, rr);
#pragma unroll
          for (int mt = 0; mt < 4; ++mt)
            if (!((q >> (2 * (mt / 2) + kk)) & 1u)) af[u & 1][mt] = u32x4{0u, 0u, 0u, 0u};
        }
        if (RAGGED && red_tail) {  // ragged reduction block: nothing past the end may reach the MFMAs
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) mask_fragment(af[u & 1][mt], kk);
          if (u < 2) {  // the W fragments stay masked for the second row block
#pragma unroll
            for (int nt = 0; nt < NT16; ++nt) mask_fragment(bf[nt][kk], kk);
          }
        }
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT16; ++nt)
            acc[rr][mt][nt] = T::mfma16(af[u & 1][mt], bf[nt][kk], acc[rr][mt][nt]);
        __builtin_amdgcn_sched_barrier(0);
        // with both row blocks at work the second wave of each SIMD issues its loads behind the last MFMAs: the two
        // waves then run a little out of step, which the dense product gains 3-5 % from
        if (DEFER && u + 1 == NR * 2 && late && step + 2 < nsteps) issue_loads(uniform(e_nn), stage);
      }
    };

    if (nsteps > 0) issue_loads(e_cur, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (nsteps > 1) issue_loads(e_next, 1);
    if (nsteps > 0) first_reads(e_cur, 0);
    for (int step = 0; step < nsteps; ++step) {
      const int stage = step & 1;
      const uint32_t e_after = step_e[step + 2];  // a VGPR until the boundary makes it uniform
      const uint32_t quads = wave_quads(e_cur);
      const uint32_t mine = wave_mine(quads);
      const bool red_tail = RAGGED && step_block(e_cur) == kb_tail;
      if constexpr (RW == 2) {
        if (mine == 3u) units(std::integral_constant<int, 3>{}, step, stage, e_next, e_after, red_tail, quads);
        else if (mine == 1u) units(std::integral_constant<int, 1>{}, step, stage, e_next, e_after, red_tail, quads);
        else if (mine == 2u) units(std::integral_constant<int, 2>{}, step, stage, e_next, e_after, red_tail, quads);
        else boundary(step, stage, e_next, e_after);
      } else {
        if (mine) units(std::integral_constant<int, 1>{}, step, stage, e_next, e_after, red_tail, quads);
        else boundary(step, stage, e_next, e_after);
      }
      e_cur = e_next;
      e_next = uniform(e_after);
    }
  } else {
  if constexpr (STEP_COPIES) {
    if (nsteps > 0) {
      tpatch_load(e_cur);
      tpatch_store(patch);
    }
    if (nsteps > 1) {
      tpatch_load(e_next);
      tpatch_store(patch1);
    }
    __syncthreads();  // the copies, their halo groups and the column table
  }
  if (nsteps > 0) issue_loads(e_cur, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int step = 0; step < nsteps; ++step) {
    const int stage = step & 1;
    const uint32_t e_after = step_e[step + 2];
    const bool more = step + 1 < nsteps;
    if constexpr (STEP_COPIES) {
      if (step + 2 < nsteps) tpatch_load(uniform(step_e[step + 2]));
      tcopy = ((step + 1) & 1) ? patch1 : patch;  // holds the rows of step + 1
    }
    // keep bits of this wave's row blocks (four per block); a block takes part when any of them is set
    const uint32_t quads = (step_flags(e_cur) >> (4 * RW * rh)) & ((1u << (4 * RW)) - 1u);
    const uint32_t mine = ((quads & 0xfu) ? 1u : 0u) | ((RW == 2 && (quads >> 4)) ? 2u : 0u);
    const bool mid = late && more && mine != 0u;
    if (more && !mid) issue_loads(e_next, stage ^ 1);
    const char* st = smem + stage * STAGE;
    const bool red_tail = RAGGED && step_block(e_cur) == kb_tail;
    if constexpr (RW == 2) {
      if (mine == 3u) compute(std::integral_constant<int, 3>{}, st, mid, e_next, stage ^ 1, red_tail, quads);
      else if (mine == 1u) compute(std::integral_constant<int, 1>{}, st, mid, e_next, stage ^ 1, red_tail, quads);
      else if (mine == 2u) compute(std::integral_constant<int, 2>{}, st, mid, e_next, stage ^ 1, red_tail, quads);
    } else {
      if (mine) compute(std::integral_constant<int, 1>{}, st, mid, e_next, stage ^ 1, red_tail, quads);
    }
    if constexpr (STEP_COPIES) {
      if (step + 2 < nsteps) tpatch_store((step & 1) ? patch1 : patch);  // last read for this step's tiles, a step ago
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    e_cur = e_next;
    e_next = uniform(e_after);
  }
  }

  // ---- epilogue: scale, round once, store ---------------------------------------------------------
  // accumulator register v of lane l is element (m, n) = (4*(l/16) + v, l%16) of the 16x16 product
  // (rows of the X tile) x (rows of the W tile).
  if (ns * 32 * NT >= nvalid) return;  // this wave's column slice overhangs N: nothing of it is stored
  float* part = nsplit > 1 ? g.ws + (int64_t)split * g.M * g.N : nullptr;
  // Each wave stages one row block's 64 x WN tile at a time in its own piece of the (now idle) stages, laid out
  // along C's contiguous index, and writes it out in 16-byte pieces.  The last step's barrier has passed, so
  // nobody reads the stages or the step table any more.
  constexpr int WN = 32 * NT;
  constexpr int WC = WN > 64 ? 64 : WN;  // columns staged at a time
  constexpr int S_ROWS = CM ? WC : BS, S_COLS = CM ? BS : WC, S_PITCH = S_COLS + 4;
  static_assert(S::NW * S_ROWS * S_PITCH * 4 <= S::SMEM_BYTES, "the staging tiles must fit in the kernel's LDS");
  float* stg = reinterpret_cast<float*>(smem) + wave * (S_ROWS * S_PITCH);
#pragma unroll
  for (int rr = 0; rr < RW; ++rr) {
    const int rb = rb0 + RW * rh + rr;
    if (rb >= Mb) continue;
#pragma unroll
    for (int h = 0; h < WN / WC; ++h) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nc = 0; nc < WC / 16; ++nc) {
          const int nt = h * (WC / 16) + nc;
          if (CM) {  // staged as [n][m]: the lane's four registers are consecutive along m
            *reinterpret_cast<f32x4*>(stg + (nc * 16 + lane % 16) * S_PITCH + mt * 16 + 4 * (lane / 16)) = acc[rr][mt][nt];
          } else {  // staged as [m][n]: four rows, one column (16 lanes x 4 row groups hit 64 distinct banks)
#pragma unroll
            for (int v = 0; v < 4; ++v)
              stg[(mt * 16 + 4 * (lane / 16) + v) * S_PITCH + nc * 16 + lane % 16] = acc[rr][mt][nt][v];
          }
        }
      const int64_t m_first = (int64_t)rb * BS, n_first = n0 + ns * WN + h * WC;
      store_staged_tile<T, false, S_ROWS, S_COLS>(g, stg, lane, !CM, CM ? n_first : m_first, CM ? m_first : n_first,
                                                  part);
    }
  }
}

template <typename T, bool TRANS, bool CM, bool RAGGED, typename S, int IMPLICIT = 0>
__global__ __launch_bounds__(S::THREADS) void dsd_kernel(GemmArgs g, int tiles_m, int tiles_n,
                                                         int Mb, int Kb_all, ImplicitConv cg) {
  dsd_body<T, TRANS, CM, RAGGED, S, IMPLICIT>(g, tiles_m, tiles_n, Mb, Kb_all, cg, (int)blockIdx.x, (int)gridDim.y,
                                              (int)blockIdx.y);
}

// The forward product and the kept lists of its mask in ONE launch: workgroups [0, n_gemm) are the product's and take
// their keep bits from the mask source itself (a handful of generator calls or mask bytes per workgroup), the others
// build the lists the backward will read, and store a drawn mask.  Nothing in the launch waits for anything else.
template <typename T, bool RAGGED, typename S>
__global__ __launch_bounds__(S::THREADS) void forward_lists_kernel(GemmArgs g, int tiles_m, int tiles_n, int Mb,
                                                                   int Kb_all, int nsplit, int n_gemm, FlatJobs f) {
  const int bid = (int)blockIdx.x;
  if (bid < n_gemm) {
    MaskSrc ms = f.job0.src;
    ms.resolve();
    const int tiles = tiles_m * tiles_n;
    dsd_body<T, false, false, RAGGED, S, 0>(g, tiles_m, tiles_n, Mb, Kb_all, ImplicitConv{}, bid % tiles, nsplit,
                                            bid / tiles, &ms);
  } else {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    flat_lists_block<S::THREADS>(f, bid - n_gemm, reinterpret_cast<int32_t*>(smem));
  }
  report_in(const_cast<uint64_t*>(f.job0.src.state), gridDim.x);
}

// ---- SDD with column groups ---------------------------------------------------------------------------
// A = dY [M, red] reduction-contiguous; B = W^T [cols, red] given with the reduction index strided
// (b.sr == 1); C row-major.  Mb x Cb is the block grid of the output (and of the mask); without a list
// every tile is kept (the dense product in this operand layout).
// With half of the tiles dropped a fixed 4x4 patch of tiles would still need nearly all of its 4 + 4 operand
// tiles per reduction step for about 8 kept tiles.  Here a workgroup owns 4 row blocks x a GROUP of consecutive
// column blocks, chosen greedily along the row so that it has at most GW column blocks with anything
// kept and at most 16 kept tiles: 4 + 6 operand tiles per step for about 12 kept tiles at p = 0.5, the
// same 4 + 4 for 16 as the patch kernel at p = 0.  Column blocks with nothing kept in these 4 rows
// cost nothing (zeros are stored for them).  Group boundaries depend on the mask, so a workgroup is launched for
// (window of 4 * GW column blocks, index of the group inside it), scans the quad's keep flags of that window and
// takes the group with its index (the grid has the worst case number of groups per window; surplus workgroups
// exit).  Groups never straddle a window, so the workgroups of different row quads stay on the same W tiles.
// A wave owns up to two WHOLE kept tiles (tile t of the group goes to wave t%8, so the two waves of a
// SIMD always carry equal work +-1): 2x2 MFMAs per 16-wide step from 2 + 2 fragments, accumulators
// statically indexed by the wave's slot, operand tiles addressed dynamically.
// SddBig   4 row blocks x groups of at most 6 active column blocks and 16 kept tiles, two tile slots per wave:
//           two 80 KB stages, all of the LDS
// SddMid   2 row blocks x at most 4 active column blocks and 8 kept tiles, one slot per wave: twice as many
//           workgroups with half the loads per step each, for outputs that give the big shape too few
template <int R_, int GW_, int SLOTS_, int NST_ = 2>
struct SddShape {
  static constexpr int NST = NST_;       // stages of LDS (steps whose tiles are resident or on their way)
  static constexpr int R = R_;           // row blocks per workgroup
  static constexpr int GW = GW_;         // column blocks with kept tiles per group
  static constexpr int SLOTS = SLOTS_;   // whole tiles a wave can own
  static constexpr int MAXT = 8 * SLOTS; // kept tiles per group
  static constexpr int BOFF = R * TILE;  // dY tiles first, then W tiles
  static constexpr int STAGE = (R + GW) * TILE;
  // two stages; at least the eight 64 x 68 fp32 staging tiles of the epilogue
  static constexpr int SMEM = NST * STAGE > 8 * BS * (BS + 4) * 4 ? NST * STAGE : 8 * BS * (BS + 4) * 4;
  static constexpr int MINCOLS = GW < MAXT / R ? GW : MAXT / R;  // column blocks a group is sure to cover
  // Groups never straddle a multiple of WINDOW column blocks, and a workgroup is launched for (window, group in
  // the window): whatever the masks of two row quads, their workgroups of one window need the same W tiles
  // (measured 1-6 % faster than groups that run freely along the row).
  static constexpr int WINDOW = 4 * GW;
  static constexpr int GPW = WINDOW / MINCOLS;  // groups a whole window can have at most
};
using SddBig = SddShape<4, 6, 2>;
using SddMid = SddShape<2, 4, 1>;
// On aligned operands, outputs too small for the big shape run with more steps in flight (a step of these shapes is
// far shorter than a load's way through L2 and memory): the shape above with three stages, and for outputs that give
// even that one too few workgroups, 2 row blocks x 2 column blocks (4 tiles, on waves 0-3; all 8 waves load) with four
using SddMidDeep = SddShape<2, 4, 1, 3>;
using SddSmall = SddShape<2, 2, 1, 4>;
constexpr int G_MAX_CB = 8192;             // per-column flags share the first stage (of either shape) before the loads start

// EDGE = the output width or the reduction length is not a multiple of 64 (both multiples of 8): the
// overhanging 16-byte chunks / rows of the last column block / reduction block are fetched from inside the
// matrix instead, as in the DSD kernel, the fragments of the last reduction block are zeroed past the end,
// and nothing is stored past the last column.  (A ragged M costs nothing worth a separate instance.)
template <typename T, bool EDGE, typename G>
__device__ __forceinline__ void sdd_body(const GemmArgs& g, int tiles_m, int gmax, int Mb, int Cb, const int bid) {
  constexpr int R = G::R, GW = G::GW, SLOTS = G::SLOTS, G_BOFF = G::BOFF, G_STAGE = G::STAGE;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // bit r: tile (row block rb0 + r, column block c) kept; bits 8 + 4r .. 11 + 4r: which of its four 32 x 32
  // quadrants (all of them unless the mask has block size 32)
  const uint32_t smem_a = lds_address(smem);
  uint32_t* flags = reinterpret_cast<uint32_t*>(smem);
  int* rec = reinterpret_cast<int*>(smem + 4 * ((Cb + 3) & ~3));  // c_lo, c_hi, ncols, kept bits, cols[GW]

  int tm, gi;
  tile_of_block<SDD_GROUP_M>(bid, tiles_m, gmax, tm, gi);
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int rb0 = tm * R;

  // ---- per-column keep flags of this row quad -------------------------------------------------------
  {
    const int rows = (rb0 + R <= Mb) ? R : Mb - rb0;
    const uint32_t all = ((1u << rows) - 1u) | (((1u << (4 * rows)) - 1u) << 8);
    const uint32_t init = g.row_ptr ? 0u : all;
    for (int i = tid; i < Cb; i += THREADS) flags[i] = init;
    if (tid < 32) rec[tid] = 0;
  }
  __syncthreads();
  if (g.row_ptr) {
    for (int r = 0; r < R; ++r) {
      if (rb0 + r >= Mb) break;
      const int beg = g.row_ptr[rb0 + r], end = g.row_ptr[rb0 + r + 1];
      for (int i = beg + tid; i < end; i += THREADS) {
        const int32_t e = g.col_idx[i];
        atomicOr(&flags[entry_block(e)], (1u << r) | (entry_quads(e) << (8 + 4 * r)));
      }
    }
    __syncthreads();
  }

  // ---- the group this workgroup was launched for ---------------------------------------------------------
  if (wave == 0) {
    // whole windows, the last one taking the remainder as well (so that the grid is as large as without windows)
    const int nwin = Cb / G::WINDOW > 1 ? Cb / G::WINDOW : 1;
    const int win = gi / G::GPW < nwin - 1 ? gi / G::GPW : nwin - 1, want = gi - win * G::GPW;
    const int w_lo = win * G::WINDOW, w_hi = win == nwin - 1 ? Cb : w_lo + G::WINDOW;
    int grp = 0, start = w_lo, width = 0, cnt = 0, lo = -1, hi = -1;
    static_assert(2 * G::WINDOW <= 64, "a window's flags are read by one wave-wide load");
    if (w_hi - w_lo <= 64) {
      const uint32_t fv = (w_lo + lane < w_hi) ? flags[w_lo + lane] : 0u;
      for (int i = 0; i < w_hi - w_lo; ++i) {
        const uint32_t f = (uint32_t)__builtin_amdgcn_readlane((int)fv, i) & 0xfu;
        if (f == 0) continue;
        const int a = __builtin_popcount(f);
        if (width == GW || cnt + a > G::MAXT) {  // the group ends in front of this column block
          if (grp == want) {
            lo = start;
            hi = w_lo + i;
            break;
          }
          ++grp;
          start = w_lo + i;
          width = 0;
          cnt = 0;
        }
        ++width;
        cnt += a;
      }
      if (hi < 0 && grp == want) {  // the window's last group runs to its end
        lo = start;
        hi = w_hi;
      }
    }
    int n = 0;
    uint32_t kept = 0;  // bit 4*j + r
    for (int c = lo; c < hi; ++c) {
      const uint32_t fq = (uint32_t)__builtin_amdgcn_readfirstlane((int)flags[c]);
      const uint32_t f = fq & 0xfu;
      if (f) {
        if (lane == 0) {
          rec[4 + n] = c;
          rec[16 + n] = (int)(fq >> 8);  // quadrant keep bits of the column block's tiles, four per row block
        }
        kept |= f << (4 * n);
        ++n;
      }
    }
    if (lane == 0) {
      rec[0] = lo;
      rec[1] = hi;
      rec[2] = n;
      rec[3] = (int)kept;
    }
  }
  __syncthreads();
  const int c_lo = __builtin_amdgcn_readfirstlane(rec[0]);
  const int c_hi = __builtin_amdgcn_readfirstlane(rec[1]);
  if (c_lo < 0) return;  // fewer groups in this row quad than the grid provides for
  const int ncols = __builtin_amdgcn_readfirstlane(rec[2]);
  const uint32_t kept = (uint32_t)__builtin_amdgcn_readfirstlane(rec[3]);
  int cols[GW];
#pragma unroll
  for (int j = 0; j < GW; ++j) cols[j] = __builtin_amdgcn_readfirstlane(rec[4 + j]);
  const int ntiles = __builtin_popcount(kept);

  // this wave's tiles: tile t of the group (set bits of `kept` in order) belongs to wave t % 8
  int my_r[SLOTS], my_j[SLOTS], my_c[SLOTS];
  bool act[SLOTS];
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int t = wave + 8 * k;
    act[k] = t < ntiles;
    uint32_t m = kept;
    for (int i = 0; i < t; ++i) m &= m - 1u;
    const int b = (act[k] && m) ? __builtin_ctz(m) : 0;
    my_j[k] = b / 4;
    my_r[k] = b % 4;
    my_c[k] = __builtin_amdgcn_readfirstlane(rec[4 + my_j[k]]);
  }
  uint32_t my_q[SLOTS];  // which quadrants of the wave's tiles are kept
#pragma unroll
  for (int k = 0; k < SLOTS; ++k)
    my_q[k] = ((uint32_t)__builtin_amdgcn_readfirstlane(rec[16 + my_j[k]]) >> (4 * my_r[k])) & 0xfu;
  uint32_t rowmask = 0;
#pragma unroll
  for (int j = 0; j < GW; ++j) rowmask |= (kept >> (4 * j)) & 0xfu;

  // ---- zeros for the dropped tiles of the group's column range ----------------------------------------
  if (!g.kept_only) {
    const int row = tid / 8, ch = tid % 8;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int c = c_lo; c < c_hi; ++c) {
      const uint32_t f = (uint32_t)__builtin_amdgcn_readfirstlane((int)flags[c]);
      for (int r = 0; r < R; ++r) {
        if (rb0 + r >= Mb) break;
        if (!((f >> r) & 1u) && (int64_t)(rb0 + r) * BS + row < g.M && (!EDGE || (int64_t)c * BS + ch * 8 < g.N))
          *reinterpret_cast<u32x4*>(g.c + ((int64_t)(rb0 + r) * BS + row) * g.c_sr + (int64_t)c * BS + ch * 8) = z;
      }
    }
  }
  if (kept == 0) return;
  __syncthreads();  // flags and rec are dead: the stages may be written

  // ---- per-lane constants -----------------------------------------------------------------------------
  // fragments of v_mfma_f32_16x16x32 per 32-wide reduction step kk (see dsd_kernel): dY tiles are
  // reduction-contiguous (b128 reads), W tiles reduction-strided (transposing reads)
  int a_off[2], b_off[2];
  {
    const int fr_sw = (lane >> 1) & 7;
    const int b4 = lane / 16, e = (lane % 16) / 4, j = lane % 4;
    const int row = 8 * b4 + e;
    const int b_ch = (j / 2) ^ swz_x(row);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      a_off[kk] = (lane % 16) * 128 + ((4 * kk + lane / 16) ^ fr_sw) * 16;  // + 16*128 per 16-row tile
      b_off[kk] = (32 * kk + row) * 128 + b_ch * 16 + (j % 2) * 8;           // ^ 32 per 16-column tile
    }
  }
  const int nsteps = (int)((g.K + BS - 1) / BS);
  // loads: wave-uniform tile bases plus this lane's 16 bytes of the wave's 8 tile rows
  const char* a_base = reinterpret_cast<const char*>(g.a.ptr + (int64_t)rb0 * BS * g.a.sr);
  const char* b_base = reinterpret_cast<const char*>(g.b.ptr);
  // M need not be a multiple of 64: rows of the last row block past M are fetched from its last valid row
  // (rows are independent, theirs are never stored)
  const int m_valid = (int)(g.M % BS), n_valid = (int)(g.N % BS), k_valid = (int)(g.K % BS);
  const int r_tail = m_valid ? Mb - 1 - rb0 : -1;
  const int c_tail = (EDGE && n_valid) ? Cb - 1 : -1;        // column block that is ragged
  const int s_tail = (EDGE && k_valid) ? nsteps - 1 : -1;    // reduction block that is ragged
  uint32_t a_lane, a_lane_m, b_lane;
  // EDGE: what to add (mod 2^32) to a lane's offset for a ragged reduction block / column block; the row and
  // the chunk term of an offset are redirected independently, so the corrections add up
  uint32_t a_delta_k, b_delta_c, b_delta_k;
  {
    const int row = wave * 8 + lane / 8;
    const int pch = lane % 8;
    auto a_at = [&](bool clamp_m, bool clamp_k) {
      const int rc = (clamp_m && row >= m_valid) ? m_valid - 1 : row;
      int c = pch ^ ((row >> 1) & 7);
      if (clamp_k && c * 8 >= k_valid) c = 0;
      return (uint32_t)(rc * g.a.sr + c * 8) * 2u;
    };
    auto b_at = [&](bool clamp_c, bool clamp_k) {  // rows of a W tile are reduction indices
      const int rc = (clamp_k && row >= k_valid) ? k_valid - 1 : row;
      int c = pch ^ swz_x(row);
      if (clamp_c && c * 8 >= n_valid) c = 0;
      return (uint32_t)(rc * g.b.sc + c * 8) * 2u;
    };
    a_lane = a_at(false, false);
    a_lane_m = a_at(r_tail >= 0, false);
    a_delta_k = a_at(false, s_tail >= 0) - a_lane;
    b_lane = b_at(false, false);
    b_delta_c = b_at(c_tail >= 0, false) - b_lane;
    b_delta_k = b_at(false, s_tail >= 0) - b_lane;
  }
  const int64_t a_tile_stride = (int64_t)BS * g.a.sr * 2;
  const int64_t b_step_stride = (int64_t)BS * g.b.sc * 2;
  auto issue_loads = [&](int step, int stage) {
    const uint32_t st = smem_a + (uint32_t)(stage * G_STAGE + wave * 1024);
    const char* ap = a_base + step * (BS * 2);
    const char* bp = b_base + step * b_step_stride;
    const bool red_tail = EDGE && step == s_tail;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (rowmask & (1u << r)) {
        uint32_t off = r == r_tail ? a_lane_m : a_lane;
        if (EDGE) off += red_tail ? a_delta_k : 0u;
        load16_to_lds(ap + r * a_tile_stride, off, st + (uint32_t)(r * TILE));
      }
#pragma unroll
    for (int j = 0; j < GW; ++j)
      if (j < ncols) {
        uint32_t off = b_lane;
        if (EDGE) off += (cols[j] == c_tail ? b_delta_c : 0u) + (red_tail ? b_delta_k : 0u);
        load16_to_lds(bp + (int64_t)cols[j] * (BS * 2), off, st + (uint32_t)(G_BOFF + j * TILE));
      }
  };
  // zeroes the elements of a fragment whose reduction index (32*kk + 8*(lane/16) + 0..7 inside the
  // block) is not below k_valid
  auto mask_fragment = [&](u32x4& f, int kk) {
    const int n = k_valid - (32 * kk + 8 * (lane / 16));
    f.x &= n >= 2 ? ~0u : (n == 1 ? 0xffffu : 0u);
    f.y &= n >= 4 ? ~0u : (n == 3 ? 0xffffu : 0u);
    f.z &= n >= 6 ? ~0u : (n == 5 ? 0xffffu : 0u);
    f.w &= n >= 8 ? ~0u : (n == 7 ? 0xffffu : 0u);
  };
  // the two waves of a SIMD (w and w + 4) issue their loads apart: the first right behind the barrier, the second
  // behind the step's last MFMAs
  const bool late = wave >= 4;

  f32x4 acc[SLOTS][4][4];  // [slot][16-row tile][16-column tile]
#pragma unroll
  for (int k = 0; k < SLOTS; ++k)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[k][a][b][v] = 0.f;

  // Units u = 2*slot + kk run as one chain over all steps: the fragments of unit u+1 are read before the MFMAs
  // of unit u, and the barrier that publishes the next stage (and frees the current one: by then the wave holds
  // all its fragments of it) stands in front of the MFMAs of the step's last unit.  Behind it the wave issues the
  // loads of the step after next and reads the next step's first fragments, under those MFMAs.
  u32x4 af[2][4], bf[2][4];
  auto read_unit = [&](int stage, int u) {
    const int k = u / 2, kk = u % 2;
    const char* st = smem + stage * G_STAGE;
    const char* at = st + my_r[k] * TILE;
    const char* bt = st + G_BOFF + my_j[k] * TILE;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      af[u & 1][h] = *reinterpret_cast<const u32x4*>(at + a_off[kk] + h * 16 * 128);
      const char* p = bt + (b_off[kk] ^ (h * 32));
      const u32x2 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * 128);
      bf[u & 1][h] = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
  };
  auto boundary = [&](int step, int stage, bool defer_loads) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads for the next step have landed
    __syncthreads();
    if (step + 2 < nsteps && !defer_loads) issue_loads(step + 2, stage);
    if (step + 1 < nsteps && act[0]) read_unit(stage ^ 1, 0);
  };
  auto mfma_unit = [&](auto k_c, int u, bool red_tail) {
    constexpr int k = decltype(k_c)::value;
    if (EDGE && red_tail) {  // nothing past the end of the reduction may reach the MFMAs
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        mask_fragment(af[u & 1][h], u % 2);
        mask_fragment(bf[u & 1][h], u % 2);
      }
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) acc[k][mt][nt] = T::mfma16(af[u & 1][mt], bf[u & 1][nt], acc[k][mt][nt]);
  };

  if constexpr (!EDGE && G::NST > 2) {
    // ---- more than one step in flight: the tiles of steps s + 1 .. s + NST - 2 are on their way while step s
    // computes; one barrier per step publishes step s and frees the stage of step s - 1, which the loads of step
    // s + NST - 1 go into right behind it.  Every step costs this wave the same number of loads, so "my loads of
    // step s have landed" is "at most (steps still in flight) x (loads per step) outstanding".
    static_assert(SLOTS == 1, "one tile per wave");
    constexpr int NST = G::NST;
    const int n_ld = __builtin_popcount(rowmask) + ncols;
    for (int s0 = 0; s0 < NST - 1 && s0 < nsteps; ++s0) issue_loads(s0, s0);
    for (int step = 0; step < nsteps; ++step) {
      const int left = nsteps - 1 - step;
      wait_loads_all_but((left < NST - 2 ? left : NST - 2) * n_ld);
      __syncthreads();
      if (step + NST - 1 < nsteps) issue_loads(step + NST - 1, (step + NST - 1) % NST);
      if (act[0]) {
        const int stage = step % NST;
        read_unit(stage, 0);
        read_unit(stage, 1);
        mfma_unit(std::integral_constant<int, 0>{}, 0, false);
        mfma_unit(std::integral_constant<int, 0>{}, 1, false);
      }
    }
    __syncthreads();  // the epilogue reuses the stages
  } else {
  issue_loads(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (nsteps > 1) issue_loads(1, 1);
  if (act[0]) read_unit(0, 0);

  for (int step = 0; step < nsteps; ++step) {
    const int stage = step & 1;
    const bool red_tail = EDGE && step == s_tail;
    const bool two = SLOTS == 2 && act[SLOTS - 1];  // the wave's second tile slot is in use: four units, else two
    const bool defer = late;  // measured: the later the second wave of a SIMD issues its loads, the better
    if (act[0]) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (u == 0) read_unit(stage, 1);
        else if (two) read_unit(stage, 2);
        else boundary(step, stage, defer);
        __builtin_amdgcn_sched_barrier(0);
        mfma_unit(std::integral_constant<int, 0>{}, u, red_tail);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (SLOTS == 2) {
        if (two) {
#pragma unroll
          for (int u = 2; u < 4; ++u) {
            if (u == 2) read_unit(stage, 3);
            else boundary(step, stage, defer);
            __builtin_amdgcn_sched_barrier(0);
            mfma_unit(std::integral_constant<int, 1>{}, u, red_tail);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      if (defer && step + 2 < nsteps) issue_loads(step + 2, stage);
    } else {
      boundary(step, stage, false);
    }
  }
  }

  // ---- epilogue ---------------------------------------------------------------------------------------
  // Each wave stages a tile in its own piece of the (now idle) stages and writes it out in 16-byte pieces, whole
  // 128-byte lines at a time; the last step's barrier has passed, so nobody reads the stages any more.
  constexpr int S_PITCH = BS + 4;
  static_assert(8 * BS * S_PITCH * 4 <= G::SMEM, "the staging tiles must fit in the kernel's LDS");
  float* stg = reinterpret_cast<float*>(smem) + wave * (BS * S_PITCH);
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    if (!act[k]) continue;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {  // register v of lane l is element (4*(l/16) + v, l%16) of the 16 x 16 tile
          // a mask of block size 32 drops 32 x 32 quadrants of a kept tile: those are stored as zeros
          const bool keep = !EDGE || ((my_q[k] >> (2 * (mt / 2) + nt / 2)) & 1u);
          stg[(mt * 16 + 4 * (lane / 16) + v) * S_PITCH + nt * 16 + lane % 16] = keep ? acc[k][mt][nt][v] : 0.f;
        }
    store_staged_tile<T, true, BS, BS>(g, stg, lane, true, (int64_t)(rb0 + my_r[k]) * BS, (int64_t)my_c[k] * BS,
                                       nullptr);
  }
}

// ---- SDD on aligned operands, 4 row blocks per workgroup: the two waves of a SIMD in opposite phases -----------------
// The step loop of the DSD kernel (memory phase: the wave's loads, then every fragment of the step; compute phase:
// MFMAs only; the second group of four waves one phase behind the first) carried over to the output-sparse product.
// For a step's fragments to fit in registers the two tiles of a wave must share an operand, so a wave owns ONE column
// block of the group and up to two of its kept tiles: the W fragments of the column (32 registers) serve both, the dY
// fragments of its one or two row blocks take 32 each.  A column block with 3 or 4 kept tiles takes two waves, and all
// waves of a column block are in one group of four (so that a W tile is read by one group only: the dY tiles are to
// this kernel what the W tile is to the DSD kernel, and the W tiles what the X tiles are).  Groups of column blocks are
// formed greedily along the row: a column block goes to the group of waves with more waves to spare, and the
// workgroup's group ends in front of the column block that fits neither, or after 6 (the LDS holds 4 + 6 tiles per
// stage).  Everything kept: 4 column blocks, 16 tiles, as before; at p = 0.5 about 6 column blocks and 12-13 tiles.
// Group 0 loads the dY tiles of the next step; group 1 its own W tiles of the next step and group 0's of the step
// after next (the DSD kernel's reasoning, see there).  Measured and slower at every drop rate but 0.5 (where it gains
// 1 %): letting a column block's two waves sit in different groups (13 instead of 10.5 tiles per group at p = 0.5)
// with the W loads shared out evenly between the groups - what a step costs is the instructions of its memory
// phase, and the fuller groups need more of them per wave.
template <typename T>
__device__ __forceinline__ void sdd_pp_body(const GemmArgs& g, int tiles_m, int gmax, int Mb, int Cb, const int bid) {
  using G = SddBig;
  constexpr int R = G::R, GW = G::GW, G_BOFF = G::BOFF, G_STAGE = G::STAGE;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t smem_a = lds_address(smem);
  // bit r: tile (row block rb0 + r, column block c) kept; bits 8 + 4r .. 11 + 4r: which of its four 32 x 32 quadrants
  // (all of them unless the mask has block size 32)
  uint32_t* flags = reinterpret_cast<uint32_t*>(smem);
  int* rec = reinterpret_cast<int*>(smem + 4 * ((Cb + 3) & ~3));        // c_lo, c_hi, ncols, group-1 slots, cols[6], waves[8]

  int tm, gi;
  tile_of_block<SDD_GROUP_M>(bid, tiles_m, gmax, tm, gi);
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int rb0 = tm * R;

  // ---- per-column keep flags of this row quad -------------------------------------------------------
  {
    const int rows = (rb0 + R <= Mb) ? R : Mb - rb0;
    const uint32_t init = g.row_ptr ? 0u : (((1u << rows) - 1u) | (((1u << (4 * rows)) - 1u) << 8));
    for (int i = tid; i < Cb; i += THREADS) flags[i] = init;
    if (tid < 32) rec[tid] = 0;
  }
  __syncthreads();
  if (g.row_ptr) {
    for (int r = 0; r < R; ++r) {
      if (rb0 + r >= Mb) break;
      const int beg = g.row_ptr[rb0 + r], end = g.row_ptr[rb0 + r + 1];
      for (int i = beg + tid; i < end; i += THREADS) {
        const int32_t e = g.col_idx[i];
        atomicOr(&flags[entry_block(e)], (1u << r) | (entry_quads(e) << (8 + 4 * r)));
      }
    }
    __syncthreads();
  }

  // ---- the group this workgroup was launched for: (window, index inside it), as in the other SDD kernel -----------
  if (wave == 0) {
    const int nwin = Cb / G::WINDOW > 1 ? Cb / G::WINDOW : 1;
    const int win = gi / G::GPW < nwin - 1 ? gi / G::GPW : nwin - 1, want = gi - win * G::GPW;
    const int w_lo = win * G::WINDOW, w_hi = win == nwin - 1 ? Cb : w_lo + G::WINDOW;
    int lo = -1, hi = -1;
    if (w_hi - w_lo <= 64) {
      const uint32_t fv = (w_lo + lane < w_hi) ? flags[w_lo + lane] : 0u;
      int grp = 0, start = w_lo, used0 = 0, used1 = 0, slots = 0;
      for (int i = 0; i < w_hi - w_lo; ++i) {
        const uint32_t f = (uint32_t)__builtin_amdgcn_readlane((int)fv, i) & 0xfu;
        if (f == 0) continue;
        const int w = (__builtin_popcount(f) + 1) / 2;  // waves the column block takes
        int gsel = used0 <= used1 ? 0 : 1;
        if (4 - (gsel ? used1 : used0) < w) gsel ^= 1;
        if (slots == GW || 4 - (gsel ? used1 : used0) < w) {  // the group ends in front of this column block
          if (grp == want) {
            lo = start;
            hi = w_lo + i;
            break;
          }
          ++grp;
          start = w_lo + i;
          used0 = used1 = slots = 0;
          gsel = 0;
        }
        if (gsel) used1 += w; else used0 += w;
        ++slots;
      }
      if (hi < 0 && grp == want) {  // the window's last group runs to its end
        lo = start;
        hi = w_hi;
      }
    }
    // slots, groups and waves of the group's column blocks (the same choices again)
    int n = 0, used0 = 0, used1 = 0;
    uint32_t g1_slots = 0, rowmask = 0;
    for (int c = lo; c < hi; ++c) {
      const uint32_t fq = (uint32_t)__builtin_amdgcn_readfirstlane((int)flags[c]), f = fq & 0xfu;
      if (!f) continue;
      const int cnt = __builtin_popcount(f), w = (cnt + 1) / 2;
      auto quads_of = [&](int r) { return (fq >> (8 + 4 * r)) & 0xfu; };
      int gsel = used0 <= used1 ? 0 : 1;
      if (4 - (gsel ? used1 : used0) < w) gsel ^= 1;
      const int wv = 4 * gsel + (gsel ? used1 : used0);
      uint32_t m = f;
      const int r_a = __builtin_ctz(m); m &= m - 1u;
      const int r_b = m ? __builtin_ctz(m) : 0; if (m) m &= m - 1u;
      const int r_c = m ? __builtin_ctz(m) : 0; if (m) m &= m - 1u;
      const int r_d = m ? __builtin_ctz(m) : 0;
      if (lane == 0) {
        rec[4 + n] = c;
        rec[10 + wv] = n | (r_a << 4) | (r_b << 8) | ((cnt >= 2 ? 2 : 1) << 12) | (int)(quads_of(r_a) << 16) | (int)(quads_of(r_b) << 20);
        if (w == 2) rec[10 + wv + 1] = n | (r_c << 4) | (r_d << 8) | ((cnt - 2) << 12) | (int)(quads_of(r_c) << 16) | (int)(quads_of(r_d) << 20);
      }
      if (gsel) { used1 += w; g1_slots |= 1u << n; } else used0 += w;
      rowmask |= f;
      ++n;
    }
    if (lane == 0) {
      rec[0] = lo;
      rec[1] = hi;
      rec[2] = n;
      rec[3] = (int)(g1_slots | (rowmask << 8));
    }
  }
  __syncthreads();
  const int c_lo = __builtin_amdgcn_readfirstlane(rec[0]);
  const int c_hi = __builtin_amdgcn_readfirstlane(rec[1]);
  if (c_lo < 0) return;  // fewer groups in this row quad than the grid provides for
  const int ncols = __builtin_amdgcn_readfirstlane(rec[2]);
  const uint32_t g1_slots = (uint32_t)__builtin_amdgcn_readfirstlane(rec[3]) & 0xffu;
  const uint32_t rowmask = ((uint32_t)__builtin_amdgcn_readfirstlane(rec[3]) >> 8) & 0xfu;
  int cols[GW];
#pragma unroll
  for (int j = 0; j < GW; ++j) cols[j] = __builtin_amdgcn_readfirstlane(rec[4 + j]);
  const uint32_t mine = (uint32_t)__builtin_amdgcn_readfirstlane(rec[10 + wave]);
  const int my_j = (int)(mine & 0xfu), n_mine = (int)((mine >> 12) & 3u);
  const int my_r[2] = {(int)((mine >> 4) & 0xfu), (int)((mine >> 8) & 0xfu)};
  const uint32_t my_q[2] = {(mine >> 16) & 0xfu, (mine >> 20) & 0xfu};  // kept quadrants of the wave's tiles
  const int my_c = __builtin_amdgcn_readfirstlane(rec[4 + my_j]);

  // ---- zeros for the dropped tiles of the group's column range ----------------------------------------
  if (!g.kept_only) {
    const int row = tid / 8, ch = tid % 8;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int c = c_lo; c < c_hi; ++c) {
      const uint32_t f = (uint32_t)__builtin_amdgcn_readfirstlane((int)flags[c]);
      for (int r = 0; r < R; ++r) {
        if (rb0 + r >= Mb) break;
        if (!((f >> r) & 1u) && (int64_t)(rb0 + r) * BS + row < g.M)
          *reinterpret_cast<u32x4*>(g.c + ((int64_t)(rb0 + r) * BS + row) * g.c_sr + (int64_t)c * BS + ch * 8) = z;
      }
    }
  }
  if (ncols == 0) return;
  __syncthreads();  // flags and rec are dead: the stages may be written

  // ---- per-lane constants -----------------------------------------------------------------------------
  int a_off[2], b_off[2];
  {
    const int fr_sw = (lane >> 1) & 7;
    const int b4 = lane / 16, e = (lane % 16) / 4, j = lane % 4;
    const int row = 8 * b4 + e;
    const int b_ch = (j / 2) ^ swz_x(row);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      a_off[kk] = (lane % 16) * 128 + ((4 * kk + lane / 16) ^ fr_sw) * 16;  // + 16*128 per 16-row tile
      b_off[kk] = (32 * kk + row) * 128 + b_ch * 16 + (j % 2) * 8;           // ^ 32 per 16-column tile
    }
  }
  const int nsteps = (int)(g.K / BS);
  const bool grp1 = wave >= 4;
  const int wg = wave & 3;
  const int m_valid = (int)(g.M % BS);
  const int r_tail = m_valid ? Mb - 1 - rb0 : -1;  // rows of the last row block past M are fetched from its last valid row
  // per-lane offsets of the wave's loads: the two 8-row pieces (wg*2, wg*2 + 1) of a tile; group 0 loads dY tiles
  // (rows of 128 B along the reduction), group 1 W tiles (reduction rows of 128 B along the columns)
  uint32_t ld_off[2], ld_off_m[2];
#pragma unroll
  for (int v = 0; v < 2; ++v) {
    const int lr = lane / 8, pch = lane % 8, row = (wg * 2 + v) * 8 + lr;
    if (!grp1) {
      const int c = pch ^ ((row >> 1) & 7);
      const int rc = (r_tail >= 0 && row >= m_valid) ? m_valid - 1 : row;
      ld_off[v] = (uint32_t)(row * g.a.sr + c * 8) * 2u;
      ld_off_m[v] = (uint32_t)(rc * g.a.sr + c * 8) * 2u;
    } else {
      ld_off[v] = ld_off_m[v] = (uint32_t)(row * g.b.sc + (pch ^ swz_x(row)) * 8) * 2u;
    }
  }
  const char* a_base = reinterpret_cast<const char*>(g.a.ptr + (int64_t)rb0 * BS * g.a.sr);
  const char* b_base = reinterpret_cast<const char*>(g.b.ptr);
  const int64_t a_tile_stride = (int64_t)BS * g.a.sr * 2;
  const int64_t b_step_stride = (int64_t)BS * g.b.sc * 2;
  const uint32_t my_dst = smem_a + (uint32_t)(wg * 2 * 1024);
  auto load_dy = [&](int step, int stage) {  // group 0: its two loads of every dY tile in use
    const char* ap = a_base + step * (BS * 2);
    const uint32_t dst = my_dst + (uint32_t)(stage * G_STAGE);
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (rowmask & (1u << r)) {
        load16_to_lds(ap + r * a_tile_stride, r == r_tail ? ld_off_m[0] : ld_off[0], dst + (uint32_t)(r * TILE));
        load16_to_lds(ap + r * a_tile_stride, r == r_tail ? ld_off_m[1] : ld_off[1], dst + (uint32_t)(r * TILE) + 1024u);
      }
  };
  auto load_w = [&](int step, int stage, uint32_t slots) {  // group 1: its two loads of the W tiles in `slots`
    const char* bp = b_base + step * b_step_stride;
    const uint32_t dst = my_dst + (uint32_t)(stage * G_STAGE + G_BOFF);
#pragma unroll
    for (int j = 0; j < GW; ++j)
      if (slots & (1u << j)) {
        load16_to_lds(bp + (int64_t)cols[j] * (BS * 2), ld_off[0], dst + (uint32_t)(j * TILE));
        load16_to_lds(bp + (int64_t)cols[j] * (BS * 2), ld_off[1], dst + (uint32_t)(j * TILE) + 1024u);
      }
  };
  const uint32_t all_slots = (1u << ncols) - 1u, g0_slots = all_slots & ~g1_slots;

  f32x4 acc[2][4][4];  // [tile of the wave][16-row tile][16-column tile]
#pragma unroll
  for (int k = 0; k < 2; ++k)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[k][a][b][v] = 0.f;
  u32x4 af[2][2][4];  // [tile][kk][16-row tile]
  u32x4 bf[2][4];     // [kk][16-column tile]

  // prologue: step 0 whole, and group 0's W tiles of step 1 (nobody's memory phase comes early enough for them);
  // here every wave loads its eighth of every tile
  {
    const int row = wave * 8 + lane / 8, pch = lane % 8;
    const int rc = (r_tail >= 0 && row >= m_valid) ? m_valid - 1 : row;
    const uint32_t a_lane = (uint32_t)(row * g.a.sr + (pch ^ ((row >> 1) & 7)) * 8) * 2u;
    const uint32_t a_lane_m = (uint32_t)(rc * g.a.sr + (pch ^ ((row >> 1) & 7)) * 8) * 2u;
    const uint32_t b_lane = (uint32_t)(row * g.b.sc + (pch ^ swz_x(row)) * 8) * 2u;
    const uint32_t dst = smem_a + (uint32_t)(wave * 1024);
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (rowmask & (1u << r)) load16_to_lds(a_base + r * a_tile_stride, r == r_tail ? a_lane_m : a_lane, dst + (uint32_t)(r * TILE));
#pragma unroll
    for (int j = 0; j < GW; ++j) {
      if (all_slots & (1u << j)) load16_to_lds(b_base + (int64_t)cols[j] * (BS * 2), b_lane, dst + (uint32_t)(G_BOFF + j * TILE));
      if (nsteps > 1 && (g0_slots & (1u << j)))
        load16_to_lds(b_base + b_step_stride + (int64_t)cols[j] * (BS * 2), b_lane, dst + (uint32_t)(G_STAGE + G_BOFF + j * TILE));
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (grp1) __syncthreads();  // phase 0 belongs to group 0
  for (int step = 0; step < nsteps; ++step) {
    const int stage = step & 1;
    // ---- memory phase
    if (!grp1) {
      if (step + 1 < nsteps) load_dy(step + 1, stage ^ 1);
    } else {
      if (step + 1 < nsteps) load_w(step + 1, stage ^ 1, g1_slots);
      if (step + 2 < nsteps) load_w(step + 2, stage, g0_slots);
    }
    const char* st = smem + stage * G_STAGE;
    if (n_mine > 0) {
      const char* bt = st + G_BOFF + my_j * TILE;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          const char* p = bt + (b_off[kk] ^ (h * 32));
          const u32x2 lo = lds_read_tr(p), hi = lds_read_tr(p + 4 * 128);
          bf[kk][h] = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
    }
#pragma unroll
    for (int k = 0; k < 2; ++k)
      if (k < n_mine) {
        const char* at = st + my_r[k] * TILE;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int h = 0; h < 4; ++h) af[k][kk][h] = *reinterpret_cast<const u32x4*>(at + a_off[kk] + h * 16 * 128);
      }
    __syncthreads();
    // ---- compute phase
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int k = 0; k < 2; ++k)
      if (k < n_mine) {
        {
          // a mask of block size 32 drops quadrants of a kept tile: their MFMAs are left out and their accumulators stay
          // zero, which is what the epilogue then stores
#pragma unroll
          for (int mh = 0; mh < 2; ++mh)
#pragma unroll
            for (int nh = 0; nh < 2; ++nh)
              if ((my_q[k] >> (2 * mh + nh)) & 1u) {
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                  for (int mt = 2 * mh; mt < 2 * mh + 2; ++mt)
#pragma unroll
                    for (int nt = 2 * nh; nt < 2 * nh + 2; ++nt) acc[k][mt][nt] = T::mfma16(af[k][kk][mt], bf[kk][nt], acc[k][mt][nt]);
              }
        }
      }
    __builtin_amdgcn_s_setprio(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads have landed
    if (!(grp1 && step + 1 == nsteps)) __syncthreads();  // (group 1's last compute phase is nobody's memory phase)
  }

  // ---- epilogue: as in the other SDD kernel.  Group 0 gets here while group 1 still computes its last step, which
  // reads no LDS any more.
  constexpr int S_PITCH = BS + 4;
  float* stg = reinterpret_cast<float*>(smem) + wave * (BS * S_PITCH);
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    if (k >= n_mine) continue;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 4; ++v)  // register v of lane l is element (4*(l/16) + v, l%16) of the 16 x 16 tile
          stg[(mt * 16 + 4 * (lane / 16) + v) * S_PITCH + nt * 16 + lane % 16] = acc[k][mt][nt][v];
    store_staged_tile<T, true, BS, BS>(g, stg, lane, true, (int64_t)(rb0 + my_r[k]) * BS, (int64_t)my_c * BS, nullptr);
  }
}

template <typename T, bool EDGE, typename G>
__device__ __forceinline__ void sdd_any_body(const GemmArgs& g, int tiles_m, int gmax, int Mb, int Cb, const int bid) {
  // aligned operands on the 4-row-block shape: the kernel whose waves alternate between memory and compute phases
  if constexpr (!EDGE && G::R == 4) sdd_pp_body<T>(g, tiles_m, gmax, Mb, Cb, bid);
  else sdd_body<T, EDGE, G>(g, tiles_m, gmax, Mb, Cb, bid);
}

template <typename T, bool EDGE, typename G>
__global__ __launch_bounds__(THREADS) void sdd_group_kernel(GemmArgs g, int tiles_m, int gmax, int Mb, int Cb) {
  sdd_any_body<T, EDGE, G>(g, tiles_m, gmax, Mb, Cb, (int)blockIdx.x);
}

// Both gradients of one layer in one launch: workgroups [0, n_dx) are the SDD product's (dX; those past its own
// grid exit: n_dx is rounded up to the 8 XCDs so that the second product's tile map keeps its XCD assignment), the
// rest the weight gradient's (DSD on reduction-strided operands, column-major C; a split reduction leaves fp32
// partials for the reduce pass as in the kernel of its own).  One launch instead of
// two, and the second product's workgroups fill the CUs the first one's last round leaves idle - for small layers,
// whose grids cover a fraction of the chip each, the two simply run side by side.
template <typename T, bool EDGE, typename G, typename S>
__global__ __launch_bounds__(THREADS) void backward_pair_kernel(GemmArgs gx, int x_tiles_m, int x_gmax, int x_Mb,
                                                                int x_Cb, int n_dx, GemmArgs gw, int w_tiles_m,
                                                                int w_tiles_n, int w_Mb, int w_Kb, int w_splits) {
  static_assert(S::THREADS == THREADS, "both products run on 512 threads");
  const int bid = (int)blockIdx.x;
  if (bid < n_dx) {
    if (bid < x_tiles_m * x_gmax) sdd_any_body<T, EDGE, G>(gx, x_tiles_m, x_gmax, x_Mb, x_Cb, bid);
  } else {
    // the weight gradient's workgroups, tile index fastest, then the part of a split reduction
    const int wb = bid - n_dx, w_tiles = w_tiles_m * w_tiles_n;
    dsd_body<T, true, true, EDGE, S, 0>(gw, w_tiles_m, w_tiles_n, w_Mb, w_Kb, ImplicitConv{}, wb % w_tiles, w_splits,
                                        wb / w_tiles);
  }
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// Raises a kernel's dynamic LDS limit once per device (the attribute belongs to the device's copy of the
// kernel); `done` is the caller's per-kernel record.
constexpr int kMaxDevices = 64;
int allow_big_lds(const void* kernel, int bytes, std::atomic<bool> (&done)[kMaxDevices]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(SD_ERR_RUNTIME, "hipGetDevice failed or device index out of range");
  // concurrent first calls may both set the attribute (to the same value): harmless
  if (!done[dev].load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(SD_ERR_RUNTIME, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    done[dev].store(true, std::memory_order_release);
  }
  return SD_OK;
}

std::atomic<int> tile_policy{0};

template <typename T, bool TRANS, bool CM, bool RAGGED, typename S>
int launch_dsd_s(const GemmArgs& g, int splits, hipStream_t stream) {
  static std::atomic<bool> configured[kMaxDevices] = {};
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(&dsd_kernel<T, TRANS, CM, RAGGED, S>), S::SMEM_BYTES,
                             configured))
    return rc;
  const int Mb = (int)((g.M + BS - 1) / BS), Kb = (int)((g.K + BS - 1) / BS);
  const int tiles_m = (Mb + S::R - 1) / S::R, tiles_n = (int)((g.N + S::BN - 1) / S::BN);
  hipLaunchKernelGGL((dsd_kernel<T, TRANS, CM, RAGGED, S>), dim3((unsigned)(tiles_m * tiles_n), (unsigned)splits),
                     dim3(S::THREADS), S::SMEM_BYTES, stream, g, tiles_m, tiles_n, Mb, Kb, ImplicitConv{});
  if (int rc = check_launch("dsd_kernel")) return rc;
  note_kernel("dsd:%s%s%s splits=%d", S::R * BS == 256 && S::BN == 256 ? "big" : "mid", TRANS ? ":strided" : "",
              RAGGED ? ":ragged" : "", splits);
  if (splits > 1) return launch_splitk_reduce(g, splits, CM, T::id, stream);
  return SD_OK;
}

template <typename S>
int64_t dsd_tiles(int64_t M, int64_t N) {
  return ((M + BS * S::R - 1) / (BS * S::R)) * ((N + S::BN - 1) / S::BN);
}
bool mid_tiles_fit_one_round(const GemmArgs& g, int splits) { return dsd_tiles<DsdMid>(g.M, g.N) * splits <= 256; }

template <typename T, bool TRANS, bool CM>
int launch_dsd(const GemmArgs& g, bool mid, int splits, hipStream_t stream) {
  // masks of block size 32 (quadrant keep bits in the lists): the 256 x 256 shape leaves out the MFMAs of dropped
  // quadrants on aligned operands; elsewhere they run on the ragged-edge instance, which zeroes fragments
  const bool ragged = g.M % BS != 0 || g.N % BS != 0 || g.K % BS != 0 || (g.quads && mid);
  if (mid) {
    if (ragged) return launch_dsd_s<T, TRANS, CM, true, DsdMid>(g, splits, stream);
    // one round of workgroups or less: a CU has one workgroup whatever its LDS, and the four-stage loop is the faster
    // one (4096 x 1024 x 4096: 67 -> 52 us; 2048^3: 39 -> 30 us).  With more, two workgroups of the two-stage shape
    // share a CU and keep its LDS busier than one of the four-stage shape can (8192^3 on this shape: 1.09 against
    // 1.34 ms).
    return mid_tiles_fit_one_round(g, splits) ? launch_dsd_s<T, TRANS, CM, false, DsdMidDeep>(g, splits, stream)
                                              : launch_dsd_s<T, TRANS, CM, false, DsdMid>(g, splits, stream);
  }
  return ragged ? launch_dsd_s<T, TRANS, CM, true, DsdBig>(g, splits, stream)
                : launch_dsd_s<T, TRANS, CM, false, DsdBig>(g, splits, stream);
}


// workgroups a tile shape gives and how many ways the reduction is then split
struct DsdPlan {
  bool mid;
  int splits;
};
// One round of workgroups (one per CU) when the output alone gives fewer than half of that and the
// reduction is long enough to pay for the extra pass: at least 8 reduction blocks per split.
int splits_for(int64_t tiles, int64_t M, int64_t N, int64_t K) {
  const int64_t kb = K / BS;
  if (tiles >= 128 || kb < 32) return 1;
  int64_t want = 256 / tiles;
  if (want > kb / 8) want = kb / 8;
  while (want > 1 && want * M * N * 4 > (256LL << 20)) --want;
  return want < 2 ? 1 : (int)want;
}
DsdPlan plan_dsd(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return {false, 1};
  const int policy = tile_policy.load(std::memory_order_relaxed);
  const int64_t big = dsd_tiles<DsdBig>(M, N), midt = dsd_tiles<DsdMid>(M, N);
  // the 256 x 256 shape when it gives more than half of the CUs a workgroup (measured: 1024^3 forward 29 us on
  // 16 big tiles, 13 us on 64 mid tiles; 2048^3 29 + 18 us on 64 big tiles x 4 splits and the reduce pass,
  // 24 us on 256 mid tiles; 8192 x 1024 x 1024, 128 big tiles, 30 against 22 us; 3072^3, 144 big tiles, 79
  // against 94 us; 4096^3, 256 big tiles, 127 against 158 us; weight gradients over 16384 to 131072 rows
  // 15-30 % faster on mid tiles x fewer splits)
  const bool mid = policy == kTileMid || (policy == kTileAuto && big <= 128);
  return {mid, splits_for(mid ? midt : big, M, N, K)};
}

template <typename T, bool EDGE, typename G>
int launch_sdd_shape(const GemmArgs& g, hipStream_t stream) {
  static std::atomic<bool> configured[kMaxDevices] = {};
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(&sdd_group_kernel<T, EDGE, G>), G::SMEM, configured)) return rc;
  const int Mb = (int)((g.M + BS - 1) / BS), Cb = (int)((g.N + BS - 1) / BS);
  // the grid provides for the most groups a row of the block grid can split into
  const int tiles_m = (Mb + G::R - 1) / G::R, gmax = (Cb + G::MINCOLS - 1) / G::MINCOLS;
  hipLaunchKernelGGL((sdd_group_kernel<T, EDGE, G>), dim3((unsigned)(tiles_m * gmax)), dim3(THREADS), G::SMEM, stream,
                     g, tiles_m, gmax, Mb, Cb);
  note_kernel("sdd:%s%s", G::R == 4 ? "big" : (G::GW == 2 ? "small" : "mid"), EDGE ? ":ragged" : "");
  return check_launch("sdd_group_kernel");
}

// the big shape when its grid (a workgroup per 4 x 4 tiles, per 4 x 6 at high drop rates) gives more than half of
// the CUs a workgroup
template <typename T>
int launch_sdd_group(const GemmArgs& g, bool ragged, hipStream_t stream) {
  const int64_t Mb = (g.M + BS - 1) / BS, Cb = (g.N + BS - 1) / BS;
  // workgroups the big shape would have: a group spans 4 column blocks with everything kept, 6 once few enough tiles
  // are kept for the width and not the tile count to end a group (measured: worth counting that way from p = 0.7).
  // The kept fraction is the caller's hint (the lists live on the device); unknown counts as everything kept.
  const float keep = (g.row_ptr && g.keep_hint >= 0.f && g.keep_hint <= 1.f) ? g.keep_hint : 1.f;
  const int64_t cols = keep <= 0.3f ? SddBig::GW : SddBig::MINCOLS;
  const int64_t big = ((Mb + 3) / 4) * ((Cb + cols - 1) / cols);
  const int policy = tile_policy.load(std::memory_order_relaxed);
  const bool mid = policy == kTileMid || (policy == kTileAuto && big <= 128);
  // masks of block size 32 (quadrant keep bits in the lists): the big shape leaves out the MFMAs of dropped quadrants
  // on aligned operands; the other instances zero them in the epilogue, which lives in the ragged-edge code
  if (!mid) return (ragged ? launch_sdd_shape<T, true, SddBig> : launch_sdd_shape<T, false, SddBig>)(g, stream);
  if (ragged || g.quads) return launch_sdd_shape<T, true, SddMid>(g, stream);
  // aligned: the loops with several steps in flight (the two-stage shape holds a CU alone as well: its epilogue's
  // staging tiles take 136 KB).  Half a round of workgroups or less on the 2 x 4 shape: the 2 x 2 shape, twice as many
  // (4096 x 4096 -> 1024 columns: 93 us on 128 workgroups of the two-stage shape).
  const int64_t mid_wgs = ((Mb + 1) / 2) * ((Cb + 3) / 4);
  if (policy == kTileAuto && mid_wgs <= 128) return launch_sdd_shape<T, false, SddSmall>(g, stream);
  return launch_sdd_shape<T, false, SddMidDeep>(g, stream);
}

int try_sdd(const GemmArgs& g, int dtype, hipStream_t stream) {
  if (g.row_ptr && g.bs != BS) return SD_ERR_UNSUPPORTED;
  const bool layout_ok = g.a.sc == 1 && g.b.sr == 1 && g.b.sc != 1 && g.c_sc == 1;
  const bool shape_ok = g.M > 0 && g.N > 0 && g.N % 8 == 0 && g.K > 0 && g.K % 8 == 0;  // any M
  const bool align_ok = aligned16(g.a.ptr) && aligned16(g.b.ptr) && aligned16(g.c) && g.a.sr % 8 == 0 &&
                        g.b.sc % 8 == 0 && g.c_sr % 8 == 0 && g.a.sr < (1 << 22) &&
                        g.b.sc < (1 << 22);  // per-lane byte offsets are 32-bit
  const int64_t Cb = (g.N + BS - 1) / BS;
  const int64_t tiles = (((g.M + BS - 1) / BS + 1) / 2) * ((Cb + 3) / 4);  // the larger of the two shapes' grids
  if (!layout_ok || !shape_ok || !align_ok || tiles > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  if (Cb > G_MAX_CB) return SD_ERR_UNSUPPORTED;
  const bool ragged = g.N % BS != 0 || g.K % BS != 0;
  return dtype == SD_BF16 ? launch_sdd_group<BF16>(g, ragged, stream) : launch_sdd_group<F16>(g, ragged, stream);
}

template <typename T, bool RAGGED, int FORM>
int launch_conv_t(const GemmArgs& g, const ImplicitConv& cg, int smem, hipStream_t stream) {
  static std::atomic<bool> configured[kMaxDevices] = {};
  auto* kernel = &dsd_kernel<T, false, false, RAGGED, DsdConv, FORM>;
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(kernel), 163840, configured)) return rc;
  const int Mb = (int)(g.M / BS), Kb = (int)((g.K + BS - 1) / BS);
  const int tiles_m = (Mb + DsdConv::R - 1) / DsdConv::R, tiles_n = (int)((g.N + DsdConv::BN - 1) / DsdConv::BN);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n), 1u), dim3(DsdConv::THREADS), smem, stream, g,
                     tiles_m, tiles_n, Mb, Kb, cg);
  note_kernel("conv_fwd:implicit:%s", FORM == 2 ? "rows-per-step" : "rows-resident");
  return check_launch("dsd_kernel (implicit conv)");
}

template <typename T, bool RAGGED>
int launch_conv_dw_t(const GemmArgs& g, const ImplicitConv& cg, int smem, int splits, hipStream_t stream) {
  static std::atomic<bool> configured[kMaxDevices] = {};
  auto* kernel = &dsd_kernel<T, true, true, RAGGED, DsdConv, 1>;
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(kernel), 163840, configured)) return rc;
  const int Mb = (int)((g.M + BS - 1) / BS), Kb = (int)(g.K / BS);
  const int tiles_m = (Mb + DsdConv::R - 1) / DsdConv::R, tiles_n = (int)((g.N + DsdConv::BN - 1) / DsdConv::BN);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n), (unsigned)splits), dim3(DsdConv::THREADS), smem, stream,
                     g, tiles_m, tiles_n, Mb, Kb, cg);
  if (int rc = check_launch("dsd_kernel (implicit conv weight gradient)")) return rc;
  note_kernel("conv_dw:implicit splits=%d", splits);
  if (splits > 1) return launch_splitk_reduce(g, splits, true, T::id, stream);
  return SD_OK;
}

}  // namespace

// g: M = C*R*S (rows of the result), N = K_out, K = N*P*Q (the reduction); b = dY^T (b.sr == 1), c column-major
// (c_sr == 1); lists = the CSC lists of the patch matrix's mask (kept row blocks per column block).
int launch_conv_implicit_dw(const GemmArgs& g, ImplicitConv cg, int64_t P, int64_t stride_h, int64_t stride_w,
                            int64_t dil_h, int64_t dil_w, int64_t R, int64_t x_sw, int dtype, hipStream_t stream) {
  if (g.row_ptr != nullptr && g.bs != BS) return SD_ERR_UNSUPPORTED;
  const bool geom_ok = stride_h == cg.sth && stride_w == cg.stw && dil_h == cg.dlh && dil_w == cg.dlw && x_sw == 1 &&
                       cg.Q > 0 && cg.Q <= BS && BS % cg.Q == 0 && (P * cg.Q) % BS == 0 && cg.W % 8 == 0 &&
                       cg.pad_h >= 0 && cg.pad_w >= 0 && cg.pad_w <= 8 && (cg.S - 1) * dil_w - cg.pad_w <= 8 &&
                       R * cg.S == cg.RS && cg.PW == cg.W + 8 &&
                       cg.PR == (cg.rpb - 1) * stride_h + (R - 1) * dil_h + 1;
  if (!geom_ok) return SD_ERR_UNSUPPORTED;
  const int64_t nch_max = (DsdConv::R * BS - 1) / cg.RS + 2;  // channels 256 consecutive columns can touch
  const int64_t copy_elems = ((nch_max < cg.C ? nch_max : cg.C) * cg.PR * cg.PW + 8 + 7) & ~7LL;
  if (copy_elems * 2 > CONV_T_PATCH_MAX) return SD_ERR_UNSUPPORTED;
  cg.patch_stride = (int)copy_elems;
  const int64_t extra = 2 * copy_elems * 2 + DsdConv::R * BS * 2;
  const int smem = ((DsdConv::SMEM_BYTES + 15) & ~15) + (int)extra;
  if (smem > 163840) return SD_ERR_UNSUPPORTED;
  const bool align_ok = aligned16(cg.x) && cg.sn % 8 == 0 && cg.sc % 8 == 0 && cg.sh % 8 == 0 && aligned16(g.b.ptr) &&
                        g.b.sr == 1 && g.b.sc % 8 == 0 && g.b.sc < (1 << 22) && g.c_sr == 1 && g.M % 8 == 0 &&
                        g.N % 8 == 0 && g.K % BS == 0 && g.K / BS < 65536;
  if (!align_ok) return SD_ERR_UNSUPPORTED;
  // the reduction over positions is long and the result small: split it over workgroups as the explicit kernel does
  const int64_t tiles = dsd_tiles<DsdConv>(g.M, g.N);
  int splits = splits_for(tiles, g.M, g.N, g.K);
  const int64_t part_bytes = g.M * g.N * 4;
  if (splits > 1 && (g.ws == nullptr || g.ws_bytes < part_bytes * splits)) splits = g.ws ? (int)(g.ws_bytes / part_bytes) : 1;
  if (splits < 1) splits = 1;
  if ((g.K / BS + splits - 1) / splits > MAX_STEPS) return SD_ERR_UNSUPPORTED;
  const bool ragged = g.M % BS != 0 || g.N % BS != 0;
  if (dtype == SD_BF16)
    return ragged ? launch_conv_dw_t<BF16, true>(g, cg, smem, splits, stream)
                  : launch_conv_dw_t<BF16, false>(g, cg, smem, splits, stream);
  return ragged ? launch_conv_dw_t<F16, true>(g, cg, smem, splits, stream)
                : launch_conv_dw_t<F16, false>(g, cg, smem, splits, stream);
}

int conv_dw_splits(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 1;
  return splits_for(dsd_tiles<DsdConv>(M, N), M, N, K);
}

int launch_conv_implicit(const GemmArgs& g, const ImplicitConv& cg, int64_t P, int64_t stride_h, int64_t stride_w,
                         int64_t dil_h, int64_t dil_w, int64_t R, int64_t x_sw, int dtype, hipStream_t stream) {
  if (g.row_ptr != nullptr && g.bs != BS) return SD_ERR_UNSUPPORTED;
  // the four row blocks of a workgroup: consecutive output rows of one image sharing their input rows (units == 1,
  // P * Q a multiple of 256), or each with its own input rows (units == 4, P * Q a multiple of 64)
  const int64_t taps_h = (R - 1) * dil_h + 1;  // input rows under one output row
  const bool units_ok =
      (cg.units == 1 && (P * cg.Q) % (BS * DsdConv::R) == 0 && cg.PR == (DsdConv::R * cg.rpb - 1) * stride_h + taps_h) ||
      (cg.units == 4 && (P * cg.Q) % BS == 0 && cg.PR == (cg.rpb - 1) * stride_h + taps_h);
  const bool geom_ok = stride_h == cg.sth && stride_w == cg.stw && dil_h == cg.dlh && dil_w == cg.dlw && x_sw == 1 &&
                       cg.Q > 0 && cg.Q <= BS && BS % cg.Q == 0 && units_ok && cg.W % 8 == 0 && cg.pad_h >= 0 &&
                       cg.pad_w >= 0 && cg.pad_w <= 8 && (cg.S - 1) * dil_w - cg.pad_w <= 8 && R * cg.S == cg.RS &&
                       cg.PW == cg.W + 8;
  if (!geom_ok) return SD_ERR_UNSUPPORTED;
  const int64_t Kb = (g.K + BS - 1) / BS;
  if (Kb > MAX_STEPS) return SD_ERR_UNSUPPORTED;
  const bool align_ok = aligned16(cg.x) && cg.sn % 8 == 0 && cg.sc % 8 == 0 && cg.sh % 8 == 0 && aligned16(g.b.ptr) &&
                        g.b.sc == 1 && g.b.sr % 8 == 0 && g.b.sr < (1 << 22) && g.c_sc == 1 && g.K % 8 == 0 &&
                        g.M % BS == 0 && (g.M / (BS * DsdConv::R) + 1) * ((g.N + 127) / 128) < 0x7fffffffLL;
  if (!align_ok) return SD_ERR_UNSUPPORTED;
  // two alternating copies of the channels one step's 64 columns touch (any number of channels; measured at least
  // as fast as the other form wherever both fit) ...
  const int64_t nch = (BS + cg.RS - 2) / cg.RS + 1;
  const int64_t copy_elems = (cg.units * nch * cg.PR * cg.PW + 8 + 7) & ~7LL;
  const int64_t stepwise = 2 * copy_elems * 2 + Kb * BS * 2;
  const bool step_ok = copy_elems * 2 <= CONV_T_PATCH_MAX && stepwise <= CONV_PATCH_MAX;
  // ... or one copy of every channel's rows for the whole kernel if that fits next to the stages (many taps per
  // 64 columns, e.g. 1 x 1 kernels, make a step's copy large; the large-tile policy prefers this form)
  const int64_t patch_elems = (int64_t)cg.C * cg.PR * cg.PW + 8;  // rows with their halo groups, one more after the last
  const int64_t whole = patch_elems * 2 + Kb * BS * 2;
  const bool whole_ok = whole <= CONV_PATCH_MAX && cg.units == 1;
  if (!step_ok && !whole_ok) return SD_ERR_UNSUPPORTED;
  const bool use_steps = step_ok && !(whole_ok && tile_policy.load(std::memory_order_relaxed) == kTileBig);
  const bool ragged = g.N % BS != 0 || g.K % BS != 0;
  if (use_steps) {
    ImplicitConv cs = cg;
    cs.patch_stride = (int)copy_elems;
    const int smem = ((DsdConv::SMEM_BYTES + 15) & ~15) + (int)stepwise;
    if (dtype == SD_BF16)
      return ragged ? launch_conv_t<BF16, true, 2>(g, cs, smem, stream) : launch_conv_t<BF16, false, 2>(g, cs, smem, stream);
    return ragged ? launch_conv_t<F16, true, 2>(g, cs, smem, stream) : launch_conv_t<F16, false, 2>(g, cs, smem, stream);
  }
  const int smem = ((DsdConv::SMEM_BYTES + 15) & ~15) + (int)whole;
  if (dtype == SD_BF16)
    return ragged ? launch_conv_t<BF16, true, 1>(g, cg, smem, stream) : launch_conv_t<BF16, false, 1>(g, cg, smem, stream);
  return ragged ? launch_conv_t<F16, true, 1>(g, cg, smem, stream) : launch_conv_t<F16, false, 1>(g, cg, smem, stream);
}

// How many ways the DSD kernel splits the reduction of this product: the plan's count cut down to what the caller's
// scratch holds; 0 = the specialised kernel should not take the product (its step table is per workgroup, and with
// scratch too small for its own partials the generic kernel's split may still fit).
int usable_splits(const GemmArgs& g, const DsdPlan& plan, int mode) {
  const int64_t tiles = plan.mid ? dsd_tiles<DsdMid>(g.M, g.N) : dsd_tiles<DsdBig>(g.M, g.N);
  int splits = plan.splits;
  const int64_t part_bytes = g.M * g.N * 4;
  if (splits > 1 && (g.ws == nullptr || g.ws_bytes < part_bytes * splits))
    splits = g.ws ? (int)(g.ws_bytes / part_bytes) : 1;
  if (splits < 1) splits = 1;
  if (((g.K + BS - 1) / BS + splits - 1) / splits > MAX_STEPS) return 0;
  if (splits == 1 && tiles < 128 && g.ws != nullptr) {
    const int gs = generic_splits(g.M, g.N, g.K, g.bs, mode);
    if (gs > 1 && g.ws_bytes >= (int64_t)gs * part_bytes) return 0;
  }
  return splits;
}

// most workgroups either product of a single-launch backward may have (SPARSEDROP_PAIR_LIMIT overrides, for measuring)
int64_t pair_limit() {
  static const int64_t limit = [] {
    const char* e = std::getenv("SPARSEDROP_PAIR_LIMIT");
    return e ? (int64_t)std::atoll(e) : (int64_t)512;
  }();
  return limit;
}

int launch_fast(const GemmArgs& g, int mode, int dtype, hipStream_t stream) {
  if (mode == kSdd) return try_sdd(g, dtype, stream);
  // a dense product of a row-major A with a reduction-strided B (dX = dY.W without dropout) is the SDD
  // kernel with every tile kept
  if (mode == kDense && g.a.sc == 1 && g.b.sr == 1 && g.b.sc != 1 && g.c_sc == 1) return try_sdd(g, dtype, stream);
  if (mode == kDsd && g.bs != BS) return SD_ERR_UNSUPPORTED;
  // everything tile-aligned and 16-byte aligned; A and B agree on whether the reduction index is contiguous
  const bool nt = g.a.sc == 1 && g.b.sc == 1;         // reduction-contiguous operands
  const bool tn = !nt && g.a.sr == 1 && g.b.sr == 1;  // reduction-strided operands
  const bool cm = g.c_sc != 1;                        // column-major C
  // ragged edges: any extent along a strided index, multiples of 8 (the 16 bytes of a load) along a contiguous one
  const bool shape_ok = g.M > 0 && (nt || g.M % 8 == 0) && g.N > 0 && (nt || g.N % 8 == 0) && g.K > 0 &&
                        (tn || g.K % 8 == 0) && (g.K + BS - 1) / BS < 65536;
  const int64_t lda = nt ? g.a.sr : g.a.sc, ldb = nt ? g.b.sr : g.b.sc;
  const bool align_ok = aligned16(g.a.ptr) && aligned16(g.b.ptr) && lda % 8 == 0 && ldb % 8 == 0 &&
                        lda < (1 << 22) && ldb < (1 << 22);  // per-lane byte offsets are 32-bit
  const DsdPlan plan = plan_dsd(g.M, g.N, g.K);
  const int64_t tiles = plan.mid ? dsd_tiles<DsdMid>(g.M, g.N) : dsd_tiles<DsdBig>(g.M, g.N);
  if (!(nt || tn) || !shape_ok || !align_ok || tiles > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  // few output tiles and a long reduction (the weight gradient of a tall matrix): split the reduction
  // over workgroups when the caller gave scratch for the fp32 partials
  const int splits = usable_splits(g, plan, mode);
  if (splits < 1) return SD_ERR_UNSUPPORTED;
  const bool mid = plan.mid;
  if (dtype == SD_BF16) {
    if (nt) return cm ? launch_dsd<BF16, false, true>(g, mid, splits, stream) : launch_dsd<BF16, false, false>(g, mid, splits, stream);
    return cm ? launch_dsd<BF16, true, true>(g, mid, splits, stream) : launch_dsd<BF16, true, false>(g, mid, splits, stream);
  }
  if (nt) return cm ? launch_dsd<F16, false, true>(g, mid, splits, stream) : launch_dsd<F16, false, false>(g, mid, splits, stream);
  return cm ? launch_dsd<F16, true, true>(g, mid, splits, stream) : launch_dsd<F16, true, false>(g, mid, splits, stream);
}

// ---- the forward product and the kept lists of its mask in one launch -------------------------------------------
// most workgroups the product may have for its lists to ride along (SPARSEDROP_FORWARD_LISTS_LIMIT overrides, for
// measuring; 0 switches the single launch off)
int64_t forward_lists_limit() {
  static const int64_t limit = [] {
    const char* e = std::getenv("SPARSEDROP_FORWARD_LISTS_LIMIT");
    return e ? (int64_t)std::atoll(e) : (int64_t)512;
  }();
  return limit;
}

template <typename T, bool RAGGED, typename S>
int launch_forward_lists_t(const GemmArgs& g, int splits, const FlatJobs& f, hipStream_t stream) {
  static std::atomic<bool> configured[kMaxDevices] = {};
  auto* kernel = &forward_lists_kernel<T, RAGGED, S>;
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(kernel), S::SMEM_BYTES, configured)) return rc;
  const int Mb = (int)((g.M + BS - 1) / BS), Kb = (int)((g.K + BS - 1) / BS);
  const int tiles_m = (Mb + S::R - 1) / S::R, tiles_n = (int)((g.N + S::BN - 1) / S::BN);
  const int n_gemm = tiles_m * tiles_n * splits;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(n_gemm + f.blocks())), dim3(S::THREADS), S::SMEM_BYTES, stream, g, tiles_m,
                     tiles_n, Mb, Kb, splits, n_gemm, f);
  if (int rc = check_launch("forward_lists_kernel")) return rc;
  note_kernel("dsd+lists:%s%s splits=%d", S::R * BS == 256 && S::BN == 256 ? "big" : "mid", RAGGED ? ":ragged" : "",
              splits);
  if (splits > 1) return launch_splitk_reduce(g, splits, false, T::id, stream);
  return SD_OK;
}

// g: the forward product (reduction-contiguous operands, row-major C) on the 64 grid; src: its mask, listed on an
// mb x kb grid into the arrays given (either list may be absent), a drawn mask stored to mask_out.
// SD_ERR_UNSUPPORTED (nothing launched, no message) unless the product runs on the specialised kernel, the mask is
// small enough for the single-launch list build and the product small enough for the saved launch to matter.
int launch_forward_with_lists(const GemmArgs& g, const MaskSrc& src, int64_t mb, int64_t kb, int32_t* row_ptr,
                              int32_t* col_idx, int32_t* col_ptr, int32_t* row_idx, uint8_t* mask_out,
                              int64_t mask_rows, int dtype, hipStream_t stream) {
  if (g.bs != BS || mb * kb > kFlatMaxEntries) return SD_ERR_UNSUPPORTED;
  if (mb != (g.M + BS - 1) / BS || kb != (g.K + BS - 1) / BS) return SD_ERR_UNSUPPORTED;
  // the forward's conditions (launch_fast)
  const bool nt = g.a.sc == 1 && g.b.sc == 1 && g.c_sc == 1;
  const bool shape_ok = g.M > 0 && g.N > 0 && g.K > 0 && g.K % 8 == 0 && (g.K + BS - 1) / BS < 65536;
  const bool align_ok = aligned16(g.a.ptr) && aligned16(g.b.ptr) && g.a.sr % 8 == 0 && g.b.sr % 8 == 0 &&
                        g.a.sr < (1 << 22) && g.b.sr < (1 << 22);
  if (!nt || !shape_ok || !align_ok) return SD_ERR_UNSUPPORTED;
  const DsdPlan plan = plan_dsd(g.M, g.N, g.K);
  const int64_t tiles = plan.mid ? dsd_tiles<DsdMid>(g.M, g.N) : dsd_tiles<DsdBig>(g.M, g.N);
  const int splits = usable_splits(g, plan, kDsd);
  if (splits < 1 || tiles * splits > forward_lists_limit()) return SD_ERR_UNSUPPORTED;
  const bool ragged = g.M % BS != 0 || g.N % BS != 0 || g.K % BS != 0 || (g.quads && plan.mid);
  const FlatJobs f = flat_jobs(src, mb, kb, row_ptr, col_idx, col_ptr, row_idx, mask_out, mask_rows,
                               plan.mid ? DsdMid::THREADS : DsdBig::THREADS);
  // the four-stage shape holds a CU alone, the list builder's blocks included: only when they all find a CU of their own
  // in one round (else the blocks that build the lists wait for a product workgroup to finish, and the two-stage shape,
  // which shares a CU with them, is as fast)
  const bool deep = plan.mid && !ragged && tiles * splits + f.blocks() <= 256;
  if (dtype == SD_BF16) {
    if (deep) return launch_forward_lists_t<BF16, false, DsdMidDeep>(g, splits, f, stream);
    if (plan.mid) return ragged ? launch_forward_lists_t<BF16, true, DsdMid>(g, splits, f, stream)
                                : launch_forward_lists_t<BF16, false, DsdMid>(g, splits, f, stream);
    return ragged ? launch_forward_lists_t<BF16, true, DsdBig>(g, splits, f, stream)
                  : launch_forward_lists_t<BF16, false, DsdBig>(g, splits, f, stream);
  }
  if (deep) return launch_forward_lists_t<F16, false, DsdMidDeep>(g, splits, f, stream);
  if (plan.mid) return ragged ? launch_forward_lists_t<F16, true, DsdMid>(g, splits, f, stream)
                              : launch_forward_lists_t<F16, false, DsdMid>(g, splits, f, stream);
  return ragged ? launch_forward_lists_t<F16, true, DsdBig>(g, splits, f, stream)
                : launch_forward_lists_t<F16, false, DsdBig>(g, splits, f, stream);
}

// ---- both gradients in one launch ------------------------------------------------------------------------
// gx: the SDD product dX = s (dY . W) on the kept tiles; gw: the DSD product dW^T = s X^T(kept blocks) . dY with
// reduction-strided operands and column-major C.  SD_ERR_UNSUPPORTED (nothing launched) unless each would run on its
// specialised kernel by itself, unsplit, and both on the same size of workgroup shape; the caller then launches them
// one after the other.
template <typename T, bool EDGE, typename G, typename S>
int launch_pair_t(const GemmArgs& gx, const GemmArgs& gw, int splits, hipStream_t stream) {
  constexpr int SMEM = G::SMEM > S::SMEM_BYTES ? G::SMEM : S::SMEM_BYTES;
  static std::atomic<bool> configured[kMaxDevices] = {};
  if (int rc = allow_big_lds(reinterpret_cast<const void*>(&backward_pair_kernel<T, EDGE, G, S>), SMEM, configured))
    return rc;
  const int x_Mb = (int)((gx.M + BS - 1) / BS), x_Cb = (int)((gx.N + BS - 1) / BS);
  const int x_tiles_m = (x_Mb + G::R - 1) / G::R, x_gmax = (x_Cb + G::MINCOLS - 1) / G::MINCOLS;
  const int64_t n_dx = ((int64_t)x_tiles_m * x_gmax + 7) / 8 * 8;
  const int w_Mb = (int)((gw.M + BS - 1) / BS), w_Kb = (int)((gw.K + BS - 1) / BS);
  const int w_tiles_m = (w_Mb + S::R - 1) / S::R, w_tiles_n = (int)((gw.N + S::BN - 1) / S::BN);
  const int64_t total = n_dx + (int64_t)w_tiles_m * w_tiles_n * splits;
  if (total > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((backward_pair_kernel<T, EDGE, G, S>), dim3((unsigned)total), dim3(THREADS), SMEM, stream, gx,
                     x_tiles_m, x_gmax, x_Mb, x_Cb, (int)n_dx, gw, w_tiles_m, w_tiles_n, w_Mb, w_Kb, splits);
  note_kernel("pair:sdd+dsd:%s%s splits=%d", G::R == 4 ? "big" : "mid", EDGE ? ":ragged" : "", splits);
  if (int rc = check_launch("backward_pair_kernel")) return rc;
  if (splits > 1) return launch_splitk_reduce(gw, splits, true, T::id, stream);
  return SD_OK;
}

int launch_backward_pair(const GemmArgs& gx, const GemmArgs& gw, int dtype, hipStream_t stream) {
  // the SDD product's conditions (try_sdd)
  if (!gx.row_ptr || gx.bs != BS || gx.kept_only) return SD_ERR_UNSUPPORTED;
  const int64_t x_Cb = (gx.N + BS - 1) / BS, x_Mb = (gx.M + BS - 1) / BS;
  const bool x_ok = gx.a.sc == 1 && gx.b.sr == 1 && gx.b.sc != 1 && gx.c_sc == 1 && gx.M > 0 && gx.N > 0 &&
                    gx.N % 8 == 0 && gx.K > 0 && gx.K % 8 == 0 && aligned16(gx.a.ptr) && aligned16(gx.b.ptr) &&
                    aligned16(gx.c) && gx.a.sr % 8 == 0 && gx.b.sc % 8 == 0 && gx.c_sr % 8 == 0 &&
                    gx.a.sr < (1 << 22) && gx.b.sc < (1 << 22) && x_Cb <= G_MAX_CB;
  // the weight gradient's (launch_fast), in the one form the autograd step produces
  if (!gw.row_ptr || gw.bs != BS || gw.act) return SD_ERR_UNSUPPORTED;
  const bool w_ok = gw.a.sr == 1 && gw.b.sr == 1 && gw.a.sc != 1 && gw.b.sc != 1 && gw.c_sc != 1 && gw.c_sr == 1 &&
                    gw.M > 0 && gw.M % 8 == 0 && gw.N > 0 && gw.N % 8 == 0 && gw.K > 0 && (gw.K + BS - 1) / BS < 65536 &&
                    aligned16(gw.a.ptr) && aligned16(gw.b.ptr) && aligned16(gw.c) && gw.a.sc % 8 == 0 &&
                    gw.b.sc % 8 == 0 && gw.c_sc % 8 == 0 && gw.a.sc < (1 << 22) && gw.b.sc < (1 << 22);
  if (!x_ok || !w_ok) return SD_ERR_UNSUPPORTED;
  const DsdPlan plan = plan_dsd(gw.M, gw.N, gw.K);
  const int splits = usable_splits(gw, plan, kDsd);
  if (splits < 1) return SD_ERR_UNSUPPORTED;
  // the SDD shape as launch_sdd_group picks it; both products must want the same size
  const float keep = (gx.keep_hint >= 0.f && gx.keep_hint <= 1.f) ? gx.keep_hint : 1.f;
  const int64_t cols = keep <= 0.3f ? SddBig::GW : SddBig::MINCOLS;
  const int64_t big = ((x_Mb + 3) / 4) * ((x_Cb + cols - 1) / cols);
  const int policy = tile_policy.load(std::memory_order_relaxed);
  const bool x_mid = policy == kTileMid || (policy == kTileAuto && big <= 128);
  if (x_mid != plan.mid) return SD_ERR_UNSUPPORTED;
  // Worth it only while neither product fills the chip by itself: side by side, two large products get in each
  // other's way in the L2 (8192^3 at p = 0.5: 1.33 ms in one launch against 1.28 in two; 1024^3: 27 us against 46).
  const int64_t x_wgs = x_mid ? ((x_Mb + 1) / 2) * ((x_Cb + 3) / 4) : big;
  const int64_t w_wgs = (plan.mid ? dsd_tiles<DsdMid>(gw.M, gw.N) : dsd_tiles<DsdBig>(gw.M, gw.N)) * splits;
  if (x_wgs > pair_limit() || w_wgs > pair_limit()) return SD_ERR_UNSUPPORTED;
  if ((x_Mb + 1) / 2 * ((x_Cb + 3) / 4) + dsd_tiles<DsdMid>(gw.M, gw.N) > 0x7fffffffLL) return SD_ERR_UNSUPPORTED;
  // either product ragged (or, on the smaller shapes, on a block-size-32 mask): the instances that handle edges, for both
  const bool edge = gx.N % BS != 0 || gx.K % BS != 0 || gw.M % BS != 0 || gw.N % BS != 0 || gw.K % BS != 0 ||
                    ((gx.quads || gw.quads) && x_mid);
  if (dtype == SD_BF16) {
    // (the smaller SDD shape holds a CU alone anyway: the loops with more stages cost nothing)
    if (x_mid) return edge ? launch_pair_t<BF16, true, SddMid, DsdMid>(gx, gw, splits, stream)
                           : launch_pair_t<BF16, false, SddMidDeep, DsdMidDeep>(gx, gw, splits, stream);
    return edge ? launch_pair_t<BF16, true, SddBig, DsdBig>(gx, gw, splits, stream)
                : launch_pair_t<BF16, false, SddBig, DsdBig>(gx, gw, splits, stream);
  }
  if (x_mid) return edge ? launch_pair_t<F16, true, SddMid, DsdMid>(gx, gw, splits, stream)
                         : launch_pair_t<F16, false, SddMidDeep, DsdMidDeep>(gx, gw, splits, stream);
  return edge ? launch_pair_t<F16, true, SddBig, DsdBig>(gx, gw, splits, stream)
              : launch_pair_t<F16, false, SddBig, DsdBig>(gx, gw, splits, stream);
}

int set_tile_policy(int policy) {
  if (policy != kTileAuto && policy != kTileBig && policy != kTileMid) return -1;
  return tile_policy.exchange(policy, std::memory_order_relaxed);
}

int fast_splits(int64_t M, int64_t N, int64_t K) { return plan_dsd(M, N, K).splits; }

}  // namespace sd
