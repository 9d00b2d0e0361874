// Grouped (per-expert) fp16 GEMM over expert-sorted rows, fp32 accumulate on MFMA.
//
//   y[start_e:end_e, :] = x[start_e:end_e, :] @ W_e^T,   W_e stored [n, k] (k contiguous)
//
// Both operands are K-contiguous, which is exactly the per-lane operand shape of
// v_mfma_f32_32x32x16_f16 (8 consecutive k per lane), so tiles go HBM -> registers -> LDS
// with 128-bit accesses and no transposition.  group_list is read on the device: every
// workgroup derives the (expert, m-tile, n-tile) it owns from a wave-level scan of the
// per-expert tile counts, so there is no host synchronisation and no planning kernel.
// Workgroups are renumbered so that each XCD (one L2 per XCD, workgroup i runs on XCD i%8)
// works through a contiguous range of experts, with the m-tiles that share a weight tile
// next to each other.
//
// Semantics: reference csrc/opdev/op_kernel/grouped_mat_mul_ex.cpp:27-44 (start/end from the
// cumulative int64 group_list, empty groups skipped), matmul_core.h:42-68 (NT product, fp32
// accumulate, fp16 result), benchmark/test_grouped_matmul.py:6-23.
#include <stdlib.h>

#include <type_traits>

#include "aops_common.h"

namespace aops {

constexpr int kBK = 64;   // k extent of one LDS stage
constexpr int kXcds = 8;

// Cumulative row end of expert e.  group_list == nullptr stands for a single group that holds
// every row (the dense NT matmul entry point).
__device__ __forceinline__ int64_t gmm_group_end(const int64_t* __restrict__ group_list, int e,
                                                 int64_t rows) {
  return group_list ? group_list[e] : rows;
}

struct GmmWork {
  int expert;
  int row_begin;  // first row of this m-tile
  int row_end;    // end of the expert's rows
  int n_tile;
  bool valid;
};

// Maps a work index to (expert, m-tile, n-tile).  Executed redundantly by every wave.
template <int kBM>
__device__ __forceinline__ GmmWork gmm_find_work(const int64_t* __restrict__ group_list,
                                                 int num_experts, int64_t rows, int n_tiles,
                                                 int wg, int num_wg) {
  const int lane = threadIdx.x & (kWave - 1);
  const int per = (num_experts + kWave - 1) / kWave;
  const int e0 = lane * per;
  auto clampr = [&](int64_t v) -> int { return (int)(v < 0 ? 0 : (v > rows ? rows : v)); };
  int tiles = 0;
  {
    int prev = (e0 == 0 || e0 > num_experts) ? 0 : clampr(gmm_group_end(group_list, e0 - 1, rows));
    for (int j = 0; j < per; ++j) {
      const int e = e0 + j;
      if (e < num_experts) {
        const int end = clampr(gmm_group_end(group_list, e, rows));
        if (end > prev) tiles += (end - prev + kBM - 1) / kBM;
        prev = end;
      }
    }
  }
  int incl = tiles;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  const int total_tiles = __shfl(incl, kWave - 1);
  const int64_t total_work = (int64_t)total_tiles * n_tiles;

  GmmWork w;
  w.valid = false;
  w.expert = w.row_begin = w.row_end = w.n_tile = 0;
  // XCD-aware renumbering: XCD x takes work items [x*share, (x+1)*share).
  const int64_t share = (total_work + kXcds - 1) / kXcds;
  const int xcd = wg % kXcds;
  const int64_t slot = wg / kXcds;
  (void)num_wg;
  if (slot >= share) return w;
  const int64_t work = (int64_t)xcd * share + slot;
  if (work >= total_work) return w;

  const int64_t lo = (int64_t)(incl - tiles) * n_tiles;
  const int64_t hi = (int64_t)incl * n_tiles;
  int f_expert = 0, f_begin = 0, f_end = 0, f_ntile = 0;
  const bool mine = work >= lo && work < hi;
  if (mine) {
    int64_t base = lo;
    int prev = (e0 == 0) ? 0 : clampr(gmm_group_end(group_list, e0 - 1, rows));
    for (int j = 0; j < per; ++j) {
      const int e = e0 + j;
      if (e >= num_experts) break;
      const int end = clampr(gmm_group_end(group_list, e, rows));
      const int t = end > prev ? (end - prev + kBM - 1) / kBM : 0;
      const int64_t span = (int64_t)t * n_tiles;
      if (work < base + span) {
        const int local = (int)(work - base);
        f_expert = e;
        f_ntile = local / t;  // m-tiles of one weight tile are adjacent
        f_begin = prev + (local - f_ntile * t) * kBM;
        f_end = end;
        break;
      }
      base += span;
      prev = end;
    }
  }
  const uint64_t mask = __ballot(mine);
  const int src = __builtin_ctzll(mask);  // exactly one lane owns the work item
  w.expert = __shfl(f_expert, src);
  w.row_begin = __shfl(f_begin, src);
  w.row_end = __shfl(f_end, src);
  w.n_tile = __shfl(f_ntile, src);
  w.valid = mask != 0;
  return w;
}

// Scheduling directive for one k step.  The step's LDS fragment reads (mask 0x100) follow its
// first two MFMAs (0x008): they feed the next step and need a full LDS round trip, so they go
// out first.  The staging LDS writes (0x200) and global loads (0x020) are then spread over the
// remaining MFMAs, so that their issue slots fall into the 32 cycles an MFMA keeps the matrix
// core busy.
template <int M, int NM, int NR, int NW, int NG>
struct MfmaInterleave {
  static __device__ __forceinline__ void run() {
    if constexpr (M < NM) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      constexpr int kReadSlots = NM < 2 ? NM : 2;
      constexpr int r = M < kReadSlots ? NR * (M + 1) / kReadSlots - NR * M / kReadSlots : 0;
      constexpr int w = NW * (M + 1) / NM - NW * M / NM;
      constexpr int g = NG * (M + 1) / NM - NG * M / NM;
      if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
      if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);
      if constexpr (g > 0) __builtin_amdgcn_sched_group_barrier(0x020, g, 0);
      MfmaInterleave<M + 1, NM, NR, NW, NG>::run();
    }
  }
};

// LDS tile [rows][kBK] halfs, 128 bytes per row.  16-byte chunk c of row r is stored in row
// r ^ ((r >> 3) & 1) at chunk position c ^ (r & 7): the 128-bit fragment reads of 8 or of 16
// consecutive rows (same c) then touch every bank once, whichever width the LDS serves per
// cycle, and so do the staging writes (8 consecutive chunks of a row per 8 lanes).
__device__ __forceinline__ int lds_off(int r, int c) {
  return (r ^ ((r >> 3) & 1)) * kBK + ((c ^ (r & 7)) << 3);
}

// Workgroup tile BM x BN = (64*MB) x (64*NB), four waves arranged 2 x 2.  Wave (wm, wn) owns
// the 32-row blocks wm, wm+2, wm+4, ... (interleaved, so that a group that fills only part of
// the tile still splits evenly between the two wave rows) and the 32*NB columns starting at
// wn*32*NB; its MB x NB accumulators of v_mfma_f32_32x32x16_f16 stay in registers for the
// whole k loop.  The products are formed as W.x^T (weight fragment as the first operand): a lane
// then holds 4 consecutive output columns of one output row, which the epilogue packs to
// 8 bytes, transposes through LDS and writes with 128-bit row-contiguous stores.
//
// Software pipeline per k tile (kBK = 64):
//   global -> registers, D tiles ahead (the loads of tile kt+1+D are issued in iteration kt),
//   registers -> LDS stage (kt+1)&1 during iteration kt, one barrier per k tile,
//   LDS -> MFMA fragments one 16-wide k step ahead of the matrix cores.
template <int MB, int NB, int D>
__global__ __launch_bounds__(4 * kWave) void grouped_matmul_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 64 * NB;
  constexpr int kThreads = 4 * kWave;
  constexpr int kAChunks = BM * (kBK / 8) / kThreads;  // 16-byte chunks per thread and tile
  constexpr int kBChunks = BN * (kBK / 8) / kThreads;
  constexpr int kRowsPerPass = kThreads / 8;           // tile rows covered by one chunk per thread
  constexpr int kSteps = kBK / 16;
  static_assert(D == 1 || D == 2, "prefetch distance");
  static_assert(kRowsPerPass % 16 == 0, "swizzle must be invariant under the row stride");

  extern __shared__ __attribute__((aligned(16))) f16 smem[];
  f16* sa = smem;                 // [2][BM * kBK]
  f16* sb = smem + 2 * BM * kBK;  // [2][BN * kBK]

  const int n_tiles = (n + BN - 1) / BN;
  const GmmWork work =
      gmm_find_work<BM>(group_list, num_experts, rows, n_tiles, blockIdx.x, gridDim.x);
  if (!work.valid) return;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1;
  const int wn = wave & 1;
  const int tile_rows = min(work.row_end - work.row_begin, BM);
  // 32-row blocks of this wave that hold at least one real row (wave uniform, 0..MB)
  const int live_blocks = (tile_rows + 31) / 32;
  const int live = (live_blocks - wm + 1) / 2;

  // Global -> register staging: thread handles chunk (row = tid/8 + kRowsPerPass*i, kc = tid%8).
  // Sources are a uniform 64-bit tile base plus a 32-bit per-lane offset; LDS destinations are
  // one per-lane offset plus compile-time strides.
  const int ld_row = tid >> 3;
  const int ld_kc = tid & 7;
  const f16* a_base = x + (int64_t)work.row_begin * k;
  const f16* b_base = w + ((int64_t)work.expert * n + (int64_t)work.n_tile * BN) * k;
  uint32_t a_off[kAChunks], b_off[kBChunks];
  const int n_left = n - work.n_tile * BN;  // rows of w available to this tile (>= 64)
#pragma unroll
  for (int i = 0; i < kAChunks; ++i) {
    int ar = ld_row + kRowsPerPass * i;
    if (ar > tile_rows - 1) ar = tile_rows - 1;  // rows past the group: duplicates, never stored
    a_off[i] = (uint32_t)ar * (uint32_t)k + ld_kc * 8;
  }
#pragma unroll
  for (int i = 0; i < kBChunks; ++i) {
    int br = ld_row + kRowsPerPass * i;
    if (br > n_left - 1) br = n_left - 1;  // n is a multiple of 64, not necessarily of BN
    b_off[i] = (uint32_t)br * (uint32_t)k + ld_kc * 8;
  }
  const int st_dst = lds_off(ld_row, ld_kc);

  f32x16 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  f16x8 ra[D][kAChunks], rb[D][kBChunks];  // D tiles in flight
  const int ktiles = k / kBK;

  auto load_tile = [&](int slot, int kt) {
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) ra[slot][i] = ld128(a_base + kt * kBK + a_off[i]);
#pragma unroll
    for (int i = 0; i < kBChunks; ++i) rb[slot][i] = ld128_stream(b_base + kt * kBK + b_off[i]);
  };
  auto store_tile = [&](int slot, int stage) {
    f16* da = sa + stage * BM * kBK;
    f16* db = sb + stage * BN * kBK;
#pragma unroll
    for (int i = 0; i < kAChunks; ++i)
      *reinterpret_cast<f16x8*>(&da[st_dst + i * kRowsPerPass * kBK]) = ra[slot][i];
#pragma unroll
    for (int i = 0; i < kBChunks; ++i)
      *reinterpret_cast<f16x8*>(&db[st_dst + i * kRowsPerPass * kBK]) = rb[slot][i];
  };

  const int fm = lane & 31;  // fragment row inside a 32-row block
  const int fq = lane >> 5;  // which half of a 16-wide k step
  // Fragment reads: block offsets are compile-time strides on top of one per-lane offset per k
  // step (the swizzle depends on fm and on the chunk only).
  int frag_off[kSteps];
#pragma unroll
  for (int st = 0; st < kSteps; ++st) frag_off[st] = lds_off(fm, st * 2 + fq);
  const f16* sa_w = sa + wm * 32 * kBK;
  const f16* sb_w = sb + wn * 32 * NB * kBK;

  // The k loop for LIVE live row blocks.  Iteration kt works on tile kt in LDS stage kt&1; the
  // register slot (kt+1)%D holds tile kt+1.  Per iteration, four k steps of 16:
  //   steps 0..2: MFMAs of the step | fragment reads of the next step (same stage) | a third of
  //               the staging: LDS writes of tile kt+1 into the other stage, each followed by
  //               the global load of tile kt+1+D into the register it just freed;
  //   barrier   : every wave has read all its fragments of tile kt and written its part of
  //               tile kt+1;
  //   step 3    : MFMAs of the step | fragment reads of step 0 of tile kt+1.
  // So the matrix cores never wait for an LDS round trip at a tile boundary, and there is one
  // barrier per k tile.  Past the end of the k loop the same code runs on the last tile again
  // (valid memory, results never consumed) instead of branching.
  auto k_loop = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    constexpr int kStageSteps = kSteps - 1;  // steps that carry staging traffic
    constexpr int kAPer = (kAChunks + kStageSteps - 1) / kStageSteps;
    constexpr int kBPer = (kBChunks + kStageSteps - 1) / kStageSteps;
    f16x8 fa[2][LIVE > 0 ? LIVE : 1], fb[2][NB];
    auto load_frags = [&](int buf, int st, int stage) {
      const f16* ca = sa_w + stage * BM * kBK;
      const f16* cb = sb_w + stage * BN * kBK;
#pragma unroll
      for (int j = 0; j < NB; ++j)
        fb[buf][j] = *reinterpret_cast<const f16x8*>(&cb[frag_off[st] + j * 32 * kBK]);
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
        fa[buf][i] = *reinterpret_cast<const f16x8*>(&ca[frag_off[st] + i * 64 * kBK]);
    };
    auto step = [&](int kload, auto slot_c, auto stage_c, auto st_c) {
      constexpr int SLOT = decltype(slot_c)::value;
      constexpr int STAGE = decltype(stage_c)::value;
      constexpr int ST = decltype(st_c)::value;
      constexpr int a_lo = ST * kAPer < kAChunks ? ST * kAPer : kAChunks;
      constexpr int a_hi = (ST + 1) * kAPer < kAChunks ? (ST + 1) * kAPer : kAChunks;
      constexpr int b_lo = ST * kBPer < kBChunks ? ST * kBPer : kBChunks;
      constexpr int b_hi = (ST + 1) * kBPer < kBChunks ? (ST + 1) * kBPer : kBChunks;
      constexpr int n_stage = ST < kStageSteps ? (a_hi - a_lo) + (b_hi - b_lo) : 0;
      if (ST + 1 < kSteps) {
        load_frags((ST + 1) & 1, ST + 1, STAGE);
        f16* da = sa + (STAGE ^ 1) * BM * kBK;
        f16* db = sb + (STAGE ^ 1) * BN * kBK;
#pragma unroll
        for (int i = a_lo; i < a_hi; ++i) {
          *reinterpret_cast<f16x8*>(&da[st_dst + i * kRowsPerPass * kBK]) = ra[SLOT][i];
          ra[SLOT][i] = ld128(a_base + kload + a_off[i]);
        }
#pragma unroll
        for (int i = b_lo; i < b_hi; ++i) {
          *reinterpret_cast<f16x8*>(&db[st_dst + i * kRowsPerPass * kBK]) = rb[SLOT][i];
          rb[SLOT][i] = ld128_stream(b_base + kload + b_off[i]);
        }
      } else {
        load_frags(0, 0, STAGE ^ 1);  // first fragments of the next tile
      }
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ST & 1][j], fa[ST & 1][i],
                                                             acc[i][j], 0, 0, 0);
      MfmaInterleave<0, LIVE * NB, LIVE + NB, n_stage, n_stage>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    auto iteration = [&](int kt, auto slot_c, auto stage_c) {
      const int kload = min(kt + 1 + D, ktiles - 1) * kBK;
      step(kload, slot_c, stage_c, std::integral_constant<int, 0>{});
      step(kload, slot_c, stage_c, std::integral_constant<int, 1>{});
      step(kload, slot_c, stage_c, std::integral_constant<int, 2>{});
      __syncthreads();
      step(kload, slot_c, stage_c, std::integral_constant<int, 3>{});
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using SlotEven = std::integral_constant<int, 1 % D>;  // slot of tile kt+1 for even kt
    using SlotOdd = std::integral_constant<int, 2 % D>;   // ... for odd kt
    __syncthreads();  // tile 0 is in stage 0
    load_frags(0, 0, 0);
    int kt = 0;
    for (; kt + 1 < ktiles; kt += 2) {
      iteration(kt, SlotEven{}, I0{});
      iteration(kt + 1, SlotOdd{}, I1{});
    }
    if (kt < ktiles) iteration(kt, SlotEven{}, I0{});
  };

  // tile t travels in register slot t % D and is consumed from LDS stage t & 1
  load_tile(0, 0);
  store_tile(0, 0);
#pragma unroll
  for (int t = 1; t <= D; ++t) load_tile(t % D, min(t, ktiles - 1));
  // One branch-free instantiation of the k loop per number of live row blocks.
  if (live >= MB) {
    k_loop(std::integral_constant<int, MB>{});
  } else if (MB > 1 && live == MB - 1) {
    k_loop(std::integral_constant<int, (MB > 1 ? MB - 1 : 0)>{});
  } else if (MB > 2 && live == MB - 2) {
    k_loop(std::integral_constant<int, (MB > 2 ? MB - 2 : 0)>{});
  } else if (live >= 1) {  // short groups: rarely worth a dedicated copy, use the next larger one
    if (MB > 3 && live <= MB - 3) k_loop(std::integral_constant<int, (MB > 3 ? MB - 3 : 0)>{});
  } else {
    k_loop(std::integral_constant<int, 0>{});
  }

  // Epilogue.  acc[i][j][r]: output row 32*(wm+2i) + lane%32, output columns
  // wn*32*NB + 32j + 8*(r/4) + 4*(lane/32) + r%4.  The C tile goes to LDS as [BM][BN] halfs in
  // 8-byte pieces, piece c of row m at position c ^ ((m & kSwz) << 1) (write conflicts at most
  // 2-way, 16-byte reads stay contiguous), and leaves as 128-bit row-contiguous global stores.
  __syncthreads();  // all waves are done with the operand stages
  f16* sc = smem;
  constexpr int kSwz = (BN / 8 < 16 ? BN / 8 : 16) - 1;  // swizzle stays inside the row
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int m = 32 * (wm + 2 * i) + fm;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f16x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (f16)acc[i][j][4 * g + e];
        const int piece = (wn * 32 * NB + 32 * j + 8 * g + 4 * fq) >> 2;
        *reinterpret_cast<f16x4*>(&sc[m * BN + ((piece ^ ((m & kSwz) << 1)) << 2)]) = v;
      }
    }
  }
  __syncthreads();
  constexpr int kChunksPerRow = BN / 8;              // 16-byte chunks per tile row
  constexpr int kRowsPerStorePass = kThreads / kChunksPerRow;
  const int c16 = tid % kChunksPerRow;
  const int col = work.n_tile * BN + c16 * 8;
  if (col < n) {
    for (int m = tid / kChunksPerRow; m < tile_rows; m += kRowsPerStorePass) {
      const f16x8 v = *reinterpret_cast<const f16x8*>(&sc[m * BN + ((c16 ^ (m & kSwz)) << 3)]);
      st128(y + (int64_t)(work.row_begin + m) * n + col, v);
    }
  }
}

#define AOPS_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define AOPS_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// s_waitcnt immediate for "at most N vector-memory operations outstanding, all LDS operations
// done" (vmcnt is split over bits 3:0 and 15:14, expcnt 6:4 left at its maximum, lgkmcnt 11:8).
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4); }

// Same tiling and MFMA work as grouped_matmul_kernel, but both operand tiles travel HBM -> LDS
// directly (global_load_lds_dwordx4: 64 lanes deposit 64 consecutive 16-byte chunks), so the k
// loop holds no staging registers and issues no LDS writes.  Because a lane cannot choose where
// its chunk lands, the swizzle is applied on the source side: the lane that owns physical chunk
// (row pr, position pc) fetches logical chunk (pr ^ ((pr>>3)&1), pc ^ (row & 7)).
// Two LDS stages.  Per tile kt (stage kt&1), four k steps of 16:
//   steps 0..2: MFMAs | fragment reads of the next step
//   then      : wait for this wave's copies of tile kt+1, barrier (tile kt+1 complete for
//               everyone, nobody reads stage kt&1 any more)
//   step 3    : MFMAs | fragment reads of step 0 of tile kt+1 | copies of tile kt+2 into stage kt&1
template <int MB, int NB, int WN>
__global__ __launch_bounds__(2 * WN * kWave) void grouped_matmul_dma_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n) {
  constexpr int kWaves = 2 * WN;  // 2 wave rows x WN wave columns
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kThreads = kWaves * kWave;
  constexpr int kSteps = kBK / 16;
  constexpr int kACopies = BM / 8 / kWaves;  // copy instructions per wave and tile (8 rows each)
  constexpr int kBCopies = BN / 8 / kWaves;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "tile rows per copy");

  extern __shared__ __attribute__((aligned(16))) f16 smem[];
  f16* sa = smem;                 // [2][BM * kBK]
  f16* sb = smem + 2 * BM * kBK;  // [2][BN * kBK]

  const int n_tiles = (n + BN - 1) / BN;
  const GmmWork work =
      gmm_find_work<BM>(group_list, num_experts, rows, n_tiles, blockIdx.x, gridDim.x);
  if (!work.valid) return;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int tile_rows = min(work.row_end - work.row_begin, BM);
  const int live_blocks = (tile_rows + 31) / 32;
  const int live = (live_blocks - wm + 1) / 2;

  // Copy sources.  Copy i of this wave fills physical rows (kWaves*i + wave)*8 .. +7 of a stage.
  const f16* a_base = x + (int64_t)work.row_begin * k;
  const f16* b_base = w + ((int64_t)work.expert * n + (int64_t)work.n_tile * BN) * k;
  const int n_left = n - work.n_tile * BN;                      // rows of w available (>= 64)
  const int64_t x_left = rows - work.row_begin;                 // rows of x available (>= 1)
  uint32_t a_off[kACopies], b_off[kBCopies];
  {
    const int pr_lo = lane >> 3;  // physical row inside the 8-row group
    const int pc = lane & 7;      // physical chunk position
#pragma unroll
    for (int i = 0; i < kACopies; ++i) {
      const int pr = (kWaves * i + wave) * 8 + pr_lo;
      int r = pr ^ ((pr >> 3) & 1);
      const int c = pc ^ (r & 7);
      // rows past the group read whatever follows in x (only dead output rows depend on them);
      // rows past the end of x are clamped
      if (r > x_left - 1) r = (int)(x_left - 1);
      a_off[i] = (uint32_t)r * (uint32_t)k + c * 8;
    }
#pragma unroll
    for (int i = 0; i < kBCopies; ++i) {
      const int pr = (kWaves * i + wave) * 8 + pr_lo;
      int r = pr ^ ((pr >> 3) & 1);
      const int c = pc ^ (r & 7);
      if (r > n_left - 1) r = n_left - 1;
      b_off[i] = (uint32_t)r * (uint32_t)k + c * 8;
    }
  }
  const int ktiles = k / kBK;
  auto copy_tile = [&](int kt, int stage) {
    const int ko = min(kt, ktiles - 1) * kBK;
    f16* da = sa + stage * BM * kBK + wave * 512;
    f16* db = sb + stage * BN * kBK + wave * 512;
#pragma unroll
    for (int i = 0; i < kACopies; ++i)
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(a_base + ko + a_off[i]),
                                       AOPS_LDS_PTR(da + i * kWaves * 512), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < kBCopies; ++i)
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(b_base + ko + b_off[i]),
                                       AOPS_LDS_PTR(db + i * kWaves * 512), 16, 0, 0);
  };

  f32x16 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int fm = lane & 31;
  const int fq = lane >> 5;
  int frag_off[kSteps];
#pragma unroll
  for (int st = 0; st < kSteps; ++st) frag_off[st] = lds_off(fm, st * 2 + fq);
  const f16* sa_w = sa + wm * 32 * kBK;
  const f16* sb_w = sb + wn * 32 * NB * kBK;

  auto k_loop = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    f16x8 fa[2][LIVE > 0 ? LIVE : 1], fb[2][NB];
    auto load_frags = [&](int buf, int st, int stage) {
      const f16* ca = sa_w + stage * BM * kBK;
      const f16* cb = sb_w + stage * BN * kBK;
#pragma unroll
      for (int j = 0; j < NB; ++j)
        fb[buf][j] = *reinterpret_cast<const f16x8*>(&cb[frag_off[st] + j * 32 * kBK]);
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
        fa[buf][i] = *reinterpret_cast<const f16x8*>(&ca[frag_off[st] + i * 64 * kBK]);
    };
    auto step = [&](int kt, auto stage_c, auto st_c) {
      constexpr int STAGE = decltype(stage_c)::value;
      constexpr int ST = decltype(st_c)::value;
      if (ST + 1 < kSteps) {
        load_frags((ST + 1) & 1, ST + 1, STAGE);
      } else {
        load_frags(0, 0, STAGE ^ 1);  // first fragments of the next tile
        copy_tile(kt + 2, STAGE);     // this stage is free: everyone is past the barrier
      }
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ST & 1][j], fa[ST & 1][i],
                                                             acc[i][j], 0, 0, 0);
      MfmaInterleave<0, LIVE * NB, LIVE + NB, 0,
                     (ST + 1 < kSteps) ? 0 : kACopies + kBCopies>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    auto iteration = [&](int kt, auto stage_c) {
      step(kt, stage_c, std::integral_constant<int, 0>{});
      step(kt, stage_c, std::integral_constant<int, 1>{});
      step(kt, stage_c, std::integral_constant<int, 2>{});
      // own copies of tile kt+1 and all own fragment reads of tile kt are complete ...
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // ... and so are everybody else's
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      step(kt, stage_c, std::integral_constant<int, 3>{});
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    // tile 0 must be complete, tile 1 may still be on its way
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kACopies + kBCopies));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frags(0, 0, 0);
    int kt = 0;
    for (; kt + 1 < ktiles; kt += 2) {
      iteration(kt, I0{});
      iteration(kt + 1, I1{});
    }
    if (kt < ktiles) iteration(kt, I0{});
  };

  copy_tile(0, 0);
  copy_tile(1, 1);
  if (live >= MB) {
    k_loop(std::integral_constant<int, MB>{});
  } else if (MB > 1 && live == MB - 1) {
    k_loop(std::integral_constant<int, (MB > 1 ? MB - 1 : 0)>{});
  } else if (MB > 2 && live == MB - 2) {
    k_loop(std::integral_constant<int, (MB > 2 ? MB - 2 : 0)>{});
  } else if (live >= 1) {
    if (MB > 3 && live <= MB - 3) k_loop(std::integral_constant<int, (MB > 3 ? MB - 3 : 0)>{});
  } else {
    k_loop(std::integral_constant<int, 0>{});
  }

  // Epilogue: as in grouped_matmul_kernel, one pass per pair of wave columns (BM x 64*NB halfs fit
  // the stages).  The last copies (a repeat of the last tile) must have landed before the stages
  // are reused for the output tile.
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  __syncthreads();
  f16* sc = smem;
  constexpr int kPassCols = 64 * NB;  // columns of two wave columns
  constexpr int kSwz = (kPassCols / 8 < 16 ? kPassCols / 8 : 16) - 1;
  constexpr int kChunksPerRow = kPassCols / 8;
  constexpr int kRowsPerStorePass = kThreads / kChunksPerRow;
#pragma unroll
  for (int pass = 0; pass < WN / 2; ++pass) {
    if (wn / 2 == pass) {
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int m = 32 * (wm + 2 * i) + fm;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (f16)acc[i][j][4 * g + e];
            const int piece = ((wn & 1) * 32 * NB + 32 * j + 8 * g + 4 * fq) >> 2;
            *reinterpret_cast<f16x4*>(&sc[m * kPassCols + ((piece ^ ((m & kSwz) << 1)) << 2)]) = v;
          }
        }
      }
    }
    __syncthreads();
    const int c16 = tid % kChunksPerRow;
    const int col = work.n_tile * BN + pass * kPassCols + c16 * 8;
    if (col < n) {
      for (int m = tid / kChunksPerRow; m < tile_rows; m += kRowsPerStorePass) {
        const f16x8 v =
            *reinterpret_cast<const f16x8*>(&sc[m * kPassCols + ((c16 ^ (m & kSwz)) << 3)]);
        st128(y + (int64_t)(work.row_begin + m) * n + col, v);
      }
    }
    if (pass + 1 < WN / 2) __syncthreads();
  }
}

// Per-lane summary of group_list for workgroups that look up many work items: lane l covers
// experts [l*per, (l+1)*per).
constexpr int kBndCache = 4;
struct GmmPlan {
  int per;          // experts per lane
  int tiles;        // m-tiles of this lane's experts
  int incl;         // inclusive prefix of tiles over the lanes
  int total_tiles;  // over all experts
  int bnd[kBndCache + 1];  // clamped row ends of experts l*per-1 .. l*per+kBndCache-1 (per <= kBndCache)
};

template <int kBM>
__device__ __forceinline__ GmmPlan gmm_make_plan(const int64_t* __restrict__ group_list,
                                                 int num_experts, int64_t rows) {
  const int lane = threadIdx.x & (kWave - 1);
  auto clampr = [&](int64_t v) -> int { return (int)(v < 0 ? 0 : (v > rows ? rows : v)); };
  GmmPlan p;
  p.per = (num_experts + kWave - 1) / kWave;
  const int e0 = lane * p.per;
  int prev = (e0 == 0 || e0 > num_experts) ? 0 : clampr(gmm_group_end(group_list, e0 - 1, rows));
  p.bnd[0] = prev;
  p.tiles = 0;
  if (p.per <= kBndCache) {
#pragma unroll
    for (int j = 0; j < kBndCache; ++j) {
      const int e = e0 + j;
      int end = prev;  // slots past the lane's experts: empty
      if (j < p.per && e < num_experts) {
        end = clampr(gmm_group_end(group_list, e, rows));
        if (end > prev) p.tiles += (end - prev + kBM - 1) / kBM;
      }
      p.bnd[j + 1] = end;
      prev = end;
    }
  } else {
#pragma unroll
    for (int j = 0; j < kBndCache; ++j) p.bnd[j + 1] = 0;
    for (int j = 0; j < p.per; ++j) {
      const int e = e0 + j;
      if (e < num_experts) {
        const int end = clampr(gmm_group_end(group_list, e, rows));
        if (end > prev) p.tiles += (end - prev + kBM - 1) / kBM;
        prev = end;
      }
    }
  }
  int incl = p.tiles;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  p.incl = incl;
  p.total_tiles = __shfl(incl, kWave - 1);
  return p;
}

// Work item `work` (0 <= work < total_tiles * n_tiles) -> (expert, m-tile, n-tile); the m-tiles
// that share a weight tile are adjacent.  With at most kBndCache experts per lane nothing is
// read from memory.
template <int kBM>
__device__ __forceinline__ GmmWork gmm_locate(const GmmPlan& p,
                                              const int64_t* __restrict__ group_list,
                                              int num_experts, int64_t rows, int n_tiles,
                                              int64_t work) {
  const int lane = threadIdx.x & (kWave - 1);
  auto clampr = [&](int64_t v) -> int { return (int)(v < 0 ? 0 : (v > rows ? rows : v)); };
  const int64_t lo = (int64_t)(p.incl - p.tiles) * n_tiles;
  const int64_t hi = (int64_t)p.incl * n_tiles;
  const bool mine = work >= lo && work < hi;
  int f_expert = 0, f_begin = 0, f_end = 0, f_ntile = 0;
  if (mine) {
    const int e0 = lane * p.per;
    int64_t base = lo;
    if (p.per <= kBndCache) {
      int prev = p.bnd[0];
      bool found = false;
#pragma unroll
      for (int j = 0; j < kBndCache; ++j) {
        const int end = p.bnd[j + 1];
        const int t = (j < p.per && end > prev) ? (end - prev + kBM - 1) / kBM : 0;
        const int64_t span = (int64_t)t * n_tiles;
        if (!found && t > 0 && work < base + span) {
          const int local = (int)(work - base);
          f_expert = e0 + j;
          f_ntile = local / t;
          f_begin = prev + (local - f_ntile * t) * kBM;
          f_end = end;
          found = true;
        }
        base += span;
        prev = end;
      }
    } else {
      int prev = (e0 == 0) ? 0 : clampr(gmm_group_end(group_list, e0 - 1, rows));
      for (int j = 0; j < p.per; ++j) {
        const int e = e0 + j;
        if (e >= num_experts) break;
        const int end = clampr(gmm_group_end(group_list, e, rows));
        const int t = end > prev ? (end - prev + kBM - 1) / kBM : 0;
        const int64_t span = (int64_t)t * n_tiles;
        if (work < base + span) {
          const int local = (int)(work - base);
          f_expert = e;
          f_ntile = local / t;
          f_begin = prev + (local - f_ntile * t) * kBM;
          f_end = end;
          break;
        }
        base += span;
        prev = end;
      }
    }
  }
  const uint64_t mask = __ballot(mine);
  GmmWork w;
  w.valid = mask != 0;
  const int src = w.valid ? __builtin_ctzll(mask) : 0;
  w.expert = __builtin_amdgcn_readfirstlane(__shfl(f_expert, src));
  w.row_begin = __builtin_amdgcn_readfirstlane(__shfl(f_begin, src));
  w.row_end = __builtin_amdgcn_readfirstlane(__shfl(f_end, src));
  w.n_tile = __builtin_amdgcn_readfirstlane(__shfl(f_ntile, src));
  return w;
}

// Persistent form of grouped_matmul_dma_kernel: one workgroup per CU walks through its share of
// the work items (XCD x owns a contiguous range of items, its workgroups take them round robin),
// and the operand pipeline never drains between items: the last two k tiles of an item issue the
// copies of the first two tiles of the next item, and the finished accumulators leave straight
// from registers (lane pairs exchange halves with v_permlane32_swap so that every lane stores 16
// contiguous bytes) while those copies are in flight, with no LDS use and no workgroup barrier.
// group_list is scanned once per workgroup; every wave keeps its copy of the scan in LDS.
// Requires k % 128 == 0 and k >= 256 (an even number of k tiles keeps the stage parity fixed).
//
// SWIGLU = true fuses the activation of a gate_up projection into the epilogue: with d = n/2 the
// kernel writes y[r, c] = silu(h[r, c]) * h[r, d + c] (h = x @ W_e^T in fp32, never stored) as a
// [rows, d] matrix.  A work item then covers 32*WN output columns; the weight stage holds, for wave
// column wn, the 32 gate rows of its columns in row block 2*wn and the matching 32 up rows in row
// block 2*wn + 1, so that a lane finds gate and up value of one output element in acc[i][0] and
// acc[i][1].
//
// GATHER = true reads the activation rows through an index: sorted row j comes from row
// row_idx[j] / idx_div of x (the routing order of a mixture of experts: row_idx = the sorted flat
// routing indices, idx_div = top-k), so the expert-sorted copy of x never exists.  The tile's
// source rows are looked up once per work item.
template <int MB, int NB, int WN, bool SWIGLU, bool GATHER>
__global__ __launch_bounds__(2 * WN * kWave) void grouped_matmul_persistent_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n,
    const int32_t* __restrict__ row_idx, int idx_div, uint32_t x_rows) {
  constexpr int kWaves = 2 * WN;
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kSteps = kBK / 16;
  constexpr int kACopies = BM / 8 / kWaves;
  constexpr int kBCopies = BN / 8 / kWaves;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "tile rows per copy");
  static_assert(!SWIGLU || (NB == 2 && kWaves == 8), "gate/up pairing assumes 64-row copies, two column blocks");
  constexpr int BNO = SWIGLU ? BN / 2 : BN;  // output columns per work item
  const int n_out = SWIGLU ? n / 2 : n;      // output row length

  extern __shared__ __attribute__((aligned(16))) f16 smem[];
  f16* sa = smem;                         // [2][BM * kBK]
  f16* sb = smem + 2 * BM * kBK;          // [2][BN * kBK]
  int* splan = reinterpret_cast<int*>(smem + 2 * (BM + BN) * kBK);  // [kWaves][kWave][8]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int n_tiles = (n_out + BNO - 1) / BNO;
  const int ktiles = k / kBK;

  int* my_plan = splan + (wave * kWave + lane) * 8;
  int plan_per, plan_total;
  {
    const GmmPlan plan = gmm_make_plan<BM>(group_list, num_experts, rows);
    plan_per = __builtin_amdgcn_readfirstlane(plan.per);
    plan_total = __builtin_amdgcn_readfirstlane(plan.total_tiles);
    my_plan[0] = plan.tiles;
    my_plan[1] = plan.incl;
#pragma unroll
    for (int j = 0; j <= kBndCache; ++j) my_plan[2 + j] = plan.bnd[j];
  }
  const int64_t total_work = (int64_t)plan_total * n_tiles;
  const int64_t share = (total_work + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int wg_in_xcd = blockIdx.x / kXcds;
  const int wgs_per_xcd = gridDim.x / kXcds;
  auto locate = [&](int64_t local) -> GmmWork {
    const int64_t item = (int64_t)xcd * share + local;
    if (local >= share || item >= total_work) {
      GmmWork none;
      none.valid = false;
      none.expert = none.row_begin = none.row_end = none.n_tile = 0;
      return none;
    }
    GmmPlan plan;  // this lane's part, written by this lane: no synchronisation needed
    plan.per = plan_per;
    plan.total_tiles = plan_total;
    plan.tiles = my_plan[0];
    plan.incl = my_plan[1];
#pragma unroll
    for (int j = 0; j <= kBndCache; ++j) plan.bnd[j] = my_plan[2 + j];
    return gmm_locate<BM>(plan, group_list, num_experts, rows, n_tiles, item);
  };

  int64_t local = wg_in_xcd;
  GmmWork cur = locate(local);
  if (!cur.valid) return;

  // Copy sources of the item whose tiles are being fetched.  Copy i of this wave fills physical
  // rows (kWaves*i + wave)*8 .. +7 of a stage, i.e. logical row 8*kWaves*i + lane_row (the row
  // swizzle only swaps rows inside the 8-row group) and chunk lane_c: one per-lane offset plus a
  // uniform stride per copy, clamped to the last valid row: tile rows past the end of the group
  // (only dead output rows depend on them) and past the end of w repeat the last valid row, which
  // costs one cache line per copy instead of eight.
  const f16* a_base;
  const f16* b_base;
  const int lane_row = wave * 8 + ((lane >> 3) ^ (wave & 1));
  const int lane_c = (lane & 7) ^ (lane_row & 7);
  const uint32_t off0 = (uint32_t)lane_row * (uint32_t)k + lane_c * 8;
  const uint32_t copy_stride = 8u * kWaves * (uint32_t)k;
  uint32_t a_last, b_last;  // offset of this lane's chunk in the last valid row
  uint32_t a_src[GATHER ? kACopies : 1];  // GATHER: offset of this lane's chunk per copy
  // SWIGLU: copy i of the weights fills row blocks 2i (gate rows 32i..32i+31 of the item) and
  // 2i+1 (the up rows d further down): per-lane offset + 32 rows per copy; b_last then holds the
  // number of valid 32-column blocks of the item instead of an offset.
  const uint32_t off0_glu = ((uint32_t)(lane_row & 31) + (lane_row >= 32 ? (uint32_t)n_out : 0u)) * (uint32_t)k + lane_c * 8;
  auto set_sources = [&](const GmmWork& it) {
    b_base = w + ((int64_t)it.expert * n + (int64_t)it.n_tile * BNO) * k;
    const int n_left = min(n_out - it.n_tile * BNO, BNO);
    const int x_left = min(it.row_end - it.row_begin, BM);  // rows of the group in this tile
    if constexpr (GATHER) {
      a_base = x;
#pragma unroll
      for (int i = 0; i < kACopies; ++i) {
        const int r = min(8 * kWaves * i + lane_row, x_left - 1);
        uint32_t src = (uint32_t)row_idx[it.row_begin + r] / (uint32_t)idx_div;
        src = src < x_rows ? src : x_rows - 1;  // an index outside x reads its last row instead of faulting
        a_src[i] = src * (uint32_t)k + lane_c * 8;
      }
    } else {
      a_base = x + (int64_t)it.row_begin * k;
    }
    a_last = (uint32_t)(x_left - 1) * (uint32_t)k + lane_c * 8;
    b_last = SWIGLU ? (uint32_t)(n_left / 32) : (uint32_t)(n_left - 1) * (uint32_t)k + lane_c * 8;
  };
  auto b_offset = [&](int i) -> uint32_t {
    if constexpr (SWIGLU) {
      const uint32_t blk = (uint32_t)i < b_last ? (uint32_t)i : 0u;  // blocks past n: repeat block 0
      return off0_glu + blk * 32u * (uint32_t)k;
    } else {
      return min(off0 + i * copy_stride, b_last);
    }
  };
  auto copy_tile = [&](int kt, int stage) {
    const int ko = kt * kBK;
    f16* da = sa + stage * BM * kBK + wave * 512;
    f16* db = sb + stage * BN * kBK + wave * 512;
    // the empty asm makes the 64-bit source address of a copy be formed right before the copy
    // instead of being kept in a register pair per copy across the k loop
#pragma unroll
    for (int i = 0; i < kACopies; ++i) {
      uint32_t o = GATHER ? a_src[i] : min(off0 + i * copy_stride, a_last);
      asm volatile("" : "+v"(o));
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(a_base + ko + o),
                                       AOPS_LDS_PTR(da + i * kWaves * 512), 16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < kBCopies; ++i) {
      uint32_t o = b_offset(i);
      asm volatile("" : "+v"(o));
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(b_base + ko + o),
                                       AOPS_LDS_PTR(db + i * kWaves * 512), 16, 0, 0);
    }
  };

  const int fm = lane & 31;
  const int fq = lane >> 5;
  // Fragment addresses: lds_off(fm, 2*st + fq) == lds_off(fm, fq) ^ (st << 4) (the k step only
  // flips two chunk bits), so one per-lane offset per operand serves every k step.
  const int fa_off0 = lds_off(fm, fq) + wm * 32 * kBK;
  const int fb_off0 = lds_off(fm, fq) + wn * 32 * NB * kBK;

  f32x16 acc[MB][NB];
  GmmWork nxt;

  auto k_loop = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    f16x8 fa[2][LIVE > 0 ? LIVE : 1], fb[2][NB];
    auto load_frags = [&](int buf, int st, int stage) {
      // the empty asm keeps the compiler from hoisting one address register per (stage, step)
      // out of the k loop, which would push the accumulators into scratch
      int fo_a = fa_off0, fo_b = fb_off0;
      asm volatile("" : "+v"(fo_a), "+v"(fo_b));
      const f16* ca = sa + stage * BM * kBK + (fo_a ^ (st << 4));
      const f16* cb = sb + stage * BN * kBK + (fo_b ^ (st << 4));
#pragma unroll
      for (int j = 0; j < NB; ++j)
        fb[buf][j] = *reinterpret_cast<const f16x8*>(&cb[j * 32 * kBK]);
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
        fa[buf][i] = *reinterpret_cast<const f16x8*>(&ca[i * 64 * kBK]);
    };
    auto step = [&](int kcopy, auto stage_c, auto st_c) {
      constexpr int STAGE = decltype(stage_c)::value;
      constexpr int ST = decltype(st_c)::value;
      if (ST + 1 < kSteps) {
        load_frags((ST + 1) & 1, ST + 1, STAGE);
      } else {
        load_frags(0, 0, STAGE ^ 1);  // first fragments of the next tile
        copy_tile(kcopy, STAGE);      // this stage is free: everyone is past the barrier
      }
#pragma unroll
      for (int i = 0; i < LIVE; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ST & 1][j], fa[ST & 1][i],
                                                             acc[i][j], 0, 0, 0);
      MfmaInterleave<0, LIVE * NB, LIVE + NB, 0,
                     (ST + 1 < kSteps) ? 0 : kACopies + kBCopies>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    auto iteration = [&](int kcopy, auto stage_c) {
      step(kcopy, stage_c, std::integral_constant<int, 0>{});
      step(kcopy, stage_c, std::integral_constant<int, 1>{});
      step(kcopy, stage_c, std::integral_constant<int, 2>{});
      // own copies of the next tile and all own fragment reads of this tile are complete ...
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // ... and so are everybody else's
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      step(kcopy, stage_c, std::integral_constant<int, 3>{});
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    load_frags(0, 0, 0);
    for (int kt = 0; kt < ktiles; kt += 2) {
      int c0 = kt + 2, c1 = kt + 3;
      if (kt + 2 >= ktiles) {  // the last two tiles fetch the head of the next item
        if (nxt.valid) {
          set_sources(nxt);
          c0 = 0;
          c1 = 1;
        } else {  // nothing follows: repeat the last tile (valid memory, never consumed)
          c0 = c1 = ktiles - 1;
        }
      }
      iteration(c0, I0{});
      iteration(c1, I1{});
    }
  };

  set_sources(cur);
  copy_tile(0, 0);
  copy_tile(1, 1);
  // tile 0 must be complete, tile 1 may still be on its way
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kACopies + kBCopies));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  for (;;) {
    local += wgs_per_xcd;
    nxt = locate(local);
    const int tile_rows = min(cur.row_end - cur.row_begin, BM);
    const int live_blocks = (tile_rows + 31) / 32;
    const int live = (live_blocks - wm + 1) / 2;
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    if (live >= MB) {
      k_loop(std::integral_constant<int, MB>{});
    } else if (MB > 1 && live == MB - 1) {
      k_loop(std::integral_constant<int, (MB > 1 ? MB - 1 : 0)>{});
    } else if (MB > 2 && live == MB - 2) {
      k_loop(std::integral_constant<int, (MB > 2 ? MB - 2 : 0)>{});
    } else if (live >= 1) {
      k_loop(std::integral_constant<int, (MB > 3 ? MB - 3 : 1)>{});
    } else {
      k_loop(std::integral_constant<int, 0>{});
    }

    // Epilogue of `cur`.  acc[i][j][4g+e]: output row 32*(wm+2i) + fm, output column
    // wn*32*NB + 32j + 8g + 4fq + e.  For a pair of column groups (g, g+1) the two lanes of a row
    // (fq = 0, 1) exchange halves: v_permlane32_swap trades the upper 32 lanes of its first
    // operand for the lower 32 lanes of its second, after which lane fq holds the 8 consecutive
    // columns of group g+fq.
    const int m_w = 32 * wm + fm;
    if constexpr (SWIGLU) {
      const int col_w = cur.n_tile * BNO + wn * 32;
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int m = m_w + 64 * i;
        if (i < live && col_w < n_out) {  // wave uniform
          const bool row_ok = m < tile_rows;
          f16* yrow = y + (int64_t)(cur.row_begin + m) * n_out + col_w + 8 * fq;
#pragma unroll
          for (int gp = 0; gp < 2; ++gp) {
            f16x4 p0, p1;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float g = acc[i][0][8 * gp + e];
              const float u = acc[i][1][8 * gp + e];
              const float ex = __builtin_amdgcn_exp2f(-1.4426950408889634f * g);
              const f16 o = (f16)(g * u * __builtin_amdgcn_rcpf(1.0f + ex));
              if (e < 4) p0[e] = o; else p1[e - 4] = o;
            }
            const u32x2 d0 = __builtin_bit_cast(u32x2, p0);
            const u32x2 d1 = __builtin_bit_cast(u32x2, p1);
            const auto lo = __builtin_amdgcn_permlane32_swap(d0[0], d1[0], false, false);
            const auto hi = __builtin_amdgcn_permlane32_swap(d0[1], d1[1], false, false);
            u32x4 out;
            out[0] = lo[0];
            out[1] = hi[0];
            out[2] = lo[1];
            out[3] = hi[1];
            if (row_ok) st128(yrow + 16 * gp, __builtin_bit_cast(f16x8, out));
          }
        }
      }
    } else {
    const int col_w = cur.n_tile * BN + wn * 32 * NB;
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int m = m_w + 64 * i;
      if (i < live) {  // wave uniform: both lanes of every pair take part in the exchange
        const bool row_ok = m < tile_rows;
        f16* yrow = y + (int64_t)(cur.row_begin + m) * n + col_w + 8 * fq;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          if (col_w + 32 * j < n) {
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
              f16x4 p0, p1;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                p0[e] = (f16)acc[i][j][8 * gp + e];
                p1[e] = (f16)acc[i][j][8 * gp + 4 + e];
              }
              const u32x2 d0 = __builtin_bit_cast(u32x2, p0);
              const u32x2 d1 = __builtin_bit_cast(u32x2, p1);
              const auto lo = __builtin_amdgcn_permlane32_swap(d0[0], d1[0], false, false);
              const auto hi = __builtin_amdgcn_permlane32_swap(d0[1], d1[1], false, false);
              u32x4 out;
              out[0] = lo[0];
              out[1] = hi[0];
              out[2] = lo[1];
              out[3] = hi[1];
              if (row_ok) st128(yrow + 32 * j + 16 * gp, __builtin_bit_cast(f16x8, out));
            }
          }
        }
      }
    }
    }
    if (!nxt.valid) break;
    cur = nxt;
  }
  // the repeated last-tile copies must have landed before the LDS is released
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
}

template <int MB, int NB, int WN, bool SWIGLU, bool GATHER = false>
static int gmm_persistent_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y,
                                 int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                                 const int32_t* row_idx = nullptr, int idx_div = 1, int64_t x_rows = 1) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kWaves = 2 * WN;
  constexpr int kLds = 2 * (BM + BN) * kBK * (int)sizeof(f16) + kWaves * kWave * 8 * (int)sizeof(int);
  static_assert(kLds <= 160 * 1024, "LDS budget");
  static int cus[64] = {0};  // per device; benign race: every writer stores the same value
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return record_launch_status(e);
  if (dev < 0 || dev >= 64) return AOPS_ERR_INVALID_ARGUMENT;
  if (cus[dev] == 0) {
    int v = 0;
    e = hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return record_launch_status(e);
    cus[dev] = v > 0 ? v : 8;
  }
  constexpr int BNO = SWIGLU ? BN / 2 : BN;
  const int64_t n_out = SWIGLU ? n / 2 : n;
  const int64_t n_tiles = (n_out + BNO - 1) / BNO;
  const int64_t max_work = ((rows + BM - 1) / BM + num_experts) * n_tiles;
  int64_t grid = cus[dev] < max_work ? cus[dev] : max_work;
  grid = grid / kXcds * kXcds;
  if (grid < kXcds) grid = kXcds;
  auto kernel = grouped_matmul_persistent_kernel<MB, NB, WN, SWIGLU, GATHER>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return record_launch_status(e);
    attr_set = true;
  }
  kernel<<<(unsigned)grid, 2 * WN * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts,
                                                          n, row_idx, idx_div, (uint32_t)x_rows);
  return record_launch_status(hipGetLastError());
}

template <int MB, int NB, int WN>
static int gmm_dma_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y,
                          int64_t rows, int k, int num_experts, int n, hipStream_t stream) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kStageBytes = 2 * (BM + BN) * kBK * (int)sizeof(f16);
  constexpr int kTileBytes = BM * 64 * NB * (int)sizeof(f16);
  constexpr int kLds = kStageBytes > kTileBytes ? kStageBytes : kTileBytes;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const int64_t n_tiles = (n + BN - 1) / BN;
  const int64_t max_m_tiles = (rows + BM - 1) / BM + num_experts;
  int64_t grid = max_m_tiles * n_tiles;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  auto kernel = grouped_matmul_dma_kernel<MB, NB, WN>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return record_launch_status(e);
    attr_set = true;
  }
  kernel<<<(unsigned)grid, 2 * WN * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts,
                                                          n);
  return record_launch_status(hipGetLastError());
}

template <int MB, int NB, int D>
static int gmm_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y, int64_t rows,
                      int k, int num_experts, int n, hipStream_t stream) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 64 * NB;
  constexpr int kStageBytes = 2 * (BM + BN) * kBK * (int)sizeof(f16);
  constexpr int kTileBytes = BM * BN * (int)sizeof(f16);
  constexpr int kLds = kStageBytes > kTileBytes ? kStageBytes : kTileBytes;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const int64_t n_tiles = (n + BN - 1) / BN;
  const int64_t max_m_tiles = (rows + BM - 1) / BM + num_experts;
  int64_t grid = max_m_tiles * n_tiles;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  auto kernel = grouped_matmul_kernel<MB, NB, D>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return record_launch_status(e);
    attr_set = true;
  }
  kernel<<<(unsigned)grid, 4 * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts, n);
  return record_launch_status(hipGetLastError());
}

}  // namespace aops

static int aops_grouped_matmul_impl(const void* x, const void* w, const int64_t* group_list, void* y,
                                    int64_t rows, int64_t k, int64_t num_experts, int64_t n,
                                    void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 64 != 0 || n % 64 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  // per-lane tile offsets are 32-bit: 320 rows x k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !y || (!group_list && num_experts != 1)) return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const f16* xp = static_cast<const f16*>(x);
  const f16* wp = static_cast<const f16*>(w);
  f16* yp = static_cast<f16*>(y);
  const char* forced_env = getenv("AOPS_GMM_VARIANT");  // tuning aid: 1..8 force one kernel / tile shape
  const int forced = forced_env ? atoi(forced_env) : 0;
  // Tile choice from what the host knows (group_list stays on the device): the largest tile
  // whose grid still gives every CU work.  320 rows cover a typical expert of a large routed
  // batch in one tile; small or dense problems (few rows, one expert) take smaller tiles so that
  // enough workgroups exist to pull the weights through all memory channels.
  int variant = forced;
  if (variant < 1 || variant > 8) {
    auto tiles = [&](int64_t bm, int64_t bn) { return ((rows + bm - 1) / bm) * ((n + bn - 1) / bn); };
    constexpr int64_t kEnough = 384;
    constexpr int64_t kMostCus = 192;  // 256-row tiles read a small batch's weights once: worth a few idle CUs
    variant = tiles(320, 256) >= kEnough ? 6 : tiles(320, 128) >= kEnough ? 2 : tiles(256, 128) >= kMostCus ? 3
              : tiles(128, 128) >= kEnough ? 4 : 5;
  }
  if (variant == 6 && (k % 128 != 0 || k < 256)) variant = 1;  // the persistent kernel's k loop
  switch (variant) {
    case 6:  // 320 x 256 tiles, eight waves, one persistent workgroup per CU
      return gmm_persistent_launch<5, 2, 4, false>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts,
                                            (int)n, s);
    case 7:  // 256 x 128 tiles, four waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<4, 2, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
    case 8:  // 128 x 128 tiles, four waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<2, 2, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
    case 1:  // 320 x 256 tiles, eight waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<5, 2, 4>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n,
                                     s);
    case 2:  // 320 x 128 tiles
      return gmm_launch<5, 2, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
    case 3:  // 256 x 128 tiles
      return gmm_launch<4, 2, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
    case 4:  // 128 x 128 tiles
      return gmm_launch<2, 2, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
    default:  // 64 x 64 tiles
      return gmm_launch<1, 1, 2>(xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
  }
}

extern "C" int aops_grouped_matmul_f16(const void* x, const void* w, const int64_t* group_list,
                                       void* y, int64_t rows, int64_t k, int64_t num_experts,
                                       int64_t n, void* stream) {
  if (rows > 0 && num_experts > 0 && !group_list) return AOPS_ERR_INVALID_ARGUMENT;
  return aops_grouped_matmul_impl(x, w, group_list, y, rows, k, num_experts, n, stream);
}

extern "C" int aops_grouped_matmul_swiglu_f16(const void* x, const void* w, const int64_t* group_list,
                                              void* y, int64_t rows, int64_t k, int64_t num_experts,
                                              int64_t n, void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 128 != 0 || k < 256 || n % 64 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  // 32-bit per-lane offsets: (n/2 + 32) weight rows of k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20) ||
      (n / 2 + 320) * k > 0x7fffffffLL)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !group_list || !y) return AOPS_ERR_INVALID_ARGUMENT;
  return gmm_persistent_launch<5, 2, 4, true>(
      static_cast<const f16*>(x), static_cast<const f16*>(w), group_list, static_cast<f16*>(y), rows,
      (int)k, (int)num_experts, (int)n, static_cast<hipStream_t>(stream));
}

extern "C" int aops_matmul_nt_f16(const void* x, const void* w, void* y, int64_t m, int64_t k, int64_t n,
                                  void* stream) {
  if (m < 0 || k <= 0 || n <= 0 || k % 64 != 0 || n % 64 != 0) return AOPS_ERR_INVALID_ARGUMENT;
  if (m == 0) return AOPS_OK;
  if (!x || !w || !y) return AOPS_ERR_INVALID_ARGUMENT;
  return aops_grouped_matmul_impl(x, w, nullptr, y, m, k, 1, n, stream);
}

extern "C" int aops_grouped_matmul_swiglu_gather_f16(const void* x, const int32_t* row_idx,
                                                     int64_t idx_div, int64_t x_rows, const void* w,
                                                     const int64_t* group_list, void* y, int64_t rows,
                                                     int64_t k, int64_t num_experts, int64_t n,
                                                     void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 128 != 0 || k < 256 || n % 64 != 0 ||
      idx_div <= 0 || idx_div > 0x7fffffff || x_rows < 0 || (rows > 0 && x_rows == 0))
    return AOPS_ERR_INVALID_ARGUMENT;
  // 32-bit per-lane offsets: x_rows activation rows and (n/2 + 32) weight rows of k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20) ||
      (n / 2 + 320) * k > 0x7fffffffLL || x_rows * k > 0xffffffffLL)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !row_idx || !w || !group_list || !y) return AOPS_ERR_INVALID_ARGUMENT;
  return gmm_persistent_launch<5, 2, 4, true, true>(
      static_cast<const f16*>(x), static_cast<const f16*>(w), group_list, static_cast<f16*>(y), rows,
      (int)k, (int)num_experts, (int)n, static_cast<hipStream_t>(stream), row_idx, (int)idx_div, x_rows);
}
