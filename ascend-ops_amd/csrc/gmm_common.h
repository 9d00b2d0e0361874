// Pieces shared by the grouped-matmul kernels: the device-side lookup of a workgroup's work item
// from group_list, the instruction-interleaving directive of the k loop, the LDS swizzle, and the
// launch functions the entry points choose from.
//
// Semantics: reference csrc/opdev/op_kernel/grouped_mat_mul_ex.cpp:27-44 (start/end from the
// cumulative int64 group_list, empty groups skipped), matmul_core.h:42-68 (NT product, fp32
// accumulate, fp16 result), benchmark/test_grouped_matmul.py:6-23.
#pragma once

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

// Order of the work items of one expert with t m-tiles and n_tiles n-tiles: bands of kBandM m-tiles;
// inside a band the m-tiles of one weight tile are adjacent and the weight tiles follow one another.
// The 32 workgroups that run side by side on an XCD then cover a 2-d block of the output (kBandM
// m-tiles x 32 / kBandM weight tiles) instead of one column of it and find most of both operands in
// that XCD's L2.  With t <= kBandM (routed batches) this is the plain "m-tiles of a weight tile
// adjacent" order.
constexpr int kBandM = 8;
__device__ __forceinline__ void gmm_item_to_tile(int local, int t, int n_tiles, int& m_tile, int& n_tile) {
  const int per_band = kBandM * n_tiles;
  const int band = local / per_band;
  const int r = local - band * per_band;
  const int m_in_band = min(kBandM, t - band * kBandM);
  n_tile = r / m_in_band;
  m_tile = band * kBandM + (r - n_tile * m_in_band);
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
        int m_tile;
        gmm_item_to_tile(local, t, n_tiles, m_tile, f_ntile);
        f_begin = prev + m_tile * kBM;
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

#define AOPS_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define AOPS_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// s_waitcnt immediate for "at most N vector-memory operations outstanding, all LDS operations
// done" (vmcnt is split over bits 3:0 and 15:14, expcnt 6:4 left at its maximum, lgkmcnt 11:8).
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4); }

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
// Index: int64_t, or int where the launcher has checked that the number of work items fits (the
// persistent kernel: 32-bit uniform values stay in scalar registers); `lane`: the caller's lane id.
template <int kBM, typename Index>
__device__ __forceinline__ GmmWork gmm_locate(const GmmPlan& p,
                                              const int64_t* __restrict__ group_list,
                                              int num_experts, int64_t rows, int n_tiles,
                                              Index work, int lane) {
  auto clampr = [&](int64_t v) -> int { return (int)(v < 0 ? 0 : (v > rows ? rows : v)); };
  const Index lo = (Index)(p.incl - p.tiles) * n_tiles;
  const Index hi = (Index)p.incl * n_tiles;
  const bool mine = work >= lo && work < hi;
  int f_expert = 0, f_begin = 0, f_end = 0, f_ntile = 0;
  if (mine) {
    const int e0 = lane * p.per;
    Index base = lo;
    if (p.per <= kBndCache) {
      int prev = p.bnd[0];
      bool found = false;
#pragma unroll
      for (int j = 0; j < kBndCache; ++j) {
        const int end = p.bnd[j + 1];
        const int t = (j < p.per && end > prev) ? (end - prev + kBM - 1) / kBM : 0;
        const Index span = (Index)t * n_tiles;
        if (!found && t > 0 && work < base + span) {
          const int local = (int)(work - base);
          f_expert = e0 + j;
          int m_tile;
          gmm_item_to_tile(local, t, n_tiles, m_tile, f_ntile);
          f_begin = prev + m_tile * kBM;
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
        const Index span = (Index)t * n_tiles;
        if (work < base + span) {
          const int local = (int)(work - base);
          f_expert = e;
          int m_tile;
          gmm_item_to_tile(local, t, n_tiles, m_tile, f_ntile);
          f_begin = prev + m_tile * kBM;
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

// Launch functions (one translation unit per kernel family).
// Tile kernels, one workgroup per work item: variant 1 = 320x256 direct copies (eight waves),
// 2 = 320x128, 3 = 256x128, 4 = 128x128, 5 = 64x64 (register staged, four waves),
// 7 = 256x128, 8 = 128x128 direct copies (four waves).
int gmm_launch_tiles(int variant, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                     int64_t rows, int k, int num_experts, int n, hipStream_t stream);
// Persistent 320x256 kernel; swiglu fuses the activation into the epilogue (y: [rows, n/2]),
// row_idx != nullptr reads the rows of x through row_idx[j] / idx_div (x has x_rows rows); ldw = elements
// from one weight row to the next (0 or k: densely packed).
int gmm_launch_persistent(bool swiglu, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                          int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                          const int32_t* row_idx, int idx_div, int64_t x_rows, int ldw = 0);
int gmm_launch_persistent_probe(int parts_off, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                                int64_t rows, int k, int num_experts, int n, hipStream_t stream, int ldw);

// Fused gate_up + SwiGLU (row_idx != nullptr: + row gather) on 128 x 128 tiles, or 64 x 64 with
// `small`; k a multiple of 64.
int gmm_launch_tiles_fused(bool small, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                           int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                           const int32_t* row_idx, int idx_div, int64_t x_rows);

// Dense [m, k] x [n, k]^T with the k range split over several workgroups per output tile and a
// second kernel adding the partial results: for few rows and a long k, where whole-k tiles would
// leave most CUs without work.  gmm_splitk_workspace returns the bytes of fp32 scratch the call
// needs on the current device, 0 when splitting does not pay for the shape.
size_t gmm_splitk_workspace(int64_t m, int64_t k, int64_t n);
// Dense products with at most 16 rows of x (matmul_fewrows.hip): one launch, no workspace.
bool matmul_fewrows_takes(int64_t m, int64_t k, int64_t n);
int matmul_fewrows_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y, int64_t m, int k,
                          int n, hipStream_t stream);
// group_list != nullptr: the single group ends at group_list[0]; rows behind it are not written.
int gmm_launch_splitk(const f16* x, const f16* w, const int64_t* group_list, f16* y, float* workspace,
                      size_t workspace_bytes, int64_t m, int k, int n, hipStream_t stream);

}  // namespace aops
