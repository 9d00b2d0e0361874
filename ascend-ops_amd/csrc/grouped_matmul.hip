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
#include "aops_common.h"

namespace aops {

constexpr int kBM = 128;
constexpr int kBN = 128;
constexpr int kBK = 64;
constexpr int kGmmThreads = 256;
constexpr int kXcds = 8;

struct GmmWork {
  int expert;
  int row_begin;  // first row of this m-tile
  int row_end;    // end of the expert's rows
  int n_tile;
  bool valid;
};

// Maps a work index to (expert, m-tile, n-tile).  Executed redundantly by every wave.
__device__ __forceinline__ GmmWork gmm_find_work(const int64_t* __restrict__ group_list,
                                                 int num_experts, int64_t rows, int n_tiles,
                                                 int wg, int num_wg) {
  const int lane = threadIdx.x & (kWave - 1);
  const int per = (num_experts + kWave - 1) / kWave;
  const int e0 = lane * per;
  auto clampr = [&](int64_t v) -> int { return (int)(v < 0 ? 0 : (v > rows ? rows : v)); };
  int tiles = 0;
  {
    int prev = (e0 == 0 || e0 > num_experts) ? 0 : clampr(group_list[e0 - 1]);
    for (int j = 0; j < per; ++j) {
      const int e = e0 + j;
      if (e < num_experts) {
        const int end = clampr(group_list[e]);
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
    int prev = (e0 == 0) ? 0 : clampr(group_list[e0 - 1]);
    for (int j = 0; j < per; ++j) {
      const int e = e0 + j;
      if (e >= num_experts) break;
      const int end = clampr(group_list[e]);
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

// LDS tile [rows][kBK] halfs; 16-byte chunk c of row r is stored at chunk (c ^ (r & 7)) so that
// the 128-bit fragment reads of 8 consecutive rows hit all banks.
__device__ __forceinline__ int lds_off(int r, int c) { return r * kBK + ((c ^ (r & 7)) << 3); }

__global__ __launch_bounds__(kGmmThreads) void grouped_matmul_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n) {
  __shared__ __attribute__((aligned(16))) f16 sa[kBM * kBK];
  __shared__ __attribute__((aligned(16))) f16 sb[kBN * kBK];

  const int n_tiles = (n + kBN - 1) / kBN;
  const GmmWork work = gmm_find_work(group_list, num_experts, rows, n_tiles, blockIdx.x, gridDim.x);
  if (!work.valid) return;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave >> 1;  // 2 x 2 waves, 64 x 64 each
  const int wn = wave & 1;

  // Global -> register staging: thread handles chunk (row = tid/8 + 32*i, kc = tid%8).
  const int ld_row = tid >> 3;
  const int ld_kc = tid & 7;
  const f16* a_src[4];
  const f16* b_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int ar = work.row_begin + ld_row + 32 * i;
    if (ar > work.row_end - 1) ar = work.row_end - 1;  // rows past the group: duplicate, never stored
    a_src[i] = x + (int64_t)ar * k + ld_kc * 8;
    int br = work.n_tile * kBN + ld_row + 32 * i;
    if (br > n - 1) br = n - 1;  // n is a multiple of 64, not necessarily of the tile width
    b_src[i] = w + ((int64_t)work.expert * n + br) * k + ld_kc * 8;
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  f16x8 ra[4], rb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ra[i] = ld128(a_src[i]);
    rb[i] = ld128(b_src[i]);
  }

  const int fm = lane & 31;  // fragment row inside a 32-row block
  const int fq = lane >> 5;  // which half of a 16-wide k step
  const int ktiles = k / kBK;
  for (int kt = 0; kt < ktiles; ++kt) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<f16x8*>(&sa[lds_off(ld_row + 32 * i, ld_kc)]) = ra[i];
      *reinterpret_cast<f16x8*>(&sb[lds_off(ld_row + 32 * i, ld_kc)]) = rb[i];
    }
    __syncthreads();
    if (kt + 1 < ktiles) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ra[i] = ld128(a_src[i] + (kt + 1) * kBK);
        rb[i] = ld128(b_src[i] + (kt + 1) * kBK);
      }
    }
#pragma unroll
    for (int s = 0; s < kBK / 16; ++s) {
      f16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *reinterpret_cast<const f16x8*>(&sa[lds_off(wm * 64 + i * 32 + fm, s * 2 + fq)]);
        fb[i] = *reinterpret_cast<const f16x8*>(&sb[lds_off(wn * 64 + i * 32 + fm, s * 2 + fq)]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }

  // C fragment: lane holds column (lane%32) and rows 8*(r/4) + 4*(lane/32) + r%4, r = 0..15.
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = work.row_begin + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * fq + (r & 3);
      if (row < work.row_end) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int col = work.n_tile * kBN + wn * 64 + j * 32 + fm;
          if (col < n) y[(int64_t)row * n + col] = (f16)acc[i][j][r];
        }
      }
    }
  }
}

}  // namespace aops

extern "C" int aops_grouped_matmul_f16(const void* x, const void* w, const int64_t* group_list,
                                       void* y, int64_t rows, int64_t k, int64_t num_experts,
                                       int64_t n, void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 64 != 0 || n % 64 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows > 0x7fffffff - kBM || k > 0x7fffffff || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !group_list || !y) return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t n_tiles = (n + kBN - 1) / kBN;
  const int64_t max_m_tiles = (rows + kBM - 1) / kBM + num_experts;
  int64_t grid = max_m_tiles * n_tiles;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  grouped_matmul_kernel<<<(unsigned)grid, kGmmThreads, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(x), static_cast<const f16*>(w), group_list, static_cast<f16*>(y),
      rows, (int)k, (int)num_experts, (int)n);
  return record_launch_status(hipGetLastError());
}
