// Grouped matmul, one workgroup per work item: the register-staged kernel (four waves) and the
// kernel that copies its operand tiles HBM -> LDS directly.
#include "gmm_common.h"

namespace aops {

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
//
// SWIGLU = true fuses the activation of a gate_up projection: with d = n/2 the kernel writes
// y[r, c] = silu(h[r, c]) * h[r, d + c] (h = x @ W_e^T) as a [rows, d] matrix.  A work item then
// covers BN/2 output columns: the first half of its weight tile holds their gate rows, the second
// half the up rows d further down, and the two meet in the LDS staging of the epilogue (after the
// rounding to fp16, as in the two-kernel chain).  GATHER = true reads activation row j of the sorted
// batch from row row_idx[j] / idx_div of x (see grouped_matmul_persistent_kernel).
template <int MB, int NB, int D, bool SWIGLU = false, bool GATHER = false>
__global__ __launch_bounds__(4 * kWave) void grouped_matmul_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n,
    const int32_t* __restrict__ row_idx, int idx_div, uint32_t x_rows) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 64 * NB;
  constexpr int BNO = SWIGLU ? BN / 2 : BN;  // output columns per work item
  const int n_out = SWIGLU ? n / 2 : n;      // output row length
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

  const int n_tiles = (n_out + BNO - 1) / BNO;
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
  const f16* a_base = GATHER ? x : x + (int64_t)work.row_begin * k;
  const f16* b_base = w + ((int64_t)work.expert * n + (int64_t)work.n_tile * BNO) * k;
  uint32_t a_off[kAChunks], b_off[kBChunks];
  const int n_left = n_out - work.n_tile * BNO;  // output columns available to this tile (>= 32)
#pragma unroll
  for (int i = 0; i < kAChunks; ++i) {
    int ar = ld_row + kRowsPerPass * i;
    if (ar > tile_rows - 1) ar = tile_rows - 1;  // rows past the group: duplicates, never stored
    if constexpr (GATHER) {
      uint32_t src = (uint32_t)row_idx[work.row_begin + ar] / (uint32_t)idx_div;
      src = src < x_rows ? src : x_rows - 1;  // an index outside x reads its last row instead of faulting
      a_off[i] = src * (uint32_t)k + ld_kc * 8;
    } else {
      a_off[i] = (uint32_t)ar * (uint32_t)k + ld_kc * 8;
    }
  }
#pragma unroll
  for (int i = 0; i < kBChunks; ++i) {
    int br = ld_row + kRowsPerPass * i;
    if constexpr (SWIGLU) {
      // tile rows [0, BN/2): gate rows of the item's columns; [BN/2, BN): the up rows n_out further down
      const bool up = br >= BN / 2;
      int c = up ? br - BN / 2 : br;
      if (c > n_left - 1) c = n_left - 1;
      b_off[i] = (uint32_t)(c + (up ? n_out : 0)) * (uint32_t)k + ld_kc * 8;
    } else {
      if (br > n_left - 1) br = n_left - 1;  // n is a multiple of 64, not necessarily of BN
      b_off[i] = (uint32_t)br * (uint32_t)k + ld_kc * 8;
    }
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
  if constexpr (SWIGLU) {
    constexpr int kChunksPerRow = BNO / 8;  // 16-byte chunks per output row of the tile
    constexpr int kRowsPerStorePass = kThreads / kChunksPerRow;
    const int c16 = tid % kChunksPerRow;
    const int col = work.n_tile * BNO + c16 * 8;
    if (col < n_out) {
      for (int m = tid / kChunksPerRow; m < tile_rows; m += kRowsPerStorePass) {
        const f16x8 gv = *reinterpret_cast<const f16x8*>(&sc[m * BN + ((c16 ^ (m & kSwz)) << 3)]);
        const f16x8 uv =
            *reinterpret_cast<const f16x8*>(&sc[m * BN + (((c16 + kChunksPerRow) ^ (m & kSwz)) << 3)]);
        f16x8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float gf = (float)gv[e];
          const float ex = __builtin_amdgcn_exp2f(-1.4426950408889634f * gf);
          v[e] = (f16)(gf * (float)uv[e] * __builtin_amdgcn_rcpf(1.0f + ex));
        }
        st128(y + (int64_t)(work.row_begin + m) * n_out + col, v);
      }
    }
    return;
  }
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

// Writes a workgroup's accumulators (acc[i][j][4g+e] of wave (wm, wn): row 32*(wm+2i) + lane%32,
// column wn*32*NB + 32j + 8g + 4*(lane/32) + e of the tile) as fp16 through LDS, one pass per pair
// of wave columns, so that y is written in 16-byte pieces along its rows.  All waves of the
// workgroup call it after a barrier; `smem` must hold BM x 64*NB halfs.
template <int MB, int NB, int WN>
__device__ __forceinline__ void gmm_store_tile(const f32x16 (&acc)[MB][NB], f16* smem, f16* __restrict__ y,
                                               int row_begin, int tile_rows, int n_tile, int n) {
  constexpr int kWaves = 2 * WN;
  constexpr int BN = 32 * NB * WN;
  constexpr int kThreads = kWaves * kWave;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int fm = lane & 31;
  const int fq = lane >> 5;
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
    const int col = n_tile * BN + pass * kPassCols + c16 * 8;
    if (col < n) {
      for (int m = tid / kChunksPerRow; m < tile_rows; m += kRowsPerStorePass) {
        const f16x8 v =
            *reinterpret_cast<const f16x8*>(&sc[m * kPassCols + ((c16 ^ (m & kSwz)) << 3)]);
        st128(y + (int64_t)(row_begin + m) * n + col, v);
      }
    }
    if (pass + 1 < WN / 2) __syncthreads();
  }
}

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
//
// SPLITK = true is the dense form for few rows and a long k (one group, group_list unused): workgroup
// blockIdx.x computes output tile blockIdx.x / splits over the k tiles of split blockIdx.x % splits
// (workgroup i runs on XCD i % 8, so with 8 splits every XCD reads one k range of x and keeps it in
// its L2) and leaves its fp32 accumulators in `partial` in register order: for (split, tile, wave)
// a block of MB*NB*4 rows of 64 float4, row (i*NB + j)*4 + g holding acc[i][j][4g..4g+3] of every
// lane, so that each store instruction writes 1 KiB of consecutive bytes.  matmul_splitk_reduce
// adds the splits in index order and writes y.
// It runs with three LDS stages instead of two: its workgroups stream weights that nobody else reads,
// and two tiles in flight per CU rather than one is what keeps enough bytes on their way from HBM.
template <int MB, int NB, int WN, bool SPLITK = false, int NS = (SPLITK ? 3 : 2)>
__global__ __launch_bounds__(2 * WN * kWave) void grouped_matmul_dma_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n, float* __restrict__ partial,
    int splits) {
  constexpr int kWaves = 2 * WN;  // 2 wave rows x WN wave columns
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kThreads = kWaves * kWave;
  constexpr int kSteps = kBK / 16;
  constexpr int kACopies = BM / 8 / kWaves;  // copy instructions per wave and tile (8 rows each)
  constexpr int kBCopies = BN / 8 / kWaves;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "tile rows per copy");

  static_assert(NS == 2 || NS == 3, "LDS stages");
  extern __shared__ __attribute__((aligned(16))) f16 smem[];
  f16* sa = smem;                  // [NS][BM * kBK]
  f16* sb = smem + NS * BM * kBK;  // [NS][BN * kBK]

  const int n_tiles = (n + BN - 1) / BN;
  GmmWork work;
  int k_begin = 0;         // first k element of this workgroup's share
  int ktiles = k / kBK;    // k tiles of this workgroup's share
  int64_t partial_block = 0;  // SPLITK: index of this workgroup's block of partial results
  if constexpr (SPLITK) {
    const int m_tiles = (int)((rows + BM - 1) / BM);
    const int tile = blockIdx.x / splits;
    const int split = blockIdx.x - tile * splits;
    if (tile >= m_tiles * n_tiles) return;
    partial_block = (int64_t)split * (m_tiles * n_tiles) + tile;
    work.valid = true;
    work.expert = 0;
    work.n_tile = tile / m_tiles;  // the m tiles of one weight tile are adjacent
    work.row_begin = (tile - work.n_tile * m_tiles) * BM;
    work.row_end = (int)rows;
    const int per = (ktiles + splits - 1) / splits;  // the host chooses splits so that none is empty
    k_begin = split * per * kBK;
    ktiles = min(per, ktiles - split * per);
  } else {
    work = gmm_find_work<BM>(group_list, num_experts, rows, n_tiles, blockIdx.x, gridDim.x);
    if (!work.valid) return;
  }

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int tile_rows = min(work.row_end - work.row_begin, BM);
  const int live_blocks = (tile_rows + 31) / 32;
  const int live = (live_blocks - wm + 1) / 2;

  // Copy sources.  Copy i of this wave fills physical rows (kWaves*i + wave)*8 .. +7 of a stage,
  // i.e. logical row 8*kWaves*i + lane_row (the row swizzle only swaps rows inside the 8-row group)
  // and chunk lane_c: one per-lane offset plus a uniform stride per copy, clamped to the last valid
  // row (tile rows past the end of the group - only dead output rows depend on them - and past
  // the end of w repeat the last valid row).
  const f16* a_base = x + (int64_t)work.row_begin * k + k_begin;
  const f16* b_base = w + ((int64_t)work.expert * n + (int64_t)work.n_tile * BN) * k + k_begin;
  const int n_left = min(n - work.n_tile * BN, BN);
  const int lane_row = wave * 8 + ((lane >> 3) ^ (wave & 1));
  const int lane_c = (lane & 7) ^ (lane_row & 7);
  const uint32_t off0 = (uint32_t)lane_row * (uint32_t)k + lane_c * 8;
  const uint32_t copy_stride = 8u * kWaves * (uint32_t)k;
  const uint32_t a_last = (uint32_t)(tile_rows - 1) * (uint32_t)k + lane_c * 8;
  const uint32_t b_last = (uint32_t)(n_left - 1) * (uint32_t)k + lane_c * 8;
  auto copy_tile = [&](int kt, int stage) {
    const int ko = min(kt, ktiles - 1) * kBK;
    f16* da = sa + stage * BM * kBK + wave * 512;
    f16* db = sb + stage * BN * kBK + wave * 512;
    // the empty asm makes the 64-bit source address of a copy be formed right before the copy
    // instead of being kept in a register pair per copy across the k loop
#pragma unroll
    for (int i = 0; i < kACopies; ++i) {
      uint32_t o = min(off0 + i * copy_stride, a_last);
      asm volatile("" : "+v"(o));
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(a_base + ko + o),
                                       AOPS_LDS_PTR(da + i * kWaves * 512), 16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < kBCopies; ++i) {
      uint32_t o = min(off0 + i * copy_stride, b_last);
      asm volatile("" : "+v"(o));
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(b_base + ko + o),
                                       AOPS_LDS_PTR(db + i * kWaves * 512), 16, 0, 0);
    }
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
  // Fragment addresses: lds_off(fm, 2*st + fq) == lds_off(fm, fq) ^ (st << 4) (the k step only
  // flips two chunk bits), so one per-lane offset per operand serves every k step.
  const int fa_off0 = lds_off(fm, fq) + wm * 32 * kBK;
  const int fb_off0 = lds_off(fm, fq) + wn * 32 * NB * kBK;

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
    auto step = [&](int kt, auto stage_c, auto st_c) {
      constexpr int STAGE = decltype(stage_c)::value;
      constexpr int ST = decltype(st_c)::value;
      if (ST + 1 < kSteps) {
        load_frags((ST + 1) & 1, ST + 1, STAGE);
      } else {
        load_frags(0, 0, (STAGE + 1) % NS);  // first fragments of the next tile
        copy_tile(kt + NS, STAGE);           // this stage is free: everyone is past the barrier
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
      // own copies of tile kt+1 (later tiles may still be on their way) and all own fragment
      // reads of tile kt are complete ...
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0((NS - 2) * (kACopies + kBCopies)));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // ... and so are everybody else's
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      step(kt, stage_c, std::integral_constant<int, 3>{});
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    // tile 0 must be complete, the later ones may still be on their way
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0((NS - 1) * (kACopies + kBCopies)));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frags(0, 0, 0);
    int kt = 0;
    if constexpr (NS == 3) {
      for (; kt + 2 < ktiles; kt += 3) {
        iteration(kt, I0{});
        iteration(kt + 1, I1{});
        iteration(kt + 2, I2{});
      }
      if (kt < ktiles) iteration(kt, I0{});
      if (kt + 1 < ktiles) iteration(kt + 1, I1{});
    } else {
      for (; kt + 1 < ktiles; kt += 2) {
        iteration(kt, I0{});
        iteration(kt + 1, I1{});
      }
      if (kt < ktiles) iteration(kt, I0{});
    }
  };

  static_assert((NS - 1) * (kACopies + kBCopies) < 64, "vmcnt range");
  copy_tile(0, 0);
  copy_tile(1, 1);
  if constexpr (NS == 3) copy_tile(2, 2);
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
  // are reused for the output tile (or released).
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  if constexpr (SPLITK) {
    f32x4* dst = reinterpret_cast<f32x4*>(partial) + (partial_block * kWaves + wave) * (MB * NB * 4 * kWave) + lane;
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      if (i < live) {  // the reduction skips the same blocks
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * g + e];
            dst[((i * NB + j) * 4 + g) * kWave] = v;
          }
      }
    }
    return;
  }
  __syncthreads();
  gmm_store_tile<MB, NB, WN>(acc, smem, y, work.row_begin, tile_rows, work.n_tile, n);
}

template <int MB, int NB, int WN, int NS = 2>
static int gmm_dma_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y,
                          int64_t rows, int k, int num_experts, int n, hipStream_t stream) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kStageBytes = NS * (BM + BN) * kBK * (int)sizeof(f16);
  constexpr int kTileBytes = BM * 64 * NB * (int)sizeof(f16);
  constexpr int kLds = kStageBytes > kTileBytes ? kStageBytes : kTileBytes;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const int64_t n_tiles = (n + BN - 1) / BN;
  const int64_t max_m_tiles = (rows + BM - 1) / BM + num_experts;
  int64_t grid = max_m_tiles * n_tiles;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  auto kernel = grouped_matmul_dma_kernel<MB, NB, WN, false, NS>;
  static std::atomic<uint64_t> lds_allowed{0};  // per device
  if (const hipError_t le = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, lds_allowed); le != hipSuccess)
    return record_launch_status(le);
  kernel<<<(unsigned)grid, 2 * WN * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts,
                                                          n, nullptr, 1);
  return record_launch_status(hipGetLastError());
}

// Second kernel of the split-k dense matmul: one wave per (output tile, wave of the first kernel,
// 64-row block i) adds that block's partial results over the splits, in index order (the result
// does not depend on which split finished first), and writes it as fp16 straight from registers:
// lane pairs exchange halves with v_permlane32_swap so that every lane stores 16 contiguous bytes.
// No LDS, no barrier; the loads of all splits are independent.
template <int MB, int NB, int WN>
__global__ __launch_bounds__(4 * kWave) void matmul_splitk_reduce(
    const float* __restrict__ partial, f16* __restrict__ y, int64_t rows, int n, int splits,
    const int64_t* __restrict__ group_list) {
  constexpr int kWaves = 2 * WN;
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  const int n_tiles = (n + BN - 1) / BN;
  const int m_tiles = (int)((rows + BM - 1) / BM);
  const int tiles = m_tiles * n_tiles;
  const int unit = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // (tile, wave, i)
  if (unit >= tiles * kWaves * MB) return;
  const int i = unit % MB;
  const int wave = (unit / MB) % kWaves;
  const int tile = unit / (MB * kWaves);
  const int n_tile = tile / m_tiles;
  const int row_begin = (tile - n_tile * m_tiles) * BM;
  const int tile_rows = min((int)rows - row_begin, BM);
  const int lane = threadIdx.x & (kWave - 1);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int live = ((tile_rows + 31) / 32 - wm + 1) / 2;
  if (i >= live) return;  // the first kernel wrote nothing for this block
  const int fm = lane & 31;
  const int fq = lane >> 5;
  f32x4 acc[NB][4];
#pragma unroll
  for (int j = 0; j < NB; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) acc[j][g] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int64_t split_stride = (int64_t)tiles * kWaves * (MB * NB * 4 * kWave);  // float4 units
  const f32x4* src = reinterpret_cast<const f32x4*>(partial) +
                     ((int64_t)tile * kWaves + wave) * (MB * NB * 4 * kWave) + (i * NB * 4) * kWave + lane;
  for (int s = 0; s < splits; ++s) {
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 v = __builtin_nontemporal_load(&src[(j * 4 + g) * kWave]);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[j][g][e] += v[e];
      }
    src += split_stride;
  }
  // acc[j][g][e]: row 32*(wm + 2i) + fm, column wn*32*NB + 32j + 8g + 4fq + e of the tile
  const int m = 32 * (wm + 2 * i) + fm;
  const int col_w = n_tile * BN + wn * 32 * NB;
  // a single group that ends before the last row: the rows behind it are not written
  const int64_t row_limit = group_list ? min(max(group_list[0], (int64_t)0), rows) : rows;
  const bool row_ok = m < tile_rows && row_begin + m < row_limit;
  f16* yrow = y + (int64_t)(row_begin + m) * n + col_w + 8 * fq;
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    if (col_w + 32 * j < n) {  // wave uniform: both lanes of every pair take part in the exchange
#pragma unroll
      for (int gp = 0; gp < 2; ++gp) {
        f16x4 p0, p1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          p0[e] = (f16)acc[j][2 * gp][e];
          p1[e] = (f16)acc[j][2 * gp + 1][e];
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

// Number of k splits worth taking for a dense [m, k] x [n, k]^T product on a device with `cus`
// CUs: as many as it takes to give every CU a workgroup when the output has too few tiles for
// that, each split keeping at least eight k tiles; 1 = do not split.
template <int MB, int NB, int WN>
static int matmul_splitk_splits(int64_t m, int64_t k, int64_t n, int cus) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  const int64_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
  const int64_t ktiles = k / kBK;
  if (tiles * 2 > cus || ktiles < 16) return 1;
  int64_t splits = cus / tiles;
  if (splits > ktiles / 8) splits = ktiles / 8;
  if (splits > 16) splits = 16;
  if (splits < 2) return 1;
  const int64_t per = (ktiles + splits - 1) / splits;
  return (int)((ktiles + per - 1) / per);  // no empty split
}

// Tiles of the split-k path: 128 columns on four waves, and as many rows as the product has, rounded
// up to 64, 128 or 256: the fp32 partial results are written and read back tile by tile, so a tile
// taller than m is wasted traffic (at m <= 64 three quarters of it with 256-row tiles).
constexpr int kSplitNB = 2, kSplitWN = 2;
static int splitk_row_blocks(int64_t m) { return m <= 64 ? 1 : m <= 128 ? 2 : 4; }

template <int MB>
static size_t splitk_workspace(int64_t m, int64_t k, int64_t n, int cus) {
  const int splits = matmul_splitk_splits<MB, kSplitNB, kSplitWN>(m, k, n, cus);
  if (splits < 2) return 0;
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * kSplitNB * kSplitWN;
  const int64_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
  return (size_t)splits * (size_t)tiles * BM * BN * sizeof(float);
}

size_t gmm_splitk_workspace(int64_t m, int64_t k, int64_t n) {
  const int cus = device_cu_count();
  switch (splitk_row_blocks(m)) {
    case 1: return splitk_workspace<1>(m, k, n, cus);
    case 2: return splitk_workspace<2>(m, k, n, cus);
    default: return splitk_workspace<4>(m, k, n, cus);
  }
}

template <int MB>
static int launch_splitk(const f16* x, const f16* w, const int64_t* group_list, f16* y, float* workspace,
                         size_t workspace_bytes, int64_t m, int k, int n, hipStream_t stream) {
  constexpr int NB = kSplitNB, WN = kSplitWN;
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  const int splits = matmul_splitk_splits<MB, NB, WN>(m, k, n, device_cu_count());
  const int64_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
  if (splits < 2) return AOPS_ERR_INVALID_ARGUMENT;
  if (!workspace || workspace_bytes < (size_t)splits * (size_t)tiles * BM * BN * sizeof(float))
    return AOPS_ERR_WORKSPACE;
  constexpr int kStageBytes = 3 * (BM + BN) * kBK * (int)sizeof(f16);
  static_assert(kStageBytes <= 160 * 1024, "LDS budget");
  auto kernel = grouped_matmul_dma_kernel<MB, NB, WN, true>;
  auto reduce = matmul_splitk_reduce<MB, NB, WN>;
  static std::atomic<uint64_t> lds_allowed{0};  // per device
  if (const hipError_t le = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kStageBytes, lds_allowed); le != hipSuccess)
    return record_launch_status(le);
  kernel<<<(unsigned)(tiles * splits), 2 * WN * kWave, kStageBytes, stream>>>(x, w, nullptr, y, m, k, 1, n,
                                                                            workspace, splits);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return record_launch_status(e);
  const int64_t units = tiles * (2 * WN) * MB;  // one wave each
  reduce<<<(unsigned)((units + 3) / 4), 4 * kWave, 0, stream>>>(workspace, y, m, n, splits, group_list);
  return record_launch_status(hipGetLastError());
}

int gmm_launch_splitk(const f16* x, const f16* w, const int64_t* group_list, f16* y, float* workspace,
                      size_t workspace_bytes, int64_t m, int k, int n, hipStream_t stream) {
  switch (splitk_row_blocks(m)) {
    case 1: return launch_splitk<1>(x, w, group_list, y, workspace, workspace_bytes, m, k, n, stream);
    case 2: return launch_splitk<2>(x, w, group_list, y, workspace, workspace_bytes, m, k, n, stream);
    default: return launch_splitk<4>(x, w, group_list, y, workspace, workspace_bytes, m, k, n, stream);
  }
}

template <int MB, int NB, int D, bool SWIGLU = false, bool GATHER = false>
static int gmm_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y, int64_t rows,
                      int k, int num_experts, int n, hipStream_t stream,
                      const int32_t* row_idx = nullptr, int idx_div = 1, int64_t x_rows = 1) {
  constexpr int BM = 64 * MB;
  constexpr int BN = 64 * NB;
  constexpr int kStageBytes = 2 * (BM + BN) * kBK * (int)sizeof(f16);
  constexpr int kTileBytes = BM * BN * (int)sizeof(f16);
  constexpr int kLds = kStageBytes > kTileBytes ? kStageBytes : kTileBytes;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  constexpr int BNO = SWIGLU ? BN / 2 : BN;
  const int64_t n_out = SWIGLU ? n / 2 : n;
  const int64_t n_tiles = (n_out + BNO - 1) / BNO;
  const int64_t max_m_tiles = (rows + BM - 1) / BM + num_experts;
  int64_t grid = max_m_tiles * n_tiles;
  grid = (grid + kXcds - 1) / kXcds * kXcds;
  if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  auto kernel = grouped_matmul_kernel<MB, NB, D, SWIGLU, GATHER>;
  static std::atomic<uint64_t> lds_allowed{0};  // per device
  if (const hipError_t le = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, lds_allowed); le != hipSuccess)
    return record_launch_status(le);
  kernel<<<(unsigned)grid, 4 * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts, n, row_idx,
                                                       idx_div, (uint32_t)x_rows);
  return record_launch_status(hipGetLastError());
}

int gmm_launch_tiles(int variant, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                     int64_t rows, int k, int num_experts, int n, hipStream_t stream) {
  switch (variant) {
    case 1:  // 320 x 256 tiles, eight waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<5, 2, 4>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 7:  // 256 x 128 tiles, four waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<4, 2, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 8:  // 128 x 128 tiles, four waves, operands copied HBM -> LDS directly
      return gmm_dma_launch<2, 2, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 9:  // 256 x 128 tiles, four waves, three LDS stages
      return gmm_dma_launch<4, 2, 2, 3>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 2:  // 320 x 128 tiles
      return gmm_launch<5, 2, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 3:  // 256 x 128 tiles
      return gmm_launch<4, 2, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
    case 4:  // 128 x 128 tiles
      return gmm_launch<2, 2, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
    default:  // 64 x 64 tiles
      return gmm_launch<1, 1, 2>(x, w, group_list, y, rows, k, num_experts, n, stream);
  }
}

// The fused gate_up + SwiGLU (+ row gather) on the small tiles, for batches with few rows per expert:
// 128 x 128 tiles (64 output columns per item) or 64 x 64 (32 output columns).
int gmm_launch_tiles_fused(bool small, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                           int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                           const int32_t* row_idx, int idx_div, int64_t x_rows) {
  if (row_idx) {
    if (small)
      return gmm_launch<1, 1, 2, true, true>(x, w, group_list, y, rows, k, num_experts, n, stream, row_idx,
                                             idx_div, x_rows);
    return gmm_launch<2, 2, 2, true, true>(x, w, group_list, y, rows, k, num_experts, n, stream, row_idx,
                                           idx_div, x_rows);
  }
  if (small) return gmm_launch<1, 1, 2, true>(x, w, group_list, y, rows, k, num_experts, n, stream);
  return gmm_launch<2, 2, 2, true>(x, w, group_list, y, rows, k, num_experts, n, stream);
}

}  // namespace aops
