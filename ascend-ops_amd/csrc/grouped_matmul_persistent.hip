// Grouped matmul, persistent kernel for large problems (optionally with the SwiGLU activation in
// the epilogue and the row gather of a routed batch in the operand copies).
#include "gmm_common.h"

namespace aops {

// Persistent form of grouped_matmul_dma_kernel: one workgroup per CU walks through its share of
// the work items (XCD x owns a contiguous range of items, its workgroups take them round robin),
// and the operand pipeline never drains between items: the last tiles of an item issue the copies
// of the first tiles of the next item (its weights two tiles ahead, its activation rows one), and
// the finished accumulators leave through a small LDS scratch of the wave's own while those copies
// are in flight, with no workgroup barrier.  The two operands have separate two-stage rings: the
// weight stage of a tile is free as soon as every wave holds its fragments in registers (barrier B
// of the k loop), the activation stage when the tile's last fragment has been read (barrier A).
// group_list is scanned once per workgroup; the scan is kept in LDS.
// Requires k % 128 == 0 and k >= 256 (an even number of k tiles keeps the stage parity fixed).
//
// SWIGLU = true fuses the activation of a gate_up projection into the epilogue: with d = n/2 the
// kernel writes y[r, c] = silu(h[r, c]) * h[r, d + c] (h = x @ W_e^T in fp32, never stored) as a
// [rows, d] matrix.  A work item then covers 32*WN output columns; the weight stage holds, for wave
// column wn, the 32 gate rows of its columns in row block 2*wn and the matching 32 up rows in row
// block 2*wn + 1, so that a lane finds gate and up value of one output element in acc[b][j] and
// acc[b][j + 2] (16-column blocks j = 0, 1 of the gate rows, 2, 3 of the up rows).
//
// GATHER = true reads the activation rows through an index: sorted row j comes from row
// row_idx[j] / idx_div of x (the routing order of a mixture of experts: row_idx = the sorted flat
// routing indices, idx_div = top-k), so the expert-sorted copy of x never exists.  The tile's
// source rows are looked up once per work item.
// Lane id taken from the hardware each time, through a volatile asm the compiler neither hoists nor
// merges.  The persistent kernel derives its per-item offsets from it instead of from values computed at
// kernel start: those would have to live across the k loop, where the accumulators fill the register
// file, and so be spilled - and reloading a spilled register means waiting for every outstanding memory
// operation, the next item's operand copies and this item's stores included.
__device__ __forceinline__ int lane_id_fresh() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

// Operand copy HBM/L2 -> LDS, 16 bytes per lane: lane l's bytes land at LDS byte address lds_addr + 16*l.
// Written as inline asm rather than through the compiler's builtin: the compiler's wait-count pass treats
// the builtin as an access to both memory and LDS and, while one is outstanding, turns every wait for an
// LDS read into a wait for all of them - and this kernel always has copies outstanding.  The kernel waits
// for its copies itself (counted s_waitcnt vmcnt before the barriers); the asm is invisible to that pass,
// which errs on the safe side for the loads and stores it does see (invisible operations only make a
// counted wait stricter, never looser, since vector memory operations complete in order).
// M0 carries the LDS address of a copy; the compiler reserves that register and warns when it appears in a
// clobber list, but nothing else in this kernel uses it.
// Two things therefore hold only as long as the compiler's output keeps them, and tests/test_gmm_waits.py
// checks both in the assembly of every instantiation at build time (no GPU needed): (1) M0 is written and
// read by these copy sequences alone, and no register is spilled; (2) between two barriers of the k loop lie
// exactly the copies the source issues there, and each barrier is directly preceded by its counted wait.
// Per-lane byte offset of a copy: lane_base + uniform_add, clamped to cap.  Volatile asm, so that the nine
// offsets of a tile's copies are computed where the copies are issued (two instructions each) instead of
// being kept in registers across the k loop, where the accumulators fill the register file.
__device__ __forceinline__ uint32_t copy_offset(uint32_t lane_base, uint32_t uniform_add, uint32_t cap) {
  uint32_t r;
  asm volatile("v_add_u32 %0, %1, %2\n\tv_min_u32 %0, %0, %3" : "=&v"(r) : "s"(uniform_add), "v"(lane_base), "v"(cap));
  return r;
}
__device__ __forceinline__ uint32_t copy_offset(uint32_t lane_base, uint32_t uniform_add) {
  uint32_t r;
  asm volatile("v_add_u32 %0, %1, %2" : "=v"(r) : "s"(uniform_add), "v"(lane_base));
  return r;
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16(const void* base, uint32_t lane_offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_addr), "v"(lane_offset), "s"(base) : "m0", "memory");
}
#pragma clang diagnostic pop

constexpr int kPlanInts = 2 + kBndCache + 1;  // per-lane record of the group_list scan kept in LDS
constexpr int kEpiScratchHalfs = 512;         // 1 KiB of LDS per wave for the epilogue's row transposition

// PROBE (measurement aid, results wrong by construction): parts of the k loop switched off, so that what
// the rest costs by itself can be timed: bit 0 = no MFMAs, bit 1 = no activation copies, bit 2 = no weight
// copies, bit 3 = no LDS fragment reads (the MFMAs then run on registers that never change), bit 4 = the weight
// copies of a k tile fetch 256 bytes of every row of one half of the tile's rows (even tiles the first half, odd
// tiles the second, both at the even tile's k offset) instead of 128 bytes of every row: the same requests per
// tile and the same bytes per pair of tiles, in pieces twice as long; where they land in LDS is meaningless, so
// only together with bits 0 and 3.  0 = the kernel.
constexpr int kProbeNoMfma = 1, kProbeNoXCopies = 2, kProbeNoWCopies = 4, kProbeNoFragments = 8, kProbeWidePieces = 16;

template <int MB, int NB, int WN, bool SWIGLU, bool GATHER, int PROBE = 0>
__global__ __launch_bounds__(2 * WN * kWave) void grouped_matmul_persistent_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int64_t rows, int k, int num_experts, int n,
    const int32_t* __restrict__ row_idx, uint32_t idx_magic, int idx_shift, uint32_t x_rows, int ldw) {
  constexpr int kWaves = 2 * WN;
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kKSteps = kBK / 32;  // k steps of a tile: one v_mfma_f32_16x16x32_f16 deep each
  constexpr int kACopies = BM / 8 / kWaves;
  constexpr int kBCopies = BN / 8 / kWaves;
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "tile rows per copy");
  static_assert(kKSteps == 2, "the k loop keeps the weight fragments of two k steps");
  static_assert(!SWIGLU || (NB == 2 && kWaves == 8), "gate/up pairing assumes 64-row copies, two column blocks");
  constexpr int BNO = SWIGLU ? BN / 2 : BN;  // output columns per work item
  const int n_out = SWIGLU ? n / 2 : n;      // output row length

  extern __shared__ __attribute__((aligned(16))) f16 smem[];
  f16* sa = smem;                         // [2][BM * kBK]
  f16* sb = smem + 2 * BM * kBK;          // [2][BN * kBK]
  int* splan = reinterpret_cast<int*>(smem + 2 * (BM + BN) * kBK);  // [kWave][kPlanInts], the same in every wave
  f16* sepi = reinterpret_cast<f16*>(splan + kWave * kPlanInts);     // [kWaves][kEpiScratchHalfs]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN;
  const int wn = wave % WN;
  const int n_tiles = (n_out + BNO - 1) / BNO;
  const int ktiles = k / kBK;

  // every wave computes the same scan and stores it to the same place: a wave reads back values that it
  // (or another wave, identically) wrote, so no synchronisation is needed
  int* my_plan = splan + lane * kPlanInts;
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
  // 32-bit on purpose (the launcher refuses problems with 2^31 work items or more): uniform 32-bit values
  // stay in scalar registers, 64-bit ones ended up in vector registers and were spilled
  const int total_work = __builtin_amdgcn_readfirstlane(plan_total * n_tiles);
  const int share = (total_work + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int wg_in_xcd = blockIdx.x / kXcds;
  const int wgs_per_xcd = gridDim.x / kXcds;
  auto locate = [&](int local) -> GmmWork {
    const int item = xcd * share + local;
    if (local >= share || item >= total_work) {
      GmmWork none;
      none.valid = false;
      none.expert = none.row_begin = none.row_end = none.n_tile = 0;
      return none;
    }
    GmmPlan plan;  // this lane's part, written by this lane (and identically by its twins in the other waves)
    const int lane_l = lane_id_fresh();
    const int* my_plan = splan + lane_l * kPlanInts;
    plan.per = plan_per;
    plan.total_tiles = plan_total;
    plan.tiles = my_plan[0];
    plan.incl = my_plan[1];
#pragma unroll
    for (int j = 0; j <= kBndCache; ++j) plan.bnd[j] = my_plan[2 + j];
    return gmm_locate<BM, int>(plan, group_list, num_experts, rows, n_tiles, item, lane_l);
  };

  int local = wg_in_xcd;
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
  // per-lane offsets of the copies, in bytes (320 rows of at most 2^22 elements: below 2^32)
  const uint32_t off0 = ((uint32_t)lane_row * (uint32_t)k + lane_c * 8) * 2u;
  const uint32_t copy_stride = 8u * kWaves * (uint32_t)k * 2u;
  // the weight rows are ldw >= k elements apart (rows padded by the caller; ldw == k: densely packed)
  const uint32_t off0_w = ((uint32_t)lane_row * (uint32_t)ldw + lane_c * 8) * 2u;
  const uint32_t copy_stride_w = 8u * kWaves * (uint32_t)ldw * 2u;
  uint32_t a_last, b_last;  // offset of this lane's chunk in the last valid row
  uint32_t b_rows = 1;      // valid weight rows of the item (used by the wide-piece measurement build only)
  uint32_t a_src[GATHER ? kACopies : 1];  // GATHER: offset of this lane's chunk per copy
  // SWIGLU: copy i of the weights fills row blocks 2i (gate rows 32i..32i+31 of the item) and
  // 2i+1 (the up rows d further down): per-lane offset + 32 rows per copy; b_last then holds the
  // number of valid 32-column blocks of the item instead of an offset.
  const uint32_t off0_glu = (((uint32_t)(lane_row & 31) + (lane_row >= 32 ? (uint32_t)n_out : 0u)) * (uint32_t)ldw + lane_c * 8) * 2u;
  auto set_w_sources = [&](const GmmWork& it) {
    const int lane_s = lane_id_fresh();
    const int lane_row = wave * 8 + ((lane_s >> 3) ^ (wave & 1));
    const int lane_c = (lane_s & 7) ^ (lane_row & 7);
    b_base = w + ((int64_t)it.expert * n + (int64_t)it.n_tile * BNO) * ldw;
    const int n_left = min(n_out - it.n_tile * BNO, BNO);
    b_last = SWIGLU ? (uint32_t)(n_left / 32) : ((uint32_t)(n_left - 1) * (uint32_t)ldw + lane_c * 8) * 2u;
    b_rows = (uint32_t)n_left;
  };
  auto set_x_sources = [&](const GmmWork& it) {
    const int lane_s = lane_id_fresh();
    const int lane_row = wave * 8 + ((lane_s >> 3) ^ (wave & 1));
    const int lane_c = (lane_s & 7) ^ (lane_row & 7);
    const int x_left = min(it.row_end - it.row_begin, BM);  // rows of the group in this tile
    if constexpr (GATHER) {
      a_base = x;
#pragma unroll
      for (int i = 0; i < kACopies; ++i) {
        const int r = min(8 * kWaves * i + lane_row, x_left - 1);
        // row_idx / idx_div as a multiplication (exact for indices below 2^31; the launcher derives the
        // constants): a division by a run-time value costs a dozen registers that the k loop does not have
        const uint32_t flat = (uint32_t)row_idx[it.row_begin + r];
        uint32_t src = idx_magic ? (__umulhi(flat, idx_magic) >> idx_shift) : flat;
        src = src < x_rows ? src : x_rows - 1;  // an index outside x reads its last row instead of faulting
        a_src[i] = (src * (uint32_t)k + lane_c * 8) * 2u;  // in bytes (the launcher refuses x of 4 GiB or more)
      }
    } else {
      a_base = x + (int64_t)it.row_begin * k;
    }
    a_last = ((uint32_t)(x_left - 1) * (uint32_t)k + lane_c * 8) * 2u;
  };
  auto b_offset = [&](int i) -> uint32_t {
    if constexpr (SWIGLU) {
      const uint32_t blk = (uint32_t)i < b_last ? (uint32_t)i : 0u;  // blocks past n: repeat block 0
      return copy_offset(off0_glu, blk * 64u * (uint32_t)ldw);
    } else {
      return copy_offset(off0_w, i * copy_stride_w, b_last);
    }
  };
  const uint32_t lds_sa = (uint32_t)(uintptr_t)AOPS_LDS_PTR(sa);  // LDS byte addresses of the stages
  const uint32_t lds_sb = (uint32_t)(uintptr_t)AOPS_LDS_PTR(sb);
  // copy i of the activation tile kt into its stage (kACopies per wave and tile), copy i of the weight tile
  auto copy_x_one = [&](int kt, int stage, int i) {
    if constexpr (PROBE & kProbeNoXCopies) return;
    const int ko = kt * kBK;
    const uint32_t da = lds_sa + (uint32_t)(stage * BM * kBK + wave * 512) * 2u;
    if constexpr (GATHER) {
      dma16(a_base + ko, a_src[i], da + i * kWaves * 1024);
    } else {
      // uniform base + 32-bit byte offset per lane: the copy takes them as they are (scalar base,
      // vector offset), no vector instructions spent on a 64-bit address
      dma16(a_base + ko, copy_offset(off0, i * copy_stride, a_last), da + i * kWaves * 1024);
    }
  };
  auto copy_x = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < kACopies; ++i) copy_x_one(kt, stage, i);
  };
  auto copy_w_one = [&](int kt, int stage, int i) {
    if constexpr (PROBE & kProbeNoWCopies) return;
    const int ko = kt * kBK;
    const uint32_t db = lds_sb + (uint32_t)(stage * BN * kBK + wave * 512) * 2u;
    if constexpr (PROBE & kProbeWidePieces) {
      static_assert(!(PROBE & kProbeWidePieces) || (!SWIGLU && BN == 256 && kBCopies * kWaves * 4 == 128), "half a tile per copy round");
      const int lane_s = lane_id_fresh();  // a copy = 4 rows x 256 bytes
      const uint32_t row = min((uint32_t)((kt & 1) * 128 + (i * kWaves + wave) * 4 + (lane_s >> 4)), b_rows - 1u);
      dma16(b_base + (kt & ~1) * kBK, (row * (uint32_t)ldw + (uint32_t)(lane_s & 15) * 8u) * 2u, db + i * kWaves * 1024);
      return;
    }
    dma16(b_base + ko, b_offset(i), db + i * kWaves * 1024);
  };
  auto copy_w = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < kBCopies; ++i) copy_w_one(kt, stage, i);
  };

  // The MFMAs are v_mfma_f32_16x16x32_f16 (with operands that change from one instruction to the next the
  // matrix cores run at the clock the power limit leaves them, and this shape sustains about a fifth more
  // there than 32x32x16 does).  A fragment is 16 rows x 32 k: lane l holds row l & 15 and the l >> 4'th group of 8
  // k values.  Which 16-byte chunk of the tile's row a group is taken from is free as long as both operands
  // take the same one (the sum over k does not care about the order): lanes l and l + 32 are served by LDS in
  // the same cycle, and with chunks 0, 2, 1, 3 for l >> 4 = 0 .. 3 their chunks differ in the lowest bit, which
  // the row swizzle turns into different bank halves (chunks l >> 4 as they come: every read a two-way conflict).
  const int fm = lane & 15;
  const int fq = ((lane >> 4) & 1) * 2 + (lane >> 5);
  // Fragment addresses: lds_off(fm, 4*st + fq) == lds_off(fm, fq) ^ (st << 5) (the k step only flips the
  // top chunk bit), so one LDS byte address per operand and stage serves both k steps: the step's XOR is one
  // vector instruction, row block and column block are immediate offsets of the reads.  (Both regions start
  // on 128-byte boundaries, so the XOR of bit 6 stays inside a row.)
  typedef const __attribute__((address_space(3))) f16x8* LdsFrag;
  const uint32_t fa_byte0 = lds_sa + (uint32_t)(lds_off(fm, fq) + wm * 32 * kBK) * 2u;
  const uint32_t fb_byte0 = lds_sb + (uint32_t)(lds_off(fm, fq) + wn * 32 * NB * kBK) * 2u;
  const uint32_t fa_byte[2] = {fa_byte0, fa_byte0 + BM * kBK * 2u};
  const uint32_t fb_byte[2] = {fb_byte0, fb_byte0 + BN * kBK * 2u};

  constexpr int JB = 2 * NB;  // 16-column blocks of a wave
  // acc[b][j]: rows 32*(wm + 2*(b/2)) + 16*(b%2) .. +15 of the tile, columns 16*j .. +15 of the wave
  f32x4 acc[2 * MB][JB];
  GmmWork nxt;

  // The k loop.  Per k tile t (stage t & 1) a wave reads its weight fragments of all four k steps into
  // registers at once and its activation fragments one at a time, row block by row block:
  //
  //   barrier A(t): tile t has landed, nobody reads the activation stage of tile t-1 any more
  //     -> fragment reads of tile t between the last eight MFMAs of tile t-1, first MFMAs of tile t; the
  //        activation copies of tile t+1 one at a time between them
  //   barrier B(t): everybody holds the weight fragments of tile t in registers
  //     -> the other MFMAs of tile t; the weight copies of tile t+2 (into the weight stage of tile t) one at a
  //        time between them
  //
  // The weights are read once, so each of their requests goes to memory and is slow; the activation
  // rows mostly hit in L2.  Freeing the weight stage at the start of the tile gives the slow requests
  // more than a tile period to arrive, and barrier A(t+1) waits only for copies that were issued most of a
  // period before: the L1's queue of pending requests (what bounds this kernel) still holds requests of
  // tile t+2 when the next ones arrive, instead of draining to empty at every barrier.
  auto k_loop = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    constexpr int NBLK = 2 * LIVE;         // 16-row blocks of this wave that hold rows of the group
    constexpr int NF = kKSteps * NBLK;     // activation fragments of a k tile, JB MFMAs each
    constexpr int kFa = 4;                 // activation fragments in flight
    f16x8 fa[LIVE > 0 ? kFa : 1], fb[kKSteps][JB];
    if constexpr (PROBE & kProbeNoFragments) {  // operands the compiler cannot fold: the MFMAs stay
      const f16x8 one = {1, 1, 1, 1, 1, 1, 1, 1};
      for (auto& f : fa) {
        f = one;
        asm volatile("" : "+v"(f));
      }
      for (auto& row : fb)
        for (auto& f : row) {
          f = one;
          asm volatile("" : "+v"(f));
        }
    }
    // The XORs are volatile asm: written as expressions they would be hoisted out of the k loop, one
    // address register per (operand, stage, step), and push the accumulators into scratch.
    auto read_fb = [&](auto st_c, auto stage_c) {  // the weight fragments of k step ST
      constexpr int ST = decltype(st_c)::value;
      constexpr int STAGE = decltype(stage_c)::value;
      if constexpr (PROBE & kProbeNoFragments) return;
      uint32_t pb = fb_byte[STAGE];
      if constexpr (ST > 0) asm volatile("v_xor_b32 %0, %1, %2" : "=v"(pb) : "n"(ST << 6), "v"(fb_byte[STAGE]));
#pragma unroll
      for (int j = 0; j < JB; ++j) fb[ST][j] = *reinterpret_cast<LdsFrag>(pb + j * 16 * kBK * 2);
    };
    // fragment n = (16-row block n / 2, k step n % 2): row block by row block (taken k step by k step the
    // compiler needs 40 registers more and spills)
    auto read_fa = [&](auto n_c, auto stage_c) {
      constexpr int N = decltype(n_c)::value;
      constexpr int STAGE = decltype(stage_c)::value;
      if constexpr (N >= 0 && N < NF && !(PROBE & kProbeNoFragments)) {
        constexpr int ST = N % kKSteps;
        constexpr int B = N / kKSteps;
        uint32_t pa = fa_byte[STAGE];
        if constexpr (ST > 0) asm volatile("v_xor_b32 %0, %1, %2" : "=v"(pa) : "n"(ST << 6), "v"(fa_byte[STAGE]));
        fa[N % kFa] = *reinterpret_cast<LdsFrag>(pa + ((B / 2) * 64 + (B % 2) * 16) * kBK * 2);
      }
    };
    auto mma = [&](auto n_c) {
      constexpr int N = decltype(n_c)::value;
      if constexpr (N >= 0 && N < NF && !(PROBE & kProbeNoMfma)) {
#pragma unroll
        for (int j = 0; j < JB; ++j)
          acc[N / kKSteps][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[N % kKSteps][j], fa[N % kFa], acc[N / kKSteps][j], 0, 0, 0);
      }
    };
    auto fence = [] {
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    };
    // The MFMA groups of fragments N .. END-1 of the tile (JB MFMAs each, one per 16-column block of the wave), each
    // followed by the copies that hook(N) issues and by the read of the fragment that takes this one's place
    auto groups = [&](auto self, auto n_c, auto end_c, auto stage_c, auto&& hook) {
      constexpr int N = decltype(n_c)::value;
      if constexpr (N < decltype(end_c)::value) {
        mma(n_c);
        hook(n_c);
        read_fa(std::integral_constant<int, N + kFa>{}, stage_c);
        __builtin_amdgcn_sched_barrier(0);
        self(self, std::integral_constant<int, N + 1>{}, end_c, stage_c, hook);
      }
    };
    // The MFMAs of the last kTail fragments of a tile run at the start of the next one, between its first
    // fragment reads, so that the matrix cores have work while those reads are on their way.  The tail is
    // the whole fragment ring: the last two row blocks at both k steps, so tail group q needs the weight
    // fragments of k step q % 2, which the next tile's reads may only replace after the last tail group that
    // uses them (k step 0: group 2, k step 1: group 3).
    constexpr int kTail = kFa;
    static_assert(kTail == 4 && kKSteps == 2, "the start of a tile is written out for a tail of four groups");
    // barrier B comes after this many MFMA groups of the tile: the burst of reads at its start has returned by
    // then, so the wait in front of the barrier costs nothing
    constexpr int kGroupsBeforeB = NF - kTail < 6 ? NF - kTail : 6;
    // The copies of a tile are spread over the MFMA groups between its barriers instead of following the
    // barrier in one burst: a copy cannot issue while the L1's queue of pending requests is full, a wave
    // stuck at a copy issues no MFMAs, and a burst of four or five copies from each of the eight waves is
    // several queues long - while the queue, once the burst is in, drains with nothing behind it until the
    // next barrier.  One copy every other group keeps the queue fed at the rate it empties and costs a wave
    // a few lines' worth of waiting at a time, which the MFMAs in flight cover.
    constexpr int kSlotsA = LIVE > 0 ? kTail + kGroupsBeforeB : 0;  // tail groups + groups between barrier A and barrier B
    constexpr int kSlotsB = NF - kTail - kGroupsBeforeB;            // groups between barrier B and the next barrier A
    auto tile = [&](auto stage_c, int kx, int kw, bool tail, bool switch_x, bool switch_w) {
      constexpr int STAGE = decltype(stage_c)::value;
      if (switch_x) set_x_sources(nxt);
      auto x_copies_of_slot = [&](int slot) {
#pragma unroll
        for (int i = 0; i < kACopies; ++i)
          if (kSlotsA > 0 && i * kSlotsA / kACopies == slot) copy_x_one(kx, STAGE ^ 1, i);
      };
      auto w_copies_of_slot = [&](int slot) {
#pragma unroll
        for (int i = 0; i < kBCopies; ++i)
          if (kSlotsB > 0 && i * kSlotsB / kBCopies == slot) copy_w_one(kw, STAGE, i);
      };
      if constexpr (kSlotsA == 0) copy_x(kx, STAGE ^ 1);
      if constexpr (LIVE > 0) {
        auto start = [&](auto q_c) {  // tail group q of the previous tile, then the reads that reuse its registers
          constexpr int Q = decltype(q_c)::value;
          if (tail) mma(std::integral_constant<int, NF - kTail + Q>{});
          x_copies_of_slot(Q);
          read_fa(q_c, stage_c);
          __builtin_amdgcn_sched_barrier(0);  // the counted wait in front of barrier B relies on this order
          if constexpr (Q == 2) read_fb(std::integral_constant<int, 0>{}, stage_c);
          if constexpr (Q == 3) read_fb(std::integral_constant<int, 1>{}, stage_c);
          __builtin_amdgcn_sched_barrier(0);
        };
        start(std::integral_constant<int, 0>{});
        start(std::integral_constant<int, 1>{});
        start(std::integral_constant<int, 2>{});
        start(std::integral_constant<int, 3>{});
        groups(groups, std::integral_constant<int, 0>{}, std::integral_constant<int, kGroupsBeforeB>{}, stage_c,
              [&](auto n_c) { x_copies_of_slot(kTail + decltype(n_c)::value); });
      }
      // all own weight fragments of this tile are in registers (LDS serves a wave's reads in order, and only
      // the kGroupsBeforeB refills of the activation ring were issued after the last of them) ...
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0xc07f | ((LIVE > 0 ? kGroupsBeforeB : 0) << 8));  // lgkmcnt only
      fence();
      __builtin_amdgcn_s_barrier();  // ... and so are everybody else's: barrier B
      fence();
      if (switch_w) set_w_sources(nxt);
      if constexpr (kSlotsB == 0) copy_w(kw, STAGE);
      if constexpr (LIVE > 0)
        groups(groups, std::integral_constant<int, kGroupsBeforeB>{}, std::integral_constant<int, NF - kTail>{}, stage_c,
              [&](auto n_c) { w_copies_of_slot(decltype(n_c)::value - kGroupsBeforeB); });
      // own copies of the next tile (all but the weight copies just issued) and all own fragment reads of
      // this tile are complete ...
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kBCopies));
      fence();
      __builtin_amdgcn_s_barrier();  // ... and so are everybody else's: barrier A of the next tile
      fence();
    };
    for (int kt = 0; kt < ktiles; kt += 2) {
      const bool last = kt + 2 >= ktiles;  // the last two tiles fetch the head of the next item
      const bool follow = last && nxt.valid;
      // nothing follows: repeat the last tile (valid memory, never consumed)
      tile(std::integral_constant<int, 0>{}, kt + 1, last ? (follow ? 0 : ktiles - 1) : kt + 2, kt > 0, false, follow);
      tile(std::integral_constant<int, 1>{}, last ? (follow ? 0 : ktiles - 1) : kt + 2,
           last ? (follow ? 1 : ktiles - 1) : kt + 3, true, follow, false);
    }
    if constexpr (LIVE > 0) {
      mma(std::integral_constant<int, NF - 4>{});
      mma(std::integral_constant<int, NF - 3>{});
      mma(std::integral_constant<int, NF - 2>{});
      mma(std::integral_constant<int, NF - 1>{});
    }
  };

  set_w_sources(cur);
  set_x_sources(cur);
  copy_w(0, 0);
  copy_x(0, 0);
  copy_w(1, 1);
  // tile 0 must be complete, the weights of tile 1 may still be on their way
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kBCopies));
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
    for (int b = 0; b < 2 * MB; ++b)
#pragma unroll
      for (int j = 0; j < JB; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[b][j][r] = 0.f;
      }

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

    // Epilogue of `cur`.  acc[b][j][e]: output row 32*(wm + 2*(b/2)) + 16*(b%2) + fm, output column
    // wn*32*NB + 16j + 4fq + e: a lane holds one output row of a 16-row block and, of the wave's columns,
    // 8-byte pieces that alternate with those of three other lanes.  Stored from there, every store
    // instruction would scatter 8-byte pieces over 16 rows, and the count of write requests, not their
    // bytes, is what the memory pipeline of a CU charges for.  So the rows go through a 1 KiB LDS scratch
    // of the wave's own, a few at a time: the lanes of those rows write their pieces (16-byte slots
    // XOR-swizzled by the row: no bank conflicts beyond the two cycles that 256 bytes take), then all 64
    // lanes read 16 bytes each in row order and store whole row segments - eight 128-byte lines per
    // instruction (SWIGLU: sixteen 64-byte halves).  The operand stages stay untouched: the next item's
    // first tiles are landing in them.
    {
      f16* scr = sepi + wave * kEpiScratchHalfs;
      constexpr int kSegHalfs = SWIGLU ? 32 : 32 * NB;       // output columns of the wave
      constexpr int kRowsPerUnit = kEpiScratchHalfs / kSegHalfs;  // 8 rows of 128 bytes, or 16 of 64
      constexpr int kSlots = kSegHalfs / 8;                  // 16-byte slots per row segment
      constexpr int kUnits = 16 / kRowsPerUnit;              // per 16-row block
      constexpr int kOutBlocks = kSegHalfs / 16;             // 16-column blocks of the wave's output
      static_assert(kSegHalfs == 128 || kSegHalfs == 64 || kSegHalfs == 32, "row segment of 256, 128 or 64 bytes");
      static_assert(kRowsPerUnit <= 16 && 16 % kRowsPerUnit == 0 && kRowsPerUnit * kSlots == kWave, "one 16-byte slot per lane");
      const int col_w = SWIGLU ? cur.n_tile * BNO + wn * 32 : cur.n_tile * BN + wn * 32 * NB;
      // the lane-derived offsets are the same for every item; taken from a fresh lane id they are not
      // hoisted out of the item loop (and spilled)
      const int lane_e = lane_id_fresh();
      const int fm_e = lane_e & 15;
      const int fq_e = lane_e >> 4;
      const int unit_of_lane = fm_e / kRowsPerUnit;
      const int r_w = fm_e % kRowsPerUnit;                    // this lane's row inside its unit
      const int r_r = lane_e / kSlots;                        // the row this lane reads back and stores
      const int q_r = lane_e % kSlots;                        // ... and its 16-byte slot
      // slot swizzle of row r: rows whose segments start in the same bank get different slot orders
      auto swz = [](int r) { return kSlots == 16 ? (r & 3) : kSlots == 8 ? (r & 7) : ((r ^ (r >> 2)) & 3); };
      const f16* rd = scr + r_r * kSegHalfs + ((q_r ^ swz(r_r)) * 8);
      // this lane's pieces of a row: columns 16*jj + 4*fq .. +3, i.e. slot 2*jj + fq/2, its half fq%2
      f16* wr = scr + r_w * kSegHalfs + 4 * (fq_e & 1);
      const int q_w = (fq_e >> 1) ^ swz(r_w);                 // (2*jj + fq/2) ^ swz == (2*jj) ^ q_w: swz < kSlots
#pragma unroll
      for (int b = 0; b < 2 * MB; ++b) {
        if (b / 2 < live && col_w < n_out) {  // wave uniform
          // (the conversion sits inside the branch of the lane's unit: no registers are held for the pieces)
#pragma unroll
          for (int u = 0; u < kUnits; ++u) {
            if (unit_of_lane == u) {
#pragma unroll
              for (int jj = 0; jj < kOutBlocks; ++jj) {
                f16x4 piece;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  if constexpr (SWIGLU) {
                    const float gt = acc[b][jj][e];
                    const float up = acc[b][jj + JB / 2][e];
                    const float ex = __builtin_amdgcn_exp2f(-1.4426950408889634f * gt);
                    piece[e] = (f16)(gt * up * __builtin_amdgcn_rcpf(1.0f + ex));
                  } else {
                    piece[e] = (f16)acc[b][jj][e];
                  }
                }
                *reinterpret_cast<f16x4*>(wr + (((2 * jj) ^ q_w) * 8)) = piece;
              }
            }
            // LDS serves a wave's accesses in order: the read sees the writes above, and the next unit's
            // writes come after this read
            asm volatile("" ::: "memory");
            const f16x8 v = *reinterpret_cast<const f16x8*>(rd);
            asm volatile("" ::: "memory");
            const int m = 32 * wm + 64 * (b / 2) + 16 * (b % 2) + u * kRowsPerUnit + r_r;
            if (m < tile_rows)
              st128_stream(y + (int64_t)(cur.row_begin + m) * n_out + col_w + q_r * 8, v);
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

template <int MB, int NB, int WN, bool SWIGLU, bool GATHER = false, int PROBE = 0>
static int gmm_persistent_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y,
                                 int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                                 const int32_t* row_idx = nullptr, int idx_div = 1, int64_t x_rows = 1, int ldw = 0) {
  if (ldw == 0) ldw = k;  // densely packed weight rows
  constexpr int BM = 64 * MB;
  constexpr int BN = 32 * NB * WN;
  constexpr int kWaves = 2 * WN;
  constexpr int kLds = 2 * (BM + BN) * kBK * (int)sizeof(f16) + kWave * kPlanInts * (int)sizeof(int) +
                       kWaves * kEpiScratchHalfs * (int)sizeof(f16);
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const int cus = device_cu_count();
  constexpr int BNO = SWIGLU ? BN / 2 : BN;
  const int64_t n_out = SWIGLU ? n / 2 : n;
  const int64_t n_tiles = (n_out + BNO - 1) / BNO;
  const int64_t max_work = ((rows + BM - 1) / BM + num_experts) * n_tiles;
  if (max_work > 0x7fffffff - 8 * kXcds) return AOPS_ERR_INVALID_ARGUMENT;  // the kernel counts work items in 32 bits
  int64_t grid = cus < max_work ? cus : max_work;
  grid = grid / kXcds * kXcds;
  if (grid < kXcds) grid = kXcds;
  auto kernel = grouped_matmul_persistent_kernel<MB, NB, WN, SWIGLU, GATHER, PROBE>;
  static std::atomic<uint64_t> lds_allowed{0};  // per device
  if (const hipError_t le = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, lds_allowed); le != hipSuccess)
    return record_launch_status(le);
  // idx_div >= 2: q = (flat * magic) >> (32 + shift) with magic = ceil(2^(31 + l) / idx_div), l = ceil(log2 idx_div),
  // shift = l - 1; exact for flat < 2^31.  idx_div == 1: magic 0 = no division.
  uint32_t idx_magic = 0;
  int idx_shift = 0;
  if (idx_div >= 2) {
    int l = 0;
    while ((1ll << l) < idx_div) ++l;
    idx_magic = (uint32_t)(((1ull << (31 + l)) + (uint64_t)idx_div - 1) / (uint64_t)idx_div);
    idx_shift = l - 1;
  }
  kernel<<<(unsigned)grid, 2 * WN * kWave, kLds, stream>>>(x, w, group_list, y, rows, k, num_experts,
                                                          n, row_idx, idx_magic, idx_shift, (uint32_t)x_rows, ldw);
  return record_launch_status(hipGetLastError());
}

// Tile height of the persistent kernel: 320 rows (one tile covers a typical expert of a large routed
// batch) or 256 rows when that takes fewer rounds of work items over the CUs times rows per tile - the
// wall time of a compute-bound product.  group_list stays on the device, so the groups are taken as
// equal plus two standard deviations of a uniform routing; a single group is exact.
static bool gmm_prefer_256_rows(int64_t rows, int64_t num_experts, int64_t n_out_tiles, int cus) {
  const int64_t groups = num_experts < rows ? num_experts : rows;
  if (groups <= 0) return false;
  int64_t avg = (rows + groups - 1) / groups;
  if (groups > 1) {
    int64_t sd = 1;
    while (sd * sd < avg) ++sd;
    avg += 2 * sd;
  }
  auto cost = [&](int64_t bm) {
    const int64_t items = groups * ((avg + bm - 1) / bm) * n_out_tiles;
    return ((items + cus - 1) / cus) * bm;
  };
  return cost(256) < cost(320);
}

int gmm_launch_persistent(bool swiglu, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                          int64_t rows, int k, int num_experts, int n, hipStream_t stream,
                          const int32_t* row_idx, int idx_div, int64_t x_rows, int ldw) {
  const int64_t n_out_tiles = swiglu ? (n / 2 + 127) / 128 : (n + 255) / 256;
  const bool small = gmm_prefer_256_rows(rows, num_experts, n_out_tiles, device_cu_count());
  if (row_idx) {  // only the fused gate_up form gathers
    if (x_rows * k * 2 > 0xffffffffLL) return AOPS_ERR_INVALID_ARGUMENT;  // 32-bit byte offsets into x
    if (small)
      return gmm_persistent_launch<4, 2, 4, true, true>(x, w, group_list, y, rows, k, num_experts, n, stream,
                                                        row_idx, idx_div, x_rows, ldw);
    return gmm_persistent_launch<5, 2, 4, true, true>(x, w, group_list, y, rows, k, num_experts, n, stream,
                                                      row_idx, idx_div, x_rows, ldw);
  }
  if (swiglu) {
    if (small)
      return gmm_persistent_launch<4, 2, 4, true>(x, w, group_list, y, rows, k, num_experts, n, stream, nullptr, 1, 1, ldw);
    return gmm_persistent_launch<5, 2, 4, true>(x, w, group_list, y, rows, k, num_experts, n, stream, nullptr, 1, 1, ldw);
  }
  if (small)
    return gmm_persistent_launch<4, 2, 4, false>(x, w, group_list, y, rows, k, num_experts, n, stream, nullptr, 1, 1, ldw);
  return gmm_persistent_launch<5, 2, 4, false>(x, w, group_list, y, rows, k, num_experts, n, stream, nullptr, 1, 1, ldw);
}

// The 320 x 256 kernel with parts of its k loop switched off (see PROBE): a measurement aid.
int gmm_launch_persistent_probe(int parts_off, const f16* x, const f16* w, const int64_t* group_list, f16* y,
                                int64_t rows, int k, int num_experts, int n, hipStream_t stream, int ldw) {
  switch (parts_off) {
#define AOPS_PROBE_CASE(P)                                                                                        \
  case (P):                                                                                                       \
    return gmm_persistent_launch<5, 2, 4, false, false, (P)>(x, w, group_list, y, rows, k, num_experts, n, stream, \
                                                             nullptr, 1, 1, ldw);
    AOPS_PROBE_CASE(kProbeNoMfma | kProbeNoFragments)                       // 9: copies and barriers only
    AOPS_PROBE_CASE(kProbeNoMfma | kProbeNoFragments | kProbeNoXCopies)     // 11: weight copies only
    AOPS_PROBE_CASE(kProbeNoMfma | kProbeNoFragments | kProbeNoWCopies)     // 13: activation copies only
    AOPS_PROBE_CASE(kProbeNoXCopies | kProbeNoWCopies)                      // 6: MFMAs and fragment reads only
    AOPS_PROBE_CASE(kProbeNoXCopies | kProbeNoWCopies | kProbeNoFragments)  // 14: MFMAs only
    AOPS_PROBE_CASE(kProbeNoMfma)                                           // 1: copies and LDS fragment reads, no MFMAs
    AOPS_PROBE_CASE(kProbeNoFragments)                                      // 8: copies and MFMAs, no LDS fragment reads
    AOPS_PROBE_CASE(kProbeWidePieces | kProbeNoMfma | kProbeNoFragments)                    // 25: as 9, weights in 256-byte pieces
    AOPS_PROBE_CASE(kProbeWidePieces | kProbeNoMfma | kProbeNoFragments | kProbeNoXCopies)  // 27: as 11, weights in 256-byte pieces
#undef AOPS_PROBE_CASE
    default:
      return AOPS_ERR_INVALID_ARGUMENT;
  }
}

}  // namespace aops
