// Paged-attention decode over the [num_blocks, Hkv*D/16, block_size, 16] fp16 KV cache.
//
//   o[b,h] = softmax_j( q[b,h] . K[j,g] / sqrt(D) ) . V[j,g],   g = h / (Hq/Hkv)
//
// Split-KV ("flash decoding"): a workgroup of 8 waves owns one (sequence, kv head, chunk of
// the context); partial (max, sum, weighted V) triples go to a workspace and a second small
// kernel merges the chunks of each (sequence, query head).  context_lens and block_tables are
// read on the device only, so the grid is sized for the longest possible context and
// workgroups past the end of their sequence exit at once.
//
// Main kernel (every head_dim that is a multiple of 16 up to 256 with pages of a multiple of 16 tokens;
// described for 128), one step = 32 tokens of one kv head = 8 KiB of K + 8 KiB of V:
//  * For one kv head a page holds K as [8 d-chunks][block_size tokens][16 halfs].  A lane
//    (n = lane%16, kg = lane/16) loads, for token n of a 16-token group, the 16 bytes that hold
//    d = 32s + 8kg ..+7 (s = 0..3).  That register IS the per-lane operand of
//    v_mfma_f32_16x16x32_f16 (8 consecutive k per lane), so S^T[token][head] = K . Q^T runs on
//    the matrix core straight from the loads, and every load instruction of a wave fetches
//    two contiguous 512-byte runs.
//  * The MFMA result leaves lane (head, kg) with the scores of tokens 4kg..4kg+3 of each group:
//    after exp2 and packing that is already the per-lane operand P^T of the second product, so
//    the softmax needs two cross-row exchanges per step (for the running maximum) and no LDS.
//  * O^T[d][head] += V^T . P^T needs V with tokens along k.  V is loaded exactly like K and
//    transposed on the matrix core: V_tile . Sel with a 0/1 selector matrix returns
//    [token][16 d] blocks whose result layout has 4 consecutive tokens per lane; converted
//    back to fp16 (exact) they are the V^T operand.
//  * The K registers are refilled for the next step as soon as the scores are out, the V
//    registers as soon as P.V is done; the eight waves of the one workgroup a CU holds cover
//    each other's waits.
//
// Semantics: signature, cache indexing, GQA mapping and the fixed 1/sqrt(D) scale follow
// reference csrc/ffi/ops.cpp:408-482, csrc/opdev/op_host/paged_attention_ex.cpp:18-36 and
// csrc/opdev/op_kernel/paged_attention_ex.cpp:90-99 (whose compute body is unfinished).
#include <mutex>

#include "aops_common.h"

namespace aops {

constexpr int kPaWaves = 8;   // waves per workgroup
constexpr int kPaStep = 32;   // tokens per wave per step (two 16-token MFMA groups)
constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;

struct PaChunking {
  int chunk_tokens;  // tokens per workgroup (multiple of kPaWaves*kPaStep)
  int max_splits;    // partial-result slots per (sequence, head): chunks of the longest possible context
  int balanced_wgs;  // > 0: workgroups per kv head of the balanced partition (see pa_decode_balanced)
};

constexpr int kPaUnit = kPaWaves * kPaStep;  // 256 tokens: one step of every wave
constexpr int kPaMaxGroup = 16;              // query heads of a sub-group: one per lane of a row of the score product
constexpr int kPaXcds = 8;                   // workgroup i runs on XCD i % 8

// Batches of up to kPaPlanMax sequences can use the balanced partition; above 64 sequences every workgroup
// of the balanced kernel computes it in LDS and one of them leaves it, for the merge kernel, in the ints
// behind the partial results.
constexpr int64_t kPaPlanMax = 4096;
constexpr int64_t kPaMaxChunks = 512;  // partial results per (sequence, head) at most
constexpr int64_t kPaMaxShares = 256;
static size_t pa_tail_ints(int64_t bs) { return bs <= 64 ? (size_t)bs : (size_t)(2 * bs + 1 + kPaMaxShares); }

static PaChunking pa_chunking(int64_t bs, int64_t num_kv_heads, int64_t block_size,
                              int64_t max_blocks_per_seq) {
  const int64_t cus = device_cu_count();
  const int64_t max_len = block_size * max_blocks_per_seq;
  // As few chunks per sequence as still give every CU two workgroups: each chunk costs a
  // partial result and a workgroup prologue, and long chunks keep the load stream steady.
  constexpr int kUnit = kPaWaves * kPaStep;
  const int64_t wanted_workgroups = 2 * cus;
  int64_t splits = (wanted_workgroups + bs * num_kv_heads - 1) / (bs * num_kv_heads > 0 ? bs * num_kv_heads : 1);
  const int64_t max_units = (max_len + kUnit - 1) / kUnit;
  if (splits > max_units) splits = max_units;
  if (splits < 1) splits = 1;
  int chunk = (int)(((max_units + splits - 1) / splits) * kUnit);
  if (chunk < kUnit) chunk = kUnit;
  if ((max_len + chunk - 1) / chunk > kPaMaxChunks)  // the merge kernel keeps one weight per chunk in LDS
    chunk = (int)(((max_units + kPaMaxChunks - 1) / kPaMaxChunks) * kUnit);
  PaChunking c;
  c.chunk_tokens = chunk;
  c.max_splits = (int)((max_len + chunk - 1) / chunk);
  if (c.max_splits < 1) c.max_splits = 1;
  c.balanced_wgs = 0;
  // Small batches: fixed chunks of a few long sequences either leave CUs idle or, cut finer, pay
  // the per-workgroup start-up many times over.  With fewer than two (sequence, kv head) pairs per
  // CU the token stream is cut into one equal share per CU instead.
  // ... and whenever the block table allows contexts beyond 4096 tokens: whole sequences per workgroup
  // would let one long sequence among short ones occupy eight CUs for the whole launch.
  constexpr int64_t kSkewFreeLen = 4096;
  if (bs <= kPaPlanMax && max_units >= 2 && (bs * num_kv_heads < 2 * cus || max_len > kSkewFreeLen)) {
    int64_t wgs = (cus + num_kv_heads - 1) / num_kv_heads;
    if (wgs > kPaMaxShares) wgs = kPaMaxShares;
    if (wgs > bs * max_units) wgs = bs * max_units;  // never more shares than units
    c.balanced_wgs = (int)wgs;
    c.max_splits = (int)(wgs < max_units ? wgs : max_units);
  }
  return c;
}

// How a head of D elements is cut up for the matrix core: kFull slices of 32 d, plus, when D is an odd
// multiple of 16, a last slice that holds 16 d in the lanes kg < 2 and zeros in the lanes kg >= 2.
template <int D>
struct PaDims {
  static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head_dim: a multiple of 16 up to 256");
  static constexpr int kFull = D / 32;
  static constexpr int kTail = (D % 32) / 16;
  static constexpr int kSlices = kFull + kTail;
  static constexpr int kOutBlocks = D / 16;  // blocks of 16 d of O^T
};

// Per-lane slice of a 32-token tile: [token group][s] holds X[token 16t + n][d = 32s + 8kg ..+7],
// s = 0 .. NS-1 with NS = PaDims<D>::kSlices.
template <int NS>
using PaRegs = f16x8[2][NS];

// tail_live: this lane holds data of the half slice (kg < 2); the other lanes must not load (their
// address lies past the head's last d-chunk row) and hold zeros.
template <int D>
__device__ __forceinline__ void pa_issue_loads(const f16* __restrict__ cache, int64_t off0, int64_t off1,
                                               uint32_t lane_off, uint32_t s_stride, bool tail_live,
                                               PaRegs<PaDims<D>::kSlices>& r) {
  constexpr int kFull = PaDims<D>::kFull;
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const f16* base = cache + (g == 0 ? off0 : off1) + lane_off;  // token group g of the step
#pragma unroll
    for (int s = 0; s < kFull; ++s) r[g][s] = ld128_stream(base + s * s_stride);
    if constexpr (PaDims<D>::kTail) {
      f16x8 t = {0, 0, 0, 0, 0, 0, 0, 0};
      if (tail_live) t = ld128_stream(base + kFull * s_stride);
      r[g][kFull] = t;
    }
  }
}

template <int D>
struct PaState {
  f32x4 o[PaDims<D>::kOutBlocks];  // O^T blocks: lane (head n, kg), o[db][i] <-> d = 16 db + 4 kg + i
  float m;     // running maximum of head n (identical in the four lanes of a head)
  float l;     // this lane's share of the running sum
};

// S^T[token][head] = K . Q^T, scaled to log2 units; lane (head n, kg) gets tokens
// 16*(e/4) + 4kg + e%4, e = 0..7, of the step.
// QLDS: the Q^T fragments are read from LDS (q_lds = this lane's slice, fragment s 512 halfs further)
// instead of being held in registers: where many of them are needed they would push the kernel into scratch.
template <int NS, bool QLDS>
__device__ __forceinline__ void pa_scores(const PaRegs<NS>& k, const f16x8 (&qreg)[QLDS ? 1 : NS],
                                          const f16* q_lds, float scale_log2, float (&sc)[8]) {
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4 sacc[2] = {zero4, zero4};
  if constexpr (QLDS) {
    // the empty asm hides that the address is the same in every step, so the fragments are not
    // hoisted out of the token loop into registers
    uint32_t off = 0;
    asm volatile("" : "+v"(off));
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const f16x8 qs = *reinterpret_cast<const f16x8*>(q_lds + off + s * (kWave * 8));
#pragma unroll
      for (int g = 0; g < 2; ++g)
        sacc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(k[g][s], qs, sacc[g], 0, 0, 0);
    }
  } else {
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int s = 0; s < NS; ++s)
        sacc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(k[g][s], qreg[s], sacc[g], 0, 0, 0);
  }
  // A matrix-core result may only be read six wait states after its instruction (four passes plus
  // two).  The compiler keeps that distance inside a basic block, but when it places the
  // accumulators in AGPRs and a taken branch (the "no further step" case of the caller) lies between
  // the last product and the first v_accvgpr_read, it emits the read two wait states after the
  // product and the last score of every step comes back stale.  Pinning the accumulators to VGPRs
  // here and spending eight idle cycles keeps the distance whatever the block layout.
  asm volatile("s_nop 7" : "+v"(sacc[0]), "+v"(sacc[1]));
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) sc[4 * g + i] = sacc[g][i] * scale_log2;
}

// Online softmax update; returns the P^T operand (lane (head n, kg), element e <-> token e).
template <int D>
__device__ __forceinline__ f16x8 pa_softmax(float (&sc)[8], PaState<D>& st) {
  float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])),
                   fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
  mx = fmaxf(mx, __shfl_xor(mx, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 32));
  const float m_new = fmaxf(st.m, mx);
  const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);
  st.m = m_new;
  f16x8 pt;
  float psum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    pt[e] = (f16)__builtin_amdgcn_exp2f(sc[e] - m_new);
    psum += (float)pt[e];
  }
  st.l = st.l * alpha + psum;
  if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {  // the maximum rarely moves after the start
#pragma unroll
    for (int db = 0; db < PaDims<D>::kOutBlocks; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) st.o[db][i] *= alpha;
  }
  return pt;
}

// O^T += V^T . P^T with V transposed on the matrix core; the transposed tile serves every sub-group of
// query heads.
template <int D, int NSUB>
__device__ __forceinline__ void pa_accumulate(const PaRegs<PaDims<D>::kSlices>& v, const f16x8 (&sel)[2],
                                              const f16x8 (&pt)[NSUB], PaState<D> (&st)[NSUB]) {
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < PaDims<D>::kSlices; ++s) {
#pragma unroll
    for (int u = 0; u < (s < PaDims<D>::kFull ? 2 : 1); ++u) {  // the half slice has d = 32s + n only
      // [token][d = 32s + 16u + n]: lane (n, kg) receives tokens 4kg..4kg+3 of each group
      const f32x4 x0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(v[0][s], sel[u], zero4, 0, 0, 0);
      const f32x4 x1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(v[1][s], sel[u], zero4, 0, 0, 0);
      f16x8 vt;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vt[i] = (f16)x0[i];
        vt[4 + i] = (f16)x1[i];
      }
#pragma unroll
      for (int sg = 0; sg < NSUB; ++sg)
        st[sg].o[2 * s + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vt, pt[sg], st[sg].o[2 * s + u], 0, 0, 0);
    }
  }
}

// LDS of the main kernels (dynamic): [Q^T fragments, where they are kept there][acc: kPaWaves x hp rows of
// D + kPaAccPad floats][m: kPaWaves x hp][l: kPaWaves x hp]; hp = query heads per pass of the cross-wave merge
// (chosen by the host so that the whole fits 64 KiB).  The pad keeps the rows of the 16 heads, which the lanes of
// a wave write side by side, out of each other's banks.
constexpr int kPaAccPad = 4;
constexpr int kPaLdsPerHead(int head_dim) { return head_dim + kPaAccPad + 2; }  // floats per wave and head
template <int D, int NSUB>
constexpr bool pa_q_in_lds() { return PaDims<D>::kSlices * NSUB > 4; }
template <int D, int NSUB>
constexpr int pa_q_lds_halfs() { return pa_q_in_lds<D, NSUB>() ? NSUB * PaDims<D>::kSlices * kWave * 8 : 0; }

// What a workgroup needs to know about the launch besides its chunk.
struct PaGeom {
  int num_heads, num_kv_heads, block_size, max_blocks_per_seq, max_splits, num_blocks;
  int group;        // query heads per kv head
  int wg_heads;     // query heads per workgroup (16 * NSUB at most); a kv head with more is served by several
  int virt;         // workgroups per kv head: ceil(group / wg_heads)
  int merge_heads;  // hp above
  float scale_log2;
};

// One chunk of one (sequence b, kv head g): tokens chunk_start .. chunk_start + chunk_len - 1, the
// steps dealt round robin to the eight waves, which are merged through LDS at the end.  The workgroup
// serves the nh query heads head0 .. head0 + nh - 1 of the kv head in NSUB sub-groups of 16 (a lane of the
// score product holds one head of a sub-group); K and V of a step are loaded once and V is transposed
// once for all sub-groups.  final: the chunk is the whole sequence, so the normalised output is written
// directly; otherwise the partial result goes to slot `split` of the (sequence, head)'s max_splits slots.
// Called by all threads of the workgroup with uniform arguments.
template <int D, int NSUB>
__device__ __forceinline__ void pa_process_chunk(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    float* __restrict__ part_o, float* __restrict__ part_ml, f16* __restrict__ out, bool final, int b, int g,
    int head0, int nh, int context_len, int chunk_start, int chunk_len, int split, const PaGeom& ge) {
  constexpr int kPaD = D;
  constexpr int NS = PaDims<D>::kSlices;
  constexpr int kFull = PaDims<D>::kFull;
  constexpr int NOB = PaDims<D>::kOutBlocks;
  const int nsteps = (chunk_len + kPaStep - 1) / kPaStep;
  const int block_size = ge.block_size;
  const int max_blocks_per_seq = ge.max_blocks_per_seq;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int n = lane & 15;
  const int kg = lane >> 4;
  const bool tail_live = kg < 2;
  const int num_heads = ge.num_heads;

  extern __shared__ __attribute__((aligned(16))) unsigned char pa_lds[];
  f16* sm_q = reinterpret_cast<f16*>(pa_lds);
  float* sm_acc = reinterpret_cast<float*>(pa_lds + pa_q_lds_halfs<D, NSUB>() * sizeof(f16));
  const int hp = ge.merge_heads;
  constexpr int kAccStride = kPaD + kPaAccPad;
  float* sm_m = sm_acc + kPaWaves * hp * kAccStride;
  float* sm_l = sm_m + kPaWaves * hp;

  // Q^T operand: lane (head n of a sub-group, kg) holds q[head][32s + 8kg ..+7]; heads >= nh are zero
  // rows, and so are d >= D in the half slice.
  constexpr bool QLDS = pa_q_in_lds<D, NSUB>();
  f16x8 qreg[QLDS ? 1 : NSUB][QLDS ? 1 : NS];
  const f16* q_lds = sm_q + lane * 8;
  {
    const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    if (!QLDS || wave == 0) {  // in LDS every wave uses the same fragments: wave 0 fetches them
#pragma unroll
      for (int sg = 0; sg < NSUB; ++sg) {
        const int hl = 16 * sg + n;
        const bool head_live = hl < nh;
        const f16* qp = q + ((int64_t)b * num_heads + head0 + (head_live ? hl : 0)) * kPaD + 8 * kg;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          f16x8 frag = zero8;
          if (head_live && (s < kFull || tail_live)) frag = ld128(qp + 32 * s);
          if constexpr (QLDS) {
            *reinterpret_cast<f16x8*>(sm_q + ((sg * NS + s) * kWave + lane) * 8) = frag;
          } else {
            qreg[sg][s] = frag;
          }
        }
      }
    }
    if constexpr (QLDS) __syncthreads();
  }
  // Selector operands of the transposing product: sel[u][k][n] = (k == n + 16u), k = 8kg + e.
  f16x8 sel[2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int e = 0; e < 8; ++e) sel[u][e] = (8 * kg + e == n + 16 * u) ? (f16)1.0f : (f16)0.0f;

  PaState<D> st[NSUB];
#pragma unroll
  for (int sg = 0; sg < NSUB; ++sg) {
#pragma unroll
    for (int db = 0; db < NOB; ++db) st[sg].o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    st[sg].m = kNegBig;
    st[sg].l = 0.f;
  }

  // Element offsets inside one page for this lane: d-chunk rows are block_size*16 halfs apart
  // (this lane starts in row kg/2), the two halves of a granule 8 halfs, tokens 16 halfs.
  const uint32_t lane_off = (uint32_t)(kg >> 1) * (uint32_t)block_size * 16u +
                            (uint32_t)(kg & 1) * 8u + (uint32_t)n * 16u;
  const uint32_t s_stride = 2u * (uint32_t)block_size * 16u;  // 32 d further = two d-chunk rows
  const int64_t page_elems = (int64_t)ge.num_kv_heads * kPaD * block_size;
  const int64_t head_off = (int64_t)g * kPaD * block_size;
  const int32_t* table = block_tables + (int64_t)b * max_blocks_per_seq;
  const int num_blocks = ge.num_blocks;

  // Offset of the 16-token group `grp` of a step (wave uniform).  Page sizes are multiples of 16, so a
  // group never straddles two pages; the two groups of a step may (page sizes that are odd multiples).
  auto page_offset = [&](int step, int grp) -> int64_t {
    const int tok = chunk_start + step * kPaStep + 16 * grp;
    const int blk = min(tok / block_size, max_blocks_per_seq - 1);  // the group past the end of the last page
    // a table entry outside the cache reads the nearest page instead of faulting
    const int64_t page = min(max(table[blk], 0), num_blocks - 1);
    return page * page_elems + head_off + (int64_t)(tok - (tok / block_size) * block_size) * 16;
  };

  // One step of this wave on the register set (kreg, vreg); the set is refilled for the step `stride`
  // steps further on: K as soon as the scores are out, V as soon as P.V is done.
  auto do_step = [&](PaRegs<NS>& kreg, PaRegs<NS>& vreg, int step, int stride) {
    const int next = step + stride;
    const bool has_next = next < nsteps;
    const int64_t next_off0 = has_next ? page_offset(next, 0) : 0;
    const int64_t next_off1 = has_next ? page_offset(next, 1) : 0;
    const int step_token0 = chunk_start + step * kPaStep;
    float sc[NSUB][8];
#pragma unroll
    for (int sg = 0; sg < NSUB; ++sg)
      pa_scores<NS, QLDS>(kreg, qreg[QLDS ? 0 : sg], q_lds + sg * (NS * kWave * 8), ge.scale_log2, sc[sg]);
    if (has_next) pa_issue_loads<D>(key_cache, next_off0, next_off1, lane_off, s_stride, tail_live, kreg);
    if (step_token0 + kPaStep > context_len) {  // wave uniform: last, partial step of the sequence
      // Cache contents past the end of the sequence are arbitrary (possibly NaN): drop their
      // scores and zero their V rows before they reach the matrix core.
      const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (step_token0 + 16 * g + 4 * kg + i >= context_len) {
#pragma unroll
            for (int sg = 0; sg < NSUB; ++sg) sc[sg][4 * g + i] = -__builtin_inff();
          }
        if (step_token0 + 16 * g + n >= context_len) {
#pragma unroll
          for (int s = 0; s < NS; ++s) vreg[g][s] = zero8;
        }
      }
    }
    f16x8 pt[NSUB];
#pragma unroll
    for (int sg = 0; sg < NSUB; ++sg) pt[sg] = pa_softmax<D>(sc[sg], st[sg]);
    pa_accumulate<D, NSUB>(vreg, sel, pt, st);
    if (has_next) pa_issue_loads<D>(value_cache, next_off0, next_off1, lane_off, s_stride, tail_live, vreg);
  };
  auto first_loads = [&](PaRegs<NS>& kreg, PaRegs<NS>& vreg, int step) {
    if (step < nsteps) {
      const int64_t off0 = page_offset(step, 0), off1 = page_offset(step, 1);
      pa_issue_loads<D>(key_cache, off0, off1, lane_off, s_stride, tail_live, kreg);
      pa_issue_loads<D>(value_cache, off0, off1, lane_off, s_stride, tail_live, vreg);
    }
  };
  // (A second register set, with the step after next in flight as well, was tried up to head_dim
  // 128: no gain where it fits, and scratch use in the balanced kernel.)
  PaRegs<NS> kreg, vreg;
  first_loads(kreg, vreg, wave);
  for (int step = wave; step < nsteps; step += kPaWaves) do_step(kreg, vreg, step, kPaWaves);

  // Merge the waves of the workgroup through LDS and emit one result per query head, hp heads of one
  // sub-group per pass.
#pragma unroll
  for (int sg = 0; sg < NSUB; ++sg) {
    // The four lanes of a head hold disjoint shares of the sum.
    float l_head = st[sg].l;
    l_head += __shfl_xor(l_head, 16);
    l_head += __shfl_xor(l_head, 32);
    const int sub_end = min(nh, 16 * sg + 16);
    for (int h0 = 16 * sg; h0 < sub_end; h0 += hp) {
      const int cnt = min(hp, sub_end - h0);
      const int r = 16 * sg + n - h0;  // this lane's head inside the pass
      if (r >= 0 && r < cnt) {
        float* dst = sm_acc + (wave * hp + r) * kAccStride + 4 * kg;
#pragma unroll
        for (int db = 0; db < NOB; ++db) *reinterpret_cast<f32x4*>(dst + 16 * db) = st[sg].o[db];
        if (kg == 0) {
          sm_m[wave * hp + r] = st[sg].m;
          sm_l[wave * hp + r] = l_head;
        }
      }
      __syncthreads();
      for (int e = threadIdx.x; e < cnt * kPaD; e += kPaWaves * kWave) {
        const int h = e / kPaD;
        const int d = e - h * kPaD;
        float mx = sm_m[h];
#pragma unroll
        for (int w = 1; w < kPaWaves; ++w) mx = fmaxf(mx, sm_m[w * hp + h]);
        float lsum = 0.f, a = 0.f;
#pragma unroll
        for (int w = 0; w < kPaWaves; ++w) {
          const float wt = __builtin_amdgcn_exp2f(sm_m[w * hp + h] - mx);
          lsum += sm_l[w * hp + h] * wt;
          a += sm_acc[(w * hp + h) * kAccStride + d] * wt;
        }
        const int64_t head = (int64_t)b * num_heads + head0 + h0 + h;
        if (final) {
          out[head * kPaD + d] = (f16)(lsum > 0.f ? a / lsum : 0.f);
        } else {
          const int64_t slot = head * ge.max_splits + split;
          part_o[slot * kPaD + d] = a;
          if (d == 0) {
            part_ml[slot * 2 + 0] = mx;
            part_ml[slot * 2 + 1] = lsum;
          }
        }
      }
      if (h0 + hp < sub_end || sg + 1 < NSUB) __syncthreads();  // the next pass reuses the arrays
    }
  }
}

constexpr int kPaRankMax = 1024;

// One workgroup: order[r] = the sequence with the r-th longest context (ties by index).
__global__ __launch_bounds__(kPaRankMax) void pa_rank_sequences(const int32_t* __restrict__ context_lens,
                                                                int bs, int32_t* __restrict__ order) {
  __shared__ int lens[kPaRankMax];
  const int t = threadIdx.x;
  const int mine = t < bs ? context_lens[t] : 0;
  lens[t] = mine;
  __syncthreads();
  if (t >= bs) return;
  int rank = 0;
  for (int j = 0; j < bs; ++j) {
    const int other = lens[j];
    rank += (other > mine || (other == mine && j < t)) ? 1 : 0;
  }
  order[rank] = t;
}

// grid = (max_splits, Hkv * virt, bs), block = 8 waves: one chunk of chunk_tokens tokens per workgroup.  A
// sequence that fits one chunk gets its output written directly; the others leave partial results.
template <int D, int NSUB>
__global__ __launch_bounds__(kPaWaves* kWave) void pa_decode_partial(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, float* __restrict__ part_o,
    float* __restrict__ part_ml, f16* __restrict__ out, const PaGeom ge, int chunk_tokens,
    const int32_t* __restrict__ order) {
  const int split = blockIdx.x;
  const int g = (int)blockIdx.y / ge.virt;
  const int v = (int)blockIdx.y - g * ge.virt;
  const int head0 = g * ge.group + v * ge.wg_heads;
  const int nh = min(ge.wg_heads, ge.group - v * ge.wg_heads);
  // Workgroups are handed out in index order, so they take the sequences longest first: with
  // one resident workgroup per CU the short sequences then fill the gaps the long ones leave
  // (longest-processing-time-first).  For batches of up to 64 sequences every wave finds the
  // sequence of rank blockIdx.z by comparing the lengths held one per lane; larger batches (up to
  // kPaRankMax sequences) get the order from pa_rank_sequences.
  int b = order ? order[blockIdx.z] : (int)blockIdx.z;
  if (gridDim.z <= kWave) {
    const int ln = threadIdx.x & (kWave - 1);
    const int mine = ln < (int)gridDim.z ? context_lens[ln] : -0x7fffffff - 1;
    int rank = 0;
    for (int j = 0; j < (int)gridDim.z; ++j) {
      const int other = __builtin_amdgcn_readlane(mine, j);
      rank += (other > mine || (other == mine && j < ln)) ? 1 : 0;
    }
    const uint64_t hit = __ballot(rank == (int)blockIdx.z && ln < (int)gridDim.z);
    if (hit) b = __builtin_ctzll(hit);  // exactly one lane has each rank
  }
  // a length beyond the block table would walk off the table row
  const int context_len = min(context_lens[b], ge.max_blocks_per_seq * ge.block_size);
  const int chunk_start = split * chunk_tokens;
  if (chunk_start >= context_len) {
    if (split == 0) {  // empty sequence: zeros
      for (int e = threadIdx.x; e < nh * D; e += kPaWaves * kWave)
        out[((int64_t)b * ge.num_heads + head0) * D + e] = (f16)0.f;
    }
    return;
  }
  pa_process_chunk<D, NSUB>(q, key_cache, value_cache, block_tables, part_o, part_ml, out,
                            context_len <= chunk_tokens, b, g, head0, nh, context_len, chunk_start,
                            min(context_len - chunk_start, chunk_tokens), split, ge);
}

// Balanced partition for batches of up to 64 sequences.  Lane l of every wave holds sequence l:
// its length, its number of 256-token units, and the number of units in front of it.
struct PaUnits {
  int len;     // context length, clamped to [0, table capacity]
  int units;   // ceil(len / 256)
  int before;  // units of the sequences 0 .. l-1
  int total;   // units of the whole batch
};

__device__ __forceinline__ PaUnits pa_units(const int32_t* __restrict__ context_lens, int bs, int max_len) {
  const int lane = threadIdx.x & (kWave - 1);
  PaUnits r;
  r.len = lane < bs ? min(max(context_lens[lane], 0), max_len) : 0;
  r.units = (r.len + kPaUnit - 1) / kPaUnit;
  int incl = r.units;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  r.before = incl - r.units;
  r.total = __shfl(incl, kWave - 1);
  return r;
}

// Share w of `wgs` covers units [w*total/wgs, (w+1)*total/wgs); this is the share that holds unit x.
__device__ __forceinline__ int pa_share_of(int x, int wgs, int total) {
  return (int)((((int64_t)x + 1) * wgs - 1) / total);
}

// The same partition for batches of 65 .. kPaPlanMax sequences: every workgroup of the balanced kernel
// scans the lengths itself (thread t holds kPaPlanPer consecutive sequences) and keeps, in LDS behind the
// merge arrays, lds_plan[b] = units in front of sequence b and lds_plan[bs + b] = its clamped length,
// then [2*bs] = total units, [2*bs + 1] = the sequence that holds the share's first unit.  Workgroup
// (0, 0) also writes   plan[0] = total, plan[1 + b] = units in front of b, plan[1 + bs + b] = its length
// to global memory for the merge kernel.
constexpr int kPaPlanPer = (int)(kPaPlanMax / (kPaWaves * kWave));  // 8 sequences per thread
static_assert(kPaPlanPer * kPaWaves * kWave == kPaPlanMax, "every sequence has a thread");

__device__ __forceinline__ void pa_block_plan(const int32_t* __restrict__ context_lens, int bs, int max_len,
                                              int wgs_max, int w, int* __restrict__ lds_plan,
                                              int32_t* __restrict__ plan, bool publish) {
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int per = (bs + kPaWaves * kWave - 1) / (kPaWaves * kWave);  // <= kPaPlanPer
  int len[kPaPlanPer], units[kPaPlanPer];
  int mine = 0;
#pragma unroll
  for (int i = 0; i < kPaPlanPer; ++i) {
    const int b = t * per + i;
    len[i] = (i < per && b < bs) ? min(max(context_lens[b], 0), max_len) : 0;
    units[i] = (len[i] + kPaUnit - 1) / kPaUnit;
    mine += units[i];
  }
  int incl = mine;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  int* wave_sum = lds_plan + 2 * bs + 2;  // kPaWaves ints
  if (lane == kWave - 1) wave_sum[wave] = incl;
  __syncthreads();
  int before = incl - mine;
  int total = 0;
#pragma unroll
  for (int v = 0; v < kPaWaves; ++v) {
    const int ws = wave_sum[v];
    if (v < wave) before += ws;
    total += ws;
  }
  const int wgs = min(wgs_max, total);
  const int lo = (total > 0 && w < wgs) ? (int)((int64_t)w * total / wgs) : -1;
  if (t == 0) {
    lds_plan[2 * bs] = total;
    lds_plan[2 * bs + 1] = bs;  // stays if the share is empty
    if (publish) plan[0] = total;
  }
  __syncthreads();  // [2*bs + 1] is initialised before the one thread below overwrites it
#pragma unroll
  for (int i = 0; i < kPaPlanPer; ++i) {
    const int b = t * per + i;
    if (i < per && b < bs) {
      lds_plan[b] = before;
      lds_plan[bs + b] = len[i];
      if (publish) {
        plan[1 + b] = before;
        plan[1 + bs + b] = len[i];
      }
      if (units[i] > 0 && before <= lo && lo < before + units[i]) lds_plan[2 * bs + 1] = b;
    }
    before += units[i];
  }
  __syncthreads();
}

// ints of LDS the plan above needs
static inline size_t pa_block_plan_ints(int64_t bs) { return bs > kWave ? (size_t)(2 * bs + 2 + kPaWaves) : 0; }

// grid = (wgs, Hkv * virt), block = 8 waves.  Workgroup w walks through its share of the batch's units,
// sequence by sequence; a sequence that lies inside one share gets its output written directly, otherwise
// the part of sequence b the share covers becomes partial result number w - (share holding b's first unit)
// of that sequence.  Up to 64 sequences the partition is computed by every wave (pa_units); above that by
// the workgroup (pa_block_plan).
template <int D, int NSUB>
__global__ __launch_bounds__(kPaWaves* kWave) void pa_decode_balanced(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, float* __restrict__ part_o,
    float* __restrict__ part_ml, f16* __restrict__ out, int bs, const PaGeom ge, int32_t* __restrict__ plan) {
  const int w = blockIdx.x;
  const int g = (int)blockIdx.y / ge.virt;
  const int v = (int)blockIdx.y - g * ge.virt;
  const int head0 = g * ge.group + v * ge.wg_heads;
  const int nh = min(ge.wg_heads, ge.group - v * ge.wg_heads);
  const int max_len = ge.max_blocks_per_seq * ge.block_size;
  const bool planned = bs > kWave;  // the partition lives in LDS (pa_block_plan), else in the lanes (pa_units)
  const int* lds_plan = nullptr;
  PaUnits pu = {0, 0, 0, 0};
  int total, next_b = 0;
  if (planned) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pa_lds[];
    int* plan_w = reinterpret_cast<int*>(pa_lds + pa_q_lds_halfs<D, NSUB>() * sizeof(f16)) +
                  kPaWaves * ge.merge_heads * kPaLdsPerHead(D);
    pa_block_plan(context_lens, bs, max_len, (int)gridDim.x, w, plan_w, plan, w == 0 && blockIdx.y == 0);
    lds_plan = plan_w;
    total = lds_plan[2 * bs];
    next_b = lds_plan[2 * bs + 1];  // the sequence that holds the share's first unit
  } else {
    pu = pa_units(context_lens, bs, max_len);
    total = pu.total;
  }
  // no more shares than units: every share then holds at least one unit, and the shares of a
  // sequence are consecutive
  const int wgs = min((int)gridDim.x, total);
  if (w >= wgs) return;
  const int lo = (int)((int64_t)w * total / wgs);
  const int hi = (int)((int64_t)(w + 1) * total / wgs);
  int cur = lo;
  while (cur < hi) {
    // the sequence that holds unit cur
    int b, before, len;
    if (planned) {
      while (next_b < bs && lds_plan[bs + next_b] <= 0) ++next_b;  // empty sequences hold no unit
      if (next_b >= bs) break;  // cannot happen: the units of the sequences tile [0, total)
      b = next_b++;
      before = lds_plan[b];
      len = lds_plan[bs + b];
    } else {
      const uint64_t hit = __ballot(pu.units > 0 && pu.before <= cur && cur < pu.before + pu.units);  // one lane
      if (hit == 0) break;  // cannot happen either
      b = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit));
      before = __builtin_amdgcn_readlane(pu.before, b);
      len = __builtin_amdgcn_readlane(pu.len, b);
    }
    const int units = (len + kPaUnit - 1) / kPaUnit;
    const int seg_end = min(hi, before + units);
    const int tok0 = (cur - before) * kPaUnit;
    const int tok1 = min((seg_end - before) * kPaUnit, len);
    const int first = pa_share_of(before, wgs, total);
    const bool whole = pa_share_of(before + units - 1, wgs, total) == first;
    pa_process_chunk<D, NSUB>(q, key_cache, value_cache, block_tables, part_o, part_ml, out, whole, b, g,
                              head0, nh, len, tok0, tok1 - tok0, w - first, ge);
    cur = seg_end;
    if (cur < hi) __syncthreads();  // the LDS arrays of the chunk are reused
  }
}

// grid = (Hq, bs), block = 4 waves.  Sequences whose output the attention kernel has written itself (one
// partial result) are left alone.  Every wave works out the weights 2^(m_s - max m) of the partial
// results (a lane per result); wave v then adds up the results s = v, v+4, ... with eight row loads in
// flight (a lane holds kPer neighbouring output elements: 1, 2 or 4 for head_dim up to 64, 128, 256), and
// the four sums meet in LDS.
constexpr int kPaMergeWaves = 4;
constexpr int kPaMergeMaxSplits = (int)kPaMaxChunks;  // weights kept in LDS; pa_chunking never cuts a sequence finer

template <int kPer>
__global__ __launch_bounds__(kPaMergeWaves* kWave) void pa_decode_merge(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int32_t* __restrict__ context_lens, f16* __restrict__ o, int head_dim, int num_heads, int chunk_tokens,
    int max_splits, int balanced_wgs, int bs, int max_len, const int32_t* __restrict__ plan) {
  typedef float fvec __attribute__((ext_vector_type(kPer)));
  __shared__ float wts[kPaMergeMaxSplits];
  __shared__ float red[kPaMergeWaves][kPer * kWave];
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int context_len = context_lens[b];
  const int64_t out = ((int64_t)b * num_heads + h) * head_dim;
  if (context_len <= 0) {
    if ((int)threadIdx.x < head_dim) o[out + threadIdx.x] = (f16)0.f;
    return;
  }
  int nsplit;
  if (balanced_wgs > 0 && plan) {
    const int total = plan[0];
    const int before = plan[1 + b];
    const int units = (plan[1 + bs + b] + kPaUnit - 1) / kPaUnit;
    const int wgs = min(balanced_wgs, total);
    nsplit = pa_share_of(before + units - 1, wgs, total) - pa_share_of(before, wgs, total) + 1;
  } else if (balanced_wgs > 0) {  // partial results of the shares that hold the sequence's first and last unit
    const PaUnits pu = pa_units(context_lens, bs, max_len);
    const int before = __builtin_amdgcn_readlane(pu.before, b);
    const int units = __builtin_amdgcn_readlane(pu.units, b);
    const int wgs = min(balanced_wgs, pu.total);
    nsplit = pa_share_of(before + units - 1, wgs, pu.total) - pa_share_of(before, wgs, pu.total) + 1;
  } else {
    nsplit = (min(context_len, max_len) + chunk_tokens - 1) / chunk_tokens;
  }
  if (nsplit <= 1) return;  // the attention kernel wrote this sequence's output itself
  nsplit = min(nsplit, min(max_splits, kPaMergeMaxSplits));
  const int64_t base = ((int64_t)b * num_heads + h) * max_splits;
  const bool act = lane * kPer < head_dim;  // lanes past the end of the head hold nothing

  // weights: the same in every wave; wave 0 leaves them in LDS
  constexpr int kMlPerLane = kPaMergeMaxSplits / kWave;
  float m_s[kMlPerLane], l_s[kMlPerLane];
  float mx = kNegBig;
#pragma unroll
  for (int i = 0; i < kMlPerLane; ++i) {
    const int s = i * kWave + lane;
    m_s[i] = kNegBig;
    l_s[i] = 0.f;
    if (i * kWave < nsplit && s < nsplit) {  // first test is wave uniform: whole rounds are skipped
      const float2 ml = *reinterpret_cast<const float2*>(&part_ml[(base + s) * 2]);
      m_s[i] = ml.x;
      l_s[i] = ml.y;
    }
    mx = fmaxf(mx, m_s[i]);
  }
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < kMlPerLane; ++i) {
    const int s = i * kWave + lane;
    const float wt = s < nsplit ? __builtin_amdgcn_exp2f(m_s[i] - mx) : 0.f;
    lsum += l_s[i] * wt;
    if (wave == 0 && i * kWave < nsplit) wts[s] = wt;
  }
  lsum = wave_sum(lsum);
  __syncthreads();

  fvec acc;
#pragma unroll
  for (int e = 0; e < kPer; ++e) acc[e] = 0.f;
  constexpr int kInFlight = 8;
  for (int s0 = wave; s0 < nsplit; s0 += kPaMergeWaves * kInFlight) {
    fvec v[kInFlight];
    float wt[kInFlight];
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const int s = s0 + j * kPaMergeWaves;
      const int sc = min(s, nsplit - 1);  // past the end: a valid row with weight 0
      v[j] = acc;                         // any finite value for the idle lanes
      if (act) v[j] = *reinterpret_cast<const fvec*>(&part_o[(base + sc) * head_dim + lane * kPer]);
      wt[j] = s < nsplit ? wts[sc] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kInFlight; ++j)
#pragma unroll
      for (int e = 0; e < kPer; ++e) acc[e] += v[j][e] * wt[j];  // fixed order: the result is deterministic
  }
#pragma unroll
  for (int e = 0; e < kPer; ++e) red[wave][lane * kPer + e] = acc[e];
  __syncthreads();
  if ((int)threadIdx.x < head_dim) {
    float a = 0.f;
#pragma unroll
    for (int v = 0; v < kPaMergeWaves; ++v) a += red[v][threadIdx.x];
    o[out + threadIdx.x] = (f16)(lsum > 0.f ? a / lsum : 0.f);
  }
}

// Arguments of a launch of the main kernels.
struct PaCall {
  const f16 *q, *kc, *vc;
  const int32_t *bt, *cl;
  f16* o;
  float *part_o, *part_ml;
  int32_t* ints;  // int area behind the partial results: length order or plan
  int bs, head_dim;
  PaGeom ge;
  PaChunking ch;
  hipStream_t s;
};

// Query-head sub-groups of 16 a workgroup serves: K and V stay in registers across them, so their number is
// bounded by the registers the accumulators of a sub-group take.
static int pa_subgroups(int64_t head_dim, int64_t group) {
  const int64_t fit = head_dim <= 128 ? 2 : 1;
  const int64_t want = (group + kPaMaxGroup - 1) / kPaMaxGroup;
  return (int)(want < fit ? want : fit);
}

static size_t pa_lds_bytes(int q_halfs, int merge_heads, int head_dim, int64_t bs, bool balanced) {
  return (size_t)q_halfs * sizeof(f16) + (size_t)kPaWaves * merge_heads * kPaLdsPerHead(head_dim) * sizeof(float) +
         (balanced ? pa_block_plan_ints(bs) * sizeof(int) : 0);
}

// Heads per pass of the cross-wave merge: as many of a sub-group's as keep the workgroup's LDS within 64 KiB,
// in passes of equal size.
static int pa_merge_heads(int q_halfs, int head_dim, int heads, int64_t bs, bool balanced) {
  const int sub = heads < kPaMaxGroup ? heads : kPaMaxGroup;
  const int64_t budget = 64 * 1024 - (int64_t)q_halfs * (int64_t)sizeof(f16) -
                         (int64_t)(balanced ? pa_block_plan_ints(bs) * sizeof(int) : 0);
  int64_t cap = budget / (int64_t)(kPaWaves * kPaLdsPerHead(head_dim) * sizeof(float));
  if (cap < 1) cap = 1;
  if (cap > sub) cap = sub;
  const int passes = (int)((sub + cap - 1) / cap);
  return (sub + passes - 1) / passes;
}

template <int D, int NSUB>
static void pa_launch(PaCall c) {
  constexpr int kQHalfs = pa_q_lds_halfs<D, NSUB>();
  const bool balanced = c.ch.balanced_wgs > 0;
  c.ge.merge_heads = pa_merge_heads(kQHalfs, D, c.ge.wg_heads < c.ge.group ? c.ge.wg_heads : c.ge.group, c.bs, balanced);
  const size_t lds = pa_lds_bytes(kQHalfs, c.ge.merge_heads, D, c.bs, balanced);
  const unsigned kv_wgs = (unsigned)(c.ge.num_kv_heads * c.ge.virt);
  const int max_len = c.ge.max_blocks_per_seq * c.ge.block_size;
  auto merge = [&](const int32_t* plan) {
    dim3 mgrid((unsigned)c.ge.num_heads, (unsigned)c.bs);
    auto kernel = D <= 64 ? pa_decode_merge<1> : D <= 128 ? pa_decode_merge<2> : pa_decode_merge<4>;
    kernel<<<mgrid, kPaMergeWaves * kWave, 0, c.s>>>(c.part_o, c.part_ml, c.cl, c.o, D, c.ge.num_heads,
                                                     c.ch.chunk_tokens, c.ch.max_splits, c.ch.balanced_wgs, c.bs,
                                                     max_len, plan);
  };
  if (balanced) {
    int32_t* plan = c.bs > kWave ? c.ints : nullptr;
    dim3 bgrid((unsigned)c.ch.balanced_wgs, kv_wgs);
    pa_decode_balanced<D, NSUB><<<bgrid, kPaWaves * kWave, lds, c.s>>>(c.q, c.kc, c.vc, c.bt, c.cl, c.part_o,
                                                                        c.part_ml, c.o, c.bs, c.ge, plan);
    merge(plan);
    return;
  }
  dim3 grid((unsigned)c.ch.max_splits, kv_wgs, (unsigned)c.bs);
  int32_t* order = (c.bs <= kWave || c.bs > kPaRankMax) ? nullptr : c.ints;  // ranked inside the kernel / not at all
  if (order) pa_rank_sequences<<<1, kPaRankMax, 0, c.s>>>(c.cl, c.bs, order);
  pa_decode_partial<D, NSUB><<<grid, kPaWaves * kWave, lds, c.s>>>(c.q, c.kc, c.vc, c.bt, c.cl, c.part_o, c.part_ml,
                                                                   c.o, c.ge, c.ch.chunk_tokens, order);
  if (c.ch.max_splits > 1) merge(nullptr);
}

// Generic path for page sizes that are not a multiple of 16 tokens (head_dim a multiple of 16 up to 256, any
// whole number of query heads per kv head): one workgroup of eight waves per (sequence, query head).
// A wave takes every eighth block of 32 tokens; lane (token = lane / 2, half = lane % 2) loads, d-chunk
// row by d-chunk row, the 16 bytes that hold d = 16c + 8*half ..+7 of its token, so that a load
// instruction of a wave covers 1 KiB of consecutive tokens of one d-chunk row (tokens of one page are
// adjacent in the layout).  Scores are finished with one exchange between the two lanes of a token, the
// block's softmax with wave reductions; every lane accumulates p * V for its own token and half, and the
// 32 tokens are added up with lane exchanges once per wave at the end.  The eight waves meet in LDS.
// Workgroups are renumbered so that the query heads of one kv head, which read the same K and V, run on
// one XCD side by side and share its L2.  CH = number of d-chunk rows the registers are sized for.
constexpr int kPaGenericMaxD = 256;
// eight waves where a wave's registers allow two waves per SIMD (head_dim <= 128), four otherwise
constexpr int pa_generic_waves(int ch) { return ch <= 8 ? 8 : 4; }

template <int CH>
__global__ __launch_bounds__(pa_generic_waves(CH) * kWave) void pa_decode_generic(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, f16* __restrict__ out, int bs, int num_heads,
    int num_kv_heads, int head_dim, int block_size, int max_blocks_per_seq, float scale_log2,
    int num_blocks) {
  constexpr int kPaGenericWaves = pa_generic_waves(CH);
  // XCD x takes the contiguous range [x * share, (x + 1) * share) of the (sequence, head) pairs
  const int total = bs * num_heads;
  const int share = (total + kPaXcds - 1) / kPaXcds;
  const int item = (int)(blockIdx.x % kPaXcds) * share + (int)(blockIdx.x / kPaXcds);
  if ((int)(blockIdx.x / kPaXcds) >= share || item >= total) return;
  const int b = item / num_heads;
  const int h = item - b * num_heads;
  const int g = h / (num_heads / num_kv_heads);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int tok = lane >> 1;
  const int half = lane & 1;
  const int chunks = head_dim / 16;
  const int context_len = min(context_lens[b], max_blocks_per_seq * block_size);
  const int64_t row_chunks = (int64_t)num_kv_heads * chunks;  // 32-byte granules per token
  const int32_t* table = block_tables + (int64_t)b * max_blocks_per_seq;

  f16x8 qv[CH];
  float acc[CH][8];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    qv[c] = c < chunks ? ld128(q + ((int64_t)b * num_heads + h) * head_dim + 16 * c + 8 * half) : zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[c][e] = 0.f;
  }
  float m = kNegBig, l = 0.f;  // running maximum (wave uniform) and this lane's share of the sum
  const int64_t chunk_stride = (int64_t)block_size * 16;
  // (token of this lane in the block that starts at j0) -> is it inside the context, and where its row starts:
  // offset of (token, kv head g, d-chunk row 0, this lane's half).  Dead lanes read a valid token and are masked.
  auto locate = [&](int j0, bool& live) -> int64_t {
    const int j = j0 + tok;
    live = j < context_len;
    const int jc = live ? j : context_len - 1;
    const int blk = jc / block_size;
    const int64_t page = min(max(table[blk], 0), num_blocks - 1);
    return ((page * row_chunks + (int64_t)g * chunks) * block_size + (jc - blk * block_size)) * 16 + 8 * half;
  };
  // K of a block is fetched while the block before it is being worked on (the wave's own blocks are its only
  // source of memory parallelism, one wave per SIMD at most): with the registers for it (head_dim <= 128) the
  // loop holds K of the next block and V of this one in flight together.
  constexpr bool kPrefetch = CH <= 8;
  constexpr int kStep = kPaGenericWaves * 32;
  f16x8 kk[CH], vv[kPrefetch ? CH : 1];
  bool live_next = false;
  int64_t base_next = 0;
  if (wave * 32 < context_len) {
    base_next = locate(wave * 32, live_next);
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (c < chunks) kk[c] = ld128_stream(key_cache + base_next + c * chunk_stride);
  }
  for (int j0 = wave * 32; j0 < context_len; j0 += kStep) {
    const bool live = live_next;
    const int64_t base = base_next;
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (c < chunks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) part += (float)qv[c][e] * (float)kk[c][e];
      }
    // V of this block; then, K of the wave's next block into the registers the scores have just freed
    auto load_v = [&](auto& dst) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
        if (c < chunks) dst[c] = ld128_stream(value_cache + base + c * chunk_stride);
    };
    auto load_next_k = [&] {
      if (j0 + kStep < context_len) {
        base_next = locate(j0 + kStep, live_next);
#pragma unroll
        for (int c = 0; c < CH; ++c)
          if (c < chunks) kk[c] = ld128_stream(key_cache + base_next + c * chunk_stride);
      }
    };
    if constexpr (kPrefetch) {
      load_v(vv);
      load_next_k();
    } else {
      load_v(kk);
    }
    part += __shfl_xor(part, 1);
    const float sc = live ? part * scale_log2 : -__builtin_inff();
    float mx = sc;
#pragma unroll
    for (int d = 2; d < kWave; d <<= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
    const float m_new = fmaxf(m, mx);  // finite: token j0 of the block is live
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    const float p = live ? __builtin_amdgcn_exp2f(sc - m_new) : 0.f;
    m = m_new;
    l = l * alpha + p;
    auto add_pv = [&](const auto& src) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
        if (c < chunks) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            // cache contents of dead tokens are arbitrary (possibly NaN): they must not reach the sum
            const float v = live ? (float)src[c][e] : 0.f;
            acc[c][e] = acc[c][e] * alpha + p * v;
          }
        }
    };
    if constexpr (kPrefetch) {
      add_pv(vv);
    } else {
      add_pv(kk);
      load_next_k();
    }
  }
  // add up the 32 tokens of the wave (lanes with the same half), then the waves
  __shared__ float sm_acc[kPaGenericWaves][kPaGenericMaxD];
  __shared__ float sm_m[kPaGenericWaves], sm_l[kPaGenericWaves];
#pragma unroll
  for (int d = 2; d < kWave; d <<= 1) l += __shfl_xor(l, d);
#pragma unroll
  for (int c = 0; c < CH; ++c)
    if (c < chunks) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = acc[c][e];
#pragma unroll
        for (int d = 2; d < kWave; d <<= 1) v += __shfl_xor(v, d);
        if (tok == 0) sm_acc[wave][16 * c + 8 * half + e] = v;
      }
    }
  if (lane == 0) {
    sm_m[wave] = m;
    sm_l[wave] = l;
  }
  __syncthreads();
  for (int d = threadIdx.x; d < head_dim; d += kPaGenericWaves * kWave) {
    float mx = sm_m[0];
#pragma unroll
    for (int w = 1; w < kPaGenericWaves; ++w) mx = fmaxf(mx, sm_m[w]);
    float lsum = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < kPaGenericWaves; ++w) {
      const float wt = __builtin_amdgcn_exp2f(sm_m[w] - mx);
      lsum += sm_l[w] * wt;
      a += sm_acc[w][d] * wt;
    }
    out[((int64_t)b * num_heads + h) * head_dim + d] = (f16)(lsum > 0.f ? a / lsum : 0.f);
  }
}

static bool pa_args_valid(int64_t bs, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                          int64_t block_size, int64_t max_blocks_per_seq) {
  if (bs < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_blocks_per_seq < 0) return false;
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > kPaGenericMaxD) return false;
  if (block_size <= 0 || num_heads % num_kv_heads != 0) return false;
  if (bs > 65535 || num_kv_heads > 65535 || num_heads > 0x7fffffff / kPaGenericMaxD) return false;
  if (block_size * max_blocks_per_seq > 0x7fffffff) return false;
  return true;
}

// Shapes served by the matrix-core kernels: every head_dim the operator admits, any number of query heads
// per kv head, pages of a multiple of 16 tokens (a 16-token group of a step never straddles two pages).
// Other page sizes take the generic kernel.
static bool pa_fast_shape(int64_t block_size) { return block_size % 16 == 0; }

// Workgroups per kv head (a workgroup serves at most 16 * pa_subgroups query heads of it).
static int64_t pa_virtual_heads(int64_t head_dim, int64_t group) {
  const int64_t per_wg = (int64_t)kPaMaxGroup * pa_subgroups(head_dim, group);
  return (group + per_wg - 1) / per_wg;
}

}  // namespace aops

extern "C" size_t aops_paged_attention_workspace(int64_t bs, int64_t num_heads,
                                                 int64_t num_kv_heads, int64_t head_dim,
                                                 int64_t block_size, int64_t max_blocks_per_seq) {
  using namespace aops;
  if (!pa_args_valid(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq))
    return 0;
  if (!pa_fast_shape(block_size)) return 16;  // not used
  const PaChunking ch = pa_chunking(bs, num_kv_heads * pa_virtual_heads(head_dim, num_heads / num_kv_heads),
                                    block_size, max_blocks_per_seq);
  // partial results, then the ints of the length order or of the balanced partition's plan
  return (size_t)bs * (size_t)num_heads * (size_t)ch.max_splits * (size_t)(head_dim + 2) * sizeof(float) +
         pa_tail_ints(bs) * sizeof(int32_t);
}

namespace aops {

// The work of both entry points: argument checks, kernel choice, launches.  `workspace` is device
// memory of at least aops_paged_attention_workspace(...) bytes (not touched by the generic kernel).
static int pa_run(const void* q, const void* key_cache, const void* value_cache,
                  const int32_t* block_tables, const int32_t* context_lens, void* o, void* workspace,
                  size_t workspace_bytes, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
                  int64_t head_dim, int64_t block_size, int64_t max_blocks_per_seq,
                  int64_t num_blocks, void* stream) {
  if (!pa_args_valid(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq) ||
      num_blocks < 0 || num_blocks > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AOPS_OK;
  if (num_blocks == 0) return AOPS_ERR_INVALID_ARGUMENT;  // sequences but no cache to read
  if (!q || !key_cache || !value_cache || !block_tables || !context_lens || !o)
    return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const f16* qp = static_cast<const f16*>(q);
  const f16* kc = static_cast<const f16*>(key_cache);
  const f16* vc = static_cast<const f16*>(value_cache);
  f16* op = static_cast<f16*>(o);
  if (!pa_fast_shape(block_size)) {
    const float scale_log2 = kLog2e / __builtin_sqrtf((float)head_dim);
    const int64_t total = bs * num_heads;
    const int64_t grid = (total + kPaXcds - 1) / kPaXcds * kPaXcds;
    if (grid > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
    const int ch = head_dim <= 64 ? 4 : head_dim <= 128 ? 8 : 16;  // d-chunk rows the registers are sized for
    auto kernel = ch == 4 ? pa_decode_generic<4> : ch == 8 ? pa_decode_generic<8> : pa_decode_generic<16>;
    const int waves = pa_generic_waves(ch);
    kernel<<<(unsigned)grid, waves * kWave, 0, s>>>(qp, kc, vc, block_tables, context_lens, op, (int)bs,
                                                             (int)num_heads, (int)num_kv_heads, (int)head_dim,
                                                             (int)block_size, (int)max_blocks_per_seq, scale_log2,
                                                             (int)num_blocks);
    return record_launch_status(hipGetLastError());
  }
  const size_t need = aops_paged_attention_workspace(bs, num_heads, num_kv_heads, head_dim,
                                                     block_size, max_blocks_per_seq);
  if (!workspace || workspace_bytes < need) return AOPS_ERR_WORKSPACE;
  const int64_t group = num_heads / num_kv_heads;
  const int nsub = pa_subgroups(head_dim, group);
  const int64_t virt = pa_virtual_heads(head_dim, group);
  if (num_kv_heads * virt > 65535) return AOPS_ERR_INVALID_ARGUMENT;  // grid dimension
  PaCall c;
  c.ch = pa_chunking(bs, num_kv_heads * virt, block_size, max_blocks_per_seq);
  c.q = qp;
  c.kc = kc;
  c.vc = vc;
  c.bt = block_tables;
  c.cl = context_lens;
  c.o = op;
  c.part_o = static_cast<float*>(workspace);
  c.part_ml = c.part_o + (size_t)bs * num_heads * c.ch.max_splits * head_dim;
  c.ints = reinterpret_cast<int32_t*>(c.part_ml + (size_t)bs * num_heads * c.ch.max_splits * 2);
  c.bs = (int)bs;
  c.head_dim = (int)head_dim;
  c.s = s;
  c.ge.num_heads = (int)num_heads;
  c.ge.num_kv_heads = (int)num_kv_heads;
  c.ge.block_size = (int)block_size;
  c.ge.max_blocks_per_seq = (int)max_blocks_per_seq;
  c.ge.max_splits = c.ch.max_splits;
  c.ge.num_blocks = (int)num_blocks;
  c.ge.group = (int)group;
  c.ge.wg_heads = kPaMaxGroup * nsub;
  c.ge.virt = (int)virt;
  c.ge.merge_heads = 0;  // set by pa_launch
  c.ge.scale_log2 = kLog2e / __builtin_sqrtf((float)head_dim);
#define AOPS_PA_CASE(D)                      \
  case D / 16:                               \
    if constexpr (D <= 128) {                \
      if (nsub == 2) {                       \
        pa_launch<D, 2>(c);                  \
        break;                               \
      }                                      \
    }                                        \
    pa_launch<D, 1>(c);                      \
    break;
  switch (head_dim / 16) {
    AOPS_PA_CASE(16)
    AOPS_PA_CASE(32)
    AOPS_PA_CASE(48)
    AOPS_PA_CASE(64)
    AOPS_PA_CASE(80)
    AOPS_PA_CASE(96)
    AOPS_PA_CASE(112)
    AOPS_PA_CASE(128)
    AOPS_PA_CASE(144)
    AOPS_PA_CASE(160)
    AOPS_PA_CASE(176)
    AOPS_PA_CASE(192)
    AOPS_PA_CASE(208)
    AOPS_PA_CASE(224)
    AOPS_PA_CASE(240)
    AOPS_PA_CASE(256)
    default:
      return AOPS_ERR_INVALID_ARGUMENT;  // pa_args_valid admits no other head_dim
  }
#undef AOPS_PA_CASE
  return record_launch_status(hipGetLastError());
}

// Scratch of the entry point that allocates nothing: the partial results and the int area of the
// split-KV kernels live in this array of the library's device image instead of a caller's workspace.
// Every GPU the library runs on holds its own copy at its own address until the process ends.
static __device__ __align__(256) unsigned char pa_static_scratch[AOPS_PA_NOALLOC_SCRATCH_BYTES];

constexpr int kPaMaxDevices = 64;
static std::mutex pa_scratch_mutex;
static void* pa_scratch_addr[kPaMaxDevices];  // device address of pa_static_scratch per device, null = not looked up

// Address of the current device's copy of the array.  In host code the array's name is only a handle
// for hipGetSymbolAddress, never a device address.
static int pa_scratch_for_current_device(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return record_launch_status(e);
  if (dev < 0 || dev >= kPaMaxDevices) return AOPS_ERR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(pa_scratch_mutex);
  if (!pa_scratch_addr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(pa_static_scratch));
    if (e != hipSuccess) return record_launch_status(e);
    if (!p) return AOPS_ERR_LAUNCH;
    pa_scratch_addr[dev] = p;
  }
  *out = pa_scratch_addr[dev];
  return AOPS_OK;
}

}  // namespace aops

extern "C" int aops_paged_attention_f16(const void* q, const void* key_cache,
                                        const void* value_cache, const int32_t* block_tables,
                                        const int32_t* context_lens, void* o, void* workspace,
                                        size_t workspace_bytes, int64_t bs, int64_t num_heads,
                                        int64_t num_kv_heads, int64_t head_dim,
                                        int64_t block_size, int64_t max_blocks_per_seq,
                                        int64_t num_blocks, void* stream) {
  return aops::pa_run(q, key_cache, value_cache, block_tables, context_lens, o, workspace,
                      workspace_bytes, bs, num_heads, num_kv_heads, head_dim, block_size,
                      max_blocks_per_seq, num_blocks, stream);
}

extern "C" int aops_paged_attention_noalloc_f16(const void* q, const void* key_cache,
                                                const void* value_cache,
                                                const int32_t* block_tables,
                                                const int32_t* context_lens, void* o, int64_t bs,
                                                int64_t num_heads, int64_t num_kv_heads,
                                                int64_t head_dim, int64_t block_size,
                                                int64_t max_blocks_per_seq, int64_t num_blocks,
                                                void* stream) {
  using namespace aops;
  if (!pa_args_valid(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq))
    return AOPS_ERR_INVALID_ARGUMENT;
  // the size test comes first: a problem beyond the fixed maximum is refused whatever else is wrong
  if (aops_paged_attention_workspace(bs, num_heads, num_kv_heads, head_dim, block_size,
                                     max_blocks_per_seq) > (size_t)AOPS_PA_NOALLOC_SCRATCH_BYTES)
    return AOPS_ERR_SCRATCH_LIMIT;
  if (bs == 0) return AOPS_OK;
  if (!q || !key_cache || !value_cache || !block_tables || !context_lens || !o)
    return AOPS_ERR_INVALID_ARGUMENT;
  void* scratch = nullptr;
  const int rc = pa_scratch_for_current_device(&scratch);
  if (rc != AOPS_OK) return rc;
  // Nothing in the scratch has to start at zero: every partial result, plan entry and rank the
  // kernels read in a call was written by an earlier kernel of the same call.
  return pa_run(q, key_cache, value_cache, block_tables, context_lens, o, scratch,
                (size_t)AOPS_PA_NOALLOC_SCRATCH_BYTES, bs, num_heads, num_kv_heads, head_dim,
                block_size, max_blocks_per_seq, num_blocks, stream);
}
