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
// Main kernel (head_dim 64, 128 or 256; described for 128), one step = 32 tokens of one kv head =
// 8 KiB of K + 8 KiB of V:
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
constexpr int kPaMaxGroup = 16;              // query heads per kv head the matrix-core kernel serves
constexpr int kPaXcds = 8;                   // workgroup i runs on XCD i % 8

// Batches of up to kPaPlanMax sequences can use the balanced partition; above 64 sequences it is
// computed by a one-workgroup kernel into kPaPlanInts(bs) ints behind the partial results.
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

// Per-lane slice of a 32-token tile: [token group][s] holds X[token 16t + n][d = 32s + 8kg ..+7],
// s = 0 .. NS-1 with NS = head_dim / 32.
template <int NS>
using PaRegs = f16x8[2][NS];

template <int NS>
__device__ __forceinline__ void pa_issue_loads(const f16* __restrict__ cache, int64_t off0, int64_t off1,
                                               uint32_t lane_off, uint32_t s_stride, PaRegs<NS>& r) {
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const f16* base = cache + (g == 0 ? off0 : off1) + lane_off;  // token group g of the step
#pragma unroll
    for (int s = 0; s < NS; ++s) r[g][s] = ld128_stream(base + s * s_stride);
  }
}

template <int NS>
struct PaState {
  f32x4 o[2 * NS];  // O^T blocks: lane (head n, kg), o[db][i] <-> d = 16 db + 4 kg + i
  float m;     // running maximum of head n (identical in the four lanes of a head)
  float l;     // this lane's share of the running sum
};

// S^T[token][head] = K . Q^T, scaled to log2 units; lane (head n, kg) gets tokens
// 16*(e/4) + 4kg + e%4, e = 0..7, of the step.
// QLDS: the Q^T fragments are read from LDS (q_lds = this lane's slice, fragment s 512 halfs further)
// instead of being held in registers: at head_dim 256 they would push the kernel into scratch.
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
template <int NS>
__device__ __forceinline__ f16x8 pa_softmax(float (&sc)[8], PaState<NS>& st) {
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
    for (int db = 0; db < 2 * NS; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) st.o[db][i] *= alpha;
  }
  return pt;
}

// O^T += V^T . P^T with V transposed on the matrix core.
template <int NS>
__device__ __forceinline__ void pa_accumulate(const PaRegs<NS>& v, const f16x8 (&sel)[2], f16x8 pt,
                                              PaState<NS>& st) {
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < NS; ++s) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      // [token][d = 32s + 16u + n]: lane (n, kg) receives tokens 4kg..4kg+3 of each group
      const f32x4 x0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(v[0][s], sel[u], zero4, 0, 0, 0);
      const f32x4 x1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(v[1][s], sel[u], zero4, 0, 0, 0);
      f16x8 vt;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vt[i] = (f16)x0[i];
        vt[4 + i] = (f16)x1[i];
      }
      st.o[2 * s + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vt, pt, st.o[2 * s + u], 0, 0, 0);
    }
  }
}

// One chunk of one (sequence b, kv head g): tokens chunk_start .. chunk_start + chunk_len - 1, the
// steps dealt round robin to the eight waves, which are merged through LDS at the end.  `group` =
// query heads per kv head, GMAX = the power of two it is rounded up to (<= 16; sizes the LDS
// arrays).  FINAL: the chunk is the whole sequence, so the normalised output is written directly;
// otherwise the partial result goes to slot `split` of the (sequence, head)'s max_splits slots.
// Called by all threads of the workgroup with uniform arguments.
template <int D, int GMAX, bool FINAL>
__device__ __forceinline__ void pa_process_chunk(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    float* __restrict__ part_o, float* __restrict__ part_ml, f16* __restrict__ out, int b, int g,
    int context_len, int chunk_start, int chunk_len, int split, int num_kv_heads, int block_size,
    int max_blocks_per_seq, int max_splits, float scale_log2, int num_blocks, int group) {
  constexpr int kPaD = D;
  constexpr int NS = D / 32;
  const int nsteps = (chunk_len + kPaStep - 1) / kPaStep;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int n = lane & 15;
  const int kg = lane >> 4;
  const int num_heads = num_kv_heads * group;

  // Q^T operand: lane (head n, kg) holds q[head n][32s + 8kg ..+7]; heads >= group are zero rows.
  constexpr bool QLDS = NS > 4;
  f16x8 qreg[QLDS ? 1 : NS];
  __shared__ __attribute__((aligned(16))) f16 sm_q[QLDS ? NS * kWave * 8 : 8];
  const f16* q_lds = sm_q + lane * 8;
  {
    const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const f16* qp = q + ((int64_t)b * num_heads + g * group + (n < group ? n : 0)) * kPaD + 8 * kg;
    if constexpr (QLDS) {  // every wave uses the same fragments: wave 0 fetches them
      if (wave == 0) {
#pragma unroll
        for (int s = 0; s < NS; ++s)
          *reinterpret_cast<f16x8*>(sm_q + (s * kWave + lane) * 8) = n < group ? ld128(qp + 32 * s) : zero8;
      }
      __syncthreads();
    } else {
#pragma unroll
      for (int s = 0; s < NS; ++s) qreg[s] = n < group ? ld128(qp + 32 * s) : zero8;
    }
  }
  // Selector operands of the transposing product: sel[u][k][n] = (k == n + 16u), k = 8kg + e.
  f16x8 sel[2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int e = 0; e < 8; ++e) sel[u][e] = (8 * kg + e == n + 16 * u) ? (f16)1.0f : (f16)0.0f;

  PaState<NS> st;
#pragma unroll
  for (int db = 0; db < 2 * NS; ++db) st.o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m = kNegBig;
  st.l = 0.f;

  // Element offsets inside one page for this lane: d-chunk rows are block_size*16 halfs apart
  // (this lane starts in row kg/2), the two halves of a granule 8 halfs, tokens 16 halfs.
  const uint32_t lane_off = (uint32_t)(kg >> 1) * (uint32_t)block_size * 16u +
                            (uint32_t)(kg & 1) * 8u + (uint32_t)n * 16u;
  const uint32_t s_stride = 2u * (uint32_t)block_size * 16u;  // 32 d further = two d-chunk rows
  const int64_t page_elems = (int64_t)num_kv_heads * kPaD * block_size;
  const int64_t head_off = (int64_t)g * kPaD * block_size;
  const int32_t* table = block_tables + (int64_t)b * max_blocks_per_seq;

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
    float sc[8];
    pa_scores<NS, QLDS>(kreg, qreg, q_lds, scale_log2, sc);
    if (has_next) pa_issue_loads(key_cache, next_off0, next_off1, lane_off, s_stride, kreg);
    if (step_token0 + kPaStep > context_len) {  // wave uniform: last, partial step of the sequence
      // Cache contents past the end of the sequence are arbitrary (possibly NaN): drop their
      // scores and zero their V rows before they reach the matrix core.
      const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (step_token0 + 16 * g + 4 * kg + i >= context_len) sc[4 * g + i] = -__builtin_inff();
        if (step_token0 + 16 * g + n >= context_len) {
#pragma unroll
          for (int s = 0; s < NS; ++s) vreg[g][s] = zero8;
        }
      }
    }
    const f16x8 pt = pa_softmax(sc, st);
    pa_accumulate(vreg, sel, pt, st);
    if (has_next) pa_issue_loads(value_cache, next_off0, next_off1, lane_off, s_stride, vreg);
  };
  auto first_loads = [&](PaRegs<NS>& kreg, PaRegs<NS>& vreg, int step) {
    if (step < nsteps) {
      const int64_t off0 = page_offset(step, 0), off1 = page_offset(step, 1);
      pa_issue_loads(key_cache, off0, off1, lane_off, s_stride, kreg);
      pa_issue_loads(value_cache, off0, off1, lane_off, s_stride, vreg);
    }
  };
  // (A second register set, with the step after next in flight as well, was tried up to head_dim
  // 128: no gain where it fits, and scratch use in the balanced kernel.)
  PaRegs<NS> kreg, vreg;
  first_loads(kreg, vreg, wave);
  for (int step = wave; step < nsteps; step += kPaWaves) do_step(kreg, vreg, step, kPaWaves);

  // The four lanes of a head hold disjoint shares of the sum.
  float l_head = st.l;
  l_head += __shfl_xor(l_head, 16);
  l_head += __shfl_xor(l_head, 32);

  // Merge the waves of the workgroup through LDS and emit one partial per query head.
  __shared__ float sm_acc[kPaWaves][GMAX][kPaD];
  __shared__ float sm_m[kPaWaves][GMAX];
  __shared__ float sm_l[kPaWaves][GMAX];
  if (n < group) {
#pragma unroll
    for (int db = 0; db < 2 * NS; ++db)
      *reinterpret_cast<f32x4*>(&sm_acc[wave][n][16 * db + 4 * kg]) = st.o[db];
    if (kg == 0) {
      sm_m[wave][n] = st.m;
      sm_l[wave][n] = l_head;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < group * kPaD; e += kPaWaves * kWave) {
    const int h = e / kPaD;
    const int d = e - h * kPaD;
    float mx = sm_m[0][h];
#pragma unroll
    for (int w = 1; w < kPaWaves; ++w) mx = fmaxf(mx, sm_m[w][h]);
    float lsum = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < kPaWaves; ++w) {
      const float wt = __builtin_amdgcn_exp2f(sm_m[w][h] - mx);
      lsum += sm_l[w][h] * wt;
      a += sm_acc[w][h][d] * wt;
    }
    if (FINAL) {
      out[((int64_t)b * num_heads + g * group + h) * kPaD + d] = (f16)(lsum > 0.f ? a / lsum : 0.f);
    } else {
      const int64_t slot = ((int64_t)b * num_heads + g * group + h) * max_splits + split;
      part_o[slot * kPaD + d] = a;
      if (d == 0) {
        part_ml[slot * 2 + 0] = mx;
        part_ml[slot * 2 + 1] = lsum;
      }
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

// grid = (max_splits, Hkv, bs), block = 8 waves: one chunk of chunk_tokens tokens per workgroup.
template <int D, int GMAX, bool FINAL>
__global__ __launch_bounds__(kPaWaves* kWave) void pa_decode_partial(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, float* __restrict__ part_o,
    float* __restrict__ part_ml, f16* __restrict__ out, int num_kv_heads, int block_size, int max_blocks_per_seq,
    int chunk_tokens, int max_splits, float scale_log2, int num_blocks, int group,
    const int32_t* __restrict__ order) {
  const int split = blockIdx.x;
  const int g = blockIdx.y;
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
  const int context_len = min(context_lens[b], max_blocks_per_seq * block_size);
  const int chunk_start = split * chunk_tokens;
  if (chunk_start >= context_len) {
    if (FINAL) {  // empty sequence: zeros
      for (int e = threadIdx.x; e < group * D; e += kPaWaves * kWave)
        out[((int64_t)b * num_kv_heads * group + g * group) * D + e] = (f16)0.f;
    }
    return;
  }
  pa_process_chunk<D, GMAX, FINAL>(q, key_cache, value_cache, block_tables, part_o, part_ml, out, b, g,
                                   context_len, chunk_start, min(context_len - chunk_start, chunk_tokens),
                                   split, num_kv_heads, block_size, max_blocks_per_seq, max_splits,
                                   scale_log2, num_blocks, group);
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

// The same partition for batches of more than 64 sequences, computed once by one workgroup into
//   plan[0] = total units, plan[1 + b] = units in front of sequence b, plan[1 + bs + b] = its clamped
//   length, plan[1 + 2*bs + w] = the sequence that holds the first unit of share w.
constexpr int kPaPlanThreads = 1024;

__global__ __launch_bounds__(kPaPlanThreads) void pa_plan_kernel(const int32_t* __restrict__ context_lens,
                                                                 int bs, int max_len, int wgs_max,
                                                                 int32_t* __restrict__ plan) {
  __shared__ int wave_sum[kPaPlanThreads / kWave];
  __shared__ int carry_s;
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  if (t == 0) carry_s = 0;
  __syncthreads();
  for (int b0 = 0; b0 < bs; b0 += kPaPlanThreads) {
    const int b = b0 + t;
    const int len = b < bs ? min(max(context_lens[b], 0), max_len) : 0;
    const int units = (len + kPaUnit - 1) / kPaUnit;
    int incl = units;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry_s + incl - units;
    for (int v = 0; v < wave; ++v) before += wave_sum[v];
    if (b < bs) {
      plan[1 + b] = before;
      plan[1 + bs + b] = len;
    }
    __syncthreads();
    if (t == kPaPlanThreads - 1) carry_s = before + units;
    __syncthreads();
  }
  const int total = carry_s;
  if (t == 0) plan[0] = total;
  if (total == 0) return;
  // every sequence names itself as the start of the shares whose first unit it holds
  const int wgs = min(wgs_max, total);
  for (int b = t; b < bs; b += kPaPlanThreads) {
    const int before = plan[1 + b];  // written by this thread
    const int units = (plan[1 + bs + b] + kPaUnit - 1) / kPaUnit;
    if (units == 0) continue;
    // shares w with before <= floor(w * total / wgs) < before + units
    int w = (int)(((int64_t)before * wgs + total - 1) / total);
    for (; w < wgs && (int)((int64_t)w * total / wgs) < before + units; ++w) plan[1 + 2 * bs + w] = b;
  }
}

// grid = (wgs, Hkv), block = 8 waves.  Workgroup w walks through its share of the batch's units,
// sequence by sequence; the part of sequence b it covers becomes partial result number
// w - (share holding b's first unit) of that sequence.  plan == nullptr: at most 64 sequences, the
// partition is computed by every wave (pa_units); otherwise it is read from pa_plan_kernel's output.
template <int D, int GMAX>
__global__ __launch_bounds__(kPaWaves* kWave) void pa_decode_balanced(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, float* __restrict__ part_o,
    float* __restrict__ part_ml, int bs, int num_kv_heads, int block_size, int max_blocks_per_seq,
    int max_splits, float scale_log2, int num_blocks, int group, const int32_t* __restrict__ plan) {
  const int w = blockIdx.x;
  const int g = blockIdx.y;
  if (plan) {
    const int total = plan[0];
    const int wgs = min((int)gridDim.x, total);
    if (w >= wgs) return;
    const int lo = (int)((int64_t)w * total / wgs);
    const int hi = (int)((int64_t)(w + 1) * total / wgs);
    int cur = lo;
    int b = plan[1 + 2 * bs + w];
    while (cur < hi && b < bs) {
      const int before = plan[1 + b];
      const int len = plan[1 + bs + b];
      const int units = (len + kPaUnit - 1) / kPaUnit;
      if (units > 0) {
        const int seg_end = min(hi, before + units);
        const int tok0 = (cur - before) * kPaUnit;
        const int tok1 = min((seg_end - before) * kPaUnit, len);
        const int slot = w - pa_share_of(before, wgs, total);
        pa_process_chunk<D, GMAX, false>(q, key_cache, value_cache, block_tables, part_o, part_ml, nullptr, b, g,
                                         len, tok0, tok1 - tok0, slot, num_kv_heads, block_size,
                                         max_blocks_per_seq, max_splits, scale_log2, num_blocks, group);
        cur = seg_end;
        if (cur < hi) __syncthreads();  // the LDS arrays of the chunk are reused
      }
      ++b;
    }
    return;
  }
  const PaUnits pu = pa_units(context_lens, bs, max_blocks_per_seq * block_size);
  // no more shares than units: every share then holds at least one unit, and the shares of a
  // sequence are consecutive
  const int wgs = min((int)gridDim.x, pu.total);
  if (w >= wgs) return;
  const int lo = (int)((int64_t)w * pu.total / wgs);
  const int hi = (int)((int64_t)(w + 1) * pu.total / wgs);
  int cur = lo;
  while (cur < hi) {
    // the sequence that holds unit cur (exactly one lane)
    const uint64_t hit = __ballot(pu.units > 0 && pu.before <= cur && cur < pu.before + pu.units);
    if (hit == 0) break;  // cannot happen: the units of the sequences tile [0, total)
    const int b = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit));
    const int before = __builtin_amdgcn_readlane(pu.before, b);
    const int units = __builtin_amdgcn_readlane(pu.units, b);
    const int len = __builtin_amdgcn_readlane(pu.len, b);
    const int seg_end = min(hi, before + units);
    const int tok0 = (cur - before) * kPaUnit;
    const int tok1 = min((seg_end - before) * kPaUnit, len);
    const int slot = w - pa_share_of(before, wgs, pu.total);
    pa_process_chunk<D, GMAX, false>(q, key_cache, value_cache, block_tables, part_o, part_ml, nullptr, b, g,
                                     len, tok0, tok1 - tok0, slot, num_kv_heads, block_size,
                                     max_blocks_per_seq, max_splits, scale_log2, num_blocks, group);
    cur = seg_end;
    if (cur < hi) __syncthreads();  // the LDS arrays of the chunk are reused
  }
}

// grid = (Hq, bs), block = 4 waves.  Every wave works out the weights 2^(m_s - max m) of the partial
// results (a lane per result); wave v then adds up the results s = v, v+4, ... with eight row loads in
// flight (a lane holds head_dim/64 neighbouring output elements), and the four sums meet in LDS.
constexpr int kPaMergeWaves = 4;
constexpr int kPaMergeMaxSplits = (int)kPaMaxChunks;  // weights kept in LDS; pa_chunking never cuts a sequence finer

template <int kPaD>
__global__ __launch_bounds__(kPaMergeWaves* kWave) void pa_decode_merge(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int32_t* __restrict__ context_lens, f16* __restrict__ o, int num_heads, int chunk_tokens,
    int max_splits, int balanced_wgs, int bs, int max_len, const int32_t* __restrict__ plan) {
  constexpr int kPer = kPaD / kWave;  // output elements per lane
  typedef float fvec __attribute__((ext_vector_type(kPer)));
  __shared__ float wts[kPaMergeMaxSplits];
  __shared__ float red[kPaMergeWaves][kPaD];
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int context_len = context_lens[b];
  const int64_t out = ((int64_t)b * num_heads + h) * kPaD;
  if (context_len <= 0) {
    if (threadIdx.x < kPaD) o[out + threadIdx.x] = (f16)0.f;
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
    nsplit = (context_len + chunk_tokens - 1) / chunk_tokens;
  }
  nsplit = min(nsplit, min(max_splits, kPaMergeMaxSplits));
  const int64_t base = ((int64_t)b * num_heads + h) * max_splits;

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
      v[j] = *reinterpret_cast<const fvec*>(&part_o[(base + sc) * kPaD + lane * kPer]);
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
  if (threadIdx.x < kPaD) {
    float a = 0.f;
#pragma unroll
    for (int v = 0; v < kPaMergeWaves; ++v) a += red[v][threadIdx.x];
    o[out + threadIdx.x] = (f16)(lsum > 0.f ? a / lsum : 0.f);
  }
}

template <int kPaD, int GMAX>
static void pa_launch(const f16* q, const f16* kc, const f16* vc, const int32_t* bt,
                      const int32_t* cl, f16* o, float* part_o, float* part_ml, int bs,
                      int num_heads, int num_kv_heads, int block_size, int max_blocks_per_seq,
                      PaChunking ch, hipStream_t s, int num_blocks, int32_t* order) {
  const float scale_log2 = kLog2e / __builtin_sqrtf((float)kPaD);
  if (ch.balanced_wgs > 0) {
    const int32_t* plan = nullptr;
    if (bs > kWave) {  // `order` is the int area behind the partial results
      pa_plan_kernel<<<1, kPaPlanThreads, 0, s>>>(cl, bs, max_blocks_per_seq * block_size, ch.balanced_wgs, order);
      plan = order;
    }
    dim3 bgrid((unsigned)ch.balanced_wgs, (unsigned)num_kv_heads);
    pa_decode_balanced<kPaD, GMAX><<<bgrid, kPaWaves * kWave, 0, s>>>(
        q, kc, vc, bt, cl, part_o, part_ml, bs, num_kv_heads, block_size, max_blocks_per_seq,
        ch.max_splits, scale_log2, num_blocks, num_heads / num_kv_heads, plan);
    dim3 mgrid((unsigned)num_heads, (unsigned)bs);
    pa_decode_merge<kPaD><<<mgrid, kPaMergeWaves * kWave, 0, s>>>(part_o, part_ml, cl, o, num_heads, ch.chunk_tokens,
                                           ch.max_splits, ch.balanced_wgs, bs,
                                           max_blocks_per_seq * block_size, plan);
    return;
  }
  dim3 grid((unsigned)ch.max_splits, (unsigned)num_kv_heads, (unsigned)bs);
  if (bs <= kWave || bs > kPaRankMax) order = nullptr;  // ranked inside the kernel / not ranked at all
  if (order) pa_rank_sequences<<<1, kPaRankMax, 0, s>>>(cl, bs, order);
  if (ch.max_splits == 1) {
    pa_decode_partial<kPaD, GMAX, true><<<grid, kPaWaves * kWave, 0, s>>>(
        q, kc, vc, bt, cl, part_o, part_ml, o, num_kv_heads, block_size, max_blocks_per_seq,
        ch.chunk_tokens, ch.max_splits, scale_log2, num_blocks, num_heads / num_kv_heads, order);
    return;
  }
  pa_decode_partial<kPaD, GMAX, false><<<grid, kPaWaves * kWave, 0, s>>>(
      q, kc, vc, bt, cl, part_o, part_ml, o, num_kv_heads, block_size, max_blocks_per_seq,
      ch.chunk_tokens, ch.max_splits, scale_log2, num_blocks, num_heads / num_kv_heads, order);
  dim3 mgrid((unsigned)num_heads, (unsigned)bs);
  pa_decode_merge<kPaD><<<mgrid, kPaMergeWaves * kWave, 0, s>>>(part_o, part_ml, cl, o, num_heads, ch.chunk_tokens,
                                         ch.max_splits, 0, bs, max_blocks_per_seq * block_size, nullptr);
}

// Generic path for every other shape (head_dim a multiple of 16 up to 256, any block size, any
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

// Shapes served by the MFMA kernel; everything else that is valid takes the generic kernel.
static bool pa_fast_shape(int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                          int64_t block_size) {
  if ((head_dim != 64 && head_dim != 128 && head_dim != 256) || block_size % 16 != 0) return false;
  // a lane of the score product holds one of at most 16 query heads of the kv head, and the cross-wave
  // merge keeps 8 x group x head_dim floats in LDS (at most 66 KB): up to 16 heads, 8 at head_dim 256
  const int64_t group = num_heads / num_kv_heads;
  return group <= kPaMaxGroup && group * head_dim <= kPaMaxGroup * 128;
}

}  // namespace aops

extern "C" size_t aops_paged_attention_workspace(int64_t bs, int64_t num_heads,
                                                 int64_t num_kv_heads, int64_t head_dim,
                                                 int64_t block_size, int64_t max_blocks_per_seq) {
  using namespace aops;
  if (!pa_args_valid(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq))
    return 0;
  if (!pa_fast_shape(num_heads, num_kv_heads, head_dim, block_size)) return 16;  // not used
  const PaChunking ch = pa_chunking(bs, num_kv_heads, block_size, max_blocks_per_seq);
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
  if (!pa_fast_shape(num_heads, num_kv_heads, head_dim, block_size)) {
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
  const PaChunking ch = pa_chunking(bs, num_kv_heads, block_size, max_blocks_per_seq);
  float* part_o = static_cast<float*>(workspace);
  float* part_ml = part_o + (size_t)bs * num_heads * ch.max_splits * head_dim;
  int32_t* order = reinterpret_cast<int32_t*>(part_ml + (size_t)bs * num_heads * ch.max_splits * 2);
#define AOPS_PA_CASE(D, G)                                                                      \
  case G:                                                                                       \
    pa_launch<D, G>(qp, kc, vc, block_tables, context_lens, op, part_o, part_ml, (int)bs,       \
                    (int)num_heads, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq, \
                    ch, s, (int)num_blocks, order);                                             \
    break;
#define AOPS_PA_GROUPS(D)     \
  switch (gmax) {             \
    AOPS_PA_CASE(D, 1)        \
    AOPS_PA_CASE(D, 2)        \
    AOPS_PA_CASE(D, 4)        \
    AOPS_PA_CASE(D, 8)        \
    AOPS_PA_CASE(D, 16)       \
  }
  const int64_t group = num_heads / num_kv_heads;
  if (group > kPaMaxGroup) return AOPS_ERR_INVALID_ARGUMENT;  // pa_fast_shape admits no such shape
  const int gmax = group <= 1 ? 1 : group <= 2 ? 2 : group <= 4 ? 4 : group <= 8 ? 8 : 16;
  if (head_dim == 64) {
    AOPS_PA_GROUPS(64)
  } else if (head_dim == 128) {
    AOPS_PA_GROUPS(128)
  } else {
    AOPS_PA_GROUPS(256)
  }
#undef AOPS_PA_GROUPS
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
