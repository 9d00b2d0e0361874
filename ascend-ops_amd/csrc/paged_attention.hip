// Paged-attention decode over the [num_blocks, Hkv*D/16, block_size, 16] fp16 KV cache.
//
//   o[b,h] = softmax_j( q[b,h] . K[j,g] / sqrt(D) ) . V[j,g],   g = h / (Hq/Hkv)
//
// Split-KV ("flash decoding"): a workgroup of 4 waves owns one (sequence, kv head, chunk of
// the context); partial (max, sum, weighted V) triples go to a workspace and a second small
// kernel merges the chunks of each (sequence, query head).  context_lens and block_tables are
// read on the device only, so the grid is sized for the longest possible context and
// workgroups past the end of their sequence exit at once.
//
// Data path of the main kernel (head_dim 128): for one kv head a page holds K as
// [8 d-chunks][block_size tokens][16 halfs], i.e. 32-byte granules.  A lane owns the 8
// consecutive d values  d = 8*(lane%16) ..+7  for good (its slice of q stays in registers,
// its slice of the output accumulates in registers) and the four 16-lane rows of a wave take
// four neighbouring tokens, so every 128-bit load instruction of a wave fetches eight whole
// 128-byte lines and each cache byte is read exactly once.  q.K is finished with DPP adds
// inside the 16-lane row (no LDS), every row keeps its own running softmax state, and rows,
// waves and chunks are merged once at the end.  K and V of the next 32 tokens are in flight
// while the current 32 are consumed.
//
// Semantics: signature, cache indexing, GQA mapping and the fixed 1/sqrt(D) scale follow
// reference csrc/ffi/ops.cpp:408-482, csrc/opdev/op_host/paged_attention_ex.cpp:18-36 and
// csrc/opdev/op_kernel/paged_attention_ex.cpp:90-99 (whose compute body is unfinished).
#include "aops_common.h"

namespace aops {

constexpr int kPaD = 128;         // head_dim of the fast path
constexpr int kPaWaves = 4;       // waves per workgroup
constexpr int kPaLoads = 8;       // 128-bit loads per lane per step (each covers 4 tokens/wave)
constexpr int kPaStep = 4 * kPaLoads;  // tokens per wave per step
constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;

struct PaChunking {
  int chunk_tokens;  // tokens per workgroup (multiple of kPaWaves*kPaStep)
  int max_splits;    // chunks needed for the longest possible context
};

static PaChunking pa_chunking(int64_t bs, int64_t num_kv_heads, int64_t block_size,
                              int64_t max_blocks_per_seq) {
  const int64_t max_len = block_size * max_blocks_per_seq;
  int chunk = 512;
  // Small problems: shorter chunks so that the grid still covers the chip.
  while (chunk > kPaWaves * kPaStep &&
         bs * num_kv_heads * ((max_len + chunk - 1) / chunk) < 1024)
    chunk /= 2;
  PaChunking c;
  c.chunk_tokens = chunk;
  c.max_splits = (int)((max_len + chunk - 1) / chunk);
  if (c.max_splits < 1) c.max_splits = 1;
  return c;
}

struct F16x8Pairs {
  f16x2 p[4];
};

template <int G, bool MASKED>
__device__ __forceinline__ void pa_step(const f16x8 (&kreg)[kPaLoads], f16x8 (&vreg)[kPaLoads],
                                        const f16x2 (&q2)[G][4], float scale_log2,
                                        int first_token, int context_len, float (&m)[G],
                                        float (&l)[G], float (&acc)[G][8]) {
  float s[kPaLoads][G];
#pragma unroll
  for (int i = 0; i < kPaLoads; ++i) {
    const F16x8Pairs kp = __builtin_bit_cast(F16x8Pairs, kreg[i]);
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float a = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) a = __builtin_amdgcn_fdot2(kp.p[c], q2[h][c], a, false);
      s[i][h] = row16_sum(a) * scale_log2;
    }
    if (MASKED) {
      const bool valid = first_token + 4 * i < context_len;
#pragma unroll
      for (int h = 0; h < G; ++h) s[i][h] = valid ? s[i][h] : -__builtin_inff();
      // Cache contents past the end of the sequence are arbitrary (possibly NaN).
      const f16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
      vreg[i] = valid ? vreg[i] : zero;
    }
  }
#pragma unroll
  for (int h = 0; h < G; ++h) {
    float mx = m[h];
#pragma unroll
    for (int i = 0; i < kPaLoads; ++i) mx = fmaxf(mx, s[i][h]);
    const float alpha = __builtin_amdgcn_exp2f(m[h] - mx);
    m[h] = mx;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[h][j] *= alpha;
#pragma unroll
    for (int i = 0; i < kPaLoads; ++i) {
      const float p = __builtin_amdgcn_exp2f(s[i][h] - mx);
      psum += p;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[h][j] += p * (float)vreg[i][j];
    }
    l[h] = l[h] * alpha + psum;
  }
}

__device__ __forceinline__ void pa_issue_loads(const f16* __restrict__ kbase,
                                               const f16* __restrict__ vbase, uint32_t lane_off,
                                               f16x8 (&kreg)[kPaLoads], f16x8 (&vreg)[kPaLoads]) {
#pragma unroll
  for (int i = 0; i < kPaLoads; ++i) kreg[i] = ld128_stream(kbase + lane_off + i * 64);
#pragma unroll
  for (int i = 0; i < kPaLoads; ++i) vreg[i] = ld128_stream(vbase + lane_off + i * 64);
}

// grid = (max_splits, Hkv, bs), block = 256.
template <int G>
__global__ __launch_bounds__(kPaWaves* kWave) void pa_decode_partial(
    const f16* __restrict__ q, const f16* __restrict__ key_cache,
    const f16* __restrict__ value_cache, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ context_lens, float* __restrict__ part_o,
    float* __restrict__ part_ml, int num_kv_heads, int block_size, int max_blocks_per_seq,
    int chunk_tokens, int max_splits, float scale_log2) {
  const int split = blockIdx.x;
  const int g = blockIdx.y;
  const int b = blockIdx.z;
  const int context_len = context_lens[b];
  const int chunk_start = split * chunk_tokens;
  if (chunk_start >= context_len) return;
  const int chunk_len = min(context_len - chunk_start, chunk_tokens);
  const int nsteps = (chunk_len + kPaStep - 1) / kPaStep;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int row = lane >> 4;     // token row inside a load instruction
  const int piece = lane & 15;   // 16-byte piece of the head: d = 8*piece ..+7
  const int num_heads = num_kv_heads * G;

  // This lane's slice of the G query heads that share kv head g.
  f16x2 q2[G][4];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    const F16x8Pairs qp = __builtin_bit_cast(
        F16x8Pairs, ld128(q + ((int64_t)b * num_heads + g * G + h) * kPaD + piece * 8));
#pragma unroll
    for (int c = 0; c < 4; ++c) q2[h][c] = qp.p[c];
  }

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = kNegBig;
    l[h] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[h][j] = 0.f;
  }

  // Element offsets inside one page for this lane: d-chunk (piece/2) rows are block_size*16
  // halfs apart, the two halves of a granule 8 halfs, neighbouring tokens 16 halfs.
  const uint32_t lane_off = (uint32_t)(piece >> 1) * (uint32_t)block_size * 16u +
                            (uint32_t)(piece & 1) * 8u + (uint32_t)row * 16u;
  const int64_t page_elems = (int64_t)num_kv_heads * kPaD * block_size;
  const int64_t head_off = (int64_t)g * kPaD * block_size;
  const int32_t* table = block_tables + (int64_t)b * max_blocks_per_seq;

  auto page_offset = [&](int step) -> int64_t {
    const int tok = chunk_start + step * kPaStep;  // first token of the step (wave uniform)
    const int blk = tok / block_size;
    const int64_t page = table[blk];
    return page * page_elems + head_off + (int64_t)(tok - blk * block_size) * 16;
  };

  f16x8 kcur[kPaLoads], vcur[kPaLoads], knext[kPaLoads], vnext[kPaLoads];
  int step = wave;
  if (step < nsteps) {
    const int64_t off = page_offset(step);
    pa_issue_loads(key_cache + off, value_cache + off, lane_off, kcur, vcur);
  }
  while (step < nsteps) {
    const int next = step + kPaWaves;
    if (next < nsteps) {
      const int64_t off = page_offset(next);
      pa_issue_loads(key_cache + off, value_cache + off, lane_off, knext, vnext);
    }
    const int first_token = chunk_start + step * kPaStep + row;
    if (chunk_start + (step + 1) * kPaStep <= context_len) {
      pa_step<G, false>(kcur, vcur, q2, scale_log2, first_token, context_len, m, l, acc);
    } else {
      pa_step<G, true>(kcur, vcur, q2, scale_log2, first_token, context_len, m, l, acc);
    }
#pragma unroll
    for (int i = 0; i < kPaLoads; ++i) {
      kcur[i] = knext[i];
      vcur[i] = vnext[i];
    }
    step = next;
  }

  // Merge the four token rows of the wave (every lane ends up with the merged state).
#pragma unroll
  for (int h = 0; h < G; ++h) {
    float mx = fmaxf(m[h], __shfl_xor(m[h], 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float w = __builtin_amdgcn_exp2f(m[h] - mx);
    float lw = l[h] * w;
    lw += __shfl_xor(lw, 16);
    lw += __shfl_xor(lw, 32);
    m[h] = mx;
    l[h] = lw;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float a = acc[h][j] * w;
      a += __shfl_xor(a, 16);
      a += __shfl_xor(a, 32);
      acc[h][j] = a;
    }
  }

  // Merge the waves of the workgroup through LDS and emit one partial per query head.
  __shared__ float sm_acc[kPaWaves][G][kPaD];
  __shared__ float sm_m[kPaWaves][G];
  __shared__ float sm_l[kPaWaves][G];
  if (row == 0) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
#pragma unroll
      for (int j = 0; j < 8; ++j) sm_acc[wave][h][piece * 8 + j] = acc[h][j];
      if (piece == 0) {
        sm_m[wave][h] = m[h];
        sm_l[wave][h] = l[h];
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < G * kPaD; e += kPaWaves * kWave) {
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
    const int64_t slot = ((int64_t)b * num_heads + g * G + h) * max_splits + split;
    part_o[slot * kPaD + d] = a;
    if (d == 0) {
      part_ml[slot * 2 + 0] = mx;
      part_ml[slot * 2 + 1] = lsum;
    }
  }
}

// grid = (Hq, bs), block = 128: one thread per output element.
__global__ __launch_bounds__(kPaD) void pa_decode_merge(const float* __restrict__ part_o,
                                                        const float* __restrict__ part_ml,
                                                        const int32_t* __restrict__ context_lens,
                                                        f16* __restrict__ o, int num_heads,
                                                        int chunk_tokens, int max_splits) {
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int d = threadIdx.x;
  const int context_len = context_lens[b];
  const int64_t out = ((int64_t)b * num_heads + h) * kPaD + d;
  if (context_len <= 0) {
    o[out] = (f16)0.f;
    return;
  }
  int nsplit = (context_len + chunk_tokens - 1) / chunk_tokens;
  if (nsplit > max_splits) nsplit = max_splits;
  const int64_t base = ((int64_t)b * num_heads + h) * max_splits;
  float mx = kNegBig;
  for (int s = 0; s < nsplit; ++s) mx = fmaxf(mx, part_ml[(base + s) * 2]);
  float lsum = 0.f, a = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float wt = __builtin_amdgcn_exp2f(part_ml[(base + s) * 2] - mx);
    lsum += part_ml[(base + s) * 2 + 1] * wt;
    a += part_o[(base + s) * kPaD + d] * wt;
  }
  o[out] = (f16)(lsum > 0.f ? a / lsum : 0.f);
}

template <int G>
static void pa_launch(const f16* q, const f16* kc, const f16* vc, const int32_t* bt,
                      const int32_t* cl, f16* o, float* part_o, float* part_ml, int bs,
                      int num_heads, int num_kv_heads, int block_size, int max_blocks_per_seq,
                      PaChunking ch, hipStream_t s) {
  const float scale_log2 = kLog2e / __builtin_sqrtf((float)kPaD);
  dim3 grid((unsigned)ch.max_splits, (unsigned)num_kv_heads, (unsigned)bs);
  pa_decode_partial<G><<<grid, kPaWaves * kWave, 0, s>>>(q, kc, vc, bt, cl, part_o, part_ml,
                                                         num_kv_heads, block_size,
                                                         max_blocks_per_seq, ch.chunk_tokens,
                                                         ch.max_splits, scale_log2);
  dim3 mgrid((unsigned)num_heads, (unsigned)bs);
  pa_decode_merge<<<mgrid, kPaD, 0, s>>>(part_o, part_ml, cl, o, num_heads, ch.chunk_tokens,
                                         ch.max_splits);
}

static bool pa_shape_supported(int64_t bs, int64_t num_heads, int64_t num_kv_heads,
                               int64_t head_dim, int64_t block_size,
                               int64_t max_blocks_per_seq) {
  if (bs < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_blocks_per_seq < 0) return false;
  if (head_dim != kPaD) return false;
  if (block_size <= 0 || block_size % kPaStep != 0) return false;
  if (num_heads % num_kv_heads != 0) return false;
  const int64_t group = num_heads / num_kv_heads;
  if (group != 1 && group != 2 && group != 4 && group != 8) return false;
  if (bs > 65535 || num_kv_heads > 65535 || num_heads > 0x7fffffff / kPaD) return false;
  if (block_size * max_blocks_per_seq > 0x7fffffff) return false;
  return true;
}

}  // namespace aops

extern "C" size_t aops_paged_attention_workspace(int64_t bs, int64_t num_heads,
                                                 int64_t num_kv_heads, int64_t head_dim,
                                                 int64_t block_size, int64_t max_blocks_per_seq) {
  using namespace aops;
  if (!pa_shape_supported(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq))
    return 0;
  const PaChunking ch = pa_chunking(bs, num_kv_heads, block_size, max_blocks_per_seq);
  return (size_t)bs * (size_t)num_heads * (size_t)ch.max_splits * (kPaD + 2) * sizeof(float);
}

extern "C" int aops_paged_attention_f16(const void* q, const void* key_cache,
                                        const void* value_cache, const int32_t* block_tables,
                                        const int32_t* context_lens, void* o, void* workspace,
                                        size_t workspace_bytes, int64_t bs, int64_t num_heads,
                                        int64_t num_kv_heads, int64_t head_dim,
                                        int64_t block_size, int64_t max_blocks_per_seq,
                                        int64_t num_blocks, void* stream) {
  using namespace aops;
  (void)num_blocks;
  if (!pa_shape_supported(bs, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AOPS_OK;
  if (!q || !key_cache || !value_cache || !block_tables || !context_lens || !o)
    return AOPS_ERR_INVALID_ARGUMENT;
  const size_t need = aops_paged_attention_workspace(bs, num_heads, num_kv_heads, head_dim,
                                                     block_size, max_blocks_per_seq);
  if (!workspace || workspace_bytes < need) return AOPS_ERR_WORKSPACE;
  const PaChunking ch = pa_chunking(bs, num_kv_heads, block_size, max_blocks_per_seq);
  float* part_o = static_cast<float*>(workspace);
  float* part_ml = part_o + (size_t)bs * num_heads * ch.max_splits * kPaD;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const f16* qp = static_cast<const f16*>(q);
  const f16* kc = static_cast<const f16*>(key_cache);
  const f16* vc = static_cast<const f16*>(value_cache);
  f16* op = static_cast<f16*>(o);
  switch (num_heads / num_kv_heads) {
    case 1:
      pa_launch<1>(qp, kc, vc, block_tables, context_lens, op, part_o, part_ml, (int)bs,
                   (int)num_heads, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq, ch,
                   s);
      break;
    case 2:
      pa_launch<2>(qp, kc, vc, block_tables, context_lens, op, part_o, part_ml, (int)bs,
                   (int)num_heads, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq, ch,
                   s);
      break;
    case 4:
      pa_launch<4>(qp, kc, vc, block_tables, context_lens, op, part_o, part_ml, (int)bs,
                   (int)num_heads, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq, ch,
                   s);
      break;
    default:
      pa_launch<8>(qp, kc, vc, block_tables, context_lens, op, part_o, part_ml, (int)bs,
                   (int)num_heads, (int)num_kv_heads, (int)block_size, (int)max_blocks_per_seq, ch,
                   s);
      break;
  }
  return record_launch_status(hipGetLastError());
}
