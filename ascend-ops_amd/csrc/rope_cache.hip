// Decode-step fusion: neox rotary embedding of q and k, with the rotated k and the untouched v
// written straight into the paged caches [num_blocks, Hkv*D/16, block_size, 16].  Equals
// aops_rope_neox_f16 followed by aops_reshape_and_cache_f16 bit for bit (same rotation routine),
// in one launch and without the round trip of the rotated k through memory.
// Order of the two steps: reference csrc/ffi/graph.cpp:255-270; semantics of each:
// csrc/opdev/op_kernel/rope_ex.cpp:56-110, csrc/opdev/op_kernel/reshape_and_cache_ex.cpp:50-58.
//
// Thread map per token: (Hq+Hkv)*D/16 rotation threads (8 pairs each, as in rope_neox_kernel)
// followed by Hkv*D/8 threads that copy 16 bytes of v.  A rotation thread of a k head writes its two
// 16-byte results into the cache; threads c and c^1 complete one 32-byte granule.
//
// NORM = true puts the per-head RMSNorm of q and k (reference csrc/ffi/graph.cpp:252-253: RMSNorm
// without residual over head_dim, one weight vector for q and one for k) in front of the rotation:
// the head_dim/16 threads of a head add up their squares with lane exchanges (when that count is a
// power of two, so that a head's threads are aligned lanes of one wave; for any other head size
// every thread adds up its whole head itself from loads its neighbours share), the normalised
// values are rounded to fp16 as the separate operator's output would be, then rotated.
#include "aops_common.h"

namespace aops {

template <bool NORM>
__global__ __launch_bounds__(256) void rope_cache_kernel(
    const f16* __restrict__ q, const f16* __restrict__ k, const f16* __restrict__ v,
    const f16* __restrict__ q_norm_weight, const f16* __restrict__ k_norm_weight, float eps,
    const int32_t* __restrict__ position_ids, const f16* __restrict__ cos_cache,
    const f16* __restrict__ sin_cache, f16* __restrict__ out_q, f16* __restrict__ out_k,
    f16* __restrict__ key_cache, f16* __restrict__ value_cache,
    const int32_t* __restrict__ slot_indices, uint32_t total, uint32_t per_token,
    uint32_t rope_threads, uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
    uint32_t block_size, int64_t num_slots) {
  // neighbouring tokens (whose cache slots share cache lines in a prefill) on one XCD
  const uint32_t i = xcd_run_index<32>(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t b = i / per_token;
  const uint32_t t = i - b * per_token;
  const uint32_t half = head_dim / 2;
  const uint32_t chunks = num_kv_heads * head_dim / 16;  // 32-byte granules per cache row
  const int64_t slot = slot_indices[b];
  const bool slot_ok = slot >= 0 && slot < num_slots;
  const uint32_t block = slot_ok ? (uint32_t)slot / block_size : 0;
  const uint32_t off = slot_ok ? (uint32_t)slot - block * block_size : 0;
  // 16-byte piece p of the token's cache row
  auto cache_at = [&](f16* cache, uint32_t p) -> f16* {
    return cache + (((int64_t)block * chunks + (p >> 1)) * block_size + off) * 16 + (p & 1) * 8;
  };
  if (t >= rope_threads) {  // v copy
    if (!slot_ok) return;
    const uint32_t p = t - rope_threads;
    st128(cache_at(value_cache, p), ld128_stream(v + ((int64_t)b * num_kv_heads * head_dim) + p * 8));
    return;
  }
  const uint32_t vec_per_head = half / 8;
  const uint32_t c = t % vec_per_head;
  const uint32_t head = t / vec_per_head;  // q heads first, then k heads
  const int64_t pos = position_ids[b];
  const f16x8 cs = ld128(cos_cache + pos * half + c * 8);
  const f16x8 sn = ld128(sin_cache + pos * half + c * 8);
  f16x8 o1, o2;
  const bool is_q = head < num_heads;
  const uint32_t hk = head - num_heads;
  const int64_t base = is_q ? ((int64_t)b * num_heads + head) * head_dim
                            : ((int64_t)b * num_kv_heads + hk) * head_dim;
  const f16* src = is_q ? q : k;
  f16x8 x1 = ld128_stream(src + base + c * 8);
  f16x8 x2 = ld128_stream(src + base + half + c * 8);
  if constexpr (NORM) {
    const f16* nw = is_q ? q_norm_weight : k_norm_weight;
    const f16x8 w1 = ld128(nw + c * 8);
    const f16x8 w2 = ld128(nw + half + c * 8);
    float ss = 0.f;
    if ((vec_per_head & (vec_per_head - 1)) == 0 && vec_per_head <= 16) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)x1[j] * (float)x1[j] + (float)x2[j] * (float)x2[j];
      // the vec_per_head threads of this head are consecutive, aligned lanes
      for (uint32_t m = 1; m < vec_per_head; m <<= 1) ss += __shfl_xor(ss, (int)m);
    } else {
      // a head's threads may lie in two waves or workgroups: every thread sums the head, all in the
      // same order, so they agree on the result bit for bit
      for (uint32_t p = 0; p < head_dim / 8; ++p) {
        const f16x8 xv = ld128(src + base + p * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += (float)xv[j] * (float)xv[j];
      }
    }
    const float inv_rms = 1.0f / __builtin_sqrtf(ss / (float)head_dim + eps);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x1[j] = (f16)((float)x1[j] * inv_rms * (float)w1[j]);
      x2[j] = (f16)((float)x2[j] * inv_rms * (float)w2[j]);
    }
  }
  rope_rotate8(x1, x2, cs, sn, o1, o2);
  if (is_q) {
    st128_stream(out_q + base + c * 8, o1);
    st128_stream(out_q + base + half + c * 8, o2);
  } else {
    if (out_k) {
      st128_stream(out_k + base + c * 8, o1);
      st128_stream(out_k + base + half + c * 8, o2);
    }
    if (slot_ok) {
      const uint32_t p = hk * (head_dim / 8) + c;
      st128(cache_at(key_cache, p), o1);
      st128(cache_at(key_cache, p + vec_per_head), o2);
    }
  }
}

}  // namespace aops

namespace aops {

static int rope_cache_launch(bool norm, const void* q, const void* k, const void* v,
                             const void* q_norm_weight, const void* k_norm_weight, float eps,
                             const int32_t* position_ids, const void* cos_cache, const void* sin_cache,
                             void* out_q, void* out_k, void* key_cache, void* value_cache,
                             const int32_t* slot_indices, int64_t bs, int64_t num_heads,
                             int64_t num_kv_heads, int64_t head_dim, int64_t num_blocks,
                             int64_t block_size, void* stream) {
  if (bs < 0 || num_heads < 0 || num_kv_heads <= 0 || head_dim <= 0 || head_dim % 16 != 0 ||
      num_blocks < 0 || block_size <= 0 || block_size > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t num_slots = num_blocks * block_size;
  if (num_slots > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;  // slots are int32
  const int64_t rope_threads = (num_heads + num_kv_heads) * (head_dim / 16);
  const int64_t per_token = rope_threads + num_kv_heads * head_dim / 8;
  const int64_t total = bs * per_token;
  if (total == 0) return AOPS_OK;
  if (total >= ((int64_t)1 << 32) - 256) return AOPS_ERR_INVALID_ARGUMENT;
  if (!k || !v || !position_ids || !cos_cache || !sin_cache || !key_cache || !value_cache ||
      !slot_indices)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (num_heads > 0 && (!q || !out_q)) return AOPS_ERR_INVALID_ARGUMENT;
  if (norm && (!k_norm_weight || (num_heads > 0 && !q_norm_weight))) return AOPS_ERR_INVALID_ARGUMENT;
  const unsigned grid = (unsigned)((total + 255) / 256);
  auto kernel = norm ? rope_cache_kernel<true> : rope_cache_kernel<false>;
  kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(q), static_cast<const f16*>(k), static_cast<const f16*>(v),
      static_cast<const f16*>(q_norm_weight), static_cast<const f16*>(k_norm_weight), eps,
      position_ids, static_cast<const f16*>(cos_cache), static_cast<const f16*>(sin_cache),
      static_cast<f16*>(out_q), static_cast<f16*>(out_k), static_cast<f16*>(key_cache),
      static_cast<f16*>(value_cache), slot_indices, (uint32_t)total, (uint32_t)per_token,
      (uint32_t)rope_threads, (uint32_t)num_heads, (uint32_t)num_kv_heads, (uint32_t)head_dim,
      (uint32_t)block_size, num_slots);
  return record_launch_status(hipGetLastError());
}

}  // namespace aops

extern "C" int aops_rope_reshape_and_cache_f16(
    const void* q, const void* k, const void* v, const int32_t* position_ids, const void* cos_cache,
    const void* sin_cache, void* out_q, void* out_k, void* key_cache, void* value_cache,
    const int32_t* slot_indices, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
    int64_t head_dim, int64_t num_blocks, int64_t block_size, void* stream) {
  return aops::rope_cache_launch(false, q, k, v, nullptr, nullptr, 0.f, position_ids, cos_cache,
                                 sin_cache, out_q, out_k, key_cache, value_cache, slot_indices, bs,
                                 num_heads, num_kv_heads, head_dim, num_blocks, block_size, stream);
}

extern "C" int aops_qknorm_rope_reshape_and_cache_f16(
    const void* q, const void* k, const void* v, const void* q_norm_weight,
    const void* k_norm_weight, float epsilon, const int32_t* position_ids, const void* cos_cache,
    const void* sin_cache, void* out_q, void* out_k, void* key_cache, void* value_cache,
    const int32_t* slot_indices, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
    int64_t head_dim, int64_t num_blocks, int64_t block_size, void* stream) {
  return aops::rope_cache_launch(true, q, k, v, q_norm_weight, k_norm_weight, epsilon, position_ids,
                                 cos_cache, sin_cache, out_q, out_k, key_cache, value_cache,
                                 slot_indices, bs, num_heads, num_kv_heads, head_dim, num_blocks,
                                 block_size, stream);
}
