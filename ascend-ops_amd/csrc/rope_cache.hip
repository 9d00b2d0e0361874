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
#include "aops_common.h"

namespace aops {

__global__ __launch_bounds__(256) void rope_cache_kernel(
    const f16* __restrict__ q, const f16* __restrict__ k, const f16* __restrict__ v,
    const int32_t* __restrict__ position_ids, const f16* __restrict__ cos_cache,
    const f16* __restrict__ sin_cache, f16* __restrict__ out_q, f16* __restrict__ out_k,
    f16* __restrict__ key_cache, f16* __restrict__ value_cache,
    const int32_t* __restrict__ slot_indices, uint32_t total, uint32_t per_token,
    uint32_t rope_threads, uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
    uint32_t block_size, int64_t num_slots) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
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
  if (head < num_heads) {
    const int64_t base = ((int64_t)b * num_heads + head) * head_dim;
    rope_rotate8(ld128_stream(q + base + c * 8), ld128_stream(q + base + half + c * 8), cs, sn, o1, o2);
    st128_stream(out_q + base + c * 8, o1);
    st128_stream(out_q + base + half + c * 8, o2);
  } else {
    const uint32_t hk = head - num_heads;
    const int64_t base = ((int64_t)b * num_kv_heads + hk) * head_dim;
    rope_rotate8(ld128_stream(k + base + c * 8), ld128_stream(k + base + half + c * 8), cs, sn, o1, o2);
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

extern "C" int aops_rope_reshape_and_cache_f16(
    const void* q, const void* k, const void* v, const int32_t* position_ids, const void* cos_cache,
    const void* sin_cache, void* out_q, void* out_k, void* key_cache, void* value_cache,
    const int32_t* slot_indices, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
    int64_t head_dim, int64_t num_blocks, int64_t block_size, void* stream) {
  using namespace aops;
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
  const unsigned grid = (unsigned)((total + 255) / 256);
  rope_cache_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(q), static_cast<const f16*>(k), static_cast<const f16*>(v),
      position_ids, static_cast<const f16*>(cos_cache), static_cast<const f16*>(sin_cache),
      static_cast<f16*>(out_q), static_cast<f16*>(out_k), static_cast<f16*>(key_cache),
      static_cast<f16*>(value_cache), slot_indices, (uint32_t)total, (uint32_t)per_token,
      (uint32_t)rope_threads, (uint32_t)num_heads, (uint32_t)num_kv_heads, (uint32_t)head_dim,
      (uint32_t)block_size, num_slots);
  return record_launch_status(hipGetLastError());
}
