// Neox (rotate-half) rotary embedding of q and k, fp16 in/out, fp32 math with one rounding.
//   out[..., i]     = x[..., i]*cos[pos, i]     - x[..., i + h]*sin[pos, i]
//   out[..., i + h] = x[..., i + h]*cos[pos, i] + x[..., i]*sin[pos, i]        (h = head_dim/2)
// One thread rotates 8 pairs: two 128-bit loads of x, one each of cos and sin, two stores.
// Semantics: reference csrc/opdev/op_kernel/rope_ex.cpp:56-110, benchmark/test_graph.py:347-367.
#include "aops_common.h"

namespace aops {

__global__ __launch_bounds__(256) void rope_neox_kernel(
    const f16* __restrict__ q, const f16* __restrict__ k, const int32_t* __restrict__ position_ids,
    const f16* __restrict__ cos_cache, const f16* __restrict__ sin_cache, f16* __restrict__ out_q,
    f16* __restrict__ out_k, uint32_t total, uint32_t heads_total, uint32_t num_heads,
    uint32_t num_kv_heads, uint32_t head_dim) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t half = head_dim / 2;
  const uint32_t vec_per_head = half / 8;
  const uint32_t c = i % vec_per_head;
  const uint32_t bh = i / vec_per_head;
  const uint32_t head = bh % heads_total;  // q heads first, then k heads
  const uint32_t b = bh / heads_total;
  const f16* src;
  f16* dst;
  if (head < num_heads) {
    const int64_t off = ((int64_t)b * num_heads + head) * head_dim;
    src = q + off;
    dst = out_q + off;
  } else {
    const int64_t off = ((int64_t)b * num_kv_heads + (head - num_heads)) * head_dim;
    src = k + off;
    dst = out_k + off;
  }
  const int64_t pos = position_ids[b];
  const f16x8 x1 = ld128_stream(src + c * 8);
  const f16x8 x2 = ld128_stream(src + half + c * 8);
  const f16x8 cs = ld128(cos_cache + pos * half + c * 8);
  const f16x8 sn = ld128(sin_cache + pos * half + c * 8);
  f16x8 o1, o2;
  rope_rotate8(x1, x2, cs, sn, o1, o2);
  st128_stream(dst + c * 8, o1);
  st128_stream(dst + half + c * 8, o2);
}

}  // namespace aops

extern "C" int aops_rope_neox_f16(const void* q, const void* k, const int32_t* position_ids,
                                  const void* cos_cache, const void* sin_cache, void* out_q,
                                  void* out_k, int64_t bs, int64_t num_heads,
                                  int64_t num_kv_heads, int64_t head_dim, void* stream) {
  using namespace aops;
  if (bs < 0 || num_heads < 0 || num_kv_heads < 0 || head_dim <= 0 || head_dim % 16 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t heads_total = num_heads + num_kv_heads;
  const int64_t total = bs * heads_total * (head_dim / 16);
  if (total == 0) return AOPS_OK;
  if (total >= ((int64_t)1 << 32) - 256) return AOPS_ERR_INVALID_ARGUMENT;
  if (!position_ids || !cos_cache || !sin_cache) return AOPS_ERR_INVALID_ARGUMENT;
  if (num_heads > 0 && (!q || !out_q)) return AOPS_ERR_INVALID_ARGUMENT;
  if (num_kv_heads > 0 && (!k || !out_k)) return AOPS_ERR_INVALID_ARGUMENT;
  const unsigned grid = (unsigned)((total + 255) / 256);
  rope_neox_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(q), static_cast<const f16*>(k), position_ids,
      static_cast<const f16*>(cos_cache), static_cast<const f16*>(sin_cache),
      static_cast<f16*>(out_q), static_cast<f16*>(out_k), (uint32_t)total, (uint32_t)heads_total,
      (uint32_t)num_heads, (uint32_t)num_kv_heads, (uint32_t)head_dim);
  return record_launch_status(hipGetLastError());
}
