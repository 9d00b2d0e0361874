// Scatter of new K/V rows into the paged cache [num_blocks, row_elems/16, block_size, 16].
//
// The layout fixes the write pattern: a token's row of row_elems halfs lands as row_elems/16
// granules of 32 bytes, block_size*32 bytes apart.  One thread moves 16 bytes, so a lane pair
// writes one whole 32-byte granule in a single store instruction and the source row is read
// with fully coalesced 128-bit loads.  K and V go in the same launch (blockIdx.y).
// Semantics: reference benchmark/test_reshape_and_cache.py:6-25; out-of-range slots are
// skipped as in csrc/opdev/op_kernel/reshape_and_cache_ex.cpp:50.
#include "aops_common.h"

namespace aops {

__global__ __launch_bounds__(256) void reshape_and_cache_kernel(
    const f16* __restrict__ key, const f16* __restrict__ value, f16* __restrict__ key_cache,
    f16* __restrict__ value_cache, const int32_t* __restrict__ slot_indices, uint32_t total,
    uint32_t pieces_per_row, uint32_t block_size, int64_t num_slots) {
  // neighbouring tokens on one XCD: 32 workgroups = 64 tokens at 1024 halfs per row
  const uint32_t wg = xcd_run_index<32>(blockIdx.x, gridDim.x);
  const uint32_t i = wg * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t token = i / pieces_per_row;
  const uint32_t piece = i - token * pieces_per_row;  // 16-byte piece of the row
  const int64_t slot = slot_indices[token];
  if (slot < 0 || slot >= num_slots) return;
  const f16* src = blockIdx.y == 0 ? key : value;
  f16* dst = blockIdx.y == 0 ? key_cache : value_cache;
  const uint32_t block = (uint32_t)slot / block_size;
  const uint32_t off = (uint32_t)slot - block * block_size;
  const uint32_t chunks = pieces_per_row / 2;  // 32-byte granules per row
  const uint32_t c = piece >> 1;
  const int64_t d = (((int64_t)block * chunks + c) * block_size + off) * 16 + (piece & 1) * 8;
  st128(dst + d, ld128_stream(src + (int64_t)i * 8));
}

}  // namespace aops

extern "C" int aops_reshape_and_cache_f16(const void* key, const void* value, void* key_cache,
                                          void* value_cache, const int32_t* slot_indices,
                                          int64_t num_tokens, int64_t row_elems,
                                          int64_t num_blocks, int64_t block_size, void* stream) {
  using namespace aops;
  if (num_tokens < 0 || row_elems <= 0 || row_elems % 16 != 0 || num_blocks < 0 ||
      block_size <= 0 || block_size > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (num_tokens == 0 || num_blocks == 0) return AOPS_OK;
  if (!key || !key_cache || !slot_indices) return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t num_slots = num_blocks * block_size;
  if (num_slots > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;  // slots are int32
  const int64_t pieces = row_elems / 8;
  const int64_t total = num_tokens * pieces;
  if (total >= ((int64_t)1 << 32) - 256) return AOPS_ERR_INVALID_ARGUMENT;
  const bool with_value = value != nullptr && value_cache != nullptr;
  dim3 grid((unsigned)((total + 255) / 256), with_value ? 2 : 1);
  reshape_and_cache_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(key), static_cast<const f16*>(value), static_cast<f16*>(key_cache),
      static_cast<f16*>(value_cache), slot_indices, (uint32_t)total, (uint32_t)pieces,
      (uint32_t)block_size, num_slots);
  return record_launch_status(hipGetLastError());
}
