// Measurement aids (no counterpart in the reference): kernels that isolate one cost of the operators so that
// the bounds quoted for them can be re-measured from this library alone.
//
//  * aops_probe_read_stream: a pure read stream with the access pattern of a GEMM operand copy.  Every
//    workgroup owns 128 consecutive rows of a [rows, row_bytes] byte matrix and walks along them in steps of
//    seg_bytes per row - with seg_bytes = 128 and row_bytes = 2 * k that is how the weight tiles of the grouped
//    matmul are fetched (128-byte pieces, one weight row apart); with row_bytes == seg_bytes the same kernel
//    reads its 128 x seg_bytes block linearly.  No arithmetic beyond a sum that keeps the loads alive.
//  * aops_grouped_matmul_probe_f16: the persistent grouped-matmul kernel with parts of its k loop switched off.
#include "gmm_common.h"

namespace aops {

template <int SEG>
__global__ __launch_bounds__(256) void probe_read_stream_kernel(const char* __restrict__ buf, float* __restrict__ sink,
                                                                int64_t row_bytes) {
  constexpr int kLanesPerRow = SEG / 16;
  constexpr int kRowsPerPass = 256 / kLanesPerRow;
  constexpr int kPasses = 128 / kRowsPerPass;
  const char* base = buf + (int64_t)blockIdx.x * 128 * row_bytes;
  const int r0 = threadIdx.x / kLanesPerRow;
  const int c = threadIdx.x % kLanesPerRow;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int64_t off = 0; off < row_bytes; off += SEG) {
    f32x4 v[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      v[p] = __builtin_nontemporal_load(
          reinterpret_cast<const f32x4*>(base + (int64_t)(r0 + p * kRowsPerPass) * row_bytes + off + c * 16));
#pragma unroll
    for (int p = 0; p < kPasses; ++p) acc += v[p];
  }
  // never true for the buffers the probe is run on (finite values): the store only keeps the loads alive
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[0] = acc[0];
}

}  // namespace aops

extern "C" int aops_probe_read_stream(const void* buf, int64_t rows, int64_t row_bytes, int64_t seg_bytes,
                                      void* sink, void* stream) {
  using namespace aops;
  if (rows <= 0 || rows % 128 != 0 || rows / 128 > 0x7fffffff || row_bytes <= 0 || !buf || !sink)
    return AOPS_ERR_INVALID_ARGUMENT;
  if ((seg_bytes != 128 && seg_bytes != 256 && seg_bytes != 512 && seg_bytes != 1024) || row_bytes % seg_bytes != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)(rows / 128);
  const char* p = static_cast<const char*>(buf);
  float* out = static_cast<float*>(sink);
  switch (seg_bytes) {
    case 128:
      probe_read_stream_kernel<128><<<grid, 256, 0, s>>>(p, out, row_bytes);
      break;
    case 256:
      probe_read_stream_kernel<256><<<grid, 256, 0, s>>>(p, out, row_bytes);
      break;
    case 512:
      probe_read_stream_kernel<512><<<grid, 256, 0, s>>>(p, out, row_bytes);
      break;
    default:
      probe_read_stream_kernel<1024><<<grid, 256, 0, s>>>(p, out, row_bytes);
      break;
  }
  return record_launch_status(hipGetLastError());
}

extern "C" int aops_grouped_matmul_probe_f16(int parts_off, const void* x, const void* w,
                                             const int64_t* group_list, void* y, int64_t rows, int64_t k,
                                             int64_t num_experts, int64_t n, void* stream) {
  using namespace aops;
  // the shapes the persistent 320 x 256 kernel takes
  if (rows <= 0 || num_experts <= 0 || k < 256 || k % 128 != 0 || k > (1 << 22) || n <= 0 || n % 64 != 0 ||
      rows > 0x7fffffff - 4096 || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (!x || !w || !y || (!group_list && num_experts != 1)) return AOPS_ERR_INVALID_ARGUMENT;
  return gmm_launch_persistent_probe(parts_off, static_cast<const f16*>(x), static_cast<const f16*>(w), group_list,
                                     static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                                     static_cast<hipStream_t>(stream));
}
