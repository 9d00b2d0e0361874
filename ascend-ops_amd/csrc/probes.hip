// Measurement aids (no counterpart in the reference): kernels that isolate one cost of the operators so that
// the bounds quoted for them can be re-measured from this library alone.
//
//  * aops_probe_read_stream: a pure read stream with the access pattern of a GEMM operand copy.  Every
//    workgroup owns 128 consecutive rows of a [rows, row_bytes] byte matrix and walks along them in steps of
//    seg_bytes per row - with seg_bytes = 128 and row_bytes = 2 * k that is how the weight tiles of the grouped
//    matmul are fetched (128-byte pieces, one weight row apart); with row_bytes == seg_bytes the same kernel
//    reads its 128 x seg_bytes block linearly.  No arithmetic beyond a sum that keeps the loads alive.  The bytes
//    go into registers or, like the operand copies of the persistent grouped-matmul kernel, straight into LDS.
//  * aops_grouped_matmul_probe_f16: the persistent grouped-matmul kernel with parts of its k loop switched off.
//  * aops_probe_mfma_rate: fp16 MFMAs of one shape on operands held in registers and nothing else - the rate the
//    matrix cores sustain for a given operand content (all-zero operands: the peak; operands that change from one
//    instruction to the next: what the power limit leaves).
#include "gmm_common.h"

namespace aops {

// VIA_LDS: the bytes are copied straight into LDS with global_load_lds_dwordx4, the instruction the persistent
// grouped-matmul kernel fetches its operands with (a wave's 64 x 16 bytes land in 1 KiB of LDS that nobody reads),
// instead of into registers.
template <int SEG, bool VIA_LDS>
__global__ __launch_bounds__(256) void probe_read_stream_kernel(const char* __restrict__ buf, float* __restrict__ sink,
                                                                int64_t row_bytes) {
  constexpr int kLanesPerRow = SEG / 16;
  constexpr int kRowsPerPass = 256 / kLanesPerRow;
  constexpr int kPasses = 128 / kRowsPerPass;
  __shared__ __attribute__((aligned(16))) char landing[VIA_LDS ? 4 * kPasses * 1024 : 16];
  const char* base = buf + (int64_t)blockIdx.x * 128 * row_bytes;
  const int r0 = threadIdx.x / kLanesPerRow;
  const int c = threadIdx.x % kLanesPerRow;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if constexpr (VIA_LDS) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t lds0 = (uint32_t)(uintptr_t)AOPS_LDS_PTR(landing) + (uint32_t)wave * kPasses * 1024u;
    for (int64_t off = 0; off < row_bytes; off += SEG) {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const char* src = base + (int64_t)(r0 + p * kRowsPerPass) * row_bytes + off + c * 16;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :: "s"(lds0 + p * 1024u), "v"(src) : "memory");
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next step reuses the landing area
    }
    acc[0] = (float)landing[threadIdx.x & 15];
  } else {
    for (int64_t off = 0; off < row_bytes; off += SEG) {
      f32x4 v[kPasses];
#pragma unroll
      for (int p = 0; p < kPasses; ++p)
        v[p] = __builtin_nontemporal_load(
            reinterpret_cast<const f32x4*>(base + (int64_t)(r0 + p * kRowsPerPass) * row_bytes + off + c * 16));
#pragma unroll
      for (int p = 0; p < kPasses; ++p) acc += v[p];
    }
  }
  // never true for the buffers the probe is run on (finite values): the store only keeps the loads alive
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[0] = acc[0];
}

// Every wave issues `iters` rounds of MFMAs of 8 x 16384 multiply-adds' worth (8 of 32x32x16 or 16 of 16x16x32) on
// eight A and eight B fragments read once from `operands`; every instruction takes another pair of them than the
// one before, and the accumulators (128 registers either way) are independent.
template <int SHAPE>
__global__ __launch_bounds__(512) void probe_mfma_rate_kernel(const f16x8* __restrict__ operands, float* __restrict__ sink,
                                                              int iters) {
  const int lane = threadIdx.x & (kWave - 1);
  f16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[i * kWave + lane];
    b[i] = operands[(i + 8) * kWave + lane];
  }
  float total = 0.f;
  if constexpr (SHAPE == 32) {
    f32x16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; it += 8) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(i + 3 * j) & 7], b[(i + j) & 7], acc[i], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) total += acc[i][r];
  } else {
    f32x4 acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; it += 8) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          acc[i + 16 * (j & 1)] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(i + 3 * j) & 7], b[(i + j) & 7],
                                                                         acc[i + 16 * (j & 1)], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 32; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) total += acc[i][r];
  }
  // never true for finite operands: the store only keeps the MFMAs alive
  if (total == 12345.678f) sink[0] = total;
}

}  // namespace aops

extern "C" int aops_probe_mfma_rate(int shape, const void* operands, int64_t iters, void* sink, void* stream) {
  using namespace aops;
  if ((shape != 16 && shape != 32) || !operands || !sink || iters <= 0 || iters % 8 != 0 || iters > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)device_cu_count();
  if (shape == 32)
    probe_mfma_rate_kernel<32><<<grid, 512, 0, s>>>(static_cast<const f16x8*>(operands), static_cast<float*>(sink), (int)iters);
  else
    probe_mfma_rate_kernel<16><<<grid, 512, 0, s>>>(static_cast<const f16x8*>(operands), static_cast<float*>(sink), (int)iters);
  return record_launch_status(hipGetLastError());
}

extern "C" int aops_probe_read_stream(const void* buf, int64_t rows, int64_t row_bytes, int64_t seg_bytes,
                                      int via_lds, void* sink, void* stream) {
  using namespace aops;
  if (rows <= 0 || rows % 128 != 0 || rows / 128 > 0x7fffffff || row_bytes <= 0 || !buf || !sink)
    return AOPS_ERR_INVALID_ARGUMENT;
  if ((seg_bytes != 128 && seg_bytes != 256 && seg_bytes != 512 && seg_bytes != 1024) || row_bytes % seg_bytes != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (via_lds != 0 && via_lds != 1) return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned grid = (unsigned)(rows / 128);
  const char* p = static_cast<const char*>(buf);
  float* out = static_cast<float*>(sink);
#define AOPS_STREAM_CASE(SEG)                                                               \
  case SEG:                                                                                 \
    if (via_lds)                                                                            \
      probe_read_stream_kernel<SEG, true><<<grid, 256, 0, s>>>(p, out, row_bytes);          \
    else                                                                                    \
      probe_read_stream_kernel<SEG, false><<<grid, 256, 0, s>>>(p, out, row_bytes);         \
    break;
  switch (seg_bytes) {
    AOPS_STREAM_CASE(128)
    AOPS_STREAM_CASE(256)
    AOPS_STREAM_CASE(512)
    AOPS_STREAM_CASE(1024)
  }
#undef AOPS_STREAM_CASE
  return record_launch_status(hipGetLastError());
}

extern "C" int aops_grouped_matmul_probe_f16(int parts_off, const void* x, const void* w, int64_t ldw,
                                             const int64_t* group_list, void* y, int64_t rows, int64_t k,
                                             int64_t num_experts, int64_t n, void* stream) {
  using namespace aops;
  // the shapes the persistent 320 x 256 kernel takes
  if (rows <= 0 || num_experts <= 0 || k < 256 || k % 128 != 0 || ldw < k || ldw % 8 != 0 || ldw > (1 << 22) || n <= 0 ||
      n % 64 != 0 || rows > 0x7fffffff - 4096 || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (!x || !w || !y || (!group_list && num_experts != 1)) return AOPS_ERR_INVALID_ARGUMENT;
  return gmm_launch_persistent_probe(parts_off, static_cast<const f16*>(x), static_cast<const f16*>(w), group_list,
                                     static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                                     static_cast<hipStream_t>(stream), (int)ldw);
}
