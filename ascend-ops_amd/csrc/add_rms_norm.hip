// Fused residual add + RMSNorm, fp16 in/out, fp32 math.
//
// One workgroup per row.  The row of t = x + residual is kept in registers between the
// sum-of-squares pass and the scaling pass, so every input byte is read from HBM once and
// every output byte written once: 4*H*2 bytes per row plus the (cache-resident) weight.
// Semantics: reference csrc/opdev/op_kernel/add_rms_norm_ex.cpp:43-122 and
// benchmark/test_add_rms_norm.py:6-10 (the mean of squares is taken over the fp16-rounded
// sum, as the reference's test function does).
#include "aops_common.h"

namespace aops {

__device__ __forceinline__ float block_sum(float v, float* smem) {
  v = wave_sum(v);
  const int nwaves = blockDim.x / kWave;
  if (nwaves == 1) return v;
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += smem[i];
  return total;
}

// ITERS 128-bit vectors per thread live in registers (ITERS*blockDim.x*8 >= H).
template <int ITERS>
__global__ __launch_bounds__(1024) void add_rms_norm_rows(const f16* __restrict__ x,
                                                          const f16* __restrict__ residual,
                                                          const f16* __restrict__ weight,
                                                          float eps, f16* __restrict__ y,
                                                          f16* __restrict__ residual_out,
                                                          int64_t num_tokens, int hidden) {
  __shared__ float smem[16];
  const int nvec = hidden / 8;
  const float inv_h = 1.0f / (float)hidden;
  for (int64_t row = blockIdx.x; row < num_tokens; row += gridDim.x) {
    const f16* xr = x + row * hidden;
    const f16* rr = residual + row * hidden;
    f16* yr = y + row * hidden;
    f16* ror = residual_out + row * hidden;

    f16x8 t16[ITERS], w16[ITERS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int v = threadIdx.x + it * blockDim.x;
      if (v < nvec) {
        const f16x8 a = ld128_stream(xr + v * 8);
        const f16x8 b = ld128_stream(rr + v * 8);
        w16[it] = ld128(weight + v * 8);  // in flight during the reduction
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const f16 s = (f16)((float)a[j] + (float)b[j]);  // correctly rounded fp16 add
          t16[it][j] = s;
          ss += (float)s * (float)s;
        }
        st128_stream(ror + v * 8, t16[it]);
      }
    }
    const float total = block_sum(ss, smem);
    const float inv_rms = 1.0f / __builtin_sqrtf(total * inv_h + eps);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int v = threadIdx.x + it * blockDim.x;
      if (v < nvec) {
        f16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (f16)((float)t16[it][j] * inv_rms * (float)w16[it][j]);
        st128_stream(yr + v * 8, o);
      }
    }
    if (row + gridDim.x < num_tokens) __syncthreads();  // smem reuse by the next row
  }
}

// Rows too long for registers: second pass re-reads residual_out (just written, cache hot).
__global__ __launch_bounds__(1024) void add_rms_norm_long_rows(const f16* __restrict__ x,
                                                               const f16* __restrict__ residual,
                                                               const f16* __restrict__ weight,
                                                               float eps, f16* __restrict__ y,
                                                               f16* residual_out,
                                                               int64_t num_tokens, int hidden) {
  __shared__ float smem[16];
  const int nvec = hidden / 8;
  const float inv_h = 1.0f / (float)hidden;
  for (int64_t row = blockIdx.x; row < num_tokens; row += gridDim.x) {
    const f16* xr = x + row * hidden;
    const f16* rr = residual + row * hidden;
    f16* yr = y + row * hidden;
    f16* ror = residual_out + row * hidden;
    float ss = 0.f;
    for (int v = threadIdx.x; v < nvec; v += blockDim.x) {
      const f16x8 a = ld128_stream(xr + v * 8);
      const f16x8 b = ld128_stream(rr + v * 8);
      f16x8 t;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        t[j] = (f16)((float)a[j] + (float)b[j]);
        ss += (float)t[j] * (float)t[j];
      }
      st128(ror + v * 8, t);
    }
    const float total = block_sum(ss, smem);
    const float inv_rms = 1.0f / __builtin_sqrtf(total * inv_h + eps);
    // Each thread re-reads exactly the vectors it wrote itself, so no fence is needed.
    for (int v = threadIdx.x; v < nvec; v += blockDim.x) {
      const f16x8 t = ld128(ror + v * 8);
      const f16x8 w = ld128(weight + v * 8);
      f16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (f16)((float)t[j] * inv_rms * (float)w[j]);
      st128_stream(yr + v * 8, o);
    }
    if (row + gridDim.x < num_tokens) __syncthreads();
  }
}

}  // namespace aops

extern "C" int aops_add_rms_norm_f16(const void* x, const void* residual, const void* weight,
                                     float epsilon, void* y, void* residual_out,
                                     int64_t num_tokens, int64_t hidden, void* stream) {
  using namespace aops;
  if (num_tokens < 0 || hidden <= 0 || hidden % 8 != 0 || hidden > (int64_t)1 << 30)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (num_tokens == 0) return AOPS_OK;
  if (!x || !residual || !weight || !y || !residual_out) return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int nvec = (int)(hidden / 8);
  const unsigned grid = (unsigned)(num_tokens < 1048576 ? num_tokens : 1048576);
  const f16* xp = static_cast<const f16*>(x);
  const f16* rp = static_cast<const f16*>(residual);
  const f16* wp = static_cast<const f16*>(weight);
  f16* yp = static_cast<f16*>(y);
  f16* op = static_cast<f16*>(residual_out);
  // Few rows: one vector per thread (shortest dependency chain).  Many rows: two vectors
  // per thread halves the number of waves that have to be scheduled per row.
  int iters = 1;
  if (nvec > 1024 || (num_tokens >= 2048 && nvec >= 256)) iters = 2;
  if (nvec > 2048) iters = 4;
  if (nvec > 4096) iters = 8;
  int threads = ((nvec + iters - 1) / iters + kWave - 1) / kWave * kWave;
  if (nvec > 8192) {
    add_rms_norm_long_rows<<<grid, 1024, 0, s>>>(xp, rp, wp, epsilon, yp, op, num_tokens,
                                                 (int)hidden);
  } else if (iters == 1) {
    add_rms_norm_rows<1><<<grid, threads, 0, s>>>(xp, rp, wp, epsilon, yp, op, num_tokens,
                                                  (int)hidden);
  } else if (iters == 2) {
    add_rms_norm_rows<2><<<grid, threads, 0, s>>>(xp, rp, wp, epsilon, yp, op, num_tokens,
                                                  (int)hidden);
  } else if (iters == 4) {
    add_rms_norm_rows<4><<<grid, threads, 0, s>>>(xp, rp, wp, epsilon, yp, op, num_tokens,
                                                  (int)hidden);
  } else {
    add_rms_norm_rows<8><<<grid, threads, 0, s>>>(xp, rp, wp, epsilon, yp, op, num_tokens,
                                                  (int)hidden);
  }
  return record_launch_status(hipGetLastError());
}
