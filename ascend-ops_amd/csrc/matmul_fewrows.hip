// Dense y = x @ W^T for at most 16 activation rows (the projections of a small decode batch):
// x [m, k], W stored [n, k] (k contiguous), y [m, n].  Every weight is used m times, so the product is
// a stream of W and the kernel is built around reading W once, in long contiguous pieces, with as
// much of it requested at once as a CU can hold.
//
// One workgroup of eight waves owns 16 consecutive rows of W, a contiguous block of 16*k halfs.  The k
// range is taken in rounds of 2048; in a round wave v owns 256 consecutive k.  It copies its 16 x 256
// piece of W and the matching piece of x from memory straight into its own 16 KiB of LDS
// (global_load_lds, 16 bytes per lane, every copy instruction two whole 512-byte row pieces), waits
// for them alone (no workgroup barrier: nobody else touches that LDS), and feeds eight
// v_mfma_f32_16x16x32_f16 from it.  The workgroup so keeps 64 KiB of W in flight.  The 16-byte chunks
// of a row are stored XOR-swizzled with the row number (applied to the source address, because a lane
// cannot choose where its 16 bytes land), so the operand reads, 16 rows at the same k, spread evenly
// over the LDS banks.  The eight partial sums meet in LDS in a fixed order: results are the same from
// call to call, and there is no workspace and no second kernel.
// Semantics as the grouped matmul with one group: reference csrc/opdev/op_kernel/matmul_core.h:42-68
// (NT product, fp32 accumulate, fp16 result); with a group_list (one entry), rows from group_list[0] on
// are not written (reference csrc/ffi/ops.cpp:179, csrc/opdev/op_kernel/grouped_mat_mul_ex.cpp:27-44).
#include "gmm_common.h"

namespace aops {

constexpr int kFrWaves = 8;
constexpr int kFrK = 256;                    // k per wave and round
constexpr int kFrChunks = kFrK / 8;          // 16-byte chunks per row piece
constexpr int kFrPiece = 16 * kFrK;          // halfs of a 16-row piece
constexpr int kFrCopies = kFrPiece * 2 / 1024;  // copy instructions per piece (1 KiB each)

// grid = n / 16, block = 8 waves; m <= 16, k a multiple of 64.
__global__ __launch_bounds__(kFrWaves* kWave) void matmul_fewrows_kernel(
    const f16* __restrict__ x, const f16* __restrict__ w, const int64_t* __restrict__ group_list,
    f16* __restrict__ y, int m, int k, int n) {
  extern __shared__ __attribute__((aligned(16))) f16 fr_smem[];
  f16* stage = fr_smem;                                                       // [wave][W, x][kFrPiece]
  float* red = reinterpret_cast<float*>(fr_smem + kFrWaves * 2 * kFrPiece);   // [wave][row of x][17]
  // neighbouring column blocks (32 bytes of every output row each) on one XCD, so that the output's
  // cache lines are completed in one L2
  const uint32_t wg = xcd_run_index<4>(blockIdx.x, gridDim.x);
  const int n0 = (int)wg * 16;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int rows = group_list ? (int)min((int64_t)m, max(group_list[0], (int64_t)0)) : m;

  // Copy side: instruction j of a piece fills rows 2j and 2j+1; this lane's 16 bytes land at chunk
  // position p of row 2j + (lane >> 5) and come from chunk p ^ (row & 15) of that row.
  const int cp_row = lane >> 5;
  const int cp_pos = lane & 31;
  // Operand side: lane (i, kg) reads row i, chunk 4*step + kg, i.e. position (4*step + kg) ^ i.
  const int i = lane & 15;
  const int kg = lane >> 4;

  f16* w_lds = stage + (wave * 2 + 0) * kFrPiece;
  f16* x_lds = stage + (wave * 2 + 1) * kFrPiece;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4 acc = zero4;

  for (int k0 = wave * kFrK; k0 < k; k0 += kFrWaves * kFrK) {
    const int klen = min(kFrK, k - k0);  // a multiple of 64; the last round of a wave may be short
    // chunks past klen would read past the end of the row: they repeat chunk 0 and are never used
#pragma unroll
    for (int j = 0; j < kFrCopies; ++j) {
      const int row = 2 * j + cp_row;
      int chunk = cp_pos ^ (row & 15);
      chunk = chunk * 8 < klen ? chunk : 0;
      const f16* wsrc = w + (int64_t)(n0 + row) * k + k0 + chunk * 8;
      const f16* xsrc = x + (int64_t)min(row, m - 1) * k + k0 + chunk * 8;
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(wsrc), AOPS_LDS_PTR(w_lds + j * 512), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(AOPS_GLOBAL_PTR(xsrc), AOPS_LDS_PTR(x_lds + j * 512), 16, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    asm volatile("" ::: "memory");
    const int steps = klen / 32;
#pragma unroll
    for (int s = 0; s < kFrK / 32; ++s) {
      if (s < steps) {  // wave uniform
        const int pos = (4 * s + kg) ^ i;
        const f16x8 a = *reinterpret_cast<const f16x8*>(w_lds + i * kFrK + pos * 8);
        const f16x8 b = *reinterpret_cast<const f16x8*>(x_lds + i * kFrK + pos * 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
      }
    }
    // the operand reads must be done before the next round's copies overwrite the stage
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    asm volatile("" ::: "memory");
  }

  // acc[r]: x row i, W row n0 + 4kg + r
#pragma unroll
  for (int r = 0; r < 4; ++r) red[(wave * 16 + i) * 17 + 4 * kg + r] = acc[r];
  __syncthreads();
  if (threadIdx.x < 256) {
    const int mi = threadIdx.x >> 4;
    const int nj = threadIdx.x & 15;
    if (mi < rows) {
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < kFrWaves; ++v) sum += red[(v * 16 + mi) * 17 + nj];
      y[(int64_t)mi * n + n0 + nj] = (f16)sum;
    }
  }
}

// Shapes the kernel takes: at most 16 rows, enough 16-row blocks of W to give every CU one, and not so
// many that the tile kernels (several workgroups per CU) do better.
bool matmul_fewrows_takes(int64_t m, int64_t k, int64_t n) {
  return m >= 1 && m <= 16 && k >= 512 && n / 16 >= 128 && n / 16 <= 1024;
}

int matmul_fewrows_launch(const f16* x, const f16* w, const int64_t* group_list, f16* y, int64_t m, int k,
                          int n, hipStream_t stream) {
  constexpr int kLds = kFrWaves * 2 * kFrPiece * (int)sizeof(f16) + kFrWaves * 16 * 17 * (int)sizeof(float);
  static_assert(kLds <= 160 * 1024, "LDS budget");
  static std::atomic<uint64_t> lds_allowed{0};  // per device
  if (const hipError_t le = allow_dynamic_lds(reinterpret_cast<const void*>(matmul_fewrows_kernel), kLds, lds_allowed); le != hipSuccess)
    return record_launch_status(le);
  matmul_fewrows_kernel<<<(unsigned)(n / 16), kFrWaves * kWave, kLds, stream>>>(x, w, group_list, y, (int)m, k, n);
  return record_launch_status(hipGetLastError());
}

}  // namespace aops
