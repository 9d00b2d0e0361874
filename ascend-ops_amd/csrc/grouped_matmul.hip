// Grouped (per-expert) fp16 GEMM over expert-sorted rows, fp32 accumulate on MFMA: the entry
// points and the choice of kernel.  Kernels: grouped_matmul_tiles.hip (one workgroup per work
// item), grouped_matmul_persistent.hip (one workgroup per CU); shared pieces: gmm_common.h.
//
//   y[start_e:end_e, :] = x[start_e:end_e, :] @ W_e^T,   W_e stored [n, k] (k contiguous)
//
// Both operands are K-contiguous, which is exactly the per-lane operand shape of
// v_mfma_f32_32x32x16_f16 (8 consecutive k per lane), so tiles go HBM -> registers -> LDS
// with 128-bit accesses and no transposition.  group_list is read on the device: every
// workgroup derives the (expert, m-tile, n-tile) it owns from a wave-level scan of the
// per-expert tile counts, so there is no host synchronisation and no planning kernel.
// Workgroups are renumbered so that each XCD (one L2 per XCD, workgroup i runs on XCD i%8)
// works through a contiguous range of experts, with the m-tiles that share a weight tile
// next to each other.
//
// Semantics: reference csrc/opdev/op_kernel/grouped_mat_mul_ex.cpp:27-44 (start/end from the
// cumulative int64 group_list, empty groups skipped), matmul_core.h:42-68 (NT product, fp32
// accumulate, fp16 result), benchmark/test_grouped_matmul.py:6-23.
#include "gmm_common.h"

// forced: 1..9 = that kernel / tile shape whatever the problem size (the override entry point), 0 = choose.
static int aops_grouped_matmul_impl(const void* x, const void* w, const int64_t* group_list, void* y,
                                    int64_t rows, int64_t k, int64_t num_experts, int64_t n,
                                    void* stream, int forced = 0) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 64 != 0 || n % 64 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  // per-lane tile offsets are 32-bit: 320 rows x k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !y || (!group_list && num_experts != 1)) return AOPS_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const f16* xp = static_cast<const f16*>(x);
  const f16* wp = static_cast<const f16*>(w);
  f16* yp = static_cast<f16*>(y);
  // Tile choice from what the host knows (group_list stays on the device, so the rows are taken
  // to be spread evenly over the experts).  With few rows per expert the weights are streamed for
  // little arithmetic and every tile row beyond the group is wasted copy and MFMA work: 128- or
  // 64-row tiles.  Otherwise the largest tile whose grid still gives most CUs a work item: 320
  // rows cover a typical expert of a large routed batch in one tile, and the persistent kernel
  // (320 x 256) wins as soon as there are enough items for one per CU.
  int variant = forced;
  // a single group of at most 16 rows (the dense projection of a small decode batch): the weight-streaming kernel
  if ((variant < 1 || variant > 9) && num_experts == 1 && matmul_fewrows_takes(rows, k, n))
    return matmul_fewrows_launch(xp, wp, group_list, yp, rows, (int)k, (int)n, s);
  if (variant < 1 || variant > 9) {
    const int64_t groups = num_experts < rows ? num_experts : rows;  // experts that can hold a row
    const int64_t avg = (rows + groups - 1) / groups;
    auto m_tiles = [&](int64_t bm) { return (avg + bm - 1) / bm; };
    auto items = [&](int64_t bm, int64_t bn) { return groups * m_tiles(bm) * ((n + bn - 1) / bn); };
    const int64_t kEnough = (int64_t)device_cu_count() * 3 / 4;  // items that still keep most CUs busy
    if (avg < 96) {
      variant = (avg >= 24 && items(128, 128) >= kEnough) ? 4 : 5;
    } else if (items(320, 256) >= kEnough) {
      variant = 6;
    } else if (items(256, 128) >= kEnough && m_tiles(256) * 256 < m_tiles(320) * 320) {
      variant = 3;  // pads the groups less than 320-row tiles would
    } else if (items(320, 128) >= kEnough) {
      variant = 2;
    } else if (items(256, 128) >= kEnough) {
      variant = 3;
    } else if (items(128, 128) >= kEnough) {
      variant = 4;
    } else {
      variant = 5;
    }
  }
  if (variant == 6 && (k % 128 != 0 || k < 256)) variant = 1;  // the persistent kernel's k loop
  if (variant == 6)  // 320 x 256 tiles, eight waves, one persistent workgroup per CU
    return gmm_launch_persistent(false, xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s,
                                 nullptr, 1, 1);
  return gmm_launch_tiles(variant, xp, wp, group_list, yp, rows, (int)k, (int)num_experts, (int)n, s);
}

extern "C" int aops_grouped_matmul_f16(const void* x, const void* w, const int64_t* group_list,
                                       void* y, int64_t rows, int64_t k, int64_t num_experts,
                                       int64_t n, void* stream) {
  if (rows > 0 && num_experts > 0 && !group_list) return AOPS_ERR_INVALID_ARGUMENT;
  return aops_grouped_matmul_impl(x, w, group_list, y, rows, k, num_experts, n, stream);
}

extern "C" int aops_grouped_matmul_variant_f16(int variant, const void* x, const void* w,
                                               const int64_t* group_list, void* y, int64_t rows,
                                               int64_t k, int64_t num_experts, int64_t n,
                                               void* stream) {
  if (variant < 1 || variant > 9) return AOPS_ERR_INVALID_ARGUMENT;
  return aops_grouped_matmul_impl(x, w, group_list, y, rows, k, num_experts, n, stream, variant);
}

extern "C" int aops_grouped_matmul_ldw_f16(const void* x, const void* w, int64_t ldw, const int64_t* group_list,
                                           void* y, int64_t rows, int64_t k, int64_t num_experts, int64_t n,
                                           void* stream) {
  using namespace aops;
  if (rows < 0 || num_experts < 0 || n <= 0 || n % 64 != 0 || k < 256 || k % 128 != 0 || ldw < k || ldw % 8 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  // per-lane byte offsets inside a weight tile are 32-bit
  if (rows > 0x7fffffff - 4096 || ldw > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20))
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !y || !group_list) return AOPS_ERR_INVALID_ARGUMENT;
  return gmm_launch_persistent(false, static_cast<const f16*>(x), static_cast<const f16*>(w), group_list,
                               static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                               static_cast<hipStream_t>(stream), nullptr, 1, 1, (int)ldw);
}

// Kernel choice of the fused entry points: 0 = persistent 320 x 256 kernel, 1 = 128 x 128 tiles,
// 2 = 64 x 64 tiles.  Under 96 rows per expert the weights are streamed for little arithmetic and the
// small tiles win (see the tile choice above); the persistent kernel also needs k % 128 == 0, k >= 256.
static int fused_tile_choice(int64_t rows, int64_t k, int64_t num_experts) {
  const int64_t groups = num_experts < rows ? num_experts : rows;
  const int64_t avg = groups > 0 ? (rows + groups - 1) / groups : 0;
  if (k % 128 != 0 || k < 256) return avg < 24 ? 2 : 1;
  if (avg >= 96) return 0;
  return avg < 24 ? 2 : 1;
}

extern "C" int aops_grouped_matmul_swiglu_f16(const void* x, const void* w, const int64_t* group_list,
                                              void* y, int64_t rows, int64_t k, int64_t num_experts,
                                              int64_t n, void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 64 != 0 || n % 64 != 0)
    return AOPS_ERR_INVALID_ARGUMENT;
  // 32-bit per-lane offsets: (n/2 + 32) weight rows of k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20) ||
      (n / 2 + 320) * k > 0x7fffffffLL)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !w || !group_list || !y) return AOPS_ERR_INVALID_ARGUMENT;
  const int choice = fused_tile_choice(rows, k, num_experts);
  if (choice != 0)
    return gmm_launch_tiles_fused(choice == 2, static_cast<const f16*>(x), static_cast<const f16*>(w),
                                  group_list, static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                                  static_cast<hipStream_t>(stream), nullptr, 1, 1);
  return gmm_launch_persistent(true, static_cast<const f16*>(x), static_cast<const f16*>(w), group_list,
                               static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                               static_cast<hipStream_t>(stream), nullptr, 1, 1);
}

extern "C" int aops_matmul_nt_f16(const void* x, const void* w, void* y, int64_t m, int64_t k, int64_t n,
                                  void* stream) {
  if (m < 0 || k <= 0 || n <= 0 || k % 64 != 0 || n % 64 != 0) return AOPS_ERR_INVALID_ARGUMENT;
  if (m == 0) return AOPS_OK;
  if (!x || !w || !y) return AOPS_ERR_INVALID_ARGUMENT;
  return aops_grouped_matmul_impl(x, w, nullptr, y, m, k, 1, n, stream);
}

static bool matmul_nt_args_valid(int64_t m, int64_t k, int64_t n) {
  return m >= 0 && k > 0 && n > 0 && k % 64 == 0 && n % 64 == 0 && m <= 0x7fffffff - 4096 &&
         k <= (1 << 22) && n <= 0x7fffffff;
}

extern "C" size_t aops_matmul_nt_workspace(int64_t m, int64_t k, int64_t n) {
  if (!matmul_nt_args_valid(m, k, n) || m == 0) return 0;
  if (aops::matmul_fewrows_takes(m, k, n)) return 0;  // one launch, no partial results
  return aops::gmm_splitk_workspace(m, k, n);
}

extern "C" int aops_matmul_nt_ws_f16(const void* x, const void* w, void* y, void* workspace,
                                     size_t workspace_bytes, int64_t m, int64_t k, int64_t n,
                                     void* stream) {
  if (!matmul_nt_args_valid(m, k, n)) return AOPS_ERR_INVALID_ARGUMENT;
  if (m == 0) return AOPS_OK;
  if (!x || !w || !y) return AOPS_ERR_INVALID_ARGUMENT;
  if (aops_matmul_nt_workspace(m, k, n) == 0)
    return aops_grouped_matmul_impl(x, w, nullptr, y, m, k, 1, n, stream);
  return aops::gmm_launch_splitk(static_cast<const aops::f16*>(x), static_cast<const aops::f16*>(w), nullptr,
                                 static_cast<aops::f16*>(y), static_cast<float*>(workspace),
                                 workspace_bytes, m, (int)k, (int)n, static_cast<hipStream_t>(stream));
}

extern "C" size_t aops_grouped_matmul_workspace(int64_t rows, int64_t k, int64_t num_experts, int64_t n) {
  // only a single group of few rows with a long k is split over k; every other shape needs no scratch
  return num_experts == 1 ? aops_matmul_nt_workspace(rows, k, n) : 0;
}

extern "C" int aops_grouped_matmul_ws_f16(const void* x, const void* w, const int64_t* group_list, void* y,
                                          void* workspace, size_t workspace_bytes, int64_t rows, int64_t k,
                                          int64_t num_experts, int64_t n, void* stream) {
  if (aops_grouped_matmul_workspace(rows, k, num_experts, n) == 0)
    return aops_grouped_matmul_f16(x, w, group_list, y, rows, k, num_experts, n, stream);
  if (!x || !w || !y || !group_list) return AOPS_ERR_INVALID_ARGUMENT;
  return aops::gmm_launch_splitk(static_cast<const aops::f16*>(x), static_cast<const aops::f16*>(w), group_list,
                                 static_cast<aops::f16*>(y), static_cast<float*>(workspace),
                                 workspace_bytes, rows, (int)k, (int)n, static_cast<hipStream_t>(stream));
}

extern "C" int aops_grouped_matmul_swiglu_gather_f16(const void* x, const int32_t* row_idx,
                                                     int64_t idx_div, int64_t x_rows, const void* w,
                                                     const int64_t* group_list, void* y, int64_t rows,
                                                     int64_t k, int64_t num_experts, int64_t n,
                                                     void* stream) {
  using namespace aops;
  if (rows < 0 || k <= 0 || n <= 0 || num_experts < 0 || k % 64 != 0 || n % 64 != 0 ||
      idx_div <= 0 || idx_div > 0x7fffffff || x_rows < 0 || (rows > 0 && x_rows == 0))
    return AOPS_ERR_INVALID_ARGUMENT;
  // 32-bit per-lane offsets: x_rows activation rows and (n/2 + 32) weight rows of k elements must fit
  if (rows > 0x7fffffff - 4096 || k > (1 << 22) || n > 0x7fffffff || num_experts > (1 << 20) ||
      (n / 2 + 320) * k > 0x7fffffffLL || x_rows * k > 0xffffffffLL)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (rows == 0 || num_experts == 0) return AOPS_OK;
  if (!x || !row_idx || !w || !group_list || !y) return AOPS_ERR_INVALID_ARGUMENT;
  int choice = fused_tile_choice(rows, k, num_experts);
  // the persistent kernel addresses the gathered rows with 32-bit byte offsets: x below 4 GiB
  if (choice == 0 && x_rows * k * 2 > 0xffffffffLL) choice = 1;
  if (choice != 0)
    return gmm_launch_tiles_fused(choice == 2, static_cast<const f16*>(x), static_cast<const f16*>(w),
                                  group_list, static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                                  static_cast<hipStream_t>(stream), row_idx, (int)idx_div, x_rows);
  return gmm_launch_persistent(true, static_cast<const f16*>(x), static_cast<const f16*>(w), group_list,
                               static_cast<f16*>(y), rows, (int)k, (int)num_experts, (int)n,
                               static_cast<hipStream_t>(stream), row_idx, (int)idx_div, x_rows);
}
