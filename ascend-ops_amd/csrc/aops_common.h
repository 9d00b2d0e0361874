// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of libaops.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include "aops.h"

namespace aops {

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// 128-bit global access: one global_load/store_dwordx4 per lane.
__device__ __forceinline__ f16x8 ld128(const f16* p) { return *reinterpret_cast<const f16x8*>(p); }
__device__ __forceinline__ void st128(f16* p, f16x8 v) { *reinterpret_cast<f16x8*>(p) = v; }
// Streaming variants: data that is touched once should not displace reusable lines.
__device__ __forceinline__ f16x8 ld128_stream(const f16* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(p));
}
__device__ __forceinline__ void st128_stream(f16* p, f16x8 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<f16x8*>(p));
}

// DPP lane exchange inside a row of 16 lanes (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside each group of 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i inside each row of 16

// Sum over the 16 lanes of a DPP row; every lane of the row receives the total.
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<kDppXor1>(v);
  v += dpp_f32<kDppXor2>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppMirror>(v);
  return v;
}

// Sum over all 64 lanes; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

// Rotate-half rotation of 8 (x1, x2) pairs in fp32 with one rounding.  The products are combined
// with explicit fused multiply-adds so that every kernel that rotates produces the same bits.
__device__ __forceinline__ void rope_rotate8(const f16x8& x1, const f16x8& x2, const f16x8& cs,
                                             const f16x8& sn, f16x8& o1, f16x8& o2) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a = (float)x1[j], b = (float)x2[j], c = (float)cs[j], s = (float)sn[j];
    o1[j] = (f16)__builtin_fmaf(a, c, -(b * s));
    o2[j] = (f16)__builtin_fmaf(b, c, a * s);
  }
}

// Workgroups are dealt to the eight XCDs (each with its own L2) round robin by their index.  Where
// neighbouring pieces of work write into the same 128-byte cache lines (tokens in neighbouring slots of
// a paged cache), a line written from two XCDs reaches memory as two partial writes.  This renumbering
// gives the workgroups with the same index mod 8 (same XCD) kRun consecutive pieces of work inside
// every run of 8 * kRun workgroups; the incomplete run at the end of the grid keeps its order.
template <uint32_t kRun>
__device__ __forceinline__ uint32_t xcd_run_index(uint32_t wg, uint32_t num_wgs) {
  static_assert((kRun & (kRun - 1)) == 0, "power of two");
  constexpr uint32_t kSpan = 8u * kRun;
  if (wg >= (num_wgs & ~(kSpan - 1u))) return wg;
  return (wg & ~(kSpan - 1u)) + (wg & 7u) * kRun + ((wg >> 3) & (kRun - 1u));
}

// Launch-status bookkeeping shared by the host launchers.
int record_launch_status(hipError_t e);

// Compute units of the current device (queried once per device; 256, an MI355X, when there is no
// device to ask).  The one source of the CU count for every launcher that sizes a grid or a
// partition by it.
int device_cu_count();

// Raises the dynamic LDS limit of `kernel` to `bytes` on the current device, once per device (the attribute
// belongs to the kernel as loaded on one device; `done` is the caller's record, one bit per device, and
// races on it are benign: the call is idempotent).
hipError_t allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done);

}  // namespace aops
