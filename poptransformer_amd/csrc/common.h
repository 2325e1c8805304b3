// Shared helpers for the gfx950 (CDNA4, wave64) decode kernels.
//
// Conventions used by every translation unit in this directory:
//   * entry points are extern "C", take raw device pointers + sizes + a hipStream_t,
//     return 0 on success or a negative PTA_E* code, and never throw;
//   * no entry point allocates, frees or synchronises: they only enqueue work on the
//     caller's stream, so they may be recorded into a HIP graph;
//   * fp16 values are `_Float16` on the device side and uint16 bit patterns on the ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/poptransformer_hip.h"

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define PTA_WAVE 64

void pta_set_error(const char* fmt, ...);

#define PTA_REQUIRE(cond, ...)                      \
  do {                                              \
    if (!(cond)) {                                  \
      pta_set_error(__VA_ARGS__);                   \
      return PTA_EINVAL;                            \
    }                                               \
  } while (0)

#define PTA_CHECK_LAUNCH(name)                                                  \
  do {                                                                          \
    hipError_t e__ = hipGetLastError();                                         \
    if (e__ != hipSuccess) {                                                    \
      pta_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));     \
      return PTA_EHIP;                                                          \
    }                                                                           \
  } while (0)

static inline bool pta_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// the same total in every lane, by four data-parallel moves within the rows of 16 lanes and four lane reads: a
// fraction of the time of the six dependent LDS-crossbar shuffles of wave_sum (every lane of the wave must be active)
__device__ __forceinline__ float wave_total_dpp(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // quad_perm [1, 0, 3, 2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // quad_perm [2, 3, 0, 1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
  const int b = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}
// the sum over each group of N (8 or 16) consecutive lanes, in every lane of the group, by data-parallel moves within
// the rows of 16 lanes (every lane of the wave must be active)
template <int N>
__device__ __forceinline__ float lane_group_sum(float v) {
  static_assert(N == 8 || N == 16, "groups of 8 or 16 lanes");
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // quad_perm [1, 0, 3, 2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // quad_perm [2, 3, 0, 1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  if (N == 16) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

template <typename T, typename U>
__device__ __forceinline__ T bitcast(U u) {
  static_assert(sizeof(T) == sizeof(U), "bitcast size");
  return __builtin_bit_cast(T, u);
}
