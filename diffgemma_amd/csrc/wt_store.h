// Write-through stores for results that the next kernel reads.
//
// Each of the chip's eight compute-unit groups (XCDs) has an L2 of its own, and the L2s are made
// consistent with memory at kernel boundaries only: a kernel does not end before every line it left
// dirty in an L2 has been written back.  A kernel that stores megabytes in its last microsecond (split
// partial rows, merged output rows) pays for that write-back after its last wave has gone.  Stores
// with the device-scope cache policy go through to memory when they are issued, while other waves
// still compute, and leave nothing to write back (a sliding layer's step: 27.0 -> 25.1 us, the
// 32k-key global layer's: -2 us).
//
// The buffer form is used because the compiler knows it (no inline assembly, wait counts kept by the
// compiler).  A window is a wave-uniform base address plus 32-bit byte offsets below 2^31; callers
// take the base per workgroup so that the offsets stay small whatever the size of the array.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dg {
namespace {

typedef uint32_t wt_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t wt_u32x2 __attribute__((ext_vector_type(2)));
constexpr int kWtPolicy = 16;   // cache-policy operand of the buffer builtins: sc1, device scope

// `base` must be the same in every lane of the wave (derived from blockIdx and kernel arguments)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wt_window(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7fffffff, 0x00020000);
}
// for a base that is the same in every lane without the compiler being able to tell (it depends on
// the wave's index within the workgroup)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wt_window_wave(const void* base) {
  const uint64_t a = (uint64_t)base;
  // (the builtin returns a signed int: through uint32_t, or the low half's top bit smears over the high half)
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  const uint64_t u = ((uint64_t)hi << 32) | (uint64_t)lo;
  return wt_window((const void*)u);
}
__device__ __forceinline__ void wt_store16(__amdgpu_buffer_rsrc_t w, uint32_t byte_off, wt_u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, w, byte_off, 0, kWtPolicy);
}
__device__ __forceinline__ void wt_store8(__amdgpu_buffer_rsrc_t w, uint32_t byte_off, wt_u32x2 v) {
  __builtin_amdgcn_raw_buffer_store_b64(v, w, byte_off, 0, kWtPolicy);
}
__device__ __forceinline__ void wt_store4(__amdgpu_buffer_rsrc_t w, uint32_t byte_off, uint32_t v) {
  __builtin_amdgcn_raw_buffer_store_b32(v, w, byte_off, 0, kWtPolicy);
}

__device__ __forceinline__ void wt_store2(__amdgpu_buffer_rsrc_t w, uint32_t byte_off, uint16_t v) {
  __builtin_amdgcn_raw_buffer_store_b16(v, w, byte_off, 0, kWtPolicy);
}

}  // namespace
}  // namespace dg
