// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <unordered_map>

namespace mg {

constexpr int kGroup = 32;  // elements per shared scale (src/reorder.cu:78-79 of the reference)

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v6u __attribute__((ext_vector_type(6)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __bf16 v32bf __attribute__((ext_vector_type(32)));
typedef short v2s __attribute__((ext_vector_type(2)));

// MFMA f8f6f4 operand format selectors (cbsz for operand A, blgp for operand B).
constexpr int kFmtE4M3 = 0;
constexpr int kFmtE3M2 = 3;
constexpr int kFmtE2M1 = 4;

// Byte offset of the scale of (row r, block kb) in a segment's scale buffer:
// 128-row x 4-block atoms of 512 bytes, atoms along K fastest
// (include/reorder.cuh:119-124, src/reorder.cu:182-185 of the reference).
__host__ __device__ inline size_t sf_offset(int r, int kb, int katoms) {
  return ((size_t)(r >> 7) * katoms + (kb >> 2)) * 512 + (r & 31) * 16 + ((r >> 5) & 3) * 4 + (kb & 3);
}

__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Raises a kernel's dynamic-LDS limit to `bytes`, once per kernel and device (the attribute is kept
// per device); safe to call from several host threads.  The library instantiates a few hundred kernels
// that need it: the record of what has been set is a hash map, so that a process that has launched many of
// them still pays one look-up per launch and no driver call.
inline hipError_t allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::unordered_map<const void*, uint64_t> done;   // kernel -> bit per device on which the attribute is set
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  std::lock_guard<std::mutex> lock(mu);
  uint64_t& devices = done[kernel];
  if (devices & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) devices |= bit;
  return e;
}

// LDS bytes a workgroup may use and the number of CUs of the current device (asked once per device).
struct DeviceLimits { int lds_bytes, cus; };
inline hipError_t device_limits(DeviceLimits* out) {
  static std::mutex mu;
  static DeviceLimits table[64] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (table[dev].cus == 0) {
    int lds = 0, cus = 0;
    e = hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    table[dev] = DeviceLimits{lds, cus};
  }
  *out = table[dev];
  return hipSuccess;
}

}  // namespace mg
