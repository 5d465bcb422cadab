// Measurement helper, not part of the hot path: the rate at which all 1024 SIMDs of the GPU
// sustain v_mfma_scale_f32_32x32x64_f8f6f4 (E2M1 x E2M1) from registers, with nothing else in the
// loop.  Operand bits are either small constants or pseudo-random: with random bits the
// chip runs into its power limit and clocks down, so the second figure is the ceiling a GEMM on
// real data can approach, whatever its memory system does.
#include "mg_common.h"

namespace mg {

namespace {

__device__ __forceinline__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

__device__ __forceinline__ v8i widen4(v4i v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1); }

template <bool RANDOM>
__global__ void __launch_bounds__(256) mfma_ceiling_kernel(float* __restrict__ out, int iters, long long* __restrict__ cycles) {
  const int lane = threadIdx.x & 63;
  const unsigned seed = blockIdx.x * 256 + threadIdx.x;
  v16f acc[16];
#pragma unroll
  for (int a = 0; a < 16; ++a)
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[a][q] = 0.0f;
  v4i wf[4], xf[4];
  int sw[4], sx[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      wf[t][j] = RANDOM ? (int)mix(seed * 16 + t * 4 + j) : lane + j;
      xf[t][j] = RANDOM ? (int)mix(seed * 16 + t * 4 + j + 7777777u) : 3 * lane + j;
    }
    sw[t] = RANDOM ? (int)(0x7c7d7e7fu ^ (mix(seed + t) & 0x03030303u)) : 0x7f7f7f7f;
    sx[t] = RANDOM ? (int)(0x7e7f7d7cu ^ (mix(seed + 99 + t) & 0x03030303u)) : 0x7f7f7f7f;
  }
  const long long t0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        acc[a * 4 + b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(widen4(wf[a]), widen4(xf[b]), acc[a * 4 + b],
                                                                         kFmtE2M1, kFmtE2M1, 0, sw[a], 0, sx[b]);
        __builtin_amdgcn_sched_barrier(0);
      }
  }
  const long long t1 = __builtin_readcyclecounter();
  float r = 0.0f;
#pragma unroll
  for (int a = 0; a < 16; ++a) r += acc[a][0] + acc[a][9];
  out[blockIdx.x * 256 + threadIdx.x] = r;
  if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
}

}  // namespace

}  // namespace mg

extern "C" __attribute__((visibility("default")))
int mg_measure_mfma_ceiling(int random_operands, int iters, double* tflops, double* shader_ghz) {
  constexpr int kGrid = 256;   // one workgroup of 4 waves per CU
  float* out = nullptr;
  long long* cyc = nullptr;
  hipEvent_t a = nullptr, b = nullptr;
  hipError_t e = hipMalloc(&out, kGrid * 256 * sizeof(float));
  if (e == hipSuccess) e = hipMalloc(&cyc, kGrid * sizeof(long long));
  if (e == hipSuccess) e = hipEventCreate(&a);
  if (e == hipSuccess) e = hipEventCreate(&b);
  float ms = 0.0f;
  long long host_cyc[kGrid];
  if (e == hipSuccess) {
    for (int rep = 0; rep < 2 && e == hipSuccess; ++rep) {   // first launch warms up clocks and code
      hipEventRecord(a, nullptr);
      if (random_operands) hipLaunchKernelGGL(mg::mfma_ceiling_kernel<true>, dim3(kGrid), dim3(256), 0, nullptr, out, iters, cyc);
      else hipLaunchKernelGGL(mg::mfma_ceiling_kernel<false>, dim3(kGrid), dim3(256), 0, nullptr, out, iters, cyc);
      hipEventRecord(b, nullptr);
      e = hipEventSynchronize(b);
    }
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, a, b);
    if (e == hipSuccess) e = hipMemcpy(host_cyc, cyc, sizeof(host_cyc), hipMemcpyDeviceToHost);
  }
  if (e == hipSuccess) {
    double avg = 0.0;
    for (int i = 0; i < kGrid; ++i) avg += (double)host_cyc[i];
    avg /= kGrid;
    const double flops = (double)kGrid * 4 * iters * 16 * (2.0 * 32 * 32 * 64);
    *tflops = flops / (ms * 1e-3) / 1e12;
    *shader_ghz = avg / (ms * 1e6);
  }
  if (a) hipEventDestroy(a);
  if (b) hipEventDestroy(b);
  if (out) hipFree(out);
  if (cyc) hipFree(cyc);
  return (int)e;
}
