// Calibration step that produces the reorder index: per-channel absolute maximum over the rows of
// a bf16 activation sample, channels sorted by it in ascending order, index as int16 (the commented
// lines main.py:31-33 of the reference: torch.max(torch.abs(X), dim=0) -> torch.sort ascending ->
// .to(torch.int16)).  Ties are broken by channel number (a stable sort; torch.sort leaves the
// order of equal keys open).
//
// Pass 1 (HBM-bound, reads X once): a workgroup reduces a strip of rows for a chunk of 2048
// columns with 16-byte loads and writes one row of partial maxima (the bf16 bit patterns with the
// sign cleared order like the values).  Pass 2 folds the partials into unique 32-bit keys
// (absmax bits << 16 | channel); pass 3 ranks every key against all others.
#include "mg_common.h"

namespace mg {

namespace {

constexpr int kStrips = 256;         // row strips of pass 1 = rows of partial maxima
constexpr int kColsPerGroup = 2048;  // 256 lanes x 8 columns

__global__ void __launch_bounds__(256)
column_absmax_kernel(const uint16_t* __restrict__ x, int rows, int K, uint16_t* __restrict__ partial) {
  const int strip = blockIdx.y, nstrips = gridDim.y;
  const int c0 = blockIdx.x * kColsPerGroup + threadIdx.x * 8;
  const int r0 = (int)((long long)rows * strip / nstrips), r1 = (int)((long long)rows * (strip + 1) / nstrips);
  v4u m = {0, 0, 0, 0};
  if (c0 < K) {   // K is a multiple of 32, so a lane's 8 columns are all inside or all outside
    const uint16_t* p = x + (size_t)r0 * K + c0;
    int r = r0;
    for (; r + 4 <= r1; r += 4) {
      v4u v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const v4u*>(p + (size_t)u * K);
      p += (size_t)4 * K;
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned a = v[u][j] & 0x7fff7fffu;   // |x| of both halves
          const unsigned lo = max(a & 0xffffu, m[j] & 0xffffu), hi = max(a >> 16, m[j] >> 16);
          m[j] = lo | (hi << 16);
        }
    }
    for (; r < r1; ++r) {
      const v4u v = *reinterpret_cast<const v4u*>(p);
      p += K;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const unsigned a = v[j] & 0x7fff7fffu;
        const unsigned lo = max(a & 0xffffu, m[j] & 0xffffu), hi = max(a >> 16, m[j] >> 16);
        m[j] = lo | (hi << 16);
      }
    }
    *reinterpret_cast<v4u*>(partial + (size_t)strip * K + c0) = m;
  }
}

// Folds the strips of partial maxima into one unique 32-bit key per channel:
// (absmax bits << 16) | channel.  Sorting the keys sorts by absmax with ties by channel number.
// A workgroup folds 64 channels: 8 lanes x 8 channels wide, 32 lanes deep over the strips.
__global__ void __launch_bounds__(256)
channel_keys_kernel(const uint16_t* __restrict__ partial, int nstrips, int K, unsigned* __restrict__ keys) {
  __shared__ v4u part[32][8];
  const int cl = threadIdx.x & 7, sl = threadIdx.x >> 3;
  const int c0 = blockIdx.x * 64 + cl * 8;
  v4u m = {0, 0, 0, 0};
  if (c0 < K) {
#pragma unroll 4
    for (int s = sl; s < nstrips; s += 32) {
      const v4u v = *reinterpret_cast<const v4u*>(partial + (size_t)s * K + c0);
#pragma unroll
      for (int j = 0; j < 4; ++j) m[j] = max(v[j] & 0xffffu, m[j] & 0xffffu) | (max(v[j] >> 16, m[j] >> 16) << 16);
    }
  }
  part[sl][cl] = m;
  __syncthreads();
  if (threadIdx.x < 64) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    const uint16_t* col = reinterpret_cast<const uint16_t*>(&part[0][0]) + threadIdx.x;
    unsigned best = 0;
#pragma unroll
    for (int s = 0; s < 32; ++s) best = max(best, (unsigned)col[s * 64]);
    if (c < K) keys[c] = (best << 16) | (unsigned)c;
  }
}

// The keys are unique, so the position of a channel in the sorted order is the number of smaller
// keys.  A workgroup ranks 64 channels (one per lane); its 16 waves each count over a sixteenth of
// the K keys, read from LDS at a wave-uniform address (a broadcast), and the counts are added
// through LDS.  K^2 compares in total over K/64 workgroups; the channel number is scattered to its rank.
constexpr int kRankWaves = 16;

__global__ void __launch_bounds__(kRankWaves * 64)
rank_channels_kernel(const unsigned* __restrict__ keys, int K, int16_t* __restrict__ idx) {
  extern __shared__ __align__(16) unsigned lds_keys[];   // K keys, then kRankWaves x 64 counts
  int* counts = reinterpret_cast<int*>(lds_keys + K);
  for (int c = threadIdx.x * 4; c < K; c += kRankWaves * 64 * 4)
    *reinterpret_cast<v4u*>(lds_keys + c) = *reinterpret_cast<const v4u*>(keys + c);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = blockIdx.x * 64 + lane;
  const unsigned mine = c < K ? lds_keys[c] : 0u;
  const int chunk = ceil_div(K / 4, kRankWaves) * 4;
  const int j0 = wave * chunk, j1 = min(K, j0 + chunk);
  int rank = 0;
#pragma unroll 4
  for (int j = j0; j < j1; j += 4) {
    const v4u q = *reinterpret_cast<const v4u*>(lds_keys + j);
#pragma unroll
    for (int e = 0; e < 4; ++e) rank += q[e] < mine ? 1 : 0;
  }
  counts[wave * 64 + lane] = rank;
  __syncthreads();
  if (wave == 0 && c < K) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kRankWaves; ++w) total += counts[w * 64 + lane];
    idx[total] = (int16_t)c;
  }
}

}  // namespace

// partial maxima (kStrips x K x 2 B, a multiple of 16) followed by the K keys
size_t calibrate_workspace_bytes(int K) { return (size_t)kStrips * K * sizeof(uint16_t) + (size_t)K * sizeof(unsigned); }

hipError_t launch_calibrate(const void* x, int rows, int K, int16_t* idx, void* workspace, hipStream_t stream) {
  uint16_t* partial = static_cast<uint16_t*>(workspace);
  unsigned* keys = reinterpret_cast<unsigned*>(partial + (size_t)kStrips * K);
  const int nstrips = rows < kStrips ? rows : kStrips;
  hipLaunchKernelGGL(column_absmax_kernel, dim3(ceil_div(K, kColsPerGroup), nstrips), dim3(256), 0, stream,
                     static_cast<const uint16_t*>(x), rows, K, partial);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(channel_keys_kernel, dim3(ceil_div(K, 64)), dim3(256), 0, stream, partial, nstrips, K, keys);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  e = allow_dynamic_lds(reinterpret_cast<const void*>(rank_channels_kernel), (32768 + kRankWaves * 64) * (int)sizeof(unsigned));
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(rank_channels_kernel, dim3(ceil_div(K, 64)), dim3(kRankWaves * 64),
                     (size_t)(K + kRankWaves * 64) * sizeof(unsigned), stream, keys, K, idx);
  return hipGetLastError();
}

}  // namespace mg
