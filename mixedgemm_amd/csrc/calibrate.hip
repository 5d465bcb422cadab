// Calibration step that produces the reorder index: per-channel absolute maximum over the rows of
// a bf16 activation sample, channels sorted by it in ascending order, index as int16 (the commented
// lines main.py:31-33 of the reference: torch.max(torch.abs(X), dim=0) -> torch.sort ascending ->
// .to(torch.int16)).  Ties are broken by channel number (a stable sort; torch.sort leaves the
// order of equal keys open).
//
// Two launches.  Pass 1 (HBM-bound, reads X once): a workgroup reduces a strip of rows for a group of
// kColLanes * 8 columns -- kColLanes lanes wide with 16-byte loads, 256 / kColLanes lanes deep over the
// rows --, folds its row lanes through LDS and writes one row of partial maxima (the bf16 bit patterns with
// the sign cleared order like the values).  The strips are few (kStrips), so that pass 2 can afford to fold
// them in every workgroup: each folds the partials of all K channels into unique 32-bit keys
// (absmax bits << 16 | channel) in LDS and ranks 16 channels against all keys.
#include "mg_common.h"

namespace mg {

namespace {

constexpr int kStrips = 8;                   // row strips of pass 1 = rows of partial maxima
constexpr int kColLanes = 16;                // lanes across the columns of a group
constexpr int kRowLanes = 256 / kColLanes;   // lanes over the rows of a strip
constexpr int kColsPerGroup = kColLanes * 8;
constexpr int kInFlight = 8;                 // loads a lane has outstanding

__device__ __forceinline__ void absmax_fold(v4u& m, const v4u& v) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned a = v[j] & 0x7fff7fffu;   // |x| of both halves
    const unsigned lo = max(a & 0xffffu, m[j] & 0xffffu), hi = max(a >> 16, m[j] >> 16);
    m[j] = lo | (hi << 16);
  }
}

__global__ void __launch_bounds__(256)
column_absmax_kernel(const uint16_t* __restrict__ x, int rows, int K, uint16_t* __restrict__ partial) {
  __shared__ v4u part[kRowLanes][kColLanes];
  const int strip = blockIdx.y, nstrips = gridDim.y;
  const int cl = threadIdx.x % kColLanes, rl = threadIdx.x / kColLanes;
  const int c0 = blockIdx.x * kColsPerGroup + cl * 8;
  const int r0 = (int)((long long)rows * strip / nstrips), r1 = (int)((long long)rows * (strip + 1) / nstrips);
  v4u m = {0, 0, 0, 0};
  if (c0 < K) {   // K is a multiple of 32, so a lane's 8 columns are all inside or all outside
    int r = r0 + rl;
    const uint16_t* p = x + (size_t)r * K + c0;
    const size_t step = (size_t)kRowLanes * K;
    for (; r + (kInFlight - 1) * kRowLanes < r1; r += kInFlight * kRowLanes) {
      v4u v[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) v[u] = *reinterpret_cast<const v4u*>(p + u * step);
      p += kInFlight * step;
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) absmax_fold(m, v[u]);
    }
    for (; r < r1; r += kRowLanes) {
      absmax_fold(m, *reinterpret_cast<const v4u*>(p));
      p += step;
    }
  }
  part[rl][cl] = m;
  __syncthreads();
  if (threadIdx.x < kColLanes && c0 < K) {
    v4u best = part[0][cl];
#pragma unroll
    for (int s = 1; s < kRowLanes; ++s) {
      const v4u v = part[s][cl];
#pragma unroll
      for (int j = 0; j < 4; ++j) best[j] = max(v[j] & 0xffffu, best[j] & 0xffffu) | (max(v[j] >> 16, best[j] >> 16) << 16);
    }
    *reinterpret_cast<v4u*>(partial + (size_t)strip * K + c0) = best;
  }
}

// The keys are unique, so the position of a channel in the sorted order is the number of smaller keys.
// Every workgroup folds the strips of partial maxima for all K channels (8 channels per lane and pass) into the
// keys, kept in LDS, and ranks 16 channels: a lane counts, for channel lane % 16, the smaller keys in one
// of kRankSlices slices of the K keys (sixteen lanes of a wave read the same 16 bytes of LDS: a broadcast), the counts
// of a channel are added through LDS, and the channel number is scattered to its rank.  K^2 compares in total over
// K/16 workgroups of 8 waves (two per SIMD: one wave's LDS latency under the other's compares).
constexpr int kRankChannels = 16, kRankSlices = 32, kRankThreads = kRankChannels * kRankSlices;

__global__ void __launch_bounds__(kRankThreads)
rank_channels_kernel(const uint16_t* __restrict__ partial, int nstrips, int K, int16_t* __restrict__ idx) {
  extern __shared__ __align__(16) unsigned lds_keys[];   // K keys, then kRankSlices x kRankChannels counts
  int* counts = reinterpret_cast<int*>(lds_keys + K);
  for (int c0 = threadIdx.x * 8; c0 < K; c0 += kRankThreads * 8) {
    // all strips requested at once (a strip past the last one reads the last one again: a maximum does not mind)
    v4u v[kStrips];
    const uint16_t* p = partial + c0;
#pragma unroll
    for (int s = 0; s < kStrips; ++s) v[s] = *reinterpret_cast<const v4u*>(p + (size_t)min(s, nstrips - 1) * K);
    v4u m = v[0];
#pragma unroll
    for (int s = 1; s < kStrips; ++s)
#pragma unroll
      for (int j = 0; j < 4; ++j) m[j] = max(v[s][j] & 0xffffu, m[j] & 0xffffu) | (max(v[s][j] >> 16, m[j] >> 16) << 16);
    v4u k0, k1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      k0[2 * j] = (m[j] << 16) | (unsigned)(c0 + 2 * j);
      k0[2 * j + 1] = (m[j] & 0xffff0000u) | (unsigned)(c0 + 2 * j + 1);
      k1[2 * j] = (m[2 + j] << 16) | (unsigned)(c0 + 4 + 2 * j);
      k1[2 * j + 1] = (m[2 + j] & 0xffff0000u) | (unsigned)(c0 + 4 + 2 * j + 1);
    }
    *reinterpret_cast<v4u*>(lds_keys + c0) = k0;
    *reinterpret_cast<v4u*>(lds_keys + c0 + 4) = k1;
  }
  __syncthreads();
  const int ch = threadIdx.x % kRankChannels, slice = threadIdx.x / kRankChannels;
  const int c = blockIdx.x * kRankChannels + ch;
  const unsigned mine = c < K ? lds_keys[c] : 0u;
  const int chunk = ceil_div(K / 4, kRankSlices) * 4;
  const int j0 = slice * chunk, j1 = min(K, j0 + chunk);
  int rank = 0;
#pragma unroll 8
  for (int j = j0; j < j1; j += 4) {
    const v4u q = *reinterpret_cast<const v4u*>(lds_keys + j);
#pragma unroll
    for (int e = 0; e < 4; ++e) rank += q[e] < mine ? 1 : 0;
  }
  counts[slice * kRankChannels + ch] = rank;
  __syncthreads();
  if (threadIdx.x < kRankChannels && c < K) {
    int total = 0;
#pragma unroll
    for (int s = 0; s < kRankSlices; ++s) total += counts[s * kRankChannels + ch];
    idx[total] = (int16_t)c;
  }
}

}  // namespace

// kStrips rows of partial maxima (K x 2 B each, a multiple of 16)
size_t calibrate_workspace_bytes(int K) { return (size_t)kStrips * K * sizeof(uint16_t); }

hipError_t launch_calibrate(const void* x, int rows, int K, int16_t* idx, void* workspace, hipStream_t stream) {
  uint16_t* partial = static_cast<uint16_t*>(workspace);
  // a strip has at least one row per row lane where the sample has that many rows
  const int nstrips = rows >= kStrips * kRowLanes ? kStrips : (rows + kRowLanes - 1) / kRowLanes;
  hipLaunchKernelGGL(column_absmax_kernel, dim3(ceil_div(K, kColsPerGroup), nstrips), dim3(256), 0, stream,
                     static_cast<const uint16_t*>(x), rows, K, partial);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const size_t lds = (size_t)(K + kRankSlices * kRankChannels) * sizeof(unsigned);
  e = allow_dynamic_lds(reinterpret_cast<const void*>(rank_channels_kernel),
                        (32768 + kRankSlices * kRankChannels) * (int)sizeof(unsigned));
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(rank_channels_kernel, dim3(ceil_div(K, kRankChannels)), dim3(kRankThreads), lds, stream, partial, nstrips, K, idx);
  return hipGetLastError();
}

}  // namespace mg
