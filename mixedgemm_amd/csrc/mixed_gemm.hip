// Mixed block-scaled GEMM for gfx950 on v_mfma_scale_f32_16x16x128_f8f6f4.
//
//   D[m][n] = bf16( sum_seg sum_kb 2^(sfa-127) 2^(sfb-127) sum_{32} a*b )
//
// replacing the reference's three chained CUTLASS segment GEMMs
// (src/gemm.cu:44-46; src/fp4.cu:35, src/fp6.cu:35, src/fp8.cu:35): all three K
// segments (E2M1, E3M2, E4M3 activations against E2M1 weights) accumulate into
// one fp32 tile and D is rounded to bf16 once.
//
// The weights are fed as the MFMA's first operand and the activations as the
// second, so the 16x16 result tile is D^T: a lane ends up with four consecutive
// output features n of one token m, which are adjacent in row-major D.
//
// Operand geometry of the instruction (measured on gfx950): lane l supplies row
// i = l % 16 of its operand; with g = l / 16,
//   E2M1 / E3M2: the 32 consecutive K elements of block g of the 128-wide K
//                step -- one MX block, 16 or 24 contiguous bytes;
//   E4M3:        K elements [16g, 16g+16) in registers 0-3 and
//                [64+16g, 64+16g+16) in registers 4-7 (two 16-byte pieces);
// and, for every format, the E8M0 scale of block g of row i in the byte of the
// scale register that op_sel selects.
#include "mg_common.h"

namespace mg {

namespace {

template <int FMT>
struct Frag;
template <> struct Frag<kFmtE2M1> { static constexpr int kBytes = 16; };
template <> struct Frag<kFmtE3M2> { static constexpr int kBytes = 24; };
template <> struct Frag<kFmtE4M3> { static constexpr int kBytes = 32; };

// Load one lane's fragment of a 128-wide K step into the low dwords of v8i.
// `step` points at the start of the K step in the lane's row; blocks at or past
// `blocks_left` (counted from the start of the step) read as zero.
template <int FMT>
__device__ __forceinline__ v8i load_frag(const uint8_t* __restrict__ step, int g, int blocks_left, bool row_ok) {
  v8i f = {0, 0, 0, 0, 0, 0, 0, 0};
  if constexpr (FMT == kFmtE2M1) {
    if (row_ok && g < blocks_left) {
      const v4i t = *reinterpret_cast<const v4i*>(step + g * 16);
      f[0] = t[0]; f[1] = t[1]; f[2] = t[2]; f[3] = t[3];
    }
  } else if constexpr (FMT == kFmtE3M2) {
    if (row_ok && g < blocks_left) {
      const v2i* q = reinterpret_cast<const v2i*>(step + g * 24);
      const v2i t0 = q[0], t1 = q[1], t2 = q[2];
      f[0] = t0[0]; f[1] = t0[1]; f[2] = t1[0]; f[3] = t1[1]; f[4] = t2[0]; f[5] = t2[1];
    }
  } else {
    // two 16-element pieces: K [16g, 16g+16) in block g/2 and K [64+16g, ...) in block 2 + g/2
    if (row_ok && (g >> 1) < blocks_left) {
      const v4i t = *reinterpret_cast<const v4i*>(step + g * 16);
      f[0] = t[0]; f[1] = t[1]; f[2] = t[2]; f[3] = t[3];
    }
    if (row_ok && 2 + (g >> 1) < blocks_left) {
      const v4i t = *reinterpret_cast<const v4i*>(step + 64 + g * 16);
      f[4] = t[0]; f[5] = t[1]; f[6] = t[2]; f[7] = t[3];
    }
  }
  return f;
}

// One K segment, operands read straight from global memory.  Wave tile:
// 16 tokens x (16*NT) output features.
template <int FMT, int NT>
__device__ __forceinline__ void segment_direct(v4f (&acc)[NT], const uint8_t* __restrict__ a, const uint8_t* __restrict__ sfa,
                                               const uint8_t* __restrict__ b, const uint8_t* __restrict__ sfb, int kseg,
                                               int m, bool m_ok, int n_base, int N, int lane) {
  const int nblk = kseg >> 5;
  if (nblk == 0) return;
  const int katoms = (kseg + 127) >> 7;
  const int g = lane >> 4, i = lane & 15;
  const size_t lda = (size_t)nblk * Frag<FMT>::kBytes;
  const size_t ldb = (size_t)nblk * 16;
  for (int q = 0; q < katoms; ++q) {
    const int kb = 4 * q + g;
    const int left = nblk - 4 * q;
    const bool k_ok = kb < nblk;
    const v8i xa = load_frag<FMT>(a + (size_t)m * lda + (size_t)q * 4 * Frag<FMT>::kBytes, g, left, m_ok);
    const int sx = (k_ok && m_ok) ? (int)sfa[sf_offset(m, kb, katoms)] : 127;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = n_base + 16 * t + i;
      const bool b_ok = k_ok && n < N;
      const v8i wb = load_frag<kFmtE2M1>(b + (size_t)n * ldb + (size_t)q * 64, g, left, n < N);
      const int sw = b_ok ? (int)sfb[sf_offset(n, kb, katoms)] : 127;
      acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wb, xa, acc[t], kFmtE2M1, FMT, 0, sw, 0, sx);
    }
  }
}

// Generic kernel for any M, N and 32-granular segments: no LDS, every wave
// fetches its own fragments.  Workgroup = 4 waves = 64 tokens x 64 features.
__global__ void __launch_bounds__(256)
mixed_gemm_direct_kernel(const uint8_t* __restrict__ an, const uint8_t* __restrict__ bn, const uint8_t* __restrict__ as_,
                         const uint8_t* __restrict__ bs, const uint8_t* __restrict__ ao, const uint8_t* __restrict__ bo,
                         const uint8_t* __restrict__ sfan, const uint8_t* __restrict__ sfbn,
                         const uint8_t* __restrict__ sfas, const uint8_t* __restrict__ sfbs,
                         const uint8_t* __restrict__ sfao, const uint8_t* __restrict__ sfbo, int M, int N, int KN, int KS,
                         int KO, uint16_t* __restrict__ d) {
  constexpr int NT = 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.y * 64 + wave * 16 + (lane & 15);
  const int n_base = blockIdx.x * 64;
  const bool m_ok = m < M;
  v4f acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

  segment_direct<kFmtE2M1, NT>(acc, an, sfan, bn, sfbn, KN, m, m_ok, n_base, N, lane);
  segment_direct<kFmtE3M2, NT>(acc, as_, sfas, bs, sfbs, KS, m, m_ok, n_base, N, lane);
  segment_direct<kFmtE4M3, NT>(acc, ao, sfao, bo, sfbo, KO, m, m_ok, n_base, N, lane);

  // result tile is D^T: lane holds token m = lane%16, features 4*(lane/16) + v
  if (!m_ok) return;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = n_base + 16 * t + 4 * (lane >> 4);
    uint16_t h[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) h[v] = __builtin_bit_cast(uint16_t, (__bf16)acc[t][v]);
    uint16_t* dst = d + (size_t)m * N + n;
    if (n + 3 < N && (N & 3) == 0) {
      *reinterpret_cast<v2u*>(dst) = v2u{(unsigned)h[0] | ((unsigned)h[1] << 16), (unsigned)h[2] | ((unsigned)h[3] << 16)};
    } else {
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (n + v < N) dst[v] = h[v];
    }
  }
}

}  // namespace

hipError_t launch_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                             const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                             const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo, int M,
                             int N, int KN, int KS, int KO, void* d, hipStream_t stream) {
  if (M == 0 || N == 0) return hipSuccess;
  dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
  hipLaunchKernelGGL(mixed_gemm_direct_kernel, grid, dim3(256), 0, stream, an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs,
                     sfao, sfbo, M, N, KN, KS, KO, static_cast<uint16_t*>(d));
  return hipGetLastError();
}

}  // namespace mg
