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


// ---------------------------------------------------------------------------
// LDS-tiled kernel on v_mfma_scale_f32_32x32x64_f8f6f4.
//
// Geometry of that instruction (measured on gfx950): lane l supplies row
// i = l % 32 of its operand; with g = l / 32,
//   E2M1 / E3M2: the 32 consecutive K elements of block g of the 64-wide K step;
//   E4M3:        K [16g, 16g+16) in registers 0-3, K [32+16g, 32+16g+16) in 4-7;
//   scale:       the E8M0 byte of (row i, block g), selected by op_sel;
//   result:      column l % 32, rows 8*(v/4) + 4*g + v%4 for v = 0..15.
//
// Workgroup = 4 waves = 256 features x 128 tokens; wave = 128 x 64 (4 x 2 MFMA
// tiles, 128 accumulator registers), two workgroups per CU so one covers the
// other's barrier and memory stalls.  One K stage = 128 elements = one dword of
// scales per row = two MFMA K steps.  Operand tiles go global -> registers ->
// LDS (double buffered) in a fragment-major order: the 16/24 bytes a lane feeds
// to one MFMA lie at (lane * 16 or 24) inside a 1 KB / 1.5 KB fragment, so every
// fragment read is one linear, conflict-free pass over LDS.
// ---------------------------------------------------------------------------
constexpr int kTileN = 256, kTileM = 128, kStageK = 128;
constexpr int kWBytes = kTileN * 64;           // weights, E2M1: 64 B per row per stage
constexpr int kXBytesMax = kTileM * 128;       // activations, E4M3 worst case
constexpr int kStageBytes = kWBytes + kXBytesMax;

struct Seg {
  const uint8_t* a;    // activation codes of the segment
  const uint8_t* b;    // weight codes
  const uint8_t* sfa;  // activation scales
  const uint8_t* sfb;  // weight scales
  int stages;          // kseg / 128
};

template <int FMT> struct RowBytes;   // activation bytes per row per 128-wide stage
template <> struct RowBytes<kFmtE2M1> { static constexpr int v = 64; };
template <> struct RowBytes<kFmtE3M2> { static constexpr int v = 96; };
template <> struct RowBytes<kFmtE4M3> { static constexpr int v = 128; };

struct Staging {
  v4i w[4];
  v4i x[4];
  v4i sw, sx;   // scale dwords of the wave's row tiles for the staged K stage
};

// Per-thread byte offsets of the 16-byte chunks a thread copies each stage,
// relative to the (uniform) start of the tile's rows in the current stage.
template <int FMT>
struct LoadOffsets {
  unsigned w;      // weight chunk k lives at w + k * 64 rows
  unsigned x[3];   // E2M1: x[0] + k * 64 rows; E3M2: x[k]; E4M3: x[0] + k * 32 rows
  __device__ __forceinline__ LoadOffsets(int tid, unsigned ldb, unsigned lda) {
    w = (unsigned)(tid >> 2) * ldb + (tid & 3) * 16;
    if constexpr (FMT == kFmtE2M1) {
      x[0] = (unsigned)(tid >> 2) * lda + (tid & 3) * 16;
    } else if constexpr (FMT == kFmtE3M2) {
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const int id = tid + 256 * k;
        x[k] = (unsigned)(id / 6) * lda + (id % 6) * 16;
      }
    } else {
      x[0] = (unsigned)(tid >> 3) * lda + (tid & 7) * 16;
    }
  }
};

// global -> registers for K stage `q` of a segment
template <int FMT>
__device__ __forceinline__ void stage_load(Staging& st, const Seg& sg, int q, int n0, int m0, int tid, int lane, int wn,
                                           int wm) {
  constexpr int RB = RowBytes<FMT>::v;
  const int nst = sg.stages;
  const unsigned ldb = (unsigned)nst * 64, lda = (unsigned)nst * RB;
  const LoadOffsets<FMT> off(tid, ldb, lda);
  const uint8_t* wbase = sg.b + (size_t)n0 * ldb + (size_t)q * 64;
#pragma unroll
  for (int k = 0; k < 4; ++k) st.w[k] = *reinterpret_cast<const v4i*>(wbase + (size_t)k * 64 * ldb + off.w);
  const uint8_t* xbase = sg.a + (size_t)m0 * lda + (size_t)q * RB;
  if constexpr (FMT == kFmtE2M1) {
#pragma unroll
    for (int k = 0; k < 2; ++k) st.x[k] = *reinterpret_cast<const v4i*>(xbase + (size_t)k * 64 * lda + off.x[0]);
  } else if constexpr (FMT == kFmtE3M2) {
#pragma unroll
    for (int k = 0; k < 3; ++k) st.x[k] = *reinterpret_cast<const v4i*>(xbase + off.x[k]);
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) st.x[k] = *reinterpret_cast<const v4i*>(xbase + (size_t)k * 32 * lda + off.x[0]);
  }
  // scales: the wave's 128 feature rows are one 512-byte atom, its 64 token rows half of one;
  // lane i reads the 16 bytes that hold the dwords of rows i, 32+i, 64+i, 96+i
  const unsigned i16 = (lane & 31) * 16;
  st.sw = *reinterpret_cast<const v4i*>(sg.sfb + ((size_t)((n0 >> 7) + wn) * nst + q) * 512 + i16);
  st.sx = *reinterpret_cast<const v4i*>(sg.sfa + ((size_t)(m0 >> 7) * nst + q) * 512 + i16);
}

// registers -> LDS, fragment-major
template <int FMT>
__device__ __forceinline__ void stage_store(const Staging& st, uint8_t* __restrict__ buf, int tid) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int id = tid + 256 * k, row = id >> 2, c = id & 3;
    // [row tile][h][g][i][16 B] with c = 2h + g
    *reinterpret_cast<v4i*>(buf + (row >> 5) * 2048 + c * 512 + (row & 31) * 16) = st.w[k];
  }
  uint8_t* xb = buf + kWBytes;
  if constexpr (FMT == kFmtE2M1) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int id = tid + 256 * k, row = id >> 2, c = id & 3;
      *reinterpret_cast<v4i*>(xb + (row >> 5) * 2048 + c * 512 + (row & 31) * 16) = st.x[k];
    }
  } else if constexpr (FMT == kFmtE3M2) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int id = tid + 256 * k, row = id / 6, c = id % 6;
      // 16-byte chunk c = 8-byte units 2c, 2c+1 of the row's 12; unit u belongs to fragment u/3
      uint8_t* rb = xb + (row >> 5) * 3072 + (row & 31) * 24;
      const int u0 = 2 * c, u1 = 2 * c + 1;
      *reinterpret_cast<v2i*>(rb + (u0 / 3) * 768 + (u0 % 3) * 8) = v2i{st.x[k][0], st.x[k][1]};
      *reinterpret_cast<v2i*>(rb + (u1 / 3) * 768 + (u1 % 3) * 8) = v2i{st.x[k][2], st.x[k][3]};
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int id = tid + 256 * k, row = id >> 3, c = id & 7;
      // chunk c: K step h = c/4, piece (c%4)/2, lane group g = c%2 -> [row tile][h][piece][g][i][16 B]
      *reinterpret_cast<v4i*>(xb + (row >> 5) * 4096 + (c >> 1) * 1024 + (c & 1) * 512 + (row & 31) * 16) = st.x[k];
    }
  }
}

template <int FMT>
__device__ __forceinline__ void stage_compute(v16f (&acc)[4][2], const uint8_t* __restrict__ buf, v4i sw, v4i sx, int lane,
                                              int wn, int wm) {
  const int g8 = (lane >> 5) * 8;
  int scw[4], scx[2];
#pragma unroll
  for (int t = 0; t < 4; ++t) scw[t] = (int)((unsigned)sw[t] >> g8);
#pragma unroll
  for (int t = 0; t < 2; ++t) scx[t] = (int)((unsigned)sx[2 * wm + t] >> g8);
  const uint8_t* wb = buf + wn * 4 * 2048 + lane * 16;
  const uint8_t* xb = buf + kWBytes;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    v8i wf[4], xf[2];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const v4i v = *reinterpret_cast<const v4i*>(wb + t * 2048 + h * 1024);
      wf[t] = __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int rt = wm * 2 + t;
      if constexpr (FMT == kFmtE2M1) {
        const v4i v = *reinterpret_cast<const v4i*>(xb + rt * 2048 + h * 1024 + lane * 16);
        xf[t] = __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1);
      } else if constexpr (FMT == kFmtE3M2) {
        const v2i* p = reinterpret_cast<const v2i*>(xb + rt * 3072 + h * 1536 + lane * 24);
        const v2i a = p[0], b = p[1], c = p[2];
        const v4i ab = __builtin_shufflevector(a, b, 0, 1, 2, 3);
        const v4i cc = __builtin_shufflevector(c, c, 0, 1, -1, -1);
        xf[t] = __builtin_shufflevector(ab, cc, 0, 1, 2, 3, 4, 5, -1, -1);
      } else {
        const v4i a = *reinterpret_cast<const v4i*>(xb + rt * 4096 + h * 2048 + lane * 16);
        const v4i b = *reinterpret_cast<const v4i*>(xb + rt * 4096 + h * 2048 + 1024 + lane * 16);
        xf[t] = v8i{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
      }
    }
#pragma unroll
    for (int tn = 0; tn < 4; ++tn)
#pragma unroll
      for (int tm = 0; tm < 2; ++tm) {
        if (h == 0)
          acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[tn], xf[tm], acc[tn][tm], kFmtE2M1, FMT, 0,
                                                                        scw[tn], 0, scx[tm]);
        else
          acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[tn], xf[tm], acc[tn][tm], kFmtE2M1, FMT, 2,
                                                                        scw[tn], 2, scx[tm]);
      }
  }
}

// Runs the stages of one segment.  On entry the staging registers hold stage 0 of
// this segment; on exit they hold stage 0 of the next segment (if any).
template <int FMT, int FMT_NEXT>
__device__ __forceinline__ void segment_tiled(v16f (&acc)[4][2], Staging& st, const Seg& sg, const Seg& next,
                                              uint8_t* __restrict__ lds, int& parity, int n0, int m0, int tid, int lane,
                                              int wn, int wm) {
  for (int q = 0; q < sg.stages; ++q) {
    uint8_t* buf = lds + parity * kStageBytes;
    stage_store<FMT>(st, buf, tid);
    const v4i sw = st.sw, sx = st.sx;
    if (q + 1 < sg.stages)
      stage_load<FMT>(st, sg, q + 1, n0, m0, tid, lane, wn, wm);
    else if (next.stages > 0)
      stage_load<FMT_NEXT>(st, next, 0, n0, m0, tid, lane, wn, wm);
    __syncthreads();
    stage_compute<FMT>(acc, buf, sw, sx, lane, wn, wm);
    parity ^= 1;
  }
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
mixed_gemm_tiled_kernel(Seg s4, Seg s6, Seg s8, int M, int N, uint16_t* __restrict__ d) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave & 1, wm = wave >> 1;
  const int n0 = blockIdx.x * kTileN, m0 = blockIdx.y * kTileM;

  v16f acc[4][2];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  Staging st;
  int parity = 0;
  const Seg none = {nullptr, nullptr, nullptr, nullptr, 0};
  // prime the staging registers with the first stage of the first non-empty segment
  if (s4.stages > 0) stage_load<kFmtE2M1>(st, s4, 0, n0, m0, tid, lane, wn, wm);
  else if (s6.stages > 0) stage_load<kFmtE3M2>(st, s6, 0, n0, m0, tid, lane, wn, wm);
  else if (s8.stages > 0) stage_load<kFmtE4M3>(st, s8, 0, n0, m0, tid, lane, wn, wm);

  if (s6.stages > 0) segment_tiled<kFmtE2M1, kFmtE3M2>(acc, st, s4, s6, lds, parity, n0, m0, tid, lane, wn, wm);
  else               segment_tiled<kFmtE2M1, kFmtE4M3>(acc, st, s4, s8, lds, parity, n0, m0, tid, lane, wn, wm);
  segment_tiled<kFmtE3M2, kFmtE4M3>(acc, st, s6, s8, lds, parity, n0, m0, tid, lane, wn, wm);
  segment_tiled<kFmtE4M3, kFmtE4M3>(acc, st, s8, none, lds, parity, n0, m0, tid, lane, wn, wm);

  // result tile is D^T: lane holds token m = lane % 32, features 8*(v/4) + 4*(lane/32) + v%4
  const int g = lane >> 5;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    const int m = m0 + wm * 64 + tm * 32 + (lane & 31);
    uint16_t* row = d + (size_t)m * N + n0 + wn * 128 + 4 * g;
#pragma unroll
    for (int tn = 0; tn < 4; ++tn)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const v2bf lo = {(__bf16)acc[tn][tm][4 * vq + 0], (__bf16)acc[tn][tm][4 * vq + 1]};
        const v2bf hi = {(__bf16)acc[tn][tm][4 * vq + 2], (__bf16)acc[tn][tm][4 * vq + 3]};
        *reinterpret_cast<v2u*>(row + tn * 32 + vq * 8) =
            v2u{__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
      }
  }
}

}  // namespace

hipError_t launch_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                             const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                             const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo, int M,
                             int N, int KN, int KS, int KO, void* d, hipStream_t stream) {
  if (M == 0 || N == 0) return hipSuccess;
  // the tiled kernel needs whole tiles and whole 128-wide K stages
  if (M % kTileM == 0 && N % kTileN == 0 && KN % kStageK == 0 && KS % kStageK == 0 && KO % kStageK == 0 &&
      KN + KS + KO > 0) {
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mixed_gemm_tiled_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kStageBytes);
      if (e != hipSuccess) return e;
      configured = true;
    }
    const Seg s4 = {an, bn, sfan, sfbn, KN / kStageK};
    const Seg s6 = {as_, bs, sfas, sfbs, KS / kStageK};
    const Seg s8 = {ao, bo, sfao, sfbo, KO / kStageK};
    hipLaunchKernelGGL(mixed_gemm_tiled_kernel, dim3(N / kTileN, M / kTileM), dim3(256), 2 * kStageBytes, stream, s4, s6,
                       s8, M, N, static_cast<uint16_t*>(d));
    return hipGetLastError();
  }
  dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
  hipLaunchKernelGGL(mixed_gemm_direct_kernel, grid, dim3(256), 0, stream, an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs,
                     sfao, sfbo, M, N, KN, KS, KO, static_cast<uint16_t*>(d));
  return hipGetLastError();
}

}  // namespace mg
