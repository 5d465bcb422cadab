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
#include <stdlib.h>

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
// Skinny kernel: few tokens (decode, small batches), weights streamed once per
// 16 * G tokens (HBM- or L2-bound).
//
// A workgroup of 4 waves owns F groups of 16 output features and G groups of 16 tokens; the K
// steps (128 elements each, counted over the three segments) are dealt to the 4
// waves in contiguous quarters.  A wave issues every load of a round of steps
// (weights, the G token groups, scales; addresses clamped, no branches) before
// the round's first MFMA; the 4 partial 16x16 tiles per group are summed through
// LDS and rounded to bf16 once.  G = 1 is the decode case.
// ---------------------------------------------------------------------------
struct DecodeSeg {
  const uint8_t* a;
  const uint8_t* b;
  const uint8_t* sfa;
  const uint8_t* sfb;
  int nblk;    // 32-element blocks in the segment
  int steps;   // ceil(nblk / 4)
};

template <int FMT>
__device__ __forceinline__ v4f decode_mfma(v8i wb, v8i xa, v4f acc, int sw, int sx) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wb, xa, acc, kFmtE2M1, FMT, 0, sw, 0, sx);
}

template <int G, int F>
__global__ void __launch_bounds__(256)
mixed_gemm_skinny_kernel(DecodeSeg s4, DecodeSeg s6, DecodeSeg s8, int M, int N, int steps_per_wave,
                         int w_tiled, uint16_t* __restrict__ d) {
  constexpr int S = G * F >= 8 ? 1 : 8 / (G * F);   // K steps a wave keeps in flight at once
  __shared__ float partial[4][F][G][16 * 16];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, g = lane >> 4;
  // The workgroup owns F groups of 16 features (group index bx = blockIdx.x * F + f) and G groups of 16
  // tokens; an activation fragment is loaded once and used for the F feature groups.
  // Row-major weights: a group is 16 consecutive features.  Tile-major weights: the 16 rows of one
  // 1 KB copy block (block j = bx % 16 of feature tile bx / 16), i.e. features
  // j + 16 * (2 * (t % 8) + t / 8) of the tile for t = 0..15, so that a weight load reads 1 KB of
  // consecutive bytes.
  int tile_row0[F], n[F], nc[F];
  bool n_ok[F];
#pragma unroll
  for (int f = 0; f < F; ++f) {
    const int bx = blockIdx.x * F + f;
    tile_row0[f] = (bx >> 4) * 256 + (bx & 15);
    n[f] = w_tiled ? tile_row0[f] + 16 * (2 * (i & 7) + (i >> 3)) : bx * 16 + i;
    n_ok[f] = n[f] < N;
    nc[f] = min(n[f], N - 1);   // clamped rows: every load is in bounds and unconditional
  }
  const int m0 = blockIdx.y * (G * 16) + i;      // this lane's token in group 0
  const int total = s4.steps + s6.steps + s8.steps;
  v4f acc[F][G];
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int gi = 0; gi < G; ++gi) acc[f][gi] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int r0 = 0; r0 < steps_per_wave; r0 += S) {
    const int t0 = wave * steps_per_wave + r0, t_end = min(total, wave * steps_per_wave + steps_per_wave);

    // Straight-line issue of every load of this round, so all of them are in
    // flight together; masking comes afterwards.
    v4i wq[S][F], xa[S][G], xb[S][G];
    int sw[S][F], sx[S][G];
#pragma unroll
    for (int k = 0; k < S; ++k) {
      const int t = min(t0 + k, total - 1);
      const int seg = t < s4.steps ? 0 : (t < s4.steps + s6.steps ? 1 : 2);
      const int q = seg == 0 ? t : (seg == 1 ? t - s4.steps : t - s4.steps - s6.steps);
      const uint8_t* pa = seg == 0 ? s4.a : (seg == 1 ? s6.a : s8.a);
      const uint8_t* pb = seg == 0 ? s4.b : (seg == 1 ? s6.b : s8.b);
      const uint8_t* psa = seg == 0 ? s4.sfa : (seg == 1 ? s6.sfa : s8.sfa);
      const uint8_t* psb = seg == 0 ? s4.sfb : (seg == 1 ? s6.sfb : s8.sfb);
      const int nblk = seg == 0 ? s4.nblk : (seg == 1 ? s6.nblk : s8.nblk);
      const int katoms = seg == 0 ? s4.steps : (seg == 1 ? s6.steps : s8.steps);
      const int xbytes = seg == 0 ? 16 : (seg == 1 ? 24 : 32);   // activation bytes per 32-element block
      const int left = nblk - 4 * q;
      const int gc = min(g, left - 1);
      // tile-major weights: 16 KB per (256-feature tile, whole step), the group's block in it, lane
      // quad i, piece g; the blocks past the last whole step as rows of (nblk % 4) blocks behind the tiled part
      const int whole = nblk >> 2, rblk = nblk & 3;
#pragma unroll
      for (int f = 0; f < F; ++f) {
        const int bx = blockIdx.x * F + f;
        const size_t w_tiled_off =
            q < whole ? ((((size_t)(bx >> 4) * whole + q) * 16 + (bx & 15)) * 1024 + i * 64 + g * 16)
                      : ((size_t)(N >> 8) * whole * 16384 + (size_t)nc[f] * rblk * 16 + gc * 16);
        const size_t w_off = w_tiled ? w_tiled_off : ((size_t)nc[f] * nblk * 16 + q * 64 + gc * 16);
        wq[k][f] = *reinterpret_cast<const v4i*>(pb + w_off);
        sw[k][f] = psb[sf_offset(nc[f], 4 * q + gc, katoms)];
      }
      // activations: two 16-byte pieces.  E2M1: block g (second piece unused);
      // E3M2: bytes [0,16) and [8,24) of block g; E4M3: K [16g,+16) and [64+16g,+16).
      const int a_blk = seg == 2 ? (g >> 1) : g, b_blk = seg == 2 ? 2 + (g >> 1) : g;
      int off_a = seg == 1 ? g * 24 : g * 16;
      int off_b = seg == 0 ? g * 16 : (seg == 1 ? g * 24 + 8 : 64 + g * 16);
      off_a = a_blk < left ? off_a : 0;
      off_b = b_blk < left ? off_b : 0;
#pragma unroll
      for (int gi = 0; gi < G; ++gi) {
        const int mc = min(m0 + gi * 16, M - 1);
        const uint8_t* xrow = pa + (size_t)mc * nblk * xbytes + q * 4 * xbytes;
        xa[k][gi] = *reinterpret_cast<const v4i*>(xrow + off_a);
        // E2M1 needs one piece only; a wave-uniform branch around the second load pays for G = 4 only (measured)
        if (G != 4 || seg != 0) xb[k][gi] = *reinterpret_cast<const v4i*>(xrow + off_b);
        else xb[k][gi] = v4i{0, 0, 0, 0};
        sx[k][gi] = psa[sf_offset(mc, 4 * q + gc, katoms)];
      }
    }

#pragma unroll
    for (int k = 0; k < S; ++k) {
      const int t = t0 + k;
      if (t < t_end) {   // wave-uniform
        const int seg = t < s4.steps ? 0 : (t < s4.steps + s6.steps ? 1 : 2);
        const int q = seg == 0 ? t : (seg == 1 ? t - s4.steps : t - s4.steps - s6.steps);
        const int nblk = seg == 0 ? s4.nblk : (seg == 1 ? s6.nblk : s8.nblk);
        const int left = nblk - 4 * q;
        const bool blk_ok = g < left;
        const v4i z = {0, 0, 0, 0};
        v8i wf[F];
        int s_w[F];
#pragma unroll
        for (int f = 0; f < F; ++f) {
          const bool w_ok = n_ok[f] && blk_ok;
          const v4i w4 = w_ok ? wq[k][f] : z;
          wf[f] = v8i{w4[0], w4[1], w4[2], w4[3], 0, 0, 0, 0};
          s_w[f] = w_ok ? sw[k][f] : 127;
        }
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
          const bool m_ok = m0 + gi * 16 < M;
          const int s_x = (m_ok && blk_ok) ? sx[k][gi] : 127;
          if (seg == 0) {
            const v4i a4 = (m_ok && blk_ok) ? xa[k][gi] : z;
            const v8i xf = {a4[0], a4[1], a4[2], a4[3], 0, 0, 0, 0};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE2M1>(wf[f], xf, acc[f][gi], s_w[f], s_x);
          } else if (seg == 1) {
            const v4i a4 = (m_ok && blk_ok) ? xa[k][gi] : z;
            const v4i b4 = (m_ok && blk_ok) ? xb[k][gi] : z;
            const v8i xf = {a4[0], a4[1], a4[2], a4[3], b4[2], b4[3], 0, 0};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE3M2>(wf[f], xf, acc[f][gi], s_w[f], s_x);
          } else {
            const v4i a4 = (m_ok && (g >> 1) < left) ? xa[k][gi] : z;
            const v4i b4 = (m_ok && 2 + (g >> 1) < left) ? xb[k][gi] : z;
            const v8i xf = {a4[0], a4[1], a4[2], a4[3], b4[0], b4[1], b4[2], b4[3]};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE4M3>(wf[f], xf, acc[f][gi], s_w[f], s_x);
          }
        }
      }
    }
  }

  // result tile is D^T: lane holds token m = lane % 16, features 4 * (lane / 16) + v
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int gi = 0; gi < G; ++gi) *reinterpret_cast<v4f*>(&partial[wave][f][gi][lane * 4]) = acc[f][gi];
  __syncthreads();
  // the F * G partial tiles are dealt to the 4 waves round-robin
#pragma unroll
  for (int fg = 0; fg < F * G; ++fg) {
    if ((fg & 3) != wave) continue;
    const int f = fg / G, gi = fg % G;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) sum += *reinterpret_cast<const v4f*>(&partial[w][f][gi][lane * 4]);
    const int nn = (blockIdx.x * F + f) * 16 + 4 * g;
    const int m = m0 + gi * 16;
    if (m < M) {
      if (w_tiled) {   // feature 4g + v of the group is row tile_row0 + 16 * (2 * (t % 8) + t / 8), t = 4g + v
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int t = 4 * g + v;
          const int row = tile_row0[f] + 16 * (2 * (t & 7) + (t >> 3));
          if (row < N) d[(size_t)m * N + row] = __builtin_bit_cast(uint16_t, (__bf16)sum[v]);
        }
      } else {
        uint16_t* dst = d + (size_t)m * N + nn;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (nn + v < N) dst[v] = __builtin_bit_cast(uint16_t, (__bf16)sum[v]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Decode kernel: 16 G tokens per workgroup (G = 1: up to 16 tokens in all; G = 2: up to 255 tokens, 32 per workgroup,
// where their codes fit the LDS), whole 128-wide K steps.
//
// The skinny kernel above issues seven loads per K step and wave, five of them for a few bytes each (the
// token fragment twice, three scale bytes); the address unit handles those as slowly as the two 1 KB weight
// loads, and with 31 MB to stream in a few microseconds that is what bounds it.  Here everything that is not
// a weight code goes global -> LDS once per workgroup in 1 KB copies (global_load_lds_dwordx4): the token
// codes of all three segments (M x 2464 bytes for K = 4096) and, per K step, the 16-byte pieces of the scale
// atoms that hold the workgroup's rows; the K loop reads them from LDS.  The weight codes go to registers,
// eight K steps per wave in flight at a time, in two rounds of four.  All
// requests are inline assembly, so that the waits can count them (requests complete in order).
//
// Which features a workgroup owns follows the scale atoms: a 16-byte piece of an atom holds rows c, c + 32,
// c + 64, c + 96 of a group of 128 (c = row % 32).  Row-major weights: the workgroup of 16 F features takes
// pieces c0 ... c0 + 4F - 1 of one group, i.e. rows c0 + (i % (4F)) + 32 (i / (4F)) for i = 0 ... 16F - 1 (its
// results are still runs of four consecutive features).  Tile-major weights: a workgroup takes F of the 1 KB
// copy blocks of a 256-feature tile (rows j + 32 t + 16 u, t = 0..7, u = 0, 1), whose scales are pieces j and
// j + 16 of both groups of the tile.  Either way the scales of a step are 64 F contiguous-by-piece bytes.
//
// Workgroup = 4 waves; the K steps (over the three segments) are dealt to the waves in contiguous quarters;
// partial tiles are summed through LDS.
// ---------------------------------------------------------------------------
struct DecodeLds {
  int x0, x1, x2;        // byte offsets of the token codes per segment
  int sfa0, sfa1, sfa2;  // of the token scale pieces: per step pa pieces of 16 bytes (piece p: tokens p, p + 32, p + 64, p + 96 of a group of 128)
  int sfb0, sfb1, sfb2;  // of the weight scale pieces: per step 4 F pieces
  int partial;           // of the partial sums
  int total;
  int pa;                // 8 (up to 8 tokens), 16, or 32 (G = 2: the whole atom of the workgroup's group of 128 tokens)
};

// value of segment seg (0, 1, 2) by masking: a select between struct fields invites the compiler to index a private
// copy of the struct, which lands in scratch memory
__device__ __forceinline__ int sel3(int seg, int v0, int v1, int v2) {
  return (v0 & (seg == 0 ? -1 : 0)) | (v1 & (seg == 1 ? -1 : 0)) | (v2 & (seg == 2 ? -1 : 0));
}
__device__ __forceinline__ const uint8_t* sel3p(int seg, const uint8_t* p0, const uint8_t* p1, const uint8_t* p2) {
  const uint64_t m0 = seg == 0 ? ~0ull : 0ull, m1 = seg == 1 ? ~0ull : 0ull, m2 = seg == 2 ? ~0ull : 0ull;
  return reinterpret_cast<const uint8_t*>((reinterpret_cast<uint64_t>(p0) & m0) | (reinterpret_cast<uint64_t>(p1) & m1) |
                                          (reinterpret_cast<uint64_t>(p2) & m2));
}

__device__ __forceinline__ void dma16_at(const uint8_t* base, unsigned voff, unsigned lds_off) {
  // base and lds_off are wave-uniform; say so to the compiler
  const uint64_t bv = reinterpret_cast<uint64_t>(base);
  // (the builtin returns int: without the casts the low half would be sign-extended over the high half)
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)bv);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(bv >> 32));
  base = reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
  lds_off = __builtin_amdgcn_readfirstlane(lds_off);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_off) : "memory", "m0");
}

// Copies `bytes` (a multiple of 16) from src to LDS offset dst in units of 1 KB, unit u by wave u % 4; lanes past
// the end copy the last 16 bytes again (into the padding that rounds every region up to whole units).
__device__ __forceinline__ void copy_region(const uint8_t* src, int bytes, unsigned dst, int wave, int lane) {
  const int units = (bytes + 1023) >> 10, chunks = bytes >> 4;
  for (int u = wave; u < units; u += 4)
    dma16_at(src, (unsigned)min(u * 64 + lane, chunks - 1) * 16u, dst + (unsigned)u * 1024u);
}

// Copies P (4, 8 or 16, a power of two) 16-byte pieces per K step of a segment's scale atoms (512 bytes per step)
// to LDS as [step][piece]; piece_off is this lane's piece (lane % P) as a byte offset inside the atom (and, for
// pieces of another group of 128 rows, that group's distance).  Units of 1 KB = 64 / P steps, unit u by wave u % 4;
// steps past the last one copy it again (into the region's padding).
// P = 1 << plog pieces per step (a power of two: no divisions by a run-time value here)
__device__ __forceinline__ void copy_pieces(const uint8_t* src, int steps, int plog, unsigned piece_off, unsigned dst,
                                            int wave, int lane) {
  const int per_unit = 64 >> plog, units = (steps + per_unit - 1) >> (6 - plog);
  for (int u = wave; u < units; u += 4) {
    const int q = min(u * per_unit + (lane >> plog), steps - 1);
    dma16_at(src, (unsigned)q * 512u + piece_off, dst + (unsigned)u * 1024u);
  }
}

// All arguments into scalar registers in one batch of loads: fetched where they are first used they cost a round trip
// to the argument buffer each time, before the first weight is requested.
__device__ __forceinline__ void pin_args(DecodeSeg& s) {
  asm volatile("" : "+s"(s.a), "+s"(s.b), "+s"(s.sfa), "+s"(s.sfb), "+s"(s.nblk), "+s"(s.steps));
}
__device__ __forceinline__ void pin_args(DecodeLds& l) {
  asm volatile("" : "+s"(l.x0), "+s"(l.x1), "+s"(l.x2), "+s"(l.sfa0), "+s"(l.sfa1), "+s"(l.sfa2), "+s"(l.sfb0), "+s"(l.sfb1),
               "+s"(l.sfb2), "+s"(l.partial), "+s"(l.total), "+s"(l.pa));
}

// 16 bytes global -> registers as an instruction the compiler does not count; use after s_waitcnt + tie()
__device__ __forceinline__ void load16_uncounted(v4i& dst, const uint8_t* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
// the same from a wave-uniform base (scalar registers), a 32-bit per-lane offset and an immediate: one instruction
// per load and no 64-bit per-lane address arithmetic in front of it.  STREAM: as a streaming (nt) load -- the weight
// codes are read once; measured on tile-major weights 8.85 -> 8.70 us (N = 14336, K = 4096), on row-major ones, whose
// 64-byte row pieces share cache lines between K steps, 9.6 -> 9.9 us.
template <int OFF, bool STREAM = false>
__device__ __forceinline__ void load16_uncounted(v4i& dst, const uint8_t* sbase, unsigned voff) {
  static_assert(OFF >= 0 && OFF < 4096, "immediate offset of a global load");
  const uint64_t v = reinterpret_cast<uint64_t>(sbase);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  const uint64_t u = ((uint64_t)hi << 32) | lo;
  if constexpr (STREAM) asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "=v"(dst) : "v"(voff), "s"(u), "n"(OFF) : "memory");
  else asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(u), "n"(OFF) : "memory");
}
__device__ __forceinline__ void tie(v4i& r) { asm volatile("" : "+v"(r)); }
template <int N>
__device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

template <int F, bool WT, int G>
__global__ void __launch_bounds__(256)
mixed_gemm_decode_kernel(DecodeSeg s4, DecodeSeg s6, DecodeSeg s8, int M, int N, int steps_per_wave, DecodeLds L,
                         uint16_t* __restrict__ d) {
  static_assert(G == 1 || G == 2, "token groups of 16 per workgroup");
  constexpr int S = 4;        // K steps per round
  constexpr int PB = 4 * F;   // weight scale pieces per step
  constexpr int PBLOG = F == 1 ? 2 : (F == 2 ? 3 : 4);
  static_assert(F == 1 || F == 2 || F == 4, "pieces per step as a power of two");
  extern __shared__ __align__(16) uint8_t lds[];
  pin_args(s4); pin_args(s6); pin_args(s8); pin_args(L);
  asm volatile("" : "+s"(M), "+s"(N), "+s"(steps_per_wave), "+s"(d));
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t*)lds;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, g = lane >> 4;
  // the segments' fields as scalars (selected by masks below, never by indexing)
  const uint8_t *b4 = s4.b, *b6 = s6.b, *b8 = s8.b;
  const int nblk4 = s4.nblk, nblk6 = s6.nblk, nblk8 = s8.nblk;
  const int total = s4.steps + s6.steps + s8.steps;
  const int t_begin = wave * steps_per_wave, t_end = min(total, t_begin + steps_per_wave);
  const int rounds = (t_end - t_begin + S - 1) / S;   // may be <= 0 for the last wave

  // ---- the workgroup's rows.  Feature group f, lane row i -> row n[f], its scale piece and its slot in the piece.
  int n[F], piece[F], slot[F];
  unsigned sfb_piece_off;   // this lane's piece (lane % PB) of the copies, as a byte offset from the segment's buffer
  int sfb_katoms_mul;       // ... plus this many times katoms * 512 (the piece's group of 128 rows)
  // Tile-major weights: which F blocks of which 256-feature tile.  The 16 / F workgroups of a tile each write 2 F of
  // every 16 consecutive output features, i.e. a part of every 32-byte sector of the tile's columns; workgroups go to
  // the 8 XCDs (one L2 each) round-robin by index, so the workgroups of a tile are given indices of one XCD, whose L2
  // then puts the sectors together instead of four L2s writing a part each (c2: 0.9 -> 0.23 MB written).
  int wg = blockIdx.x;
  if constexpr (WT) {
    constexpr int kPer = 16 / F;   // workgroups per tile
    if ((int)gridDim.x % (8 * kPer) == 0) {
      const int xcd = wg & 7, slot = wg >> 3;
      wg = ((slot / kPer) * 8 + xcd) * kPer + slot % kPer;
    }
  }
  if constexpr (WT) {
    // blocks j0 + f of tile `tile`; pieces ordered [group of 128][u][f]
    const int tile = (wg * F) >> 4, j0 = (wg * F) & 15;
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const int t = i & 7, u = i >> 3;
      n[f] = tile * 256 + j0 + f + 32 * t + 16 * u;
      piece[f] = (t >> 2) * 2 * F + u * F + f;
      slot[f] = t & 3;
    }
    const int pl = lane % PB, pf = pl % F, pu = (pl / F) & 1, pg = pl / (2 * F);
    sfb_piece_off = (unsigned)(j0 + pf + 16 * pu) * 16u;
    sfb_katoms_mul = tile * 2 + pg;
  } else {
    // pieces c0 ... c0 + PB - 1 of group blockIdx.x / (32 / PB)
    const int per_group = 32 / PB, group = blockIdx.x / per_group, c0 = (blockIdx.x % per_group) * PB;
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const int e = 16 * f + i;   // 0 ... 16 F - 1
      n[f] = group * 128 + c0 + e % PB + 32 * (e / PB);
      piece[f] = e % PB;
      slot[f] = e / PB;
    }
    sfb_piece_off = (unsigned)(c0 + lane % PB) * 16u;
    sfb_katoms_mul = group;
  }

  // ---- weight codes: per lane 16 bytes per step and feature group (row n[f], block g of the step)
  int nc[F];
#pragma unroll
  for (int f = 0; f < F; ++f) nc[f] = min(n[f], N - 1);   // clamped rows: every load is in bounds
  v4i wq[2][S][F];
  // Per-lane byte offsets of the loads.  Tile-major: 16 KB per (256-feature tile, step), the workgroup's F blocks of
  // 1 KB consecutive in it, lane quad i, piece g.  Row-major: row nc[f] of the segment, piece g of the step.
  unsigned vrow4[F], vrow6[F], vrow8[F];
  const unsigned vlane = (unsigned)(i * 64 + g * 16);
#pragma unroll
  for (int f = 0; f < F; ++f) {
    vrow4[f] = (unsigned)nc[f] * (unsigned)nblk4 * 16u + (unsigned)g * 16u;
    vrow6[f] = (unsigned)nc[f] * (unsigned)nblk6 * 16u + (unsigned)g * 16u;
    vrow8[f] = (unsigned)nc[f] * (unsigned)nblk8 * 16u + (unsigned)g * 16u;
  }
  const int wtile = (wg * F) >> 4, wj0 = (wg * F) & 15;
  auto request_round = [&](int r, auto buf_c) {
    constexpr int B = decltype(buf_c)::value;
#pragma unroll
    for (int k = 0; k < S; ++k) {
      const int t = min(t_begin + r * S + k, total - 1);
      const int seg = t < s4.steps ? 0 : (t < s4.steps + s6.steps ? 1 : 2);
      const int q = seg == 0 ? t : (seg == 1 ? t - s4.steps : t - s4.steps - s6.steps);
      const uint8_t* pb = sel3p(seg, b4, b6, b8);
      if constexpr (WT) {
        const int nst = sel3(seg, nblk4, nblk6, nblk8) >> 2;
        const uint8_t* sb = pb + (((size_t)wtile * nst + q) * 16 + wj0) * 1024;
        constexpr bool kStream = G == 1;   // several token groups' workgroups read the same weights: those stay ordinary loads
        if constexpr (F >= 1) load16_uncounted<0, kStream>(wq[B][k][0], sb, vlane);
        if constexpr (F >= 2) load16_uncounted<1024, kStream>(wq[B][k][F >= 2 ? 1 : 0], sb, vlane);
        if constexpr (F >= 4) {
          load16_uncounted<2048, kStream>(wq[B][k][F >= 4 ? 2 : 0], sb, vlane);
          load16_uncounted<3072, kStream>(wq[B][k][F >= 4 ? 3 : 0], sb, vlane);
        }
      } else {
        const uint8_t* sb = pb + (size_t)q * 64;
#pragma unroll
        for (int f = 0; f < F; ++f)
          load16_uncounted<0>(wq[B][k][f], sb, (unsigned)sel3(seg, (int)vrow4[f], (int)vrow6[f], (int)vrow8[f]));
      }
    }
  };
  // ---- what is not a weight code, into LDS: requested first (measured: with the first round of weights ahead of
  // them the kernel is slower, by 2 % on tile-major and 7 % on row-major weights)
  // the workgroup's tokens: m_base ... m_base + rows_here - 1 (G = 2: workgroup blockIdx.y takes 32 of them)
  const int m_base = G == 1 ? 0 : (int)blockIdx.y * 32;
  const int rows_here = min(M - m_base, 16 * G);
  copy_region(s4.a + (size_t)m_base * nblk4 * 16, rows_here * nblk4 * 16, lds0 + L.x0, wave, lane);
  copy_region(s6.a + (size_t)m_base * nblk6 * 24, rows_here * nblk6 * 24, lds0 + L.x1, wave, lane);
  copy_region(s8.a + (size_t)m_base * nblk8 * 32, rows_here * nblk8 * 32, lds0 + L.x2, wave, lane);
  {
    const int palog = L.pa == 8 ? 3 : (L.pa == 16 ? 4 : 5);
    // token scale pieces 0 ... pa - 1 of the tokens' group of 128 rows
    const unsigned pa_off = (unsigned)(lane & (L.pa - 1)) * 16u;
    const unsigned agrp = (unsigned)(m_base >> 7) * 512u;   // times the segment's atoms along K
    if (s4.steps) copy_pieces(s4.sfa, s4.steps, palog, pa_off + agrp * (unsigned)s4.steps, lds0 + L.sfa0, wave, lane);
    if (s6.steps) copy_pieces(s6.sfa, s6.steps, palog, pa_off + agrp * (unsigned)s6.steps, lds0 + L.sfa1, wave, lane);
    if (s8.steps) copy_pieces(s8.sfa, s8.steps, palog, pa_off + agrp * (unsigned)s8.steps, lds0 + L.sfa2, wave, lane);
    if (s4.steps) copy_pieces(s4.sfb, s4.steps, PBLOG, sfb_piece_off + (unsigned)(sfb_katoms_mul * s4.steps) * 512u, lds0 + L.sfb0, wave, lane);
    if (s6.steps) copy_pieces(s6.sfb, s6.steps, PBLOG, sfb_piece_off + (unsigned)(sfb_katoms_mul * s6.steps) * 512u, lds0 + L.sfb1, wave, lane);
    if (s8.steps) copy_pieces(s8.sfb, s8.steps, PBLOG, sfb_piece_off + (unsigned)(sfb_katoms_mul * s8.steps) * 512u, lds0 + L.sfb2, wave, lane);
  }

  if (rounds > 0) request_round(0, std::integral_constant<int, 0>{});
  if (rounds > 1) request_round(1, std::integral_constant<int, 1>{});

  // ---- the copies and the first round are older than the second round: done when only that is in flight
  if (rounds > 1) wait_vmcnt<S * F>();
  else wait_vmcnt<0>();
  asm volatile("s_barrier" ::: "memory");

  v4f acc[F][G];
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int gi = 0; gi < G; ++gi) acc[f][gi] = v4f{0.f, 0.f, 0.f, 0.f};
  // token of this lane in token group gi, as a row of the workgroup's LDS image (tokens past M: the last one again,
  // never stored), and where its scale bytes sit in a step's pieces
  int mc[G], sx_off[G];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    mc[gi] = min(16 * gi + i, rows_here - 1);
    const int mg = m_base + mc[gi];
    sx_off[gi] = (mg & (L.pa - 1)) * 16 + ((mg >> 5) & 3) * 4;
  }
  const int pa16 = L.pa * 16;

  auto compute_round = [&](int r, auto buf_c) {
    constexpr int B = decltype(buf_c)::value;
#pragma unroll
    for (int k = 0; k < S; ++k) {
      const int t = t_begin + r * S + k;
      if (t < t_end) {   // wave-uniform
        const int seg = t < s4.steps ? 0 : (t < s4.steps + s6.steps ? 1 : 2);
        const int q = seg == 0 ? t : (seg == 1 ? t - s4.steps : t - s4.steps - s6.steps);
        const uint8_t* sfa_l = lds + sel3(seg, L.sfa0, L.sfa1, L.sfa2) + q * pa16;
        const uint8_t* sfb_l = lds + sel3(seg, L.sfb0, L.sfb1, L.sfb2) + q * (PB * 16);
        int s_x[G];
#pragma unroll
        for (int gi = 0; gi < G; ++gi) s_x[gi] = sfa_l[sx_off[gi] + g];
        v8i wf[F];
        int s_w[F];
#pragma unroll
        for (int f = 0; f < F; ++f) {
          s_w[f] = sfb_l[piece[f] * 16 + slot[f] * 4 + g];
          const v4i w4 = wq[B][k][f];
          wf[f] = v8i{w4[0], w4[1], w4[2], w4[3], 0, 0, 0, 0};
        }
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
          if (seg == 0) {
            const v4i a4 = *reinterpret_cast<const v4i*>(lds + L.x0 + mc[gi] * (nblk4 * 16) + q * 64 + g * 16);
            const v8i xf = {a4[0], a4[1], a4[2], a4[3], 0, 0, 0, 0};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE2M1>(wf[f], xf, acc[f][gi], s_w[f], s_x[gi]);
          } else if (seg == 1) {
            const v2i* p = reinterpret_cast<const v2i*>(lds + L.x1 + mc[gi] * (nblk6 * 24) + q * 96 + g * 24);
            const v2i a = p[0], b = p[1], c = p[2];
            const v8i xf = {a[0], a[1], b[0], b[1], c[0], c[1], 0, 0};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE3M2>(wf[f], xf, acc[f][gi], s_w[f], s_x[gi]);
          } else {
            const uint8_t* p = lds + L.x2 + mc[gi] * (nblk8 * 32) + q * 128 + g * 16;
            const v4i a4 = *reinterpret_cast<const v4i*>(p), b4v = *reinterpret_cast<const v4i*>(p + 64);
            const v8i xf = {a4[0], a4[1], a4[2], a4[3], b4v[0], b4v[1], b4v[2], b4v[3]};
#pragma unroll
            for (int f = 0; f < F; ++f) acc[f][gi] = decode_mfma<kFmtE4M3>(wf[f], xf, acc[f][gi], s_w[f], s_x[gi]);
          }
        }
      }
    }
  };
  // the registers of a round are tied to the wait that precedes their use
  auto settle = [&](auto buf_c, auto n_c) {
    constexpr int B = decltype(buf_c)::value;
    constexpr int NW = decltype(n_c)::value;
    wait_vmcnt<NW>();
#pragma unroll
    for (int k = 0; k < S; ++k)
#pragma unroll
      for (int f = 0; f < F; ++f) tie(wq[B][k][f]);
  };
  // Two rounds at a time, both requested before the first is used.  The first pair (requested above) is straight-line
  // code, the loop requests its pairs itself: nothing is in flight across a loop edge (a register that an uncounted
  // load is still to fill must not be moved by the compiler, which a value carried around a loop may be).
  if (rounds > 0) {
#pragma unroll
    for (int k = 0; k < S; ++k)
#pragma unroll
      for (int f = 0; f < F; ++f) tie(wq[0][k][f]);
    compute_round(0, std::integral_constant<int, 0>{});
  }
  if (rounds > 1) {
    settle(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
    compute_round(1, std::integral_constant<int, 1>{});
  }
  for (int r = 2; r < rounds; r += 2) {
    request_round(r, std::integral_constant<int, 0>{});
    if (r + 1 < rounds) {
      request_round(r + 1, std::integral_constant<int, 1>{});
      settle(std::integral_constant<int, 0>{}, std::integral_constant<int, S * F>{});
    } else {
      settle(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    }
    compute_round(r, std::integral_constant<int, 0>{});
    if (r + 1 < rounds) {
      settle(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
      compute_round(r + 1, std::integral_constant<int, 1>{});
    }
  }

  // ---- sum the four waves' partial tiles (D^T: lane holds token lane % 16, feature slots 4 * (lane / 16) + v of a group)
  float* partial = reinterpret_cast<float*>(lds + L.partial);
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
      *reinterpret_cast<v4f*>(partial + ((wave * (F * G) + f * G + gi) * 64 + lane) * 4) = acc[f][gi];
  __syncthreads();
#pragma unroll
  for (int fg = 0; fg < F * G; ++fg) {
    if ((fg & 3) != wave) continue;
    const int f = fg / G, gi = fg % G;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) sum += *reinterpret_cast<const v4f*>(partial + ((w * (F * G) + fg) * 64 + lane) * 4);
    const int m = m_base + 16 * gi + i;
    if (m < M) {
      uint16_t h[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) h[v] = __builtin_bit_cast(uint16_t, (__bf16)sum[v]);
      if constexpr (WT) {
        // feature slot e = 4 g + v of the block is row j + 32 (e % 8) + 16 (e / 8) of the tile
        const int bx = wg * F + f, row0 = (bx >> 4) * 256 + (bx & 15);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int e = 4 * g + v, row = row0 + 32 * (e & 7) + 16 * (e >> 3);
          if (row < N) d[(size_t)m * N + row] = h[v];
        }
      } else {
        // feature slots 4 g ... 4 g + 3 of the group are four consecutive rows
        const int per_group = 32 / PB, group = blockIdx.x / per_group, c0 = (blockIdx.x % per_group) * PB;
        const int e = 16 * f + 4 * g;
        const int nn = group * 128 + c0 + e % PB + 32 * (e / PB);
        uint16_t* dst = d + (size_t)m * N + nn;
        if (nn + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<v2u*>(dst) = v2u{(unsigned)h[0] | ((unsigned)h[1] << 16), (unsigned)h[2] | ((unsigned)h[3] << 16)};
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (nn + v < N) dst[v] = h[v];
        }
      }
    }
  }
}

static int round_up_1k(int v) { return (v + 1023) & ~1023; }

// The decode kernel takes whole 128-wide steps in every segment and, with one token group per workgroup (G = 1), up to
// 16 tokens and an LDS image of at most 76 KB (two workgroups per CU); with two (G = 2: 32 tokens per workgroup, any
// number of tokens below 256) whatever fits the LDS of a CU.
constexpr int kDecodeLds1 = 76 * 1024, kDecodeLds2 = 156 * 1024;
static bool decode_lds_plan(const DecodeSeg& d4, const DecodeSeg& d6, const DecodeSeg& d8, int M, int F, int G, DecodeLds* L) {
  int pos = 0;
  auto take = [&](int bytes) { const int at = pos; pos += round_up_1k(bytes); return at; };
  const int rows = G == 1 ? M : (M < 32 ? M : 32);   // token rows of a workgroup's image
  L->pa = G == 2 ? 32 : (M <= 8 ? 8 : 16);
  L->x0 = take(rows * d4.nblk * 16); L->x1 = take(rows * d6.nblk * 24); L->x2 = take(rows * d8.nblk * 32);
  L->sfa0 = take(d4.steps * L->pa * 16); L->sfa1 = take(d6.steps * L->pa * 16); L->sfa2 = take(d8.steps * L->pa * 16);
  L->sfb0 = take(d4.steps * F * 64); L->sfb1 = take(d6.steps * F * 64); L->sfb2 = take(d8.steps * F * 64);
  L->partial = pos;
  pos += 4 * F * G * 1024;
  L->total = pos;
  return pos <= (G == 1 ? kDecodeLds1 : kDecodeLds2);
}

// Feature groups of 16 per workgroup of the decode kernel (and what the cost model below assumes of the skinny one).
static int skinny_feature_groups(int rows, int N, int cus) {
  const int g = rows <= 16 ? 1 : (rows <= 32 ? 2 : (rows <= 64 ? 4 : 8));
  return ceil_div(N, 32) * ceil_div(rows, 16 * g) >= cus ? 2 : 1;
}

// Token groups (g) and feature groups (f) of 16 per workgroup of the skinny kernel.  A wave's loads per K step are
// f weight fragments, 2 g token fragments and f + g scale bytes, and the token fragments (16 rows x 16 bytes each)
// are what the address unit is slowest at: two feature groups per workgroup halve them per output, and more than
// four token groups per workgroup never paid (M = 128, N = 4096, K = 4096: g = 8, f = 1 22.3 us; g = 4, f = 2 16.9 us;
// M = 64: g = 4, f = 1 12.0 us; g = 2, f = 2 10.5 us; M = 200: g = 8, f = 2 26.4 us; g = 4, f = 2 23.0 us).  The largest of
// these that still gives every CU a workgroup.
static void skinny_groups(int rows, int N, int cus, int* g_out, int* f_out) {
  const int gmax = rows <= 16 ? 1 : (rows <= 32 ? 2 : 4);
  for (int f = 2; f >= 1; --f)
    for (int g = gmax; g >= 1; g >>= 1)
      if (ceil_div(N, 16 * f) * ceil_div(rows, 16 * g) >= cus) {
        *g_out = g;
        *f_out = f;
        return;
      }
  *g_out = 1;
  *f_out = 1;
}
// Feature groups of 16 per workgroup (4, 2 or 1) for the decode kernel with two token groups per workgroup: the most
// that still leave most CUs a workgroup and whose LDS image fits; 0 if none does (then *L is not valid).
static int decode2_feature_groups(const DecodeSeg& d4, const DecodeSeg& d6, const DecodeSeg& d8, int M, int N, int cus,
                                  DecodeLds* L) {
  const int tg = ceil_div(M, 32);
  int f = ceil_div(N, 64) * tg >= cus * 3 / 4 ? 4 : (ceil_div(N, 32) * tg >= cus * 3 / 4 ? 2 : 1);
  while (f > 1 && !decode_lds_plan(d4, d6, d8, M, f, 2, L)) f >>= 1;
  return decode_lds_plan(d4, d6, d8, M, f, 2, L) ? f : 0;
}

hipError_t launch_skinny(const DecodeSeg& d4, const DecodeSeg& d6, const DecodeSeg& d8, int M, int N,
                         bool w_tiled, uint16_t* d, hipStream_t stream) {
  const int rows = M;
  DeviceLimits lim;
  if (hipError_t e = device_limits(&lim); e != hipSuccess) return e;
  // decode: the kernel that stages everything but the weight codes in LDS
  // (a segment's weight codes below 4 GB: the kernel addresses them with 32-bit per-lane offsets)
  const size_t widest = (size_t)(d4.nblk > d6.nblk ? (d4.nblk > d8.nblk ? d4.nblk : d8.nblk) : (d6.nblk > d8.nblk ? d6.nblk : d8.nblk));
  typedef void (*kernel_t)(DecodeSeg, DecodeSeg, DecodeSeg, int, int, int, DecodeLds, uint16_t*);
  const bool whole_steps = ((d4.nblk | d6.nblk | d8.nblk) & 3) == 0 && (size_t)N * widest * 16 < ((size_t)1 << 32);
  const int spw = (d4.steps + d6.steps + d8.steps + 3) / 4;
  if (M <= 16 && whole_steps) {
    // feature groups of 16 per workgroup: 4 (tile-major weights; measured on N = 14336: 9.0 against 9.6 us) or 2 as
    // long as that leaves most CUs a workgroup
    int f = skinny_feature_groups(rows, N, lim.cus);
    if (w_tiled && ceil_div(N, 64) >= lim.cus * 3 / 4) f = 4;
    DecodeLds L;
    if (f == 4 && !decode_lds_plan(d4, d6, d8, M, f, 1, &L)) f = 2;
    if (decode_lds_plan(d4, d6, d8, M, f, 1, &L)) {
      // row-major: per group of 128 rows 8 / F workgroups (the last group whole, rows past N clamped and not stored)
      const dim3 grid(w_tiled ? ceil_div(N, 16 * f) : ceil_div(N, 128) * (8 / f));
      const kernel_t kernels[2][3] = {
          {mixed_gemm_decode_kernel<1, false, 1>, mixed_gemm_decode_kernel<2, false, 1>, mixed_gemm_decode_kernel<4, false, 1>},
          {mixed_gemm_decode_kernel<1, true, 1>, mixed_gemm_decode_kernel<2, true, 1>, mixed_gemm_decode_kernel<4, true, 1>}};
      const kernel_t kernel = kernels[w_tiled ? 1 : 0][f == 4 ? 2 : f - 1];
      if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kDecodeLds1); e != hipSuccess) return e;
      hipLaunchKernelGGL(kernel, grid, dim3(256), (size_t)L.total, stream, d4, d6, d8, M, N, spw, L, d);
      return hipGetLastError();
    }
  }
  // More tokens, in groups of 32 per workgroup, while their codes fit the LDS (K = 4096: 79 KB; not K = 14336): the
  // token fragments and scales then come from LDS once per workgroup instead of from memory in every K step, which
  // is what the kernel below spends most of its time on (M = 128, N = 4096, K = 4096: 17 -> 9 us).  The most feature
  // groups per workgroup (4, 2, 1) that still leave most CUs a workgroup.
  if (M > 16 && whole_steps) {
    const int tg = ceil_div(M, 32);
    DecodeLds L;
    const int f = decode2_feature_groups(d4, d6, d8, M, N, lim.cus, &L);
    if (f > 0) {
      const dim3 grid(w_tiled ? ceil_div(N, 16 * f) : ceil_div(N, 128) * (8 / f), tg);
      const kernel_t kernels[2][3] = {
          {mixed_gemm_decode_kernel<1, false, 2>, mixed_gemm_decode_kernel<2, false, 2>, mixed_gemm_decode_kernel<4, false, 2>},
          {mixed_gemm_decode_kernel<1, true, 2>, mixed_gemm_decode_kernel<2, true, 2>, mixed_gemm_decode_kernel<4, true, 2>}};
      const kernel_t kernel = kernels[w_tiled ? 1 : 0][f == 4 ? 2 : f - 1];
      if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kDecodeLds2); e != hipSuccess) return e;
      hipLaunchKernelGGL(kernel, grid, dim3(256), (size_t)L.total, stream, d4, d6, d8, M, N, spw, L, d);
      return hipGetLastError();
    }
  }
  const int steps_per_wave = (d4.steps + d6.steps + d8.steps + 3) / 4;
  int g, f;
  skinny_groups(rows, N, lim.cus, &g, &f);
  const dim3 grid(ceil_div(N, 16 * f), ceil_div(rows, 16 * g));
  const int wt = w_tiled ? 1 : 0;
  switch (g) {
    case 1:
      if (f == 2) hipLaunchKernelGGL((mixed_gemm_skinny_kernel<1, 2>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      else hipLaunchKernelGGL((mixed_gemm_skinny_kernel<1, 1>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      break;
    case 2:
      if (f == 2) hipLaunchKernelGGL((mixed_gemm_skinny_kernel<2, 2>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      else hipLaunchKernelGGL((mixed_gemm_skinny_kernel<2, 1>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      break;
    default:   // 4 token groups: skinny_groups takes no more
      if (f == 2) hipLaunchKernelGGL((mixed_gemm_skinny_kernel<4, 2>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      else hipLaunchKernelGGL((mixed_gemm_skinny_kernel<4, 1>), grid, dim3(256), 0, stream, d4, d6, d8, M, N, steps_per_wave, wt, d);
      break;
  }
  return hipGetLastError();
}

}  // namespace

// 256 x 256 tiles, one workgroup per CU (mixed_gemm_256.hip)
bool mixed_gemm_256_supported(int M, int N, int KN, int KS, int KO);
hipError_t launch_mixed_gemm_256(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                                 const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                                 const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo,
                                 int m_store, int a_rows, int N, int KN, int KS, int KO, bool w_tiled, void* d,
                                 hipStream_t stream);

// Rough launch times in microseconds, only to choose between the kernels for fewer than 256 tokens (measured on
// MI355X, 256 CUs, K = 4096: the whole-tile kernel runs such problems as 256 x 128 tiles when that is at most one
// round -- a 128-wide stage then takes ~0.42 us with at most half of the CUs busy, ~0.45 us with more, plus ~2.5 us --
// and as 256 x 256 tiles at ~0.95 us a stage plus ~3 us a round otherwise; the decode kernel with two token groups
// per workgroup takes ~5.5 us plus 22 ns per K step and feature group for each round of one workgroup per CU; the
// skinny kernel 0.25-0.33 ns per 16 tokens x 16 features x 128 K plus ~5 us: K = 14336, N = 4096, 64 / 128 tokens 28 / 62 us).
static double pipelined_us(int M, int N, int stages, int cus) {
  const int whole = ceil_div(M, 256) * ceil_div(N, 256);
  if (whole <= cus / 2) return stages * (ceil_div(M, 128) * ceil_div(N, 256) <= cus / 2 ? 0.42 : 0.45) + 2.5;
  return (double)ceil_div(whole, cus) * (stages * 0.95 + 3.0);
}
static double skinny_us(const DecodeSeg& d4, const DecodeSeg& d6, const DecodeSeg& d8, int rows, int N, int steps, int cus,
                        bool w_tiled) {
  if (rows > 16 && ((d4.nblk | d6.nblk | d8.nblk) & 3) == 0) {
    DecodeLds L;
    const int f2 = decode2_feature_groups(d4, d6, d8, rows, N, cus, &L);
    if (f2 > 0) {
      const int wgs = (w_tiled ? ceil_div(N, 16 * f2) : ceil_div(N, 128) * (8 / f2)) * ceil_div(rows, 32);
      return 1.0 + ceil_div(wgs, cus) * (5.5 + steps * f2 * 0.022);
    }
  }
  int g, f;
  skinny_groups(rows, N, cus, &g, &f);
  return 5.0 + (double)ceil_div(rows, 16) * ceil_div(N, 16) * steps * (f == 2 ? 0.25e-3 : 0.33e-3);
}

// a_rows: token rows for which the activation codes and scales are readable (>= M)
hipError_t launch_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                             const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                             const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo, int M,
                             int a_rows, int N, int KN, int KS, int KO, unsigned flags, void* d, hipStream_t stream) {
  if (M == 0 || N == 0) return hipSuccess;
  const bool w_tiled = (flags & 1u) != 0;   // MG_FLAG_W_TILED
  // tile-major weights exist only for shapes the 256x256 kernel takes
  if (w_tiled && (N % 256 != 0 || !mixed_gemm_256_supported(256, N, KN, KS, KO))) return hipErrorInvalidValue;
  const int m_pad = (M + 255) / 256 * 256;
  const int steps = (KN + 127) / 128 + (KS + 127) / 128 + (KO + 127) / 128;
  int cus = 256;
  if (M < 256) {
    DeviceLimits lim;
    if (hipError_t e = device_limits(&lim); e != hipSuccess) return e;
    cus = lim.cus;
  }
  // whole 256-row tiles; the last one does not write rows past M and reads no activation row past
  // a_rows (lanes that would are pointed at the last readable row)
  const DecodeSeg d4 = {an, bn, sfan, sfbn, KN / 32, (KN + 127) / 128};
  const DecodeSeg d6 = {as_, bs, sfas, sfbs, KS / 32, (KS + 127) / 128};
  const DecodeSeg d8 = {ao, bo, sfao, sfbo, KO / 32, (KO + 127) / 128};
  if (mixed_gemm_256_supported(m_pad, N, KN, KS, KO) &&
      (M >= 256 || pipelined_us(M, N, steps, cus) < skinny_us(d4, d6, d8, M, N, steps, cus, w_tiled)))
    return launch_mixed_gemm_256(an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs, sfao, sfbo, M, a_rows, N, KN, KS, KO,
                                 w_tiled, d, stream);
  if (M < 256 && KN + KS + KO > 0) return launch_skinny(d4, d6, d8, M, N, w_tiled, static_cast<uint16_t*>(d), stream);
  // what is left (256 tokens or more with N not a multiple of 8, or with a segment that is not whole 128-wide
  // stages next to an empty one): the direct kernel
  dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
  hipLaunchKernelGGL(mixed_gemm_direct_kernel, grid, dim3(256), 0, stream, an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs,
                     sfao, sfbo, M, N, KN, KS, KO, static_cast<uint16_t*>(d));
  return hipGetLastError();
}

}  // namespace mg
