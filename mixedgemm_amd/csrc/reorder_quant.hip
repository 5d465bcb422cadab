// Reorder-quantize kernels for gfx950: gather bf16 channels by a reorder index,
// then per-32-element power-of-two (E8M0) scaling and quantization into packed
// MXFP4 (E2M1) / MXFP6 (E3M2) / MXFP8 (E4M3) segments.
//
// Semantics follow the reference kernels reorder_bf16_mixed_kernel
// (src/reorder.cu:94-269) and reorder_bf16_fp4_kernel (src/reorder.cu:271-432):
//   scale  = 2^e, e = min{e : amax <= MAX * 2^e}  (= ceil(log2(amax/MAX)), :180),
//            0.5 for an all-zero block (:179); E8M0 byte = e + 127
//   code   = RNE_fmt( bf16( clamp( roundf(x / scale) ) ) )   (:221-248)
// The design is not the reference's: a workgroup stages R rows at a time into
// LDS in channel-major order with the R rows of one channel adjacent, so one
// 2R-byte LDS read fetches a gathered channel for all R rows; one lane owns one
// 32-element block (no cross-lane reduction), the scale exponent comes from
// integer arithmetic on the float bits, and the element conversion is done by
// the gfx950 cvt_scalef32 instructions on the already integer-rounded values.
#include <type_traits>

#include "mg_common.h"

namespace mg {

namespace {

__device__ __forceinline__ unsigned perm(unsigned hi, unsigned lo, unsigned sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// E8M0 byte of the block scale from the bits of amax (a non-negative float).
// MAX = fm * 2^pm with fm in [0.5,1): the exponent steps up by one when the
// mantissa of amax exceeds the mantissa of MAX, which the add below carries
// into the exponent field.  `fmt` may differ between the lanes of a wave.
__device__ __forceinline__ int scale_byte(float amax, int fmt) {
  const unsigned thr = fmt == kFmtE2M1 ? 0x400000u : 0x600000u;  // 6 = 1.5*4, 28 = 1.75*16, 448 = 1.75*256
  const int pm = fmt == kFmtE2M1 ? 3 : (fmt == kFmtE3M2 ? 5 : 9);
  const unsigned bits = __float_as_uint(amax);
  int byte = (int)((bits + (0x7FFFFFu - thr)) >> 23) + 1 - pm;
  byte = byte < 0 ? 0 : byte;
  return amax == 0.0f ? 126 : byte;
}

// roundf(x * rs): half away from zero, sign of zero kept.
__device__ __forceinline__ float round_scaled(float x, float rs) {
  float half = __uint_as_float((__float_as_uint(x) & 0x80000000u) | 0x3f000000u);
  return __builtin_truncf(__builtin_fmaf(x, rs, half));
}

// Quantize one gathered block (32 floats holding bf16 values) and store its codes and scale.
// Everything up to the integer-valued v[] is the same instruction stream for the three
// formats (a wave that straddles a segment boundary runs it once, not once per format); only
// the final conversion and store differ.
__device__ __forceinline__ void quantize_store(const float (&f)[32], int fmt, uint8_t* __restrict__ q,
                                               uint8_t* __restrict__ sf) {
  float amax = 0.0f;
#pragma unroll
  for (int p = 0; p < 32; p += 2) amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fabsf(f[p])), __builtin_fabsf(f[p + 1]));
  const int byte = scale_byte(amax, fmt);
  const float rs = __uint_as_float((unsigned)(254 - byte) << 23);
  float v[32];
#pragma unroll
  for (int p = 0; p < 32; ++p) v[p] = round_scaled(f[p], rs);
  *sf = (uint8_t)byte;

  if (fmt == kFmtE2M1) {
    v4u out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      unsigned w = 0;
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 0], v[8 * j + 1], 1.0f, 0);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 2], v[8 * j + 3], 1.0f, 1);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 4], v[8 * j + 5], 1.0f, 2);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 6], v[8 * j + 7], 1.0f, 3);
      out[j] = w;
    }
    *reinterpret_cast<v4u*>(q) = out;
  } else {
    // the bf16 hop of the reference (src/reorder.cu:223) is a real rounding above 256
    v32bf h;
#pragma unroll
    for (int p = 0; p < 32; ++p) h[p] = (__bf16)v[p];
    if (fmt == kFmtE3M2) {
      // the ISA calls E3M2 "bf6" (its "fp6" is E2M3)
      const v6u w = __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(h, 1.0f);
      v2u* p = reinterpret_cast<v2u*>(q);
      p[0] = v2u{w[0], w[1]};
      p[1] = v2u{w[2], w[3]};
      p[2] = v2u{w[4], w[5]};
    } else {
      unsigned out[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const v2bf lo = {h[4 * j + 0], h[4 * j + 1]};
        const v2bf hi = {h[4 * j + 2], h[4 * j + 3]};
        v2s z = {0, 0};
        z = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, lo, 1.0f, false);
        z = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, hi, 1.0f, true);
        out[j] = __builtin_bit_cast(unsigned, z);
      }
      v4u* p = reinterpret_cast<v4u*>(q);
      p[0] = v4u{out[0], out[1], out[2], out[3]};
      p[1] = v4u{out[4], out[5], out[6], out[7]};
    }
  }
}

// A workgroup handles groups of R consecutive rows, group blockIdx.x first and then every
// gridDim.x-th one; blockDim.x >= K/32 (at most MAXT).  The global loads of the next group are
// issued before the current group is gathered and quantized, and the LDS tile is double buffered
// (buf_stride bytes apart; 0 when every workgroup has a single group), so loads, arithmetic and
// stores of different groups overlap inside the workgroup and one barrier per group suffices.
//
// NORM: an RMSNorm (weight gamma, bf16 in and out, the arithmetic of the usual fp32 implementation)
// is applied to each row before the gather:
//   var = fl32( (sum over the row of x^2, accumulated in fp64) / K )
//   r   = fl32( 1 / sqrt( fl32(var + eps) ) )      (division and square root in fp64)
//   y   = bf16( gamma * bf16( x * r ) )            (both products in fp32)
// The fp64 sum makes the result independent of the order in which the lanes add their parts
// (up to the last bit of a double, which the rounding to fp32 all but never sees).
template <int R, bool IS_W, int MAXT, bool NORM>
__global__ void __launch_bounds__(MAXT)
reorder_quant_kernel(const uint16_t* __restrict__ x, const int16_t* __restrict__ idx, int rows, int K, int KN, int KS,
                     int KO, uint8_t* __restrict__ qn, uint8_t* __restrict__ qs, uint8_t* __restrict__ qo,
                     uint8_t* __restrict__ sfn, uint8_t* __restrict__ sfs, uint8_t* __restrict__ sfo, int buf_stride,
                     const uint16_t* __restrict__ gamma, float eps) {
  extern __shared__ __align__(16) uint8_t lds_all[];
  __shared__ double row_sums[R][MAXT / 64];
  const int tid = threadIdx.x;
  const int nthr = blockDim.x;
  const int ngroups = (rows + R - 1) / R;

  // ---- the lane's 32 reorder indices (the same for every row): requested first, needed only
  //      after the first barrier
  const int b = tid;
  const bool has_block = b < (K >> 5);
  v4u iv[4];
  {
    const v4u* ip = reinterpret_cast<const v4u*>(idx + (size_t)(has_block ? b : 0) * 32);
#pragma unroll
    for (int q = 0; q < 4; ++q) iv[q] = ip[q];
  }

  // per-lane block constants
  const int nbn = KN >> 5, nbs = KS >> 5;
  const int seg = b < nbn ? 0 : (b < nbn + nbs ? 1 : 2);
  const int j = seg == 0 ? b : (seg == 1 ? b - nbn : b - nbn - nbs);
  const int kseg = seg == 0 ? KN : (seg == 1 ? KS : KO);
  const int katoms = (kseg + 127) >> 7;
  const int fmt = IS_W ? kFmtE2M1 : (seg == 0 ? kFmtE2M1 : (seg == 1 ? kFmtE3M2 : kFmtE4M3));
  const int blk_bytes = fmt == kFmtE2M1 ? 16 : (fmt == kFmtE3M2 ? 24 : 32);
  const size_t pitch = (size_t)(kseg >> 5) * blk_bytes;
  uint8_t* qbase = (seg == 0 ? qn : (seg == 1 ? qs : qo)) + j * blk_bytes;
  uint8_t* sfbase = seg == 0 ? sfn : (seg == 1 ? sfs : sfo);

  // ---- stage R rows: all 16-byte loads issued up front (row and chunk clamped instead of
  //      branched, so nothing waits), R x 8 transpose in registers, 16-byte LDS stores.
  //      Channel c of row r lands at lds[(c*R + r)*2].
  const int nchunks = K >> 3;
  v4u a[4][R];
  auto issue_loads = [&](int group) {
    const int row0 = group * R;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int c = min(tid + it * nthr, nchunks - 1);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int row = min(row0 + r, rows - 1);
        a[it][r] = *reinterpret_cast<const v4u*>(x + (size_t)row * K + (size_t)c * 8);
      }
    }
  };

  int group = blockIdx.x;
  if (group >= ngroups) return;
  issue_loads(group);
  v4u gv[4];   // the RMSNorm weights of this lane's chunks (the same for every row)
  if constexpr (NORM) {
#pragma unroll
    for (int it = 0; it < 4; ++it)
      gv[it] = *reinterpret_cast<const v4u*>(gamma + (size_t)min(tid + it * nthr, nchunks - 1) * 8);
  }
  // Byte offsets of the lane's 32 gathered channels inside a tile (the same for every row).  An entry outside
  // [0, K) is read as channel K - 1, so that the gather stays inside the tile whatever the index holds.
  unsigned ga[32];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      ga[q * 8 + e] = min((e & 1) ? (iv[q][e >> 1] >> 16) : (iv[q][e >> 1] & 0xffffu), (unsigned)(K - 1)) * (2 * R);

  // The loop body exists once per LDS buffer, so that the buffer's offset is a compile-time
  // constant wherever the buffers are a fixed distance apart (kFixed) and folds into the LDS
  // instructions' immediate offsets: the gather is then one instruction per channel.
  constexpr bool kFixed = MAXT == 256;
  constexpr int kBuf1 = MAXT * 64 * R;   // largest tile of this instantiation
  auto body = [&](auto parity_c) {
    constexpr int parity = decltype(parity_c)::value;
    uint8_t* lds = lds_all + (kFixed ? parity * kBuf1 : parity * buf_stride);
    const int row0 = group * R;
    if constexpr (NORM) {
      double ss[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        ss[r] = 0.0;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          if (tid + it * nthr < nchunks) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const unsigned d = a[it][r][e];
              const double lo = (double)__uint_as_float(d << 16), hi = (double)__uint_as_float(d & 0xffff0000u);
              ss[r] = __builtin_fma(lo, lo, ss[r]);
              ss[r] = __builtin_fma(hi, hi, ss[r]);
            }
          }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ss[r] += __shfl_xor(ss[r], off, 64);
        if ((tid & 63) == 0) row_sums[r][tid >> 6] = ss[r];
      }
      __syncthreads();
#pragma unroll
      for (int r = 0; r < R; ++r) {
        double tot = 0.0;
        for (int w = 0; w < (nthr >> 6); ++w) tot += row_sums[r][w];
        const float var = (float)(tot / (double)K);
        const float rn = (float)(1.0 / __builtin_sqrt((double)(var + eps)));
#pragma unroll
        for (int it = 0; it < 4; ++it) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned d = a[it][r][e], g = gv[it][e];
            const float h0 = (float)(__bf16)(__uint_as_float(d << 16) * rn);
            const float h1 = (float)(__bf16)(__uint_as_float(d & 0xffff0000u) * rn);
            const v2bf y = {(__bf16)(__uint_as_float(g << 16) * h0), (__bf16)(__uint_as_float(g & 0xffff0000u) * h1)};
            a[it][r][e] = __builtin_bit_cast(unsigned, y);
          }
        }
      }
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int c = tid + it * nthr;
      if (c < nchunks) {
        v4u* dst = reinterpret_cast<v4u*>(lds + (size_t)c * 16 * R);
        if constexpr (R == 1) {
          dst[0] = a[it][0];
        } else if constexpr (R == 2) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            v4u o;
            o[0] = perm(a[it][1][2 * h], a[it][0][2 * h], 0x05040100u);
            o[1] = perm(a[it][1][2 * h], a[it][0][2 * h], 0x07060302u);
            o[2] = perm(a[it][1][2 * h + 1], a[it][0][2 * h + 1], 0x05040100u);
            o[3] = perm(a[it][1][2 * h + 1], a[it][0][2 * h + 1], 0x07060302u);
            dst[h] = o;
          }
        } else {
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            v4u o;
            o[0] = perm(a[it][1][jj], a[it][0][jj], 0x05040100u);
            o[1] = perm(a[it][3][jj], a[it][2][jj], 0x05040100u);
            o[2] = perm(a[it][1][jj], a[it][0][jj], 0x07060302u);
            o[3] = perm(a[it][3][jj], a[it][2][jj], 0x07060302u);
            dst[jj] = o;
          }
        }
      }
    }
    __syncthreads();
    // the registers are free again: request the next group's rows while this one is processed
    if (group + (int)gridDim.x < ngroups) issue_loads(group + gridDim.x);

    // ---- one lane per 32-element block
    if (has_block) {
      unsigned g[32][(R + 1) / 2];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int p = q * 8 + e;
          if constexpr (R == 4) {
            const v2u d = *reinterpret_cast<const v2u*>(lds + ga[p]);
            g[p][0] = d[0];
            g[p][1] = d[1];
          } else if constexpr (R == 2) {
            g[p][0] = *reinterpret_cast<const unsigned*>(lds + ga[p]);
          } else {
            g[p][0] = *reinterpret_cast<const uint16_t*>(lds + ga[p]);
          }
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int row = row0 + r;
        if (row >= rows) break;
        float f[32];
#pragma unroll
        for (int p = 0; p < 32; ++p) {
          const unsigned d = g[p][r >> 1];
          f[p] = __uint_as_float((r & 1) ? (d & 0xffff0000u) : (d << 16));
        }
        // per-lane format, code row pitch and byte offset of the block inside its row
        quantize_store(f, fmt, qbase + (size_t)row * pitch, sfbase + sf_offset(row, j, katoms));
      }
    }
    // with one buffer (buf_stride == 0) there is exactly one group per workgroup; with two, the
    // barrier of the next iteration separates this gather from the stores two iterations on
  };
  while (true) {
    body(std::integral_constant<int, 0>{});
    group += gridDim.x;
    if (group >= ngroups) break;
    body(std::integral_constant<int, 1>{});
    group += gridDim.x;
    if (group >= ngroups) break;
  }
}

}  // namespace

// gamma != nullptr: RMSNorm with that weight and eps before the gather (activations only)
template <bool IS_W>
hipError_t launch_reorder_quant(const void* x, const int16_t* idx, int rows, int K, int KN, int KS, int KO, uint8_t* qn,
                                uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo,
                                const void* gamma, float eps, hipStream_t stream) {
  if (rows == 0 || K == 0) return hipSuccess;
  if (gamma != nullptr && IS_W) return hipErrorInvalidValue;
  const uint16_t* gm = static_cast<const uint16_t*>(gamma);
  const int threads = ((K >> 5) + 63) & ~63;
  const uint16_t* xb = static_cast<const uint16_t*>(x);
  DeviceLimits lim;
  if (hipError_t e = device_limits(&lim); e != hipSuccess) return e;
  hipError_t err = hipSuccess;
  // R rows interleaved in LDS.  More row groups than `resident` workgroups: each workgroup
  // streams several groups through a double-buffered tile.
  auto launch = [&](auto kernel, int R) {
    const int tile = K * 2 * R;
    const int ngroups = ceil_div(rows, R);
    // second LDS buffer: a fixed 16 KB * R behind the first for the 256-lane kernels (see kFixed), else one tile behind
    const int second = K <= 8192 ? 256 * 64 * R : tile;
    const int usable = lim.lds_bytes - 1024;   // the kernels' static LDS (row sums of the RMSNorm) stays below 1 KB
    int per_cu = usable / (second + tile);
    per_cu = per_cu < 1 ? 1 : (per_cu > 4 ? 4 : per_cu);
    const int resident = lim.cus * per_cu;
    const bool stream_groups = ngroups > resident && second + tile <= usable;
    const int grid = stream_groups ? resident : ngroups;
    const int lds = stream_groups ? second + tile : tile;
    if (lds > usable) { err = hipErrorInvalidValue; return; }
    err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), usable);
    if (err != hipSuccess) return;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), (size_t)lds, stream, xb, idx, rows, K,
                       KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, stream_groups ? tile : 0, gm, eps);
    err = hipGetLastError();
  };
  constexpr int R = 1;
  if constexpr (!IS_W) {
    if (gamma != nullptr) {
      if (K <= 8192) launch(reorder_quant_kernel<R, false, 256, true>, R);
      else if (K <= 16384) launch(reorder_quant_kernel<2, false, 512, true>, 2);
      else launch(reorder_quant_kernel<1, false, 1024, true>, 1);
      return err;
    }
  }
  if (K <= 8192) {
    launch(reorder_quant_kernel<R, IS_W, 256, false>, R);
  } else if (K <= 16384) {
    launch(reorder_quant_kernel<2, IS_W, 512, false>, 2);
  } else {
    launch(reorder_quant_kernel<1, IS_W, 1024, false>, 1);
  }
  return err;
}

template hipError_t launch_reorder_quant<false>(const void*, const int16_t*, int, int, int, int, int, uint8_t*, uint8_t*,
                                                uint8_t*, uint8_t*, uint8_t*, uint8_t*, const void*, float, hipStream_t);
template hipError_t launch_reorder_quant<true>(const void*, const int16_t*, int, int, int, int, int, uint8_t*, uint8_t*,
                                               uint8_t*, uint8_t*, uint8_t*, uint8_t*, const void*, float, hipStream_t);

}  // namespace mg
