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

// roundf(x * rs) for a bf16 value x and a power of two rs, as one multiplication and one round-to-nearest-even:
// rs1 = rs * (1 + 2^-12).  x * rs has at most 8 significant bits, so x * rs1 is exact in fp32 (21 bits), a
// tie n + 0.5 moves off the tie away from zero, and every other value stays on its side of the nearest tie
// (it is at least one 8-bit step from it, the nudge is 2^-12 of the value).  The sign of zero is kept.
__device__ __forceinline__ float round_scaled(float x, float rs1) { return __builtin_rintf(x * rs1); }

// Stores of the codes and the scale byte.  COUNTED: as inline assembly, one instruction each, so that a kernel
// which waits with s_waitcnt vmcnt(n) on older requests knows exactly how many stores it has issued since;
// the codes go out as streaming (nt) stores, which leave the L2 while the kernel runs instead of in the
// write-back at its end, the scale bytes as ordinary stores (the 32 rows that share a 128-byte line of a scale
// atom are written by different workgroups; the L2 merges them).  KEEP: ordinary stores for the codes too -- for
// the fused call, whose GEMM reads them next: the quantizer is then about a microsecond slower and the GEMM five
// to six faster (measured on M = 4096, K = 4096, N = 14336).
template <bool COUNTED, bool KEEP = false>
__device__ __forceinline__ void store16(uint8_t* q, v4u v) {
  if constexpr (COUNTED && KEEP) asm volatile("global_store_dwordx4 %0, %1, off" : : "v"(q), "v"(v) : "memory");
  else if constexpr (COUNTED) asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(q), "v"(v) : "memory");
  else *reinterpret_cast<v4u*>(q) = v;
}
template <bool COUNTED, bool KEEP = false>
__device__ __forceinline__ void store8(uint8_t* q, v2u v) {
  if constexpr (COUNTED && KEEP) asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(q), "v"(v) : "memory");
  else if constexpr (COUNTED) asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(q), "v"(v) : "memory");
  else *reinterpret_cast<v2u*>(q) = v;
}
template <bool COUNTED>
__device__ __forceinline__ void store1(uint8_t* q, int byte) {
  if constexpr (COUNTED) asm volatile("global_store_byte %0, %1, off" : : "v"(q), "v"(byte) : "memory");
  else *q = (uint8_t)byte;
}
// store instructions a wave issues per row for a block format (plus one for the scale byte)
__device__ __forceinline__ constexpr int code_stores(int fmt) { return fmt == kFmtE2M1 ? 1 : (fmt == kFmtE3M2 ? 3 : 2); }

// Quantize one gathered block (32 floats holding bf16 values) and store its codes and scale.
// Everything up to the integer-valued v[] is the same instruction stream for the three
// formats (a wave that straddles a segment boundary runs it once, not once per format); only
// the final conversion and store differ.
template <bool COUNTED = false, bool KEEP = false>
__device__ __forceinline__ void quantize_store(const float (&f)[32], int fmt, uint8_t* __restrict__ q,
                                               uint8_t* __restrict__ sf) {
  float amax = 0.0f;
#pragma unroll
  for (int p = 0; p < 32; p += 2) amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fabsf(f[p])), __builtin_fabsf(f[p + 1]));
  const int byte = scale_byte(amax, fmt);
  const float rs1 = __uint_as_float(((unsigned)(254 - byte) << 23) | 0x800u);   // 2^(127 - byte) * (1 + 2^-12)
  float v[32];
#pragma unroll
  for (int p = 0; p < 32; ++p) v[p] = round_scaled(f[p], rs1);
  store1<COUNTED>(sf, byte);

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
    store16<COUNTED, KEEP>(q, out);
  } else {
    // the bf16 hop of the reference (src/reorder.cu:223) is a real rounding above 256
    v32bf h;
#pragma unroll
    for (int p = 0; p < 32; ++p) h[p] = (__bf16)v[p];
    if (fmt == kFmtE3M2) {
      // the ISA calls E3M2 "bf6" (its "fp6" is E2M3)
      const v6u w = __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(h, 1.0f);
      store8<COUNTED, KEEP>(q, v2u{w[0], w[1]});
      store8<COUNTED, KEEP>(q + 8, v2u{w[2], w[3]});
      store8<COUNTED, KEEP>(q + 16, v2u{w[4], w[5]});
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
      store16<COUNTED, KEEP>(q, v4u{out[0], out[1], out[2], out[3]});
      store16<COUNTED, KEEP>(q + 16, v4u{out[4], out[5], out[6], out[7]});
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The kernel (activations and weights): rows go global -> LDS directly.
//
// A workgroup owns rows first, first + gridDim.x, ... and a ring of NS row slots in LDS (row-major, as in
// memory).  The rows of the first NS iterations are requested before anything else happens
// (global_load_lds_dwordx4: no staging registers, nothing to wait for in the requesting wave); the slot a row
// leaves is refilled one iteration later, behind the barrier that also publishes the next row.  A lane gathers
// its channels with ds_read_u16_d16_hi, which puts the bf16 into the upper half of a register whose lower half
// is zero and stays zero -- the value is a float without a conversion instruction.
//
// EPL = 32: one lane per 32-element block (K/32 lanes).  EPL = 16: two lanes per block (K/16 lanes, K up to
// 16384): half the dependent work per lane and row, which is what bounds small problems -- the time from a
// row's arrival to its last store; the block's absmax is one cross-lane step.
//
// Everything a wave requests or stores goes through inline assembly, one instruction each, so that the waits
// on a row (s_waitcnt vmcnt(n): requests and stores complete in order) can count what was issued after it.
//
// T > 0: blockDim.x == T and the slot offsets are immediates of the LDS reads; T == 0: any blockDim.x, the
// slot offset is added to the addresses per row.
// ---------------------------------------------------------------------------------------------
// Sum of a double over the 64 lanes of a wave, the same value in every lane: four data-parallel-primitive steps inside
// the rows of 16 lanes (two register moves and an add each, no trip through the LDS crossbar), then the four row sums
// through scalar registers.
template <int CTRL>
__device__ __forceinline__ double dpp_add(double v) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const int lo = __builtin_amdgcn_mov_dpp((int)(uint32_t)b, CTRL, 0xF, 0xF, true);
  const int hi = __builtin_amdgcn_mov_dpp((int)(uint32_t)(b >> 32), CTRL, 0xF, 0xF, true);
  return v + __builtin_bit_cast(double, ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
}
__device__ __forceinline__ double wave_sum(double v) {
  v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141>(v);   // row_half_mirror: the other quad of the 8
  v = dpp_add<0x140>(v);   // row_mirror: the other 8 of the 16
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  double rows[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)b, 16 * r), hi = __builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), 16 * r);
    rows[r] = __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
  }
  return (rows[0] + rows[1]) + (rows[2] + rows[3]);
}

__device__ __forceinline__ void dma16(const uint8_t* base, unsigned voff, unsigned lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_off) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vm_imm() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

// s_waitcnt vmcnt(n) for a wave-uniform n: the wave's n most recent requests and stores may still be in flight
__device__ __forceinline__ void wait_vm(int n) {
  switch (n) {
#define MG_VM_CASE(N) case N: wait_vm_imm<N>(); break;
    MG_VM_CASE(0) MG_VM_CASE(1) MG_VM_CASE(2) MG_VM_CASE(3) MG_VM_CASE(4) MG_VM_CASE(5) MG_VM_CASE(6) MG_VM_CASE(7)
    MG_VM_CASE(8) MG_VM_CASE(9) MG_VM_CASE(10) MG_VM_CASE(11) MG_VM_CASE(12) MG_VM_CASE(13) MG_VM_CASE(14) MG_VM_CASE(15)
    MG_VM_CASE(16) MG_VM_CASE(17) MG_VM_CASE(18) MG_VM_CASE(19) MG_VM_CASE(20) MG_VM_CASE(21) MG_VM_CASE(22) MG_VM_CASE(23)
    MG_VM_CASE(24) MG_VM_CASE(25) MG_VM_CASE(26) MG_VM_CASE(27) MG_VM_CASE(28) MG_VM_CASE(29) MG_VM_CASE(30) MG_VM_CASE(31)
    MG_VM_CASE(32) MG_VM_CASE(33) MG_VM_CASE(34) MG_VM_CASE(35) MG_VM_CASE(36) MG_VM_CASE(37) MG_VM_CASE(38) MG_VM_CASE(39)
#undef MG_VM_CASE
    default: wait_vm_imm<40>(); break;   // n > 40: wait for a little more than necessary
  }
}

// 16 gathered channels: u[p] <- bf16 at LDS address ga[p] + OFF (an immediate), as the upper half.  OFF < 0 (the
// kernel with a run-time workgroup size, 1024 lanes and 128 registers each, which spills): at ga[p] + add, through
// reads the compiler sees and waits for itself, so that a spilled register is always a loaded one.
template <int OFF>
__device__ __forceinline__ void gather16(unsigned (&u)[16], const unsigned (&ga)[16], unsigned add) {
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    if constexpr (OFF >= 0) {
      asm volatile("ds_read_u16_d16_hi %0, %1 offset:%2" : "+v"(u[p]) : "v"(ga[p]), "n"(OFF));
    } else {
      typedef __attribute__((address_space(3))) const uint16_t* lds_u16;
      u[p] = (unsigned)*reinterpret_cast<lds_u16>((size_t)(ga[p] + add)) << 16;
    }
  }
}
// the reads above are invisible to the compiler's own wait insertion: wait here, with the registers tied to the wait
__device__ __forceinline__ void gather_wait(unsigned (&u)[16]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(u[0]), "+v"(u[1]), "+v"(u[2]), "+v"(u[3]), "+v"(u[4]), "+v"(u[5]), "+v"(u[6]), "+v"(u[7]),
                 "+v"(u[8]), "+v"(u[9]), "+v"(u[10]), "+v"(u[11]), "+v"(u[12]), "+v"(u[13]), "+v"(u[14]), "+v"(u[15]));
}

// Half a block (16 gathered values, lane pair 2b / 2b + 1 holds block b): the pair's absmax by one cross-lane
// step, then the same arithmetic as quantize_store; `half` (0 or 1) says which 16 elements these are.
template <bool KEEP = false>
__device__ __forceinline__ void quantize_store_half(const float (&f)[16], int fmt, int half, uint8_t* __restrict__ q,
                                                    uint8_t* __restrict__ sf) {
  float amax = 0.0f;
#pragma unroll
  for (int p = 0; p < 16; p += 2) amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fabsf(f[p])), __builtin_fabsf(f[p + 1]));
  // quad_perm [1, 0, 3, 2]: the other lane of the pair
  const float other = __uint_as_float((unsigned)__builtin_amdgcn_mov_dpp((int)__float_as_uint(amax), 0xB1, 0xF, 0xF, true));
  amax = __builtin_fmaxf(amax, other);
  const int byte = scale_byte(amax, fmt);
  const float rs1 = __uint_as_float(((unsigned)(254 - byte) << 23) | 0x800u);
  float v[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) v[p] = round_scaled(f[p], rs1);
  if (half == 0) store1<true>(sf, byte);
  if (fmt == kFmtE2M1) {
    v2u out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      unsigned w = 0;
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 0], v[8 * j + 1], 1.0f, 0);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 2], v[8 * j + 3], 1.0f, 1);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 4], v[8 * j + 5], 1.0f, 2);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[8 * j + 6], v[8 * j + 7], 1.0f, 3);
      out[j] = w;
    }
    store8<true, KEEP>(q + half * 8, out);
  } else {
    if (fmt == kFmtE3M2) {
      // 16 codes are the first 96 bits of the 32-code conversion
      v32bf h;
#pragma unroll
      for (int p = 0; p < 16; ++p) h[p] = (__bf16)v[p];
#pragma unroll
      for (int p = 16; p < 32; ++p) h[p] = (__bf16)0.0f;
      const v6u w = __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(h, 1.0f);
      typedef unsigned v3u __attribute__((ext_vector_type(3)));
      const v3u w3 = {w[0], w[1], w[2]};
      if constexpr (KEEP) asm volatile("global_store_dwordx3 %0, %1, off" : : "v"(q + half * 12), "v"(w3) : "memory");
      else asm volatile("global_store_dwordx3 %0, %1, off nt" : : "v"(q + half * 12), "v"(w3) : "memory");
    } else {
      unsigned out[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v2bf lo = {(__bf16)v[4 * j + 0], (__bf16)v[4 * j + 1]};
        const v2bf hi = {(__bf16)v[4 * j + 2], (__bf16)v[4 * j + 3]};
        v2s z = {0, 0};
        z = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, lo, 1.0f, false);
        z = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, hi, 1.0f, true);
        out[j] = __builtin_bit_cast(unsigned, z);
      }
      store16<true, KEEP>(q + half * 16, v4u{out[0], out[1], out[2], out[3]});
    }
  }
}


// Which rows a workgroup takes (see the kernel).  With a whole number `a` of rows per workgroup the plain schedule
// is `a` full iterations; the skewed one is a - 1 full iterations, one without the last generation of workgroups
// and one with the first generation only.  A CU's workgroups are dispatched one generation (gridDim.x / per-CU
// count) after the other and its memory requests are served in the order they were made, so the workgroup
// dispatched last gets its first row after everything its neighbours asked for at their start: it runs a row
// or two behind them for the whole launch, and the kernel ends when it does.  One row less for it and one more
// for the first generation evens that out (c1, 4 rows per workgroup: 10.2 -> 9.65 us).
struct RowSchedule {
  int head;       // iterations in which every workgroup takes a row
  int width[3];   // then: the first width[j] workgroups take one (0: nobody)
};

template <int EPL, int T, int NS, bool IS_W, int MAXT, bool KEEP = false, bool NORM = false>
__global__ void __launch_bounds__(MAXT)
reorder_quant_dma_kernel(const uint8_t* __restrict__ x, const int16_t* __restrict__ idx, int rows, int K, int KN, int KS,
                         int KO, uint8_t* __restrict__ qn, uint8_t* __restrict__ qs, uint8_t* __restrict__ qo,
                         uint8_t* __restrict__ sfn, uint8_t* __restrict__ sfs, uint8_t* __restrict__ sfo, RowSchedule sched,
                         const uint16_t* __restrict__ gamma, float eps) {
  extern __shared__ __align__(16) uint8_t lds[];
  __shared__ double row_sums[NORM ? 2 : 1][NORM ? MAXT / 64 : 1];   // RMSNorm: the waves' sums of squares, by row parity
  static_assert(EPL == 32 || EPL == 16, "one or two lanes per block");
  constexpr int kPieces = EPL / 8;   // 16-byte pieces of a row (and of the index) per lane
  constexpr int kParts = EPL / 16;   // gathers of 16 per lane and row
  constexpr bool kImm = T > 0;
  static_assert(!kImm || (NS - 1) * 2 * EPL * T <= 65535, "slot offsets must fit the LDS instructions' immediate");
  const int tid = threadIdx.x;
  const int nthr = kImm ? T : (int)blockDim.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned stride = 2u * EPL * nthr;   // bytes per slot: kPieces copies of nthr x 16 bytes, at least one row
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t*)lds;
  const int grid = gridDim.x;
  // Which row a workgroup starts with.  The scale bytes of 32 rows -- r % 32 in [8k, 8k + 8) for one k, any
  // (r / 32) % 4, of one group of 128 rows -- share a 128-byte line of a scale atom, and each row is written by
  // another workgroup.  Workgroups go to the 8 XCDs (one L2 each) round-robin by index, so the rows of a line
  // are given to workgroups of one XCD (row bits 3, 4, 7 = workgroup bits 0, 1, 2): its L2 then assembles the
  // whole line instead of eight L2s holding an eighth each until the write-back at the end of the kernel.
  int first = blockIdx.x;
  if (first < (grid & ~255)) {
    const int xcd = first & 7, y = (first >> 3) & 31;
    first = (first & ~255) | (y & 7) | ((xcd & 3) << 3) | (((y >> 3) & 3) << 5) | ((xcd >> 2) << 7);
  }
  // The rows of this workgroup: `sched.head` iterations in which every workgroup takes a row (iteration k: row
  // k * grid + first), then up to three iterations in which the first sched.width[j] workgroups do.
  const bool in_tail[3] = {first < sched.width[0], first < sched.width[1], first < sched.width[2]};
  const int count = sched.head + in_tail[0] + in_tail[1] + in_tail[2];
  auto row_of = [&](int k) {
    if (k < sched.head) return k * grid + first;
    int off = sched.head * grid, t = k - sched.head;   // the t-th tail iteration this workgroup is part of
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      if (in_tail[j]) {
        if (t == 0) break;
        --t;
      }
      off += sched.width[j];
    }
    return off + first;
  };
  const size_t row_bytes = (size_t)K * 2;

  // per-lane byte offsets of the lane's 16-byte pieces of a row (pieces past the row's end: the last one
  // again, into the slot's padding)
  const int nchunks = K >> 3;
  unsigned voff[kPieces];
#pragma unroll
  for (int it = 0; it < kPieces; ++it) voff[it] = (unsigned)min(it * nthr + tid, nchunks - 1) * 16u;
  const unsigned wave_lds = lds0 + (unsigned)wave * 1024u;
  auto request = [&](const uint8_t* base, unsigned slot_off) {
#pragma unroll
    for (int it = 0; it < kPieces; ++it) dma16(base, voff[it], wave_lds + slot_off + (unsigned)it * nthr * 16u);
  };

  // the lane's block and, with two lanes per block, its half
  const int b = EPL == 32 ? tid : tid >> 1;
  const int half = EPL == 32 ? 0 : tid & 1;
  const bool has_block = b < (K >> 5);

  // ---- everything this workgroup can have in flight, requested up front: the lane's EPL index entries (into
  //      registers), then the first NS rows
  v4u iv[kPieces];
  {
    const v4u* ip = reinterpret_cast<const v4u*>(idx + (size_t)(has_block ? b : 0) * 32 + half * 16);
    // (kernels with a compile-time workgroup size: as uncounted loads, waited for below; they compile without scratch
    // memory -- the build checks it --, so that no register is moved before its load has landed)
#pragma unroll
    for (int q = 0; q < kPieces; ++q) {
      if constexpr (kImm) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(iv[q]) : "v"(ip + q) : "memory");
      else iv[q] = ip[q];
    }
  }
#pragma unroll
  for (int s = 0; s < NS; ++s)
    if (s < count) request(x + (size_t)row_of(s) * row_bytes, s * stride);
  // RMSNorm: the weights of this lane's pieces of a row (the same for every row); ordinary loads, which the compiler
  // waits for itself where they are first used (with vmcnt(0): once, in the first row)
  v4u gv[kPieces];
  if constexpr (NORM) {
#pragma unroll
    for (int it = 0; it < kPieces; ++it)
      gv[it] = *reinterpret_cast<const v4u*>(gamma + (size_t)min(it * nthr + tid, nchunks - 1) * 8);
  }

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

  // ---- the index entries are the oldest requests: they are there when at most the row copies are in flight
  wait_vm(kPieces * min(NS, count));
  if constexpr (kPieces == 4) asm volatile("" : "+v"(iv[0]), "+v"(iv[1]), "+v"(iv[2]), "+v"(iv[3]));
  else asm volatile("" : "+v"(iv[0]), "+v"(iv[1]));
  // LDS byte addresses of the lane's gathered channels in slot 0.  An entry outside [0, K) is read as
  // channel K - 1, so that the gather stays inside the row whatever the index holds.
  unsigned ga[kParts][16];
#pragma unroll
  for (int q = 0; q < kPieces; ++q)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      ga[q >> 1][(q & 1) * 8 + e] =
          lds0 + min((e & 1) ? (iv[q][e >> 1] >> 16) : (iv[q][e >> 1] & 0xffffu), (unsigned)(K - 1)) * 2u;
  unsigned u[kParts][16];
#pragma unroll
  for (int h = 0; h < kParts; ++h)
#pragma unroll
    for (int p = 0; p < 16; ++p) u[h][p] = 0u;
  // store instructions this wave issues per row: the scale byte, and the codes once per format its lanes have
  const int fmt_or_none = has_block ? fmt : -1;
  const int row_stores =
      1 + (__builtin_amdgcn_ballot_w64(fmt_or_none == kFmtE2M1) ? (EPL == 32 ? code_stores(kFmtE2M1) : 1) : 0) +
      (__builtin_amdgcn_ballot_w64(fmt_or_none == kFmtE3M2) ? (EPL == 32 ? code_stores(kFmtE3M2) : 1) : 0) +
      (__builtin_amdgcn_ballot_w64(fmt_or_none == kFmtE4M3) ? (EPL == 32 ? code_stores(kFmtE4M3) : 1) : 0);

  int i = 0;
  auto body = [&](auto slot_c) {
    constexpr int S = decltype(slot_c)::value;
    const int row = row_of(i);
    // Row i has landed when at most what was issued after its request is in flight (requests and stores complete
    // in order): the requests of the rows after it -- NS - 1 of them at the start, NS - 2 once refills follow the
    // iterations -- and the stores of the iterations since, at most NS - 1 of them.
    wait_vm(kPieces * min(i == 0 ? NS - 1 : NS - 2, count - 1 - i) + row_stores * min(i, NS - 1));
    if constexpr (NORM) {
      // RMSNorm of the row, in place, before anyone gathers from it (the arithmetic of the usual fp32 implementation):
      //   var = fl32( (sum over the row of x^2, accumulated in fp64) / K )
      //   r   = fl32( 1 / sqrt( fl32(var + eps) ) )      (division and square root in fp64)
      //   y   = bf16( gamma * bf16( x * r ) )            (both products in fp32)
      // The fp64 sum makes the result independent of the order in which the lanes add their parts (up to the last
      // bit of a double, which the rounding to fp32 all but never sees).  A lane works on the pieces it copied.
      uint8_t* slot = lds + S * stride;
      v4u a[kPieces];
      double part[4] = {0.0, 0.0, 0.0, 0.0};   // four chains: one chain of dependent fp64 fmas would wait for each in turn
#pragma unroll
      for (int it = 0; it < kPieces; ++it) {
        a[it] = *reinterpret_cast<const v4u*>(slot + (size_t)(it * nthr + tid) * 16);
        if (it * nthr + tid < nchunks) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned d = a[it][e];
            const double lo = (double)__uint_as_float(d << 16), hi = (double)__uint_as_float(d & 0xffff0000u);
            part[e] = __builtin_fma(lo, lo, part[e]);
            part[e] = __builtin_fma(hi, hi, part[e]);
          }
        }
      }
      double ss = wave_sum((part[0] + part[1]) + (part[2] + part[3]));
      if ((tid & 63) == 0) row_sums[i & 1][tid >> 6] = ss;
      __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the sum is in the LDS (a raw barrier implies no wait of the compiler's)
      asm volatile("s_barrier" ::: "memory");   // also: every wave's copies of row i have landed, every wave is past its gather of row i - 1
      if (i >= 1 && i - 1 + NS < count)
        request(x + (size_t)row_of(i + NS - 1) * row_bytes, ((S + NS - 1) % NS) * stride);
      double tot = 0.0;
      for (int w = 0; w < (nthr >> 6); ++w) tot += row_sums[i & 1][w];
      const float var = (float)(tot / (double)K);
      const float rn = (float)(1.0 / __builtin_sqrt((double)(var + eps)));
#pragma unroll
      for (int it = 0; it < kPieces; ++it) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const unsigned d = a[it][e], g = gv[it][e];
          const float h0 = (float)(__bf16)(__uint_as_float(d << 16) * rn);
          const float h1 = (float)(__bf16)(__uint_as_float(d & 0xffff0000u) * rn);
          const v2bf y = {(__bf16)(__uint_as_float(g << 16) * h0), (__bf16)(__uint_as_float(g & 0xffff0000u) * h1)};
          a[it][e] = __builtin_bit_cast(unsigned, y);
        }
        if (it * nthr + tid < nchunks) *reinterpret_cast<v4u*>(slot + (size_t)(it * nthr + tid) * 16) = a[it];
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);
      asm volatile("s_barrier" ::: "memory");   // the normalized row is complete
    } else {
      asm volatile("s_barrier" ::: "memory");
      // every wave is past its gather of row i - 1: refill that row's slot
      if (i >= 1 && i - 1 + NS < count)
        request(x + (size_t)row_of(i + NS - 1) * row_bytes, ((S + NS - 1) % NS) * stride);
    }
    if (has_block) {
      constexpr int kOff = kImm ? S * 2 * EPL * T : -1;
#pragma unroll
      for (int h = 0; h < kParts; ++h) gather16<kOff>(u[h], ga[h], S * stride);
#pragma unroll
      for (int h = 0; h < kParts; ++h) gather_wait(u[h]);
      uint8_t* q = qbase + (size_t)row * pitch;
      uint8_t* sf = sfbase + sf_offset(row, j, katoms);
      if constexpr (EPL == 32) {
        float f[32];
#pragma unroll
        for (int p = 0; p < 32; ++p) f[p] = __uint_as_float(u[p >> 4][p & 15]);
        quantize_store<true, KEEP>(f, fmt, q, sf);
      } else {
        float f[16];
#pragma unroll
        for (int p = 0; p < 16; ++p) f[p] = __uint_as_float(u[0][p]);
        quantize_store_half<KEEP>(f, fmt, half, q, sf);
      }
    }
  };
  auto run = [&](auto self, auto slot_c) -> void {
    constexpr int S = decltype(slot_c)::value;
    body(slot_c);
    ++i;
    if constexpr (S + 1 < NS) {
      if (i < count) self(self, std::integral_constant<int, S + 1>{});
    }
  };
  while (i < count) run(run, std::integral_constant<int, 0>{});
}

}  // namespace

// gamma != nullptr: RMSNorm with that weight and eps before the gather (activations only)
template <bool IS_W>
hipError_t launch_reorder_quant(const void* x, const int16_t* idx, int rows, int K, int KN, int KS, int KO, uint8_t* qn,
                                uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo,
                                const void* gamma, float eps, bool keep_codes, hipStream_t stream) {
  if (rows == 0 || K == 0) return hipSuccess;
  if (gamma != nullptr && IS_W) return hipErrorInvalidValue;
  const uint16_t* gm = static_cast<const uint16_t*>(gamma);
  const int threads = ((K >> 5) + 63) & ~63;
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  DeviceLimits lim;
  if (hipError_t e = device_limits(&lim); e != hipSuccess) return e;
  hipError_t err = hipSuccess;
  // rows global -> LDS directly; NS row slots per workgroup, as many workgroups per CU as fit
  const int usable = lim.lds_bytes - 1024;   // the kernels' static LDS (row sums of the RMSNorm) stays below 1 KB
  auto launch_dma = [&](auto kernel, int epl, int NS, int nthreads, int max_per_cu) {
    const int lds = NS * 2 * epl * nthreads;   // NS row slots
    if (lds > usable) { err = hipErrorInvalidValue; return; }
    int per_cu = usable / lds;
    per_cu = per_cu > max_per_cu ? max_per_cu : per_cu;
    const int by_waves = 16 / (nthreads / 64);
    per_cu = per_cu > by_waves ? (by_waves < 1 ? 1 : by_waves) : per_cu;
    const int resident = lim.cus * per_cu;
    const int grid = rows < resident ? rows : resident;
    const int a = rows / grid, rem = rows - a * grid;
    RowSchedule sched;
    if (a >= 2 && per_cu >= 3 && grid == resident) {
      sched = RowSchedule{a - 1, {grid - lim.cus, lim.cus, rem}};
    } else {
      sched = RowSchedule{a - 1, {grid, rem, 0}};
    }
    err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), usable);
    if (err != hipSuccess) return;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(nthreads), (size_t)lds, stream, xb, idx, rows, K, KN, KS, KO, qn, qs, qo, sfn,
                       sfs, sfo, sched, gm, eps);
    err = hipGetLastError();
  };
  // Measured on M = 4096 ... 16384 rows of K = 3584 ... 18944: two row slots per workgroup, and per CU up to four
  // workgroups but no more than 16 waves (K = 5120: 3 x 5 waves, K = 12288: 2 x 6); more of either puts more requests
  // in front of a workgroup's first row and was slower.
  constexpr int kNS = 2;
  constexpr int kPerCu = 4;
  // keep: the codes stay in the L2 for the kernel that reads them next (activations only); norm: RMSNorm of the row
  // before the gather (activations only; its codes are always kept: what follows a norm is the layer's GEMM)
  auto dispatch = [&](auto keep_c, auto norm_c) {
    constexpr bool KP = decltype(keep_c)::value;
    constexpr bool NM = decltype(norm_c)::value;
    if (K <= 8192) {
      // two lanes per block: K/16 lanes, rounded up to whole waves
      const int t2 = ((K >> 4) + 63) & ~63;
      switch (t2) {
        case 64: launch_dma(reorder_quant_dma_kernel<16, 64, kNS, IS_W, 64, KP, NM>, 16, kNS, 64, kPerCu); break;
        case 128: launch_dma(reorder_quant_dma_kernel<16, 128, kNS, IS_W, 128, KP, NM>, 16, kNS, 128, kPerCu); break;
        case 192: launch_dma(reorder_quant_dma_kernel<16, 192, kNS, IS_W, 192, KP, NM>, 16, kNS, 192, kPerCu); break;
        case 256: launch_dma(reorder_quant_dma_kernel<16, 256, kNS, IS_W, 256, KP, NM>, 16, kNS, 256, kPerCu); break;
        case 320: launch_dma(reorder_quant_dma_kernel<16, 320, kNS, IS_W, 320, KP, NM>, 16, kNS, 320, kPerCu); break;
        case 384: launch_dma(reorder_quant_dma_kernel<16, 384, kNS, IS_W, 384, KP, NM>, 16, kNS, 384, kPerCu); break;
        case 448: launch_dma(reorder_quant_dma_kernel<16, 448, kNS, IS_W, 448, KP, NM>, 16, kNS, 448, kPerCu); break;
        default: launch_dma(reorder_quant_dma_kernel<16, 512, kNS, IS_W, 512, KP, NM>, 16, kNS, 512, kPerCu); break;
      }
    } else if (K <= 20480) {
      // one lane per block: the workgroups are large enough as it is, and LDS (two rows per workgroup) bounds how
      // many a CU holds
      switch (threads) {
        case 320: launch_dma(reorder_quant_dma_kernel<32, 320, kNS, IS_W, 320, KP, NM>, 32, kNS, 320, kPerCu); break;
        case 384: launch_dma(reorder_quant_dma_kernel<32, 384, kNS, IS_W, 384, KP, NM>, 32, kNS, 384, kPerCu); break;
        case 448: launch_dma(reorder_quant_dma_kernel<32, 448, kNS, IS_W, 448, KP, NM>, 32, kNS, 448, kPerCu); break;
        case 512: launch_dma(reorder_quant_dma_kernel<32, 512, kNS, IS_W, 512, KP, NM>, 32, kNS, 512, kPerCu); break;
        case 576: launch_dma(reorder_quant_dma_kernel<32, 576, kNS, IS_W, 576, KP, NM>, 32, kNS, 576, kPerCu); break;
        default: launch_dma(reorder_quant_dma_kernel<32, 640, kNS, IS_W, 640, KP, NM>, 32, kNS, 640, kPerCu); break;
      }
    } else {
      launch_dma(reorder_quant_dma_kernel<32, 0, 2, IS_W, 1024, KP, NM>, 32, 2, threads, kPerCu);
    }
  };
  if constexpr (IS_W) {
    dispatch(std::false_type{}, std::false_type{});
  } else {
    if (gamma != nullptr) dispatch(std::true_type{}, std::true_type{});
    else if (keep_codes) dispatch(std::true_type{}, std::false_type{});
    else dispatch(std::false_type{}, std::false_type{});
  }
  return err;
}

template hipError_t launch_reorder_quant<false>(const void*, const int16_t*, int, int, int, int, int, uint8_t*, uint8_t*,
                                                uint8_t*, uint8_t*, uint8_t*, uint8_t*, const void*, float, bool, hipStream_t);
template hipError_t launch_reorder_quant<true>(const void*, const int16_t*, int, int, int, int, int, uint8_t*, uint8_t*,
                                               uint8_t*, uint8_t*, uint8_t*, uint8_t*, const void*, float, bool, hipStream_t);

}  // namespace mg
