// Mixed block-scaled GEMM for large whole-tile shapes: 256 x 256 workgroup tiles, one workgroup
// of 8 waves per CU (two per SIMD), each wave 128 features x 64 tokens = 4 x 2 tiles of
// v_mfma_scale_f32_32x32x64_f8f6f4 (128 accumulator registers).  Replaces the three CUTLASS GEMMs
// of the reference (src/fp4.cu:35, src/fp6.cu:35, src/fp8.cu:35, driver src/gemm.cu:22-47) for
// N a multiple of 8 and every K segment at least 128 wide (a multiple of 32), or absent.
//
// Next to an MFMA (32 cycles in the matrix pipe) a wave gets only a handful of other instructions
// for free; with two waves per SIMD one wave's copy and fragment-read instructions issue while the
// other's MFMA runs (with one wave of 128 x 128 per SIMD the K loop took 10 % more cycles), and the
// steady state is written to need few of them:
//   * operands and scale atoms go global -> LDS directly (global_load_lds_dwordx4 / _dword); a copy
//     is a scalar base (advanced once per stage), a per-lane offset fixed for the segment, and an LDS
//     offset that is an immediate (the three stage buffers are three copies of the loop body);
//   * fragment reads use per-lane LDS addresses fixed for the segment plus immediates;
//   * copies are spread between the MFMAs, one after every second MFMA.
// Pipeline per K stage q (128 elements), three LDS buffers:
//   read second half of q | 8 MFMAs first half, last copies of q+2 | own reads done, own copies
//   of q+1 landed (those of q+2 stay in flight) | barrier | read first half + scales of q+1 |
//   8 MFMAs second half, first copies of q+3 into the buffer stage q just freed.
// The last three stages of a segment copy stages of the next segment(s); plans whose segments are
// too short for that run a generic body whose copy format is a run-time, wave-uniform value.
// The result tile is transposed through LDS so that stores write 256 contiguous bytes per row.
#include "mg_common.h"

#include <type_traits>

namespace mg {

namespace {

constexpr int kT = 256;                   // tile edge (features and tokens)
constexpr int kBlk = 1040;                // 16 rows x 64 B + 16
constexpr int kBlk6 = 3088;               // 32 rows x 96 B + 16
constexpr int kWOff = 0;
constexpr int kXOff = 16 * kBlk;          // 16640
constexpr int kSOff = kXOff + 32 * kBlk;  // E4M3 worst case: two K halves x 16 blocks -> 49920
constexpr int kStage = kSOff + 2048;      // 51968
constexpr int kBuffers = 3;
constexpr int kStartSkew = 8000;          // see the kernel: largest start delay, in ticks of s_memtime (about 4 us)

// Eight waves per workgroup, two per SIMD: a wave's tile is 128 features x 32 * TM tokens (TM = 2: the workgroup's
// tile is 256 x 256; TM = 1: 256 x 128), 64 * TM accumulator registers, so that two waves fit a SIMD's register file
// and one wave's copy and fragment-read instructions issue while the other's MFMA runs.  A stage's copies are dealt to
// the waves so that the workgroup moves every byte exactly once: per wave 2 weight blocks, 2 / 3 / 4 token copies
// (E2M1 / E3M2 / E4M3) and a quarter of a scale atom pair (a 4-byte copy).
constexpr int kWaves = 8;
constexpr int kWCopies = 2;                            // weight copy blocks per wave and stage
constexpr int kXSlots = 4;                             // token copy slots per wave and stage (E4M3 uses them all)
constexpr int kCopySlots = kWCopies + kXSlots + 1;     // + the scale copy
constexpr int kSplit = 3;                              // slots [0, kSplit) go out in the second half of a stage, the rest in the next first half

typedef int v6i __attribute__((ext_vector_type(6)));

// Kernel arguments: per K segment (0: E2M1, 1: E3M2, 2: E4M3 activations) the code and scale
// pointers and the number of 128-wide stages.
struct Plan {
  const uint8_t *a0, *a1, *a2;        // activation codes
  const uint8_t *b0, *b1, *b2;        // weight codes
  const uint8_t *sfa0, *sfa1, *sfa2;  // activation scales
  const uint8_t *sfb0, *sfb1, *sfb2;  // weight scales
  int st0, st1, st2;                  // whole 128-wide stages per segment
  int blk0, blk1, blk2;               // 32-element blocks per segment (row pitches and scale atoms; up to 3 more than 4 * st)
  int total;                          // stages over all segments
  int w_tiled;                        // weights in tile-major order (see tile_weights_kernel): a copy reads 1 KB of consecutive bytes
};

__device__ __forceinline__ const uint8_t* uni(const uint8_t* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
}

// Field of segment sg (0, 1, 2) by masking rather than by select: a select between adjacent struct
// fields is rewritten by the compiler into a dynamically indexed load from a private copy.
__device__ __forceinline__ uint64_t pick3(int sg, uint64_t v0, uint64_t v1, uint64_t v2) {
  const uint64_t m0 = sg == 0 ? ~0ull : 0ull, m1 = sg == 1 ? ~0ull : 0ull, m2 = sg == 2 ? ~0ull : 0ull;
  return (v0 & m0) | (v1 & m1) | (v2 & m2);
}
__device__ __forceinline__ const uint8_t* pick3(int sg, const uint8_t* p0, const uint8_t* p1, const uint8_t* p2) {
  return reinterpret_cast<const uint8_t*>(pick3(sg, reinterpret_cast<uint64_t>(p0), reinterpret_cast<uint64_t>(p1),
                                                reinterpret_cast<uint64_t>(p2)));
}
__device__ __forceinline__ unsigned pick3u(int sg, unsigned v0, unsigned v1, unsigned v2) {
  const unsigned m0 = sg == 0 ? ~0u : 0u, m1 = sg == 1 ? ~0u : 0u, m2 = sg == 2 ? ~0u : 0u;
  return (v0 & m0) | (v1 & m1) | (v2 & m2);
}

// Which segment a global stage index falls in (uniform).
__device__ __forceinline__ int seg_of(const Plan& p, int q, int& local) {
  if (q < p.st0) { local = q; return 0; }
  q -= p.st0;
  if (q < p.st1) { local = q; return 1; }
  local = q - p.st1;
  return 2;
}

constexpr int kFmtNone = -1;   // "no stage": copies of a stage past the end of K

template <int FMT> struct Fmt;
template <> struct Fmt<kFmtNone> { static constexpr int seg = 3, row_bytes = 0, x_copies = 0; typedef v4i xfrag; };
template <> struct Fmt<kFmtE2M1> { static constexpr int seg = 0, row_bytes = 64, x_copies = 4; typedef v4i xfrag; };
template <> struct Fmt<kFmtE3M2> { static constexpr int seg = 1, row_bytes = 96, x_copies = 6; typedef v6i xfrag; };
template <> struct Fmt<kFmtE4M3> { static constexpr int seg = 2, row_bytes = 128, x_copies = 8; typedef v8i xfrag; };

// ---------------------------------------------------------------------------------------------
// Copies.  One instruction moves 64 x 16 B to 1 KB of consecutive LDS.  Weights and E2M1 / E4M3
// tokens: 16 rows x 64 B (a lane quad reads 64 contiguous bytes of one row), rows j, j+16, ...,
// j+240 of the tile into block j at j * 1040 (E4M3: one set of 16 blocks per 64-wide K half).
// E3M2 rows are 96 B: three instructions move the 32 rows j, j+8, ..., j+248 as one row-major
// block of 3072 B at j * 3088.  Last slot: the stage's four scale atoms (two of the features, two
// of the tokens, 2 KB) as eight 4-byte copies, one per wave.
// ---------------------------------------------------------------------------------------------

// global[base + voff(lane)] -> LDS[lds_off + 16 * lane]; base and lds_off are wave-uniform
__device__ __forceinline__ void copy16(const uint8_t* base, unsigned voff, unsigned lds_off) {
  base = uni(base);
  lds_off = __builtin_amdgcn_readfirstlane(lds_off);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_off) : "memory", "m0");
}

// the same with the LDS offset as scalar register + immediate
template <int OFF>
__device__ __forceinline__ void copy16i(const uint8_t* base, unsigned voff, unsigned lds_sreg) {
  base = uni(base);                                         // no-ops when the values are already in scalar registers
  lds_sreg = __builtin_amdgcn_readfirstlane(lds_sreg);
  asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_sreg), "n"(OFF) : "memory", "m0", "scc");
}

// the same with an immediate byte offset on the global address as well.  The hardware adds the
// instruction's immediate to the LDS address too, so M0 gets the LDS offset less the immediate.
template <int OFF, int GOFF>
__device__ __forceinline__ void copy16io(const uint8_t* base, unsigned voff, unsigned lds_sreg) {
  static_assert(GOFF >= 0 && GOFF < 4096 && OFF >= GOFF, "global_load immediate offset");
  base = uni(base);
  lds_sreg = __builtin_amdgcn_readfirstlane(lds_sreg);
  asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%4"
               : : "v"(voff), "s"(base), "s"(lds_sreg), "n"(OFF - GOFF), "n"(GOFF) : "memory", "m0", "scc");
}

// 4-byte copies: global[base + voff(lane)] -> LDS[lds_off + 4 * lane] (a quarter of a scale atom pair per wave)
__device__ __forceinline__ void copy4(const uint8_t* base, unsigned voff, unsigned lds_off) {
  base = uni(base);
  lds_off = __builtin_amdgcn_readfirstlane(lds_off);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_off) : "memory", "m0");
}
template <int OFF>
__device__ __forceinline__ void copy4i(const uint8_t* base, unsigned voff, unsigned lds_sreg) {
  base = uni(base);
  lds_sreg = __builtin_amdgcn_readfirstlane(lds_sreg);
  asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               : : "v"(voff), "s"(base), "s"(lds_sreg), "n"(OFF) : "memory", "m0", "scc");
}

struct Ctx {
  int n0, m0, lane, wave, wn, wm, total;
  int xatom, xtile;    // the wave's token tiles: scale atom (of 128 rows) of the workgroup's tile, and the first one's index (0 ... 3) in that atom
  int rows_avail;      // activation rows that may be read from m0 on (codes and scales); 1 ... 256
  int cols_avail;      // features of the tile that exist (weight rows and scales that may be read from n0 on); 1 ... 256
  unsigned lds_base;   // LDS byte offset of the dynamic shared memory
};

// Per-lane byte offsets of the copies, fixed for the whole kernel.
// Token rows are clamped to the last readable row of the tile (rows_avail - 1): in the last, partial
// token tile the lanes of rows past it copy that row again, into LDS rows of tokens that are never stored.
struct LaneOffsets {
  unsigned s0, s1, s2;      // the wave's quarter of a segment's scale atom pair, 4 bytes per lane
  int lane, wave, last_row, last_col, prow;

  __device__ __forceinline__ LaneOffsets(const Plan& p, const Ctx& cx) {
    lane = cx.lane;
    wave = cx.wave;
    last_row = cx.rows_avail - 1;
    last_col = cx.cols_avail - 1;
    // quad k of a copy holds tile row j + 16 * (2 * (k % 8) + k / 8): rows 32t + i and 32t + i + 16 of a
    // fragment end up 512 B apart in their block, which the LDS reads conflict-free (64 B apart they collide)
    const unsigned k = lane >> 2, pr = 2 * (k & 7) + (k >> 3);
    prow = 16 * pr;
    // scale atoms: waves 0-3 copy a quarter each (256 bytes, 4 per lane) of the tile's two feature atoms, waves 4-7
    // of its two token atoms; the second atom of a tile exists only past 128 features / readable token rows
    const unsigned hi = (wave >= 4 ? cx.rows_avail : cx.cols_avail) <= 128 ? 0 : (wave >> 1) & 1;
    const unsigned lo = (wave & 1) * 256 + lane * 4;
    s0 = hi * ((p.blk0 + 3) >> 2) * 512 + lo;
    s1 = hi * ((p.blk1 + 3) >> 2) * 512 + lo;
    s2 = hi * ((p.blk2 + 3) >> 2) * 512 + lo;
  }

  // Byte offset, from the tile's first weight row, that this lane reads in weight copy k of a stage (row-major
  // weights, row pitch ldb): 64 bytes of row 2 * wave + k + 16 * pr, clamped to the last feature that exists.
  __device__ __forceinline__ unsigned woff(int k, unsigned ldb) const {
    return (unsigned)min(prow + kWCopies * wave + k, last_col) * ldb + (lane & 3) * 16;
  }

  // Byte offset, from the tile's first token row, that this lane reads in token copy kx of a stage of
  // segment sg (row pitch lda).  E2M1: rows 2 * wave + kx + 16 * pr, 16-byte piece lane % 4; E4M3: rows
  // 4 * (wave % 4) + kx + 16 * pr; E3M2: piece c % 6 of row wave + 8 * (c / 6), c = 64 * kx + lane.
  __device__ __forceinline__ unsigned xoff(int sg, int kx, unsigned lda) const {
    if (sg == 1) {
      const int c = 64 * kx + lane;
      return (unsigned)min(8 * (c / 6) + wave, last_row) * lda + (c % 6) * 16;
    }
    const int first = sg == 0 ? 2 * wave : 4 * (wave & 3);
    return (unsigned)min(prow + first + kx, last_row) * lda + (lane & 3) * 16;
  }
};

struct StageBases {
  const uint8_t *w, *x, *s;
  unsigned ldb, lda;
  int seg;   // -1: no such stage
  bool tiled;   // tile-major weights

  __device__ __forceinline__ StageBases() : w(nullptr), x(nullptr), s(nullptr), ldb(0), lda(0), seg(-1), tiled(false) {}

  __device__ __forceinline__ StageBases(const Plan& plan, int q, const Ctx& c) {
    int ql;
    const int sg = seg_of(plan, q, ql);
    seg = q < plan.total ? sg : -1;
    const uint8_t* pa = pick3(sg, plan.a0, plan.a1, plan.a2);
    const uint8_t* pb = pick3(sg, plan.b0, plan.b1, plan.b2);
    const uint8_t* psa = pick3(sg, plan.sfa0, plan.sfa1, plan.sfa2);
    const uint8_t* psb = pick3(sg, plan.sfb0, plan.sfb1, plan.sfb2);
    const unsigned blk = (unsigned)pick3(sg, (uint64_t)plan.blk0, (uint64_t)plan.blk1, (uint64_t)plan.blk2);
    const unsigned nst = (blk + 3) >> 2;   // scale atoms along K
    const unsigned rb = sg == 0 ? 64 : (sg == 1 ? 96 : 128);
    ldb = blk * 16;
    lda = blk * (rb >> 2);
    tiled = plan.w_tiled != 0;
    if (plan.w_tiled) {
      // 16 KB per (feature tile, stage), 1 KB per copy block: the wave's 4 blocks are consecutive
      const unsigned nstg = (unsigned)pick3(sg, (uint64_t)plan.st0, (uint64_t)plan.st1, (uint64_t)plan.st2);
      w = pb + (((size_t)(c.n0 >> 8) * nstg + ql) * 16 + c.wave * kWCopies) * 1024;
      ldb = 1024;
    } else {
      w = pb + (size_t)c.n0 * ldb + (size_t)ql * 64;   // the lanes' offsets carry the wave's rows
    }
    // the tile's first token row (the lanes' offsets carry the wave's rows); E4M3: K half wave / 4
    x = pa + (size_t)c.m0 * lda + (size_t)ql * rb + (sg == 2 ? (c.wave >> 2) * 64 : 0);
    s = c.wave < 4 ? psb + ((size_t)(c.n0 >> 7) * nst + ql) * 512 : psa + ((size_t)(c.m0 >> 7) * nst + ql) * 512;
  }
};

// Copies of a stage whose format is only known at run time (segment boundaries, prologue).
struct GenericCopy {
  StageBases b;
  unsigned buf;   // LDS byte offset of the target stage buffer

  __device__ __forceinline__ GenericCopy() : buf(0) {}
  __device__ __forceinline__ GenericCopy(const Plan& plan, int q, const Ctx& c)
      : b(plan, q, c), buf(c.lds_base + (q % kBuffers) * kStage) {}

  __device__ __forceinline__ int count() const {
    return b.seg < 0 ? 0 : kWCopies + (b.seg == 0 ? kXSlots / 2 : (b.seg == 1 ? 3 * kXSlots / 4 : kXSlots)) + 1;
  }

  template <int K>
  __device__ __forceinline__ void issue(const LaneOffsets& lo, int wave) const {
    if (b.seg < 0) return;
    if constexpr (K < kWCopies) {
      if (b.tiled) copy16(b.w + (size_t)K * 1024, lo.lane * 16, buf + kWOff + (wave * kWCopies + K) * kBlk);
      else copy16(b.w, lo.woff(K, b.ldb), buf + kWOff + (wave * kWCopies + K) * kBlk);
    } else if constexpr (K < kCopySlots - 1) {
      constexpr int kx = K - kWCopies;
      if (b.seg == 0) {
        if constexpr (kx < kXSlots / 2) copy16(b.x, lo.xoff(0, kx, b.lda), buf + kXOff + (wave * (kXSlots / 2) + kx) * kBlk);
      } else if (b.seg == 1) {
        if constexpr (kx < 3 * kXSlots / 4) copy16(b.x, lo.xoff(1, kx, b.lda), buf + kXOff + wave * kBlk6 + kx * 1024);
      } else {
        copy16(b.x, lo.xoff(2, kx, b.lda), buf + kXOff + (wave * kXSlots + kx) * kBlk);
      }
    } else {
      copy4(b.s, pick3u(b.seg, lo.s0, lo.s1, lo.s2), buf + kSOff + wave * 256);
    }
  }
};

template <int K0, int K1>
__device__ __forceinline__ void issue_range(const GenericCopy& cp, const LaneOffsets& lo, int wave) {
  if constexpr (K0 < K1) {
    cp.template issue<K0>(lo, wave);
    issue_range<K0 + 1, K1>(cp, lo, wave);
  }
}

// Copies of stages inside one segment of format FMT: scalar bases advanced by one stage at a time,
// per-lane offsets (one register per copy, the row step of the copy folded in) fixed.
// WT: weights in tile-major order -- one per-lane offset (16 * lane) and immediates for all four
// weight copies; vw[] is then unused.
template <int FMT, bool WT>
struct LeanCopy {
  static constexpr int WC = kWCopies;
  static constexpr int NX = Fmt<FMT>::x_copies / 2;
  // token copies, rows clamped to the last readable one.  E2M1, E3M2: one offset per copy.  E4M3, of which
  // there are few stages: the first copy's offset, and in its bits 0-2 how many of the three row steps that
  // follow stay inside the readable rows.  (These offsets are multiples of 16.)
  static constexpr int NV = FMT == kFmtE4M3 ? 1 : (FMT == kFmtE3M2 ? 3 : NX);
  const uint8_t *w, *x, *s;        // bases of the stage being copied
  unsigned lds_w, lds_x, lds_s;    // LDS offsets of the wave's first weight / token block and scale atom pair in buffer 0
  unsigned lda;
  unsigned vw[WC], vx[NV], vs, vlin;

  __device__ __forceinline__ void init(const Plan& plan, int q, const LaneOffsets&, const Ctx& c) {
    const LaneOffsets lo(plan, c);   // recomputed here rather than kept in registers across the K loop
    const StageBases b(plan, q, c);
    w = uni(b.w);
    x = uni(b.x);
    s = uni(b.s);
    constexpr int sg = Fmt<FMT>::seg;
    vlin = c.lane * 16;
    if constexpr (!WT) {
#pragma unroll
      for (int k = 0; k < WC; ++k) vw[k] = lo.woff(k, b.ldb);
    }
    lda = __builtin_amdgcn_readfirstlane(b.lda);
    if constexpr (FMT == kFmtE4M3) {
      const int row0 = lo.prow + 4 * (c.wave & 3);
      vx[0] = lo.xoff(2, 0, b.lda) | (unsigned)min(max(lo.last_row - row0, 0), NX - 1);
    } else if constexpr (FMT == kFmtE3M2) {
#pragma unroll
      for (int t = 0; t < 3; ++t) vx[t] = lo.xoff(1, t, b.lda);
    } else {
#pragma unroll
      for (int k = 0; k < NX; ++k) vx[k] = lo.xoff(0, k, b.lda);
    }
    vs = sg == 0 ? lo.s0 : (sg == 1 ? lo.s1 : lo.s2);
    lds_w = __builtin_amdgcn_readfirstlane(c.lds_base + kWOff + c.wave * WC * kBlk);
    lds_x = __builtin_amdgcn_readfirstlane(c.lds_base + kXOff +
                                           c.wave * (FMT == kFmtE3M2 ? kBlk6 : NX * kBlk));
    lds_s = __builtin_amdgcn_readfirstlane(c.lds_base + kSOff + c.wave * 256);
  }

  __device__ __forceinline__ void advance() {
    w += WT ? 16384 : 64;
    x += Fmt<FMT>::row_bytes;
    s += 512;
  }

  static constexpr int count() { return WC + NX + 1; }

  // slot K into the stage buffer at byte offset boff (wave-uniform)
  template <int K>
  __device__ __forceinline__ void issue(unsigned boff) const {
    if constexpr (K < WC) {
      if constexpr (WT) copy16io<K * kBlk, K * 1024>(w, vlin, lds_w + boff);
      else copy16i<K * kBlk>(w, vw[K], lds_w + boff);
    } else if constexpr (K < WC + NX) {
      constexpr int kx = K - WC;
      if constexpr (FMT == kFmtE3M2) copy16i<kx * 1024>(x, vx[kx], lds_x + boff);
      else if constexpr (FMT == kFmtE4M3)
        copy16i<kx * kBlk>(x, (vx[0] & ~15u) + min((unsigned)kx, vx[0] & 7u) * lda, lds_x + boff);
      else copy16i<kx * kBlk>(x, vx[kx], lds_x + boff);
    } else if constexpr (K == kCopySlots - 1) {
      copy4i<0>(s, vs, lds_s + boff);
    }
  }
};

template <bool WT>
struct LeanCopy<kFmtNone, WT> {
  __device__ __forceinline__ void init(const Plan&, int, const LaneOffsets&, const Ctx&) {}
  __device__ __forceinline__ void advance() {}
  static constexpr int count() { return 0; }
  template <int K>
  __device__ __forceinline__ void issue(unsigned) const {}
};

template <int K0, int K1, int FMT, bool WT>
__device__ __forceinline__ void issue_range(const LeanCopy<FMT, WT>& lc, unsigned boff) {
  if constexpr (K0 < K1) {
    lc.template issue<K0>(boff);
    issue_range<K0 + 1, K1>(lc, boff);
  }
}

// s_waitcnt vmcnt(n) for a run-time, wave-uniform n: the n most recent copies may stay in flight
__device__ __forceinline__ void wait_copies_but(int n) {
  switch (n) {
#define MG_VMCNT_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    MG_VMCNT_CASE(1) MG_VMCNT_CASE(2) MG_VMCNT_CASE(3) MG_VMCNT_CASE(4) MG_VMCNT_CASE(5) MG_VMCNT_CASE(6)
    MG_VMCNT_CASE(7) MG_VMCNT_CASE(8) MG_VMCNT_CASE(9) MG_VMCNT_CASE(10) MG_VMCNT_CASE(11) MG_VMCNT_CASE(12)
    MG_VMCNT_CASE(13) MG_VMCNT_CASE(14) MG_VMCNT_CASE(15) MG_VMCNT_CASE(16) MG_VMCNT_CASE(17) MG_VMCNT_CASE(18)
    MG_VMCNT_CASE(19) MG_VMCNT_CASE(20)
#undef MG_VMCNT_CASE
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}
template <int N>
__device__ __forceinline__ void wait_copies_but_imm() {
  static_assert(N >= 0 && N < 64, "vmcnt immediate");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// s_waitcnt lgkmcnt(0) as a compiler-visible instruction (vmcnt and expcnt fields at their maxima),
// so that the compiler's own wait insertion knows the LDS reads are done
__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }

// ---------------------------------------------------------------------------------------------
// Fragments
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ v8i widen(v4i v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1); }
__device__ __forceinline__ v8i widen(v6i v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3, 4, 5, -1, -1); }
__device__ __forceinline__ v8i widen(v8i v) { return v; }

// Fragments of one 64-wide K half of a stage: 4 feature tiles, 4 token tiles.
template <int FMT, int TM>
struct HalfFrags {
  v4i w[4];
  typename Fmt<FMT>::xfrag x[TM];
};

// Per-lane LDS addresses of a wave's fragments in stage buffer 0.
struct WeightPtrs {
  const uint8_t* w;    // weights: row 32*t + i at block i%16, quad 8*(i/16) + t; + t*64 + h*32
  const uint8_t* sw;   // scale dwords of the 4 feature tiles
  const uint8_t* sx;   // scale dwords of the wave's token tiles

  // the wave's token tiles lie in scale atom c.xatom of the workgroup's tile
  __device__ __forceinline__ WeightPtrs(const uint8_t* lds, const Ctx& c) {
    const int i = c.lane & 31, g = c.lane >> 5;
    w = lds + kWOff + (i & 15) * kBlk + (i >> 4) * 512 + c.wn * 256 + g * 16;
    sw = lds + kSOff + c.wn * 512 + i * 16;
    sx = lds + kSOff + 1024 + c.xatom * 512 + i * 16 + c.xtile * 4;
  }
};

template <int FMT, int TM>
struct TokenPtrs {
  const uint8_t* x;

  // the wave's token tiles are tiles TM * wm ... TM * wm + TM - 1 of the workgroup's
  __device__ __forceinline__ TokenPtrs(const uint8_t* lds, const Ctx& c) {
    const int i = c.lane & 31, g = c.lane >> 5;
    if constexpr (FMT == kFmtE3M2) {
      // row 32*rt + i: block i%8, row slot 4*rt + i/8, fragment 2h+g of 24 bytes
      x = lds + kXOff + (i & 7) * kBlk6 + (4 * TM * c.wm + (i >> 3)) * 96 + g * 24;
    } else {
      x = lds + kXOff + (i & 15) * kBlk + (i >> 4) * 512 + c.wm * (64 * TM) + g * 16;
    }
  }
};

// Reads of the fragments of K half H of one stage, one fragment per call so that they can be
// spread between MFMAs: R = 0..3 weight tile R, 4..7 token tile R-4, 8 / 9 the scale dwords of
// the feature / token tiles (only when SC).
template <int FMT, int H, bool SC, int TM>
struct FragReader {
  HalfFrags<FMT, TM>& f;
  v4i& sw;
  v4i& sx;
  const uint8_t* pw;
  const uint8_t* px;
  const uint8_t* psw;
  const uint8_t* psx;
  bool on;   // wave-uniform

  static constexpr int kReads = SC ? 6 + TM : 4 + TM;

  template <int R>
  __device__ __forceinline__ void read() const {
    if (!on) return;
    if constexpr (R < 4) {
      f.w[R] = *reinterpret_cast<const v4i*>(pw + R * 64 + H * 32);
    } else if constexpr (R < 4 + TM) {
      constexpr int t = R - 4;
      if constexpr (FMT == kFmtE2M1) {
        f.x[t] = *reinterpret_cast<const v4i*>(px + t * 64 + H * 32);
      } else if constexpr (FMT == kFmtE3M2) {
        const v2i* p = reinterpret_cast<const v2i*>(px + t * 384 + H * 48);
        const v2i a = p[0], b = p[1], c = p[2];
        f.x[t] = v6i{a[0], a[1], b[0], b[1], c[0], c[1]};
      } else {
        const uint8_t* p = px + H * 16 * kBlk + t * 64;
        const v4i a = *reinterpret_cast<const v4i*>(p);        // K [16g, 16g+16) of the half
        const v4i b = *reinterpret_cast<const v4i*>(p + 32);   // K [32+16g, 32+16g+16)
        f.x[t] = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    } else if constexpr (SC && R == 4 + TM) {
      sw = *reinterpret_cast<const v4i*>(psw);
    } else if constexpr (SC && R == 5 + TM) {
      // the dwords of the wave's own token tiles only (TM consecutive ones of the atom's four)
      if constexpr (TM == 2) {
        const v2i t = *reinterpret_cast<const v2i*>(psx);
        sx[0] = t[0];
        sx[1] = t[1];
      } else {
        sx[0] = *reinterpret_cast<const int*>(psx);
      }
    }
  }
};

template <int R = 0, int FMT, int H, bool SC, int TM>
__device__ __forceinline__ void read_all(const FragReader<FMT, H, SC, TM>& rd) {
  if constexpr (R < FragReader<FMT, H, SC, TM>::kReads) {
    rd.template read<R>();
    read_all<R + 1>(rd);
  }
}

// reads [R0, R1) of a half's fragments, as far as there are that many
template <int R0, int R1, class Reader>
__device__ __forceinline__ void read_some(const Reader& rd) {
  if constexpr (R0 < R1 && R0 < Reader::kReads) {
    rd.template read<R0>();
    read_some<R0 + 1, R1>(rd);
  }
}

template <int TM>
struct Scales {
  int w[4], x[TM];   // scale dwords of the 4 feature / TM token tiles, shifted so that byte 0 / 2 is block g / 2+g
};

// sw holds the scale dwords of the four feature tiles, sx[0 .. TM - 1] those of the wave's token tiles
template <int TM>
__device__ __forceinline__ void shift_scales(Scales<TM>& sc, v4i sw, v4i sx, int lane) {
  const int g8 = (lane >> 5) * 8;
#pragma unroll
  for (int t = 0; t < 4; ++t) sc.w[t] = (int)((unsigned)sw[t] >> g8);
#pragma unroll
  for (int t = 0; t < TM; ++t) sc.x[t] = (int)((unsigned)sx[t] >> g8);
}

// ---------------------------------------------------------------------------------------------
// One K stage
// ---------------------------------------------------------------------------------------------
template <int FMT, int H>
__device__ __forceinline__ void mfma_one(v16f& acc, v4i w, const typename Fmt<FMT>::xfrag& x, int scw, int scx) {
  acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(widen(w), widen(x), acc, kFmtE2M1, FMT, 2 * H, scw, 2 * H, scx);
}

// first copy slot >= K that a stage of format FMT has (the token slots past the format's copies are empty)
template <int FMT>
constexpr int next_slot(int k) {
  return (k >= kWCopies + Fmt<FMT>::x_copies / 2 && k < kCopySlots - 1) ? kCopySlots - 1 : k;
}

// The 4 * TM MFMAs of one K half.  Between them: the fragment reads of `rd` (for the next half: one after
// each of the first MFMAs -- two where a half has fewer MFMAs than reads --, so that the waves do not all
// queue at the LDS at once with their MFMAs stuck behind) and the copy slots [K0, K1) of one stage, one after
// every second MFMA of 8, after every one of 4.
// LEAN: slots of `lc` (a stage of format CF, skipped when !on) into the buffer at byte offset boff;
// otherwise slots of the run-time plan `gc`.
template <int FMT, int H, bool LEAN, int CF, int M0, int K0, int K1, class Reader, bool WT, int TM>
__device__ __forceinline__ void mfma_half(v16f (&acc)[4][TM], const HalfFrags<FMT, TM>& f, const Scales<TM>& sc, const Reader& rd,
                                          const LeanCopy<CF, WT>& lc, bool on, unsigned boff, const GenericCopy& gc,
                                          const LaneOffsets& lo, int wave) {
  if constexpr (M0 < 4 * TM) {
    constexpr int tn = M0 / TM, tm = M0 % TM;
    mfma_one<FMT, H>(acc[tn][tm], f.w[tn], f.x[tm], sc.w[tn], sc.x[tm]);
    // The fragment reads go out after the first MFMAs, as few per MFMA as leaves the last two MFMAs of the half
    // without one: what is read last is needed first afterwards, and its LDS latency would stand between two halves.
    constexpr int RP = (Reader::kReads + 4 * TM - 3) / (4 * TM - 2);
    read_some<M0 * RP, (M0 + 1) * RP>(rd);
    constexpr int KS = LEAN ? (CF == kFmtNone ? K1 : next_slot<CF>(K0)) : K0;
    // a copy slot after every second MFMA where a wave has twice as many MFMAs per half as copy slots, else after every one
    constexpr bool kEvery = 4 * TM <= kCopySlots - kSplit;
    if constexpr ((kEvery || (M0 & 1) == 1) && KS < K1) {
      if constexpr (LEAN) {
        if (on) lc.template issue<KS>(boff);
      } else {
        gc.template issue<KS>(lo, wave);
      }
      __builtin_amdgcn_sched_barrier(0);
      mfma_half<FMT, H, LEAN, CF, M0 + 1, KS + 1, K1>(acc, f, sc, rd, lc, on, boff, gc, lo, wave);
    } else {
      __builtin_amdgcn_sched_barrier(0);
      mfma_half<FMT, H, LEAN, CF, M0 + 1, K0, K1>(acc, f, sc, rd, lc, on, boff, gc, lo, wave);
    }
  }
}

// The three stage buffers as byte offsets, rotated once per stage (wave-uniform).
struct Ring {
  unsigned cur, nxt, lst;   // buffers of stage q, q+1, q+2
  __device__ __forceinline__ explicit Ring(int q) {
    cur = (q % kBuffers) * kStage;
    nxt = ((q + 1) % kBuffers) * kStage;
    lst = ((q + 2) % kBuffers) * kStage;
  }
  __device__ __forceinline__ void rotate() {
    const unsigned t = cur;
    cur = nxt;
    nxt = lst;
    lst = t;
  }
};

// Stage q of format FMT; FR = format of stage q+1, whose first half is prefetched into `a`
// (FR == FMT) or `a_next`.  `xp` / `xpn`: token fragment addresses for FMT / FR.
// LEAN: the late copy slots (of stage q+2, format CL) come from `lcl` when late_on, the early ones
// (of stage q+3, format CE) from `lce` when early_on; MID says what happens to `lce` between the
// halves: 1 = advance by one stage, 2 = nothing (stage q+3 is the first of its segment, where lce stands).
// !LEAN: both from the run-time plan `gc`.  next_on: there is a stage q+1.
template <int FMT, int FR, bool LEAN, int CL, int CE, int MID, bool WT, int TM>
__device__ __forceinline__ void stage_body(v16f (&acc)[4][TM], HalfFrags<FMT, TM>& a, HalfFrags<FR, TM>& a_next, Scales<TM>& sc,
                                           const LeanCopy<CL, WT>& lcl, bool late_on, LeanCopy<CE, WT>& lce, bool early_on,
                                           GenericCopy& gc, const LaneOffsets& lo, const Plan& plan, int q,
                                           bool next_on, const Ring& ring, const WeightPtrs& wp, const TokenPtrs<FMT, TM>& xp,
                                           const TokenPtrs<FR, TM>& xpn, const Ctx& c) {
  HalfFrags<FMT, TM> b;
  HalfFrags<FR, TM> nx;
  v4i sw = {0, 0, 0, 0}, sx = {0, 0, 0, 0};
  wait_lds_reads();   // nothing is outstanding here; tells the compiler so (it cannot see it across the loop edge)
  // first half; reads the second half's fragments; the remaining copies of stage q+2 go to the last buffer
  const FragReader<FMT, 1, false, TM> rd_b{b, sw, sx, wp.w + ring.cur, xp.x + ring.cur, nullptr, nullptr, true};
  mfma_half<FMT, 0, LEAN, CL, 0, kSplit, kCopySlots>(acc, a, sc, rd_b, lcl, late_on, ring.lst, gc, lo, c.wave);
  __builtin_amdgcn_sched_barrier(0);
  wait_lds_reads();
  if constexpr (LEAN) {
    if (late_on) wait_copies_but_imm<LeanCopy<CL, WT>::count()>();
    else wait_copies_but_imm<0>();
  } else {
    wait_copies_but(gc.count());
  }
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (LEAN) {
    if constexpr (MID == 1) lce.advance();   // MID == 2: lce was set up for its segment's first stage before the K loop
  } else {
    gc = GenericCopy(plan, q + 3, c);
  }
  // second half; reads the first half and the scales of stage q+1; the first copies of stage q+3
  // go to the buffer this stage just released
  const FragReader<FR, 0, true, TM> rd_n{nx, sw, sx, wp.w + ring.nxt, xpn.x + ring.nxt, wp.sw + ring.nxt, wp.sx + ring.nxt,
                                     next_on};
  mfma_half<FMT, 1, LEAN, CE, 0, 0, kSplit>(acc, b, sc, rd_n, lce, early_on, ring.cur, gc, lo, c.wave);
  __builtin_amdgcn_sched_barrier(0);
  wait_lds_reads();
  shift_scales(sc, sw, sx, c.lane);
  if constexpr (FR == FMT) a = nx;
  else a_next = nx;
}

// Runs the n >= 1 stages [q0, q0 + n) of one segment whose format is FMT; the next segment has
// format F1 (kFmtNone after the last one) and n1 stages; FR1 = F1, or FMT after the last segment.
// NLAST (REGULAR kernels): how many stages the plan's last segment has -- 1, 2, or 3 for three or
// more; 0 = not known at compile time (plans of one segment) or, for a segment before the last
// but one, not needed.  It makes "does the stage that would be copied exist" a compile-time
// constant in every stage body: a run-time switch around each copy costs a branch per copy, at
// every branch the wait for the fragment reads just issued, and registers (the kernels spilled).
// On entry `a` holds the first K half of stage q0 and `sc` its scales; on exit `a_next` holds the
// first half of stage q0 + n when there is one.
// REGULAR (every segment but the last has at least 3 stages): `lc` describes the copies of local
// stage 2 on entry; the last three stages copy the first three of the next segment through
// `lcn`, which the next segment then continues to use as its `lc`.
// !REGULAR: `gc` describes stage q0 + 2 (whose first copies are out) on entry and exit; the
// stages that copy across a segment boundary take the run-time path.
template <int FMT, int F1, int FR1, bool REGULAR, int NLAST = 0, bool WT, int TM>
__device__ __forceinline__ void run_segment(v16f (&acc)[4][TM], HalfFrags<FMT, TM>& a, Scales<TM>& sc, HalfFrags<FR1, TM>& a_next,
                                            LeanCopy<FMT, WT>& lc, LeanCopy<F1, WT>& lcn, GenericCopy& gc, const LaneOffsets& lo,
                                            const Plan& plan, int n, int n1, int q0, const WeightPtrs& wp,
                                            const uint8_t* lds, const Ctx& c) {
  const TokenPtrs<FMT, TM> xp(lds, c);
  const TokenPtrs<FR1, TM> xpn(lds, c);
  Ring ring(q0);
  int ql = 0;
  HalfFrags<FMT, TM> unused;
  if constexpr (REGULAR && F1 != kFmtNone) {
    for (; ql + 3 < n; ++ql) {
      stage_body<FMT, FMT, true, FMT, FMT, 1>(acc, a, unused, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                              xp, c);
      ring.rotate();
    }
    // the last three stages copy stages 0, 1, 2 of the next segment; only the plan's last segment can have
    // fewer than three (NLAST = 1, 2)
    constexpr bool s1 = NLAST != 1, s2 = NLAST != 1 && NLAST != 2;
    stage_body<FMT, FMT, true, FMT, F1, 2>(acc, a, unused, sc, lc, true, lcn, true, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                           xp, c);
    ring.rotate();
    ++ql;
    stage_body<FMT, FMT, true, F1, F1, 1>(acc, a, unused, sc, lcn, true, lcn, s1, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                          xp, c);
    ring.rotate();
    ++ql;
    stage_body<FMT, FR1, true, F1, F1, 1>(acc, a, a_next, sc, lcn, s1, lcn, s2, gc, lo, plan, q0 + ql, true, ring, wp, xp, xpn,
                                          c);
  } else if constexpr (REGULAR) {
    // last segment: its own stages only, any n >= 1; first the stages whose copies all exist (no run-time
    // switches in the body), then the last three
    for (; ql + 3 < n; ++ql) {
      stage_body<FMT, FMT, true, FMT, FMT, 1>(acc, a, unused, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                              xp, c);
      ring.rotate();
    }
    if ((NLAST == 0 && n >= 3) || NLAST >= 3) {   // third from last: the last stage's remaining copies
      stage_body<FMT, FMT, true, FMT, FMT, 1>(acc, a, unused, sc, lc, true, lc, false, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                              xp, c);
      ring.rotate();
      ++ql;
    }
    if ((NLAST == 0 && n >= 2) || NLAST >= 2) {   // second from last: nothing left to copy
      stage_body<FMT, FMT, true, FMT, FMT, 1>(acc, a, unused, sc, lc, false, lc, false, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                              xp, c);
      ring.rotate();
      ++ql;
    }
    stage_body<FMT, FMT, true, kFmtNone, kFmtNone, 0>(acc, a, unused, sc, lcn, false, lcn, false, gc, lo, plan, q0 + ql,
                                                      false, ring, wp, xp, xp, c);
  } else {
    if (n > 3) {
      // stages whose stage-after-next-but-one is still in this segment
      lc.init(plan, q0 + 2, lo, c);
      for (; ql + 3 < n; ++ql) {
        stage_body<FMT, FMT, true, FMT, FMT, 1>(acc, a, unused, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, true, ring, wp,
                                                xp, xp, c);
        ring.rotate();
      }
      gc = GenericCopy(plan, q0 + ql + 2, c);
    }
    for (; ql + 1 < n; ++ql) {
      stage_body<FMT, FMT, false, FMT, FMT, 0>(acc, a, unused, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                               xp, c);
      ring.rotate();
    }
    if constexpr (FR1 == FMT) {
      stage_body<FMT, FMT, false, FMT, FMT, 0>(acc, a, unused, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, false, ring, wp, xp,
                                               xp, c);
    } else {
      stage_body<FMT, FR1, false, FMT, FMT, 0>(acc, a, a_next, sc, lc, true, lc, true, gc, lo, plan, q0 + ql, true, ring, wp, xp,
                                               xpn, c);
    }
  }
}


// The 0..3 blocks of 32 elements a segment has beyond its whole 128-wide stages (e.g. 4928 = 38 * 128
// + 64): straight from global memory, by up to two more MFMA steps per segment (K half h = blocks 2h and
// 2h + 1), ahead of the pipelined stages.  A half is loaded whole (block index clamped into the segment) and
// the blocks it does not have are turned into zero codes with scale 2^0 before the MFMAs; a half without any
// block is skipped by a wave-uniform branch.  Loading and computing are separate steps: the kernel requests the
// first halves of all three segments before its first stage copies, so that these loads -- 16 bytes per lane from
// rows far apart, each the first touch of its cache line -- are in flight together and with the copies, and
// computes them while stages 1 and 2 are still landing.  (After the K loop, one half after the other, they cost
// 4 to 9 % of the kernel: every load was waited for with nothing else to do; and branches there, around code
// that touches the live accumulator, make the register allocator spill it.  Here the accumulator is still zero.)
template <int FMT, int TM>
struct RemainderHalf {
  v4i w[4];
  typename Fmt<FMT>::xfrag x[TM];
  int sw[4], sx[TM];
};

template <int FMT, int TM>
__device__ __forceinline__ void remainder_load(RemainderHalf<FMT, TM>& f, int h, const uint8_t* __restrict__ a,
                                               const uint8_t* __restrict__ b, const uint8_t* __restrict__ sfa,
                                               const uint8_t* __restrict__ sfb, int blk, bool w_tiled, int tiles_n,
                                               const Ctx& c) {
  const int r = blk & 3, q = blk >> 2;
  // weights: row-major rows of blk blocks, or (tile-major) the r blocks past the whole stages as rows of
  // r blocks behind the tiled part; with r == 0 nothing is used and any valid address will do
  const uint8_t* wbase = w_tiled ? (r ? b + (size_t)tiles_n * q * 16384 : b) : b;
  const unsigned wpitch = w_tiled ? (unsigned)r * 16 : (unsigned)blk * 16;
  const int wfirst = w_tiled ? 4 * q : 0;   // block index of the first block of a row
  constexpr int XB = Fmt<FMT>::row_bytes / 4;   // token bytes per block
  const int i = c.lane & 31, g = c.lane >> 5;
  const int katoms = (blk + 3) >> 2;
  const unsigned lda = (unsigned)blk * XB;
  const int kb = 2 * h + g;
  const int kbc = min(4 * q + kb, blk - 1);           // a block that exists
  const int kb1 = min(4 * q + 2 * h + 1, blk - 1);    // E4M3: the second block of the half
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const unsigned n = c.n0 + min(c.wn * 128 + t * 32 + i, c.cols_avail - 1);   // features past the last one are never stored
    f.w[t] = *reinterpret_cast<const v4i*>(wbase + (size_t)n * wpitch + (size_t)max(kbc - wfirst, 0) * 16);
    f.sw[t] = sfb[sf_offset(n, kbc, katoms)];
  }
#pragma unroll
  for (int t = 0; t < TM; ++t) {
    const unsigned m = c.m0 + min(c.wm * (32 * TM) + t * 32 + i, c.rows_avail - 1);   // rows past the last readable one are never stored
    f.sx[t] = sfa[sf_offset(m, kbc, katoms)];
    const uint8_t* xr = a + (size_t)m * lda;
    if constexpr (FMT == kFmtE2M1) {
      f.x[t] = *reinterpret_cast<const v4i*>(xr + (size_t)kbc * 16);
    } else if constexpr (FMT == kFmtE3M2) {
      const v2i* p = reinterpret_cast<const v2i*>(xr + (size_t)kbc * 24);
      const v2i p0 = p[0], p1 = p[1], p2 = p[2];
      f.x[t] = v6i{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1]};
    } else {
      // K [16g, 16g+16) of the half lies in block 2h, K [32+16g, ...) in block 2h+1
      const int kb0 = min(4 * q + 2 * h, blk - 1);
      const v4i pa = *reinterpret_cast<const v4i*>(xr + (size_t)kb0 * 32 + g * 16);
      const v4i pb = *reinterpret_cast<const v4i*>(xr + (size_t)kb1 * 32 + g * 16);
      f.x[t] = __builtin_shufflevector(pa, pb, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }
}

template <int FMT, int TM>
__device__ __forceinline__ void remainder_mfma(v16f (&acc)[4][TM], RemainderHalf<FMT, TM>& f, int h, int blk, const Ctx& c) {
  const int r = blk & 3;
  const int g = c.lane >> 5;
  const bool ok = 2 * h + g < r;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int e = 0; e < 4; ++e) f.w[t][e] = ok ? f.w[t][e] : 0;
    f.sw[t] = ok ? f.sw[t] : 127;
  }
#pragma unroll
  for (int t = 0; t < TM; ++t) {
    f.sx[t] = ok ? f.sx[t] : 127;
    if constexpr (FMT == kFmtE4M3) {
      const bool oka = 2 * h < r, okb = 2 * h + 1 < r;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f.x[t][e] = oka ? f.x[t][e] : 0;
        f.x[t][4 + e] = okb ? f.x[t][4 + e] : 0;
      }
    } else {
      constexpr int NE = FMT == kFmtE2M1 ? 4 : 6;
#pragma unroll
      for (int e = 0; e < NE; ++e) f.x[t][e] = ok ? f.x[t][e] : 0;
    }
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int tn = 0; tn < 4; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) mfma_one<FMT, 0>(acc[tn][tm], f.w[tn], f.x[tm], f.sw[tn], f.sx[tm]);
  __builtin_amdgcn_sched_barrier(0);
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give each XCD a contiguous band of
// feature tiles and walk it feature tile by feature tile inside groups of at most 8 feature tiles, token tile
// after token tile: the ~32 tiles an XCD works on at a time are then about as many feature tiles as token tiles
// (7 x 4.6 for 56 x 16 tiles), which is what keeps the bytes that pass its L2 lowest.
// A launch of at most one tile per CU (cus > 0 says so: all its tiles run at once) gives each XCD a rectangle of
// bn x bm tiles instead, the one of the 8 / 4 / 2 / 1 column splits that needs the fewest operand bytes per stage
// (a weight tile is 16 KB per stage, a token tile of `tokens` rows about 80 bytes per row): M = 2048, N = 4096 as
// 256 tiles of 256 x 128 fetches 140 MB past the L2s as 4 x 8 rectangles, 186 MB as 2 x 16 bands.
// Returns whether the banded walk applies (tile counts that divide accordingly).
__device__ __forceinline__ bool tile_of(int wg, int nwg, int tiles_n, int& tile_n, int& tile_m, int cus = 0, int tokens = kT) {
  const int tiles_m = nwg / tiles_n;
  tile_n = wg / tiles_m;
  tile_m = wg % tiles_m;
  bool banded = false;
  if ((nwg & 7) == 0 && nwg <= cus) {
    // (a rectangle must beat what the walk below gives an XCD: its tiles in feature-major order, i.e. all token tiles of
    // one or two feature tiles, and of a third where the XCDs' shares do not end with a column)
    const int share = nwg >> 3;
    int best = 0, best_cost = ((share + tiles_m - 1) / tiles_m + (share % tiles_m != 0 ? 1 : 0)) * 16384 +
                              min(tiles_m, share) * tokens * 80;
#pragma unroll
    for (int gx = 8; gx >= 1; gx >>= 1) {
      const int gy = 8 / gx;
      if (tiles_n % gx == 0 && tiles_m % gy == 0) {
        const int cost = (tiles_n / gx) * 16384 + (tiles_m / gy) * tokens * 80;
        if (cost < best_cost) {
          best_cost = cost;
          best = gx;
        }
      }
    }
    if (best > 0) {
      const int xcd = wg & 7, j = wg >> 3, bn = tiles_n / best, bm = tiles_m / (8 / best);
      tile_n = (xcd % best) * bn + j % bn;
      tile_m = (xcd / best) * bm + j / bn;
      return false;
    }
  }
  if ((nwg & 7) == 0) {
    const int per_xcd = nwg >> 3;
    const int j = wg >> 3;                       // position in this XCD's list
    const int tile = (wg & 7) * per_xcd + j;     // feature-major tile index
    tile_n = tile / tiles_m;
    tile_m = tile % tiles_m;
    if (per_xcd % tiles_m == 0) {
      const int cols = per_xcd / tiles_m;        // feature tiles of the band
      const int groups = (cols + 7) / 8;
      if (cols % groups == 0) {
        const int gw = cols / groups, per_group = gw * tiles_m;
        const int g = j / per_group, r = j % per_group;
        tile_n = (wg & 7) * cols + g * gw + r % gw;
        tile_m = r / gw;
        banded = true;
      }
    }
  }
  return banded;
}

// What a workgroup does before its tile: the staggered start and the plan into scalar registers.
// Staggered start: with several tiles per CU, the first workgroup of each CU (the first `first_round` of the
// grid) starts up to `skew` clock ticks late, each by a different amount.  Every tile takes the same time, so
// without this all CUs load their first stages and store their result tiles in the same microseconds, tile after
// tile, and queue at the memory; the few microseconds lost once come back several times over.
template <bool WT>
__device__ __forceinline__ Plan start_workgroup(const Plan& plan_arg, int first_round, int skew) {
  if (skew > 0 && (int)blockIdx.x < first_round) {
    const long long delay = (long long)skew * (((int)blockIdx.x >> 3) * 8 + ((int)blockIdx.x & 7)) / first_round;
    const long long t0 = __builtin_amdgcn_s_memtime();
    while ((long long)__builtin_amdgcn_s_memtime() - t0 < delay) __builtin_amdgcn_s_sleep(4);
  }
  Plan plan;
  plan.a0 = uni(plan_arg.a0); plan.a1 = uni(plan_arg.a1); plan.a2 = uni(plan_arg.a2);
  plan.b0 = uni(plan_arg.b0); plan.b1 = uni(plan_arg.b1); plan.b2 = uni(plan_arg.b2);
  plan.sfa0 = uni(plan_arg.sfa0); plan.sfa1 = uni(plan_arg.sfa1); plan.sfa2 = uni(plan_arg.sfa2);
  plan.sfb0 = uni(plan_arg.sfb0); plan.sfb1 = uni(plan_arg.sfb1); plan.sfb2 = uni(plan_arg.sfb2);
  plan.st0 = __builtin_amdgcn_readfirstlane(plan_arg.st0);
  plan.st1 = __builtin_amdgcn_readfirstlane(plan_arg.st1);
  plan.st2 = __builtin_amdgcn_readfirstlane(plan_arg.st2);
  plan.blk0 = __builtin_amdgcn_readfirstlane(plan_arg.blk0);
  plan.blk1 = __builtin_amdgcn_readfirstlane(plan_arg.blk1);
  plan.blk2 = __builtin_amdgcn_readfirstlane(plan_arg.blk2);
  plan.total = __builtin_amdgcn_readfirstlane(plan_arg.total);
  plan.w_tiled = WT ? 1 : 0;
  return plan;
}

// Format of the k-th segment that exists in a plan (segs: bit 0 E2M1, bit 1 E3M2, bit 2 E4M3), kFmtNone past the last.
constexpr int nth_format(int segs, int k) {
  constexpr int fmts[3] = {kFmtE2M1, kFmtE3M2, kFmtE4M3};
  for (int sg = 0; sg < 3; ++sg)
    if (segs & (1 << sg)) {
      if (k == 0) return fmts[sg];
      --k;
    }
  return kFmtNone;
}
template <int FMT>
__device__ __forceinline__ int stages_of(const Plan& p) {
  return FMT == kFmtE2M1 ? p.st0 : (FMT == kFmtE3M2 ? p.st1 : (FMT == kFmtE4M3 ? p.st2 : 0));
}

// REGULAR: see run_segment.  REM: some segment is not a multiple of 128 wide.  WT: tile-major weights.
// SEGS: which activation segments the plan has, bit 0 E2M1, bit 1 E3M2, bit 2 E4M3 -- the
// prefetched fragments pass from a segment to the next one that exists, and their types are fixed here.
// TM: token tiles of 32 per wave.  2: the workgroup's tile is 256 features x 256 tokens.  1: 256 x 128, for
// problems with fewer than 256 whole tiles (every CU still gets a workgroup): same copies (the lanes of token
// rows 128 ... 255 read the last row again, which costs the address unit next to nothing), same LDS image,
// half the MFMAs per stage, a copy slot after every MFMA instead of every second one.
// NLAST: see run_segment (the launcher picks the instance from the plan).
// Computes one tile of 256 features x 128 * TM tokens: feature tile tile_n, token tile tile_m (of 128 * TM rows).
template <bool REGULAR, bool REM, bool WT, int SEGS, int TM, int NLAST>
__device__ __forceinline__ void compute_tile(const Plan& plan, int tile_n, int tile_m, int tiles_n, int N, int m_store,
                                             int a_rows, uint16_t* __restrict__ d, uint8_t* lds) {
  static_assert(TM == 2 || TM == 1, "wave tiles of 128 features x 32 * TM tokens");
  const int tid = threadIdx.x;
  Ctx c;
  c.lane = tid & 63;
  c.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  c.wn = c.wave & 1;
  c.wm = c.wave >> 1;
  c.xatom = (c.wm * TM) >> 2;
  c.xtile = (c.wm * TM) & 3;
  constexpr int kTokens = 16 * kWaves * TM;   // token rows of the workgroup's tile
  c.n0 = tile_n * kT;
  c.m0 = tile_m * kTokens;
  c.total = plan.total;
  c.rows_avail = min(a_rows - c.m0, kTokens);
  c.cols_avail = min(N - c.n0, kT);
  c.lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t*)lds;

  const LaneOffsets lo(plan, c);
  const WeightPtrs wp(lds, c);

  // the blocks past the whole stages first (see RemainderHalf): first K halves requested ahead of the copies
  RemainderHalf<kFmtE2M1, TM> p0;
  RemainderHalf<kFmtE3M2, TM> s0;
  RemainderHalf<kFmtE4M3, TM> o0;
  if constexpr (REM) {
    if ((plan.blk0 & 3) > 0) remainder_load<kFmtE2M1>(p0, 0, plan.a0, plan.b0, plan.sfa0, plan.sfb0, plan.blk0, WT, tiles_n, c);
    if ((plan.blk1 & 3) > 0) remainder_load<kFmtE3M2>(s0, 0, plan.a1, plan.b1, plan.sfa1, plan.sfb1, plan.blk1, WT, tiles_n, c);
    if ((plan.blk2 & 3) > 0) remainder_load<kFmtE4M3>(o0, 0, plan.a2, plan.b2, plan.sfa2, plan.sfb2, plan.blk2, WT, tiles_n, c);
    __builtin_amdgcn_sched_barrier(0);
  }
  // prologue: stages 0 and 1 and the first copies of stage 2 in flight; wait for stage 0 only.  The copies go out
  // before anything else that can wait (the accumulators are cleared while they are in flight); in REGULAR kernels
  // the first three stages belong to the plan's first segment, or do not exist, and take the compile-time form of the copies.
  constexpr int FA = nth_format(SEGS, 0), FB = nth_format(SEGS, 1), FC = nth_format(SEGS, 2);   // the segments that exist, in order
  static_assert(FA != kFmtNone, "a plan has at least one segment");
  const int nA = stages_of<FA>(plan), nB = stages_of<FB>(plan), nC = stages_of<FC>(plan);
  GenericCopy gc;
  LeanCopy<FA, WT> la;
  int in_flight;   // copies that may stay in flight while stage 0 is awaited
  if constexpr (REGULAR) {
    la.init(plan, 0, lo, c);
    issue_range<0, kCopySlots>(la, 0);
    in_flight = 0;
    if (plan.total > 1) {
      la.advance();
      issue_range<0, kCopySlots>(la, kStage);
      in_flight = la.count();
    }
    if (plan.total > 2) {
      la.advance();   // stays on stage 2: where the segment loop expects it
      issue_range<0, kSplit>(la, 2 * kStage);
      in_flight += kSplit;
    }
  } else {
    const GenericCopy g0(plan, 0, c);
    issue_range<0, kCopySlots>(g0, lo, c.wave);
    const GenericCopy g1(plan, 1, c);
    issue_range<0, kCopySlots>(g1, lo, c.wave);
    gc = GenericCopy(plan, 2, c);
    issue_range<0, kSplit>(gc, lo, c.wave);
    in_flight = g1.count() + (gc.b.seg < 0 ? 0 : kSplit);
  }
  // the copy state of the later segments, while the first copies are in flight: set up between two halves of a
  // stage it would hold up the MFMAs for several hundred cycles
  LeanCopy<FB, WT> lb;
  LeanCopy<FC, WT> lcc;
  if constexpr (REGULAR) {
    lb.init(plan, nA, lo, c);          // (no-ops for segments that do not exist)
    lcc.init(plan, nA + nB, lo, c);
  }
  __builtin_amdgcn_sched_barrier(0);

  v16f acc[4][TM];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;
  __builtin_amdgcn_sched_barrier(0);

  if constexpr (REM) {
    if ((plan.blk0 & 3) > 0) remainder_mfma<kFmtE2M1>(acc, p0, 0, plan.blk0, c);
    if ((plan.blk1 & 3) > 0) remainder_mfma<kFmtE3M2>(acc, s0, 0, plan.blk1, c);
    if ((plan.blk2 & 3) > 0) remainder_mfma<kFmtE4M3>(acc, o0, 0, plan.blk2, c);
    // second K halves: segments with three blocks past their whole stages
    RemainderHalf<kFmtE2M1, TM> p1;
    RemainderHalf<kFmtE3M2, TM> s1;
    RemainderHalf<kFmtE4M3, TM> o1;
    if ((plan.blk0 & 3) > 2) remainder_load<kFmtE2M1>(p1, 1, plan.a0, plan.b0, plan.sfa0, plan.sfb0, plan.blk0, WT, tiles_n, c);
    if ((plan.blk1 & 3) > 2) remainder_load<kFmtE3M2>(s1, 1, plan.a1, plan.b1, plan.sfa1, plan.sfb1, plan.blk1, WT, tiles_n, c);
    if ((plan.blk2 & 3) > 2) remainder_load<kFmtE4M3>(o1, 1, plan.a2, plan.b2, plan.sfa2, plan.sfb2, plan.blk2, WT, tiles_n, c);
    __builtin_amdgcn_sched_barrier(0);
    if ((plan.blk0 & 3) > 2) remainder_mfma<kFmtE2M1>(acc, p1, 1, plan.blk0, c);
    if ((plan.blk1 & 3) > 2) remainder_mfma<kFmtE3M2>(acc, s1, 1, plan.blk1, c);
    if ((plan.blk2 & 3) > 2) remainder_mfma<kFmtE4M3>(acc, o1, 1, plan.blk2, c);
    __builtin_amdgcn_sched_barrier(0);
  }

  wait_copies_but(in_flight);
  asm volatile("s_barrier" ::: "memory");

  static_assert(SEGS >= 1 && SEGS <= 7 && (SEGS == 7 || !REM), "plans with an empty segment: whole stages only");
  HalfFrags<FA, TM> fa, da;   // d*: never-read targets of the prefetch past a plan's last stage
  HalfFrags<FB, TM> fb, db;
  HalfFrags<FC, TM> fc, dc;
  Scales<TM> sc;
  {
    const TokenPtrs<FA, TM> xp(lds, c);
    v4i sw, sx;
    const FragReader<FA, 0, true, TM> rd{fa, sw, sx, wp.w, xp.x, wp.sw, wp.sx, true};
    read_all(rd);
    wait_lds_reads();
    shift_scales(sc, sw, sx, c.lane);
  }
  LeanCopy<kFmtNone, WT> l0;
  // NLAST goes to the plan's last segment and the one before it (see run_segment)
  if constexpr (FB == kFmtNone) {
    run_segment<FA, kFmtNone, FA, REGULAR>(acc, fa, sc, da, la, l0, gc, lo, plan, nA, 0, 0, wp, lds, c);
  } else if constexpr (FC == kFmtNone) {
    run_segment<FA, FB, FB, REGULAR, NLAST>(acc, fa, sc, fb, la, lb, gc, lo, plan, nA, nB, 0, wp, lds, c);
    run_segment<FB, kFmtNone, FB, REGULAR, NLAST>(acc, fb, sc, db, lb, l0, gc, lo, plan, nB, 0, nA, wp, lds, c);
  } else {
    run_segment<FA, FB, FB, REGULAR>(acc, fa, sc, fb, la, lb, gc, lo, plan, nA, nB, 0, wp, lds, c);
    run_segment<FB, FC, FC, REGULAR, NLAST>(acc, fb, sc, fc, lb, lcc, gc, lo, plan, nB, nC, nA, wp, lds, c);
    run_segment<FC, kFmtNone, FC, REGULAR, NLAST>(acc, fc, sc, dc, lcc, l0, gc, lo, plan, nC, 0, nA + nB, wp, lds, c);
  }

  // Result tile is D^T: lane holds token m = lane % 32, features 8*(v/4) + 4*(lane/32) + v%4.
  // Each wave transposes its 128 tokens x 128 features through its own part of the (now idle)
  // LDS, so that a store instruction writes 4 rows x 256 contiguous bytes instead of 32 rows x 16.
  // No barrier: the last stage reads no fragments after its barrier, before which every wave's copies had landed,
  // and from here on a wave touches only its own part of the LDS.
  constexpr int kPitch = 256 + 16;   // bytes per token row in LDS
  static_assert(kWaves * 32 * TM * kPitch <= kBuffers * kStage, "epilogue staging must fit the stage buffers");
  uint8_t* stage = lds + c.wave * (32 * TM) * kPitch;
  {
    const int g = c.lane >> 5;
    uint8_t* wr = stage + (c.lane & 31) * kPitch + 8 * g;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const v2bf lo2 = {(__bf16)acc[tn][tm][4 * vq + 0], (__bf16)acc[tn][tm][4 * vq + 1]};
          const v2bf hi2 = {(__bf16)acc[tn][tm][4 * vq + 2], (__bf16)acc[tn][tm][4 * vq + 3]};
          *reinterpret_cast<v2u*>(wr + tm * 32 * kPitch + tn * 64 + vq * 16) =
              v2u{__builtin_bit_cast(unsigned, lo2), __builtin_bit_cast(unsigned, hi2)};
        }
  }
  {
    const int r = c.lane >> 4, cc = c.lane & 15;
    const uint8_t* rd = stage + r * kPitch + cc * 16;
    uint16_t* out = d + (size_t)(c.m0 + c.wm * (32 * TM) + r) * N + c.n0 + c.wn * 128 + cc * 8;
    // token rows at or past m_store are not written, nor the 8-feature pieces past the layer's last feature
    const int rows_left = (c.wn * 128 + cc * 8 < c.cols_avail) ? m_store - (c.m0 + c.wm * (32 * TM) + r) : 0;
    // Eight reads in flight, then their eight stores: a read that is waited for before its own store costs a
    // full LDS latency per row (which is what the compiler makes of the predicated form: it sinks each read
    // into its store's block -- hence the separate path for tiles that are stored whole).  Streaming stores: the result is not read again here, and the XCD's L2 is
    // better spent on the operands.
    auto write_rows = [&](auto whole) {
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        v4u v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const v4u*>(rd + (b * 8 + j) * 4 * kPitch);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = b * 8 + j;
          if (decltype(whole)::value || i * 4 < rows_left)
            __builtin_nontemporal_store(v[j], reinterpret_cast<v4u*>(out + (size_t)i * 4 * N));
        }
      }
    };
    if (m_store - c.m0 >= kTokens && c.cols_avail == kT) write_rows(std::true_type{});   // wave-uniform: the whole tile is stored
    else write_rows(std::false_type{});
  }
}


template <bool REGULAR, bool REM, bool WT, int SEGS = 7, int TM = 2, int NLAST = 0>
__global__ void __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
mixed_gemm_256_kernel(Plan plan_arg, int tiles_n, int N, int m_store, int a_rows, uint16_t* __restrict__ d, int first_round,
                      int skew) {
  extern __shared__ __align__(16) uint8_t lds[];
  const Plan plan = start_workgroup<WT>(plan_arg, first_round, skew);
  int tile_n, tile_m;
  tile_of(blockIdx.x, gridDim.x, tiles_n, tile_n, tile_m, first_round, 128 * TM);
  compute_tile<REGULAR, REM, WT, SEGS, TM, NLAST>(plan, tile_n, tile_m, tiles_n, N, m_store, a_rows, d, lds);
}

// The same for problems whose last round of 256 x 256 tiles would leave at least half of the CUs idle: the first
// n_whole workgroups compute whole tiles (n_whole a multiple of the CU count), the others the remaining whole tiles
// as two tiles of 256 x 128 each.  Measured: M = 4096, N = 5120, K = 8576 / 4800 / 448 (320 tiles) 166 -> 147 us; where the
// last round is exactly half full (M = 4096, N = 14336: 896 tiles) it changes nothing -- the chip is at its power limit,
// and the CUs that work while the others idle get the clock the others do not use.
template <bool REM, bool WT, int NLAST>
__global__ void __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
mixed_gemm_256_tail_kernel(Plan plan_arg, int tiles_n, int N, int m_store, int a_rows, uint16_t* __restrict__ d, int first_round,
                           int skew, int n_whole) {
  extern __shared__ __align__(16) uint8_t lds[];
  const Plan plan = start_workgroup<WT>(plan_arg, first_round, skew);
  const int wg = blockIdx.x;
  const int ntiles = n_whole + (((int)gridDim.x - n_whole) >> 1);   // whole tiles of the problem
  int tile_n, tile_m;
  if (wg < n_whole) {
    tile_of(wg, ntiles, tiles_n, tile_n, tile_m);
    compute_tile<true, REM, WT, 7, 2, NLAST>(plan, tile_n, tile_m, tiles_n, N, m_store, a_rows, d, lds);
  } else {
    // Where the XCDs walk bands of feature tiles, the two halves of a tile go to the XCD that holds the tile's band
    // (workgroups 8 apart): its L2 then fetches the weight tile once for both, and the tiles left over in a band
    // share their token rows (M = 4096, N = 14336: 250 -> 226 MB past the L2s).  Elsewhere the halves of a tile are
    // neighbouring workgroups: an XCD then holds upper or lower halves only, of two XCDs' leftovers, which for the
    // feature-major walk are the same token tiles (M = 4096, N = 5120, K = 13824: 443 MB that way, 502 MB paired).
    const int h = wg - n_whole, nh = (int)gridDim.x - n_whole;
    int t = ((h >> 4) << 3) | (h & 7), upper = (h >> 3) & 1;
    const bool paired = tile_of(n_whole + t, ntiles, tiles_n, tile_n, tile_m) && (n_whole & 7) == 0 && (nh & 15) == 0;
    if (!paired) {
      t = h >> 1;
      upper = h & 1;
      tile_of(n_whole + t, ntiles, tiles_n, tile_n, tile_m);
    }
    const int half_m = 2 * tile_m + upper;
    if (half_m * 128 >= m_store) return;   // the lower half of a ragged last tile: no token of it exists
    compute_tile<true, REM, WT, 7, 1, NLAST>(plan, tile_n, half_m, tiles_n, N, m_store, a_rows, d, lds);
  }
}

}  // namespace


bool mixed_gemm_256_supported(int M, int N, int KN, int KS, int KO) {
  if (M <= 0 || N <= 0 || KN < 0 || KS < 0 || KO < 0) return false;
  // N: whole 8-feature store pieces (tile-major weights need whole tiles: mg_weights_tileable)
  if (M % kT != 0 || N % 8 != 0 || KN % 32 != 0 || KS % 32 != 0 || KO % 32 != 0) return false;
  // all three segments with at least one whole 128-wide stage: the pipeline hands the prefetched
  // fragments from one segment's loop to the next, in the order E2M1 -> E3M2 -> E4M3
  if (KN >= 128 && KS >= 128 && KO >= 128) return true;
  // plans without one or two of the segments (pure E3M2 x E2M1 and E4M3 x E2M1 products among them, the reference's
  // matmul_host6 / matmul_host8 on their own): whole stages only
  return (KN | KS | KO) % 128 == 0 && KN + KS + KO > 0;
}

// Token rows per workgroup tile for a problem of m_store tokens: 256, or 128 when the 256 x 256 tiles would leave
// at least half of the CUs without one.  A half tile takes most of a whole tile's time (the copies of a stage
// bound it, not its MFMAs), so halves pay only where they put idle CUs to work.
static int tile_tokens(int m_store, int N, int cus) {
  const long long tiles = (long long)((m_store + kT - 1) / kT) * ((N + kT - 1) / kT);
  return tiles <= cus / 2 ? 128 : 256;
}

typedef void (*kernel_t)(Plan, int, int, int, int, uint16_t*, int, int);

// The kernel for a plan: segs = which activation segments exist (bit 0 E2M1, 1 E3M2, 2 E4M3), nlast = stages of the
// last one (3 = three or more), regular = every segment but the last has at least three stages.  Plans with an empty
// segment exist in the whole-stage form only (!REM).
template <bool REM, bool WT, int TM, int SEGS>
static kernel_t select_by_length(bool regular, int nlast) {
  constexpr bool kOne = SEGS == 1 || SEGS == 2 || SEGS == 4;   // one segment: nothing to hand over, any length
  if constexpr (kOne) return mixed_gemm_256_kernel<true, REM, WT, SEGS, TM, 0>;
  if (!regular) return mixed_gemm_256_kernel<false, REM, WT, SEGS, TM, 0>;
  return nlast == 1 ? mixed_gemm_256_kernel<true, REM, WT, SEGS, TM, 1>
                    : (nlast == 2 ? mixed_gemm_256_kernel<true, REM, WT, SEGS, TM, 2> : mixed_gemm_256_kernel<true, REM, WT, SEGS, TM, 3>);
}
template <bool REM, bool WT, int TM>
static kernel_t select_kernel(bool regular, int segs, int nlast) {
  if (segs == 7) return select_by_length<REM, WT, TM, 7>(regular, nlast);
  if constexpr (!REM) {
    switch (segs) {
      case 1: return select_by_length<false, WT, TM, 1>(regular, nlast);
      case 2: return select_by_length<false, WT, TM, 2>(regular, nlast);
      case 3: return select_by_length<false, WT, TM, 3>(regular, nlast);
      case 4: return select_by_length<false, WT, TM, 4>(regular, nlast);
      case 5: return select_by_length<false, WT, TM, 5>(regular, nlast);
      case 6: return select_by_length<false, WT, TM, 6>(regular, nlast);
      default: break;
    }
  }
  return nullptr;
}

typedef void (*tail_kernel_t)(Plan, int, int, int, int, uint16_t*, int, int, int);

template <bool REM, bool WT>
static tail_kernel_t select_tail_kernel(int nlast) {
  return nlast == 1 ? mixed_gemm_256_tail_kernel<REM, WT, 1>
                    : (nlast == 2 ? mixed_gemm_256_tail_kernel<REM, WT, 2> : mixed_gemm_256_tail_kernel<REM, WT, 3>);
}

hipError_t launch_mixed_gemm_256(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                                 const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                                 const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo,
                                 int m_store, int a_rows, int N, int KN, int KS, int KO, bool w_tiled, void* d,
                                 hipStream_t stream) {
  // m_store tokens are computed in whole tiles of 256 or 128 token rows; rows past m_store are computed but not
  // stored; the activation buffers are read up to row a_rows - 1 only
  if (m_store <= 0 || a_rows < m_store) return hipErrorInvalidValue;
  DeviceLimits lim;
  if (hipError_t e = device_limits(&lim); e != hipSuccess) return e;
  const int tokens = tile_tokens(m_store, N, lim.cus);
  const int M = (m_store + tokens - 1) / tokens * tokens;
  const bool rem = (KN | KS | KO) % 128 != 0;
  const int half = tokens == 128 ? 1 : 0;
  const int segs = (KN > 0 ? 1 : 0) | (KS > 0 ? 2 : 0) | (KO > 0 ? 4 : 0);
  // every segment that another follows has at least 3 whole stages: the copies across segment boundaries are compiled in
  const bool regular = (KN == 0 || KN >= 384 || (KS == 0 && KO == 0)) && (KS == 0 || KS >= 384 || KO == 0);
  const int last_stages = KO > 0 ? KO / 128 : (KS > 0 ? KS / 128 : KN / 128);
  const int nlast = last_stages >= 3 ? 3 : last_stages;
  // token tiles of 32 per wave: 2 for 256 x 256 workgroup tiles, 1 for 256 x 128
  kernel_t kernel = nullptr;
  if (rem) {
    if (w_tiled) kernel = half ? select_kernel<true, true, 1>(regular, segs, nlast) : select_kernel<true, true, 2>(regular, segs, nlast);
    else kernel = half ? select_kernel<true, false, 1>(regular, segs, nlast) : select_kernel<true, false, 2>(regular, segs, nlast);
  } else {
    if (w_tiled) kernel = half ? select_kernel<false, true, 1>(regular, segs, nlast) : select_kernel<false, true, 2>(regular, segs, nlast);
    else kernel = half ? select_kernel<false, false, 1>(regular, segs, nlast) : select_kernel<false, false, 2>(regular, segs, nlast);
  }
  if (kernel == nullptr) return hipErrorInvalidValue;
  // a last round of whole tiles on at most half of the CUs: those tiles as twice as many half tiles
  const int whole_tiles = ((N + kT - 1) / kT) * (M / tokens);
  const int rest = whole_tiles % lim.cus;
  const bool tail = !half && regular && segs == 7 && whole_tiles > lim.cus && rest > 0 && 2 * rest <= lim.cus;
  tail_kernel_t tail_kernel = nullptr;
  if (tail) {
    if (rem) tail_kernel = w_tiled ? select_tail_kernel<true, true>(nlast) : select_tail_kernel<true, false>(nlast);
    else tail_kernel = w_tiled ? select_tail_kernel<false, true>(nlast) : select_tail_kernel<false, false>(nlast);
    if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(tail_kernel), kBuffers * kStage); e != hipSuccess) return e;
  }
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kBuffers * kStage); e != hipSuccess) return e;
  Plan p;
  p.a0 = an; p.a1 = as_; p.a2 = ao;
  p.b0 = bn; p.b1 = bs; p.b2 = bo;
  p.sfa0 = sfan; p.sfa1 = sfas; p.sfa2 = sfao;
  p.sfb0 = sfbn; p.sfb1 = sfbs; p.sfb2 = sfbo;
  p.st0 = KN / 128; p.st1 = KS / 128; p.st2 = KO / 128;
  p.blk0 = KN / 32; p.blk1 = KS / 32; p.blk2 = KO / 32;
  p.total = p.st0 + p.st1 + p.st2;
  p.w_tiled = w_tiled ? 1 : 0;
  if (w_tiled && N % kT != 0) return hipErrorInvalidValue;
  const int tiles_n = (N + kT - 1) / kT, tiles_m = M / tokens;
  // more tiles than CUs: staggered start (see the kernel), up to kStartSkew ticks of the shader's clock counter
  const int ntiles = tiles_n * tiles_m;
  const int skew = ntiles > lim.cus ? kStartSkew : 0;
  if (tail)
    hipLaunchKernelGGL(tail_kernel, dim3(ntiles + rest), dim3(64 * kWaves), kBuffers * kStage, stream, p, tiles_n, N, m_store, a_rows,
                       static_cast<uint16_t*>(d), lim.cus, skew, ntiles - rest);
  else
    hipLaunchKernelGGL(kernel, dim3(ntiles), dim3(64 * kWaves), kBuffers * kStage, stream, p, tiles_n, N, m_store, a_rows,
                       static_cast<uint16_t*>(d), lim.cus, skew);
  return hipGetLastError();
}

// Tile-major weight order of one segment (N a multiple of 256): per feature tile of 256 rows and per
// whole 128-wide stage one block of 16 KB, inside it the 16 copy blocks of 1 KB in the order the
// kernel's LDS image wants them -- block j holds rows j + 16 * (2 * (k % 8) + k / 8) for lane quad
// k = 0..15, 64 bytes (the stage's K range) each.  A copy instruction then reads 1 KB of consecutive
// bytes (8 lines of 128 B) instead of 64 bytes from each of 16 rows (16 lines), and the address
// unit, which limits the loop, has two thirds of the work.  The 1-3 blocks of 32 elements a segment
// may have past its last whole stage follow behind the tiled part as N row-major rows.
__global__ void __launch_bounds__(256) tile_weights_kernel(const v4u* __restrict__ src, v4u* __restrict__ dst, int N, int blk) {
  const int nst = blk >> 2, rem = blk & 3;
  const size_t tiled = (size_t)N * nst * 4;   // 16-byte units in whole stages
  // Whole stages: 128 lanes move the 1 KB copy block j of two neighbouring stages (lane = 8 * quad + 4 * stage parity +
  // piece), so that the eight lanes of a quad read 128 consecutive bytes of one row -- a whole cache line -- and a wave
  // writes 512 consecutive bytes of each of the two stages.
  const int npairs = (nst + 1) >> 1;
  const size_t groups = (size_t)(N >> 8) * npairs * 16;
  const int t7 = threadIdx.x & 127;
  const unsigned c = t7 & 3, sp = (t7 >> 2) & 1, k = t7 >> 3;
  for (size_t g = (size_t)blockIdx.x * 2 + (threadIdx.x >> 7); g < groups; g += (size_t)gridDim.x * 2) {
    const unsigned j = g & 15;
    const size_t tp = g >> 4;
    const unsigned pair = tp % npairs;
    const size_t tile_n = tp / npairs;
    const unsigned ql = 2 * pair + sp;
    if (ql < (unsigned)nst) {
      const size_t row = tile_n * 256 + j + 16 * (2 * (k & 7) + (k >> 3));
      dst[(((tile_n * nst + ql) * 16 + j) << 6) + k * 4 + c] = src[row * blk + ql * 4 + c];
    }
  }
  // the 1-3 blocks past the last whole stage: N row-major rows behind the tiled part
  if (rem) {
    const size_t total = (size_t)N * blk;
    for (size_t u = tiled + (size_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (size_t)gridDim.x * 256) {
      const size_t v = u - tiled;
      dst[u] = src[(v / rem) * blk + nst * 4 + v % rem];
    }
  }
}

hipError_t launch_tile_weights(const uint8_t* src, uint8_t* dst, int N, int kseg, hipStream_t stream) {
  if (N % 256 != 0 || kseg % 32 != 0) return hipErrorInvalidValue;
  if (N == 0 || kseg == 0) return hipSuccess;
  const size_t units = (size_t)N * (kseg / 32);
  const int grid = (int)((units + 255) / 256 < 8192 ? (units + 255) / 256 : 8192);
  hipLaunchKernelGGL(tile_weights_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<const v4u*>(src),
                     reinterpret_cast<v4u*>(dst), N, kseg / 32);
  return hipGetLastError();
}

}  // namespace mg
