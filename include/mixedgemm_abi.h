/*
 * C-ABI of the MI355X (gfx950) reorder-quantize + mixed MXFP4/6/8 GEMM library.
 *
 * Plain C types only: device pointers, sizes, a HIP stream passed as void*.
 * Every entry point validates its arguments on the host, enqueues its kernels
 * on `stream` and returns without synchronizing (mg_device_synchronize and
 * mg_check_reorder_index, whose job it is to wait, excepted); none allocates.  The return
 * value is a status code: 0 on success, a hipError_t value for a HIP failure, or
 * one of the MG_ERR_* codes below.  mg_status_string() names any of them.
 *
 * Citations give the reference interface each entry point replaces, relative
 * to the reference tree.
 */
#ifndef MIXEDGEMM_ABI_H
#define MIXEDGEMM_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MG_OK 0
#define MG_ERR_BAD_SHAPE 10001   /* a segment is not a multiple of 32, K mismatch, negative size */
#define MG_ERR_BAD_POINTER 10002 /* null or insufficiently aligned pointer (16 bytes required) */
#define MG_ERR_BAD_INDEX 10003   /* reorder index entry outside [0, K): mg_check_reorder_index[_host] */
#define MG_ERR_UNSUPPORTED 10004 /* shape outside what the kernels handle (K > 32736) */
#define MG_ERR_TOO_LARGE 10005   /* mg_fused_linear_static: the activations do not fit the static scratch memory */

/* Operand selector for mg_sf_bytes(). */
#define MG_OPERAND_A 0 /* activations: (rows/128 + 1)*128*kseg/32, src/bindings.cpp:91-93 */
#define MG_OPERAND_B 1 /* weights:     rows*kseg/32,               src/bindings.cpp:210-212 */

/*
 * Activation reorder-quantize.  Replaces run_reorder_bf16_mixed<32,K>
 * (include/reorder.cuh:295-308, src/reorder.cu:434-469) and its kernel
 * reorder_bf16_mixed_kernel (src/reorder.cu:94-269), for any K that is a
 * multiple of 32 (the reference instantiates seven values of K only).
 *
 *   x_bf16 [M, K] bf16 row-major, idx [K] int16 (output position j takes input
 *   channel idx[j]); K = KN + KS + KO, each a multiple of 32.
 *   qn [M, KN/2]   E2M1 codes, element 2i in the low nibble of byte i
 *   qs [M, 3KS/4]  E3M2 codes, 4 codes per 3 bytes, little-endian bit stream
 *   qo [M, KO]     E4M3 codes
 *   sfn/sfs/sfo    E8M0 scale bytes, one per 32 elements, in the 128-row x
 *                  4-block interleaved layout; mg_sf_bytes(M, Kseg, MG_OPERAND_A)
 *                  bytes each.  Entries of rows >= M are left untouched.
 * Inputs are expected to be finite.  A 32-element block that holds an infinity or a NaN gets codes
 * and a scale that are not specified (the reference's own arithmetic, log2 and a division by the
 * scale, src/reorder.cu:172-197, is undefined there too); other blocks are not affected.
 */
int mg_reorder_quantize_x(const void* x_bf16, const int16_t* idx, int M, int K, int KN, int KS, int KO,
                          uint8_t* qn, uint8_t* qs, uint8_t* qo,
                          uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream);

/*
 * Weight reorder-quantize: same gather and scale rule, all three segments to
 * E2M1.  Replaces run_reorder_bf16_fp4<32,K> (include/reorder.cuh:310-323,
 * src/reorder.cu:471-506) and reorder_bf16_fp4_kernel (src/reorder.cu:271-432).
 *   qn [N, KN/2], qs [N, KS/2], qo [N, KO/2]; scale buffers of
 *   mg_sf_bytes(N, Kseg, MG_OPERAND_B) bytes.
 */
int mg_reorder_quantize_w(const void* w_bf16, const int16_t* idx, int N, int K, int KN, int KS, int KO,
                          uint8_t* qn, uint8_t* qs, uint8_t* qo,
                          uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream);

/*
 * mg_reorder_quantize_x with an RMSNorm in front, in the same pass over the rows (the layer that feeds
 * a quantized linear in a transformer block; the reference leaves it to the caller and reads the
 * normalised activations back from memory):
 *   var = fl32( (sum of x^2 over the row, accumulated in fp64) / K ),  r = fl32( 1 / sqrt( fl32(var + eps) ) ),
 *   y = bf16( gamma * bf16( x * r ) )   -- both products in fp32, gamma bf16 [K] --
 * and y is what gets gathered and quantized.  eps >= 0.
 */
int mg_rmsnorm_reorder_quantize_x(const void* x_bf16, const void* gamma_bf16, float eps, const int16_t* idx,
                                  int M, int K, int KN, int KS, int KO,
                                  uint8_t* qn, uint8_t* qs, uint8_t* qo,
                                  uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream);

/*
 * Mixed block-scaled GEMM: D[M,N] = bf16( sum over the three K segments of
 * A_seg . B_seg^T ), fp32 accumulation across all segments, one bf16 rounding.
 * Replaces matmul_host (include/gemm.h:21-41, src/gemm.cu:22-47) and the three
 * segment GEMMs it chains (src/fp4.cu:35, src/fp6.cu:35, src/fp8.cu:35).
 * Operand layouts are the ones the two quantizers above produce.
 */
int mg_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                  const uint8_t* ao, const uint8_t* bo,
                  const uint8_t* sfan, const uint8_t* sfbn, const uint8_t* sfas, const uint8_t* sfbs,
                  const uint8_t* sfao, const uint8_t* sfbo,
                  int M, int N, int KN, int KS, int KO, void* d_bf16, void* stream);

/*
 * The same GEMM with two things a caller may know about its buffers:
 *   a_rows -- an, as_, ao are readable for a_rows >= M token rows and sfan, sfas, sfao for
 *     mg_sf_bytes(a_rows, kseg, MG_OPERAND_A) bytes (what lies past row M is never used for a
 *     result).  a_rows == M is always valid: the whole-tile kernel never reads past row a_rows - 1
 *     (lanes of later rows read that row again) and never writes past row M - 1.
 *   flags  -- MG_FLAG_W_TILED: bn, bs, bo hold the codes in the tile-major order mg_tile_weights
 *     writes (same sizes; mg_weights_tileable(N, KN, KS, KO) must hold).  The prefill kernel's copies
 *     then read consecutive kilobytes, which is worth 10-15 % of its time.
 * mg_mixed_gemm is this with a_rows = M, flags = 0.  The reference has no counterpart: its CUTLASS
 * GEMMs (src/fp4.cu:164-182) predicate partial tiles themselves and fix their operand layouts.
 */
#define MG_FLAG_W_TILED 1u
#define MG_STATIC_SCRATCH_BYTES ((size_t)20 << 20) /* mg_fused_linear_static */
int mg_mixed_gemm_ex(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                     const uint8_t* ao, const uint8_t* bo,
                     const uint8_t* sfan, const uint8_t* sfbn, const uint8_t* sfas, const uint8_t* sfbs,
                     const uint8_t* sfao, const uint8_t* sfbo,
                     int M, int a_rows, int N, int KN, int KS, int KO, unsigned flags, void* d_bf16, void* stream);
/* Rewrites one segment's weight codes src[N, kseg/2] (row-major, as mg_reorder_quantize_w wrote them;
 * the weight path of src/bindings.cpp:188-305) into tile-major order in dst (same size, dst != src):
 * per 256-feature tile and 128-wide K stage one block of 16 KB, ordered as the prefill kernel stages
 * it; the 1-3 blocks of 32 a segment may have past its last whole stage follow as row-major rows.
 * N a multiple of 256, kseg a multiple of 32.  Done once per layer, offline. */
int mg_tile_weights(const uint8_t* src, uint8_t* dst, int N, int kseg, void* stream);
/* 1 when weights of this shape can be tiled (the shapes the whole-tile kernel takes, whole tiles only): N a multiple of
 * 256 and either every segment a multiple of 32 and at least 128 wide, or one or two of the segments empty and
 * the others multiples of 128 (pure E3M2 x E2M1 and E4M3 x E2M1 products among them: what matmul_host6 and
 * matmul_host8 of the reference, src/fp6.cu:35 and src/fp8.cu:35, compute on their own). */
int mg_weights_tileable(int N, int KN, int KS, int KO);
/* M rounded up to whole 256-token tiles. */
int mg_padded_rows(int M);

/*
 * Activation reorder-quantize followed by the mixed GEMM on the same stream
 * (the sequence src/bindings.cpp:69-186 then :9-67 performs with a device-wide
 * synchronize in between; bench_reorder_gemm.cu:163-167 times the same pair).
 * `workspace` receives the quantized activations and their scales;
 * mg_fused_workspace_bytes(M, KN, KS, KO) bytes, 256-byte aligned.
 */
int mg_fused_linear(const void* x_bf16, const int16_t* idx,
                    const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                    const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo,
                    int M, int N, int KN, int KS, int KO,
                    void* d_bf16, void* workspace, size_t workspace_bytes, void* stream);
/* mg_fused_linear with the flags of mg_mixed_gemm_ex (MG_FLAG_W_TILED). */
int mg_fused_linear_ex(const void* x_bf16, const int16_t* idx,
                       const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                       const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo,
                       int M, int N, int KN, int KS, int KO, unsigned flags,
                       void* d_bf16, void* workspace, size_t workspace_bytes, void* stream);
/* mg_fused_linear_ex with the RMSNorm of mg_rmsnorm_reorder_quantize_x in front (gamma_bf16 == NULL: none). */
int mg_fused_norm_linear(const void* x_bf16, const void* gamma_bf16, float eps, const int16_t* idx,
                         const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                         const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo,
                         int M, int N, int KN, int KS, int KO, unsigned flags,
                         void* d_bf16, void* workspace, size_t workspace_bytes, void* stream);
size_t mg_fused_workspace_bytes(int M, int KN, int KS, int KO);

/*
 * mg_fused_linear_ex without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart
 * in the reference.  The quantized activations go through memory the library owns: a static device array
 * of MG_STATIC_SCRATCH_BYTES = 20 MiB per GPU, held from the loading of the library until the process
 * ends.  Problems with mg_fused_workspace_bytes(M, KN, KS, KO) above that size (M = 4096 at K = 4096 and
 * M = 2048 at K = 14336 fit) are rejected with MG_ERR_TOO_LARGE.  The call allocates and frees nothing;
 * its first call on a device looks up the array's address on that device (make it outside a capture).
 * Every call on a GPU uses that GPU's one array: calls that may overlap there (different streams without
 * an ordering between them, several host threads) race -- order them, or use mg_fused_linear_ex.  Nothing
 * in the array has to start at zero: a call rewrites every byte its GEMM's results depend on.
 */
int mg_fused_linear_static(const void* x_bf16, const int16_t* idx,
                           const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                           const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo,
                           int M, int N, int KN, int KS, int KO, unsigned flags,
                           void* d_bf16, void* stream);

/* Size in bytes of one segment's scale buffer (src/bindings.cpp:91-93, 210-212);
 * never smaller than the interleaved layout spans. */
size_t mg_sf_bytes(int rows, int kseg, int operand);

/* Byte offset of the scale of (row, 32-element block kb) inside a segment's
 * scale buffer (include/reorder.cuh:119-124; src/reorder.cu:182-185). */
size_t mg_sf_offset(int row, int kb, int kseg);

/* Calibration step that produces the reorder index (the commented lines main.py:31-33 of the
 * reference: per-channel max |x| over the rows of a bf16 sample X[M,K], channels sorted by it in
 * ascending order, as int16).  Ties are ordered by channel number.  K a multiple of 32, <= 32736.
 * `workspace`: mg_calibrate_workspace_bytes(K) bytes of device memory, 16-byte aligned. */
int mg_calibrate_reorder_index(const void* x_bf16, int M, int K, int16_t* idx,
                               void* workspace, size_t workspace_bytes, void* stream);
size_t mg_calibrate_workspace_bytes(int K);

/* Range check of a reorder index, for the places where an index enters the system (calibration, a
 * pack file, a caller's own tensor): MG_OK when every entry lies in [0, K), MG_ERR_BAD_INDEX otherwise.
 * The reference never checks: its K is a template constant and an out-of-range entry reads outside the
 * staged row (src/reorder.cu:154-158, 187).  The quantizers here clamp such an entry to channel K - 1, so
 * that they stay inside the row whatever the index holds; these calls are how a caller finds out.
 *   _host: idx is host memory.  The other: idx is device memory; copies it to the host behind the work
 *   already enqueued on `stream` and BLOCKS until that copy has finished (a pack-time call). */
int mg_check_reorder_index_host(const int16_t* idx, int K);
int mg_check_reorder_index(const int16_t* idx, int K, void* stream);

/* Blocks the host until all work on the current device has finished
 * (src/bindings.cpp:59,178,297 do this after every operator). */
int mg_device_synchronize(void);

/* Text for a status code returned by any function above. */
const char* mg_status_string(int status);

#ifdef __cplusplus
}
#endif
#endif /* MIXEDGEMM_ABI_H */
