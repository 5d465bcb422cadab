// extern "C" surface of the library: argument validation on the host, then the
// kernel launchers.  Nothing here allocates device memory or synchronizes (except
// mg_device_synchronize and mg_check_reorder_index, whose job that is).
#include "../../include/mixedgemm_abi.h"

#include "mg_common.h"

#include <vector>

namespace mg {
template <bool IS_W>
hipError_t launch_reorder_quant(const void* x, const int16_t* idx, int rows, int K, int KN, int KS, int KO, uint8_t* qn,
                                uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, const void* gamma,
                                float eps, bool keep_codes, hipStream_t stream);
hipError_t launch_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs,
                             const uint8_t* ao, const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn,
                             const uint8_t* sfas, const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo, int M,
                             int a_rows, int N, int KN, int KS, int KO, unsigned flags, void* d, hipStream_t stream);
hipError_t launch_tile_weights(const uint8_t* src, uint8_t* dst, int N, int kseg, hipStream_t stream);
bool mixed_gemm_256_supported(int M, int N, int KN, int KS, int KO);
size_t calibrate_workspace_bytes(int K);
hipError_t launch_calibrate(const void* x, int rows, int K, int16_t* idx, void* workspace, hipStream_t stream);
}  // namespace mg

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A segment pointer may be null only when that segment is empty.
bool ptr_ok(const void* p, bool needed) { return needed ? (p != nullptr && aligned16(p)) : true; }

int check_split(int rows, int KN, int KS, int KO) {
  if (rows < 0 || KN < 0 || KS < 0 || KO < 0) return MG_ERR_BAD_SHAPE;
  if ((KN | KS | KO) & 31) return MG_ERR_BAD_SHAPE;
  if ((long long)KN + KS + KO > 32736) return MG_ERR_UNSUPPORTED;  // int16 index, one lane per block, <= 1024 lanes
  return MG_OK;
}

template <bool IS_W>
int reorder_quantize(const void* x, const int16_t* idx, int rows, int K, int KN, int KS, int KO, uint8_t* qn,
                     uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream,
                     const void* gamma = nullptr, float eps = 0.0f, bool keep_codes = false) {
  if (int s = check_split(rows, KN, KS, KO)) return s;
  if (K != KN + KS + KO) return MG_ERR_BAD_SHAPE;
  if (rows == 0 || K == 0) return MG_OK;
  if (!ptr_ok(x, true) || !ptr_ok(idx, true)) return MG_ERR_BAD_POINTER;
  if (!ptr_ok(qn, KN > 0) || !ptr_ok(qs, KS > 0) || !ptr_ok(qo, KO > 0)) return MG_ERR_BAD_POINTER;
  if ((KN > 0 && !sfn) || (KS > 0 && !sfs) || (KO > 0 && !sfo)) return MG_ERR_BAD_POINTER;
  return (int)mg::launch_reorder_quant<IS_W>(x, idx, rows, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, gamma, eps, keep_codes,
                                             static_cast<hipStream_t>(stream));
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// Library-owned scratch memory of mg_fused_linear_static: the quantized activations and their scales
// between the two kernels of a fused call.  One copy per GPU, allocated with the code object and held
// until the process ends.  `scratch` is a host-side stand-in for the symbol, never a device address:
// host code uses the per-device pointer scratch_ptr() returns.
constexpr size_t kScratchBytes = MG_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[kScratchBytes];

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device, looked up once per device.
hipError_t scratch_ptr(uint8_t** out) {
  static std::mutex mu;
  static uint8_t* table[kMaxDevices] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (table[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    table[dev] = static_cast<uint8_t*>(p);
  }
  *out = table[dev];
  return hipSuccess;
}

}  // namespace

extern "C" {

int mg_reorder_quantize_x(const void* x_bf16, const int16_t* idx, int M, int K, int KN, int KS, int KO, uint8_t* qn,
                          uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream) {
  return reorder_quantize<false>(x_bf16, idx, M, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, stream);
}

int mg_rmsnorm_reorder_quantize_x(const void* x_bf16, const void* gamma_bf16, float eps, const int16_t* idx, int M, int K,
                                  int KN, int KS, int KO, uint8_t* qn, uint8_t* qs, uint8_t* qo, uint8_t* sfn,
                                  uint8_t* sfs, uint8_t* sfo, void* stream) {
  if (!ptr_ok(gamma_bf16, true) || !(eps >= 0.0f)) return gamma_bf16 ? MG_ERR_BAD_SHAPE : MG_ERR_BAD_POINTER;
  return reorder_quantize<false>(x_bf16, idx, M, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, stream, gamma_bf16, eps);
}

int mg_reorder_quantize_w(const void* w_bf16, const int16_t* idx, int N, int K, int KN, int KS, int KO, uint8_t* qn,
                          uint8_t* qs, uint8_t* qo, uint8_t* sfn, uint8_t* sfs, uint8_t* sfo, void* stream) {
  return reorder_quantize<true>(w_bf16, idx, N, K, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, stream);
}

int mg_mixed_gemm_ex(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs, const uint8_t* ao,
                     const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn, const uint8_t* sfas,
                     const uint8_t* sfbs, const uint8_t* sfao, const uint8_t* sfbo, int M, int a_rows, int N, int KN,
                     int KS, int KO, unsigned flags, void* d_bf16, void* stream) {
  if (int s = check_split(M, KN, KS, KO)) return s;
  if (N < 0 || a_rows < M) return MG_ERR_BAD_SHAPE;
  if (flags & ~MG_FLAG_W_TILED) return MG_ERR_BAD_SHAPE;
  if ((flags & MG_FLAG_W_TILED) && !mg_weights_tileable(N, KN, KS, KO)) return MG_ERR_UNSUPPORTED;
  if (M == 0 || N == 0) return MG_OK;
  if (!ptr_ok(d_bf16, true)) return MG_ERR_BAD_POINTER;
  if (!ptr_ok(an, KN > 0) || !ptr_ok(bn, KN > 0) || !ptr_ok(as_, KS > 0) || !ptr_ok(bs, KS > 0) ||
      !ptr_ok(ao, KO > 0) || !ptr_ok(bo, KO > 0))
    return MG_ERR_BAD_POINTER;
  if ((KN > 0 && (!sfan || !sfbn)) || (KS > 0 && (!sfas || !sfbs)) || (KO > 0 && (!sfao || !sfbo)))
    return MG_ERR_BAD_POINTER;
  return (int)mg::launch_mixed_gemm(an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs, sfao, sfbo, M, a_rows, N, KN, KS, KO,
                                    flags, d_bf16, static_cast<hipStream_t>(stream));
}

int mg_mixed_gemm(const uint8_t* an, const uint8_t* bn, const uint8_t* as_, const uint8_t* bs, const uint8_t* ao,
                  const uint8_t* bo, const uint8_t* sfan, const uint8_t* sfbn, const uint8_t* sfas, const uint8_t* sfbs,
                  const uint8_t* sfao, const uint8_t* sfbo, int M, int N, int KN, int KS, int KO, void* d_bf16,
                  void* stream) {
  return mg_mixed_gemm_ex(an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs, sfao, sfbo, M, M, N, KN, KS, KO, 0u, d_bf16, stream);
}

int mg_padded_rows(int M) { return M <= 0 ? 0 : (M + 255) / 256 * 256; }

int mg_weights_tileable(int N, int KN, int KS, int KO) {
  return N > 0 && N % 256 == 0 && mg::mixed_gemm_256_supported(256, N, KN, KS, KO);   // what the whole-tile kernel takes
}

int mg_tile_weights(const uint8_t* src, uint8_t* dst, int N, int kseg, void* stream) {
  if (N < 0 || kseg < 0 || N % 256 != 0 || kseg % 32 != 0) return MG_ERR_BAD_SHAPE;
  if (N == 0 || kseg == 0) return MG_OK;
  if (!ptr_ok(src, true) || !ptr_ok(dst, true) || src == dst) return MG_ERR_BAD_POINTER;
  return (int)mg::launch_tile_weights(src, dst, N, kseg, static_cast<hipStream_t>(stream));
}

size_t mg_sf_bytes(int rows, int kseg, int operand) {
  if (rows < 0 || kseg < 0) return 0;
  const size_t span = (size_t)((rows + 127) / 128) * (size_t)((kseg + 127) / 128) * 512;
  const size_t ref = operand == MG_OPERAND_A ? (size_t)(rows / 128 + 1) * 128 * (size_t)kseg / 32
                                             : (size_t)rows * (size_t)kseg / 32;
  return ref > span ? ref : span;
}

size_t mg_sf_offset(int row, int kb, int kseg) { return mg::sf_offset(row, kb, (kseg + 127) / 128); }

// The quantized activations live in the workspace with room for whole 256-row tiles, so that the
// GEMM may read (and ignore) the rows between M and the next multiple of 256.
size_t mg_fused_workspace_bytes(int M, int KN, int KS, int KO) {
  if (M < 0 || KN < 0 || KS < 0 || KO < 0) return 0;
  const int R = mg_padded_rows(M);
  return align256((size_t)R * (KN / 2)) + align256((size_t)R * (KS / 4 * 3)) + align256((size_t)R * KO) +
         align256(mg_sf_bytes(R, KN, MG_OPERAND_A)) + align256(mg_sf_bytes(R, KS, MG_OPERAND_A)) +
         align256(mg_sf_bytes(R, KO, MG_OPERAND_A));
}

int mg_fused_norm_linear(const void* x_bf16, const void* gamma_bf16, float eps, const int16_t* idx, const uint8_t* bn,
                         const uint8_t* bs, const uint8_t* bo, const uint8_t* sfbn, const uint8_t* sfbs,
                         const uint8_t* sfbo, int M, int N, int KN, int KS, int KO, unsigned flags, void* d_bf16,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (gamma_bf16 != nullptr && !(eps >= 0.0f)) return MG_ERR_BAD_SHAPE;
  if (int s = check_split(M, KN, KS, KO)) return s;
  if (N < 0) return MG_ERR_BAD_SHAPE;
  if (M == 0 || N == 0) return MG_OK;
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return MG_ERR_BAD_POINTER;
  if (workspace_bytes < mg_fused_workspace_bytes(M, KN, KS, KO)) return MG_ERR_BAD_SHAPE;
  const int R = mg_padded_rows(M);
  uint8_t* p = static_cast<uint8_t*>(workspace);
  uint8_t* qn = p;  p += align256((size_t)R * (KN / 2));
  uint8_t* qs = p;  p += align256((size_t)R * (KS / 4 * 3));
  uint8_t* qo = p;  p += align256((size_t)R * KO);
  uint8_t* sfn = p; p += align256(mg_sf_bytes(R, KN, MG_OPERAND_A));
  uint8_t* sfs = p; p += align256(mg_sf_bytes(R, KS, MG_OPERAND_A));
  uint8_t* sfo = p;
  // the GEMM reads the codes next: ordinary stores, so that they are in the L2 when it starts
  if (int s = reorder_quantize<false>(x_bf16, idx, M, KN + KS + KO, KN, KS, KO, qn, qs, qo, sfn, sfs, sfo, stream, gamma_bf16, eps,
                                      /*keep_codes=*/true))
    return s;
  return mg_mixed_gemm_ex(qn, bn, qs, bs, qo, bo, sfn, sfbn, sfs, sfbs, sfo, sfbo, M, R, N, KN, KS, KO, flags, d_bf16, stream);
}

int mg_fused_linear_ex(const void* x_bf16, const int16_t* idx, const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                       const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo, int M, int N, int KN, int KS, int KO,
                       unsigned flags, void* d_bf16, void* workspace, size_t workspace_bytes, void* stream) {
  return mg_fused_norm_linear(x_bf16, nullptr, 0.0f, idx, bn, bs, bo, sfbn, sfbs, sfbo, M, N, KN, KS, KO, flags, d_bf16,
                              workspace, workspace_bytes, stream);
}

int mg_fused_linear(const void* x_bf16, const int16_t* idx, const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                    const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo, int M, int N, int KN, int KS, int KO,
                    void* d_bf16, void* workspace, size_t workspace_bytes, void* stream) {
  return mg_fused_linear_ex(x_bf16, idx, bn, bs, bo, sfbn, sfbs, sfbo, M, N, KN, KS, KO, 0u, d_bf16, workspace,
                            workspace_bytes, stream);
}

int mg_fused_linear_static(const void* x_bf16, const int16_t* idx, const uint8_t* bn, const uint8_t* bs, const uint8_t* bo,
                           const uint8_t* sfbn, const uint8_t* sfbs, const uint8_t* sfbo, int M, int N, int KN, int KS,
                           int KO, unsigned flags, void* d_bf16, void* stream) {
  if (int s = check_split(M, KN, KS, KO)) return s;
  if (N < 0) return MG_ERR_BAD_SHAPE;
  if (mg_fused_workspace_bytes(M, KN, KS, KO) > kScratchBytes) return MG_ERR_TOO_LARGE;
  if (M == 0 || N == 0) return MG_OK;
  uint8_t* ws = nullptr;
  if (hipError_t e = scratch_ptr(&ws); e != hipSuccess) return (int)e;
  return mg_fused_norm_linear(x_bf16, nullptr, 0.0f, idx, bn, bs, bo, sfbn, sfbs, sfbo, M, N, KN, KS, KO, flags, d_bf16, ws,
                              kScratchBytes, stream);
}

size_t mg_calibrate_workspace_bytes(int K) { return K > 0 ? mg::calibrate_workspace_bytes(K) : 0; }

int mg_calibrate_reorder_index(const void* x_bf16, int M, int K, int16_t* idx, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (M <= 0 || K <= 0 || (K & 31)) return MG_ERR_BAD_SHAPE;
  if (K > 32736) return MG_ERR_UNSUPPORTED;
  if (!x_bf16 || !aligned16(x_bf16) || !idx || !workspace || !aligned16(workspace)) return MG_ERR_BAD_POINTER;
  if (workspace_bytes < mg::calibrate_workspace_bytes(K)) return MG_ERR_BAD_SHAPE;
  return (int)mg::launch_calibrate(x_bf16, M, K, idx, workspace, static_cast<hipStream_t>(stream));
}

int mg_check_reorder_index_host(const int16_t* idx, int K) {
  if (K < 0) return MG_ERR_BAD_SHAPE;
  if (K > 0 && idx == nullptr) return MG_ERR_BAD_POINTER;
  for (int i = 0; i < K; ++i)
    if (idx[i] < 0 || idx[i] >= K) return MG_ERR_BAD_INDEX;
  return MG_OK;
}

int mg_check_reorder_index(const int16_t* idx, int K, void* stream) {
  if (K < 0) return MG_ERR_BAD_SHAPE;
  if (K > 32767) return MG_ERR_UNSUPPORTED;
  if (K == 0) return MG_OK;
  if (idx == nullptr) return MG_ERR_BAD_POINTER;
  std::vector<int16_t> host((size_t)K);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(host.data(), idx, (size_t)K * sizeof(int16_t), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return (int)e;
  return mg_check_reorder_index_host(host.data(), K);
}

int mg_device_synchronize(void) { return (int)hipDeviceSynchronize(); }

const char* mg_status_string(int status) {
  switch (status) {
    case MG_OK: return "success";
    case MG_ERR_BAD_SHAPE: return "invalid shape: segment sizes must be non-negative multiples of 32 and K = KN + KS + KO";
    case MG_ERR_BAD_POINTER: return "null or misaligned pointer (16-byte alignment required)";
    case MG_ERR_BAD_INDEX: return "reorder index entry out of range";
    case MG_ERR_UNSUPPORTED: return "unsupported shape: K must not exceed 32736";
    case MG_ERR_TOO_LARGE: return "problem too large for the library's static scratch memory (MG_STATIC_SCRATCH_BYTES)";
    default: return hipGetErrorString(static_cast<hipError_t>(status));
  }
}

}  // extern "C"
