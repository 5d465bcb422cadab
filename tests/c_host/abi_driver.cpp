// A host program that uses the library the way a C or C++ application without torch would:
// HIP runtime calls for memory and the stream, the C-ABI of include/mixedgemm_abi.h for everything
// else.  It runs the whole path on one problem read from a file and writes every result to
// another; tests/test_gpu_c_host.py compares them with the golden vectors.
//
//   abi_driver <in.bin> <out.bin>
//   in.bin : int32 M, N, KN, KS, KO; bf16 X[M,K]; bf16 W[N,K]          (K = KN + KS + KO)
//   out.bin: int16 idx[K] (calibrated on X); the six activation outputs and the six weight outputs of
//            the quantizers, each as its raw buffer; bf16 D[M,N] from mg_mixed_gemm; bf16 D[M,N] from
//            mg_fused_linear_ex with tile-major weights
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "mixedgemm_abi.h"

#define HIP_OK(call)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));              \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)
#define MG_CALL(call)                                                                     \
  do {                                                                                    \
    int s_ = (call);                                                                      \
    if (s_ != MG_OK) {                                                                    \
      std::fprintf(stderr, "%s failed: %s\n", #call, mg_status_string(s_));               \
      return 3;                                                                           \
    }                                                                                     \
  } while (0)

namespace {

struct DeviceBuffer {
  void* p = nullptr;
  size_t bytes = 0;
  hipError_t alloc(size_t n) {
    bytes = n;
    return hipMalloc(&p, n ? n : 1);
  }
  ~DeviceBuffer() {
    if (p) (void)hipFree(p);
  }
  uint8_t* u8() const { return static_cast<uint8_t*>(p); }
};

bool write_back(std::FILE* f, const DeviceBuffer& b) {
  std::vector<uint8_t> h(b.bytes);
  if (b.bytes && hipMemcpy(h.data(), b.p, b.bytes, hipMemcpyDeviceToHost) != hipSuccess) return false;
  return std::fwrite(h.data(), 1, h.size(), f) == h.size();
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 3) {
    std::fprintf(stderr, "usage: %s <in.bin> <out.bin>\n", argv[0]);
    return 1;
  }
  std::FILE* in = std::fopen(argv[1], "rb");
  if (!in) return 1;
  int32_t dims[5];
  if (std::fread(dims, sizeof(int32_t), 5, in) != 5) return 1;
  const int M = dims[0], N = dims[1], KN = dims[2], KS = dims[3], KO = dims[4], K = KN + KS + KO;
  std::vector<uint16_t> hx((size_t)M * K), hw((size_t)N * K);
  if (std::fread(hx.data(), 2, hx.size(), in) != hx.size() || std::fread(hw.data(), 2, hw.size(), in) != hw.size()) return 1;
  std::fclose(in);

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  DeviceBuffer x, w, idx, cal_ws, d1, d2, fused_ws;
  HIP_OK(x.alloc(hx.size() * 2));
  HIP_OK(w.alloc(hw.size() * 2));
  HIP_OK(idx.alloc((size_t)K * 2));
  HIP_OK(cal_ws.alloc(mg_calibrate_workspace_bytes(K)));
  HIP_OK(d1.alloc((size_t)M * N * 2));
  HIP_OK(d2.alloc((size_t)M * N * 2));
  HIP_OK(fused_ws.alloc(mg_fused_workspace_bytes(M, KN, KS, KO)));
  HIP_OK(hipMemcpyAsync(x.p, hx.data(), x.bytes, hipMemcpyHostToDevice, stream));
  HIP_OK(hipMemcpyAsync(w.p, hw.data(), w.bytes, hipMemcpyHostToDevice, stream));

  // activation outputs: XN [M, KN/2], XS [M, 3KS/4], XO [M, KO] + three scale buffers;
  // weight outputs: WN [N, KN/2], WS [N, KS/2], WO [N, KO/2] + three scale buffers
  DeviceBuffer a[6], b[6], bt[3];
  const size_t a_bytes[6] = {(size_t)M * KN / 2, (size_t)M * KS / 4 * 3, (size_t)M * KO,
                             mg_sf_bytes(M, KN, MG_OPERAND_A), mg_sf_bytes(M, KS, MG_OPERAND_A), mg_sf_bytes(M, KO, MG_OPERAND_A)};
  const size_t b_bytes[6] = {(size_t)N * KN / 2, (size_t)N * KS / 2, (size_t)N * KO / 2,
                             mg_sf_bytes(N, KN, MG_OPERAND_B), mg_sf_bytes(N, KS, MG_OPERAND_B), mg_sf_bytes(N, KO, MG_OPERAND_B)};
  for (int i = 0; i < 6; ++i) {
    HIP_OK(a[i].alloc(a_bytes[i]));
    HIP_OK(b[i].alloc(b_bytes[i]));
    HIP_OK(hipMemsetAsync(a[i].p, 0, a[i].bytes ? a[i].bytes : 1, stream));   // scale entries of rows >= M are never written
    HIP_OK(hipMemsetAsync(b[i].p, 0, b[i].bytes ? b[i].bytes : 1, stream));
  }

  MG_CALL(mg_calibrate_reorder_index(x.p, M, K, static_cast<int16_t*>(idx.p), cal_ws.p, cal_ws.bytes, stream));
  const int16_t* index = static_cast<const int16_t*>(idx.p);
  MG_CALL(mg_reorder_quantize_x(x.p, index, M, K, KN, KS, KO, a[0].u8(), a[1].u8(), a[2].u8(), a[3].u8(), a[4].u8(),
                                a[5].u8(), stream));
  MG_CALL(mg_reorder_quantize_w(w.p, index, N, K, KN, KS, KO, b[0].u8(), b[1].u8(), b[2].u8(), b[3].u8(), b[4].u8(),
                                b[5].u8(), stream));
  MG_CALL(mg_mixed_gemm(a[0].u8(), b[0].u8(), a[1].u8(), b[1].u8(), a[2].u8(), b[2].u8(), a[3].u8(), b[3].u8(), a[4].u8(),
                        b[4].u8(), a[5].u8(), b[5].u8(), M, N, KN, KS, KO, d1.p, stream));

  // the fused entry point, with tile-major weights when the shape allows
  unsigned flags = 0;
  const uint8_t* wc[3] = {b[0].u8(), b[1].u8(), b[2].u8()};
  if (mg_weights_tileable(N, KN, KS, KO)) {
    const int kseg[3] = {KN, KS, KO};
    for (int i = 0; i < 3; ++i) {
      HIP_OK(bt[i].alloc(b_bytes[i]));
      MG_CALL(mg_tile_weights(b[i].u8(), bt[i].u8(), N, kseg[i], stream));
      wc[i] = bt[i].u8();
    }
    flags = MG_FLAG_W_TILED;
  }
  MG_CALL(mg_fused_linear_ex(x.p, index, wc[0], wc[1], wc[2], b[3].u8(), b[4].u8(), b[5].u8(), M, N, KN, KS, KO, flags, d2.p,
                             fused_ws.p, fused_ws.bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));

  std::FILE* out = std::fopen(argv[2], "wb");
  if (!out) return 1;
  bool ok = write_back(out, idx);
  for (int i = 0; i < 6; ++i) ok = ok && write_back(out, a[i]);
  for (int i = 0; i < 6; ++i) ok = ok && write_back(out, b[i]);
  ok = ok && write_back(out, d1) && write_back(out, d2);
  std::fclose(out);
  (void)hipStreamDestroy(stream);
  std::printf("abi_driver: M=%d N=%d K=%d/%d/%d flags=%u %s\n", M, N, KN, KS, KO, flags, ok ? "ok" : "write failed");
  return ok ? 0 : 4;
}
