// Python module `mixedgemm`: the reference's operator surface
// (src/bindings.cpp:311-343 of the reference -- matmul, reorder_quantize_x,
// reorder_quantize_w, test_function, same keyword names, same return tuples,
// same tensor shapes and dtypes) on top of the C-ABI of the HIP library.
//
// Conventions kept from the reference boundary:
//   * inputs are borrowed through data_ptr<T>() (dtype mismatch raises the torch
//     error), assumed contiguous row-major and on one device; outputs are
//     allocated here and owned by the returned tensors
//     (src/bindings.cpp:30-36, 85-93, 204-212);
//   * each operator blocks until the device has finished and turns a launch or
//     execution failure into std::runtime_error -> Python RuntimeError
//     (src/bindings.cpp:51-64, 170-183, 289-302);
//   * an invalid K raises RuntimeError("Value error in run_reorder_bf16_mixed ")
//     / ("... run_reorder_bf16_fp4 ") after "K value is not valid !" on stderr
//     (src/bindings.cpp:165-168, 284-287).  The reference accepts seven values
//     of K; this module accepts every split whose parts are multiples of 32.
// The reference's one-line progress print per operator is emitted only when the
// environment variable MIXEDGEMM_VERBOSE is set.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <tuple>

#include "mixedgemm_abi.h"

namespace {

using torch::Tensor;
using SixTensors = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor>;

bool verbose() {
  static const bool v = std::getenv("MIXEDGEMM_VERBOSE") != nullptr;
  return v;
}

void* current_stream(const Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

// Launch status, then device-wide synchronize, both mapped to runtime_error.
void finish(int launch_status, const char* what) {
  if (launch_status != MG_OK) {
    std::cerr << "GPU error after launching " << what << ": " << mg_status_string(launch_status) << std::endl;
    throw std::runtime_error(std::string("CUDA error in ") + what + ": " + mg_status_string(launch_status));
  }
  const int sync_status = mg_device_synchronize();
  if (sync_status != MG_OK) {
    std::cerr << "GPU error during/after " << what << " synchronization: " << mg_status_string(sync_status) << std::endl;
    throw std::runtime_error(std::string("CUDA sync error in ") + what + ": " + mg_status_string(sync_status));
  }
  if (verbose()) std::cout << what << " kernel finished and synced successfully." << std::endl;
}

Tensor bytes(const Tensor& like, std::initializer_list<int64_t> shape) {
  return torch::empty(shape, torch::dtype(torch::kUInt8).device(like.device()));
}

// uint8 [rows, cols] (or [n] when cols < 0) at the start of a larger allocation: the tensor has the
// reference's shape, its storage the room for whole 256-row tiles
Tensor roomy(const Tensor& like, int64_t alloc, int64_t shown, int64_t cols) {
  if (cols < 0) return bytes(like, {alloc < shown ? shown : alloc}).narrow(0, 0, shown);
  return bytes(like, {alloc < shown ? shown : alloc, cols}).narrow(0, 0, shown);
}

// bytes readable from the tensor's first element to the end of its storage
int64_t capacity(const Tensor& t) {
  return static_cast<int64_t>(t.storage().nbytes()) - t.storage_offset() * static_cast<int64_t>(t.element_size());
}

Tensor matmul(const Tensor& AN, const Tensor& BN, const Tensor& AS, const Tensor& BS, const Tensor& AO, const Tensor& BO,
              const Tensor& SFAN, const Tensor& SFBN, const Tensor& SFAS, const Tensor& SFBS, const Tensor& SFAO,
              const Tensor& SFBO) {
  // shapes recovered from the packed operands exactly as the reference does
  const int M = static_cast<int>(AN.size(0));
  const int N = static_cast<int>(BN.size(0));
  const int KN = static_cast<int>(AN.size(1)) * 2;
  const int KS = static_cast<int>(AS.size(1)) * 4 / 3;
  const int KO = static_cast<int>(AO.size(1));
  Tensor C = torch::zeros({M, N}, torch::dtype(torch::kBFloat16).device(AN.device()));
  // activation buffers that reorder_quantize_x of this module made have room for whole tiles
  const int R = mg_padded_rows(M);
  const bool room = capacity(AN) >= (int64_t)R * AN.size(1) && capacity(AS) >= (int64_t)R * AS.size(1) &&
                    capacity(AO) >= (int64_t)R * AO.size(1) &&
                    capacity(SFAN) >= (int64_t)mg_sf_bytes(R, KN, MG_OPERAND_A) &&
                    capacity(SFAS) >= (int64_t)mg_sf_bytes(R, KS, MG_OPERAND_A) &&
                    capacity(SFAO) >= (int64_t)mg_sf_bytes(R, KO, MG_OPERAND_A);
  const int status = mg_mixed_gemm_ex(AN.data_ptr<uint8_t>(), BN.data_ptr<uint8_t>(), AS.data_ptr<uint8_t>(),
                                        BS.data_ptr<uint8_t>(), AO.data_ptr<uint8_t>(), BO.data_ptr<uint8_t>(),
                                        SFAN.data_ptr<uint8_t>(), SFBN.data_ptr<uint8_t>(), SFAS.data_ptr<uint8_t>(),
                                        SFBS.data_ptr<uint8_t>(), SFAO.data_ptr<uint8_t>(), SFBO.data_ptr<uint8_t>(), M,
                                        room ? R : M, N, KN, KS, KO, 0u, C.data_ptr<at::BFloat16>(), current_stream(AN));
  finish(status, "GEMM");
  return C;
}

template <bool kWeights>
SixTensors reorder_quantize(const Tensor& T, const Tensor& reorder_index, int KN, int KS, int KO) {
  const char* what = kWeights ? "run_reorder_bf16_fp4" : "run_reorder_bf16_mixed";
  const int rows = static_cast<int>(T.size(0));
  const int K = KN + KS + KO;
  if (KN < 0 || KS < 0 || KO < 0 || ((KN | KS | KO) & 31) || K > 32736) {
    std::cerr << "K value is not valid !" << std::endl;
    throw std::runtime_error(std::string("Value error in ") + what + " ");
  }
  const int operand = kWeights ? MG_OPERAND_B : MG_OPERAND_A;
  const int R = kWeights ? rows : mg_padded_rows(rows);
  Tensor QN = roomy(T, R, rows, KN / 2);
  Tensor QS = roomy(T, R, rows, kWeights ? KS / 2 : KS / 4 * 3);
  Tensor QO = roomy(T, R, rows, kWeights ? KO / 2 : KO);
  Tensor SFN = roomy(T, static_cast<int64_t>(mg_sf_bytes(R, KN, operand)), static_cast<int64_t>(mg_sf_bytes(rows, KN, operand)), -1);
  Tensor SFS = roomy(T, static_cast<int64_t>(mg_sf_bytes(R, KS, operand)), static_cast<int64_t>(mg_sf_bytes(rows, KS, operand)), -1);
  Tensor SFO = roomy(T, static_cast<int64_t>(mg_sf_bytes(R, KO, operand)), static_cast<int64_t>(mg_sf_bytes(rows, KO, operand)), -1);
  auto* fn = kWeights ? &mg_reorder_quantize_w : &mg_reorder_quantize_x;
  const int status = fn(T.data_ptr<at::BFloat16>(), reorder_index.data_ptr<int16_t>(), rows, K, KN, KS, KO,
                        QN.data_ptr<uint8_t>(), QS.data_ptr<uint8_t>(), QO.data_ptr<uint8_t>(), SFN.data_ptr<uint8_t>(),
                        SFS.data_ptr<uint8_t>(), SFO.data_ptr<uint8_t>(), current_stream(T));
  finish(status, what);
  return std::make_tuple(QN, QS, QO, SFN, SFS, SFO);
}

// seqlen and outfeatures are accepted and ignored, as in the reference (rows come
// from the tensor; outfeatures only reached a layout call that does not use it).
SixTensors reorder_quantize_x(const Tensor& X, const Tensor& reorder_index, int KN, int KS, int KO, int /*seqlen*/,
                              int /*outfeatures*/) {
  return reorder_quantize<false>(X, reorder_index, KN, KS, KO);
}

SixTensors reorder_quantize_w(const Tensor& W, const Tensor& reorder_index, int KN, int KS, int KO, int /*seqlen*/,
                              int /*outfeatures*/) {
  return reorder_quantize<true>(W, reorder_index, KN, KS, KO);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("matmul", &matmul,
        "Mixed MXFP4/6/8 block-scaled GEMM: bf16 [M, N] = A @ B^T from the packed segment operands and their "
        "E8M0 scale buffers.",
        py::arg("AN"), py::arg("BN"), py::arg("AS"), py::arg("BS"), py::arg("AO"), py::arg("BO"), py::arg("SFAN"),
        py::arg("SFBN"), py::arg("SFAS"), py::arg("SFBS"), py::arg("SFAO"), py::arg("SFBO"));
  m.def("test_function", []() { return "Hello from test_function!"; });
  m.def("reorder_quantize_x", &reorder_quantize_x, "Reorder and quantize activation", py::arg("X"),
        py::arg("reorder_index"), py::arg("KN"), py::arg("KS"), py::arg("KO"), py::arg("seqlen"), py::arg("outfeatures"));
  m.def("reorder_quantize_w", &reorder_quantize_w, "Reorder and quantize weight", py::arg("W"),
        py::arg("reorder_index"), py::arg("KN"), py::arg("KS"), py::arg("KO"), py::arg("seqlen"), py::arg("outfeatures"));
}
