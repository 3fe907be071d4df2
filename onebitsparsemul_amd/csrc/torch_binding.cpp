// pybind11 / ATen binding `onebit_sparse_cuda.onebit_mul(A, B, meta, C)`.
// Same module name, function name, positional order and docstring as the reference binding
// (onebit_sparse_mul/torch_kernel_cuda.cpp:10-38; module name from setup.py:14). The reference derives
// m and k from A's shape, which matches none of the layouts its own Python side produces, and raises when
// the shapes agree (:13-18); here the problem size comes from the operands' defined shapes and every
// mismatch raises a Python exception:
//   A    uint8  (k/2, m/8)   one-bit values as written by BinaryLinear_2_4.pack()
//   B    fp16   (k, n)       contiguous
//   meta int16  (m, k/16)    reordered metadata
//   C    fp32 or fp16 (m, n) destination (the reference passes it as both source and destination, :23-24)
// The work is enqueued on PyTorch's current HIP stream of C's device.
#include <torch/extension.h>
// PyTorch on ROCm presents its devices as type "cuda"; these are the guard and stream accessors for that.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "onebit_sparse_tensor.h"

namespace {

void check_operand(const torch::Tensor& t, const char* name, c10::ScalarType dtype, const c10::Device& device) {
  TORCH_CHECK(t.device() == device, name, " must be on ", device, ", got ", t.device());
  TORCH_CHECK(t.scalar_type() == dtype, name, " must have dtype ", dtype, ", got ", t.scalar_type());
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

void onebit_mul(const torch::Tensor& A, const torch::Tensor& B, const torch::Tensor& meta, torch::Tensor& C) {
  TORCH_CHECK(C.is_cuda(), "C must be a GPU tensor");
  TORCH_CHECK(meta.dim() == 2 && B.dim() == 2 && C.dim() == 2, "meta, B and C must be 2-dimensional");
  const c10::Device device = C.device();
  check_operand(A, "A", torch::kUInt8, device);
  check_operand(B, "B", torch::kFloat16, device);
  check_operand(meta, "meta", torch::kInt16, device);
  TORCH_CHECK(C.scalar_type() == torch::kFloat32 || C.scalar_type() == torch::kFloat16,
              "C must be float32 or float16, got ", C.scalar_type());
  TORCH_CHECK(C.is_contiguous(), "C must be contiguous");

  const int64_t prob_m = meta.size(0);
  const int64_t prob_k = meta.size(1) * 16;
  const int64_t prob_n = B.size(1);
  TORCH_CHECK(A.numel() == prob_m * prob_k / 16, "A holds ", A.numel(), " bytes, expected m*k/16 = ",
              prob_m * prob_k / 16, " for meta of shape (", prob_m, ", ", meta.size(1), ")");
  TORCH_CHECK(B.size(0) == prob_k, "B.size(0) = ", B.size(0), " != k = ", prob_k);
  TORCH_CHECK(C.size(0) == prob_m && C.size(1) == prob_n, "C must have shape (", prob_m, ", ", prob_n, ")");
  TORCH_CHECK(prob_m < (1ll << 31) && prob_n < (1ll << 31) && prob_k < (1ll << 31), "problem size exceeds int range");

  const c10::hip::HIPGuardMasqueradingAsCUDA guard(device);
  void* stream = static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device.index()).stream());
  const int d_dtype = C.scalar_type() == torch::kFloat16 ? ONEBIT_DTYPE_F16 : ONEBIT_DTYPE_F32;
  const int rc = onebit_sparse_matmul_ex(A.data_ptr(), B.data_ptr(), C.data_ptr(), C.data_ptr(), meta.data_ptr(),
                                         (int)prob_m, (int)prob_n, (int)prob_k, 1.0f, 0.0f, d_dtype, d_dtype,
                                         ONEBIT_META_REFERENCE, stream);
  TORCH_CHECK(rc == ONEBIT_OK, "onebit_sparse_matmul_ex failed: ", onebit_sparse_last_error());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("onebit_mul", &onebit_mul, "A32 = Sparse W1 * A16 matmul.");
}
