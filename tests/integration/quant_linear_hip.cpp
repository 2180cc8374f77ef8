// quant_linear_hip.cpp — built with torch.utils.cpp_extension, links -luniql_amd
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include "uniql_amd.h"

torch::Tensor w4a16o16_gemm(const torch::Tensor& A, const torch::Tensor& B, const torch::Tensor& s,
                            torch::Tensor& workspace, int64_t m, int64_t n, int64_t k,
                            bool output_transpose, int64_t, int64_t, int64_t, int64_t) {
  auto D = output_transpose ? torch::zeros({n, (m + 7) / 8 * 8}, A.options()) : torch::empty({m, n}, A.options());
  static thread_local torch::Tensor accum;          // zero between calls, one per stream in real code
  size_t need = uniql_w4a16_gemm_accum_bytes(m, n, k);
  if (!accum.defined() || (size_t)accum.nbytes() < need)
    accum = torch::zeros({(int64_t)need}, A.options().dtype(torch::kUInt8));
  size_t tmp = uniql_w4a16_gemm_temp_bytes(m, n, k, /*had_block=*/0);   // partial tiles when K is split
  auto temp = torch::empty({(int64_t)tmp}, A.options().dtype(torch::kUInt8));
  int rc = uniql_w4a16_gemm(A.data_ptr(), A.stride(0), B.data_ptr(), s.data_ptr(), D.data_ptr(),
                            workspace.data_ptr<int32_t>(), workspace.numel(),
                            accum.data_ptr(), accum.nbytes(), tmp ? temp.data_ptr() : nullptr, tmp,
                            m, n, k, s.size(0), /*had_block=*/0, 0.f,
                            /*flags=*/output_transpose ? UNIQL_F_TRANSPOSE_OUT : 0,
                            c10::hip::getCurrentHIPStream().stream());
  TORCH_CHECK(rc == 0, uniql_status_string(rc));
  return D;
}
PYBIND11_MODULE(quant_linear_cuda, m) { m.def("w4a16o16_gemm", &w4a16o16_gemm); }
