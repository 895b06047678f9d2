// PyTorch binding: module `attention_cutlass_fp8`, function `flash_attention_v2_cutlass`.
//
// Drop-in for the reference extension (reference csrc/attention_api.cpp:6-10, declaration
// include/attention_api.h:10-11, host body csrc/flash_attention.cu:639-668): same module and function
// name, same five leading arguments (q, k, v, is_causal, softmax_scale), returns a one-element list.
// Host C++ only: all GPU work goes through the C ABI of libfa8.so (include/fa8_api.h).
//
// Deliberate differences from the reference host code:
//   * v is [B,H,N,d] like k by default; `v_transposed=True` takes the reference's [B,H,d,N] (test.py:71);
//   * O is fp16 by default; `out_dtype=q.dtype` gives the reference's fp8 O in the input element type (:557, :656);
//   * the kernel runs on torch's current stream and the call does not synchronise the device (:661-665);
//   * bad arguments and HIP errors raise RuntimeError instead of printf + exit (include/attention_api.cuh:20-29).
// Additions the reference declares but never implements (csrc/flash.h:36-45,56): k/v may have fewer heads than q
// (grouped-query attention), `return_lse=True` appends the fp32 log-sum-exp [B,H,Nq] to the returned list, and
// `causal_bottom_right=True` aligns the causal diagonal with the last key when seqlen_q != seqlen_k.  `schedule`
// (FA8_SCHEDULE_*, include/fa8_api.h) picks the kernel's main loop by hand: a performance hint, the result is the same.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <vector>

#include "fa8_api.h"

namespace {

void check_input(const torch::Tensor& t, const char* name) {
  // same two conditions as the reference CHECK_INPUT (include/attention_api.cuh:12-18)
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.dim() == 4, name, " must be 4-dimensional [batch, heads, seqlen, head_dim], got ", t.dim(), " dims");
}

}  // namespace

std::vector<torch::Tensor> flash_attention_v2_cutlass(torch::Tensor q, torch::Tensor k, torch::Tensor v, bool is_causal,
                                                      float softmax_scale, bool v_transposed,
                                                      c10::optional<at::ScalarType> out_dtype, bool return_lse,
                                                      bool causal_bottom_right, int64_t schedule) {
  check_input(q, "q");
  check_input(k, "k");
  check_input(v, "v");
  const auto in_type = q.scalar_type();
  TORCH_CHECK(in_type == at::kFloat8_e4m3fn || in_type == at::kFloat8_e5m2,
              "q must be torch.float8_e4m3fn or torch.float8_e5m2 (OCP fp8), got ", in_type);
  TORCH_CHECK(k.scalar_type() == in_type && v.scalar_type() == in_type, "q, k and v must have the same dtype");
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "q, k and v must be on the same device");
  const int64_t B = q.size(0), H = q.size(1), Nq = q.size(2), D = q.size(3);
  const int64_t Nk = k.size(2), Hk = k.size(1);
  TORCH_CHECK(k.size(0) == B && k.size(3) == D, "k must be [", B, ", heads_k, seqlen_k, ", D, "], got ", k.sizes());
  TORCH_CHECK(Hk >= 1 && H % Hk == 0, "the number of q heads (", H, ") must be a multiple of the number of k/v heads (", Hk, ")");
  if (v_transposed) {
    TORCH_CHECK(v.size(0) == B && v.size(1) == Hk && v.size(2) == D && v.size(3) == Nk, "v (transposed) must be [", B, ", ",
                Hk, ", ", D, ", ", Nk, "], got ", v.sizes());
  } else {
    TORCH_CHECK(v.size(0) == B && v.size(1) == Hk && v.size(2) == Nk && v.size(3) == D, "v must be [", B, ", ", Hk, ", ", Nk,
                ", ", D, "], got ", v.sizes());
  }
  TORCH_CHECK(B >= 1 && H >= 1 && Nq >= 1 && Nk >= 1, "empty tensors are not supported");
  TORCH_CHECK(Nq <= INT32_MAX && Nk <= INT32_MAX && B <= INT32_MAX && H <= INT32_MAX, "tensor too large");
  const at::ScalarType o_type = out_dtype.value_or(at::kHalf);
  TORCH_CHECK(o_type == at::kHalf || o_type == in_type,
              "out_dtype must be torch.float16 or the fp8 type of the inputs (the reference's output type), got ", o_type);

  auto out = torch::empty({B, H, Nq, D}, q.options().dtype(o_type));
  torch::Tensor lse;
  if (return_lse) lse = torch::empty({B, H, Nq}, q.options().dtype(at::kFloat));

  Fa8FwdParams p = {};
  p.q = q.data_ptr();
  p.k = k.data_ptr();
  p.v = v.data_ptr();
  p.o = out.data_ptr();
  p.batch = (int32_t)B;
  p.heads = (int32_t)H;
  p.seqlen_q = (int32_t)Nq;
  p.seqlen_k = (int32_t)Nk;
  p.head_dim = (int32_t)D;
  p.is_causal = is_causal ? 1 : 0;
  p.in_dtype = in_type == at::kFloat8_e5m2 ? FA8_DTYPE_E5M2 : FA8_DTYPE_E4M3;
  p.out_dtype = o_type == at::kHalf ? FA8_OUT_FP16 : (o_type == at::kFloat8_e5m2 ? FA8_OUT_E5M2 : FA8_OUT_E4M3);
  p.v_layout = v_transposed ? FA8_V_TRANSPOSED : FA8_V_ROWS;
  p.softmax_scale = softmax_scale;
  p.q_batch_stride = q.stride(0); p.q_head_stride = q.stride(1); p.q_row_stride = q.stride(2);
  p.k_batch_stride = k.stride(0); p.k_head_stride = k.stride(1); p.k_row_stride = k.stride(2);
  p.v_batch_stride = v.stride(0); p.v_head_stride = v.stride(1); p.v_row_stride = v.stride(2);
  p.o_batch_stride = out.stride(0); p.o_head_stride = out.stride(1); p.o_row_stride = out.stride(2);
  p.heads_k = (int32_t)Hk;
  p.causal_align = causal_bottom_right ? FA8_CAUSAL_BOTTOM_RIGHT : FA8_CAUSAL_TOP_LEFT;
  TORCH_CHECK(schedule >= FA8_SCHEDULE_AUTO && schedule <= FA8_SCHEDULE_DENSE, "schedule must be one of the FA8_SCHEDULE_* codes 0..",
              FA8_SCHEDULE_DENSE, ", got ", schedule);
  p.schedule = (int32_t)schedule;
  if (return_lse) {
    p.lse = lse.data_ptr();
    p.lse_batch_stride = lse.stride(0);
    p.lse_head_stride = lse.stride(1);
  }

  // PyTorch-ROCm presents HIP devices under the "cuda" device type; these are its guard and stream for them.
  const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(q.device());
  const hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
  const int rc = fa8_fwd(&p, (void*)stream);
  TORCH_CHECK(rc == FA8_OK, "flash_attention_v2_cutlass: ", fa8_error_string(rc), " (code ", rc, ")");
  if (return_lse) return {out, lse};
  return {out};
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "FP8 flash-attention forward for AMD MI355X (gfx950)";
  m.def("flash_attention_v2_cutlass", &flash_attention_v2_cutlass,
        "FP8 flash attention forward: fp8 q/k/v [B,H,N,d] -> [O] (fp16 by default)", py::arg("q"), py::arg("k"),
        py::arg("v"), py::arg("is_causal"), py::arg("softmax_scale"), py::kw_only(), py::arg("v_transposed") = false,
        py::arg("out_dtype") = py::none(), py::arg("return_lse") = false, py::arg("causal_bottom_right") = false,
        py::arg("schedule") = 0);
  m.def("kv_block", []() { return fa8_query(FA8_QUERY_KV_BLOCK); }, "kv rows per online-softmax step of the kernel");
}
