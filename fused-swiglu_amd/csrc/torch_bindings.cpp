// PyTorch-ROCm operator surface of `fused_mlp_module`, rebuilt on the C ABI of include/fsw.h.
//
// Kept from the reference (csrc/torch_bindings.cpp:31-50): the module name, the two pybind functions
// `fused_swiglu_bf16(X, W1W3)` and `swiglu_fwd_bf16(m, n, k, A, ldA, B, ldB, C, ldC)`, the dispatcher library
// `ASMLLM` with the same two schema strings, and the CUDA dispatch key (HIP tensors dispatch through it on
// PyTorch-ROCm). Added beside them, because the full MLP forward and the fp16 configuration need them:
// `fused_swiglu_fp16`, `swiglu_down_{bf16,fp16}`, `fused_swiglu_mlp_{bf16,fp16}`, and for the reference's build with
// a float output type (constants.cuh:9-14) `fused_swiglu_bf16_f32out` and a float C in `swiglu_fwd_bf16`.
//
// This file is plain host C++ (no device code, no CUDA spellings): torch is used for tensors, the device guard
// and the current stream only.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/all.h>
#include <torch/extension.h>

#include <algorithm>

#include "fsw.h"

namespace {

using at::Tensor;

void* current_stream() { return (void*)at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

int dtype_code(at::ScalarType t) { return t == at::kBFloat16 ? FSW_BF16 : FSW_FP16; }

void check_rc(int rc, const char* op) {
  TORCH_CHECK(rc == FSW_OK, op, ": ", fsw_strerror(rc), " (code ", rc, ", hip error ", fsw_last_hip_error(), ")");
}

void check_device_tensor(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), "Expected tensor ", name, " to be on the GPU, but got device ", t.device());
}

// swiglu_fwd<bf16,bf16,bf16> of the reference (swiglu.cu:397-525). n and ldC are the FULL N = 2*ff; the dense
// [m, n/2] result is written with row stride ldC/2 (swiglu.cu:408,414,353).
void swiglu_fwd_typed(at::ScalarType want, int64_t m, int64_t n, int64_t k, Tensor const& A, int64_t ldA,
                      Tensor const& B, int64_t ldB, Tensor& C, int64_t ldC) {
  // dtype guards as at swiglu.cu:475-480 (same failure mode: c10::Error -> RuntimeError)
  TORCH_CHECK(A.scalar_type() == want, "Expected tensor A to be of type ", want, ", but got: ", A.scalar_type());
  TORCH_CHECK(B.scalar_type() == want, "Expected tensor B to be of type ", want, ", but got: ", B.scalar_type());
  // C: the element type (the reference as shipped, C_TYPE bf16), or float: its other build (constants.cuh:9-14,
  // "C can work with either bf16 or fp32", swiglu.cu:470-471), which stores the gated fp32 value unrounded
  const bool c_f32 = C.scalar_type() == at::kFloat;
  TORCH_CHECK(C.scalar_type() == want || c_f32, "Expected tensor C to be of type ", want, " or ", at::kFloat,
              ", but got: ", C.scalar_type());
  check_device_tensor(A, "A");
  check_device_tensor(B, "B");
  check_device_tensor(C, "C");
  TORCH_CHECK(A.device() == B.device() && A.device() == C.device(), "A, B and C must live on the same device");
  TORCH_CHECK(m >= 0 && n >= 0 && k >= 0, "negative problem size");
  // the raw-pointer interface trusts m/n/k/ld*; bound them by what the tensors actually hold
  if (m > 0 && n > 0) {
    TORCH_CHECK(A.numel() >= (m - 1) * ldA + k, "tensor A is smaller than m x k with leading dimension ldA");
    TORCH_CHECK(B.numel() >= (n - 1) * ldB + k, "tensor B is smaller than n x k with leading dimension ldB");
    TORCH_CHECK(C.numel() >= (m - 1) * (ldC / 2) + n / 2, "tensor C is smaller than m x n/2 with row stride ldC/2");
  }
  const at::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(A));
  // like the reference's launcher this allocates nothing: the kernels read A and B where they lie
  const int rc = c_f32 ? fsw_gateup_f32out(dtype_code(want), m, n, k, A.data_ptr(), ldA, B.data_ptr(), ldB,
                                           (float*)C.data_ptr(), ldC / 2, current_stream())
                       : fsw_gateup(dtype_code(want), m, n, k, A.data_ptr(), ldA, B.data_ptr(), ldB, C.data_ptr(),
                                    ldC / 2, current_stream());
  check_rc(rc, "swiglu_fwd");
}

void swiglu_fwd_bf16(int64_t m, int64_t n, int64_t k, Tensor const& A, int64_t ldA, Tensor const& B, int64_t ldB,
                     Tensor& C, int64_t ldC) {
  swiglu_fwd_typed(at::kBFloat16, m, n, k, A, ldA, B, ldB, C, ldC);
}

// fused_swiglu_bf16 of the reference (swiglu.cu:538-553): shapes from the tensors, out[M, N/2] with X's options.
Tensor fused_swiglu_typed(at::ScalarType want, Tensor const& X, Tensor const& W1W3, bool f32_out = false) {
  TORCH_CHECK(X.dim() == 2 && W1W3.dim() == 2, "X and W1W3 must be 2-D");
  TORCH_CHECK(X.size(1) == W1W3.size(1), "X is [M, K] and W1W3 is [2*ff, K]: K differs (", X.size(1), " vs ",
              W1W3.size(1), ")");
  TORCH_CHECK(X.stride(1) == 1 || X.size(1) <= 1, "X must be K-contiguous");
  TORCH_CHECK(W1W3.stride(1) == 1 || W1W3.size(1) <= 1, "W1W3 must be K-contiguous");
  const int64_t M = X.size(0), N = W1W3.size(0), K = X.size(1);
  TORCH_CHECK(N % 2 == 0, "W1W3 must hold an even number of rows (interleaved up/gate pairs)");
  Tensor out = at::empty({M, N / 2}, X.options().dtype(f32_out ? at::kFloat : want));
  const int64_t ldx = M > 1 ? X.stride(0) : K;
  const int64_t ldw = N > 1 ? W1W3.stride(0) : K;
  swiglu_fwd_typed(want, M, N, K, X, ldx, W1W3, ldw, out, N);
  return out;
}

Tensor fused_swiglu_bf16(Tensor const& X, Tensor const& W1W3) { return fused_swiglu_typed(at::kBFloat16, X, W1W3); }
Tensor fused_swiglu_fp16(Tensor const& X, Tensor const& W1W3) { return fused_swiglu_typed(at::kHalf, X, W1W3); }
// fused_swiglu_bf16 as the reference's C_TYPE float build returns it: float32, no rounding of the gated value
Tensor fused_swiglu_bf16_f32out(Tensor const& X, Tensor const& W1W3) {
  return fused_swiglu_typed(at::kBFloat16, X, W1W3, true);
}

// Y[M, D] = H[M, FF] @ W2[D, FF].T  (no counterpart in the reference)
Tensor swiglu_down_typed(at::ScalarType want, Tensor const& H, Tensor const& W2) {
  TORCH_CHECK(H.scalar_type() == want, "Expected tensor H to be of type ", want, ", but got: ", H.scalar_type());
  TORCH_CHECK(W2.scalar_type() == want, "Expected tensor W2 to be of type ", want, ", but got: ", W2.scalar_type());
  check_device_tensor(H, "H");
  check_device_tensor(W2, "W2");
  TORCH_CHECK(H.device() == W2.device(), "H and W2 must live on the same device");
  TORCH_CHECK(H.dim() == 2 && W2.dim() == 2, "H and W2 must be 2-D");
  TORCH_CHECK(H.size(1) == W2.size(1), "H is [M, FF] and W2 is [D, FF]: FF differs");
  TORCH_CHECK(H.stride(1) == 1 || H.size(1) <= 1, "H must be FF-contiguous");
  TORCH_CHECK(W2.stride(1) == 1 || W2.size(1) <= 1, "W2 must be FF-contiguous");
  const int64_t M = H.size(0), FF = H.size(1), D = W2.size(0);
  Tensor Y = at::empty({M, D}, H.options());
  const int64_t ldh = M > 1 ? H.stride(0) : FF;
  const int64_t ldw = D > 1 ? W2.stride(0) : FF;
  const at::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(H));
  const int code = dtype_code(want);
  const size_t ws_bytes = fsw_down_workspace_bytes(code, M, D, FF);
  Tensor ws;
  if (ws_bytes > 0) ws = at::empty({(int64_t)ws_bytes}, H.options().dtype(at::kByte));
  const int rc = fsw_down(code, M, D, FF, H.data_ptr(), ldh, W2.data_ptr(), ldw, Y.data_ptr(), D,
                          ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream());
  check_rc(rc, "swiglu_down");
  return Y;
}

Tensor swiglu_down_bf16(Tensor const& H, Tensor const& W2) { return swiglu_down_typed(at::kBFloat16, H, W2); }
Tensor swiglu_down_fp16(Tensor const& H, Tensor const& W2) { return swiglu_down_typed(at::kHalf, H, W2); }

// Y = (silu(X @ Wg) * (X @ Wu)) @ Wd with W1W3 = interleaved [up; gate] rows and W2 = Wd^T.
Tensor fused_swiglu_mlp_typed(at::ScalarType want, Tensor const& X, Tensor const& W1W3, Tensor const& W2) {
  TORCH_CHECK(X.scalar_type() == want && W1W3.scalar_type() == want && W2.scalar_type() == want,
              "Expected tensors X, W1W3 and W2 to be of type ", want);
  check_device_tensor(X, "X");
  check_device_tensor(W1W3, "W1W3");
  check_device_tensor(W2, "W2");
  TORCH_CHECK(X.device() == W1W3.device() && X.device() == W2.device(), "X, W1W3 and W2 must live on the same device");
  TORCH_CHECK(X.dim() == 2 && W1W3.dim() == 2 && W2.dim() == 2, "X, W1W3 and W2 must be 2-D");
  const int64_t M = X.size(0), D = X.size(1), N = W1W3.size(0), FF = N / 2;
  TORCH_CHECK(N % 2 == 0 && W1W3.size(1) == D, "W1W3 must be [2*ff, d] for X [M, d]");
  TORCH_CHECK(W2.size(0) == D && W2.size(1) == FF, "W2 must be [d, ff]");
  TORCH_CHECK((X.stride(1) == 1 || D <= 1) && (W1W3.stride(1) == 1 || D <= 1) && (W2.stride(1) == 1 || FF <= 1),
              "X, W1W3 and W2 must be contiguous in their last dimension");
  Tensor Y = at::empty({M, D}, X.options());
  const at::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(X));
  const int code = dtype_code(want);
  // one call: H (panel-blocked for large problems) and the split-K partials live in this scratch, never as a tensor
  const size_t ws_bytes = fsw_mlp_workspace_bytes(code, M, D, FF);
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, X.options().dtype(at::kByte));
  const int rc = fsw_mlp(code, M, D, FF, X.data_ptr(), M > 1 ? X.stride(0) : D, W1W3.data_ptr(),
                         N > 1 ? W1W3.stride(0) : D, W2.data_ptr(), D > 1 ? W2.stride(0) : FF, Y.data_ptr(), D,
                         ws.data_ptr(), ws_bytes, current_stream());
  check_rc(rc, "fused_swiglu_mlp");
  return Y;
}

Tensor fused_swiglu_mlp_bf16(Tensor const& X, Tensor const& W1W3, Tensor const& W2) {
  return fused_swiglu_mlp_typed(at::kBFloat16, X, W1W3, W2);
}
Tensor fused_swiglu_mlp_fp16(Tensor const& X, Tensor const& W1W3, Tensor const& W2) {
  return fused_swiglu_mlp_typed(at::kHalf, X, W1W3, W2);
}

// ---- shape-only ("meta") implementations: let the ops trace under torch.compile / FakeTensor without a GPU.
// The reference registers no such kernels and its swiglu_fwd_bf16 schema hides that C is written
// (torch_bindings.cpp:42); `swiglu_fwd_bf16_out` below is the same call with the mutation declared.
Tensor meta_gateup(at::ScalarType want, Tensor const& X, Tensor const& W1W3) {
  TORCH_CHECK(X.scalar_type() == want, "Expected tensor A to be of type ", want, ", but got: ", X.scalar_type());
  TORCH_CHECK(W1W3.scalar_type() == want, "Expected tensor B to be of type ", want, ", but got: ", W1W3.scalar_type());
  TORCH_CHECK(X.dim() == 2 && W1W3.dim() == 2 && X.size(1) == W1W3.size(1) && W1W3.size(0) % 2 == 0,
              "X is [M, K] and W1W3 is [2*ff, K]");
  return at::empty({X.size(0), W1W3.size(0) / 2}, X.options());
}
Tensor meta_down(at::ScalarType want, Tensor const& H, Tensor const& W2) {
  TORCH_CHECK(H.scalar_type() == want && W2.scalar_type() == want, "Expected tensors of type ", want);
  TORCH_CHECK(H.dim() == 2 && W2.dim() == 2 && H.size(1) == W2.size(1), "H is [M, FF] and W2 is [D, FF]");
  return at::empty({H.size(0), W2.size(0)}, H.options());
}
Tensor meta_fused_swiglu_bf16(Tensor const& X, Tensor const& W) { return meta_gateup(at::kBFloat16, X, W); }
Tensor meta_fused_swiglu_fp16(Tensor const& X, Tensor const& W) { return meta_gateup(at::kHalf, X, W); }
Tensor meta_fused_swiglu_bf16_f32out(Tensor const& X, Tensor const& W) {
  return meta_gateup(at::kBFloat16, X, W).to(at::kFloat);
}
Tensor meta_down_bf16(Tensor const& H, Tensor const& W2) { return meta_down(at::kBFloat16, H, W2); }
Tensor meta_down_fp16(Tensor const& H, Tensor const& W2) { return meta_down(at::kHalf, H, W2); }
Tensor meta_mlp_bf16(Tensor const& X, Tensor const& W, Tensor const& W2) {
  return meta_down(at::kBFloat16, meta_gateup(at::kBFloat16, X, W), W2);
}
Tensor meta_mlp_fp16(Tensor const& X, Tensor const& W, Tensor const& W2) {
  return meta_down(at::kHalf, meta_gateup(at::kHalf, X, W), W2);
}
void meta_swiglu_fwd_bf16(int64_t, int64_t, int64_t, Tensor const&, int64_t, Tensor const&, int64_t, Tensor&, int64_t) {}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("fused_swiglu_bf16", &fused_swiglu_bf16, "fused SwiGLU for bf16");
  m.def("swiglu_fwd_bf16", &swiglu_fwd_bf16, "SwiGLU fwd bf16");
  // additions
  m.def("fused_swiglu_fp16", &fused_swiglu_fp16, "fused SwiGLU for fp16");
  m.def("fused_swiglu_bf16_f32out", &fused_swiglu_bf16_f32out, "fused SwiGLU for bf16 inputs, float32 output");
  m.def("swiglu_down_bf16", &swiglu_down_bf16, "down projection H @ W2.T, bf16");
  m.def("swiglu_down_fp16", &swiglu_down_fp16, "down projection H @ W2.T, fp16");
  m.def("fused_swiglu_mlp_bf16", &fused_swiglu_mlp_bf16, "full SwiGLU MLP forward, bf16");
  m.def("fused_swiglu_mlp_fp16", &fused_swiglu_mlp_fp16, "full SwiGLU MLP forward, fp16");
  m.def("variant_name", [](int family, int64_t M, int64_t n, int64_t k) {
    return std::string(fsw_variant_name(family, FSW_BF16, M, n, k));
  }, "kernel variant the dispatcher picks (family 0 = gate/up, 1 = down)");
}

TORCH_LIBRARY(ASMLLM, m) {
  m.def("fused_swiglu_bf16(Tensor X, Tensor W1W3) -> Tensor");
  m.def("swiglu_fwd_bf16(int m, int n, int k, Tensor A, int ldA, Tensor B, int ldB, Tensor C, int ldC) -> ()");
  // additions
  m.def("fused_swiglu_fp16(Tensor X, Tensor W1W3) -> Tensor");
  m.def("fused_swiglu_bf16_f32out(Tensor X, Tensor W1W3) -> Tensor");
  m.def("swiglu_down_bf16(Tensor H, Tensor W2) -> Tensor");
  m.def("swiglu_down_fp16(Tensor H, Tensor W2) -> Tensor");
  m.def("fused_swiglu_mlp_bf16(Tensor X, Tensor W1W3, Tensor W2) -> Tensor");
  m.def("fused_swiglu_mlp_fp16(Tensor X, Tensor W1W3, Tensor W2) -> Tensor");
  // swiglu_fwd_bf16 with the write to C declared, for tracing compilers
  m.def("swiglu_fwd_bf16_out(int m, int n, int k, Tensor A, int ldA, Tensor B, int ldB, Tensor(a!) C, int ldC) -> ()");
}

TORCH_LIBRARY_IMPL(ASMLLM, CUDA, m) {
  m.impl("fused_swiglu_bf16", &fused_swiglu_bf16);
  m.impl("swiglu_fwd_bf16", &swiglu_fwd_bf16);
  m.impl("fused_swiglu_fp16", &fused_swiglu_fp16);
  m.impl("fused_swiglu_bf16_f32out", &fused_swiglu_bf16_f32out);
  m.impl("swiglu_down_bf16", &swiglu_down_bf16);
  m.impl("swiglu_down_fp16", &swiglu_down_fp16);
  m.impl("fused_swiglu_mlp_bf16", &fused_swiglu_mlp_bf16);
  m.impl("fused_swiglu_mlp_fp16", &fused_swiglu_mlp_fp16);
  m.impl("swiglu_fwd_bf16_out", &swiglu_fwd_bf16);
}

TORCH_LIBRARY_IMPL(ASMLLM, Meta, m) {
  m.impl("fused_swiglu_bf16", &meta_fused_swiglu_bf16);
  m.impl("fused_swiglu_fp16", &meta_fused_swiglu_fp16);
  m.impl("fused_swiglu_bf16_f32out", &meta_fused_swiglu_bf16_f32out);
  m.impl("swiglu_down_bf16", &meta_down_bf16);
  m.impl("swiglu_down_fp16", &meta_down_fp16);
  m.impl("fused_swiglu_mlp_bf16", &meta_mlp_bf16);
  m.impl("fused_swiglu_mlp_fp16", &meta_mlp_fp16);
  m.impl("swiglu_fwd_bf16", &meta_swiglu_fwd_bf16);
  m.impl("swiglu_fwd_bf16_out", &meta_swiglu_fwd_bf16);
}
