// Python module gemm_kernels._C: the thin PyTorch boundary over the C ABI in mi355_gemm.h.
//
// Keeps the reference's module name, function name, keyword names and return value
// (kernels/gemm_kernels/__init__.cpp:4-9: m.def("gemm_tn_test", ..., arg("A"), arg("B"),
// arg("C")) returning the C tensor) and the argument checks of its host launcher
// (kernels/gemm_kernels/sm90a/gemm_test.cu:15-41).  Differences, all supersets: fp16 inputs are
// accepted as well as bf16, C is validated, shapes need not be multiples of the tile, and the
// launch goes to torch's current stream of A's device instead of the legacy default stream
// (gemm_test.cu:82-85).  Every check that does not need a GPU runs before the first HIP call.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <string>

#include "../../include/mi355_gemm.h"

namespace {

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kBFloat16: return MI355_BF16;
    case at::kHalf: return MI355_F16;
    case at::kFloat8_e4m3fn: return MI355_E4M3;
    default: return -1;
  }
}

int variant_code(const std::string& v) {
  if (v == "auto") return MI355_VARIANT_AUTO;
  if (v == "basic") return MI355_VARIANT_BASIC;
  if (v == "pingpong") return MI355_VARIANT_PINGPONG;
  if (v == "skinny") return MI355_VARIANT_SKINNY;
  if (v == "simple") return MI355_VARIANT_SIMPLE;
  if (v == "alternate") return MI355_VARIANT_ALTERNATE;
  TORCH_CHECK(false, "unknown variant '", v, "' (expected auto, basic, pingpong, alternate, skinny or simple)");
}

const char* variant_name(int v) {
  switch (v) {
    case MI355_VARIANT_AUTO: return "auto";
    case MI355_VARIANT_BASIC: return "basic";
    case MI355_VARIANT_PINGPONG: return "pingpong";
    case MI355_VARIANT_SKINNY: return "skinny";
    case MI355_VARIANT_SIMPLE: return "simple";
    case MI355_VARIANT_ALTERNATE: return "alternate";
  }
  return "?";
}

// A scale given as a one-element tensor on the GEMM's device is passed by address (no host
// synchronisation); a Python number or a CPU tensor is folded into the scalar factor.
struct Scale {
  float host = 1.0f;
  const float* device = nullptr;
  torch::Tensor keep;
};

torch::Tensor run(const torch::Tensor& A, const torch::Tensor& B, torch::Tensor C, float scale,
                  int variant, bool fp8, const Scale& sa = Scale(), const Scale& sb = Scale()) {
  // Same order as the reference's checks (gemm_test.cu:15-28), then the ones it lacks.
  TORCH_CHECK(A.device() == B.device(), "All tensors must be on the same device");
  TORCH_CHECK(A.is_contiguous() && B.is_contiguous(), "All tensors must be contiguous");
  TORCH_CHECK(A.dim() == 2 && B.dim() == 2, "Both tensors must be 2D (matrix) tensors");
  TORCH_CHECK(A.size(1) == B.size(1), "Inner dimensions of A and B must match (A: ", A.size(1),
              ", B: ", B.size(1), ")");
  TORCH_CHECK(A.scalar_type() == B.scalar_type(), "A and B must have the same dtype");
  const int in_dt = dtype_code(A.scalar_type());
  if (fp8) {
    TORCH_CHECK(in_dt == MI355_E4M3, "Both tensors must be of type float8_e4m3fn");
  } else {
    TORCH_CHECK(in_dt == MI355_BF16 || in_dt == MI355_F16,
                "Both tensors must be of type bfloat16 or float16");
  }
  const int64_t M = A.size(0), N = B.size(0), K = A.size(1);
  TORCH_CHECK(C.dim() == 2 && C.size(0) == M && C.size(1) == N, "C must have shape (", M, ", ", N, ")");
  TORCH_CHECK(C.device() == A.device(), "All tensors must be on the same device");
  const int out_dt = dtype_code(C.scalar_type());
  if (fp8) {
    TORCH_CHECK(out_dt == MI355_BF16 || out_dt == MI355_F16, "C must be bfloat16 or float16");
  } else {
    TORCH_CHECK(out_dt == in_dt, "C must have the dtype of A and B");
  }
  TORCH_CHECK(N <= 1 || C.stride(1) == 1, "C must be contiguous in its last dimension");
  const int64_t ldc = M > 1 ? C.stride(0) : N;
  int st = mi355_gemm_check(M, N, K, K, K, ldc, in_dt, out_dt, variant);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st), " [M=", M, " N=", N,
              " K=", K, " variant=", variant_name(variant), "]");
  TORCH_CHECK(A.is_cuda(), "gemm_kernels runs on a HIP device only; got tensors on ", A.device());

  if (M == 0 || N == 0) return C;
  c10::DeviceGuard guard(A.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(A.device().index()).stream();
  const size_t ws_bytes = mi355_gemm_workspace_bytes(M, N, K, in_dt, variant);
  torch::Tensor ws;
  void* ws_ptr = nullptr;
  if (ws_bytes) {
    // From torch's caching allocator, so the memory is stream-ordered with the launch below.
    ws = torch::empty({(int64_t)ws_bytes}, A.options().dtype(torch::kUInt8));
    ws_ptr = ws.data_ptr();
  }
  st = mi355_gemm_tn_scaled(A.const_data_ptr(), B.const_data_ptr(), C.mutable_data_ptr(), M, N, K, K, K,
                            ldc, in_dt, out_dt, scale * sa.host * sb.host, sa.device, sb.device, variant,
                            ws_ptr, ws_bytes, (void*)stream);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st));
  return C;
}

Scale scale_of(const pybind11::object& o, const torch::Tensor& like) {
  Scale s;
  if (THPVariable_Check(o.ptr())) {
    const torch::Tensor& t = THPVariable_Unpack(o.ptr());
    TORCH_CHECK(t.numel() == 1, "a scale tensor must hold exactly one element");
    if (t.is_cuda() && t.device() == like.device() && t.scalar_type() == at::kFloat) {
      s.keep = t;
      s.device = t.const_data_ptr<float>();
    } else {
      s.host = t.item<float>();
    }
  } else {
    s.host = o.cast<float>();
  }
  return s;
}

}  // namespace

namespace test {

// C = A · B^T, A (M,K) and B (N,K) contiguous bf16 or fp16, C (M,N) of the same dtype.
torch::Tensor gemm_tn_test(const torch::Tensor A, const torch::Tensor B, torch::Tensor C) {
  return run(A, B, C, 1.0f, MI355_VARIANT_AUTO, false);
}

torch::Tensor gemm_tn(const torch::Tensor A, const torch::Tensor B, torch::Tensor C,
                      const std::string& variant) {
  return run(A, B, C, 1.0f, variant_code(variant), false);
}

// C = (scale_a*scale_b) * A_q · B_q^T for per-tensor-scaled float8_e4m3fn operands.
torch::Tensor gemm_tn_fp8(const torch::Tensor A_q, const torch::Tensor B_q, pybind11::object scale_a,
                          pybind11::object scale_b, torch::Tensor C, const std::string& variant) {
  return run(A_q, B_q, C, 1.0f, variant_code(variant), true, scale_of(scale_a, A_q), scale_of(scale_b, A_q));
}

// (x_q, scale): x_q float8_e4m3fn of x's shape, scale a 0-dim fp32 tensor on x's device, with
// x ~= scale * x_q, scale = amax|x| / 448.  No host synchronisation.
std::pair<torch::Tensor, torch::Tensor> quantize_e4m3(const torch::Tensor x) {
  TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
  int dt;
  switch (x.scalar_type()) {
    case at::kBFloat16: dt = MI355_BF16; break;
    case at::kHalf: dt = MI355_F16; break;
    case at::kFloat: dt = MI355_F32; break;
    default: TORCH_CHECK(false, "x must be bfloat16, float16 or float32");
  }
  TORCH_CHECK(x.is_cuda(), "gemm_kernels runs on a HIP device only; got a tensor on ", x.device());
  c10::DeviceGuard guard(x.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  torch::Tensor q = torch::empty(x.sizes(), x.options().dtype(at::kFloat8_e4m3fn));
  torch::Tensor sa = torch::empty({2}, x.options().dtype(at::kFloat));
  int st = mi355_quantize_e4m3(x.const_data_ptr(), dt, x.numel(), q.mutable_data_ptr(), sa.data_ptr<float>(),
                               (void*)stream);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st));
  return {q, sa[0]};
}

// Scale bytes of an MX operand: a uint8 (or float8_e8m0fnu) tensor (rows, K/32), rows contiguous.
const uint8_t* mx_scale_ptr(const torch::Tensor& s, const torch::Tensor& x, const char* name) {
  TORCH_CHECK(s.scalar_type() == at::kByte || s.scalar_type() == at::kFloat8_e8m0fnu, name,
              " must be uint8 or float8_e8m0fnu (E8M0 scale bytes)");
  TORCH_CHECK(s.dim() == 2 && s.size(0) == x.size(0) && s.size(1) * 32 == x.size(1), name,
              " must have shape (rows, K/32) = (", x.size(0), ", ", x.size(1) / 32, ")");
  TORCH_CHECK(s.device() == x.device(), "All tensors must be on the same device");
  TORCH_CHECK(s.size(1) <= 1 || s.stride(1) == 1, name, " must be contiguous in its last dimension");
  return (const uint8_t*)s.const_data_ptr();
}

// C = A · B^T for MX-quantised operands: A_q, B_q float8_e4m3fn (M,K), (N,K); scale_a, scale_b
// E8M0 bytes (M,K/32), (N,K/32); C bf16 or fp16.
// With scales_shuffled the scale tensors are outputs of shuffle_mx_scales (flat uint8).
torch::Tensor gemm_tn_mxfp8(const torch::Tensor A_q, const torch::Tensor B_q, const torch::Tensor scale_a,
                            const torch::Tensor scale_b, torch::Tensor C, bool scales_shuffled) {
  TORCH_CHECK(A_q.device() == B_q.device(), "All tensors must be on the same device");
  TORCH_CHECK(A_q.is_contiguous() && B_q.is_contiguous(), "All tensors must be contiguous");
  TORCH_CHECK(A_q.dim() == 2 && B_q.dim() == 2, "Both tensors must be 2D (matrix) tensors");
  TORCH_CHECK(A_q.size(1) == B_q.size(1), "Inner dimensions of A and B must match (A: ", A_q.size(1),
              ", B: ", B_q.size(1), ")");
  TORCH_CHECK(A_q.scalar_type() == at::kFloat8_e4m3fn && B_q.scalar_type() == at::kFloat8_e4m3fn,
              "Both tensors must be of type float8_e4m3fn");
  const int64_t M = A_q.size(0), N = B_q.size(0), K = A_q.size(1);
  TORCH_CHECK(K % 32 == 0, "K must be a multiple of the MX block (32); the kernel needs K % 128 == 0");
  TORCH_CHECK(C.dim() == 2 && C.size(0) == M && C.size(1) == N, "C must have shape (", M, ", ", N, ")");
  TORCH_CHECK(C.device() == A_q.device(), "All tensors must be on the same device");
  const int out_dt = dtype_code(C.scalar_type());
  TORCH_CHECK(out_dt == MI355_BF16 || out_dt == MI355_F16, "C must be bfloat16 or float16");
  TORCH_CHECK(N <= 1 || C.stride(1) == 1, "C must be contiguous in its last dimension");
  const int64_t ldc = M > 1 ? C.stride(0) : N;
  int st = mi355_gemm_mx_check(M, N, K, K, K, ldc, out_dt);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st), " [mxfp8 M=", M, " N=", N, " K=", K, "]");
  TORCH_CHECK(A_q.is_cuda(), "gemm_kernels runs on a HIP device only; got tensors on ", A_q.device());
  if (M == 0 || N == 0) return C;
  c10::DeviceGuard guard(A_q.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(A_q.device().index()).stream();
  const uint8_t *sa, *sb;
  if (scales_shuffled) {
    auto shuffled = [&](const torch::Tensor& t, int64_t rows, const char* name) {
      TORCH_CHECK(t.scalar_type() == at::kByte && t.dim() == 1 && t.is_contiguous() && t.device() == A_q.device() &&
                      (size_t)t.numel() == mi355_mx_shuffled_bytes(rows, K),
                  name, " must be the output of shuffle_mx_scales for this operand");
      return (const uint8_t*)t.const_data_ptr();
    };
    sa = shuffled(scale_a, M, "scale_a");
    sb = shuffled(scale_b, N, "scale_b");
  } else {
    sa = mx_scale_ptr(scale_a, A_q, "scale_a");
    sb = mx_scale_ptr(scale_b, B_q, "scale_b");
  }
  const size_t ws_bytes = mi355_gemm_mx_workspace_bytes(M, N, K, scales_shuffled ? 1 : 0);
  torch::Tensor ws;
  void* ws_ptr = nullptr;
  if (ws_bytes) {
    ws = torch::empty({(int64_t)ws_bytes}, A_q.options().dtype(torch::kUInt8));
    ws_ptr = ws.data_ptr();
  }
  st = mi355_gemm_tn_mxfp8(A_q.const_data_ptr(), B_q.const_data_ptr(), C.mutable_data_ptr(), M, N, K, K, K, ldc, sa,
                           !scales_shuffled && M > 1 ? scale_a.stride(0) : K / 32, sb,
                           !scales_shuffled && N > 1 ? scale_b.stride(0) : K / 32, scales_shuffled ? 1 : 0, out_dt,
                           ws_ptr, ws_bytes, (void*)stream);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st));
  return C;
}

// Scale bytes (rows, K/32) of one operand -> the layout the kernel reads (a flat uint8 tensor); do
// it once for weights and pass scales_shuffled=True to gemm_tn_mxfp8.
torch::Tensor shuffle_mx_scales(const torch::Tensor scales) {
  TORCH_CHECK(scales.scalar_type() == at::kByte || scales.scalar_type() == at::kFloat8_e8m0fnu,
              "scales must be uint8 or float8_e8m0fnu");
  TORCH_CHECK(scales.dim() == 2 && (scales.size(1) <= 1 || scales.stride(1) == 1), "scales must be (rows, K/32), rows contiguous");
  const int64_t rows = scales.size(0), K = scales.size(1) * 32;
  TORCH_CHECK(K % 128 == 0, "K must be a multiple of 128");
  TORCH_CHECK(scales.is_cuda(), "gemm_kernels runs on a HIP device only; got a tensor on ", scales.device());
  c10::DeviceGuard guard(scales.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(scales.device().index()).stream();
  torch::Tensor out = torch::empty({(int64_t)mi355_mx_shuffled_bytes(rows, K)}, scales.options().dtype(at::kByte));
  int st = mi355_mx_shuffle_scales((const uint8_t*)scales.const_data_ptr(), rows, K, rows > 1 ? scales.stride(0) : K / 32,
                                   out.data_ptr<uint8_t>(), (void*)stream);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st));
  return out;
}

// (x_q, scales): x (rows, K) -> float8_e4m3fn (rows, K) and uint8 E8M0 scale bytes (rows, K/32),
// one per 32 consecutive elements of a row, x ~= x_q * 2^(scales - 127).
// With shuffled the scales come back flat, in the layout gemm_tn_mxfp8(..., scales_shuffled=True) takes.
std::pair<torch::Tensor, torch::Tensor> quantize_mxfp8(const torch::Tensor x, bool shuffled) {
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "x must be a contiguous 2D tensor");
  int dt;
  switch (x.scalar_type()) {
    case at::kBFloat16: dt = MI355_BF16; break;
    case at::kHalf: dt = MI355_F16; break;
    case at::kFloat: dt = MI355_F32; break;
    default: TORCH_CHECK(false, "x must be bfloat16, float16 or float32");
  }
  const int64_t rows = x.size(0), K = x.size(1);
  TORCH_CHECK(K % 32 == 0, "the last dimension must be a multiple of the MX block (32)");
  TORCH_CHECK(x.is_cuda(), "gemm_kernels runs on a HIP device only; got a tensor on ", x.device());
  c10::DeviceGuard guard(x.device());
  hipStream_t stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  torch::Tensor q = torch::empty({rows, K}, x.options().dtype(at::kFloat8_e4m3fn));
  TORCH_CHECK(!shuffled || K % 128 == 0, "shuffled scales need the last dimension to be a multiple of 128");
  torch::Tensor sc = shuffled ? torch::empty({(int64_t)mi355_mx_shuffled_bytes(rows, K)}, x.options().dtype(at::kByte))
                              : torch::empty({rows, K / 32}, x.options().dtype(at::kByte));
  int st = mi355_quantize_mxfp8(x.const_data_ptr(), dt, rows, K, K, q.mutable_data_ptr(), sc.data_ptr<uint8_t>(),
                                shuffled ? 1 : 0, (void*)stream);
  TORCH_CHECK(st == MI355_OK, "gemm_kernels: ", mi355_gemm_strerror(st));
  return {q, sc};
}

std::string select_variant(int64_t M, int64_t N, int64_t K, at::ScalarType dtype) {
  const int dt = dtype_code(dtype);
  TORCH_CHECK(dt >= 0, "dtype must be bfloat16, float16 or float8_e4m3fn");
  const int v = mi355_gemm_select_variant(M, N, K, dt);
  TORCH_CHECK(v >= 0, "gemm_kernels: ", mi355_gemm_strerror(v));
  return variant_name(v);
}

}  // namespace test

PYBIND11_MODULE(_C, m) {
  namespace py = pybind11;
  m.def("gemm_tn_test", &test::gemm_tn_test, "C = A @ B.T (bf16/fp16 in and out, fp32 accumulate)",
        py::arg("A"), py::arg("B"), py::arg("C"));
  m.def("gemm_tn", &test::gemm_tn, "gemm_tn_test with an explicit kernel variant", py::arg("A"),
        py::arg("B"), py::arg("C"), py::arg("variant") = "auto");
  m.def("gemm_tn_fp8", &test::gemm_tn_fp8,
        "C = scale_a*scale_b * A_q @ B_q.T for float8_e4m3fn operands, bf16/fp16 out",
        py::arg("A_q"), py::arg("B_q"), py::arg("scale_a"), py::arg("scale_b"), py::arg("C"),
        py::arg("variant") = "auto");
  m.def("quantize_e4m3", &test::quantize_e4m3,
        "per-tensor fp8 quantisation on the device: returns (x_q float8_e4m3fn, scale 0-dim fp32 tensor)",
        py::arg("x"));
  m.def("gemm_tn_mxfp8", &test::gemm_tn_mxfp8,
        "C = A @ B.T for MX block-scaled float8_e4m3fn operands (one E8M0 scale byte per 32 elements of K)",
        py::arg("A_q"), py::arg("B_q"), py::arg("scale_a"), py::arg("scale_b"), py::arg("C"),
        py::arg("scales_shuffled") = false);
  m.def("shuffle_mx_scales", &test::shuffle_mx_scales,
        "re-lay MX scale bytes (rows, K/32) into the layout the kernel reads", py::arg("scales"));
  m.def("quantize_mxfp8", &test::quantize_mxfp8,
        "MX quantisation on the device: returns (x_q float8_e4m3fn, scales uint8 (rows, K/32), or flat in the "
        "GEMM's layout with shuffled=True)",
        py::arg("x"), py::arg("shuffled") = false);
  m.def("select_variant", &test::select_variant, py::arg("M"), py::arg("N"), py::arg("K"),
        py::arg("dtype"));
  m.def("version", []() { return mi355_gemm_version(); });
}
