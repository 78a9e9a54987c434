// The thin ATen/pybind layer over libllmq_hip.so.
//
// It owns what a C ABI cannot: tensor checks, output allocation from torch's caching
// allocator, the device guard and torch's current stream. The Python names, argument names
// and defaults of the first two ops are those of the reference's extension
// (llmquant/cuda/csrc/fake_quant.cpp:21-51), so KernelQuantLinear-style callers bind
// unchanged; the error fragments its tests match ("must be a CUDA tensor",
// "float32, float16 or bfloat16", reference tests/test_cuda_kernel.py:84-89) are kept.
// No kernel lives here and nothing here synchronises, so every op stays graph-capturable.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <tuple>

#include "llmq.h"

namespace {

int dtype_code(const at::Tensor& t, const char* name) {
  switch (t.scalar_type()) {
    case at::kFloat: return LLMQ_F32;
    case at::kHalf: return LLMQ_F16;
    case at::kBFloat16: return LLMQ_BF16;
    default:
      TORCH_CHECK(false, name, " must be float32, float16 or bfloat16, got ", t.scalar_type());
  }
  return -1;
}

llmq_stream_t current_stream(const at::Tensor& t) {
  return static_cast<llmq_stream_t>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

void check_rc(int rc, const char* op) {
  TORCH_CHECK(rc == 0, op, " failed (", rc, "): ", llmq_last_error());
}

std::tuple<at::Tensor, at::Tensor> fake_quant_group(const at::Tensor& x, int64_t num_bits,
                                                    int64_t group_size, bool return_scale) {
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  TORCH_CHECK(x.dim() >= 1, "x must have at least one dimension");
  TORCH_CHECK(num_bits >= 2 && num_bits <= 8, "num_bits must be in [2, 8], got ", num_bits);
  TORCH_CHECK(group_size > 0, "group_size must be positive, got ", group_size);
  const int dtype = dtype_code(x, "x");
  const auto xc = x.contiguous();
  const int64_t k = xc.size(-1);
  TORCH_CHECK(k % group_size == 0, "last dim ", k, " is not divisible by group_size ", group_size);

  auto out = at::empty_like(xc);
  const auto scale_opts = xc.options().dtype(at::kFloat);
  if (xc.numel() == 0) return std::make_tuple(out.reshape(x.sizes()), at::empty({0}, scale_opts));

  auto scale_sizes = xc.sizes().vec();
  scale_sizes.back() = k / group_size;
  auto scale = return_scale ? at::empty(scale_sizes, scale_opts) : at::empty({0}, scale_opts);

  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_fake_quant_group(xc.const_data_ptr(), out.mutable_data_ptr(),
                                 return_scale ? scale.mutable_data_ptr<float>() : nullptr,
                                 xc.numel() / group_size, static_cast<int>(group_size),
                                 static_cast<int>(num_bits), dtype, current_stream(xc)),
           "fake_quant_group");
  return std::make_tuple(out.reshape(x.sizes()), scale);
}

std::tuple<at::Tensor, at::Tensor> quant_group_codes(const at::Tensor& x, int64_t num_bits,
                                                     int64_t group_size, bool pack4) {
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  TORCH_CHECK(x.dim() >= 1, "x must have at least one dimension");
  TORCH_CHECK(num_bits >= 2 && num_bits <= 8, "num_bits must be in [2, 8], got ", num_bits);
  TORCH_CHECK(group_size > 0, "group_size must be positive, got ", group_size);
  TORCH_CHECK(!pack4 || (num_bits <= 4 && group_size % 2 == 0),
              "nibble packing needs num_bits <= 4 and an even group_size");
  const int dtype = dtype_code(x, "x");
  const auto xc = x.contiguous();
  const int64_t k = xc.size(-1);
  TORCH_CHECK(k % group_size == 0, "last dim ", k, " is not divisible by group_size ", group_size);

  auto code_sizes = xc.sizes().vec();
  if (pack4) code_sizes.back() = k / 2;
  auto codes = at::empty(code_sizes, xc.options().dtype(pack4 ? at::kByte : at::kChar));
  auto scale_sizes = xc.sizes().vec();
  scale_sizes.back() = k / group_size;
  auto scale = at::empty(scale_sizes, xc.options().dtype(at::kFloat));
  if (xc.numel() == 0) return std::make_tuple(codes, scale);

  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_quant_group_codes(xc.const_data_ptr(), codes.mutable_data_ptr(),
                                  scale.mutable_data_ptr<float>(), xc.numel() / group_size,
                                  static_cast<int>(group_size), static_cast<int>(num_bits),
                                  pack4 ? 1 : 0, dtype, current_stream(xc)),
           "quant_group_codes");
  return std::make_tuple(codes, scale);
}

// qweight is either the reference's int8 [N, G, gs] or nibble-packed uint8 [N, G, gs/2].
at::Tensor wq_gemv(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale,
                   int64_t out_group) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar,
              "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat, "wscale must be float32");
  TORCH_CHECK(wscale.dim() == 2, "wscale must be [scale_rows, groups]");
  const int dtype = dtype_code(x, "x");

  const auto xc = x.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t N = wc.size(0);
  const int64_t groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(xc.dim() >= 1 && xc.size(-1) > 0, "x needs a non-empty last dimension");
  const int64_t M = xc.numel() / xc.size(-1);
  TORCH_CHECK(group_size % (packed ? 8 : 4) == 0, "group_size must be a multiple of ",
              packed ? 8 : 4, ", got ", group_size);
  TORCH_CHECK(xc.size(-1) == groups * group_size, "x last dim ", xc.size(-1),
              " does not match qweight ", groups, "x", group_size);
  TORCH_CHECK(out_group >= 0, "out_group must be >= 0");
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows,
              ", ", groups, "], got [", sc.size(0), ", ", sc.size(1), "]");

  auto out = at::empty({M, N}, xc.options());
  if (M == 0 || N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_wq_gemv(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                        out.mutable_data_ptr(), static_cast<int>(M), static_cast<int>(N),
                        static_cast<int>(groups), static_cast<int>(group_size),
                        static_cast<int>(out_group), packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8,
                        dtype, current_stream(xc)),
           "wq_gemv");
  return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("fake_quant_group", &fake_quant_group,
        "Fused symmetric RTN quant-dequant, grouped along the last axis (HIP, gfx950)",
        py::arg("x"), py::arg("num_bits"), py::arg("group_size"), py::arg("return_scale") = false);
  m.def("quant_group_codes", &quant_group_codes,
        "Symmetric RTN quantize to integer codes + fp32 scales, grouped along the last axis",
        py::arg("x"), py::arg("num_bits"), py::arg("group_size"), py::arg("pack4") = false);
  m.def("wq_gemv", &wq_gemv,
        "Weight-only quantized matmul for a few rows: int8 or packed-int4 weight (HIP, gfx950)",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0);
  m.def("abi_version", []() { return llmq_abi_version(); });
}
