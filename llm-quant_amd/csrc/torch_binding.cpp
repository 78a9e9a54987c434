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
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
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

// x [R, G*gs]; qweight [E, N, G, gs] int8 or [E, N, G, gs/2] packed; wscale [E, scale_rows, G]; the plan is
// three int32 device tensors of equal length. Returns [R, N]; rows no plan entry covers are zero.
at::Tensor wq_gemv_batched(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale,
                           const at::Tensor& block_expert, const at::Tensor& block_row0,
                           const at::Tensor& block_rows, int64_t out_group) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda() && block_expert.is_cuda() &&
                  block_row0.is_cuda() && block_rows.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 4, "qweight must be [experts, N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar,
              "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 3, "wscale must be float32 [experts, scale_rows, groups]");
  const int dtype = dtype_code(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [rows, in_features]");
  const auto xc = x.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const auto be = block_expert.to(at::kInt).contiguous();
  const auto b0 = block_row0.to(at::kInt).contiguous();
  const auto br = block_rows.to(at::kInt).contiguous();
  TORCH_CHECK(be.dim() == 1 && b0.sizes() == be.sizes() && br.sizes() == be.sizes(),
              "block_expert, block_row0 and block_rows must be 1-D and of equal length");
  const int64_t E = wc.size(0), N = wc.size(1), groups = wc.size(2);
  const int64_t group_size = packed ? wc.size(3) * 2 : wc.size(3);
  TORCH_CHECK(xc.size(1) == groups * group_size, "x last dim ", xc.size(1), " does not match qweight ", groups,
              "x", group_size);
  TORCH_CHECK(out_group >= 0, "out_group must be >= 0");
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == E && sc.size(1) == scale_rows && sc.size(2) == groups, "wscale must be [", E, ", ",
              scale_rows, ", ", groups, "]");
  auto out = at::zeros({xc.size(0), N}, xc.options());
  if (out.numel() == 0 || be.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_wq_gemv_batched(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                                out.mutable_data_ptr(), be.const_data_ptr<int32_t>(), b0.const_data_ptr<int32_t>(),
                                br.const_data_ptr<int32_t>(), static_cast<int>(be.numel()),
                                static_cast<int>(xc.size(0)), static_cast<int>(E), static_cast<int>(N),
                                static_cast<int>(groups), static_cast<int>(group_size), static_cast<int>(out_group),
                                packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, current_stream(xc)),
           "wq_gemv_batched");
  return out;
}

// qweight [N, G, gs] int8 or [N, G, gs/2] packed uint8 -> dense [N, G*keep] in out_dtype.
at::Tensor dequant_weight(const at::Tensor& qweight, const at::Tensor& wscale, int64_t out_group,
                          int64_t keep_per_group, at::ScalarType out_dtype) {
  TORCH_CHECK(qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 3 && qweight.is_contiguous(), "qweight must be contiguous [N, groups, group_size]");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar,
              "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2 && wscale.is_contiguous(),
              "wscale must be contiguous float32 [scale_rows, groups]");
  const int64_t N = qweight.size(0), groups = qweight.size(1);
  const int64_t group_size = packed ? qweight.size(2) * 2 : qweight.size(2);
  if (keep_per_group <= 0) keep_per_group = group_size;
  TORCH_CHECK(out_group >= 0, "out_group must be >= 0");
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(wscale.size(0) == scale_rows && wscale.size(1) == groups, "wscale must be [", scale_rows,
              ", ", groups, "], got [", wscale.size(0), ", ", wscale.size(1), "]");
  auto out = at::empty({N, groups * keep_per_group}, qweight.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  if (out.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(qweight));
  check_rc(llmq_dequant_weight(qweight.const_data_ptr(), wscale.const_data_ptr<float>(), out.mutable_data_ptr(),
                               static_cast<int>(N), static_cast<int>(groups), static_cast<int>(group_size),
                               static_cast<int>(keep_per_group), static_cast<int>(out_group),
                               packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, current_stream(qweight)),
           "dequant_weight");
  return out;
}

// ---- the dense branch in one call: dequantize, then the BLAS library's matmul ----------------------
// at::mm spends ~19 us of host time per call on this stack, most of it on building descriptors and
// asking the library's heuristic again; a prompt pass makes four such calls per layer and the host
// is what bounds it. Here the descriptors and the heuristic's first choice are kept per
// (dtype, M, N, K) and a call costs ~10 us. The algorithm is the one at::mm gets from the same
// heuristic, so the results are the same bits.
struct DensePlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo;
  bool usable = true;   // false: the heuristic had nothing for this shape within the workspace; torch's matmul takes it
};
struct DenseState {
  hipblasLtHandle_t handle = nullptr;
  std::map<std::tuple<int, int64_t, int64_t, int64_t>, DensePlan> plans;
  std::map<void*, at::Tensor> workspaces;  // one per stream: calls on two streams may overlap
};
constexpr int64_t kDenseWorkspaceBytes = 32 << 20;
constexpr size_t kDenseMaxPlans = 4096;
std::mutex g_dense_lock;

DenseState& dense_state(int device) {
  // never destroyed: at process exit the HIP runtime may already be gone when statics are torn down
  static auto* states = new std::map<int, DenseState>;
  return (*states)[device];
}

void check_lt(hipblasStatus_t status, const char* what) {
  TORCH_CHECK(status == HIPBLAS_STATUS_SUCCESS, "hipBLASLt ", what, " failed with status ", static_cast<int>(status));
}

const DensePlan& dense_plan(DenseState& st, bool bf16, int64_t M, int64_t N, int64_t K) {
  const auto key = std::make_tuple(static_cast<int>(bf16), M, N, K);
  auto found = st.plans.find(key);
  if (found != st.plans.end()) return found->second;
  if (st.plans.size() >= kDenseMaxPlans) {  // a caller with ever-changing row counts: start over
    for (auto& kept : st.plans) {
      hipblasLtMatmulDescDestroy(kept.second.desc);
      hipblasLtMatrixLayoutDestroy(kept.second.w);
      hipblasLtMatrixLayoutDestroy(kept.second.x);
      hipblasLtMatrixLayoutDestroy(kept.second.out);
    }
    st.plans.clear();
  }
  DensePlan p;
  const hipDataType t = bf16 ? HIP_R_16BF : HIP_R_16F;
  check_lt(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "MatmulDescCreate");
  const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  check_lt(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)), "TRANSA");
  check_lt(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)), "TRANSB");
  // in the library's column-major terms: out^T [N, M] = (w as [K, N])^T * (x as [K, M])
  check_lt(hipblasLtMatrixLayoutCreate(&p.w, t, K, N, K), "MatrixLayoutCreate");
  check_lt(hipblasLtMatrixLayoutCreate(&p.x, t, K, M, K), "MatrixLayoutCreate");
  check_lt(hipblasLtMatrixLayoutCreate(&p.out, t, N, M, N), "MatrixLayoutCreate");
  hipblasLtMatmulPreference_t pref = nullptr;
  check_lt(hipblasLtMatmulPreferenceCreate(&pref), "MatmulPreferenceCreate");
  const size_t cap = static_cast<size_t>(kDenseWorkspaceBytes);
  check_lt(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap)),
           "MAX_WORKSPACE_BYTES");
  hipblasLtMatmulHeuristicResult_t results[4];
  int n_results = 0;
  const hipblasStatus_t status =
      hipblasLtMatmulAlgoGetHeuristic(st.handle, p.desc, p.w, p.x, p.out, p.out, pref, 4, results, &n_results);
  hipblasLtMatmulPreferenceDestroy(pref);
  check_lt(status, "MatmulAlgoGetHeuristic");
  int pick = -1;
  for (int i = 0; i < n_results && pick < 0; ++i) {
    if (results[i].state == HIPBLAS_STATUS_SUCCESS && results[i].workspaceSize <= cap) pick = i;
  }
  if (pick >= 0) {
    p.algo = results[pick].algo;
  } else {
    p.usable = false;   // (seen for 31000 x 16384 x 2048: remembered, so that the heuristic is not asked again per call)
  }
  return st.plans.emplace(key, p).first->second;
}

at::Tensor dense_linear(const at::Tensor& x, const at::Tensor& w) {
  TORCH_CHECK(x.is_cuda() && w.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.is_contiguous() && w.is_contiguous(),
              "x [M, K] and w [N, K] must be contiguous matrices");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf, "x must be float16 or bfloat16, got ",
              x.scalar_type());
  TORCH_CHECK(w.scalar_type() == x.scalar_type(), "w must have x's dtype");
  TORCH_CHECK(x.size(1) == w.size(1), "x has ", x.size(1), " columns, w ", w.size(1));
  const int64_t M = x.size(0), K = x.size(1), N = w.size(0);
  auto out = at::empty({M, N}, x.options());
  if (out.numel() == 0) return out;
  if (K == 0) return out.zero_();
  // the kept plan is chosen once per shape, for operands as the allocator hands them out; rows that are
  // not whole 16-byte packets, or a view at an odd offset, go the general way
  const bool packets = K % 8 == 0 &&
                       ((reinterpret_cast<uintptr_t>(x.const_data_ptr()) | reinterpret_cast<uintptr_t>(w.const_data_ptr())) & 15u) == 0;
  if (!packets) return at::mm(x, w.t());
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  const auto stream = c10::hip::getCurrentHIPStream(x.device().index());
  const std::lock_guard<std::mutex> lock(g_dense_lock);
  DenseState& st = dense_state(x.device().index());
  if (st.handle == nullptr) check_lt(hipblasLtCreate(&st.handle), "Create");
  at::Tensor& workspace = st.workspaces[static_cast<void*>(stream.stream())];
  if (!workspace.defined()) workspace = at::empty({kDenseWorkspaceBytes}, x.options().dtype(at::kByte));
  const DensePlan& plan = dense_plan(st, x.scalar_type() == at::kBFloat16, M, N, K);
  if (!plan.usable) return at::mm(x, w.t());
  const float one = 1.0f, zero = 0.0f;
  check_lt(hipblasLtMatmul(st.handle, plan.desc, &one, w.const_data_ptr(), plan.w, x.const_data_ptr(), plan.x, &zero,
                           out.const_data_ptr(), plan.out, out.mutable_data_ptr(), plan.out, &plan.algo,
                           workspace.mutable_data_ptr(), static_cast<size_t>(kDenseWorkspaceBytes), stream.stream()),
           "Matmul");
  return out;
}

at::Tensor wq_dense_linear(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale, int64_t out_group,
                           int64_t keep_per_group) {
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  return dense_linear(x, dequant_weight(qweight, wscale, out_group, keep_per_group, x.scalar_type()));
}

// One activation row through a quantized Linear with the surrounding elementwise operations
// folded in (see llmq_wq_gemv_fused). x: [K] (or [2K] gate|up for prologue 2); returns [N].
at::Tensor wq_gemv_fused(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale,
                         int64_t out_group, int64_t prologue, const c10::optional<at::Tensor>& norm_weight,
                         double eps, int64_t in_head_dim, const c10::optional<at::Tensor>& residual) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 3 && qweight.is_contiguous(), "qweight must be contiguous [N, groups, group_size]");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2 && wscale.is_contiguous(),
              "wscale must be contiguous float32 [scale_rows, groups]");
  TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
  const int dtype = dtype_code(x, "x");
  const int64_t N = qweight.size(0), groups = qweight.size(1);
  const int64_t group_size = packed ? qweight.size(2) * 2 : qweight.size(2);
  TORCH_CHECK(group_size == 128, "the fused GEMV needs group_size 128, got ", group_size);
  const int64_t k_real = in_head_dim > 0 ? groups * in_head_dim : groups * group_size;
  TORCH_CHECK(x.numel() == (prologue == LLMQ_PRO_SILU_MUL ? 2 * k_real : k_real), "x has ", x.numel(),
              " elements, expected ", prologue == LLMQ_PRO_SILU_MUL ? 2 * k_real : k_real);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(wscale.size(0) == scale_rows && wscale.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  const void* norm_ptr = nullptr;
  if (prologue == LLMQ_PRO_RMSNORM) {
    TORCH_CHECK(norm_weight.has_value() && norm_weight->is_cuda() && norm_weight->is_contiguous() &&
                    norm_weight->numel() == k_real && norm_weight->scalar_type() == x.scalar_type(),
                "the RMSNorm prologue needs a contiguous weight of x's dtype with ", k_real, " elements");
    norm_ptr = norm_weight->const_data_ptr();
  }
  const void* res_ptr = nullptr;
  if (residual.has_value() && residual->defined()) {
    TORCH_CHECK(residual->is_cuda() && residual->is_contiguous() && residual->numel() == N &&
                    residual->scalar_type() == x.scalar_type(),
                "residual must be a contiguous tensor of x's dtype with ", N, " elements");
    res_ptr = residual->const_data_ptr();
  }
  auto out = at::empty({1, N}, x.options());
  if (N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_wq_gemv_fused(x.const_data_ptr(), qweight.const_data_ptr(), wscale.const_data_ptr<float>(),
                              out.mutable_data_ptr(), static_cast<int>(N), static_cast<int>(groups),
                              static_cast<int>(out_group), packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype,
                              static_cast<int>(prologue), norm_ptr, static_cast<float>(eps),
                              static_cast<int>(in_head_dim), res_ptr, current_stream(x)),
           "wq_gemv_fused");
  return out;
}

// The batched GEMV's routing plan in one launch (see llmq_route_plan). top_k_index: integer tensor of
// any shape; returns (order int64 [rows], block_expert, block_row0, block_rows int32 [experts * B]).
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> route_plan(const at::Tensor& top_k_index,
                                                                      int64_t num_experts, int64_t limit) {
  TORCH_CHECK(top_k_index.is_cuda(), "top_k_index must be a CUDA tensor");
  TORCH_CHECK(at::isIntegralType(top_k_index.scalar_type(), false), "top_k_index must hold integers");
  const at::Tensor flat = top_k_index.reshape({-1}).to(at::kLong).contiguous();
  const int64_t rows = flat.numel();
  TORCH_CHECK(limit > 0, "limit must be positive, got ", limit);
  TORCH_CHECK(llmq_route_plan_supported(static_cast<int>(std::min<int64_t>(rows, INT32_MAX)),
                                        static_cast<int>(std::min<int64_t>(num_experts, INT32_MAX))),
              "the routing-plan kernel does not take ", rows, " rows and ", num_experts, " experts");
  const int64_t per_expert = llmq_route_plan_blocks_per_expert(static_cast<int>(rows), static_cast<int>(limit));
  auto order = at::empty({rows}, flat.options());
  auto i32 = flat.options().dtype(at::kInt);
  auto block_expert = at::empty({num_experts * per_expert}, i32);
  auto block_row0 = at::empty({num_experts * per_expert}, i32);
  auto block_rows = at::empty({num_experts * per_expert}, i32);
  const c10::OptionalDeviceGuard guard(at::device_of(flat));
  check_rc(llmq_route_plan(flat.const_data_ptr<int64_t>(), static_cast<int>(rows), static_cast<int>(num_experts),
                           static_cast<int>(limit), order.mutable_data_ptr<int64_t>(),
                           block_expert.mutable_data_ptr<int32_t>(), block_row0.mutable_data_ptr<int32_t>(),
                           block_rows.mutable_data_ptr<int32_t>(), current_stream(flat)),
           "route_plan");
  return {order, block_expert, block_row0, block_rows};
}

// A projection of a gated MoE block over every routed expert (see llmq_wq_gemv_batched_fused).
// x: [n_rows, K] rows in sorted order, or [1, K] with broadcast_x (every row is that one token).
// Returns [n_rows, N], or [n_rows, N / 2] = silu(gate) * up with act_pair.
at::Tensor wq_gemv_batched_fused(const at::Tensor& x, bool broadcast_x, int64_t n_rows, const at::Tensor& qweight,
                                 const at::Tensor& wscale, const at::Tensor& block_expert,
                                 const at::Tensor& block_row0, const at::Tensor& block_rows, bool act_pair) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda() && block_expert.is_cuda() &&
                  block_row0.is_cuda() && block_rows.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 4 && qweight.is_contiguous(), "qweight must be contiguous [experts, N, groups, group_size]");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  const int64_t E = qweight.size(0), N = qweight.size(1), groups = qweight.size(2);
  const int64_t group_size = packed ? qweight.size(3) * 2 : qweight.size(3);
  TORCH_CHECK(group_size == 128, "the fused batched GEMV needs group_size 128, got ", group_size);
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.is_contiguous() && wscale.dim() == 3 &&
                  wscale.size(0) == E && wscale.size(1) == N && wscale.size(2) == groups,
              "wscale must be contiguous float32 [", E, ", ", N, ", ", groups, "]");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && x.size(1) == groups * group_size, "x must be contiguous [rows, ",
              groups * group_size, "]");
  TORCH_CHECK(broadcast_x ? x.size(0) == 1 : x.size(0) == n_rows, "x has ", x.size(0), " rows, expected ",
              broadcast_x ? 1 : n_rows);
  for (const at::Tensor* t : {&block_expert, &block_row0, &block_rows}) {
    TORCH_CHECK(t->scalar_type() == at::kInt && t->is_contiguous() && t->dim() == 1 &&
                    t->numel() == block_expert.numel(), "the plan must be three contiguous int32 vectors of one length");
  }
  TORCH_CHECK(!act_pair || N % 16 == 0, "gate|up needs halves that are multiples of 8 rows, got ", N);
  const int dtype = dtype_code(x, "x");
  auto out = at::empty({n_rows, act_pair ? N / 2 : N}, x.options());
  if (out.numel() == 0 || block_expert.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_wq_gemv_batched_fused(x.const_data_ptr(), broadcast_x ? 0 : x.size(1), qweight.const_data_ptr(),
                                      wscale.const_data_ptr<float>(), out.mutable_data_ptr(),
                                      block_expert.const_data_ptr<int32_t>(), block_row0.const_data_ptr<int32_t>(),
                                      block_rows.const_data_ptr<int32_t>(), static_cast<int>(block_expert.numel()),
                                      static_cast<int>(n_rows), static_cast<int>(E), static_cast<int>(N),
                                      static_cast<int>(groups), packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype,
                                      act_pair ? 1 : 0, current_stream(x)),
           "wq_gemv_batched_fused");
  return out;
}

// final[t] = sum of the rows routed from token t times their routing weights (see llmq_moe_combine).
at::Tensor moe_combine(const at::Tensor& rows_out, const at::Tensor& order, const at::Tensor& weights,
                       int64_t n_tokens) {
  TORCH_CHECK(rows_out.is_cuda() && order.is_cuda() && weights.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(rows_out.dim() == 2 && rows_out.is_contiguous(), "rows_out must be contiguous [rows, width]");
  TORCH_CHECK(order.scalar_type() == at::kLong && order.is_contiguous() && order.numel() == rows_out.size(0),
              "order must be a contiguous int64 vector with one entry per row");
  TORCH_CHECK(weights.dim() == 2 && weights.is_contiguous() && weights.size(0) == n_tokens &&
                  weights.scalar_type() == rows_out.scalar_type() && weights.numel() == order.numel(),
              "weights must be contiguous [tokens, top_k] of the rows' dtype, one per row");
  const int dtype = dtype_code(rows_out, "rows_out");
  auto out = at::empty({n_tokens, rows_out.size(1)}, rows_out.options());
  if (out.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(rows_out));
  check_rc(llmq_moe_combine(rows_out.const_data_ptr(), order.const_data_ptr<int64_t>(), weights.const_data_ptr(),
                            out.mutable_data_ptr(), static_cast<int>(rows_out.size(0)),
                            static_cast<int>(weights.size(1)), static_cast<int>(n_tokens),
                            static_cast<int>(rows_out.size(1)), dtype, current_stream(rows_out)),
           "moe_combine");
  return out;
}

// One-row gate|up Linear of a gated MLP with act(gate) * up folded into the store (see
// llmq_wq_gemv_gate_up_silu). qweight: [2I, groups, group_size], gate rows first; returns [1, I].
at::Tensor wq_gemv_gate_up_silu(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale,
                                int64_t prologue, const c10::optional<at::Tensor>& norm_weight, double eps) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(qweight.dim() == 3 && qweight.is_contiguous(), "qweight must be contiguous [2I, groups, group_size]");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2 && wscale.is_contiguous(),
              "wscale must be contiguous float32 [2I, groups]");
  TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
  const int dtype = dtype_code(x, "x");
  const int64_t N = qweight.size(0), groups = qweight.size(1);
  const int64_t group_size = packed ? qweight.size(2) * 2 : qweight.size(2);
  TORCH_CHECK(group_size == 128, "the fused GEMV needs group_size 128, got ", group_size);
  TORCH_CHECK(N % 16 == 0, "gate|up needs an even number of rows with halves that are multiples of 8, got ", N);
  TORCH_CHECK(x.numel() == groups * group_size, "x has ", x.numel(), " elements, expected ", groups * group_size);
  TORCH_CHECK(wscale.size(0) == N && wscale.size(1) == groups, "wscale must be [", N, ", ", groups, "]");
  const void* norm_ptr = nullptr;
  if (prologue == LLMQ_PRO_RMSNORM) {
    TORCH_CHECK(norm_weight.has_value() && norm_weight->is_cuda() && norm_weight->is_contiguous() &&
                    norm_weight->numel() == x.numel() && norm_weight->scalar_type() == x.scalar_type(),
                "the RMSNorm prologue needs a contiguous weight of x's dtype with ", x.numel(), " elements");
    norm_ptr = norm_weight->const_data_ptr();
  }
  auto out = at::empty({1, N / 2}, x.options());
  if (N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_wq_gemv_gate_up_silu(x.const_data_ptr(), qweight.const_data_ptr(), wscale.const_data_ptr<float>(),
                                     out.mutable_data_ptr(), static_cast<int>(N / 2), static_cast<int>(groups),
                                     packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, static_cast<int>(prologue),
                                     norm_ptr, static_cast<float>(eps), current_stream(x)),
           "wq_gemv_gate_up_silu");
  return out;
}

// Integer GEMM: a int8 [M, K], sx fp32 [M, G]; qweight / wscale as for wq_gemv; optional fp32 or
// half-width bias (converted to fp32 here, as RealQuantLinear adds bias.float()).
// exact = true: RealQuantLinear's fp32 roundings and group order, bit for bit. exact = false: the same integer
// group sums folded in with one multiply-add fewer per output and group, the reduction axis split across
// workgroups where the output has few tiles: agrees to fp32 rounding. sx is [M, groups], or [M, 1] for one scale
// per token (the exact form multiplies by the broadcast scale group by group; the fast form takes the scale
// out of the sum over groups).
at::Tensor wq_gemm_a8(const at::Tensor& a, const at::Tensor& sx, const at::Tensor& qweight,
                      const at::Tensor& wscale, const c10::optional<at::Tensor>& bias, int64_t out_group,
                      at::ScalarType out_dtype, bool exact) {
  TORCH_CHECK(a.is_cuda() && sx.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(a.scalar_type() == at::kChar && a.dim() == 2, "a must be int8 [M, K]");
  TORCH_CHECK(sx.scalar_type() == at::kFloat && sx.dim() == 2, "sx must be float32 [M, groups]");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto ac = a.contiguous();
  auto sxc = sx.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = ac.size(0), N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the integer GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(ac.size(1) == groups * group_size, "a last dim ", ac.size(1), " does not match qweight ",
              groups, "x", group_size);
  TORCH_CHECK(sxc.size(0) == M && (sxc.size(1) == groups || sxc.size(1) == 1), "sx must be [", M, ", ", groups,
              "] or [", M, ", 1]");
  const int64_t sx_groups = sxc.size(1);
  if (exact && sx_groups != groups) sxc = sxc.expand({M, groups}).contiguous();
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  at::Tensor bias_f;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->numel() == N, "bias must have ", N, " elements");
    bias_f = bias->to(at::kFloat).contiguous();
  }
  auto out = at::empty({M, N}, ac.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  if (M == 0 || N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(ac));
  if (!exact) {
    const size_t need = llmq_wq_gemm_a8_fast_workspace_bytes(static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups));
    auto workspace = at::empty({static_cast<int64_t>((need + 3) / 4)}, ac.options().dtype(at::kFloat));
    check_rc(llmq_wq_gemm_a8_fast(ac.const_data_ptr<int8_t>(), sxc.const_data_ptr<float>(), wc.const_data_ptr(),
                                  sc.const_data_ptr<float>(), bias_f.defined() ? bias_f.const_data_ptr<float>() : nullptr,
                                  out.mutable_data_ptr(), need ? workspace.mutable_data_ptr() : nullptr, need, static_cast<int>(M),
                                  static_cast<int>(N), static_cast<int>(groups), static_cast<int>(sx_groups),
                                  static_cast<int>(group_size), static_cast<int>(out_group),
                                  packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, current_stream(ac)),
             "wq_gemm_a8 (fast form)");
    return out;
  }
  check_rc(llmq_wq_gemm_a8(ac.const_data_ptr<int8_t>(), sxc.const_data_ptr<float>(), wc.const_data_ptr(),
                           sc.const_data_ptr<float>(), bias_f.defined() ? bias_f.const_data_ptr<float>() : nullptr,
                           out.mutable_data_ptr(), static_cast<int>(M), static_cast<int>(N),
                           static_cast<int>(groups), static_cast<int>(group_size), static_cast<int>(out_group),
                           packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, current_stream(ac)),
           "wq_gemm_a8");
  return out;
}

// x [M, K] bf16 / fp16 -> (int8 codes in the operand order of the exact integer GEMM's group-parallel kernel, for
// weights of `weight_bits` bits; scales [M, K / 128]): quant_group_codes(x, 8, 128) with the codes laid out for
// wq_gemm_a8_tiled.
std::tuple<at::Tensor, at::Tensor> quant_act_codes_tiled(const at::Tensor& x, int64_t weight_bits) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2, "x must be a CUDA tensor [M, K]");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf, "x must be bfloat16 or float16");
  TORCH_CHECK(weight_bits == 4 || weight_bits == 8, "weight_bits must be 4 or 8, got ", weight_bits);
  const auto xc = x.contiguous();
  const int64_t M = xc.size(0), K = xc.size(1);
  TORCH_CHECK(K % 128 == 0, "last dim ", K, " is not a multiple of 128");
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  auto codes = at::empty({static_cast<int64_t>(llmq_act_codes_tiled_bytes(static_cast<int>(M), static_cast<int>(K)))},
                         xc.options().dtype(at::kChar));
  auto scale = at::empty({M, K / 128}, xc.options().dtype(at::kFloat));
  if (xc.numel() == 0) return std::make_tuple(codes, scale);
  check_rc(llmq_quant_act_codes_tiled(xc.const_data_ptr(), codes.mutable_data_ptr(), scale.mutable_data_ptr<float>(),
                                      static_cast<int>(M), static_cast<int>(K),
                                      weight_bits == 4 ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype_code(xc, "x"),
                                      current_stream(xc)),
           "quant_act_codes_tiled");
  return std::make_tuple(codes, scale);
}

// wq_gemm_a8 (exact form) on the codes of quant_act_codes_tiled for `rows` activation rows.
at::Tensor wq_gemm_a8_tiled(const at::Tensor& codes, const at::Tensor& sx, int64_t rows, const at::Tensor& qweight,
                            const at::Tensor& wscale, const c10::optional<at::Tensor>& bias, int64_t out_group,
                            at::ScalarType out_dtype) {
  TORCH_CHECK(codes.is_cuda() && sx.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(codes.scalar_type() == at::kChar && codes.dim() == 1 && codes.is_contiguous(),
              "codes must be the tensor quant_act_codes_tiled returned");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto sxc = sx.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = rows, N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the integer GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(sxc.scalar_type() == at::kFloat && sxc.dim() == 2 && sxc.size(0) == M && sxc.size(1) == groups,
              "sx must be float32 [", M, ", ", groups, "]");
  TORCH_CHECK(static_cast<size_t>(codes.numel()) >= llmq_act_codes_tiled_bytes(static_cast<int>(M), static_cast<int>(groups * 128)),
              "codes hold ", codes.numel(), " bytes: not the codes of ", M, " rows of ", groups * 128);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  at::Tensor bias_f;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->numel() == N, "bias must have ", N, " elements");
    bias_f = bias->to(at::kFloat).contiguous();
  }
  auto out = at::empty({M, N}, codes.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  if (M == 0 || N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(codes));
  check_rc(llmq_wq_gemm_a8_tiled(codes.const_data_ptr(), sxc.const_data_ptr<float>(), wc.const_data_ptr(),
                                 sc.const_data_ptr<float>(), bias_f.defined() ? bias_f.const_data_ptr<float>() : nullptr,
                                 out.mutable_data_ptr(), static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups),
                                 static_cast<int>(group_size), static_cast<int>(out_group),
                                 packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, current_stream(codes)),
           "wq_gemm_a8_tiled");
  return out;
}

// Weight-only GEMM for a few dozen rows: x fp16/bf16 [M, K]; qweight / wscale as for wq_gemv.
at::Tensor wq_gemm_a16(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale, int64_t out_group,
                       bool split) {
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  TORCH_CHECK(qweight.is_cuda() && wscale.is_cuda(), "qweight and wscale must be CUDA tensors");
  TORCH_CHECK(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16,
              "the fused GEMM takes float16 or bfloat16 activations");
  TORCH_CHECK(x.dim() == 2, "x must be [M, K]");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto xc = x.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = xc.size(0), N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the fused GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(xc.size(1) == groups * group_size, "x last dim ", xc.size(1), " does not match qweight ", groups, "x",
              group_size);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  auto out = at::empty({M, N}, xc.options());
  if (M == 0 || N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  if (split) {
    const size_t need = llmq_wq_gemm_a16_workspace_bytes(static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups));
    auto workspace = at::empty({static_cast<int64_t>((need + 3) / 4)}, xc.options().dtype(at::kFloat));
    check_rc(llmq_wq_gemm_a16_split(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                                    out.mutable_data_ptr(), need ? workspace.mutable_data_ptr() : nullptr, need,
                                    static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups),
                                    static_cast<int>(group_size), static_cast<int>(out_group),
                                    packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype_code(xc, "x"), current_stream(xc)),
             "wq_gemm_a16_split");
    return out;
  }
  check_rc(llmq_wq_gemm_a16(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                            out.mutable_data_ptr(), static_cast<int>(M), static_cast<int>(N),
                            static_cast<int>(groups), static_cast<int>(group_size), static_cast<int>(out_group),
                            packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype_code(xc, "x"), current_stream(xc)),
           "wq_gemm_a16");
  return out;
}

// The fused GEMM for prompt-sized M (bf16 / fp16): 128 x 256 or 64 x 128 tiles, no dense weight.
at::Tensor wq_gemm_a16_tile(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale, int64_t out_group) {
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  TORCH_CHECK(qweight.is_cuda() && wscale.is_cuda(), "qweight and wscale must be CUDA tensors");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf,
              "the tiled fused GEMM takes bfloat16 or float16 activations");
  TORCH_CHECK(x.dim() == 2, "x must be [M, K]");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto xc = x.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = xc.size(0), N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the tiled fused GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(xc.size(1) == groups * group_size, "x last dim ", xc.size(1), " does not match qweight ", groups, "x",
              group_size);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  auto out = at::empty({M, N}, xc.options());
  if (M == 0 || N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  const size_t need = llmq_wq_gemm_a16_tile_workspace_bytes(static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups));
  auto workspace = at::empty({static_cast<int64_t>((need + 3) / 4)}, xc.options().dtype(at::kFloat));
  check_rc(llmq_wq_gemm_a16_tile(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                                 out.mutable_data_ptr(), workspace.mutable_data_ptr(), need, static_cast<int>(M),
                                 static_cast<int>(N), static_cast<int>(groups), static_cast<int>(group_size),
                                 static_cast<int>(out_group), packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8,
                                 dtype_code(xc, "x"), current_stream(xc)),
           "wq_gemm_a16_tile");
  return out;
}

// gate|up GEMM with silu(gate) * up written as the prepared activation of the next tiled GEMM (down_proj, next_n
// rows): returns that GEMM's workspace, to be handed to wq_gemm_a16_tile_prepared.
at::Tensor wq_gemm_a16_tile_gate_up_silu(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& wscale,
                                         int64_t out_group, int64_t next_n) {
  TORCH_CHECK(x.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "x, qweight and wscale must be CUDA tensors");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf,
              "the tiled fused GEMM takes bfloat16 or float16 activations");
  TORCH_CHECK(x.dim() == 2, "x must be [M, K]");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [2 * intermediate, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto xc = x.contiguous();
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = xc.size(0), N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the tiled fused GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(N % 256 == 0, "gate rows followed by up rows, a multiple of 128 each: got ", N, " rows");
  TORCH_CHECK(xc.size(1) == groups * group_size, "x last dim ", xc.size(1), " does not match qweight ", groups, "x", group_size);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  TORCH_CHECK(M > 0 && next_n > 0, "empty activation");
  const int64_t inter = N / 2, next_groups = inter / 128;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  const size_t need = llmq_wq_gemm_a16_tile_prepared_bytes(static_cast<int>(M), static_cast<int>(groups));
  const size_t next_need = llmq_wq_gemm_a16_tile_workspace_bytes(static_cast<int>(M), static_cast<int>(next_n), static_cast<int>(next_groups));
  auto workspace = at::empty({static_cast<int64_t>((need + 3) / 4)}, xc.options().dtype(at::kFloat));
  auto next = at::empty({static_cast<int64_t>((next_need + 3) / 4)}, xc.options().dtype(at::kFloat));
  check_rc(llmq_wq_gemm_a16_tile_gate_up_silu(xc.const_data_ptr(), wc.const_data_ptr(), sc.const_data_ptr<float>(),
                                              workspace.mutable_data_ptr(), need, next.mutable_data_ptr(), next_need,
                                              static_cast<int>(M), static_cast<int>(inter), static_cast<int>(groups),
                                              static_cast<int>(group_size), static_cast<int>(out_group),
                                              packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype_code(xc, "x"),
                                              current_stream(xc)),
           "wq_gemm_a16_tile_gate_up_silu");
  return next;
}

// The same launch on an activation that is already in prepared form in `workspace` (from add_rmsnorm_prepared).
at::Tensor wq_gemm_a16_tile_gate_up_silu_prepared(const at::Tensor& workspace, int64_t rows, const at::Tensor& qweight,
                                                  const at::Tensor& wscale, int64_t out_group, int64_t next_n,
                                                  at::ScalarType dtype) {
  TORCH_CHECK(dtype == at::kBFloat16 || dtype == at::kHalf, "dtype must be bfloat16 or float16");
  TORCH_CHECK(workspace.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "workspace, qweight and wscale must be CUDA tensors");
  TORCH_CHECK(workspace.scalar_type() == at::kFloat && workspace.dim() == 1 && workspace.is_contiguous(),
              "workspace must be the tensor add_rmsnorm_prepared returned");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [2 * intermediate, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = rows, N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the tiled fused GEMM needs group_size 128, got ", group_size);
  TORCH_CHECK(N % 256 == 0, "gate rows followed by up rows, a multiple of 128 each: got ", N, " rows");
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  TORCH_CHECK(M > 0 && next_n > 0, "empty activation");
  const int64_t inter = N / 2, next_groups = inter / 128;
  const c10::OptionalDeviceGuard guard(at::device_of(workspace));
  const size_t need = llmq_wq_gemm_a16_tile_prepared_bytes(static_cast<int>(M), static_cast<int>(groups));
  TORCH_CHECK(static_cast<size_t>(workspace.numel()) * 4 >= need, "workspace holds ", workspace.numel() * 4, " bytes, this GEMM needs ", need);
  const size_t next_need = llmq_wq_gemm_a16_tile_workspace_bytes(static_cast<int>(M), static_cast<int>(next_n), static_cast<int>(next_groups));
  auto next = at::empty({static_cast<int64_t>((next_need + 3) / 4)}, workspace.options());
  check_rc(llmq_wq_gemm_a16_tile_gate_up_silu_prepared(wc.const_data_ptr(), sc.const_data_ptr<float>(),
                                                       workspace.mutable_data_ptr(), static_cast<size_t>(workspace.numel()) * 4,
                                                       next.mutable_data_ptr(), next_need, static_cast<int>(M),
                                                       static_cast<int>(inter), static_cast<int>(groups),
                                                       static_cast<int>(group_size), static_cast<int>(out_group),
                                                       packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8,
                                                       dtype == at::kHalf ? LLMQ_F16 : LLMQ_BF16, current_stream(workspace)),
           "wq_gemm_a16_tile_gate_up_silu_prepared");
  return next;
}

// The tiled GEMM on a prepared activation of `rows` rows sitting in `workspace` (from wq_gemm_a16_tile_gate_up_silu).
at::Tensor wq_gemm_a16_tile_prepared(const at::Tensor& workspace, int64_t rows, const at::Tensor& qweight,
                                     const at::Tensor& wscale, int64_t out_group, at::ScalarType dtype) {
  TORCH_CHECK(dtype == at::kBFloat16 || dtype == at::kHalf, "dtype must be bfloat16 or float16");
  TORCH_CHECK(workspace.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "workspace, qweight and wscale must be CUDA tensors");
  TORCH_CHECK(workspace.scalar_type() == at::kFloat && workspace.dim() == 1 && workspace.is_contiguous(),
              "workspace must be the tensor wq_gemm_a16_tile_gate_up_silu or add_rmsnorm_prepared returned");
  TORCH_CHECK(qweight.dim() == 3, "qweight must be [N, groups, group_size], got ", qweight.dim(), "D");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2, "wscale must be float32 [scale_rows, groups]");
  const auto wc = qweight.contiguous();
  const auto sc = wscale.contiguous();
  const int64_t M = rows, N = wc.size(0), groups = wc.size(1);
  const int64_t group_size = packed ? wc.size(2) * 2 : wc.size(2);
  TORCH_CHECK(group_size == 128, "the tiled fused GEMM needs group_size 128, got ", group_size);
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(sc.size(0) == scale_rows && sc.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  TORCH_CHECK(M > 0 && N > 0, "empty activation or weight");
  const size_t need = llmq_wq_gemm_a16_tile_workspace_bytes(static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups));
  TORCH_CHECK(static_cast<size_t>(workspace.numel()) * 4 >= need, "workspace holds ", workspace.numel() * 4, " bytes, this GEMM needs ", need);
  auto out = at::empty({M, N}, workspace.options().dtype(dtype));
  const c10::OptionalDeviceGuard guard(at::device_of(workspace));
  check_rc(llmq_wq_gemm_a16_tile_prepared(wc.const_data_ptr(), sc.const_data_ptr<float>(), out.mutable_data_ptr(),
                                          workspace.mutable_data_ptr(), static_cast<size_t>(workspace.numel()) * 4,
                                          static_cast<int>(M), static_cast<int>(N), static_cast<int>(groups),
                                          static_cast<int>(group_size), static_cast<int>(out_group),
                                          packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8,
                                          dtype == at::kHalf ? LLMQ_F16 : LLMQ_BF16, current_stream(workspace)),
           "wq_gemm_a16_tile_prepared");
  return out;
}

// ---- elementwise pieces of a prompt pass ----------------------------------------------------------------
at::Tensor rmsnorm(const at::Tensor& x, const at::Tensor& weight, double eps) {
  TORCH_CHECK(x.is_cuda() && weight.is_cuda(), "x and weight must be CUDA tensors");
  TORCH_CHECK(x.dim() >= 1 && weight.dim() == 1 && weight.size(0) == x.size(-1), "weight must be [hidden]");
  TORCH_CHECK(weight.scalar_type() == x.scalar_type(), "weight must have x's dtype");
  const auto xc = x.contiguous();
  const auto wc = weight.contiguous();
  auto out = at::empty_like(xc);
  const int64_t hidden = xc.size(-1);
  const int64_t rows = hidden ? xc.numel() / hidden : 0;
  if (rows == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_rmsnorm(xc.const_data_ptr(), wc.const_data_ptr(), out.mutable_data_ptr(), static_cast<int>(rows),
                        static_cast<int>(hidden), static_cast<float>(eps), dtype_code(xc, "x"), current_stream(xc)),
           "rmsnorm");
  return out;
}

// (x + delta, LlamaRMSNorm(x + delta)): the residual add in front of a norm, one launch.
std::tuple<at::Tensor, at::Tensor> add_rmsnorm(const at::Tensor& x, const at::Tensor& delta, const at::Tensor& weight,
                                               double eps) {
  TORCH_CHECK(x.is_cuda() && delta.is_cuda() && weight.is_cuda(), "x, delta and weight must be CUDA tensors");
  TORCH_CHECK(x.sizes() == delta.sizes() && x.scalar_type() == delta.scalar_type(), "x and delta must match");
  TORCH_CHECK(x.dim() >= 1 && weight.dim() == 1 && weight.size(0) == x.size(-1), "weight must be [hidden]");
  TORCH_CHECK(weight.scalar_type() == x.scalar_type(), "weight must have x's dtype");
  const auto xc = x.contiguous();
  const auto dc = delta.contiguous();
  const auto wc = weight.contiguous();
  auto sum = at::empty_like(xc);
  auto out = at::empty_like(xc);
  const int64_t hidden = xc.size(-1);
  const int64_t rows = hidden ? xc.numel() / hidden : 0;
  if (rows == 0) return {sum, out};
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  check_rc(llmq_add_rmsnorm(xc.const_data_ptr(), dc.const_data_ptr(), wc.const_data_ptr(), sum.mutable_data_ptr(),
                            out.mutable_data_ptr(), static_cast<int>(rows), static_cast<int>(hidden),
                            static_cast<float>(eps), dtype_code(xc, "x"), current_stream(xc)),
           "add_rmsnorm");
  return {sum, out};
}

// LlamaRMSNorm(x + delta) (delta None: of x) written as the prepared activation of a tiled GEMM on a weight of
// next_n rows: returns (x + delta or x, that GEMM's workspace), the workspace to be handed to
// wq_gemm_a16_tile_prepared or wq_gemm_a16_tile_gate_up_silu_prepared with rows = the rows of x.
std::tuple<at::Tensor, at::Tensor> add_rmsnorm_prepared(const at::Tensor& x, const c10::optional<at::Tensor>& delta,
                                                        const at::Tensor& weight, double eps, int64_t next_n) {
  TORCH_CHECK(x.is_cuda() && weight.is_cuda(), "x and weight must be CUDA tensors");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf,
              "the prepared form is of bfloat16 or float16 activations");
  TORCH_CHECK(x.dim() == 2 && weight.dim() == 1 && weight.size(0) == x.size(1), "x must be [rows, hidden], weight [hidden]");
  TORCH_CHECK(weight.scalar_type() == x.scalar_type(), "weight must have x's dtype");
  TORCH_CHECK(x.size(0) > 0 && next_n > 0, "empty activation");
  const auto xc = x.contiguous();
  const auto wc = weight.contiguous();
  at::Tensor dc, sum = xc;
  if (delta.has_value()) {
    TORCH_CHECK(delta->is_cuda() && delta->sizes() == x.sizes() && delta->scalar_type() == x.scalar_type(), "x and delta must match");
    dc = delta->contiguous();
    sum = at::empty_like(xc);
  }
  const int64_t rows = xc.size(0), hidden = xc.size(1);
  TORCH_CHECK(hidden % 128 == 0, "hidden must be a multiple of 128, got ", hidden);
  const c10::OptionalDeviceGuard guard(at::device_of(xc));
  const size_t need = llmq_wq_gemm_a16_tile_workspace_bytes(static_cast<int>(rows), static_cast<int>(next_n), static_cast<int>(hidden / 128));
  auto workspace = at::empty({static_cast<int64_t>((need + 3) / 4)}, xc.options().dtype(at::kFloat));
  check_rc(llmq_add_rmsnorm_prepared(xc.const_data_ptr(), delta.has_value() ? dc.const_data_ptr() : nullptr,
                                     wc.const_data_ptr(), delta.has_value() ? sum.mutable_data_ptr() : nullptr,
                                     workspace.mutable_data_ptr(), need, static_cast<int>(rows), static_cast<int>(hidden),
                                     static_cast<float>(eps), dtype_code(xc, "x"), current_stream(xc)),
           "add_rmsnorm_prepared");
  return {sum, workspace};
}

// q [tokens, q_heads * D], k [tokens, kv_heads * D] (rows may be strided), cos / sin [tokens, D].
std::tuple<at::Tensor, at::Tensor> rope_qk(const at::Tensor& q, const at::Tensor& k, const at::Tensor& cos,
                                           const at::Tensor& sin, int64_t q_heads, int64_t kv_heads) {
  TORCH_CHECK(q.is_cuda() && k.is_cuda() && cos.is_cuda() && sin.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && cos.dim() == 2 && sin.dim() == 2, "q, k, cos, sin must be 2-D");
  TORCH_CHECK(q.stride(1) == 1 && k.stride(1) == 1, "q and k need a contiguous last axis");
  TORCH_CHECK(q_heads > 0 && kv_heads > 0, "head counts must be positive");
  const int64_t tokens = q.size(0), head_dim = cos.size(1);
  TORCH_CHECK(k.size(0) == tokens && cos.size(0) == tokens && sin.size(0) == tokens && sin.size(1) == head_dim,
              "q, k, cos and sin must cover the same tokens");
  TORCH_CHECK(q.size(1) == q_heads * head_dim && k.size(1) == kv_heads * head_dim, "q / k widths do not match the heads");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && cos.scalar_type() == q.scalar_type() &&
                  sin.scalar_type() == q.scalar_type(), "k, cos and sin must have q's dtype");
  const auto cc = cos.contiguous();
  const auto sc = sin.contiguous();
  auto q_out = at::empty({tokens, q_heads, head_dim}, q.options());
  auto k_out = at::empty({tokens, kv_heads, head_dim}, k.options());
  if (tokens == 0) return {q_out, k_out};
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  check_rc(llmq_rope_qk(q.const_data_ptr(), k.const_data_ptr(), cc.const_data_ptr(), sc.const_data_ptr(),
                        q_out.mutable_data_ptr(), k_out.mutable_data_ptr(), static_cast<int>(tokens),
                        static_cast<int>(q_heads), static_cast<int>(kv_heads), static_cast<int>(head_dim), q.stride(0),
                        k.stride(0), dtype_code(q, "q"), current_stream(q)),
           "rope_qk");
  return {q_out, k_out};
}

// gate, up: same shape; 2-D inputs may be column blocks of a wider tensor (row strides, contiguous last axis).
at::Tensor silu_mul(const at::Tensor& gate, const at::Tensor& up) {
  TORCH_CHECK(gate.is_cuda() && up.is_cuda(), "gate and up must be CUDA tensors");
  TORCH_CHECK(gate.sizes() == up.sizes() && gate.scalar_type() == up.scalar_type(), "gate and up must match");
  const bool strided = gate.dim() == 2 && gate.stride(1) == 1 && up.stride(1) == 1;
  const auto gc = strided ? gate : gate.contiguous();
  const auto uc = strided ? up : up.contiguous();
  auto out = at::empty(gate.sizes(), gate.options());
  if (gate.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(gc));
  if (strided) {
    check_rc(llmq_silu_mul_rows(gc.const_data_ptr(), uc.const_data_ptr(), out.mutable_data_ptr(), gc.size(0),
                                static_cast<int>(gc.size(1)), gc.stride(0), uc.stride(0), dtype_code(gc, "gate"),
                                current_stream(gc)),
             "silu_mul");
  } else {
    check_rc(llmq_silu_mul(gc.const_data_ptr(), uc.const_data_ptr(), out.mutable_data_ptr(), gc.numel(),
                           dtype_code(gc, "gate"), current_stream(gc)),
             "silu_mul");
  }
  return out;
}

// ---- quantized KV cache -------------------------------------------------------------------------------
// Cache tensors of one layer: codes [kv_heads, t_max, head_dim] int8 or [kv_heads, t_max,
// head_dim / 2] uint8, scales [kv_heads, t_max] fp32. `position` is a device int32 tensor.

struct CacheGeometry {
  int kv_heads, t_max, head_dim, bits;
};

CacheGeometry cache_geometry(const at::Tensor& codes, const at::Tensor& scale, const char* what) {
  TORCH_CHECK(codes.is_cuda() && scale.is_cuda(), what, " cache tensors must be CUDA");
  TORCH_CHECK(codes.dim() == 3 && codes.is_contiguous(), what, " codes must be contiguous [kv_heads, t_max, head_dim]");
  const bool packed = codes.scalar_type() == at::kByte;
  // (fp16 / bf16 "codes": an unquantized cache, bits 16, which only the split attention step takes)
  const bool unquantized = codes.scalar_type() == at::kHalf || codes.scalar_type() == at::kBFloat16;
  TORCH_CHECK(packed || unquantized || codes.scalar_type() == at::kChar, what, " codes must be int8, or uint8 for 4-bit");
  TORCH_CHECK(scale.scalar_type() == at::kFloat && scale.is_contiguous() && scale.dim() == 2 &&
                  scale.size(0) == codes.size(0) && scale.size(1) == codes.size(1),
              what, " scales must be contiguous float32 [kv_heads, t_max]");
  return {static_cast<int>(codes.size(0)), static_cast<int>(codes.size(1)),
          static_cast<int>(packed ? codes.size(2) * 2 : codes.size(2)), unquantized ? 16 : (packed ? 4 : 8)};
}

void check_position(const at::Tensor& position) {
  TORCH_CHECK(position.is_cuda() && position.scalar_type() == at::kInt && position.numel() >= 1,
              "position must be a CUDA int32 tensor");
}

// key / value: [kv_heads, n_new, head_dim] views (last axis contiguous, both with the same
// strides). Returns the dequantized new tokens when asked, else two empty tensors.
std::tuple<at::Tensor, at::Tensor> kv_append(const at::Tensor& key, const at::Tensor& value,
                                             at::Tensor& k_codes, at::Tensor& v_codes, at::Tensor& k_scale,
                                             at::Tensor& v_scale, const at::Tensor& position,
                                             bool return_dequantized) {
  TORCH_CHECK(key.is_cuda() && value.is_cuda(), "key and value must be CUDA tensors");
  TORCH_CHECK(key.dim() == 3 && value.sizes() == key.sizes() && value.strides() == key.strides() &&
                  key.scalar_type() == value.scalar_type(),
              "key and value must be [kv_heads, n_new, head_dim] with equal shapes, strides and dtypes");
  TORCH_CHECK(key.stride(2) == 1 || key.size(2) == 1, "the head_dim axis must be contiguous");
  const int dtype = dtype_code(key, "key");
  const CacheGeometry g = cache_geometry(k_codes, k_scale, "key");
  const CacheGeometry gv = cache_geometry(v_codes, v_scale, "value");
  TORCH_CHECK(g.kv_heads == gv.kv_heads && g.t_max == gv.t_max && g.head_dim == gv.head_dim && g.bits == gv.bits,
              "key and value caches differ in geometry");
  TORCH_CHECK(key.size(0) == g.kv_heads && key.size(2) == g.head_dim, "key is [", key.size(0), ", ",
              key.size(1), ", ", key.size(2), "] but the cache holds ", g.kv_heads, " heads of ", g.head_dim);
  check_position(position);
  const int64_t n_new = key.size(1);
  at::Tensor dq_k = at::empty({0}, key.options()), dq_v = at::empty({0}, key.options());
  if (return_dequantized) {
    dq_k = at::empty({g.kv_heads, n_new, g.head_dim}, key.options());
    dq_v = at::empty({g.kv_heads, n_new, g.head_dim}, key.options());
  }
  if (n_new == 0) return std::make_tuple(dq_k, dq_v);
  const c10::OptionalDeviceGuard guard(at::device_of(key));
  check_rc(llmq_kv_append(key.const_data_ptr(), value.const_data_ptr(), key.stride(0), key.stride(1),
                          k_codes.mutable_data_ptr(), v_codes.mutable_data_ptr(),
                          k_scale.mutable_data_ptr<float>(), v_scale.mutable_data_ptr<float>(),
                          return_dequantized ? dq_k.mutable_data_ptr() : nullptr,
                          return_dequantized ? dq_v.mutable_data_ptr() : nullptr,
                          position.const_data_ptr<int32_t>(), static_cast<int>(n_new), g.kv_heads,
                          g.head_dim, g.t_max, g.bits, dtype, current_stream(key)),
           "kv_append");
  return std::make_tuple(dq_k, dq_v);
}

// q [tokens, q_heads*head_dim], k / v [tokens, kv_heads*head_dim]: rows of the projections (column
// slices of one q|k|v output are fine). Returns (q rotated [tokens, q_heads, head_dim], dq_k, dq_v
// [kv_heads, tokens, head_dim]; the last two empty without return_dequantized).
std::tuple<at::Tensor, at::Tensor, at::Tensor> rope_kv_append(
    const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& cos, const at::Tensor& sin,
    at::Tensor& k_codes, at::Tensor& v_codes, at::Tensor& k_scale, at::Tensor& v_scale, const at::Tensor& position,
    int64_t q_heads, bool return_dequantized) {
  TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda() && cos.is_cuda() && sin.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && v.dim() == 2 && q.stride(1) == 1 && k.stride(1) == 1 && v.stride(1) == 1,
              "q, k and v must be [tokens, heads * head_dim] with a contiguous last axis");
  const int dtype = dtype_code(q, "q");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type() &&
                  cos.scalar_type() == q.scalar_type() && sin.scalar_type() == q.scalar_type(),
              "q, k, v, cos and sin must share a dtype");
  const CacheGeometry g = cache_geometry(k_codes, k_scale, "key");
  const CacheGeometry gv = cache_geometry(v_codes, v_scale, "value");
  TORCH_CHECK(g.kv_heads == gv.kv_heads && g.t_max == gv.t_max && g.head_dim == gv.head_dim && g.bits == gv.bits,
              "key and value caches differ in geometry");
  const int64_t tokens = q.size(0);
  TORCH_CHECK(q_heads > 0 && q.size(1) == q_heads * g.head_dim, "q has ", q.size(1), " columns, expected ",
              q_heads * g.head_dim);
  TORCH_CHECK(k.size(0) == tokens && v.size(0) == tokens && k.size(1) == g.kv_heads * g.head_dim &&
                  v.size(1) == k.size(1),
              "k and v must be [", tokens, ", ", g.kv_heads * g.head_dim, "]");
  TORCH_CHECK(cos.dim() == 2 && cos.is_contiguous() && sin.is_contiguous() && cos.sizes() == sin.sizes() &&
                  cos.size(0) == tokens && cos.size(1) == g.head_dim,
              "cos and sin must be contiguous [tokens, head_dim]");
  check_position(position);
  auto q_out = at::empty({tokens, q_heads, g.head_dim}, q.options());
  at::Tensor dq_k = at::empty({0}, q.options()), dq_v = at::empty({0}, q.options());
  if (return_dequantized) {
    dq_k = at::empty({g.kv_heads, tokens, g.head_dim}, q.options());
    dq_v = at::empty({g.kv_heads, tokens, g.head_dim}, q.options());
  }
  if (tokens == 0) return std::make_tuple(q_out, dq_k, dq_v);
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  check_rc(llmq_rope_kv_append(q.const_data_ptr(), k.const_data_ptr(), v.const_data_ptr(), q.stride(0), k.stride(0),
                               v.stride(0), cos.const_data_ptr(), sin.const_data_ptr(), q_out.mutable_data_ptr(),
                               k_codes.mutable_data_ptr(), v_codes.mutable_data_ptr(),
                               k_scale.mutable_data_ptr<float>(), v_scale.mutable_data_ptr<float>(),
                               return_dequantized ? dq_k.mutable_data_ptr() : nullptr,
                               return_dequantized ? dq_v.mutable_data_ptr() : nullptr,
                               position.const_data_ptr<int32_t>(), static_cast<int>(tokens),
                               static_cast<int>(q_heads), g.kv_heads, g.head_dim, g.t_max, g.bits, dtype,
                               current_stream(q)),
           "rope_kv_append");
  return std::make_tuple(q_out, dq_k, dq_v);
}

at::Tensor kv_dequant(const at::Tensor& codes, const at::Tensor& scale, int64_t n_tokens,
                      at::ScalarType out_dtype) {
  const CacheGeometry g = cache_geometry(codes, scale, "cache");
  TORCH_CHECK(n_tokens >= 0 && n_tokens <= g.t_max, "n_tokens ", n_tokens, " outside [0, ", g.t_max, "]");
  auto out = at::empty({g.kv_heads, n_tokens, g.head_dim}, codes.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  if (out.numel() == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(codes));
  check_rc(llmq_kv_dequant(codes.const_data_ptr(), scale.const_data_ptr<float>(), out.mutable_data_ptr(),
                           g.kv_heads, g.head_dim, g.t_max, static_cast<int>(n_tokens), g.bits, dtype,
                           current_stream(codes)),
           "kv_dequant");
  return out;
}

int64_t kv_decode_workspace_floats(int64_t q_heads, int64_t head_dim, int64_t t_max) {
  return static_cast<int64_t>(llmq_kv_decode_workspace_floats(static_cast<int>(q_heads),
                                                              static_cast<int>(head_dim),
                                                              static_cast<int>(t_max)));
}

// query: [q_heads, head_dim]; length: device int32, tokens valid in the cache. Returns [q_heads, head_dim].
at::Tensor kv_decode_attention(const at::Tensor& query, const at::Tensor& k_codes, const at::Tensor& v_codes,
                               const at::Tensor& k_scale, const at::Tensor& v_scale, at::Tensor& workspace,
                               const at::Tensor& length, double sm_scale) {
  TORCH_CHECK(query.is_cuda(), "query must be a CUDA tensor");
  TORCH_CHECK(query.dim() == 2 && query.is_contiguous(), "query must be contiguous [q_heads, head_dim]");
  const int dtype = dtype_code(query, "query");
  const CacheGeometry g = cache_geometry(k_codes, k_scale, "key");
  const CacheGeometry gv = cache_geometry(v_codes, v_scale, "value");
  TORCH_CHECK(g.kv_heads == gv.kv_heads && g.t_max == gv.t_max && g.head_dim == gv.head_dim && g.bits == gv.bits,
              "key and value caches differ in geometry");
  TORCH_CHECK(query.size(1) == g.head_dim, "query head_dim ", query.size(1), " != cache head_dim ", g.head_dim);
  const int q_heads = static_cast<int>(query.size(0));
  check_position(length);
  TORCH_CHECK(workspace.is_cuda() && workspace.scalar_type() == at::kFloat && workspace.is_contiguous() &&
                  workspace.numel() >= kv_decode_workspace_floats(q_heads, g.head_dim, g.t_max),
              "workspace must be a contiguous CUDA float32 tensor of at least kv_decode_workspace_floats() elements");
  auto out = at::empty_like(query);
  const c10::OptionalDeviceGuard guard(at::device_of(query));
  check_rc(llmq_kv_decode_attention(query.const_data_ptr(), k_codes.const_data_ptr(), v_codes.const_data_ptr(),
                                    k_scale.const_data_ptr<float>(), v_scale.const_data_ptr<float>(),
                                    out.mutable_data_ptr(), workspace.mutable_data_ptr<float>(),
                                    length.const_data_ptr<int32_t>(), static_cast<float>(sm_scale), q_heads,
                                    g.kv_heads, g.head_dim, g.t_max, g.bits, dtype, current_stream(query)),
           "kv_decode_attention");
  return out;
}

// qkv: [(q_heads + 2*kv_heads) * head_dim]; returns the attention output [1, q_heads * head_dim].
at::Tensor kv_rope_append_attend(const at::Tensor& qkv, const at::Tensor& cos_table, const at::Tensor& sin_table,
                                 at::Tensor& k_codes, at::Tensor& v_codes, at::Tensor& k_scale, at::Tensor& v_scale,
                                 const at::Tensor& position, double sm_scale, int64_t q_heads) {
  TORCH_CHECK(qkv.is_cuda() && qkv.is_contiguous(), "qkv must be a contiguous CUDA tensor");
  const int dtype = dtype_code(qkv, "qkv");
  const CacheGeometry g = cache_geometry(k_codes, k_scale, "key");
  const CacheGeometry gv = cache_geometry(v_codes, v_scale, "value");
  TORCH_CHECK(g.kv_heads == gv.kv_heads && g.t_max == gv.t_max && g.head_dim == gv.head_dim && g.bits == gv.bits,
              "key and value caches differ in geometry");
  TORCH_CHECK(qkv.numel() == (q_heads + 2 * g.kv_heads) * g.head_dim, "qkv has ", qkv.numel(), " elements, expected ",
              (q_heads + 2 * g.kv_heads) * g.head_dim);
  for (const at::Tensor* t : {&cos_table, &sin_table}) {
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->dim() == 2 && t->size(1) == g.head_dim &&
                    t->size(0) >= g.t_max && t->scalar_type() == qkv.scalar_type(),
                "cos/sin tables must be contiguous [>= t_max, head_dim] tensors of qkv's dtype");
  }
  check_position(position);
  auto out = at::empty({1, q_heads * g.head_dim}, qkv.options());
  const c10::OptionalDeviceGuard guard(at::device_of(qkv));
  check_rc(llmq_kv_rope_append_attend(qkv.const_data_ptr(), cos_table.const_data_ptr(), sin_table.const_data_ptr(),
                                      k_codes.mutable_data_ptr(), v_codes.mutable_data_ptr(),
                                      k_scale.mutable_data_ptr<float>(), v_scale.mutable_data_ptr<float>(),
                                      out.mutable_data_ptr(), position.const_data_ptr<int32_t>(),
                                      static_cast<float>(sm_scale), static_cast<int>(q_heads), g.kv_heads,
                                      g.head_dim, g.t_max, g.bits, dtype, current_stream(qkv)),
           "kv_rope_append_attend");
  return out;
}

// The split form: fills `partials` (fp32, at least kv_attend_partials_floats(...) elements) and returns it.
at::Tensor kv_rope_append_attend_split(const at::Tensor& qkv, const at::Tensor& cos_table,
                                       const at::Tensor& sin_table, at::Tensor& k_codes, at::Tensor& v_codes,
                                       at::Tensor& k_scale, at::Tensor& v_scale, at::Tensor& partials,
                                       const at::Tensor& position, double sm_scale, int64_t q_heads,
                                       int64_t n_splits) {
  TORCH_CHECK(qkv.is_cuda() && qkv.is_contiguous(), "qkv must be a contiguous CUDA tensor");
  const int dtype = dtype_code(qkv, "qkv");
  const CacheGeometry g = cache_geometry(k_codes, k_scale, "key");
  const CacheGeometry gv = cache_geometry(v_codes, v_scale, "value");
  TORCH_CHECK(g.kv_heads == gv.kv_heads && g.t_max == gv.t_max && g.head_dim == gv.head_dim && g.bits == gv.bits,
              "key and value caches differ in geometry");
  TORCH_CHECK(qkv.numel() == (q_heads + 2 * g.kv_heads) * g.head_dim, "qkv has ", qkv.numel(), " elements, expected ",
              (q_heads + 2 * g.kv_heads) * g.head_dim);
  for (const at::Tensor* t : {&cos_table, &sin_table}) {
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->dim() == 2 && t->size(1) == g.head_dim &&
                    t->size(0) >= g.t_max && t->scalar_type() == qkv.scalar_type(),
                "cos/sin tables must be contiguous [>= t_max, head_dim] tensors of qkv's dtype");
  }
  check_position(position);
  TORCH_CHECK(g.bits != 16 || k_codes.scalar_type() == qkv.scalar_type(),
              "an unquantized cache must hold values of qkv's dtype");
  TORCH_CHECK(n_splits >= 1 && n_splits <= 256, "n_splits must be in [1, 256], got ", n_splits);
  const auto need = static_cast<int64_t>(llmq_kv_attend_partials_floats(static_cast<int>(q_heads), g.head_dim,
                                                                        static_cast<int>(n_splits)));
  TORCH_CHECK(partials.is_cuda() && partials.is_contiguous() && partials.scalar_type() == at::kFloat &&
                  partials.numel() >= need,
              "partials must be a contiguous CUDA float32 tensor of at least ", need, " elements");
  const c10::OptionalDeviceGuard guard(at::device_of(qkv));
  check_rc(llmq_kv_rope_append_attend_split(
               qkv.const_data_ptr(), cos_table.const_data_ptr(), sin_table.const_data_ptr(), k_codes.mutable_data_ptr(),
               v_codes.mutable_data_ptr(), k_scale.mutable_data_ptr<float>(), v_scale.mutable_data_ptr<float>(),
               partials.mutable_data_ptr<float>(), position.const_data_ptr<int32_t>(), static_cast<float>(sm_scale),
               static_cast<int>(q_heads), g.kv_heads, g.head_dim, g.t_max, g.bits, static_cast<int>(n_splits), dtype,
               current_stream(qkv)),
           "kv_rope_append_attend_split");
  return partials;
}

at::Tensor kv_attend_merge(const at::Tensor& partials, int64_t q_heads, int64_t head_dim, int64_t n_splits,
                           at::ScalarType out_dtype) {
  TORCH_CHECK(partials.is_cuda() && partials.is_contiguous() && partials.scalar_type() == at::kFloat,
              "partials must be a contiguous CUDA float32 tensor");
  TORCH_CHECK(q_heads >= 0 && head_dim > 0 && n_splits >= 1, "bad sizes");
  TORCH_CHECK(partials.numel() >= static_cast<int64_t>(llmq_kv_attend_partials_floats(
                                      static_cast<int>(q_heads), static_cast<int>(head_dim), static_cast<int>(n_splits))),
              "partials is too small for ", q_heads, " heads x ", n_splits, " splits");
  auto out = at::empty({1, q_heads * head_dim}, partials.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  const c10::OptionalDeviceGuard guard(at::device_of(partials));
  check_rc(llmq_kv_attend_merge(partials.const_data_ptr<float>(), out.mutable_data_ptr(), static_cast<int>(q_heads),
                                static_cast<int>(head_dim), static_cast<int>(n_splits), dtype, current_stream(partials)),
           "kv_attend_merge");
  return out;
}

// The GEMV that consumes split attention: activation = out_dtype(merge(partials)), [q_heads * head_dim].
at::Tensor wq_gemv_attn_merge(const at::Tensor& partials, int64_t n_splits, int64_t head_dim,
                              const at::Tensor& qweight, const at::Tensor& wscale, int64_t out_group,
                              int64_t in_head_dim, const c10::optional<at::Tensor>& residual,
                              at::ScalarType out_dtype) {
  TORCH_CHECK(partials.is_cuda() && qweight.is_cuda() && wscale.is_cuda(), "all tensors must be CUDA");
  TORCH_CHECK(partials.is_contiguous() && partials.scalar_type() == at::kFloat, "partials must be contiguous float32");
  TORCH_CHECK(qweight.dim() == 3 && qweight.is_contiguous(), "qweight must be contiguous [N, groups, group_size]");
  const bool packed = qweight.scalar_type() == at::kByte;
  TORCH_CHECK(packed || qweight.scalar_type() == at::kChar, "qweight must be int8, or uint8 for nibble-packed int4");
  TORCH_CHECK(wscale.scalar_type() == at::kFloat && wscale.dim() == 2 && wscale.is_contiguous(),
              "wscale must be contiguous float32 [scale_rows, groups]");
  const int64_t N = qweight.size(0), groups = qweight.size(1);
  const int64_t group_size = packed ? qweight.size(2) * 2 : qweight.size(2);
  TORCH_CHECK(group_size == 128, "the fused GEMV needs group_size 128, got ", group_size);
  const int64_t k_real = in_head_dim > 0 ? groups * in_head_dim : groups * group_size;
  TORCH_CHECK(head_dim > 0 && k_real % head_dim == 0, "input width ", k_real, " is not a whole number of heads of ", head_dim);
  TORCH_CHECK(n_splits >= 1 && partials.numel() >= static_cast<int64_t>(llmq_kv_attend_partials_floats(
                                   static_cast<int>(k_real / head_dim), static_cast<int>(head_dim), static_cast<int>(n_splits))),
              "partials is too small for ", k_real / head_dim, " heads x ", n_splits, " splits");
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  TORCH_CHECK(wscale.size(0) == scale_rows && wscale.size(1) == groups, "wscale must be [", scale_rows, ", ", groups, "]");
  auto out = at::empty({1, N}, partials.options().dtype(out_dtype));
  const int dtype = dtype_code(out, "output dtype");
  const void* res_ptr = nullptr;
  if (residual.has_value() && residual->defined()) {
    TORCH_CHECK(residual->is_cuda() && residual->is_contiguous() && residual->numel() == N &&
                    residual->scalar_type() == out_dtype,
                "residual must be a contiguous tensor of the output dtype with ", N, " elements");
    res_ptr = residual->const_data_ptr();
  }
  if (N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(partials));
  check_rc(llmq_wq_gemv_attn_merge(partials.const_data_ptr<float>(), static_cast<int>(n_splits),
                                   static_cast<int>(head_dim), qweight.const_data_ptr(),
                                   wscale.const_data_ptr<float>(), out.mutable_data_ptr(), static_cast<int>(N),
                                   static_cast<int>(groups), static_cast<int>(out_group),
                                   packed ? LLMQ_W_INT4_PACKED : LLMQ_W_INT8, dtype, static_cast<int>(in_head_dim),
                                   res_ptr, current_stream(partials)),
           "wq_gemv_attn_merge");
  return out;
}

// The decode-step GEMV over an unquantized fp16 / bf16 weight [N, K] (the 16-bit baseline's kernel).
// prologue 0 / 1 (RMSNorm): x is [1, K]; prologue 3 (attention merge): x is the fp32 records of split
// attention, n_splits per head of head_dim. pair_half > 0: weight is gate rows over up rows, out [1, pair_half].
at::Tensor dense_gemv_fused(const at::Tensor& x, const at::Tensor& weight, int64_t prologue,
                            const c10::optional<at::Tensor>& norm_weight, double eps,
                            const c10::optional<at::Tensor>& residual, int64_t pair_half, int64_t n_splits,
                            int64_t head_dim) {
  TORCH_CHECK(x.is_cuda() && weight.is_cuda(), "x and weight must be CUDA tensors");
  TORCH_CHECK(weight.dim() == 2 && weight.is_contiguous(), "weight must be contiguous [N, K]");
  TORCH_CHECK(weight.scalar_type() == at::kHalf || weight.scalar_type() == at::kBFloat16,
              "weight must be float16 or bfloat16");
  TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
  const int64_t N = weight.size(0), K = weight.size(1);
  const bool merge = prologue == LLMQ_PRO_ATTN_MERGE;
  if (merge) {
    TORCH_CHECK(x.scalar_type() == at::kFloat && head_dim > 0 && K % head_dim == 0 && n_splits >= 1 &&
                    x.numel() >= static_cast<int64_t>(llmq_kv_attend_partials_floats(
                                     static_cast<int>(K / head_dim), static_cast<int>(head_dim), static_cast<int>(n_splits))),
                "the attention-merge prologue takes the float32 records of ", K / std::max<int64_t>(head_dim, 1), " heads x ",
                n_splits, " splits");
  } else {
    TORCH_CHECK(x.scalar_type() == weight.scalar_type() && x.numel() == K, "x must be [1, ", K, "] of the weight's dtype");
  }
  const void* norm_ptr = nullptr;
  if (prologue == LLMQ_PRO_RMSNORM) {
    TORCH_CHECK(norm_weight.has_value() && norm_weight->defined() && norm_weight->is_cuda() &&
                    norm_weight->is_contiguous() && norm_weight->numel() == K &&
                    norm_weight->scalar_type() == weight.scalar_type(),
                "the RMSNorm prologue needs norm_weight [", K, "] of the weight's dtype");
    norm_ptr = norm_weight->const_data_ptr();
  }
  const int64_t n_out = pair_half > 0 ? pair_half : N;
  const void* res_ptr = nullptr;
  if (residual.has_value() && residual->defined()) {
    TORCH_CHECK(residual->is_cuda() && residual->is_contiguous() && residual->numel() == n_out &&
                    residual->scalar_type() == weight.scalar_type(),
                "residual must be a contiguous tensor of the weight's dtype with ", n_out, " elements");
    res_ptr = residual->const_data_ptr();
  }
  auto out = at::empty({1, n_out}, weight.options());
  const int dtype = dtype_code(weight, "weight");
  if (N == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(weight));
  check_rc(llmq_dense_gemv_fused(x.const_data_ptr(), weight.const_data_ptr(), out.mutable_data_ptr(),
                                 static_cast<int>(N), static_cast<int>(K), dtype, static_cast<int>(prologue), norm_ptr,
                                 static_cast<float>(eps), res_ptr, static_cast<int>(pair_half),
                                 static_cast<int>(n_splits), static_cast<int>(head_dim), current_stream(weight)),
           "dense_gemv_fused");
  return out;
}

// x: one row (any shape, contiguous); returns a [1] int64 tensor with the index of its first maximum.
at::Tensor argmax_row(const at::Tensor& x) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && x.numel() > 0, "x must be a non-empty contiguous CUDA tensor");
  const int dtype = dtype_code(x, "x");
  auto out = at::empty({1}, x.options().dtype(at::kLong));
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_argmax_row(x.const_data_ptr(), static_cast<int>(x.numel()), out.mutable_data_ptr<int64_t>(), dtype,
                           current_stream(x)),
           "argmax_row");
  return out;
}

// Causal grouped-query attention of a prompt. q [tokens, q_heads, head_dim]; k, v [kv_heads, tokens, head_dim]
// (contiguous, fp16 / bf16, head_dim 64 or 128) -> [tokens, q_heads * head_dim].
at::Tensor prefill_attention(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, double scale) {
  TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), "q, k, v must be CUDA tensors");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, "q must be [tokens, q_heads, head_dim], k and v [kv_heads, tokens, head_dim]");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(), "q, k, v must share a dtype");
  TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q, k, v must be float16 or bfloat16");
  const auto qc = q.contiguous(), kc = k.contiguous(), vc = v.contiguous();
  const int64_t tokens = qc.size(0), q_heads = qc.size(1), head_dim = qc.size(2), kv_heads = kc.size(0);
  TORCH_CHECK(kc.size(1) == tokens && kc.size(2) == head_dim && vc.sizes() == kc.sizes(),
              "k and v must be [kv_heads, ", tokens, ", ", head_dim, "]");
  auto out = at::empty({tokens, q_heads * head_dim}, qc.options());
  if (tokens == 0) return out;
  const c10::OptionalDeviceGuard guard(at::device_of(qc));
  check_rc(llmq_prefill_attention(qc.const_data_ptr(), kc.const_data_ptr(), vc.const_data_ptr(), out.mutable_data_ptr(),
                                  static_cast<int>(tokens), static_cast<int>(q_heads), static_cast<int>(kv_heads),
                                  static_cast<int>(head_dim), static_cast<float>(scale), dtype_code(qc, "q"),
                                  current_stream(qc)),
           "prefill_attention");
  return out;
}

// argmax_advance over 32 workgroups, and the winner's row of the embedding table copied to hidden_out (both or
// neither of embed / hidden_out). workspace: int32 zeros of argmax_workspace_ints() elements, kept by the caller.
at::Tensor argmax_advance_embed(const at::Tensor& x, at::Tensor& token, at::Tensor& step64, at::Tensor& step32,
                                const c10::optional<at::Tensor>& embed, const c10::optional<at::Tensor>& hidden_out,
                                at::Tensor& workspace) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && x.numel() > 0, "x must be a non-empty contiguous CUDA tensor");
  TORCH_CHECK(token.is_cuda() && token.scalar_type() == at::kLong && token.numel() == 1, "token must be one int64");
  TORCH_CHECK(step64.is_cuda() && step64.scalar_type() == at::kLong && step64.numel() == 1, "step64 must be one int64");
  TORCH_CHECK(step32.is_cuda() && step32.scalar_type() == at::kInt && step32.numel() == 1, "step32 must be one int32");
  TORCH_CHECK(workspace.is_cuda() && workspace.is_contiguous() &&
                  static_cast<size_t>(workspace.numel() * workspace.element_size()) >= llmq_argmax_workspace_bytes(),
              "workspace must be a contiguous CUDA tensor of at least ", llmq_argmax_workspace_bytes(), " bytes");
  const bool hand_off = embed.has_value() && embed->defined();
  TORCH_CHECK(hand_off == (hidden_out.has_value() && hidden_out->defined()), "embed and hidden_out go together");
  int64_t hidden = 0;
  if (hand_off) {
    TORCH_CHECK(embed->is_cuda() && embed->is_contiguous() && embed->dim() == 2 && embed->scalar_type() == x.scalar_type(),
                "embed must be a contiguous [vocab, hidden] CUDA tensor of x's dtype");
    TORCH_CHECK(embed->size(0) >= x.numel(), "embed has ", embed->size(0), " rows for ", x.numel(), " logits");
    hidden = embed->size(1);
    TORCH_CHECK(hidden_out->is_cuda() && hidden_out->is_contiguous() && hidden_out->numel() == hidden &&
                    hidden_out->scalar_type() == x.scalar_type(),
                "hidden_out must be a contiguous CUDA tensor of ", hidden, " elements of x's dtype");
  }
  const int dtype = dtype_code(x, "x");
  auto out = at::empty({1}, x.options().dtype(at::kLong));
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_argmax_advance_embed(x.const_data_ptr(), static_cast<int>(x.numel()), out.mutable_data_ptr<int64_t>(),
                                     token.mutable_data_ptr<int64_t>(), step64.mutable_data_ptr<int64_t>(),
                                     step32.mutable_data_ptr<int32_t>(), hand_off ? embed->const_data_ptr() : nullptr,
                                     hand_off ? hidden_out->mutable_data_ptr() : nullptr, static_cast<int>(hidden),
                                     workspace.mutable_data_ptr(), dtype, current_stream(x)),
           "argmax_advance_embed");
  return out;
}

// argmax_row plus: token <- index, step64 += 1, step32 += 1 (one-element int64 / int64 / int32 device tensors).
at::Tensor argmax_advance(const at::Tensor& x, at::Tensor& token, at::Tensor& step64, at::Tensor& step32) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && x.numel() > 0, "x must be a non-empty contiguous CUDA tensor");
  TORCH_CHECK(token.is_cuda() && token.scalar_type() == at::kLong && token.numel() == 1, "token must be one int64");
  TORCH_CHECK(step64.is_cuda() && step64.scalar_type() == at::kLong && step64.numel() == 1, "step64 must be one int64");
  TORCH_CHECK(step32.is_cuda() && step32.scalar_type() == at::kInt && step32.numel() == 1, "step32 must be one int32");
  const int dtype = dtype_code(x, "x");
  auto out = at::empty({1}, x.options().dtype(at::kLong));
  const c10::OptionalDeviceGuard guard(at::device_of(x));
  check_rc(llmq_argmax_advance(x.const_data_ptr(), static_cast<int>(x.numel()), out.mutable_data_ptr<int64_t>(),
                               token.mutable_data_ptr<int64_t>(), step64.mutable_data_ptr<int64_t>(),
                               step32.mutable_data_ptr<int32_t>(), dtype, current_stream(x)),
           "argmax_advance");
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
  m.def("wq_gemv_fused", &wq_gemv_fused,
        "One-row quantized Linear with RMSNorm / SiLU*up prologue, head padding and residual epilogue",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0, py::arg("prologue") = 0,
        py::arg("norm_weight") = py::none(), py::arg("eps") = 0.0, py::arg("in_head_dim") = 0,
        py::arg("residual") = py::none());
  m.def("wq_gemv_batched_fused", &wq_gemv_batched_fused,
        "Batched expert GEMV with the row gather (one token) and silu(gate) * up folded in",
        py::arg("x"), py::arg("broadcast_x"), py::arg("n_rows"), py::arg("qweight"), py::arg("wscale"),
        py::arg("block_expert"), py::arg("block_row0"), py::arg("block_rows"), py::arg("act_pair"));
  m.def("moe_combine", &moe_combine, "Routing-weighted sum of the experts' rows per token",
        py::arg("rows_out"), py::arg("order"), py::arg("weights"), py::arg("n_tokens"));
  m.def("route_plan", &route_plan, "Routing plan of the batched GEMV in one launch",
        py::arg("top_k_index"), py::arg("num_experts"), py::arg("limit"));
  m.def("route_plan_supported", [](int64_t rows, int64_t experts) {
    return rows <= INT32_MAX && experts <= INT32_MAX &&
           llmq_route_plan_supported(static_cast<int>(rows), static_cast<int>(experts)) != 0;
  }, py::arg("rows"), py::arg("num_experts"));
  m.def("wq_gemv_gate_up_silu", &wq_gemv_gate_up_silu,
        "One-row gate|up Linear that stores act(gate) * up, optional RMSNorm prologue",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("prologue") = 0,
        py::arg("norm_weight") = py::none(), py::arg("eps") = 0.0);
  m.def("kv_rope_append_attend", &kv_rope_append_attend,
        "RoPE + KV quantize-append + attention for one decode token of one layer, one launch",
        py::arg("qkv"), py::arg("cos_table"), py::arg("sin_table"), py::arg("k_codes"), py::arg("v_codes"),
        py::arg("k_scale"), py::arg("v_scale"), py::arg("position"), py::arg("sm_scale"), py::arg("q_heads"));
  m.def("argmax_row", &argmax_row, "Index of the first maximum of one row", py::arg("x"));
  m.def("wq_gemm_a8", &wq_gemm_a8,
        "Integer GEMM: int8 activations x int4/int8 group-quantized weights, real-mode rounding order",
        py::arg("a"), py::arg("sx"), py::arg("qweight"), py::arg("wscale"), py::arg("bias") = py::none(),
        py::arg("out_group") = 0, py::arg("out_dtype") = at::kBFloat16, py::arg("exact") = true);
  m.def("quant_act_codes_tiled", &quant_act_codes_tiled,
        "int8 activation codes (groups of 128) in the operand order of wq_gemm_a8_tiled, and their scales",
        py::arg("x"), py::arg("weight_bits"));
  m.def("wq_gemm_a8_tiled", &wq_gemm_a8_tiled,
        "the exact integer GEMM on the codes of quant_act_codes_tiled (group-parallel kernel, no operand staging pass)",
        py::arg("codes"), py::arg("sx"), py::arg("rows"), py::arg("qweight"), py::arg("wscale"),
        py::arg("bias") = py::none(), py::arg("out_group") = 0, py::arg("out_dtype") = at::kBFloat16);
  m.def("wq_gemm_a8_takes_groups", [](int64_t m_rows, int64_t n, int64_t groups) {
          return llmq_wq_gemm_a8_takes_groups(static_cast<int>(m_rows), static_cast<int>(n), static_cast<int>(groups)) != 0;
        }, "whether wq_gemm_a8 (exact) runs its group-parallel kernel for the shape: then wq_gemm_a8_tiled is the faster call",
        py::arg("rows"), py::arg("out_features"), py::arg("groups"));
  m.def("wq_gemm_a16", &wq_gemm_a16,
        "Weight-only GEMM for a few dozen rows: fp16/bf16 activations x int4/int8 group-quantized weights, no dense copy",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0, py::arg("split") = false);
  m.def("wq_gemm_a16_tile_gate_up_silu", &wq_gemm_a16_tile_gate_up_silu,
        "gate|up tiled GEMM whose workgroups write silu(gate) * up as the next tiled GEMM's prepared activation",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0, py::arg("next_n"));
  m.def("wq_gemm_a16_tile_gate_up_silu_prepared", &wq_gemm_a16_tile_gate_up_silu_prepared,
        "wq_gemm_a16_tile_gate_up_silu on the prepared activation add_rmsnorm_prepared left in its workspace",
        py::arg("workspace"), py::arg("rows"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0,
        py::arg("next_n"), py::arg("dtype") = at::kBFloat16);
  m.def("add_rmsnorm_prepared", &add_rmsnorm_prepared,
        "(x + delta, workspace): LlamaRMSNorm(x + delta) written as the prepared activation of a tiled GEMM, one launch",
        py::arg("x"), py::arg("delta"), py::arg("weight"), py::arg("eps"), py::arg("next_n"));
  m.def("wq_gemm_a16_tile_prepared", &wq_gemm_a16_tile_prepared,
        "the tiled GEMM on the prepared activation wq_gemm_a16_tile_gate_up_silu left in its workspace",
        py::arg("workspace"), py::arg("rows"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0,
        py::arg("dtype") = at::kBFloat16);
  m.def("wq_gemm_a16_tile", &wq_gemm_a16_tile,
        "Fused weight-only GEMM for prompt-sized bf16 activations: 128 x 256 tiles on the bf16 matrix cores, no dense weight",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0);
  m.def("rmsnorm", &rmsnorm, "LlamaRMSNorm over the last axis, one launch", py::arg("x"), py::arg("weight"), py::arg("eps"));
  m.def("add_rmsnorm", &add_rmsnorm, "(x + delta, LlamaRMSNorm(x + delta)), one launch", py::arg("x"), py::arg("delta"),
        py::arg("weight"), py::arg("eps"));
  m.def("rope_qk", &rope_qk, "apply_rotary_pos_emb on the q and k projections of a prompt, one launch",
        py::arg("q"), py::arg("k"), py::arg("cos"), py::arg("sin"), py::arg("q_heads"), py::arg("kv_heads"));
  m.def("silu_mul", &silu_mul, "silu(gate) * up with both roundings, one launch", py::arg("gate"), py::arg("up"));
  m.def("kv_append", &kv_append,
        "Quantize new K/V tokens into one layer's cache at the device-side position",
        py::arg("key"), py::arg("value"), py::arg("k_codes"), py::arg("v_codes"), py::arg("k_scale"),
        py::arg("v_scale"), py::arg("position"), py::arg("return_dequantized") = false);
  m.def("rope_kv_append", &rope_kv_append,
        "Prompt pass: RoPE on q and k, then quantize-and-append of k and v, in one launch (rope_qk + kv_append, same bits)",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("cos"), py::arg("sin"), py::arg("k_codes"),
        py::arg("v_codes"), py::arg("k_scale"), py::arg("v_scale"), py::arg("position"), py::arg("q_heads"),
        py::arg("return_dequantized") = false);
  m.def("kv_dequant", &kv_dequant, "Dequantize the first n_tokens of one layer's cache",
        py::arg("codes"), py::arg("scale"), py::arg("n_tokens"), py::arg("out_dtype"));
  m.def("kv_decode_workspace_floats", &kv_decode_workspace_floats, py::arg("q_heads"),
        py::arg("head_dim"), py::arg("t_max"));
  m.def("kv_decode_attention", &kv_decode_attention,
        "Single-token GQA attention reading the quantized cache",
        py::arg("query"), py::arg("k_codes"), py::arg("v_codes"), py::arg("k_scale"), py::arg("v_scale"),
        py::arg("workspace"), py::arg("length"), py::arg("sm_scale"));
  m.def("wq_gemv_batched", &wq_gemv_batched,
        "One launch over every routed expert: rows block_row0[b].. of x through expert block_expert[b]",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("block_expert"), py::arg("block_row0"),
        py::arg("block_rows"), py::arg("out_group") = 0);
  m.def("wq_gemv_batched_max_rows", []() { return llmq_wq_gemv_batched_max_rows(); });
  m.def("dequant_weight", &dequant_weight,
        "Dense [N, groups*keep_per_group] matrix of a quantized weight (keep_per_group <= 0: whole groups)",
        py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0, py::arg("keep_per_group") = 0,
        py::arg("out_dtype") = at::kBFloat16);
  m.def("dense_linear", &dense_linear,
        "x [M, K] @ w [N, K].T for float16 / bfloat16 through hipBLASLt with the descriptors and the heuristic's "
        "choice kept per shape (the same algorithm, and bits, as torch's matmul at half the host time)",
        py::arg("x"), py::arg("w"));
  m.def("wq_dense_linear", &wq_dense_linear,
        "The dense branch in one call: dequant_weight into x's dtype, then dense_linear",
        py::arg("x"), py::arg("qweight"), py::arg("wscale"), py::arg("out_group") = 0, py::arg("keep_per_group") = 0);
  m.def("kv_attend_partials_floats", [](int64_t q_heads, int64_t head_dim, int64_t n_splits) {
    return static_cast<int64_t>(llmq_kv_attend_partials_floats(static_cast<int>(q_heads), static_cast<int>(head_dim),
                                                               static_cast<int>(n_splits)));
  }, py::arg("q_heads"), py::arg("head_dim"), py::arg("n_splits"));
  m.def("dense_gemv_fused", &dense_gemv_fused, py::arg("x"), py::arg("weight"), py::arg("prologue") = 0,
        py::arg("norm_weight") = py::none(), py::arg("eps") = 0.0, py::arg("residual") = py::none(),
        py::arg("pair_half") = 0, py::arg("n_splits") = 0, py::arg("head_dim") = 0,
        "Decode-step GEMV over an unquantized fp16 / bf16 weight with the fused step's prologues and epilogues");
  m.def("kv_rope_append_attend_split", &kv_rope_append_attend_split,
        "RoPE + quantize-append + attention spread over n_splits workgroups per head; fills and returns partials",
        py::arg("qkv"), py::arg("cos_table"), py::arg("sin_table"), py::arg("k_codes"), py::arg("v_codes"),
        py::arg("k_scale"), py::arg("v_scale"), py::arg("partials"), py::arg("position"), py::arg("sm_scale"),
        py::arg("q_heads"), py::arg("n_splits"));
  m.def("kv_attend_merge", &kv_attend_merge, py::arg("partials"), py::arg("q_heads"), py::arg("head_dim"),
        py::arg("n_splits"), py::arg("out_dtype") = at::kBFloat16);
  m.def("wq_gemv_attn_merge", &wq_gemv_attn_merge,
        "GEMV whose activation is the merged split-attention output",
        py::arg("partials"), py::arg("n_splits"), py::arg("head_dim"), py::arg("qweight"), py::arg("wscale"),
        py::arg("out_group") = 0, py::arg("in_head_dim") = 0, py::arg("residual") = py::none(),
        py::arg("out_dtype") = at::kBFloat16);
  m.def("prefill_attention", &prefill_attention, "causal grouped-query attention of a prompt on the matrix core",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale"));
  m.def("argmax_advance_embed", &argmax_advance_embed,
        "argmax_advance over 32 workgroups; with embed / hidden_out also hidden_out <- embed[index]", py::arg("x"),
        py::arg("token"), py::arg("step64"), py::arg("step32"), py::arg("embed") = py::none(),
        py::arg("hidden_out") = py::none(), py::arg("workspace"));
  m.def("argmax_workspace_ints", []() { return static_cast<int64_t>((llmq_argmax_workspace_bytes() + 3) / 4); },
        "elements of the int32 zeros tensor argmax_advance_embed takes as workspace");
  m.def("argmax_advance", &argmax_advance, "argmax_row, then token <- index, step64 += 1, step32 += 1",
        py::arg("x"), py::arg("token"), py::arg("step64"), py::arg("step32"));
  m.def("abi_version", []() { return llmq_abi_version(); });
}
