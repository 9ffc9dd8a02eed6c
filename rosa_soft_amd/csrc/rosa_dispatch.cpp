// PyTorch dispatcher layer of the MI355X rosa_soft operators (module rosa_soft_amd._C).
//
// Declares the four `rosa_soft::` operator schemas, byte for byte those of the
// reference (rosa_soft/csrc/export.cpp:24-31), and registers their device
// implementations under the CUDA dispatch key, which is the key HIP tensors
// carry in PyTorch-ROCm (reference: rosa_soft/csrc/rosa_soft.cpp:542-549).
// The implementations validate like the reference's boundary
// (rosa_soft.cpp:84-374: same conditions, same message texts), make inputs
// contiguous, narrow the scalars to float32, allocate outputs and workspace
// with ATen, and hand raw pointers plus the current HIP stream to the C ABI of
// librosa_soft_hip.so.  No device code lives in this file.  (PyTorch-ROCm labels
// HIP devices "cuda", so the device guard and stream accessors used here are
// its HIP classes that carry that label.)

#include <ATen/Context.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <Python.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <tuple>

#include "../../include/rosa_soft_hip.h"

namespace {

using torch::Tensor;
using Triple = std::tuple<Tensor, Tensor, Tensor>;

constexpr int64_t kIndexMargin = 128;
constexpr int64_t kIntMax = std::numeric_limits<int>::max();

int dtype_code(c10::ScalarType dtype) {
  switch (dtype) {
    case torch::kFloat32: return ROSA_DTYPE_F32;
    case torch::kFloat16: return ROSA_DTYPE_F16;
    case torch::kBFloat16: return ROSA_DTYPE_BF16;
    default: return -1;
  }
}

struct Scalars {
  float scale, dropout_p, inverse_keep, mismatch_scale;
};

float positive_normal_float(double value, const char* name) {
  const float narrowed = static_cast<float>(value);
  TORCH_CHECK(narrowed > 0.0f && std::isnormal(narrowed), name,
              " must be representable as a positive normal float32 value");
  return narrowed;
}

Scalars narrow_scalars(int64_t horizon, double scale, double dropout_p, double mismatch_scale) {
  TORCH_CHECK(std::isfinite(scale) && scale > 0.0, "scale must be finite and > 0");
  TORCH_CHECK(std::isfinite(dropout_p) && dropout_p >= 0.0 &&
                  dropout_p <= 1.0 - std::ldexp(1.0, -24),
              "dropout_p must be finite and in [0, 1 - 2^-24]");
  TORCH_CHECK(std::isfinite(mismatch_scale) && mismatch_scale > 0.0,
              "mismatch_scale must be finite and > 0");
  Scalars s;
  s.scale = positive_normal_float(scale, "scale");
  s.dropout_p = static_cast<float>(dropout_p);
  s.inverse_keep = 1.0f / (1.0f - s.dropout_p);
  const double float_max = static_cast<double>(std::numeric_limits<float>::max());
  TORCH_CHECK(scale <= float_max / static_cast<double>(horizon),
              "max_suffix_length * scale must fit in float32");
  s.mismatch_scale = positive_normal_float(mismatch_scale, "mismatch_scale");
  TORCH_CHECK(mismatch_scale <= float_max / (static_cast<double>(horizon) * scale),
              "mismatch_scale * max_suffix_length * scale must fit in float32");
  return s;
}

void check_device_float_inputs(const Tensor& query, const Tensor& key, const Tensor& value) {
  TORCH_CHECK(query.is_cuda(), "query must be a CUDA tensor");
  TORCH_CHECK(key.is_cuda(), "key must be a CUDA tensor");
  TORCH_CHECK(value.is_cuda(), "value must be a CUDA tensor");
  TORCH_CHECK(dtype_code(query.scalar_type()) >= 0,
              "query must be float32, float16, or bfloat16");
  TORCH_CHECK(query.scalar_type() == key.scalar_type(), "query/key dtype mismatch");
  TORCH_CHECK(query.scalar_type() == value.scalar_type(), "query/value dtype mismatch");
}

void check_dense(const Tensor& query, const Tensor& key, const Tensor& value, int64_t horizon) {
  check_device_float_inputs(query, key, value);
  TORCH_CHECK(query.device() == key.device(), "query and key must be on the same CUDA device");
  TORCH_CHECK(query.device() == value.device(),
              "query and value must be on the same CUDA device");
  TORCH_CHECK(query.dim() == 4, "query must have shape (B, T, H, D)");
  TORCH_CHECK(key.dim() == 4, "key must have shape (B, T, H, D)");
  TORCH_CHECK(value.dim() == 4, "value must have shape (B, T, H_p, D_p)");
  TORCH_CHECK(query.size(0) > 0, "batch size must be positive");
  TORCH_CHECK(query.size(1) > 0, "sequence length must be positive");
  TORCH_CHECK(query.size(2) > 0, "query head count must be positive");
  TORCH_CHECK(value.size(2) > 0, "value head count must be positive");
  TORCH_CHECK(value.size(3) > 0, "value dimension must be positive");
  TORCH_CHECK(query.size(0) == key.size(0), "query/key batch mismatch");
  TORCH_CHECK(query.size(1) == key.size(1), "query/key sequence mismatch");
  TORCH_CHECK(query.size(2) == key.size(2), "query/key head mismatch");
  TORCH_CHECK(query.size(3) == key.size(3), "query/key bit dimension mismatch");
  TORCH_CHECK(query.size(0) == value.size(0), "query/value batch mismatch");
  TORCH_CHECK(query.size(1) == value.size(1), "query/value sequence mismatch");
  TORCH_CHECK(query.size(2) % value.size(2) == 0,
              "query heads must be divisible by value heads");
  TORCH_CHECK(query.size(3) > 0 && query.size(3) <= 32,
              "query/key bit dimension must be in [1, 32]");
  TORCH_CHECK(query.numel() / query.size(3) <= kIntMax, "B * T * H must fit in int32");
  TORCH_CHECK(query.size(1) <= kIntMax - kIndexMargin,
              "sequence length is too large for the CUDA kernel index stride");
  TORCH_CHECK(value.size(3) <= kIntMax - kIndexMargin,
              "value dimension is too large for the CUDA kernel index stride");
  TORCH_CHECK(horizon >= 1, "max_suffix_length must be >= 1");
}

void check_packed(const Tensor& query, const Tensor& key, const Tensor& value,
                  const Tensor& cu_seqlens, int64_t horizon) {
  check_device_float_inputs(query, key, value);
  TORCH_CHECK(cu_seqlens.is_cuda(), "cu_seqlens must be a CUDA tensor");
  TORCH_CHECK(query.device() == key.device() && query.device() == value.device() &&
                  query.device() == cu_seqlens.device(),
              "all inputs and cu_seqlens must be on the same CUDA device");
  TORCH_CHECK(query.dim() == 3, "query must have shape (N, H, D)");
  TORCH_CHECK(key.dim() == 3, "key must have shape (N, H, D)");
  TORCH_CHECK(value.dim() == 3, "value must have shape (N, H_p, D_p)");
  TORCH_CHECK(query.size(0) > 0, "packed token count must be positive");
  TORCH_CHECK(query.size(1) > 0, "query head count must be positive");
  TORCH_CHECK(value.size(1) > 0, "value head count must be positive");
  TORCH_CHECK(value.size(2) > 0, "value dimension must be positive");
  TORCH_CHECK(query.size(0) == key.size(0), "query/key token mismatch");
  TORCH_CHECK(query.size(0) == value.size(0), "query/value token mismatch");
  TORCH_CHECK(query.size(1) == key.size(1), "query/key head mismatch");
  TORCH_CHECK(query.size(2) == key.size(2), "query/key bit dimension mismatch");
  TORCH_CHECK(query.size(1) % value.size(1) == 0,
              "query heads must be divisible by value heads");
  TORCH_CHECK(query.size(2) > 0 && query.size(2) <= 32,
              "query/key bit dimension must be in [1, 32]");
  TORCH_CHECK(query.size(0) * query.size(1) <= kIntMax, "N * H must fit in int32");
  TORCH_CHECK(query.size(0) <= kIntMax - kIndexMargin,
              "packed token count is too large for CUDA kernel indexing");
  TORCH_CHECK(value.size(2) <= kIntMax - kIndexMargin,
              "value dimension is too large for the CUDA kernel index stride");
  TORCH_CHECK(cu_seqlens.scalar_type() == torch::kInt32, "cu_seqlens must be int32");
  TORCH_CHECK(cu_seqlens.dim() == 1 && cu_seqlens.numel() >= 2,
              "cu_seqlens must be one-dimensional with at least two entries");
  TORCH_CHECK(cu_seqlens.numel() - 1 <= kIntMax - kIndexMargin,
              "number of packed sequences is too large for CUDA indexing");
  TORCH_CHECK(horizon >= 1, "max_suffix_length must be >= 1");
}

void check_words(const Tensor& words, const Tensor& query, bool packed, const char* name) {
  TORCH_CHECK(words.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(words.device() == query.device(), name,
              " must be on the same CUDA device as query");
  TORCH_CHECK(words.scalar_type() == torch::kInt32, name, " must be int32");
  if (packed) {
    TORCH_CHECK(words.dim() == 2, name, " must have shape (H, N)");
    TORCH_CHECK(words.size(0) == query.size(1) && words.size(1) == query.size(0), name,
                " shape mismatch");
  } else {
    TORCH_CHECK(words.dim() == 3, name, " must have shape (B, H, T)");
    TORCH_CHECK(words.size(0) == query.size(0), name, " batch mismatch");
    TORCH_CHECK(words.size(1) == query.size(2), name, " head mismatch");
    TORCH_CHECK(words.size(2) == query.size(1), name, " sequence mismatch");
  }
}

void check_grad_output(const Tensor& grad_output, const Tensor& query, const Tensor& value,
                       bool packed) {
  TORCH_CHECK(grad_output.is_cuda(), "grad_output must be a CUDA tensor");
  TORCH_CHECK(grad_output.device() == query.device(),
              "grad_output must be on the same CUDA device as query");
  TORCH_CHECK(grad_output.scalar_type() == query.scalar_type(), "grad_output dtype mismatch");
  if (packed) {
    TORCH_CHECK(grad_output.sizes() ==
                    torch::IntArrayRef({query.size(0), query.size(1), value.size(2)}),
                "grad_output shape mismatch");
  } else {
    TORCH_CHECK(grad_output.sizes() == torch::IntArrayRef({query.size(0), query.size(1),
                                                           query.size(2), value.size(3)}),
                "grad_output shape mismatch");
  }
}

void check_seed(const Tensor& seed, const Tensor& query, double dropout_p) {
  TORCH_CHECK(seed.is_cuda(), "dropout_seed must be a CUDA tensor");
  TORCH_CHECK(seed.device() == query.device(),
              "dropout_seed must be on the same CUDA device as query");
  TORCH_CHECK(seed.scalar_type() == torch::kInt64, "dropout_seed must have dtype int64");
  TORCH_CHECK(seed.numel() == (dropout_p > 0.0 ? 1 : 0),
              "dropout_seed must be scalar exactly when dropout_p > 0");
}

rosa_problem describe(const Tensor& query, const Tensor& value, const Tensor* cu_seqlens,
                      int64_t horizon) {
  rosa_problem p{};
  p.dtype = dtype_code(query.scalar_type());
  if (cu_seqlens == nullptr) {
    p.B = static_cast<int>(query.size(0));
    p.T = static_cast<int>(query.size(1));
    p.N = p.B * p.T;
    p.S = 0;
    p.H = static_cast<int>(query.size(2));
    p.D = static_cast<int>(query.size(3));
    p.Hv = static_cast<int>(value.size(2));
    p.Dv = static_cast<int>(value.size(3));
    p.cu_seqlens = nullptr;
  } else {
    p.N = static_cast<int>(query.size(0));
    p.S = static_cast<int>(cu_seqlens->numel() - 1);
    p.H = static_cast<int>(query.size(1));
    p.D = static_cast<int>(query.size(2));
    p.Hv = static_cast<int>(value.size(1));
    p.Dv = static_cast<int>(value.size(2));
    p.cu_seqlens = cu_seqlens->data_ptr<int32_t>();
  }
  p.W = static_cast<int>(horizon);
  return p;
}

void raise_on_failure(int status, const char* what) {
  TORCH_CHECK(status == 0, what, " failed (", status, "): ", rosa_hip_last_error());
}

Triple forward_common(Tensor query, Tensor key, Tensor value, const Tensor* cu_seqlens,
                      int64_t horizon) {
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(query.device());
  query = query.contiguous();
  key = key.contiguous();
  value = value.contiguous();
  Tensor offsets;
  if (cu_seqlens != nullptr) offsets = cu_seqlens->contiguous();
  const rosa_problem problem = describe(query, value, cu_seqlens ? &offsets : nullptr, horizon);
  const auto word_options = query.options().dtype(torch::kInt32);
  Tensor packed_query, packed_key, output;
  if (cu_seqlens == nullptr) {
    packed_query = torch::empty({problem.B, problem.H, problem.T}, word_options);
    packed_key = torch::empty({problem.B, problem.H, problem.T}, word_options);
    output = torch::empty({problem.B, problem.T, problem.H, problem.Dv}, query.options());
  } else {
    packed_query = torch::empty({problem.H, problem.N}, word_options);
    packed_key = torch::empty({problem.H, problem.N}, word_options);
    output = torch::empty({problem.N, problem.H, problem.Dv}, query.options());
  }
  const size_t bytes = rosa_hip_forward_workspace_bytes(&problem);
  TORCH_CHECK(bytes > 0, "hard_forward: ", rosa_hip_last_error());
  Tensor workspace =
      torch::empty({static_cast<int64_t>(bytes)}, query.options().dtype(torch::kUInt8));
  const auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  raise_on_failure(
      rosa_hip_hard_forward(&problem, query.data_ptr(), key.data_ptr(), value.data_ptr(),
                            output.data_ptr(), packed_query.data_ptr<int32_t>(),
                            packed_key.data_ptr<int32_t>(), nullptr, workspace.data_ptr(), bytes,
                            stream.stream()),
      "rosa_hip_hard_forward");
  return std::make_tuple(output, packed_query, packed_key);
}

Triple vjp_common(Tensor query, Tensor key, Tensor value, const Tensor* cu_seqlens,
                  Tensor grad_output, Tensor packed_query, Tensor packed_key, Tensor seed,
                  int64_t horizon, const Scalars& scalars, int64_t gradient_mask) {
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(query.device());
  {
    // Recording the surrogate backward into a HIP graph has crashed the host process on
    // this platform (cause unknown), whichever way the backward is reached: refuse before
    // anything is allocated or launched.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const hipError_t queried = hipStreamIsCapturing(
        c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(), &capture);
    TORCH_CHECK(queried == hipSuccess, "surrogate_vjp: hipStreamIsCapturing failed: ",
                hipGetErrorString(queried));
    TORCH_CHECK(capture == hipStreamCaptureStatusNone,
                "surrogate_vjp: the surrogate backward cannot be recorded into a HIP graph in "
                "this build; run the backward eagerly");
  }
  query = query.contiguous();
  key = key.contiguous();
  value = value.contiguous();
  grad_output = grad_output.contiguous();
  packed_query = packed_query.contiguous();
  packed_key = packed_key.contiguous();
  seed = seed.contiguous();
  Tensor offsets;
  if (cu_seqlens != nullptr) offsets = cu_seqlens->contiguous();
  const rosa_problem problem = describe(query, value, cu_seqlens ? &offsets : nullptr, horizon);
  const auto grad_options = query.options().dtype(torch::kFloat32);
  const auto make_grad = [&](int bit, const Tensor& like) {
    return (gradient_mask & bit) != 0 ? torch::empty(like.sizes(), grad_options)
                                      : torch::empty({0}, grad_options);
  };
  Tensor grad_query = make_grad(ROSA_GRAD_QUERY, query);
  Tensor grad_key = make_grad(ROSA_GRAD_KEY, key);
  Tensor grad_value = make_grad(ROSA_GRAD_VALUE, value);
  const int mask = static_cast<int>(gradient_mask);
  const size_t bytes = rosa_hip_vjp_workspace_bytes(&problem, mask, scalars.scale,
                                                    scalars.dropout_p > 0.0f ? 1 : 0);
  TORCH_CHECK(bytes > 0, "surrogate_vjp: ", rosa_hip_last_error());
  Tensor workspace =
      torch::empty({static_cast<int64_t>(bytes)}, query.options().dtype(torch::kUInt8));
  const auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  raise_on_failure(
      rosa_hip_surrogate_vjp(
          &problem, query.data_ptr(), key.data_ptr(), value.data_ptr(), grad_output.data_ptr(),
          packed_query.data_ptr<int32_t>(), packed_key.data_ptr<int32_t>(),
          scalars.dropout_p > 0.0f ? seed.data_ptr<int64_t>() : nullptr, scalars.scale,
          scalars.dropout_p, scalars.inverse_keep, scalars.mismatch_scale, mask,
          (mask & ROSA_GRAD_QUERY) ? grad_query.data_ptr<float>() : nullptr,
          (mask & ROSA_GRAD_KEY) ? grad_key.data_ptr<float>() : nullptr,
          (mask & ROSA_GRAD_VALUE) ? grad_value.data_ptr<float>() : nullptr,
          workspace.data_ptr(), bytes, stream.stream()),
      "rosa_hip_surrogate_vjp");
  return std::make_tuple(grad_query, grad_key, grad_value);
}

void check_gradient_mask(int64_t gradient_mask) {
  TORCH_CHECK(gradient_mask >= 1 && gradient_mask <= 7,
              "gradient_mask must be an integer bit mask in [1, 7]");
}

Triple hard_forward_op(Tensor query, Tensor key, Tensor value, int64_t max_suffix_length) {
  check_dense(query, key, value, max_suffix_length);
  const int64_t horizon = std::min<int64_t>(max_suffix_length, query.size(1));
  return forward_common(query, key, value, nullptr, horizon);
}

Triple hard_forward_varlen_op(Tensor query, Tensor key, Tensor value, Tensor cu_seqlens,
                              int64_t max_suffix_length) {
  check_packed(query, key, value, cu_seqlens, max_suffix_length);
  const int64_t horizon = std::min<int64_t>(max_suffix_length, query.size(0));
  return forward_common(query, key, value, &cu_seqlens, horizon);
}

Triple surrogate_vjp_masked_op(Tensor query, Tensor key, Tensor value, Tensor grad_output,
                               Tensor packed_query_symbols, Tensor packed_key_symbols,
                               Tensor dropout_seed, int64_t max_suffix_length, double scale,
                               double dropout_p, double mismatch_scale, int64_t gradient_mask) {
  check_dense(query, key, value, max_suffix_length);
  check_grad_output(grad_output, query, value, false);
  check_words(packed_query_symbols, query, false, "packed_query_symbols");
  check_words(packed_key_symbols, query, false, "packed_key_symbols");
  const int64_t horizon = std::min<int64_t>(max_suffix_length, query.size(1));
  const Scalars scalars = narrow_scalars(horizon, scale, dropout_p, mismatch_scale);
  check_seed(dropout_seed, query, dropout_p);
  check_gradient_mask(gradient_mask);
  at::globalContext().alertNotDeterministic("rosa_soft::surrogate_vjp_masked");
  return vjp_common(query, key, value, nullptr, grad_output, packed_query_symbols,
                    packed_key_symbols, dropout_seed, horizon, scalars, gradient_mask);
}

Triple surrogate_vjp_varlen_masked_op(Tensor query, Tensor key, Tensor value, Tensor cu_seqlens,
                                      Tensor grad_output, Tensor packed_query_symbols,
                                      Tensor packed_key_symbols, Tensor dropout_seed,
                                      int64_t max_suffix_length, double scale, double dropout_p,
                                      double mismatch_scale, int64_t gradient_mask) {
  check_packed(query, key, value, cu_seqlens, max_suffix_length);
  check_grad_output(grad_output, query, value, true);
  check_words(packed_query_symbols, query, true, "packed_query_symbols");
  check_words(packed_key_symbols, query, true, "packed_key_symbols");
  const int64_t horizon = std::min<int64_t>(max_suffix_length, query.size(0));
  const Scalars scalars = narrow_scalars(horizon, scale, dropout_p, mismatch_scale);
  check_seed(dropout_seed, query, dropout_p);
  check_gradient_mask(gradient_mask);
  at::globalContext().alertNotDeterministic("rosa_soft::surrogate_vjp_varlen_masked");
  return vjp_common(query, key, value, &cu_seqlens, grad_output, packed_query_symbols,
                    packed_key_symbols, dropout_seed, horizon, scalars, gradient_mask);
}

}  // namespace

TORCH_LIBRARY(rosa_soft, m) {
  m.def(
      "hard_forward(Tensor query, Tensor key, Tensor value, int max_suffix_length) -> "
      "(Tensor output, Tensor packed_query_symbols, Tensor packed_key_symbols)");
  m.def(
      "hard_forward_varlen(Tensor query, Tensor key, Tensor value, Tensor cu_seqlens, "
      "int max_suffix_length) -> "
      "(Tensor output, Tensor packed_query_symbols, Tensor packed_key_symbols)");
  m.def(
      "surrogate_vjp_masked(Tensor query, Tensor key, Tensor value, Tensor grad_output, "
      "Tensor packed_query_symbols, Tensor packed_key_symbols, Tensor dropout_seed, "
      "int max_suffix_length, float scale, float dropout_p, float mismatch_scale, "
      "int gradient_mask) -> (Tensor grad_query, Tensor grad_key, Tensor grad_value)");
  m.def(
      "surrogate_vjp_varlen_masked(Tensor query, Tensor key, Tensor value, Tensor cu_seqlens, "
      "Tensor grad_output, Tensor packed_query_symbols, Tensor packed_key_symbols, "
      "Tensor dropout_seed, int max_suffix_length, float scale, float dropout_p, "
      "float mismatch_scale, int gradient_mask) -> "
      "(Tensor grad_query, Tensor grad_key, Tensor grad_value)");
}

TORCH_LIBRARY_IMPL(rosa_soft, CUDA, m) {
  m.impl("hard_forward", &hard_forward_op);
  m.impl("hard_forward_varlen", &hard_forward_varlen_op);
  m.impl("surrogate_vjp_masked", &surrogate_vjp_masked_op);
  m.impl("surrogate_vjp_varlen_masked", &surrogate_vjp_varlen_masked_op);
}

// Importing the module is what runs the static registrations above.
static struct PyModuleDef rosa_module = {PyModuleDef_HEAD_INIT, "_C", nullptr, -1, nullptr,
                                         nullptr, nullptr, nullptr, nullptr};

PyMODINIT_FUNC PyInit__C(void) { return PyModule_Create(&rosa_module); }
