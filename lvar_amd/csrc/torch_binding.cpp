// Compiled fast path of the dense attention op for torch callers: argument checks, output allocation and the
// launch happen in C++, which takes the host cost of a call from ~15 us (Python + ctypes) to ~6.5 us -- the
// small scales of a next-scale-prediction model are bound by exactly that.  The reference registers its
// native ops the same way (kernels/chipmunk/csrc/chipmunk.cu:50-89, dense_attn at :57).
//
// The module does not link the C-ABI library: bind() receives the entry point's address from the Python
// side (which has loaded the library with ctypes), so both paths always call the same library.
// fast_dense_attn() only takes the common case (bf16, 4-d, contiguous, 16-byte aligned, consistent shapes,
// tensors on the current device) and returns None otherwise; the Python path then runs, with its layout
// fallbacks and error messages.
#include <optional>
#include <torch/extension.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include "../../include/lvar_sparse_attn.h"

namespace {

using dense_fn_t = decltype(&lvar_dense_attn_fwd);
dense_fn_t g_dense = nullptr;

bool plain(const at::Tensor& t) {
  return t.defined() && t.is_cuda() && t.dim() == 4 && t.scalar_type() == at::kBFloat16 && t.is_contiguous() &&
         (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15u) == 0;
}

lvar_tensor_t view(const at::Tensor& t) {
  lvar_tensor_t v;
  v.ptr = t.data_ptr();
  v.stride_b = t.stride(0);
  v.stride_h = t.stride(1);
  v.stride_row = t.stride(2);
  return v;
}

void bind(uintptr_t dense_attn_fwd) { g_dense = reinterpret_cast<dense_fn_t>(dense_attn_fwd); }

// (o, M, L) like lvar_amd.sparse_attn_ops.dense_attn, or None when the inputs need the general path
py::object fast_dense_attn(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, std::optional<double> scale) {
  if (!g_dense || !plain(q) || !plain(k) || !plain(v)) return py::none();
  const int64_t B = q.size(0), H = q.size(1), Lq = q.size(2), d = q.size(3), Lk = k.size(2);
  if (k.sizes() != v.sizes() || k.size(0) != B || k.size(1) != H || k.size(3) != d || (d != 64 && d != 128)) return py::none();
  if (Lq <= 0 || Lk <= 0 || B <= 0 || H <= 0 || Lq > INT32_MAX || Lk > INT32_MAX) return py::none();
  const auto dev = q.get_device();
  if (k.get_device() != dev || v.get_device() != dev || c10::hip::current_device() != dev) return py::none();
  const float s = scale ? static_cast<float>(*scale) : 1.0f / std::sqrt(static_cast<float>(d));
  at::Tensor o = at::empty_like(q);
  at::Tensor ml = at::empty({2, B, H, Lq, 1}, q.options().dtype(at::kFloat));   // M and L in one allocation
  float* mp = ml.data_ptr<float>();
  void* stream = c10::hip::getCurrentHIPStream(dev).stream();
  const int st = g_dense(view(q), view(k), view(v), view(o), mp, mp + B * H * Lq, nullptr, static_cast<int>(B),
                         static_cast<int>(H), static_cast<int>(Lq), static_cast<int>(Lk), static_cast<int>(d), s, stream);
  if (st != LVAR_OK) return py::none();   // the general path reports the error
  return py::make_tuple(o, ml.select(0, 0), ml.select(0, 1));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("bind", &bind, "address of lvar_dense_attn_fwd");
  m.def("fast_dense_attn", &fast_dense_attn);
}
