// Compiled host path of the dense attention op for torch callers: argument checks, output allocation and the
// launch happen in C++, which takes the host cost of a call from ~15 us (Python + ctypes) to ~6.5 us -- the
// small scales of a next-scale-prediction model are bound by exactly that.  Two forms:
//   fast_dense_attn(q, k, v, scale)   (o, M, L) for lvar_amd.sparse_attn_ops.dense_attn; plain inputs only
//   register_dense_attn(ns)           defines and implements the torch-library op
//                                     `<ns>::dense_attn(Tensor q, Tensor k, Tensor v) -> Tensor[]`
//                                     natively, as the reference registers torch.ops.chipmunk.dense_attn
//                                     (kernels/chipmunk/csrc/chipmunk.cu:50-89, dense_attn at :57):
//                                     returns [o, 1/(2^M L)], softmax scale fixed to 1 (dense_attn.cu:161-163)
//
// The module does not link the C-ABI library: bind() receives the entry points' addresses from the Python
// side (which has loaded the library with ctypes), so both paths always call the same library.
#include <memory>
#include <optional>
#include <string>
#include <vector>
#include <torch/extension.h>
#include <torch/library.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include "../../include/lvar_sparse_attn.h"

namespace {

using dense_fn_t = decltype(&lvar_dense_attn_fwd);
using dense_rcp_fn_t = decltype(&lvar_dense_attn_rcp_fwd);
dense_fn_t g_dense = nullptr;
dense_rcp_fn_t g_dense_rcp = nullptr;

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

void bind(uintptr_t dense_attn_fwd, uintptr_t dense_attn_rcp_fwd) {
  g_dense = reinterpret_cast<dense_fn_t>(dense_attn_fwd);
  g_dense_rcp = reinterpret_cast<dense_rcp_fn_t>(dense_attn_rcp_fwd);
}

// (o, M, L) like lvar_amd.sparse_attn_ops.dense_attn, or None when the inputs need the general path
py::object fast_dense_attn(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, std::optional<double> scale) {
  if (!g_dense || !plain(q) || !plain(k) || !plain(v)) return py::none();
  const int64_t B = q.size(0), H = q.size(1), Lq = q.size(2), d = q.size(3), Lk = k.size(2);
  const int64_t Hkv = k.size(1);
  if (k.sizes() != v.sizes() || k.size(0) != B || Hkv <= 0 || H % Hkv != 0 || k.size(3) != d || (d != 64 && d != 128)) return py::none();
  if (Lq <= 0 || Lk <= 0 || B <= 0 || H <= 0 || Lq > INT32_MAX || Lk > INT32_MAX) return py::none();
  const auto dev = q.get_device();
  if (k.get_device() != dev || v.get_device() != dev || c10::hip::current_device() != dev) return py::none();
  const float s = scale ? static_cast<float>(*scale) : 1.0f / std::sqrt(static_cast<float>(d));
  at::Tensor o = at::empty_like(q);
  at::Tensor ml = at::empty({2, B, H, Lq, 1}, q.options().dtype(at::kFloat));   // M and L in one allocation
  float* mp = ml.data_ptr<float>();
  void* stream = c10::hip::getCurrentHIPStream(dev).stream();
  const int st = g_dense(view(q), view(k), view(v), view(o), mp, mp + B * H * Lq, nullptr, static_cast<int>(B),
                         static_cast<int>(H), static_cast<int>(Hkv), static_cast<int>(Lq), static_cast<int>(Lk), static_cast<int>(d), s, stream);
  if (st != LVAR_OK) return py::none();   // the general path reports the error
  return py::make_tuple(o, ml.select(0, 0), ml.select(0, 1));
}

// rows are read with 16-byte accesses: anything else is copied into a plain tensor first
at::Tensor as_plain(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 4, name, " must be [B,H,L,d], got ", t.sizes());
  TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16, got ", t.scalar_type());
  TORCH_CHECK(t.is_cuda(), name, " must live on a HIP device; lvar_amd has no CPU path");
  if (plain(t)) return t;
  at::Tensor c = t.contiguous();
  if (reinterpret_cast<uintptr_t>(c.data_ptr()) & 15u) c = c.clone();
  return c;
}

// <ns>::dense_attn(q, k, v) -> [o, 1/(2^M L)]
std::vector<at::Tensor> op_dense_attn(const at::Tensor& q_in, const at::Tensor& k_in, const at::Tensor& v_in) {
  TORCH_CHECK(g_dense_rcp, "lvar_amd: the C-ABI library is not bound");
  const at::Tensor q = as_plain(q_in, "q"), k = as_plain(k_in, "k"), v = as_plain(v_in, "v");
  const int64_t B = q.size(0), H = q.size(1), Lq = q.size(2), d = q.size(3), Lk = k.size(2);
  TORCH_CHECK(k.sizes() == v.sizes(), "k/v shape mismatch: ", k.sizes(), " vs ", v.sizes());
  const int64_t Hkv = k.size(1);
  TORCH_CHECK(k.size(0) == B && Hkv > 0 && H % Hkv == 0 && k.size(3) == d, "q/k batch, head or head_dim mismatch: ", q.sizes(), " vs ", k.sizes());
  TORCH_CHECK(q.get_device() == k.get_device() && q.get_device() == v.get_device(), "q, k, v must be on the same device");
  TORCH_CHECK(Lq <= INT32_MAX && Lk <= INT32_MAX, "sequence too long");
  const c10::DeviceGuard guard(q.device());   // the tensors' device is current for the allocations and the launch
  at::Tensor o = at::empty_like(q);
  at::Tensor rcp = at::empty({B, H, Lq, 1}, q.options().dtype(at::kFloat));
  void* stream = c10::hip::getCurrentHIPStream(q.get_device()).stream();
  const int st = g_dense_rcp(view(q), view(k), view(v), view(o), rcp.data_ptr<float>(), static_cast<int>(B), static_cast<int>(H), static_cast<int>(Hkv),
                             static_cast<int>(Lq), static_cast<int>(Lk), static_cast<int>(d), 1.0f, stream);
  TORCH_CHECK(st == LVAR_OK, "lvar_dense_attn_rcp_fwd failed with status ", st,
              st == LVAR_EUNSUPPORTED ? " (unsupported head_dim)" : st == LVAR_EINVAL ? " (invalid argument)" : " (launch failed)");
  return {o, rcp};
}

// Libraries registered by register_dense_attn live until the process ends (as a TORCH_LIBRARY block's would).
std::vector<std::unique_ptr<torch::Library>>& libraries() {
  static std::vector<std::unique_ptr<torch::Library>> libs;
  return libs;
}

void register_dense_attn(const std::string& ns) {
  auto lib = std::make_unique<torch::Library>(torch::Library::FRAGMENT, ns, std::nullopt, __FILE__, __LINE__);
  lib->def("dense_attn(Tensor q, Tensor k, Tensor v) -> Tensor[]");
  lib->impl("dense_attn", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(op_dense_attn)));
  libraries().push_back(std::move(lib));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("bind", &bind, "addresses of lvar_dense_attn_fwd and lvar_dense_attn_rcp_fwd");
  m.def("fast_dense_attn", &fast_dense_attn);
  m.def("register_dense_attn", &register_dense_attn, "define and implement <ns>::dense_attn natively");
}
