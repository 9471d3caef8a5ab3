// PyTorch-side autograd node of the WTConv layer in C++ (host code only; the kernels live behind the C ABI of
// include/wtconv_hip.h, whose entry points this module receives as addresses from the ctypes loader, so that the
// process holds one copy of the library).
//
// Why C++: an eager training step of a small plane spends more time in PyTorch's Python autograd machinery than on
// the GPU -- a torch.autograd.Function with the 9-13 differentiable inputs of this layer (the reference's own
// parameter structure, wtconv/wtconv2d.py:19-31) costs ~13 us of host time per input and pass.  The node below does
// the same work as wtconv_amd/functional.py (_forward_impl / _backward_impl) without the interpreter: allocate
// the outputs, fill the parameter tables, call the library on the current stream.
//
// Only the canonical case is handled here: every parameter on the device of x, contiguous, all in one of the three
// kernel dtypes.  layer() returns None for anything else and the caller takes the Python path, which converts.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/function.h>
#include <torch/csrc/autograd/functions/basic_ops.h>

#include <optional>
#include <vector>

#include "../../include/wtconv_hip.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

// The C ABI as function pointers (filled once by bind()).
struct Abi {
  int (*fwd2)(const void*, void*, const wtconv_params*, int, int, int, int, int, int, int, int, void*, size_t, void*);
  int (*bwd2)(const void*, const void*, void*, const wtconv_params*, const wtconv_param_grads*, int, int, int, int, int,
              int, int, int, void*, size_t, void*);
  int (*bwdin2)(const void*, void*, const wtconv_params*, int, int, int, int, int, int, int, int, void*, size_t, void*);
  int (*bwdpar2)(const void*, const void*, const wtconv_params*, const wtconv_param_grads*, int, int, int, int, int, int,
                 int, int, void*, size_t, void*);
  size_t (*ws2)(int, int, int, int, int, int, int);
  int (*fwd1)(const void*, void*, const wtconv_params*, int, int, int, int, int, int, int, void*, size_t, void*);
  int (*bwd1)(const void*, const void*, void*, const wtconv_params*, const wtconv_param_grads*, int, int, int, int, int,
              int, int, void*, size_t, void*);
  int (*bwdin1)(const void*, void*, const wtconv_params*, int, int, int, int, int, int, int, void*, size_t, void*);
  int (*bwdpar1)(const void*, const void*, const wtconv_params*, const wtconv_param_grads*, int, int, int, int, int, int,
                 int, void*, size_t, void*);
  size_t (*ws1)(int, int, int, int, int, int);
  const char* (*last_error)();
  bool bound = false;
} abi;

template <typename F>
void take(F& slot, uintptr_t addr) { slot = reinterpret_cast<F>(addr); }

// Addresses in the order of the names in wtconv_amd/_ext.py.
void bind(const std::vector<uintptr_t>& a) {
  TORCH_CHECK(a.size() == 11, "bind: expected 11 addresses, got ", a.size());
  take(abi.fwd2, a[0]); take(abi.bwd2, a[1]); take(abi.bwdin2, a[2]); take(abi.bwdpar2, a[3]); take(abi.ws2, a[4]);
  take(abi.fwd1, a[5]); take(abi.bwd1, a[6]); take(abi.bwdin1, a[7]); take(abi.bwdpar1, a[8]); take(abi.ws1, a[9]);
  take(abi.last_error, a[10]);
  abi.bound = true;
}

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return WTCONV_F32;
    case at::kBFloat16: return WTCONV_BF16;
    case at::kHalf: return WTCONV_F16;
    default: return -1;
  }
}

void fail(int rc, const char* what) {
  const char* msg = abi.last_error ? abi.last_error() : "";
  if (rc == WTCONV_E_ARG) throw py::value_error(std::string(msg && *msg ? msg : what));
  TORCH_CHECK(false, (msg && *msg) ? msg : what, " (code ", rc, ")");
}

struct Shape { int B, C, H, W; };      // 1-D rows: H = 1, W = N

size_t workspace_bytes(int dims, const Shape& s, int K, int L, int pass) {
  size_t n = dims == 2 ? abi.ws2(s.B, s.C, s.H, s.W, K, L, pass) : abi.ws1(s.B, s.C, s.W, K, L, pass);
  return n < 256 ? 256 : n;
}

template <typename Table>
void fill(Table& t, const Tensor& base_w, const Tensor& base_b, const Tensor& base_s, at::TensorList wt, int L) {
  t = Table{};
  t.base_weight = static_cast<decltype(t.base_weight)>(base_w.data_ptr());
  t.base_bias = base_b.defined() ? static_cast<decltype(t.base_bias)>(base_b.data_ptr()) : nullptr;
  t.base_scale = static_cast<decltype(t.base_scale)>(base_s.data_ptr());
  for (int l = 0; l < L; ++l) {
    t.wt_weight[l] = static_cast<decltype(t.base_weight)>(wt[l].data_ptr());
    t.wt_scale[l] = static_cast<decltype(t.base_weight)>(wt[L + l].data_ptr());
  }
}

class WTConvNode : public torch::autograd::Function<WTConvNode> {
 public:
  // wt = the L level weights followed by the L level scales.
  static Tensor forward(AutogradContext* ctx, const Tensor& x_in, const Tensor& base_w,
                        const std::optional<Tensor>& base_b_opt, const Tensor& base_s, at::TensorList wt,
                        int64_t dims, int64_t K, int64_t L) {
    const Tensor x = x_in.contiguous();
    const Tensor base_b = base_b_opt.has_value() ? *base_b_opt : Tensor();
    const c10::DeviceGuard guard(x.device());      // (PyTorch on ROCm names the device type "cuda")
    const Shape s = dims == 2 ? Shape{(int)x.size(0), (int)x.size(1), (int)x.size(2), (int)x.size(3)}
                              : Shape{(int)x.size(0), (int)x.size(1), 1, (int)x.size(2)};
    Tensor out = at::empty_like(x, at::MemoryFormat::Contiguous);
    const size_t wsz = workspace_bytes(dims, s, K, L, 0);
    Tensor ws = at::empty({static_cast<int64_t>(wsz)}, x.options().dtype(at::kByte));
    wtconv_params p;
    fill(p, base_w, base_b, base_s, wt, L);
    void* stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
    const int dt = dtype_code(x.scalar_type()), pdt = dtype_code(base_w.scalar_type());
    const int rc = dims == 2 ? abi.fwd2(x.data_ptr(), out.data_ptr(), &p, s.B, s.C, s.H, s.W, K, L, dt, pdt,
                                        ws.data_ptr(), wsz, stream)
                             : abi.fwd1(x.data_ptr(), out.data_ptr(), &p, s.B, s.C, s.W, K, L, dt, pdt, ws.data_ptr(),
                                        wsz, stream);
    if (rc) fail(rc, "wtconv forward");
    variable_list saved = {x, base_w, base_b, base_s};
    saved.insert(saved.end(), wt.begin(), wt.end());
    ctx->save_for_backward(saved);
    ctx->saved_data["dims"] = dims;
    ctx->saved_data["K"] = K;
    ctx->saved_data["L"] = L;
    return out;
  }

  static variable_list backward(AutogradContext* ctx, variable_list grad_outputs) {
    const variable_list saved = ctx->get_saved_variables();
    const int dims = ctx->saved_data["dims"].toInt(), K = ctx->saved_data["K"].toInt(), L = ctx->saved_data["L"].toInt();
    const Tensor &x = saved[0], &base_w = saved[1], &base_b = saved[2], &base_s = saved[3];
    const at::TensorList wt(saved.data() + 4, 2 * L);
    const bool has_bias = base_b.defined();
    // one result per argument of forward: x, base_w, base_b, base_s, 2L level tensors, dims, K, L
    variable_list res(4 + 2 * L + 3);
    Tensor g = grad_outputs[0];
    if (!g.defined()) return res;
    // needs_input_grad counts the tensor arguments only (a missing bias is not one of them)
    const int nt = 3 + (has_bias ? 1 : 0) + 2 * L;
    const bool need_x = ctx->needs_input_grad(0);
    bool need_params = false;
    for (int i = 1; i < nt; ++i) need_params = need_params || ctx->needs_input_grad(i);
    if (!need_x && !need_params) return res;
    if (g.scalar_type() != x.scalar_type()) g = g.to(x.scalar_type());
    g = g.contiguous();
    const c10::DeviceGuard guard(x.device());      // (PyTorch on ROCm names the device type "cuda")
    const Shape s = dims == 2 ? Shape{(int)x.size(0), (int)x.size(1), (int)x.size(2), (int)x.size(3)}
                              : Shape{(int)x.size(0), (int)x.size(1), 1, (int)x.size(2)};
    const int pass = need_x && need_params ? 3 : (need_x ? 1 : 2);
    const size_t wsz = workspace_bytes(dims, s, K, L, pass);
    Tensor ws = at::empty({static_cast<int64_t>(wsz)}, x.options().dtype(at::kByte));
    wtconv_params p;
    fill(p, base_w, base_b, base_s, wt, L);
    void* stream = c10::hip::getCurrentHIPStream(x.device().index()).stream();
    const int dt = dtype_code(x.scalar_type()), pdt = dtype_code(base_w.scalar_type());
    Tensor grad_x;
    if (need_x) grad_x = at::empty_like(x, at::MemoryFormat::Contiguous);
    // parameter gradients are written as fp32 into one flat buffer (one allocation for the 5 + 2 L tensors): fp32
    // parameters get views of it in their own shapes, others views of one cast of it
    const bool f32 = base_w.scalar_type() == at::kFloat;
    std::vector<Tensor> views(3 + 2 * L);      // base_w, base_b, base_s, levels
    Tensor flat;
    wtconv_param_grads gt;
    if (need_params) {
      std::vector<const Tensor*> plist = {&base_w, &base_b, &base_s};
      for (int i = 0; i < 2 * L; ++i) plist.push_back(&wt[i]);
      int64_t total = 0;
      for (const Tensor* t : plist) total += t->defined() ? t->numel() : 0;
      flat = at::empty({total}, x.options().dtype(at::kFloat));
      int64_t pos = 0;
      for (size_t i = 0; i < plist.size(); ++i)
        if (plist[i]->defined()) {
          views[i] = flat.narrow(0, pos, plist[i]->numel());
          if (f32) views[i] = views[i].view(plist[i]->sizes());
          pos += plist[i]->numel();
        }
      const at::TensorList lv(views.data() + 3, 2 * L);
      fill(gt, views[0], views[1], views[2], lv, L);
    }
    int rc;
    if (dims == 2) {
      if (pass == 3)
        rc = abi.bwd2(x.data_ptr(), g.data_ptr(), grad_x.data_ptr(), &p, &gt, s.B, s.C, s.H, s.W, K, L, dt, pdt,
                      ws.data_ptr(), wsz, stream);
      else if (pass == 1)
        rc = abi.bwdin2(g.data_ptr(), grad_x.data_ptr(), &p, s.B, s.C, s.H, s.W, K, L, dt, pdt, ws.data_ptr(), wsz, stream);
      else
        rc = abi.bwdpar2(x.data_ptr(), g.data_ptr(), &p, &gt, s.B, s.C, s.H, s.W, K, L, dt, pdt, ws.data_ptr(), wsz, stream);
    } else {
      if (pass == 3)
        rc = abi.bwd1(x.data_ptr(), g.data_ptr(), grad_x.data_ptr(), &p, &gt, s.B, s.C, s.W, K, L, dt, pdt, ws.data_ptr(),
                      wsz, stream);
      else if (pass == 1)
        rc = abi.bwdin1(g.data_ptr(), grad_x.data_ptr(), &p, s.B, s.C, s.W, K, L, dt, pdt, ws.data_ptr(), wsz, stream);
      else
        rc = abi.bwdpar1(x.data_ptr(), g.data_ptr(), &p, &gt, s.B, s.C, s.W, K, L, dt, pdt, ws.data_ptr(), wsz, stream);
    }
    if (rc) fail(rc, "wtconv backward");
    // The gradients come from raw pointers and carry no graph.  Under create_graph=True every result that something
    // differentiable went into gets a node that raises when it is differentiated (what once_differentiable does for
    // the Python function): a second-order term is refused instead of being treated as a constant.
    bool twice = false;
    if (at::GradMode::is_enabled()) {
      twice = grad_outputs[0].requires_grad();
      for (const Tensor& t : saved) twice = twice || (t.defined() && t.requires_grad());
    }
    auto refuse = [&](Tensor& t) {
      if (!twice || !t.defined()) return;
      auto err = std::make_shared<torch::autograd::Error>(
          "the backward pass of the WTConv layer is not differentiable (double backward / create_graph=True through "
          "this layer is not supported)", torch::autograd::edge_list());
      torch::autograd::create_gradient_edge(t, err);
    };
    res[0] = grad_x;
    refuse(res[0]);
    if (need_params) {
      if (!f32) {
        const Tensor cast = flat.to(base_w.scalar_type());
        int64_t pos = 0;
        std::vector<const Tensor*> plist = {&base_w, &base_b, &base_s};
        for (int i = 0; i < 2 * L; ++i) plist.push_back(&wt[i]);
        for (size_t i = 0; i < plist.size(); ++i)
          if (plist[i]->defined()) {
            views[i] = cast.narrow(0, pos, plist[i]->numel()).view(plist[i]->sizes());
            pos += plist[i]->numel();
          }
      }
      res[1] = views[0];
      res[2] = views[1];
      res[3] = views[2];
      for (int i = 0; i < 2 * L; ++i) res[4 + i] = views[3 + i];
      for (int i = 1; i < 4 + 2 * L; ++i) refuse(res[i]);
    }
    return res;
  }
};

bool canonical(const Tensor& t, const at::Device& dev, at::ScalarType pd) {
  return t.device() == dev && t.scalar_type() == pd && t.is_contiguous();
}

// The layer with its C++ autograd node, or None when the arguments need the conversions of the Python path.
py::object layer(const Tensor& x, const Tensor& base_w, const std::optional<Tensor>& base_b, const Tensor& base_s,
                 const std::vector<Tensor>& wt_ws, const std::vector<Tensor>& wt_ss, int64_t dims, int64_t K, int64_t L) {
  TORCH_CHECK(abi.bound, "wtconv binding used before bind()");
  if (!x.is_cuda() || dtype_code(x.scalar_type()) < 0) return py::none();
  const at::ScalarType pd = base_w.scalar_type();
  if (dtype_code(pd) < 0) return py::none();
  if (static_cast<int64_t>(wt_ws.size()) != L || static_cast<int64_t>(wt_ss.size()) != L) return py::none();
  const at::Device dev = x.device();
  if (!canonical(base_w, dev, pd) || !canonical(base_s, dev, pd)) return py::none();
  if (base_b.has_value() && base_b->defined() && !canonical(*base_b, dev, pd)) return py::none();
  std::vector<Tensor> wt;
  wt.reserve(2 * L);
  for (const Tensor& t : wt_ws) { if (!canonical(t, dev, pd)) return py::none(); wt.push_back(t); }
  for (const Tensor& t : wt_ss) { if (!canonical(t, dev, pd)) return py::none(); wt.push_back(t); }
  const std::optional<Tensor> bias = (base_b.has_value() && base_b->defined()) ? base_b : std::nullopt;
  Tensor out;
  {
    py::gil_scoped_release nogil;
    out = WTConvNode::apply(x, base_w, bias, base_s, at::TensorList(wt), dims, K, L);
  }
  return py::cast(out);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("bind", &bind, "hand over the addresses of the C-ABI entry points");
  m.def("layer", &layer, "WTConv layer (2-D or 1-D) with a C++ autograd node; None if the arguments are not canonical");
}
