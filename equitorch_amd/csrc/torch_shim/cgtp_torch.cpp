// PyTorch C++ extension over the C ABI of libcgtp for the fused edge product (gather, channel-wise tensor product,
// segment sum; compiled table): the autograd node, the argument block, output and workspace allocation and the stream
// lookup of one forward + backward live here instead of in Python, which is what a training step pays per call on the
// host.  Everything numeric happens behind cgtp_uvu_fwd / cgtp_uvu_bwd (include/cgtp.h); this file holds no kernel.
// Mirrors the reference's autograd Functions for this path (equitorch/nn/functional/linears.py:18-83 composed with
// index_select and indexed_scale_segment, equitorch/ops/indexed_scale_segment_op.py:143-170).
#include <torch/extension.h>

#include <memory>
#include <unordered_map>

// torch's ROCm build presents its HIP devices as device type "cuda": the guard and stream types that follow that
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "cgtp.h"

namespace {

using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

// One sorted view of the edge list (by destination for the forward, by source for the backward) and how it is cut
// into ranges: wave_seg (segment-aligned) or wave_pos (anywhere), at most one of them defined.
struct SegView {
  at::Tensor ptr, perm, seg_ids, gather, wave_seg, wave_pos;
};

// Callables (grad_out, x, y, w, need_x, need_y, need_w) -> (gx, gy, gw) that evaluate the gradients of an edge product
// through differentiable functions, for a backward that runs with gradient mode on (a gradient of the gradient is
// wanted).  One per EdgeHandle, looked up by number when the backward runs, dropped with the last copy of the handle.
std::unordered_map<int64_t, py::object>& edge_fallbacks() {
  static auto* m = new std::unordered_map<int64_t, py::object>();   // never destroyed: outlives the interpreter's teardown
  return *m;
}

struct EdgeHandle {
  SegView fwd, bwd;
  at::Tensor path_scale;   // undefined = all ones
  int64_t cfg, d_out, y_vec;
  int64_t fallback = -1;
  std::shared_ptr<void> fallback_guard;

  void set_fallback(py::object fn) {
    static int64_t next = 0;
    const int64_t id = next++;
    edge_fallbacks()[id] = std::move(fn);
    fallback = id;
    fallback_guard = std::shared_ptr<void>(nullptr, [id](void*) {
      if (!Py_IsInitialized()) return;
      py::gil_scoped_acquire gil;
      edge_fallbacks().erase(id);
    });
  }
};

const void* ptr_or_null(const at::Tensor& t) { return t.defined() ? t.data_ptr() : nullptr; }

void check_index(const at::Tensor& t, const at::Tensor& like, const char* what, at::ScalarType type = at::kLong) {
  TORCH_CHECK(!t.defined() || (t.scalar_type() == type && t.is_contiguous() && t.device() == like.device()), what,
              ": expected a contiguous ", type, " tensor on ", like.device());
}

cgtp_uvu_args base_args(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, const SegView& s,
                        const at::Tensor& path_scale, int64_t cfg, int64_t y_vec) {
  TORCH_CHECK(x.is_cuda() && y.is_cuda() && w.is_cuda(), "cgtp: operands must live on the GPU");
  TORCH_CHECK(x.is_contiguous() && y.is_contiguous() && w.is_contiguous(), "cgtp: operands must be contiguous");
  TORCH_CHECK(x.scalar_type() == y.scalar_type() && x.scalar_type() == w.scalar_type() &&
                  (x.scalar_type() == at::kFloat || x.scalar_type() == at::kDouble),
              "cgtp: operands must share one dtype, float32 or float64");
  TORCH_CHECK(x.dim() == 3 && y.dim() == 2 && (w.dim() == 2 || w.dim() == 3), "cgtp: x (N, D1, C), y (E, D2), w (E, P, C) | (P, C)");
  check_index(s.ptr, x, "ptr");
  check_index(s.perm, x, "perm");
  check_index(s.seg_ids, x, "seg_ids");
  check_index(s.gather, x, "gather");
  check_index(s.wave_seg, x, "wave_seg", at::kInt);
  check_index(s.wave_pos, x, "wave_pos");
  TORCH_CHECK(s.seg_ids.size(0) == y.size(0) && s.gather.size(0) == y.size(0), "cgtp: the edge list and y differ in length");
  cgtp_uvu_args a{};
  a.cfg = (int32_t)cfg;
  a.dtype = x.scalar_type() == at::kFloat ? CGTP_F32 : CGTP_F64;
  a.C = (int32_t)x.size(2);
  a.w_shared = w.dim() == 2;
  a.n_rows = y.size(0);
  a.n_x_rows = x.size(0);
  a.n_seg = s.ptr.size(0) - 1;
  a.ptr = (const int64_t*)s.ptr.data_ptr();
  a.perm = (const int64_t*)ptr_or_null(s.perm);
  a.seg_ids = (const int64_t*)s.seg_ids.data_ptr();
  a.gather = (const int64_t*)s.gather.data_ptr();
  a.y_vec = (int32_t)y_vec;
  if (s.wave_pos.defined()) {
    a.wave_pos = (const int64_t*)s.wave_pos.data_ptr();
    a.n_waves = s.wave_pos.size(0) - 1;
  } else if (s.wave_seg.defined()) {
    a.wave_seg = (const int32_t*)s.wave_seg.data_ptr();
    a.n_waves = s.wave_seg.size(0) - 1;
  }
  a.x = x.data_ptr();
  a.y = y.data_ptr();
  a.w = w.data_ptr();
  a.path_scale = ptr_or_null(path_scale);
  return a;
}

at::Tensor workspace_for(cgtp_uvu_args& a, int backward, const at::Tensor& like) {
  const int64_t bytes = cgtp_uvu_workspace_bytes(&a, backward);
  TORCH_CHECK(bytes >= 0, "cgtp_uvu_workspace_bytes: these operands have no launch shape");
  at::Tensor ws;
  if (bytes > 0) {
    ws = at::empty({bytes}, like.options().dtype(at::kByte));
    a.workspace = ws.data_ptr();
  }
  return ws;
}

void check_status(int status, const char* what) {
  TORCH_CHECK(status == CGTP_OK, what, ": ", cgtp_status_string(status), " (status ", status, ")");
}

void* current_stream(const at::Tensor& t) { return (void*)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream(); }

at::Tensor seg_forward(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, const EdgeHandle& h) {
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  cgtp_uvu_args a = base_args(x, y, w, h.fwd, h.path_scale, h.cfg, h.y_vec);
  at::Tensor out = at::empty({a.n_seg, h.d_out, x.size(2)}, x.options());
  a.out = out.data_ptr();
  at::Tensor ws = workspace_for(a, 0, x);
  check_status(cgtp_uvu_fwd(&a, current_stream(x)), "cgtp_uvu_fwd");
  return out;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> seg_backward(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w,
                                                            const at::Tensor& grad_out, const SegView& bwd,
                                                            const at::Tensor& path_scale, int64_t cfg, int64_t y_vec,
                                                            bool need_x, bool need_y, bool need_w) {
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  cgtp_uvu_args a = base_args(x, y, w, bwd, path_scale, cfg, y_vec);
  const at::Tensor g = grad_out.contiguous();
  TORCH_CHECK(g.scalar_type() == x.scalar_type() && g.dim() == 3 && g.size(2) == x.size(2), "cgtp: grad_out (N, DO, C) of the operands' dtype");
  a.grad_out = g.data_ptr();
  at::Tensor gx, gy, gw;
  if (need_x) gx = at::empty_like(x);
  if (need_y) gy = at::empty_like(y);
  if (need_w) gw = at::empty_like(w);
  a.grad_x = const_cast<void*>(ptr_or_null(gx));
  a.grad_y = const_cast<void*>(ptr_or_null(gy));
  a.grad_w = const_cast<void*>(ptr_or_null(gw));
  at::Tensor ws = workspace_for(a, 1, x);
  check_status(cgtp_uvu_bwd(&a, current_stream(x)), "cgtp_uvu_bwd");
  return {gx, gy, gw};
}

// The autograd node of the fused edge product.  A backward under gradient mode hands over to the handle's callable.
class EdgeUvu : public torch::autograd::Function<EdgeUvu> {
 public:
  static at::Tensor forward(AutogradContext* ctx, const at::Tensor& x, const at::Tensor& y, const at::Tensor& w,
                            const EdgeHandle* h) {
    at::Tensor out = seg_forward(x, y, w, *h);
    ctx->save_for_backward({x, y, w, h->bwd.ptr, h->bwd.perm, h->bwd.seg_ids, h->bwd.gather, h->bwd.wave_seg,
                            h->bwd.wave_pos, h->path_scale});
    ctx->saved_data["cfg"] = h->cfg;
    ctx->saved_data["y_vec"] = h->y_vec;
    ctx->saved_data["fallback"] = h->fallback;
    return out;
  }

  static variable_list backward(AutogradContext* ctx, variable_list grad_outputs) {
    const variable_list s = ctx->get_saved_variables();
    if (at::GradMode::is_enabled()) {
      py::gil_scoped_acquire gil;
      const auto it = edge_fallbacks().find(ctx->saved_data["fallback"].toInt());
      TORCH_CHECK(it != edge_fallbacks().end(),
                  "cgtp: a gradient of higher order of an edge product was asked for after its EdgePlan was released");
      const py::tuple r = it->second(grad_outputs[0], s[0], s[1], s[2], ctx->needs_input_grad(0),
                                     ctx->needs_input_grad(1), ctx->needs_input_grad(2));
      variable_list out(4);
      for (int i = 0; i < 3; ++i)
        if (!r[i].is_none()) out[i] = r[i].cast<at::Tensor>();
      return out;
    }
    const SegView bwd{s[3], s[4], s[5], s[6], s[7], s[8]};
    at::NoGradGuard no_grad;
    auto [gx, gy, gw] = seg_backward(s[0], s[1], s[2], grad_outputs[0], bwd, s[9], ctx->saved_data["cfg"].toInt(),
                                     ctx->saved_data["y_vec"].toInt(), ctx->needs_input_grad(0),
                                     ctx->needs_input_grad(1), ctx->needs_input_grad(2));
    return {gx, gy, gw, at::Tensor()};
  }
};

at::Tensor edge_uvu(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, const EdgeHandle& h) {
  return EdgeUvu::apply(x, y, w, &h);
}

// ---- row mode: the channel-wise product on a plain batch (SO3Linear('uu') on its compiled table) -----------------
// Gradients of higher order are re-expressed in Python through the differentiable contraction family; the callables
// that do it are registered once per table and looked up by number when a backward runs with gradient mode on.
std::vector<py::object>& fallbacks() {
  static std::vector<py::object>* v = new std::vector<py::object>();   // never destroyed: outlives the interpreter's teardown
  return *v;
}

cgtp_uvu_args row_args(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, const at::Tensor& path_scale,
                       int64_t cfg) {
  TORCH_CHECK(x.is_cuda() && y.is_cuda() && w.is_cuda(), "cgtp: operands must live on the GPU");
  TORCH_CHECK(x.is_contiguous() && y.is_contiguous() && w.is_contiguous(), "cgtp: operands must be contiguous");
  TORCH_CHECK(x.scalar_type() == y.scalar_type() && x.scalar_type() == w.scalar_type() &&
                  (x.scalar_type() == at::kFloat || x.scalar_type() == at::kDouble),
              "cgtp: operands must share one dtype, float32 or float64");
  TORCH_CHECK(x.dim() == 3 && y.dim() == 2 && x.size(0) == y.size(0) && (w.dim() == 2 || (w.dim() == 3 && w.size(0) == x.size(0))),
              "cgtp: x (N, D1, C), y (N, D2), w (N, P, C) | (P, C)");
  cgtp_uvu_args a{};
  a.cfg = (int32_t)cfg;
  a.dtype = x.scalar_type() == at::kFloat ? CGTP_F32 : CGTP_F64;
  a.C = (int32_t)x.size(2);
  a.w_shared = w.dim() == 2;
  a.n_rows = y.size(0);
  a.n_x_rows = x.size(0);
  a.x = x.data_ptr();
  a.y = y.data_ptr();
  a.w = w.data_ptr();
  a.path_scale = ptr_or_null(path_scale);
  return a;
}

class RowUvu : public torch::autograd::Function<RowUvu> {
 public:
  // scale: handed over by address, not as an argument tensor (it is no input of the node, and may be undefined)
  static at::Tensor forward(AutogradContext* ctx, const at::Tensor& x, const at::Tensor& y, const at::Tensor& w,
                            const at::Tensor* scale, int64_t cfg, int64_t d_out, int64_t fallback) {
    const at::Tensor& path_scale = *scale;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    cgtp_uvu_args a = row_args(x, y, w, path_scale, cfg);
    at::Tensor out = at::empty({x.size(0), d_out, x.size(2)}, x.options());
    a.out = out.data_ptr();
    at::Tensor ws = workspace_for(a, 0, x);
    check_status(cgtp_uvu_fwd(&a, current_stream(x)), "cgtp_uvu_fwd");
    ctx->save_for_backward({x, y, w, path_scale});
    ctx->saved_data["cfg"] = cfg;
    ctx->saved_data["fallback"] = fallback;
    return out;
  }

  static variable_list backward(AutogradContext* ctx, variable_list grad_outputs) {
    const variable_list s = ctx->get_saved_variables();
    const bool need_x = ctx->needs_input_grad(0), need_y = ctx->needs_input_grad(1), need_w = ctx->needs_input_grad(2);
    if (at::GradMode::is_enabled()) {   // a gradient of the gradient is wanted: the differentiable route, in Python
      py::gil_scoped_acquire gil;
      const py::object fn = fallbacks().at((size_t)ctx->saved_data["fallback"].toInt());
      const py::tuple r = fn(grad_outputs[0], s[0], s[1], s[2], need_x, need_y, need_w);
      variable_list out(7);
      for (int i = 0; i < 3; ++i)
        if (!r[i].is_none()) out[i] = r[i].cast<at::Tensor>();
      return out;
    }
    const at::Tensor& x = s[0];
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    cgtp_uvu_args a = row_args(x, s[1], s[2], s[3], ctx->saved_data["cfg"].toInt());
    const at::Tensor g = grad_outputs[0].contiguous();
    a.grad_out = g.data_ptr();
    at::Tensor gx, gy, gw;
    if (need_x) gx = at::empty_like(x);
    if (need_y) gy = at::empty_like(s[1]);
    if (need_w) gw = at::empty_like(s[2]);
    a.grad_x = const_cast<void*>(ptr_or_null(gx));
    a.grad_y = const_cast<void*>(ptr_or_null(gy));
    a.grad_w = const_cast<void*>(ptr_or_null(gw));
    at::Tensor ws = workspace_for(a, 1, x);
    check_status(cgtp_uvu_bwd(&a, current_stream(x)), "cgtp_uvu_bwd");
    return {gx, gy, gw, at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
  }
};

// Bytes of workspace the row-mode backward with all gradients would ask for (the Python side splits batches whose
// per-row weight gradients exceed its budget before it comes here).
int64_t row_backward_workspace(const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, int64_t cfg) {
  cgtp_uvu_args a = row_args(x, y, w, at::Tensor(), cfg);
  a.grad_out = a.x;                      // any non-null pointers: the query asks which gradients are wanted
  a.grad_w = const_cast<void*>(a.w);
  return cgtp_uvu_workspace_bytes(&a, 1);
}

at::Tensor opt(const c10::optional<at::Tensor>& t) { return t.has_value() ? *t : at::Tensor(); }

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "torch C++ shim over libcgtp's C ABI for the fused edge tensor product";
  py::class_<EdgeHandle>(m, "EdgeHandle")
      .def(py::init([](int64_t cfg, int64_t d_out, int64_t y_vec, c10::optional<at::Tensor> path_scale,
                       at::Tensor f_ptr, c10::optional<at::Tensor> f_perm, at::Tensor f_seg_ids, at::Tensor f_gather,
                       c10::optional<at::Tensor> f_wave_seg, c10::optional<at::Tensor> f_wave_pos, at::Tensor b_ptr,
                       c10::optional<at::Tensor> b_perm, at::Tensor b_seg_ids, at::Tensor b_gather,
                       c10::optional<at::Tensor> b_wave_seg, c10::optional<at::Tensor> b_wave_pos) {
        EdgeHandle h;
        h.cfg = cfg; h.d_out = d_out; h.y_vec = y_vec; h.path_scale = opt(path_scale);
        h.fwd = SegView{f_ptr, opt(f_perm), f_seg_ids, f_gather, opt(f_wave_seg), opt(f_wave_pos)};
        h.bwd = SegView{b_ptr, opt(b_perm), b_seg_ids, b_gather, opt(b_wave_seg), opt(b_wave_pos)};
        return h;
      }))
      .def("set_fallback", &EdgeHandle::set_fallback,
           "callable (grad_out, x, y, w, need_x, need_y, need_w) -> (gx, gy, gw) for gradients of higher order");
  m.def("edge_uvu", &edge_uvu, "fused edge product with its autograd node: x (N, D1, C), y (E, D2 | 3), w (E, P, C) | (P, C)");
  m.def("row_uvu", [](const at::Tensor& x, const at::Tensor& y, const at::Tensor& w, c10::optional<at::Tensor> path_scale,
                      int64_t cfg, int64_t d_out, int64_t fallback) {
    const at::Tensor scale = opt(path_scale);
    return RowUvu::apply(x, y, w, &scale, cfg, d_out, fallback);
  }, "channel-wise product on a batch with its autograd node: x (N, D1, C), y (N, D2), w (N, P, C) | (P, C)");
  m.def("row_backward_workspace", &row_backward_workspace);
  m.def("register_fallback", [](py::object fn) {
    fallbacks().push_back(std::move(fn));
    return (int64_t)fallbacks().size() - 1;
  }, "keeps a callable (grad_out, x, y, w, need_x, need_y, need_w) -> (gx, gy, gw) for gradients of higher order");
  m.def("abi_version", []() { return cgtp_version(); });
}
