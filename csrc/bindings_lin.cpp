// Torch bindings of the sandwich-norm / depth-average / linear-attention kernels (csrc/kernels/lin_mix.hip);
// registered into src/_Cmix by register_lin_ops(). Shapes, dtypes, devices and index ranges that the host can see
// are validated here; the launchers trust them.
#include <ATen/hip/HIPContext.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include "kernels/lin_launchers.h"

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

namespace {

inline hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define HIP_OK(call)                                                                                   \
  do {                                                                                                  \
    hipError_t e_ = (call);                                                                             \
    TORCH_CHECK(e_ == hipSuccess, "HIP launch failed: ", hipGetErrorString(e_), " (", #call, ")");      \
  } while (0)

bool is_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

void check_rows(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be [rows, n] with unit inner stride");
}

void check_c(const Tensor& t, at::ScalarType d, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == d && t.is_contiguous(), name, ": wrong device / dtype / layout");
}

const float* f32_vec(const OptTensor& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  check_c(*t, at::kFloat, name);
  TORCH_CHECK(t->numel() == n, name, ": expected ", n, " values, got ", t->numel());
  return t->data_ptr<float>();
}

void embed_pos(Tensor out, Tensor embed, Tensor pos, Tensor ids, Tensor positions) {
  check_c(out, at::kFloat, "out");
  TORCH_CHECK(out.dim() == 2, "out [T, W]");
  const int64_t T = out.size(0), W = out.size(1);
  const bool f = is_f32(embed, "embed");
  TORCH_CHECK(is_f32(pos, "pos") == f && embed.dim() == 2 && pos.dim() == 2 && embed.is_contiguous() &&
                  pos.is_contiguous() && embed.size(1) == W && pos.size(1) == W,
              "embed [V, W], pos [P, W], one dtype");
  check_c(ids, at::kLong, "ids");
  check_c(positions, at::kLong, "positions");
  TORCH_CHECK(ids.numel() >= T && positions.numel() >= T, "ids / positions [T]");
  HIP_OK(die::launch_embed_pos(out.data_ptr<float>(), embed.data_ptr(), pos.data_ptr(), f, ids.data_ptr<int64_t>(),
                               positions.data_ptr<int64_t>(), (int)T, (int)W, cur_stream()));
}

// y (+ ybias) of a sublayer: pointer, stride, type; checked against [T, W]
struct SubOut {
  const void* y = nullptr;
  int64_t stride = 0;
  bool f32 = false;
  const void* bias = nullptr;
};
SubOut sub_out(const OptTensor& y, const OptTensor& ybias, int64_t T, int64_t W) {
  SubOut o;
  if (!y.has_value()) {
    TORCH_CHECK(!ybias.has_value(), "ybias without y");
    return o;
  }
  check_rows(*y, "y");
  o.f32 = is_f32(*y, "y");
  TORCH_CHECK(y->size(0) == T && y->size(1) == W, "y [T, W]");
  o.y = y->data_ptr();
  o.stride = y->stride(0);
  if (ybias.has_value()) {
    TORCH_CHECK(is_f32(*ybias, "ybias") == o.f32 && ybias->is_contiguous() && ybias->numel() == W,
                "ybias [W] in y's dtype");
    o.bias = ybias->data_ptr();
  }
  return o;
}

void post_pre_norm(Tensor resid, Tensor y, OptTensor ybias, Tensor w_post, OptTensor w_pre, OptTensor h, double eps) {
  check_c(resid, at::kFloat, "resid");
  TORCH_CHECK(resid.dim() == 2, "resid [T, W]");
  const int64_t T = resid.size(0), W = resid.size(1);
  const SubOut so = sub_out(y, ybias, T, W);
  die::PostPreNormArgs a;
  a.resid = resid.data_ptr<float>();
  a.y = so.y;
  a.ystride = so.stride;
  a.y_f32 = so.f32;
  a.ybias = so.bias;
  a.w_post = f32_vec(w_post, W, "w_post");
  a.w_pre = f32_vec(w_pre, W, "w_pre");
  a.h = nullptr;
  a.h_f32 = false;
  if (h.has_value()) {
    a.h_f32 = is_f32(*h, "h");
    TORCH_CHECK(h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W && w_pre.has_value(),
                "h [T, W] contiguous, with w_pre");
    a.h = h->data_ptr();
  }
  a.eps = (float)eps;
  a.T = (int)T;
  a.W = (int)W;
  HIP_OK(die::launch_post_pre_norm(a, cur_stream()));
}

void depth_avg_norm(Tensor planes, int64_t n, OptTensor dw, OptTensor y, OptTensor ybias, OptTensor w_post,
                    OptTensor w_pre, OptTensor h, double eps) {
  check_c(planes, at::kFloat, "planes");
  TORCH_CHECK(planes.dim() == 3 && n >= 1 && planes.size(0) >= n + 1, "planes [>= n + 1, T, W]");
  const int64_t T = planes.size(1), W = planes.size(2);
  const SubOut so = sub_out(y, ybias, T, W);
  die::DepthAvgArgs a;
  a.planes = planes.data_ptr<float>();
  a.plane_stride = planes.stride(0);
  a.n = (int)n;
  a.dw = f32_vec(dw, n, "dw");
  a.y = so.y;
  a.ystride = so.stride;
  a.y_f32 = so.f32;
  a.ybias = so.bias;
  a.w_post = f32_vec(w_post, W, "w_post");
  TORCH_CHECK(!y.has_value() || w_post.has_value(), "y needs w_post");
  a.w_pre = f32_vec(w_pre, W, "w_pre");
  a.h = nullptr;
  a.h_f32 = false;
  if (h.has_value()) {
    a.h_f32 = is_f32(*h, "h");
    TORCH_CHECK(h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W && w_pre.has_value(),
                "h [T, W] contiguous, with w_pre");
    a.h = h->data_ptr();
  }
  a.eps = (float)eps;
  a.T = (int)T;
  a.W = (int)W;
  HIP_OK(die::launch_depth_avg_norm(a, cur_stream()));
}

void bias_relu2(Tensor out, Tensor z, Tensor b) {
  const bool f = is_f32(z, "z");
  TORCH_CHECK(is_f32(out, "out") == f && is_f32(b, "b") == f && z.dim() == 2 && z.is_contiguous() &&
                  out.is_contiguous() && out.sizes() == z.sizes() && b.is_contiguous() && b.numel() == z.size(1),
              "bias_relu2: z, out [rows, n] contiguous, b [n], one dtype");
  HIP_OK(die::launch_bias_relu2(out.data_ptr(), z.data_ptr(), b.data_ptr(), f, (int)z.size(0), (int)z.size(1),
                                cur_stream()));
}

void tanh_cap(Tensor out, Tensor z, double cap) {
  const bool f = is_f32(z, "z");
  check_c(out, at::kFloat, "out");
  TORCH_CHECK(z.is_contiguous() && out.numel() == z.numel() && cap > 0.0, "tanh_cap: z contiguous, out fp32 of its size, cap > 0");
  HIP_OK(die::launch_tanh_cap(out.data_ptr<float>(), z.data_ptr(), f, (float)cap, z.numel(), cur_stream()));
}

void head_gate(Tensor out, Tensor o, Tensor g) {
  const bool f = is_f32(o, "o");
  TORCH_CHECK(o.dim() == 3 && o.is_contiguous(), "o [H, T, v] contiguous");
  const int64_t H = o.size(0), T = o.size(1), v = o.size(2);
  check_rows(g, "g");
  TORCH_CHECK(is_f32(g, "g") == f && g.size(0) == T && g.size(1) == H, "g [T, H] in o's dtype");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.numel() == o.numel(), "out [T, H * v]");
  HIP_OK(die::launch_head_gate(out.data_ptr(), o.data_ptr(), g.data_ptr(), g.stride(0), f, (int)T, (int)H, (int)v,
                               cur_stream()));
}

void norm_sigmoid_gate(Tensor out, Tensor o, Tensor g, Tensor w, double eps) {
  check_c(o, at::kFloat, "o");
  TORCH_CHECK(o.dim() == 2, "o [T, n]");
  const int64_t T = o.size(0), n = o.size(1);
  check_rows(g, "g");
  const bool f = is_f32(g, "g");
  TORCH_CHECK(g.size(0) == T && g.size(1) == n, "g [T, n]");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.sizes() == o.sizes(),
              "out [T, n] in g's dtype");
  HIP_OK(die::launch_norm_sigmoid_gate(out.data_ptr(), o.data_ptr<float>(), g.data_ptr(), g.stride(0), f,
                                       f32_vec(w, n, "w"), (float)eps, (int)T, (int)n, cur_stream()));
}

void lightning_attn(Tensor out, Tensor x, int64_t qoff, int64_t koff, int64_t voff, Tensor decay, Tensor state,
                    int64_t heads, int64_t dim, int64_t vdim, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_rows(x, "x");
  const int64_t T = x.size(0);
  check_c(out, at::kFloat, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == heads * vdim, "out [T, H * vdim] fp32");
  TORCH_CHECK(heads >= 1 && dim >= 1 && dim <= 128 && vdim >= 1 && vdim <= 256, "dim <= 128, vdim <= 256");
  TORCH_CHECK(qoff >= 0 && koff >= 0 && voff >= 0 && qoff + heads * dim <= x.size(1) &&
                  koff + heads * dim <= x.size(1) && voff + heads * vdim <= x.size(1),
              "q / k / v columns outside x");
  check_c(state, at::kFloat, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dim && state.size(3) == vdim,
              "state [slots, H, dim, vdim]");
  check_c(positions, at::kLong, "positions");
  check_c(state_slots, at::kInt, "state_slots");
  TORCH_CHECK(positions.numel() >= T, "positions [T]");
  die::RaggedRows r;
  r.positions = positions.data_ptr<int64_t>();
  r.state_slots = state_slots.data_ptr<int>();
  r.total_rows = (int)T;
  r.cu_q = nullptr;
  if (cu_q.has_value()) {
    check_c(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= 2, "cu_q [S + 1]");
    r.cu_q = cu_q->data_ptr<int>();
    r.num_seqs = (int)cu_q->numel() - 1;
  } else {
    r.num_seqs = (int)T;
  }
  TORCH_CHECK(state_slots.numel() >= r.num_seqs, "state_slots [S]");
  die::LightningArgs a;
  a.out = out.data_ptr<float>();
  a.x = x.data_ptr();
  a.xstride = x.stride(0);
  a.qoff = (int)qoff;
  a.koff = (int)koff;
  a.voff = (int)voff;
  a.f32 = is_f32(x, "x");
  a.decay = f32_vec(decay, heads, "decay");
  a.state = state.data_ptr<float>();
  a.heads = (int)heads;
  a.dim = (int)dim;
  a.vdim = (int)vdim;
  HIP_OK(die::launch_lightning_attn(a, r, cur_stream()));
}

}  // namespace

void register_lin_ops(pybind11::module& m) {
  m.def("embed_pos", &embed_pos);
  m.def("post_pre_norm", &post_pre_norm);
  m.def("depth_avg_norm", &depth_avg_norm);
  m.def("bias_relu2", &bias_relu2);
  m.def("tanh_cap", &tanh_cap);
  m.def("head_gate", &head_gate);
  m.def("norm_sigmoid_gate", &norm_sigmoid_gate);
  m.def("lightning_attn", &lightning_attn);
}
