// Torch bindings of the recurrent-mixer kernels (csrc/kernels/rec_mix.hip); registered into src/_Cmix by
// register_rec_ops(). Shapes, dtypes, devices and index ranges that the host can see are validated here; the
// launchers trust them.
#include <ATen/hip/HIPContext.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include "kernels/rec_launchers.h"

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

die::RaggedRows ragged(int64_t T, const Tensor& positions, const OptTensor& cu_q, const Tensor& state_slots) {
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
  return r;
}

void embed_scaled(Tensor resid, OptTensor act, Tensor embed, Tensor ids, double scale) {
  check_c(resid, at::kFloat, "resid");
  TORCH_CHECK(resid.dim() == 2, "resid [T, W]");
  const int64_t T = resid.size(0), W = resid.size(1);
  const bool f = is_f32(embed, "embed");
  TORCH_CHECK(embed.dim() == 2 && embed.is_contiguous() && embed.size(1) == W, "embed [V, W]");
  check_c(ids, at::kLong, "ids");
  TORCH_CHECK(ids.numel() >= T, "ids [T]");
  void* ap = nullptr;
  if (act.has_value()) {
    TORCH_CHECK(is_f32(*act, "act") == f && act->is_contiguous() && act->sizes() == resid.sizes(),
                "act: the table's dtype, the residual's shape");
    ap = act->data_ptr();
  }
  HIP_OK(die::launch_embed_scaled(resid.data_ptr<float>(), ap, embed.data_ptr(), f, ids.data_ptr<int64_t>(),
                                  (float)scale, (int)T, (int)W, cur_stream()));
}

void conv_silu(Tensor y, Tensor x, Tensor w, OptTensor wt, OptTensor bias, Tensor conv_state, OptTensor dt,
               OptTensor dt_bias, OptTensor A_log, OptTensor ab, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_rows(x, "x");
  const int64_t T = x.size(0), C = x.size(1);
  die::ConvSiluArgs a;
  a.f32 = is_f32(x, "x");
  TORCH_CHECK(is_f32(y, "y") == a.f32 && y.is_contiguous() && y.dim() == 2 && y.size(0) == T && y.size(1) == C,
              "y [T, C] contiguous in x's dtype");
  check_c(w, at::kFloat, "w");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && w.size(1) >= 1 && w.size(1) <= 16, "w [C, taps], taps <= 16");
  const int64_t taps = w.size(1);
  check_c(conv_state, at::kFloat, "conv_state");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(1) == taps - 1 && conv_state.size(2) == C,
              "conv_state [slots, taps - 1, C]");
  a.y = y.data_ptr();
  a.x = x.data_ptr();
  a.xstride = x.stride(0);
  a.w = w.data_ptr<float>();
  a.wt = f32_vec(wt, C * taps, "wt");
  a.bias = f32_vec(bias, C, "bias");
  a.conv_state = conv_state.data_ptr<float>();
  a.C = (int)C;
  a.taps = (int)taps;
  a.dt = nullptr;
  a.dt_bias = a.A_log = nullptr;
  a.ab = nullptr;
  a.H = 0;
  if (dt.has_value()) {
    check_rows(*dt, "dt");
    const int64_t H = dt->size(1);
    TORCH_CHECK(is_f32(*dt, "dt") == a.f32 && dt->size(0) == T && dt->stride(0) == x.stride(0) && ab.has_value(),
                "dt [T, H]: a slice of the projection x comes from; with ab");
    check_c(*ab, at::kFloat, "ab");
    TORCH_CHECK(ab->numel() == T * H * 2, "ab [T, H, 2]");
    a.dt = dt->data_ptr();
    a.dt_bias = f32_vec(dt_bias, H, "dt_bias");
    a.A_log = f32_vec(A_log, H, "A_log");
    TORCH_CHECK(a.dt_bias != nullptr && a.A_log != nullptr, "dt needs dt_bias and A_log");
    a.ab = ab->data_ptr<float>();
    a.H = (int)H;
  }
  HIP_OK(die::launch_conv_silu(a, ragged(T, positions, cu_q, state_slots), cur_stream()));
}

void conv_tail_update(Tensor conv_state, Tensor x, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_c(conv_state, at::kFloat, "conv_state");
  check_rows(x, "x");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(2) == x.size(1) && conv_state.size(1) < 16,
              "conv_state [slots, taps - 1, C], x [T, C]");
  HIP_OK(die::launch_conv_tail_update(conv_state.data_ptr<float>(), x.data_ptr(), x.stride(0), is_f32(x, "x"),
                                      (int)x.size(1), (int)conv_state.size(1) + 1,
                                      ragged(x.size(0), positions, cu_q, state_slots), cur_stream()));
}

void selective_scan(Tensor out, Tensor x, Tensor dt, Tensor dt_bias, Tensor bc, int64_t boff, int64_t coff, Tensor A,
                    Tensor D, Tensor z, Tensor state, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_rows(x, "x");
  check_rows(dt, "dt");
  check_rows(bc, "bc");
  check_rows(z, "z");
  const int64_t T = x.size(0), I = x.size(1);
  die::SelectiveScanArgs a;
  a.f32 = is_f32(x, "x");
  TORCH_CHECK(is_f32(dt, "dt") == a.f32 && is_f32(bc, "bc") == a.f32 && is_f32(z, "z") == a.f32 &&
                  is_f32(out, "out") == a.f32,
              "one dtype");
  TORCH_CHECK(dt.size(0) == T && dt.size(1) == I && z.size(0) == T && z.size(1) == I && bc.size(0) == T &&
                  out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == I,
              "x, dt, z, out [T, I]; bc [T, *]");
  check_c(A, at::kFloat, "A");
  TORCH_CHECK(A.dim() == 2 && A.size(0) == I && A.size(1) >= 1 && A.size(1) <= 256, "A [I, N], N <= 256");
  const int64_t N = A.size(1);
  TORCH_CHECK(boff >= 0 && coff >= 0 && boff + N <= bc.size(1) && coff + N <= bc.size(1), "B / C columns outside bc");
  check_c(state, at::kFloat, "state");
  TORCH_CHECK(state.dim() == 3 && state.size(1) == I && state.size(2) == N, "state [slots, I, N]");
  a.out = out.data_ptr();
  a.x = x.data_ptr();
  a.dt = dt.data_ptr();
  a.bc = bc.data_ptr();
  a.z = z.data_ptr();
  a.xstride = x.stride(0);
  a.dtstride = dt.stride(0);
  a.bcstride = bc.stride(0);
  a.zstride = z.stride(0);
  a.boff = (int)boff;
  a.coff = (int)coff;
  a.dt_bias = f32_vec(dt_bias, I, "dt_bias");
  a.A = A.data_ptr<float>();
  a.D = f32_vec(D, I, "D");
  a.state = state.data_ptr<float>();
  a.I = (int)I;
  a.N = (int)N;
  HIP_OK(die::launch_selective_scan(a, ragged(T, positions, cu_q, state_slots), cur_stream()));
}

void exp_gate_scan(Tensor abe, Tensor x, int64_t ioff, int64_t foff, Tensor i_bias, Tensor f_bias, double cap,
                   Tensor m_state, int64_t heads, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_rows(x, "x");
  const int64_t T = x.size(0);
  check_c(abe, at::kFloat, "abe");
  TORCH_CHECK(abe.numel() == T * heads * 3, "abe [T, H, 3]");
  TORCH_CHECK(heads >= 1 && ioff >= 0 && foff >= 0 && ioff + heads <= x.size(1) && foff + heads <= x.size(1) && cap > 0.0,
              "gate columns outside x, or cap <= 0");
  check_c(m_state, at::kFloat, "m_state");
  TORCH_CHECK(m_state.dim() == 2 && m_state.size(1) == heads, "m_state [slots, H]");
  HIP_OK(die::launch_exp_gate_scan(abe.data_ptr<float>(), x.data_ptr(), x.stride(0), (int)ioff, (int)foff,
                                   is_f32(x, "x"), f32_vec(i_bias, heads, "i_bias"), f32_vec(f_bias, heads, "f_bias"),
                                   (float)cap, m_state.data_ptr<float>(), (int)heads,
                                   ragged(T, positions, cu_q, state_slots), cur_stream()));
}

void gated_linear_attn(Tensor out, OptTensor nq, Tensor x, int64_t qoff, int64_t koff, int64_t voff, Tensor ab,
                       Tensor state, OptTensor n_state, int64_t heads, int64_t groups, int64_t dim, int64_t vdim,
                       double qscale, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_rows(x, "x");
  const int64_t T = x.size(0);
  check_c(out, at::kFloat, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == heads * vdim, "out [T, H * vdim] fp32");
  TORCH_CHECK(heads >= 1 && groups >= 1 && heads % groups == 0 && dim >= 1 && dim <= 256 && vdim >= 1,
              "heads a multiple of groups, dim <= 256");
  TORCH_CHECK(qoff >= 0 && koff >= 0 && voff >= 0 && qoff + groups * dim <= x.size(1) &&
                  koff + groups * dim <= x.size(1) && voff + heads * vdim <= x.size(1),
              "q / k / v columns outside x");
  check_c(ab, at::kFloat, "ab");
  TORCH_CHECK(ab.dim() == 3 && ab.size(0) == T && ab.size(1) == heads && ab.size(2) >= 2, "ab [T, H, >= 2]");
  check_c(state, at::kFloat, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dim && state.size(3) == vdim,
              "state [slots, H, dim, vdim]");
  die::GatedLinearArgs a;
  a.out = out.data_ptr<float>();
  a.nq = nullptr;
  a.n_state = nullptr;
  TORCH_CHECK(nq.has_value() == n_state.has_value(), "nq and n_state come together");
  if (nq.has_value()) {
    check_c(*nq, at::kFloat, "nq");
    check_c(*n_state, at::kFloat, "n_state");
    TORCH_CHECK(nq->numel() == T * heads && n_state->dim() == 3 && n_state->size(0) == state.size(0) &&
                    n_state->size(1) == heads && n_state->size(2) == dim,
                "nq [T, H], n_state [slots, H, dim]");
    a.nq = nq->data_ptr<float>();
    a.n_state = n_state->data_ptr<float>();
  }
  a.x = x.data_ptr();
  a.xstride = x.stride(0);
  a.qoff = (int)qoff;
  a.koff = (int)koff;
  a.voff = (int)voff;
  a.f32 = is_f32(x, "x");
  a.ab = ab.data_ptr<float>();
  a.abw = (int)ab.size(2);
  a.state = state.data_ptr<float>();
  a.heads = (int)heads;
  a.groups = (int)groups;
  a.dim = (int)dim;
  a.vdim = (int)vdim;
  a.qscale = (float)qscale;
  HIP_OK(die::launch_gated_linear_attn(a, ragged(T, positions, cu_q, state_slots), cur_stream()));
}

void head_norm_gate(Tensor out, Tensor o, Tensor nq, Tensor abe, Tensor g, Tensor w, int64_t heads, int64_t vdim,
                    double eps) {
  check_c(o, at::kFloat, "o");
  check_c(nq, at::kFloat, "nq");
  check_c(abe, at::kFloat, "abe");
  TORCH_CHECK(o.dim() == 2 && o.size(1) == heads * vdim, "o [T, H * vdim]");
  const int64_t T = o.size(0);
  TORCH_CHECK(nq.numel() == T * heads && abe.numel() == T * heads * 3, "nq [T, H], abe [T, H, 3]");
  check_rows(g, "g");
  const bool f = is_f32(g, "g");
  TORCH_CHECK(g.size(0) == T && g.size(1) == heads * vdim, "g [T, H * vdim]");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.sizes() == o.sizes(),
              "out [T, H * vdim] in g's dtype");
  HIP_OK(die::launch_head_norm_gate(out.data_ptr(), o.data_ptr<float>(), nq.data_ptr<float>(), abe.data_ptr<float>(),
                                    g.data_ptr(), g.stride(0), f, f32_vec(w, heads * vdim, "w"), (int)T, (int)heads,
                                    (int)vdim, (float)eps, cur_stream()));
}

void skip_gate_group_norm(Tensor out, Tensor o, Tensor x, Tensor D, Tensor z, Tensor w, int64_t heads, int64_t vdim,
                          int64_t parts, double eps) {
  check_c(o, at::kFloat, "o");
  const int64_t n = heads * vdim;
  TORCH_CHECK(o.dim() == 2 && o.size(1) == n, "o [T, H * vdim]");
  const int64_t T = o.size(0);
  check_rows(x, "x");
  check_rows(z, "z");
  const bool f = is_f32(z, "z");
  TORCH_CHECK(is_f32(x, "x") == f && x.size(0) == T && x.size(1) == n && z.size(0) == T && z.size(1) == n,
              "x, z [T, H * vdim], one dtype");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.dim() == 2 && out.sizes() == o.sizes(),
              "out [T, H * vdim] in z's dtype");
  TORCH_CHECK(parts >= 1 && n % parts == 0, "the row must split into equal parts");
  HIP_OK(die::launch_skip_gate_group_norm(out.data_ptr(), o.data_ptr<float>(), x.data_ptr(), x.stride(0),
                                          f32_vec(D, heads, "D"), z.data_ptr(), z.stride(0), f, f32_vec(w, n, "w"),
                                          (int)T, (int)heads, (int)vdim, (int)parts, (float)eps, cur_stream()));
}

void pair_post_norm_residual(Tensor resid, OptTensor act, Tensor y1, Tensor w1, Tensor y2, Tensor w2, Tensor w,
                             double mult, double eps) {
  check_c(resid, at::kFloat, "resid");
  TORCH_CHECK(resid.dim() == 2, "resid [T, W]");
  const int64_t T = resid.size(0), W = resid.size(1);
  check_rows(y1, "y1");
  check_rows(y2, "y2");
  const bool f = is_f32(y1, "y1");
  TORCH_CHECK(is_f32(y2, "y2") == f && is_f32(w, "w") == f && y1.size(0) == T && y1.size(1) == W && y2.size(0) == T &&
                  y2.size(1) == W && w.is_contiguous() && w.numel() == W,
              "y1, y2 [T, W], w [W], one dtype");
  void* ap = nullptr;
  if (act.has_value()) {
    TORCH_CHECK(is_f32(*act, "act") == f && act->is_contiguous() && act->sizes() == resid.sizes(),
                "act: the activation dtype, the residual's shape");
    ap = act->data_ptr();
  }
  HIP_OK(die::launch_pair_post_norm_residual(resid.data_ptr<float>(), ap, y1.data_ptr(), y1.stride(0),
                                             f32_vec(w1, W, "w1"), y2.data_ptr(), y2.stride(0), f32_vec(w2, W, "w2"),
                                             f, w.data_ptr(), (float)mult, (float)eps, (int)T, (int)W, cur_stream()));
}

}  // namespace

void register_rec_ops(pybind11::module& m) {
  m.def("embed_scaled", &embed_scaled);
  m.def("conv_silu", &conv_silu);
  m.def("conv_tail_update", &conv_tail_update);
  m.def("selective_scan", &selective_scan);
  m.def("exp_gate_scan", &exp_gate_scan);
  m.def("gated_linear_attn", &gated_linear_attn);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("skip_gate_group_norm", &skip_gate_group_norm);
  m.def("pair_post_norm_residual", &pair_post_norm_residual);
}
