// Torch bindings of the dtype-generic kernels (csrc/kernels/mix_ops.hip, latent_attn.hip) and of the expert
// alignment kernel they share with the Mixtral path (moe.hip). Built as src/_Cmix: a model that needs only
// these compiles only these. Shapes, dtypes and devices are validated here; the launchers trust them.
#include <ATen/hip/HIPContext.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include "kernels/launchers.h"
#include "kernels/mix_launchers.h"

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

namespace {

inline hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define HIP_OK(call)                                                                                   \
  do {                                                                                                  \
    hipError_t e_ = (call);                                                                             \
    TORCH_CHECK(e_ == hipSuccess, "HIP launch failed: ", hipGetErrorString(e_), " (", #call, ")");      \
  } while (0)

// storage type of an activation / weight tensor: true = fp32, false = bf16
bool is_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

void check_rows(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be [rows, n] with unit inner stride");
}

void check_i(const Tensor& t, at::ScalarType d, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == d && t.is_contiguous(), name, ": wrong device / dtype / layout");
}

void rms_norm_ext(Tensor out, Tensor x, OptTensor w, bool unit_offset, double eps) {
  check_rows(out, "out");
  check_rows(x, "x");
  const bool of = is_f32(out, "out"), xf = is_f32(x, "x");
  TORCH_CHECK(out.size(0) == x.size(0) && out.size(1) == x.size(1), "rms_norm_ext shapes");
  bool wf = false;
  const void* wp = nullptr;
  if (w.has_value()) {
    wf = is_f32(*w, "w");
    TORCH_CHECK(w->is_contiguous() && w->numel() == x.size(1), "w [n]");
    wp = w->data_ptr();
  }
  HIP_OK(die::launch_rms_norm_ext(out.data_ptr(), out.stride(0), of, x.data_ptr(), x.stride(0), xf, wp, wf,
                                  unit_offset, (float)eps, (int)x.size(0), (int)x.size(1), cur_stream()));
}

void post_norm_residual(Tensor resid, OptTensor act, Tensor y, Tensor w, bool unit_offset, double eps, double mult) {
  TORCH_CHECK(resid.is_cuda() && resid.scalar_type() == at::kFloat && resid.is_contiguous() && resid.dim() == 2,
              "resid must be a contiguous fp32 [rows, n] GPU tensor");
  check_rows(y, "y");
  const bool yf = is_f32(y, "y"), wf = is_f32(w, "w");
  TORCH_CHECK(y.size(0) == resid.size(0) && y.size(1) == resid.size(1) && w.is_contiguous() &&
                  w.numel() == resid.size(1),
              "post_norm_residual shapes");
  void* ap = nullptr;
  if (act.has_value()) {
    TORCH_CHECK(act->is_cuda() && act->scalar_type() == at::kBFloat16 && act->is_contiguous() &&
                    act->sizes() == resid.sizes(),
                "act must be a contiguous bf16 tensor of the residual's shape");
    ap = act->data_ptr();
  }
  HIP_OK(die::launch_post_norm_residual(resid.data_ptr<float>(), ap, y.data_ptr(), y.stride(0), yf, w.data_ptr(), wf,
                                        unit_offset, (float)eps, (float)mult, (int)resid.size(0), (int)resid.size(1),
                                        cur_stream()));
}

void gated_act(Tensor out, Tensor gu, int64_t kind, double limit, double alpha) {
  const bool f = is_f32(gu, "gu");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && gu.is_contiguous() && gu.dim() == 2 &&
                  out.dim() == 2 && gu.size(1) == 2 * out.size(1) && gu.size(0) == out.size(0),
              "gated_act: gu [rows, 2f] -> out [rows, f], same dtype, contiguous");
  HIP_OK(die::launch_gated_act(out.data_ptr(), gu.data_ptr(), f, (int)out.size(0), (int)out.size(1), (int)kind,
                               (float)limit, (float)alpha, cur_stream()));
}

void route_sigmoid_topk(Tensor w, Tensor ids, Tensor x, Tensor wr) {
  check_rows(x, "x");
  const bool xf = is_f32(x, "x"), wf = is_f32(wr, "wr");
  check_i(w, at::kFloat, "w");
  check_i(ids, at::kInt, "ids");
  TORCH_CHECK(wr.dim() == 2 && wr.is_contiguous() && wr.size(1) == x.size(1), "wr [E, H]");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == x.size(0) && ids.sizes() == w.sizes() && w.size(1) <= wr.size(0),
              "w, ids [T, K], K <= E");
  HIP_OK(die::launch_route_sigmoid_topk(w.data_ptr<float>(), ids.data_ptr<int>(), x.data_ptr(), x.stride(0), xf,
                                        wr.data_ptr(), wf, (int)x.size(0), (int)x.size(1), (int)wr.size(0),
                                        (int)w.size(1), cur_stream()));
}

void topk_sigmoid(Tensor w, Tensor ids, Tensor z) {
  check_i(w, at::kFloat, "w");
  check_i(ids, at::kInt, "ids");
  check_i(z, at::kFloat, "z");
  TORCH_CHECK(z.dim() == 2 && w.dim() == 2 && w.size(0) == z.size(0) && ids.sizes() == w.sizes() &&
                  w.size(1) <= z.size(1),
              "z [T, E]; w, ids [T, K], K <= E");
  HIP_OK(die::launch_topk_sigmoid(w.data_ptr<float>(), ids.data_ptr<int>(), z.data_ptr<float>(), (int)z.size(0),
                                  (int)z.size(1), (int)w.size(1), cur_stream()));
}

void gather_scaled(Tensor xs, Tensor x, OptTensor sorted, OptTensor w, int64_t topk) {
  const bool f = is_f32(x, "x");
  const float* wp = nullptr;
  if (w.has_value()) {
    check_i(*w, at::kFloat, "w");
    wp = w->data_ptr<float>();
  }
  TORCH_CHECK(is_f32(xs, "xs") == f && xs.is_contiguous() && x.is_contiguous() && xs.dim() == 2 && x.dim() == 2 &&
                  xs.size(1) == x.size(1) && xs.size(0) == x.size(0) * topk && (!w.has_value() || w->numel() == xs.size(0)),
              "gather_scaled shapes");
  const int* sp = nullptr;
  if (sorted.has_value()) {
    check_i(*sorted, at::kInt, "sorted");
    TORCH_CHECK(sorted->numel() == xs.size(0), "sorted [T * K]");
    sp = sorted->data_ptr<int>();
  }
  HIP_OK(die::launch_gather_scaled(xs.data_ptr(), x.data_ptr(), f, sp, wp, (int)xs.size(0),
                                   (int)topk, (int)x.size(1), cur_stream()));
}

const float* opt_f32(const OptTensor& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  check_i(*t, at::kFloat, name);
  TORCH_CHECK(t->numel() == n, name, ": expected ", n, " values");
  return t->data_ptr<float>();
}

void route_softmax_topk(Tensor w, Tensor ids, OptTensor gate, Tensor x, Tensor wr, int64_t n_route, OptTensor corr) {
  check_rows(x, "x");
  const bool xf = is_f32(x, "x"), wf = is_f32(wr, "wr");
  check_i(w, at::kFloat, "w");
  check_i(ids, at::kInt, "ids");
  const int64_t T = x.size(0);
  TORCH_CHECK(wr.dim() == 2 && wr.is_contiguous() && wr.size(1) == x.size(1) &&
                  wr.size(0) >= n_route + (gate.has_value() ? 1 : 0),
              "wr [>= n_route (+ 1 with a gate), H]");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == T && ids.sizes() == w.sizes() && w.size(1) <= n_route,
              "w, ids [T, K], K <= n_route");
  float* gp = const_cast<float*>(opt_f32(gate, T, "gate"));
  HIP_OK(die::launch_route_softmax_topk(w.data_ptr<float>(), ids.data_ptr<int>(), gp, x.data_ptr(), x.stride(0), xf,
                                        wr.data_ptr(), wf, opt_f32(corr, n_route, "corr"), (int)T, (int)x.size(1),
                                        (int)n_route, (int)w.size(1), cur_stream()));
}

void topk_softmax_corrected(Tensor w, Tensor ids, OptTensor gate, Tensor z, int64_t n_route, OptTensor corr) {
  check_i(w, at::kFloat, "w");
  check_i(ids, at::kInt, "ids");
  check_i(z, at::kFloat, "z");
  TORCH_CHECK(z.dim() == 2 && w.dim() == 2 && w.size(0) == z.size(0) && ids.sizes() == w.sizes() &&
                  w.size(1) <= n_route && z.size(1) >= n_route + (gate.has_value() ? 1 : 0),
              "z [T, >= n_route (+ 1 with a gate)]; w, ids [T, K], K <= n_route");
  float* gp = const_cast<float*>(opt_f32(gate, z.size(0), "gate"));
  HIP_OK(die::launch_topk_softmax_corrected(w.data_ptr<float>(), ids.data_ptr<int>(), gp, z.data_ptr<float>(),
                                            (int)z.size(1), opt_f32(corr, n_route, "corr"), (int)z.size(0),
                                            (int)n_route, (int)w.size(1), cur_stream()));
}

void combine_weighted(OptTensor out, OptTensor resid, OptTensor act, Tensor ys, OptTensor pos, Tensor x, Tensor wk,
                      Tensor ids, int64_t num_experts, OptTensor extra, OptTensor gate, OptTensor w, bool unit_offset,
                      double eps, double mult) {
  const bool f = is_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "x [T, H] contiguous");
  const int64_t T = x.size(0), H = x.size(1);
  check_i(wk, at::kFloat, "wk");
  check_i(ids, at::kInt, "ids");
  TORCH_CHECK(wk.dim() == 2 && wk.size(0) == T && ids.sizes() == wk.sizes(), "wk, ids [T, K]");
  const int64_t K = wk.size(1);
  TORCH_CHECK(is_f32(ys, "ys") == f && ys.is_contiguous() && ys.dim() == 2 && ys.size(1) == H &&
                  (ys.size(0) == T * K || num_experts == 0),
              "ys [T * K, H] in x's dtype");
  const int* pp = nullptr;
  if (pos.has_value()) {
    check_i(*pos, at::kInt, "pos");
    TORCH_CHECK(pos->numel() == T * K, "pos [T * K]");
    pp = pos->data_ptr<int>();
  }
  const void* ep = nullptr;
  if (extra.has_value()) {
    TORCH_CHECK(is_f32(*extra, "extra") == f && extra->is_contiguous() && extra->dim() == 2 && extra->size(0) == T &&
                    extra->size(1) == H,
                "extra [T, H] in x's dtype");
    ep = extra->data_ptr();
  }
  TORCH_CHECK(!gate.has_value() || extra.has_value(), "gate without extra");
  float* op = nullptr;
  if (out.has_value()) {
    check_i(*out, at::kFloat, "out");
    TORCH_CHECK(out->dim() == 2 && out->size(0) == T && out->size(1) == H, "out [T, H]");
    op = out->data_ptr<float>();
  }
  float* rp = nullptr;
  void* ap = nullptr;
  const void* wp = nullptr;
  bool wf = false;
  if (resid.has_value()) {
    check_i(*resid, at::kFloat, "resid");
    TORCH_CHECK(resid->dim() == 2 && resid->size(0) == T && resid->size(1) == H && w.has_value(), "resid [T, H], with w");
    rp = resid->data_ptr<float>();
    wf = is_f32(*w, "w");
    TORCH_CHECK(w->is_contiguous() && w->numel() == H, "w [H]");
    wp = w->data_ptr();
    if (act.has_value()) {
      TORCH_CHECK(is_f32(*act, "act") == f && act->is_contiguous() && act->sizes() == resid->sizes(),
                  "act: x's dtype, the residual's shape");
      ap = act->data_ptr();
    }
  }
  TORCH_CHECK(op != nullptr || rp != nullptr, "out or resid");
  HIP_OK(die::launch_combine_weighted(op, rp, ap, ys.data_ptr(), f, pp, x.data_ptr(), wk.data_ptr<float>(),
                                      ids.data_ptr<int>(), (int)num_experts, ep, opt_f32(gate, T, "gate"), (int)T,
                                      (int)K, (int)H, wp, wf, unit_offset, (float)eps, (float)mult, cur_stream()));
}

void combine_sum(Tensor out, Tensor ys, OptTensor pos, OptTensor extra, int64_t topk) {
  const bool f = is_f32(ys, "ys");
  check_i(out, at::kFloat, "out");
  TORCH_CHECK(out.dim() == 2 && ys.dim() == 2 && ys.is_contiguous() && ys.size(1) == out.size(1) &&
                  ys.size(0) == out.size(0) * topk,
              "combine_sum shapes");
  const int* pp = nullptr;
  if (pos.has_value()) {
    check_i(*pos, at::kInt, "pos");
    TORCH_CHECK(pos->numel() == ys.size(0), "pos [T * K]");
    pp = pos->data_ptr<int>();
  }
  const void* ep = nullptr;
  if (extra.has_value()) {
    TORCH_CHECK(is_f32(*extra, "extra") == f && extra->is_contiguous() && extra->sizes() == out.sizes(),
                "extra: same dtype as ys, shape of out");
    ep = extra->data_ptr();
  }
  HIP_OK(die::launch_combine_sum(out.data_ptr<float>(), ys.data_ptr(), f, pp, ep, (int)out.size(0), (int)topk,
                                 (int)out.size(1), cur_stream()));
}

die::LatentShape latent_shape(int64_t rank, int64_t rot_dim, const Tensor& inv_freq) {
  check_i(inv_freq, at::kFloat, "inv_freq");
  TORCH_CHECK(rank >= 1 && rot_dim >= 0 && inv_freq.numel() * 2 <= rot_dim, "latent shape");
  die::LatentShape sh;
  sh.rank = (int)rank;
  sh.rot_dim = (int)rot_dim;
  sh.rot_pairs = (int)inv_freq.numel();
  sh.inv_freq = inv_freq.data_ptr<float>();
  return sh;
}

// cache [num_blocks, block_size, rank + rot_dim]; kv [T, >= rank + rot_dim]
void latent_kv_write(Tensor cache, Tensor kv, Tensor w, Tensor positions, Tensor slots, int64_t rank, int64_t rot_dim,
                     Tensor inv_freq, double eps) {
  check_rows(kv, "kv");
  const bool f = is_f32(kv, "kv"), wf = is_f32(w, "w");
  TORCH_CHECK(is_f32(cache, "cache") == f && cache.is_contiguous() && cache.dim() == 3 &&
                  cache.size(2) == rank + rot_dim && kv.size(1) == rank + rot_dim,
              "latent_kv_write: cache [blocks, block_size, rank + rot_dim], kv [T, rank + rot_dim], same dtype");
  TORCH_CHECK(w.is_contiguous() && w.numel() == rank, "w [rank]");
  check_i(positions, at::kLong, "positions");
  check_i(slots, at::kLong, "slots");
  TORCH_CHECK(positions.numel() >= kv.size(0) && slots.numel() >= kv.size(0), "positions / slots [T]");
  HIP_OK(die::launch_latent_kv_write(cache.data_ptr(), kv.data_ptr(), kv.stride(0), f, w.data_ptr(), wf,
                                     positions.data_ptr<int64_t>(), slots.data_ptr<int64_t>(), (int)kv.size(0),
                                     latent_shape(rank, rot_dim, inv_freq), (float)eps, cur_stream()));
}

// p [T, q_rank + rank + rot_dim]: cq [T, q_rank] = rmsnorm(p[:, :q_rank]) * wq; cache rows from p[:, q_rank:]
void latent_qkv_prep(Tensor cq, Tensor cache, Tensor p, Tensor wq, Tensor wkv, Tensor positions, Tensor slots,
                     int64_t rank, int64_t rot_dim, Tensor inv_freq, double eps) {
  check_rows(p, "p");
  const bool f = is_f32(p, "p"), wf = is_f32(wq, "wq");
  const int64_t q_rank = p.size(1) - rank - rot_dim;
  TORCH_CHECK(q_rank >= 1, "p narrower than the cache row");
  TORCH_CHECK(is_f32(cq, "cq") == f && cq.is_contiguous() && cq.dim() == 2 && cq.size(0) == p.size(0) &&
                  cq.size(1) == q_rank,
              "cq [T, q_rank], dtype of p");
  TORCH_CHECK(is_f32(cache, "cache") == f && cache.is_contiguous() && cache.dim() == 3 &&
                  cache.size(2) == rank + rot_dim,
              "cache [blocks, block_size, rank + rot_dim], dtype of p");
  TORCH_CHECK(is_f32(wkv, "wkv") == wf && wq.is_contiguous() && wkv.is_contiguous() && wq.numel() == q_rank &&
                  wkv.numel() == rank,
              "wq [q_rank], wkv [rank], one dtype");
  check_i(positions, at::kLong, "positions");
  check_i(slots, at::kLong, "slots");
  TORCH_CHECK(positions.numel() >= p.size(0) && slots.numel() >= p.size(0), "positions / slots [T]");
  HIP_OK(die::launch_latent_qkv_prep(cq.data_ptr(), p.data_ptr(), p.stride(0), f, (int)q_rank, wq.data_ptr(),
                                     wkv.data_ptr(), wf, cache.data_ptr(), positions.data_ptr<int64_t>(),
                                     slots.data_ptr<int64_t>(), (int)p.size(0), latent_shape(rank, rot_dim, inv_freq),
                                     (float)eps, cur_stream()));
}

void combine_post_norm(Tensor resid, OptTensor act, Tensor ys, OptTensor pos, OptTensor extra, int64_t topk, Tensor w,
                       bool unit_offset, double eps) {
  const bool f = is_f32(ys, "ys"), wf = is_f32(w, "w");
  check_i(resid, at::kFloat, "resid");
  TORCH_CHECK(resid.dim() == 2 && ys.dim() == 2 && ys.is_contiguous() && ys.size(1) == resid.size(1) &&
                  ys.size(0) == resid.size(0) * topk && w.is_contiguous() && w.numel() == resid.size(1),
              "combine_post_norm shapes");
  const int* pp = nullptr;
  if (pos.has_value()) {
    check_i(*pos, at::kInt, "pos");
    TORCH_CHECK(pos->numel() == ys.size(0), "pos [T * K]");
    pp = pos->data_ptr<int>();
  }
  const void* ep = nullptr;
  if (extra.has_value()) {
    TORCH_CHECK(is_f32(*extra, "extra") == f && extra->is_contiguous() && extra->sizes() == resid.sizes(),
                "extra: same dtype as ys, shape of resid");
    ep = extra->data_ptr();
  }
  void* ap = nullptr;
  if (act.has_value()) {
    TORCH_CHECK(act->is_cuda() && act->scalar_type() == at::kBFloat16 && act->is_contiguous() &&
                    act->sizes() == resid.sizes(),
                "act must be a contiguous bf16 tensor of the residual's shape");
    ap = act->data_ptr();
  }
  HIP_OK(die::launch_combine_post_norm(resid.data_ptr<float>(), ap, ys.data_ptr(), f, pp, ep, (int)resid.size(0),
                                       (int)topk, (int)resid.size(1), w.data_ptr(), wf, unit_offset, (float)eps,
                                       cur_stream()));
}

// out, q_lat [H, T, rank]; q [T, H * qh] whose head h keeps its rotary part at [h * qh + rot_off, + rot_dim)
void latent_attn(Tensor out, Tensor q_lat, Tensor q, int64_t rot_off, Tensor cache, Tensor block_tables,
                 OptTensor cu_q, Tensor ctx_lens, Tensor positions, OptTensor sink, int64_t max_q, int64_t window,
                 double scale, int64_t rot_dim, Tensor inv_freq, int64_t impl) {
  const bool f = is_f32(q_lat, "q_lat");
  TORCH_CHECK(is_f32(out, "out") == f && is_f32(q, "q") == f && is_f32(cache, "cache") == f, "one dtype");
  TORCH_CHECK(q_lat.dim() == 3 && q_lat.is_contiguous() && out.is_contiguous() && out.sizes() == q_lat.sizes(),
              "q_lat, out [H, T, rank] contiguous");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), rank = q_lat.size(2);
  check_rows(q, "q");
  TORCH_CHECK(q.size(0) == T && q.size(1) % H == 0, "q [T, H * qh]");
  const int64_t qh = q.size(1) / H;
  TORCH_CHECK(rot_off >= 0 && rot_off + rot_dim <= qh, "rotary part outside the head");
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && cache.size(2) == rank + rot_dim, "cache layout");
  check_i(ctx_lens, at::kInt, "ctx_lens");
  check_i(positions, at::kLong, "positions");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                  block_tables.stride(1) == 1,
              "block_tables [S, W] int32");
  const int64_t S = block_tables.size(0);
  TORCH_CHECK(ctx_lens.numel() >= S && positions.numel() >= T, "ctx_lens [S], positions [T]");
  die::LatentAttnArgs a;
  a.out = out.data_ptr();
  a.q_lat = q_lat.data_ptr();
  a.q_rot = static_cast<const char*>(q.data_ptr()) + rot_off * q.element_size();
  a.q_stride = q.stride(0);
  a.q_hstride = qh;
  a.cache = cache.data_ptr();
  a.block_tables = block_tables.data_ptr<int>();
  a.bt_stride = (int)block_tables.stride(0);
  a.cu_q = nullptr;
  if (cu_q.has_value()) {
    check_i(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= S + 1, "cu_q [S + 1]");
    a.cu_q = cu_q->data_ptr<int>();
  } else {
    TORCH_CHECK(T >= S && max_q == 1, "without cu_q every sequence has one row");
  }
  a.ctx_lens = ctx_lens.data_ptr<int>();
  a.positions = positions.data_ptr<int64_t>();
  a.sink = nullptr;
  if (sink.has_value()) {
    check_i(*sink, at::kFloat, "sink");
    TORCH_CHECK(sink->numel() == H, "sink [H]");
    a.sink = sink->data_ptr<float>();
  }
  a.num_seqs = (int)S;
  a.total_q = (int)T;
  a.max_q = (int)max_q;
  a.heads = (int)H;
  a.block_size = (int)cache.size(1);
  a.window = (int)window;
  a.scale = (float)scale;
  a.sh = latent_shape(rank, rot_dim, inv_freq);
  a.f32 = f;
  a.impl = (int)impl;
  a.ws_o = a.ws_ml = nullptr;
  a.nsplit = 1;
  a.chunk = 0;
  Tensor ws_o, ws_ml;
  if (die::latent_attn_uses_mfma(a)) {
    // few row tiles (decode steps): split the keys over workgroups until about 256 are in flight. The key range
    // is bounded by the window, else by the block table's width (under a captured graph: the model length;
    // splits beyond a sequence's keys exit at once)
    const int64_t rows_wg = max_q * H <= 32 ? 32 : 128;
    const int64_t tiles = S * ((max_q * H + rows_wg - 1) / rows_wg);
    int64_t bound = block_tables.size(1) * cache.size(1);
    if (window > 0) bound = std::min<int64_t>(bound, window + max_q);
    int64_t ns = std::min<int64_t>({(int64_t)16, 512 / std::max<int64_t>(1, tiles), (bound + 63) / 64});
    if (ns > 1) {
      a.chunk = (int)((((bound + ns - 1) / ns) + 31) / 32 * 32);
      a.nsplit = (int)((bound + a.chunk - 1) / a.chunk);
      if (a.nsplit > 1) {
        ws_o = at::empty({a.nsplit, H * T, rank}, q_lat.options().dtype(at::kFloat));
        ws_ml = at::empty({a.nsplit, H * T, 2}, q_lat.options().dtype(at::kFloat));
        a.ws_o = ws_o.data_ptr<float>();
        a.ws_ml = ws_ml.data_ptr<float>();
      } else {
        a.nsplit = 1;
      }
    }
  }
  HIP_OK(die::launch_latent_attn(a, cur_stream()));
}

void moe_align(Tensor offsets, Tensor sorted, Tensor pos, Tensor ids, int64_t num_experts) {
  check_i(offsets, at::kInt, "offsets");
  check_i(sorted, at::kInt, "sorted");
  check_i(pos, at::kInt, "pos");
  check_i(ids, at::kInt, "ids");
  TORCH_CHECK(offsets.numel() >= num_experts + 1 && sorted.numel() >= ids.numel() && pos.numel() >= ids.numel(),
              "moe_align buffers");
  HIP_OK(die::launch_moe_align(offsets.data_ptr<int>(), sorted.data_ptr<int>(), pos.data_ptr<int>(),
                               ids.data_ptr<int>(), (int)ids.numel(), (int)num_experts, cur_stream()));
}

}  // namespace

void register_seq_ops(pybind11::module& m);  // csrc/bindings_seq.cpp
void register_lin_ops(pybind11::module& m);  // csrc/bindings_lin.cpp
void register_rec_ops(pybind11::module& m);  // csrc/bindings_rec.cpp

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  register_seq_ops(m);
  register_lin_ops(m);
  register_rec_ops(m);
  m.def("route_softmax_topk", &route_softmax_topk);
  m.def("topk_softmax_corrected", &topk_softmax_corrected);
  m.def("combine_weighted", &combine_weighted);
  m.def("rms_norm_ext", &rms_norm_ext);
  m.def("post_norm_residual", &post_norm_residual);
  m.def("gated_act", &gated_act);
  m.def("route_sigmoid_topk", &route_sigmoid_topk);
  m.def("topk_sigmoid", &topk_sigmoid);
  m.def("gather_scaled", &gather_scaled);
  m.def("combine_sum", &combine_sum);
  m.def("latent_kv_write", &latent_kv_write);
  m.def("latent_attn", &latent_attn);
  m.def("latent_qkv_prep", &latent_qkv_prep);
  m.def("combine_post_norm", &combine_post_norm);
  m.def("moe_align", &moe_align);
}
