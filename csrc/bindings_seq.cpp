// Torch bindings of the sequence-state kernels (csrc/kernels/seq_mix.hip) and the sink attention
// (csrc/kernels/sink_attn.hip); registered into src/_Cmix by register_seq_ops(). Shapes, dtypes, devices and
// index ranges that the host can see are validated here; the launchers trust them.
#include <ATen/hip/HIPContext.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include "kernels/seq_launchers.h"

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

const float* f32_ptr(const OptTensor& t, int64_t n, const char* name) {
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

void embed_hash(Tensor streams, Tensor embed, OptTensor bigram, Tensor ids, Tensor positions, OptTensor cu_q,
                Tensor state_slots, Tensor prev_tok, double scale, int64_t buckets, int64_t mul_prev,
                int64_t mul_cur) {
  check_c(streams, at::kFloat, "streams");
  TORCH_CHECK(streams.dim() == 3, "streams [T, S, W]");
  const int64_t T = streams.size(0), S = streams.size(1), W = streams.size(2);
  const bool f = is_f32(embed, "embed");
  TORCH_CHECK(embed.dim() == 2 && embed.is_contiguous() && embed.size(1) == W, "embed [V, W]");
  check_c(ids, at::kLong, "ids");
  check_c(prev_tok, at::kLong, "prev_tok");
  TORCH_CHECK(ids.numel() >= T, "ids [T]");
  const void* bp = nullptr;
  if (bigram.has_value()) {
    TORCH_CHECK(is_f32(*bigram, "bigram") == f && bigram->dim() == 2 && bigram->is_contiguous() &&
                    bigram->size(1) == W && bigram->size(0) == buckets + 1 && buckets >= 1 && mul_prev >= 0 &&
                    mul_cur >= 0,
                "bigram [buckets + 1, W] of the embedding's dtype");
    bp = bigram->data_ptr();
  }
  auto r = ragged(T, positions, cu_q, state_slots);
  HIP_OK(die::launch_embed_hash(streams.data_ptr<float>(), (int)S, (int)W, embed.data_ptr(), bp, f,
                                ids.data_ptr<int64_t>(), r, prev_tok.data_ptr<int64_t>(), (float)scale, buckets,
                                mul_prev, mul_cur, cur_stream()));
}

void store_last_token(Tensor prev_tok, Tensor ids, Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_c(ids, at::kLong, "ids");
  check_c(prev_tok, at::kLong, "prev_tok");
  auto r = ragged(ids.numel(), positions, cu_q, state_slots);
  HIP_OK(die::launch_store_last_token(prev_tok.data_ptr<int64_t>(), ids.data_ptr<int64_t>(), r, cur_stream()));
}

void stream_mix_norm(Tensor streams, OptTensor y1, OptTensor y2, double a1, double a2, OptTensor mix, OptTensor outw,
                     OptTensor inw, OptTensor gain, double eps, OptTensor h) {
  check_c(streams, at::kFloat, "streams");
  TORCH_CHECK(streams.dim() == 3, "streams [T, S, W]");
  die::StreamMixArgs a;
  a.streams = streams.data_ptr<float>();
  a.T = (int)streams.size(0);
  a.S = (int)streams.size(1);
  a.W = (int)streams.size(2);
  a.y1 = a.y2 = nullptr;
  a.ys1 = a.ys2 = 0;
  a.y_f32 = true;
  if (y1.has_value()) {
    check_rows(*y1, "y1");
    a.y_f32 = is_f32(*y1, "y1");
    TORCH_CHECK(y1->size(0) == a.T && y1->size(1) == a.W, "y1 [T, W]");
    a.y1 = y1->data_ptr();
    a.ys1 = y1->stride(0);
    if (y2.has_value()) {
      check_rows(*y2, "y2");
      TORCH_CHECK(is_f32(*y2, "y2") == a.y_f32 && y2->size(0) == a.T && y2->size(1) == a.W, "y2 like y1");
      a.y2 = y2->data_ptr();
      a.ys2 = y2->stride(0);
    }
  }
  a.a1 = (float)a1;
  a.a2 = (float)a2;
  a.mix = f32_ptr(mix, (int64_t)a.S * a.S, "mix");
  a.outw = f32_ptr(outw, a.S, "outw");
  a.inw = f32_ptr(inw, a.S, "inw");
  a.gain = f32_ptr(gain, 1, "gain");
  a.eps = (float)eps;
  a.h = nullptr;
  a.h_f32 = true;
  if (h.has_value()) {
    a.h_f32 = is_f32(*h, "h");
    TORCH_CHECK(h->dim() == 2 && h->is_contiguous() && h->size(0) == a.T && h->size(1) == a.W, "h [T, W]");
    TORCH_CHECK(a.gain != nullptr, "h needs the norm's gain");
    a.h = h->data_ptr();
  }
  HIP_OK(die::launch_stream_mix_norm(a, cur_stream()));
}

void poly_norm_act(Tensor out, Tensor z, Tensor coef, double eps) {
  check_rows(z, "z");
  const bool f = is_f32(z, "z");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.sizes() == z.sizes(), "out like z, contiguous");
  HIP_OK(die::launch_poly_norm_act(out.data_ptr(), z.data_ptr(), z.stride(0), f, f32_ptr(coef, 4, "coef"), (float)eps,
                                   (int)z.size(0), (int)z.size(1), cur_stream()));
}

die::DeltaShape delta_shape(int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, int64_t taps) {
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1 && dim <= 256 && vdim >= 1 &&
                  vdim <= 256 && taps >= 1 && taps <= 16,
              "gated delta rule: heads % kv_heads == 0, dim and vdim in 1..256, taps in 1..16");
  die::DeltaShape sh;
  sh.heads = (int)heads;
  sh.kv_heads = (int)kv_heads;
  sh.dim = (int)dim;
  sh.vdim = (int)vdim;
  sh.taps = (int)taps;
  return sh;
}

// x [T, C], b [T, heads], a [T, heads]: column slices of ONE projection output (same row stride)
void delta_prep(Tensor qkv32, Tensor bg, Tensor x, Tensor b, Tensor a, Tensor conv_w, OptTensor conv_wt,
                Tensor conv_state, Tensor A_log, Tensor dt_bias, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, Tensor positions,
                OptTensor cu_q, Tensor state_slots) {
  TORCH_CHECK(conv_w.dim() == 2, "conv_w [C, taps]");
  auto sh = delta_shape(heads, kv_heads, dim, vdim, conv_w.size(1));
  const int64_t C = sh.channels(), T = x.size(0);
  check_rows(x, "x");
  check_rows(b, "b");
  check_rows(a, "a");
  const bool f = is_f32(x, "x");
  TORCH_CHECK(is_f32(b, "b") == f && is_f32(a, "a") == f, "one dtype");
  TORCH_CHECK(x.size(1) == C && b.size(0) == T && a.size(0) == T && b.size(1) == heads && a.size(1) == heads &&
                  b.stride(0) == x.stride(0) && a.stride(0) == x.stride(0),
              "x [T, C], b / a [T, heads], slices of one projection");
  check_c(qkv32, at::kFloat, "qkv32");
  check_c(bg, at::kFloat, "bg");
  TORCH_CHECK(qkv32.numel() == T * C && bg.numel() == T * 2 * heads, "qkv32 [T, C], bg [T, 2 heads]");
  check_c(conv_state, at::kFloat, "conv_state");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(1) == sh.taps - 1 && conv_state.size(2) == C,
              "conv_state [slots, taps - 1, C]");
  auto r = ragged(T, positions, cu_q, state_slots);
  HIP_OK(die::launch_delta_prep(qkv32.data_ptr<float>(), bg.data_ptr<float>(), x.data_ptr(), b.data_ptr(),
                                a.data_ptr(), x.stride(0), f, f32_ptr(conv_w, C * sh.taps, "conv_w"),
                                f32_ptr(conv_wt, C * sh.taps, "conv_wt"), conv_state.data_ptr<float>(), f32_ptr(A_log, heads, "A_log"),
                                f32_ptr(dt_bias, heads, "dt_bias"), sh, r, cur_stream()));
}

void conv_state_update(Tensor conv_state, Tensor x, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                       Tensor positions, OptTensor cu_q, Tensor state_slots) {
  check_c(conv_state, at::kFloat, "conv_state");
  TORCH_CHECK(conv_state.dim() == 3, "conv_state [slots, taps - 1, C]");
  auto sh = delta_shape(heads, kv_heads, dim, vdim, conv_state.size(1) + 1);
  check_rows(x, "x");
  TORCH_CHECK(x.size(1) == sh.channels() && conv_state.size(2) == sh.channels(), "x [T, C]");
  auto r = ragged(x.size(0), positions, cu_q, state_slots);
  HIP_OK(die::launch_conv_state_update(conv_state.data_ptr<float>(), x.data_ptr(), x.stride(0), is_f32(x, "x"), sh, r,
                                       cur_stream()));
}

void gated_delta(Tensor out, Tensor qkv32, Tensor bg, Tensor gate, Tensor norm_w, double eps, Tensor state,
                 int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, Tensor positions, OptTensor cu_q,
                 Tensor state_slots) {
  auto sh = delta_shape(heads, kv_heads, dim, vdim, 1);
  const int64_t C = sh.channels();
  check_c(qkv32, at::kFloat, "qkv32");
  check_c(bg, at::kFloat, "bg");
  TORCH_CHECK(qkv32.dim() == 2 && qkv32.size(1) == C, "qkv32 [T, C]");
  const int64_t T = qkv32.size(0);
  TORCH_CHECK(bg.numel() == T * 2 * heads, "bg [T, 2 heads]");
  check_rows(gate, "gate");
  const bool f = is_f32(gate, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == heads * vdim, "gate [T, heads * vdim]");
  TORCH_CHECK(is_f32(out, "out") == f && out.is_contiguous() && out.numel() == T * heads * vdim,
              "out [T, heads * vdim] contiguous");
  check_c(state, at::kFloat, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dim && state.size(3) == vdim,
              "state [slots, heads, dim, vdim]");
  auto r = ragged(T, positions, cu_q, state_slots);
  HIP_OK(die::launch_gated_delta(out.data_ptr(), qkv32.data_ptr<float>(), bg.data_ptr<float>(), gate.data_ptr(),
                                 gate.stride(0), f, f32_ptr(norm_w, vdim, "norm_w"), (float)eps,
                                 state.data_ptr<float>(), sh, r, cur_stream()));
}

// q [T, H * dim], k [T, G * dim], v [T, G * vdim]: column slices of ONE projection output
void qkv_prep(Tensor q_out, Tensor cache, Tensor q, Tensor k, OptTensor v, int64_t heads, int64_t kv_heads,
              int64_t dim, int64_t vdim, OptTensor q_norm, OptTensor k_norm, int64_t rot_dims, OptTensor inv_freq,
              bool v_unit, OptTensor v_lambda, OptTensor v_first, double eps, Tensor positions, Tensor slots,
              bool head_norm, double q_temp_coef, int64_t q_temp_every, bool norm_after_rot) {
  check_rows(q, "q");
  check_rows(k, "k");
  die::QkvPrepArgs a;
  a.f32 = is_f32(q, "q");
  const int64_t T = q.size(0);
  TORCH_CHECK(is_f32(k, "k") == a.f32 && is_f32(q_out, "q_out") == a.f32 && is_f32(cache, "cache") == a.f32,
              "one dtype");
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0, "heads % kv_heads == 0");
  TORCH_CHECK(q.size(1) == heads * dim && k.size(1) == kv_heads * dim && k.size(0) == T &&
                  k.stride(0) == q.stride(0),
              "q / k: slices of one projection");
  if (v.has_value()) {
    check_rows(*v, "v");
    TORCH_CHECK(is_f32(*v, "v") == a.f32 && v->size(1) == kv_heads * vdim && v->size(0) == T &&
                    v->stride(0) == q.stride(0),
                "v: a slice of the same projection");
  } else {
    TORCH_CHECK(vdim == dim && !v_lambda.has_value(), "values taken from the keys: vdim == dim, no value mixing");
  }
  TORCH_CHECK(q_temp_coef == 0.0 || q_temp_every >= 1, "q_temp_every >= 1");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == T * heads * dim, "q_out [T, H * dim]");
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == kv_heads * (dim + vdim),
              "cache [blocks, block_size, G * (dim + vdim)]");
  check_c(positions, at::kLong, "positions");
  check_c(slots, at::kLong, "slots");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "positions, slots [T]");
  a.q = q.data_ptr();
  a.k = k.data_ptr();
  a.v = v.has_value() ? v->data_ptr() : nullptr;
  a.xstride = q.stride(0);
  a.T = (int)T;
  a.heads = (int)heads;
  a.kv_heads = (int)kv_heads;
  a.dim = (int)dim;
  a.vdim = (int)vdim;
  a.head_norm = head_norm;
  TORCH_CHECK(!norm_after_rot || (head_norm && v.has_value()),
              "norm_after_rot is a form of head_norm, and not for values taken from the keys");
  a.norm_after_rot = norm_after_rot;
  TORCH_CHECK(!head_norm || q_norm.has_value(), "head_norm needs the norm weights");
  a.q_norm = f32_ptr(q_norm, head_norm ? dim : heads * dim, "q_norm");
  a.k_norm = f32_ptr(k_norm, head_norm ? dim : kv_heads * dim, "k_norm");
  a.q_temp_coef = (float)q_temp_coef;
  a.q_temp_every = (int)q_temp_every;
  a.rot_dims = (int)rot_dims;
  a.inv_freq = f32_ptr(inv_freq, rot_dims / 2, "inv_freq");
  a.v_unit = v_unit;
  a.v_lambda = f32_ptr(v_lambda, 1, "v_lambda");
  a.v_first = nullptr;
  a.vfstride = 0;
  if (v_first.has_value()) {
    check_rows(*v_first, "v_first");
    TORCH_CHECK(is_f32(*v_first, "v_first") == a.f32 && v_first->size(0) == T && v_first->size(1) == kv_heads * vdim,
                "v_first [T, G * vdim]");
    a.v_first = v_first->data_ptr();
    a.vfstride = v_first->stride(0);
  }
  a.eps = (float)eps;
  a.positions = positions.data_ptr<int64_t>();
  a.slots = slots.data_ptr<int64_t>();
  a.q_out = q_out.data_ptr();
  a.cache = cache.data_ptr();
  a.block_size = (int)cache.size(1);
  HIP_OK(die::launch_qkv_prep(a, cur_stream()));
}

void sink_attn(Tensor out, Tensor q, Tensor cache, Tensor block_tables, OptTensor cu_q, Tensor ctx_lens,
               Tensor positions, OptTensor sink, OptTensor bias, int64_t max_q, int64_t heads, int64_t kv_heads,
               int64_t dim, int64_t vdim, int64_t window, double scale, int64_t impl, double softcap,
               OptTensor slopes) {
  die::SinkAttnArgs a;
  a.f32 = is_f32(q, "q");
  TORCH_CHECK(is_f32(out, "out") == a.f32 && is_f32(cache, "cache") == a.f32, "one dtype");
  TORCH_CHECK(q.dim() == 2 && q.is_contiguous() && q.size(1) == heads * dim, "q [T, H * dim] contiguous");
  const int64_t T = q.size(0);
  TORCH_CHECK(out.is_contiguous() && out.numel() == T * heads * vdim, "out [T, H * vdim] contiguous");
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0, "heads % kv_heads == 0");
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && cache.size(2) == kv_heads * (dim + vdim), "cache layout");
  check_c(ctx_lens, at::kInt, "ctx_lens");
  check_c(positions, at::kLong, "positions");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                  block_tables.stride(1) == 1,
              "block_tables [S, W] int32");
  const int64_t S = block_tables.size(0);
  TORCH_CHECK(ctx_lens.numel() >= S && positions.numel() >= T, "ctx_lens [S], positions [T]");
  a.out = out.data_ptr();
  a.q = q.data_ptr();
  a.cache = cache.data_ptr();
  a.block_tables = block_tables.data_ptr<int>();
  a.bt_stride = (int)block_tables.stride(0);
  a.cu_q = nullptr;
  if (cu_q.has_value()) {
    check_c(*cu_q, at::kInt, "cu_q");
    TORCH_CHECK(cu_q->numel() >= S + 1, "cu_q [S + 1]");
    a.cu_q = cu_q->data_ptr<int>();
  } else {
    TORCH_CHECK(T >= S && max_q == 1, "without cu_q every sequence has one row");
  }
  a.ctx_lens = ctx_lens.data_ptr<int>();
  a.positions = positions.data_ptr<int64_t>();
  a.sink = f32_ptr(sink, heads, "sink");
  a.bias = nullptr;
  a.bias_rows = 0;
  if (bias.has_value()) {
    check_c(*bias, at::kFloat, "bias");
    TORCH_CHECK(bias->dim() == 2 && bias->size(1) == heads && bias->size(0) >= 1, "bias [rows, H]");
    a.bias = bias->data_ptr<float>();
    a.bias_rows = (int)bias->size(0);
  }
  TORCH_CHECK(softcap >= 0.0, "softcap >= 0");
  a.softcap = (float)softcap;
  a.slopes = f32_ptr(slopes, heads, "slopes");
  a.num_seqs = (int)S;
  a.total_q = (int)T;
  a.max_q = (int)max_q;
  a.heads = (int)heads;
  a.kv_heads = (int)kv_heads;
  a.dim = (int)dim;
  a.vdim = (int)vdim;
  a.block_size = (int)cache.size(1);
  a.window = (int)window;
  a.scale = (float)scale;
  a.impl = (int)impl;
  a.ws_o = a.ws_ml = nullptr;
  a.nsplit = 1;
  a.chunk = 0;
  Tensor ws_o, ws_ml;
  // The key range is bounded by the window, else by the block table's width (under a captured graph: the model
  // length; splits beyond a sequence's keys exit at once)
  int64_t bound = block_tables.size(1) * cache.size(1);
  if (window > 0) bound = std::min<int64_t>(bound, window + max_q);
  int64_t ns = 1;
  if (die::sink_attn_uses_decode(a)) {
    // decode steps: a workgroup per (sequence, key/value head, split); trips of 128 keys, splits until about 2048
    // workgroups are in flight
    const int64_t wgs = S * kv_heads;
    ns = std::min<int64_t>({(int64_t)128, std::max<int64_t>(1, 2048 / std::max<int64_t>(1, wgs)), (bound + 127) / 128});
    if (ns > 1) a.chunk = (int)((((bound + ns - 1) / ns) + 127) / 128 * 128);
  } else if (die::sink_attn_uses_mfma(a)) {
    // few row tiles: split the keys over workgroups until about 2048 are in flight
    const int64_t qpg = heads / kv_heads;
    const int64_t rows_wg = max_q * qpg <= 32 ? 32 : 128;
    const int64_t tiles = S * kv_heads * ((max_q * qpg + rows_wg - 1) / rows_wg);
    ns = std::min<int64_t>({(int64_t)16, 2048 / std::max<int64_t>(1, tiles), (bound + 63) / 64});
    if (ns > 1) a.chunk = (int)((((bound + ns - 1) / ns) + 31) / 32 * 32);
  }
  if (ns > 1) {
    a.nsplit = (int)((bound + a.chunk - 1) / a.chunk);
    if (a.nsplit > 1) {
      ws_o = at::empty({a.nsplit, T * heads, vdim}, q.options().dtype(at::kFloat));
      ws_ml = at::empty({a.nsplit, T * heads, 2}, q.options().dtype(at::kFloat));
      a.ws_o = ws_o.data_ptr<float>();
      a.ws_ml = ws_ml.data_ptr<float>();
    } else {
      a.nsplit = 1;
    }
  }
  HIP_OK(die::launch_sink_attn(a, cur_stream()));
}

}  // namespace

void register_seq_ops(pybind11::module& m) {
  m.def("embed_hash", &embed_hash);
  m.def("store_last_token", &store_last_token);
  m.def("stream_mix_norm", &stream_mix_norm);
  m.def("poly_norm_act", &poly_norm_act);
  m.def("delta_prep", &delta_prep);
  m.def("conv_state_update", &conv_state_update);
  m.def("gated_delta", &gated_delta);
  m.def("qkv_prep", &qkv_prep);
  m.def("sink_attn", &sink_attn);
}
