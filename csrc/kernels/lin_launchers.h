// Host launchers of the kernels for layer stacks with sandwich norms (a norm before and after every sublayer),
// a learned weighted average over the results of all earlier layers ("depth-weighted average"), learned position
// vectors, biased squared-ReLU feed-forwards, per-head and per-channel sigmoid output gates, and linear attention
// with a fixed decay per head (a recurrent fp32 matrix state per head). Raw pointers + an explicit stream, no
// allocation and no synchronisation: every launcher is hipGraph-capturable. `f32` selects the storage type of
// activations and weight matrices (false: bf16); norm weights, decays and the residual planes are always fp32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "seq_launchers.h"

namespace die {

// out[t] (fp32) = embed[ids[t]] + pos[positions[t]]
hipError_t launch_embed_pos(float* out, const void* embed, const void* pos, bool f32, const int64_t* ids,
                            const int64_t* positions, int T, int W, hipStream_t s);

// One launch at a sublayer boundary inside a layer: resid[t] (fp32, in place) += rms(y[t] + ybias) * w_post, then
// h[t] = rms(resid[t]) * w_pre (h == nullptr: no second norm). rms(v) = v / sqrt(mean(v^2) + eps).
struct PostPreNormArgs {
  float* resid;          // [T, W]
  const void* y;         // [T, W], row stride ystride
  int64_t ystride;
  bool y_f32;
  const void* ybias;     // [W] in y's storage type, or nullptr
  const float* w_post;   // [W]
  const float* w_pre;    // [W] or nullptr
  void* h;               // [T, W] or nullptr
  bool h_f32;
  float eps;
  int T, W;
};
hipError_t launch_post_pre_norm(const PostPreNormArgs& a, hipStream_t s);

// One launch at a layer boundary. planes [>= n + 1, T, W] fp32 hold X_0 .. X_(n-1): the embedding output and the
// results of the layers so far, plane n - 1 being the running residual of the layer that just ended.
//   y != nullptr:  planes[n - 1] += rms(y + ybias) * w_post      (the layer's last post-norm, finishing X_(n-1))
//   planes[n]  = sum_(j < n) dw[j] * planes[j]                   (the next layer's input and running residual;
//                                                                 dw == nullptr: a copy of plane n - 1)
//   h          = rms(planes[n]) * w_pre                          (the next layer's first norm, or the final norm)
struct DepthAvgArgs {
  float* planes;
  int64_t plane_stride;  // T * W
  int n;
  const float* dw;       // [n] or nullptr
  const void* y;
  int64_t ystride;
  bool y_f32;
  const void* ybias;
  const float* w_post;
  const float* w_pre;
  void* h;
  bool h_f32;
  float eps;
  int T, W;
};
hipError_t launch_depth_avg_norm(const DepthAvgArgs& a, hipStream_t s);

// out[r, c] = relu(z[r, c] + b[c])^2
hipError_t launch_bias_relu2(void* out, const void* z, const void* b, bool f32, int rows, int n, hipStream_t s);

// out[i] (fp32) = cap * tanh(z[i] / cap), cap > 0
hipError_t launch_tanh_cap(float* out, const void* z, bool f32, float cap, int64_t total, hipStream_t s);

// out[t, h * v + c] = o[h, t, c] * sigmoid(g[t * gstride + h]): per-head output gate, fused with the move from
// head-major to token-major
hipError_t launch_head_gate(void* out, const void* o, const void* g, int64_t gstride, bool f32, int T, int H, int v,
                            hipStream_t s);

// out[t] = rms(o[t]) * w * sigmoid(g[t]) over rows of n values; o fp32, g (row stride gstride) and out in the
// activation type
hipError_t launch_norm_sigmoid_gate(void* out, const float* o, const void* g, int64_t gstride, bool f32,
                                    const float* w, float eps, int T, int n, hipStream_t s);

// Linear attention with a fixed decay per head. x [T, xstride] holds the projections q | k (H * dim each) and
// v (H * vdim) at column offsets qoff / koff / voff; SiLU is applied on load (and rounded to the storage type).
// Per (sequence, head), token by token: S <- decay[h] * S + k v^T; o = S^T q, with S [dim, vdim] fp32 kept in
// state [slots, H, dim, vdim]. out [T, H * vdim] fp32.
struct LightningArgs {
  float* out;
  const void* x;
  int64_t xstride;
  int qoff, koff, voff;
  bool f32;
  const float* decay;    // [H]
  float* state;
  int heads, dim, vdim;
};
hipError_t launch_lightning_attn(const LightningArgs& a, RaggedRows r, hipStream_t s);

}  // namespace die
