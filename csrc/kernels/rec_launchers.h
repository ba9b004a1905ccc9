// Host launchers of the kernels for recurrent mixers whose state is a vector per channel or a matrix per head:
// short causal convolutions with bias, the selective scan (diagonal state per channel, input-dependent step size
// and maps), log-space exponential gates under a running maximum, the matrix recurrence S <- a S + b k v^T with one
// (a, b) per token and head (scalar-decay state-space layers, matrix-memory LSTMs), their read-out epilogues, and
// the residual update of two side-by-side sublayers. Raw pointers + an explicit stream, no allocation and no
// synchronisation: every launcher is hipGraph-capturable. `f32` selects the storage type of activations and weight
// matrices (false: bf16); gates, decays, step sizes, norm weights, recurrent state and the residual are always fp32.
//
// A step is a ragged batch (RaggedRows, seq_launchers.h): a sequence whose first row of the step is at position 0
// starts from zero state, whatever its slot holds.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "seq_launchers.h"

namespace die {

// resid[t] (fp32) = embed[ids[t]] * scale; act[t] (optional, the table's type) = the same, rounded
hipError_t launch_embed_scaled(float* resid, void* act, const void* embed, bool f32, const int64_t* ids, float scale,
                               int T, int W, hipStream_t s);

struct ConvSiluArgs {
  void* y;                 // [T, C] contiguous, x's type
  const void* x;           // [T, C], row stride xstride
  int64_t xstride;
  bool f32;
  const float* w;          // [C, taps]
  const float* wt;         // [taps, C] or nullptr (16-byte loads in bf16 steps)
  const float* bias;       // [C] or nullptr
  float* conv_state;       // [slots, taps - 1, C], the most recent input last
  int C, taps;
  // optional: per-head step size and decay of a scalar-decay state-space layer, from dt [T, H] (row stride xstride,
  // x's type): d = softplus(dt + dt_bias[h]); ab[t, h] = (exp(-exp(A_log[h]) * d), d)
  const void* dt;
  const float* dt_bias;
  const float* A_log;
  float* ab;               // [T, H, 2]
  int H;
};
// y[t, c] = silu(bias[c] + sum_j w[c, j] * x[t - (taps - 1 - j), c]); rows before the step come from conv_state, rows
// before the sequence's start are zero. A step with one row per sequence (cu_q == nullptr) also moves the row's input
// into conv_state.
hipError_t launch_conv_silu(const ConvSiluArgs& a, RaggedRows r, hipStream_t s);
// conv_state[slot(s)] = the last taps - 1 inputs of sequence s after this step (nothing to do when cu_q == nullptr)
hipError_t launch_conv_tail_update(float* conv_state, const void* x, int64_t xstride, bool f32, int C, int taps,
                                   RaggedRows r, hipStream_t s);

struct SelectiveScanArgs {
  void* out;               // [T, I] contiguous, x's type: y * silu(z)
  const void* x;           // [T, I] row stride xstride: the convolved, activated input
  const void* dt;          // [T, I] row stride dtstride: the step size before bias and softplus
  const void* bc;          // [T, *] row stride bcstride: B_t at column boff, C_t at column coff, N values each
  const void* z;           // [T, I] row stride zstride
  int64_t xstride, dtstride, bcstride, zstride;
  int boff, coff;
  bool f32;
  const float* dt_bias;    // [I]
  const float* A;          // [I, N], negative
  const float* D;          // [I]
  float* state;            // [slots, I, N]
  int I, N;
};
// Per (sequence, channel c), token by token, d = softplus(dt + dt_bias[c]):
//   S[c, n] <- exp(d * A[c, n]) * S[c, n] + d * x * B[n];   y = sum_n S[c, n] * C[n] + D[c] * x;   out = y * silu(z)
hipError_t launch_selective_scan(const SelectiveScanArgs& a, RaggedRows r, hipStream_t s);

// Log-space gates of a matrix-memory LSTM. x [T, *] (row stride xstride) holds the raw pre-activations of H heads
// at columns ioff / foff. i = cap * tanh((x_i + i_bias) / cap); f = logsigmoid(cap * tanh((x_f + f_bias) / cap));
// m_t = max(f + m_(t-1), i) with m (per sequence and head) in m_state [slots, H], 0 at a sequence's start.
// abe[t, h] = (exp(f + m_(t-1) - m_t), exp(i - m_t), exp(-m_t)).
hipError_t launch_exp_gate_scan(float* abe, const void* x, int64_t xstride, int ioff, int foff, bool f32,
                                const float* i_bias, const float* f_bias, float cap, float* m_state, int H,
                                RaggedRows r, hipStream_t s);

struct GatedLinearArgs {
  float* out;              // [T, H * vdim]
  float* nq;               // [T, H] or nullptr: n . q of the normaliser
  const void* x;           // [T, *] row stride xstride: q | k (G * dim each) at qoff / koff, v (H * vdim) at voff
  int64_t xstride;
  int qoff, koff, voff;
  bool f32;
  const float* ab;         // [T, H, abw]: (a, b) = the first two entries
  int abw;
  float* state;            // [slots, H, dim, vdim]
  float* n_state;          // [slots, H, dim] or nullptr
  int heads, groups, dim, vdim;
  float qscale;
};
// Per (sequence, head), token by token: S <- a S + b k v^T; o = S^T (q * qscale); with n_state also
// n <- a n + b k and nq = n . (q * qscale). Head h reads q and k of group h / (heads / groups).
hipError_t launch_gated_linear_attn(const GatedLinearArgs& a, RaggedRows r, hipStream_t s);

// out[t, h, :] = rms(o[t, h, :] / (max(|nq[t, h]|, abe[t, h, 2]) + 1e-6)) * w[h, :] * sigmoid(g[t, h, :]); o fp32,
// g (row stride gstride) and out in the activation type
hipError_t launch_head_norm_gate(void* out, const float* o, const float* nq, const float* abe, const void* g,
                                 int64_t gstride, bool f32, const float* w, int T, int H, int vdim, float eps,
                                 hipStream_t s);

// y = (o + D[h] * x) * silu(z); out = rms(y) over each of `parts` equal parts of the row * w; o fp32 [T, H * vdim];
// x, z (row strides xstride / zstride) and out in the activation type
hipError_t launch_skip_gate_group_norm(void* out, const float* o, const void* x, int64_t xstride, const float* D,
                                       const void* z, int64_t zstride, bool f32, const float* w, int T, int H, int vdim,
                                       int parts, float eps, hipStream_t s);

// resid[t] (fp32) += mult * rms(u) * (1 + w), u = (rms(y1[t]) * w1 + rms(y2[t]) * w2) / 2; act[t] (optional, the
// activation type) = resid[t]. w in the activation type, w1 / w2 fp32.
hipError_t launch_pair_post_norm_residual(float* resid, void* act, const void* y1, int64_t ys1, const float* w1,
                                          const void* y2, int64_t ys2, const float* w2, bool f32, const void* w,
                                          float mult, float eps, int T, int W, hipStream_t s);

}  // namespace die
