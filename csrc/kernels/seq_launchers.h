// Host launchers of the kernels for models that carry per-sequence state besides a paged KV cache: hashed
// bigram embeddings (the previous token is state), several residual streams with learned mixing
// ("hyper-connections"), a polynomial feed-forward activation, short causal convolutions and the gated delta
// rule (a recurrent fp32 matrix state per head), and grouped-query softmax attention with a per-head sink, an
// optional sliding window and an optional learned bias per (distance, head). Raw pointers + an explicit
// stream, no allocation and no synchronisation: every launcher is hipGraph-capturable. `f32` selects the
// storage type of activation / cache tensors (false: bf16); small parameter vectors are always fp32.
//
// A step is a ragged batch: sequence s owns rows cu_q[s] .. cu_q[s + 1] - 1 (cu_q == nullptr: one row per
// sequence, row s), positions[row] is the row's position in its sequence, state_slots[s] the sequence's slot in
// every state tensor. A sequence whose first row of the step is at position 0 starts from zero state, whatever
// its slot holds.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace die {

struct RaggedRows {
  const int* cu_q;            // [S + 1] or nullptr
  const int64_t* positions;   // [T]
  const int* state_slots;     // [S]
  int num_seqs, total_rows;
};

// streams[t, s, :] (fp32, s < S) = embed[ids[t]] * scale + bigram[row(t)] for all s. row(t) = buckets at
// position 0, else (prev * mul_prev + ids[t] * mul_cur) mod buckets, prev = the sequence's previous token (the
// row before, or prev_tok[slot] for the first row of the step). bigram == nullptr: no such term. A step with one row
// per sequence (cu_q == nullptr) also stores the row's token as the slot's new previous token.
hipError_t launch_embed_hash(float* streams, int S, int W, const void* embed, const void* bigram, bool f32,
                             const int64_t* ids, RaggedRows r, int64_t* prev_tok, float scale, int64_t buckets,
                             int64_t mul_prev, int64_t mul_cur, hipStream_t s);
// prev_tok[slot(s)] = the last token of sequence s in this step (nothing to do when cu_q == nullptr, see above)
hipError_t launch_store_last_token(int64_t* prev_tok, const int64_t* ids, RaggedRows r, hipStream_t s);

struct StreamMixArgs {
  float* streams;       // [T, S, W] fp32, updated in place
  int T, S, W;
  // sublayer output y = a1 * y1 (+ a2 * y2): [T, W] rows with strides ys1 / ys2; y1 == nullptr: no update
  const void* y1;
  const void* y2;
  int64_t ys1, ys2;
  bool y_f32;
  float a1, a2;
  const float* mix;     // [S, S] (from, to); with outw: x_t <- sum_s mix[s, t] x_s + outw[t] * y
  const float* outw;    // [S]
  // next sublayer's input: h = rmsnorm(sum_t inw[t] x_t) * gain[0]; inw == nullptr: plain sum; h == nullptr: none
  const float* inw;
  const float* gain;
  float eps;
  void* h;
  bool h_f32;
};
hipError_t launch_stream_mix_norm(const StreamMixArgs& a, hipStream_t s);

// out[t] = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, powers elementwise, N(v) = v / sqrt(mean(v^2) + eps) over the row
hipError_t launch_poly_norm_act(void* out, const void* z, int64_t zstride, bool f32, const float* coef, float eps,
                                int rows, int n, hipStream_t s);

struct DeltaShape {
  int heads, kv_heads, dim, vdim, taps;
  __host__ __device__ int channels() const { return 2 * kv_heads * dim + heads * vdim; }
};
// Per row: the short causal convolution (+ SiLU) of the C = [q | k | v] channels of x, with the taps - 1 inputs
// before the step taken from conv_state [slots, taps - 1, C] (fp32, the most recent last); q and k heads made
// unit vectors (q also times dim^-1/2); beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias)).
// Writes qkv32 [T, C] and bg [T, 2 * heads] = [beta | g], both fp32. A step with one row per sequence
// (cu_q == nullptr) also moves the row's input into conv_state. conv_w is [C, taps]; conv_wt, optional, the same
// weights tap-major ([taps, C]), which lets prompt-sized bf16 steps load them 16 bytes at a time.
hipError_t launch_delta_prep(float* qkv32, float* bg, const void* x, const void* b, const void* a, int64_t xstride,
                             bool f32, const float* conv_w, const float* conv_wt, float* conv_state,
                             const float* A_log, const float* dt_bias, DeltaShape sh, RaggedRows r, hipStream_t s);
// conv_state[slot(s)] = the last taps - 1 inputs of sequence s after this step (nothing to do when cu_q == nullptr)
hipError_t launch_conv_state_update(float* conv_state, const void* x, int64_t xstride, bool f32, DeltaShape sh,
                                    RaggedRows r, hipStream_t s);
// Per (sequence, head), token by token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with
// S [dim, vdim] fp32 kept in state [slots, heads, dim, vdim]. out[t, h, :] = o / rms(o) * norm_w * silu(gate[t, h, :]).
hipError_t launch_gated_delta(void* out, const float* qkv32, const float* bg, const void* gate, int64_t gstride,
                              bool f32, const float* norm_w, float eps, float* state, DeltaShape sh, RaggedRows r,
                              hipStream_t s);

struct QkvPrepArgs {
  const void* q;          // [T, H * dim], [T, G * dim], [T, G * vdim]: slices of one projection, row stride xstride
  const void* k;
  const void* v;          // nullptr: the values are the keys as projected, before any norm or rotation (vdim == dim)
  int64_t xstride;
  bool f32;
  int T, heads, kv_heads, dim, vdim;
  const float* q_norm;    // [H * dim], [G * dim]: RMS norm over the whole projection, or nullptr
  const float* k_norm;
  bool head_norm;         // q_norm and k_norm are [dim], shared by all heads: RMS norm of every head by itself
  bool norm_after_rot;    // with head_norm: the rotation comes first and the norm acts on the rotated heads
  float q_temp_coef;      // != 0: q, after its norm, times 1 + coef * ln(floor((p + 1) / q_temp_every) + 1) at position p
  int q_temp_every;
  int rot_dims;           // rotated dims per head (pairs i, i + rot_dims / 2), 0: none
  const float* inv_freq;  // [rot_dims / 2]
  bool v_unit;            // each value head divided by its root mean square
  const float* v_lambda;  // v <- (1 - l) v + l v_first with l = v_lambda[0], or nullptr
  const void* v_first;    // [T, G * vdim], row stride vfstride
  int64_t vfstride;
  float eps;
  const int64_t* positions;
  const int64_t* slots;   // cache slot per row, < 0: not written
  void* q_out;            // [T, H * dim]
  void* cache;            // blocks of block_size tokens, head-major: [G][block_size][K: dim | V: vdim]
  int block_size;
};
hipError_t launch_qkv_prep(const QkvPrepArgs& a, hipStream_t s);

struct SinkAttnArgs {
  void* out;              // [T, H * vdim]
  const void* q;          // [T, H * dim]
  const void* cache;      // [num_blocks][G][block_size][K: dim | V: vdim]
  const int* block_tables;
  int bt_stride;
  const int* cu_q;        // nullptr: one row per sequence
  const int* ctx_lens;    // [S] keys after this step
  const int64_t* positions;
  const float* sink;      // [H] or nullptr
  const float* bias;      // [bias_rows, H]: added to the scaled score of a key at distance n, row min(n, bias_rows - 1)
  int bias_rows;
  float softcap;          // > 0: the scaled score s becomes softcap * tanh(s / softcap), before bias and slope
  const float* slopes;    // [H] or nullptr: slopes[h] * n is taken off the score of a key at distance n
  int num_seqs, total_q, max_q, heads, kv_heads, dim, vdim, block_size;
  int window;             // keys j with 0 <= p - j < window (0: all j <= p)
  float scale;
  bool f32;
  int impl;               // 0: the decode-step kernel or matrix cores where they apply, else FMA; 1: FMA;
                          // 2: matrix cores or fail
  // split keys (matrix-core kernel only): nsplit > 1 workgroups per row tile take `chunk` keys each and write
  // unnormalised partial sums to ws_o [nsplit, T * H, vdim] and (running max in log2 units, sum) to
  // ws_ml [nsplit, T * H, 2]; a merge kernel then writes `out`
  float* ws_o;
  float* ws_ml;
  int nsplit, chunk;
};
hipError_t launch_sink_attn(const SinkAttnArgs& a, hipStream_t s);
bool sink_attn_uses_mfma(const SinkAttnArgs& a);
// whether launch_sink_attn would run the decode-step kernel (impl 0, one bf16 query token per sequence); it splits
// the keys in multiples of 128
bool sink_attn_uses_decode(const SinkAttnArgs& a);

}  // namespace die
