// Host launchers of the dtype-generic kernels (bf16 or fp32 storage, fp32 arithmetic): sublayer-output
// norms into an fp32 residual stream, gated activations, sigmoid top-k routing with input-scaled experts,
// and latent (compressed-KV) attention with a sliding window and a softmax sink. Raw pointers + an explicit
// stream, no allocation and no synchronisation: every launcher is hipGraph-capturable. `f32` selects the
// storage type of the activation / cache / weight tensors (false: bf16).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace die {

// out[r] = x[r] / sqrt(mean(x[r]^2) + eps) * (w or 1 + w); in_f32 / out_f32 / w_f32 give each tensor's storage
hipError_t launch_rms_norm_ext(void* out, int64_t ostride, bool out_f32, const void* x, int64_t xstride, bool in_f32,
                               const void* w, bool w_f32, bool unit_offset, float eps, int rows, int n,
                               hipStream_t s);
// resid[r] (fp32) += mult * y[r] / sqrt(mean(y[r]^2) + eps) * (w or 1 + w); act[r] (optional, bf16) = resid[r]
hipError_t launch_post_norm_residual(float* resid, void* act, const void* y, int64_t ystride, bool y_f32,
                                     const void* w, bool w_f32, bool unit_offset, float eps, float mult, int rows,
                                     int n, hipStream_t s);
// out[r, :f] = act(gu[r, :f]) * f(gu[r, f:2f]).  kind 0: silu(g) * u.  kind 1: g' = min(g, limit),
// u' = clamp(u, -limit, limit), g' * sigmoid(alpha * g') * (u' + 1).  kind 2: gelu(g) * u, tanh form
hipError_t launch_gated_act(void* out, const void* gu, bool f32, int rows, int f, int kind, float limit, float alpha,
                            hipStream_t s);

// Router: z = x . Wr[e] in fp32, score = sigmoid(z), the K largest per token (lowest index on ties);
// w [T, K] fp32 = the chosen scores (not renormalised), ids [T, K] int32
hipError_t launch_route_sigmoid_topk(float* w, int* ids, const void* x, int64_t xstride, bool x_f32, const void* wr,
                                     bool wr_f32, int T, int H, int E, int K, hipStream_t s);
// the same selection from fp32 logits z [T, E] computed elsewhere
hipError_t launch_topk_sigmoid(float* w, int* ids, const float* z, int T, int E, int K, hipStream_t s);
// Router with softmax scores over E choices: z = x . Wr[e] in fp32, s = softmax(z); the K largest s + corr (corr
// optional; lowest index on ties) are chosen; w [T, K] = their s over the sum of the chosen s (+ 1e-20).
// gate != nullptr: Wr has one more row, gate[t] = sigmoid(x . Wr[E]).
hipError_t launch_route_softmax_topk(float* w, int* ids, float* gate, const void* x, int64_t xstride, bool x_f32,
                                     const void* wr, bool wr_f32, const float* corr, int T, int H, int E, int K,
                                     hipStream_t s);
// the same selection from fp32 logits z [T, zstride] computed elsewhere (the gate's logit at column E)
hipError_t launch_topk_softmax_corrected(float* w, int* ids, float* gate, const float* z, int zstride,
                                         const float* corr, int T, int E, int K, hipStream_t s);
// sum[t] = sum_k wk[t, k] * (ids[t, k] < E ? ys[pos[t * K + k]] : x[t]) + gate[t] * extra[t]  (pos == nullptr:
// t * K + k; extra, gate optional). out != nullptr: out[t] (fp32) = sum[t]. resid != nullptr:
// resid[t] += mult * rmsnorm(sum[t]) * (w or 1 + w), act[t] (optional, the activation type) = resid[t].
hipError_t launch_combine_weighted(float* out, float* resid, void* act, const void* ys, bool f32, const int* pos,
                                   const void* x, const float* wk, const int* ids, int E, const void* extra,
                                   const float* gate, int T, int K, int H, const void* w, bool w_f32, bool unit_offset,
                                   float eps, float mult, hipStream_t s);
// xs[j] = w[sorted[j]] * x[sorted[j] / K]  (sorted == nullptr: j itself; w == nullptr: a plain gather)
hipError_t launch_gather_scaled(void* xs, const void* x, bool f32, const int* sorted, const float* w, int n, int K,
                                int H, hipStream_t s);
// out[t] (fp32) = sum_k ys[pos[t * K + k]] (+ extra[t]);  pos == nullptr: t * K + k
hipError_t launch_combine_sum(float* out, const void* ys, bool f32, const int* pos, const void* extra, int T, int K,
                              int H, hipStream_t s);

struct LatentShape {
  int rank;      // latent (compressed KV) width, normalised
  int rot_dim;   // shared rotary key width, stored after the latent
  int rot_pairs; // rotated pairs (2i, 2i + 1), i < rot_pairs <= rot_dim / 2; the rest passes unchanged
  const float* inv_freq;  // [rot_pairs] fp32 (device): the angle of pair i at position p is p * inv_freq[i]
};
// cache row of token t (at slot_mapping[t] >= 0): [ rmsnorm(kv[t, :rank]) * w | rotate(kv[t, rank:]) ]
hipError_t launch_latent_kv_write(void* cache, const void* kv, int64_t kvstride, bool f32, const void* w, bool w_f32,
                                  const int64_t* positions, const int64_t* slots, int T, LatentShape sh, float eps,
                                  hipStream_t s);

// p [T, q_rank + rank + rot_dim] (row stride pstride): cq[t] = rmsnorm(p[t, :q_rank]) * wq and the cache row of
// token t from p[t, q_rank:], as launch_latent_kv_write — one launch for both
hipError_t launch_latent_qkv_prep(void* cq, const void* p, int64_t pstride, bool f32, int q_rank, const void* wq,
                                  const void* wkv, bool w_f32, void* cache, const int64_t* positions,
                                  const int64_t* slots, int T, LatentShape sh, float eps, hipStream_t s);
// resid[t] (fp32) += rmsnorm(sum_k ys[pos[t * K + k]] + extra[t]) * (w or 1 + w); act[t] (optional, bf16) = resid[t]
hipError_t launch_combine_post_norm(float* resid, void* act, const void* ys, bool f32, const int* pos,
                                    const void* extra, int T, int K, int H, const void* w, bool w_f32,
                                    bool unit_offset, float eps, hipStream_t s);

struct LatentAttnArgs {
  void* out;              // [H, T, rank] latent-space attention output
  const void* q_lat;      // [H, T, rank] queries projected into the latent space
  const void* q_rot;      // rotary part of the queries: row t, head h at q_rot + t * q_stride + h * q_hstride
  int64_t q_stride, q_hstride;
  const void* cache;      // [num_blocks, block_size, rank + rot_dim]
  const int* block_tables;
  int bt_stride;
  const int* cu_q;        // [S + 1] first row of each sequence (nullptr: one row per sequence)
  const int* ctx_lens;    // [S] keys after this step
  const int64_t* positions;
  const float* sink;      // [H] or nullptr
  int num_seqs, total_q, max_q, heads, block_size;
  int window;             // keys j with 0 <= p - j < window (0: all j <= p)
  float scale;
  LatentShape sh;
  bool f32;
  // split keys (matrix-core kernel only): nsplit > 1 workgroups per row tile take `chunk` keys each and write
  // unnormalised partial sums to ws_o [nsplit, H * T, rank] and (running max in log2 units, sum) to
  // ws_ml [nsplit, H * T, 2]; a merge kernel then writes `out`
  float* ws_o;
  float* ws_ml;
  int nsplit, chunk;
  int impl;               // 0: matrix cores where they apply, else the FMA form; 1: FMA form; 2: matrix cores or fail;
                          // 3: as 2, but never the register-query variant (A/B)
};
hipError_t launch_latent_attn(const LatentAttnArgs& a, hipStream_t s);
// whether launch_latent_attn would run the matrix-core kernel for these arguments (the split workspace is only
// used by it)
bool latent_attn_uses_mfma(const LatentAttnArgs& a);

}  // namespace die
