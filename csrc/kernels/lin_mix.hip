// Kernels for layer stacks with sandwich norms, depth-weighted averaging of layer results, learned position
// vectors, biased squared-ReLU feed-forwards, sigmoid output gates and decayed linear attention (gfx950). Storage of
// activations is bf16 or fp32 (a run-time flag), arithmetic is fp32; the residual planes, every norm, the decays and
// the recurrent state are fp32 in both modes.
//
//   embed_pos            token vector + learned position vector -> fp32 residual
//   post_pre_norm        resid += rms(y + bias) * w_post and the next sublayer's input rms(resid) * w_pre, one launch
//   depth_avg_norm       the layer's last post-norm, the weighted average over all layer results so far and the
//                        next layer's first norm (or the final norm), one launch
//   bias_relu2           relu(z + b)^2
//   tanh_cap             cap * tanh(z / cap) into fp32 (capped logits)
//   head_gate            per-head sigmoid gate fused with the head-major -> token-major move
//   norm_sigmoid_gate    rms(o) * w * sigmoid(g)
//   lightning_attn       S <- decay S + k v^T, o = S^T q: one workgroup per (sequence, head), the state in
//                        registers (a column per lane quad), prompt portions and decode rows alike
#include "common.h"
#include "lin_launchers.h"

namespace die {

namespace {

constexpr int NT = 256;

__device__ __forceinline__ float ldv(const void* p, int64_t i, bool f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void stv(void* p, int64_t i, bool f32, float v) {
  if (f32)
    reinterpret_cast<float*>(p)[i] = v;
  else
    reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}
__device__ __forceinline__ float rnd(float v, bool f32) { return f32 ? v : bf2f(f2bf(v)); }
__device__ __forceinline__ float siluf(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }

__device__ __forceinline__ bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// 4 consecutive values (element index i a multiple of 4, the base 16-byte aligned)
__device__ __forceinline__ float4 ld4(const void* p, int64_t i, bool f32) {
  if (f32) return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
  const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const bf16_t*>(p) + i);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                     __uint_as_float(w.y & 0xffff0000u));
}
__device__ __forceinline__ void st4(void* p, int64_t i, bool f32, float4 v) {
  if (f32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + i) = v;
  } else {
    uint2 w;
    w.x = pack2(v.x, v.y);
    w.y = pack2(v.z, v.w);
    *reinterpret_cast<uint2*>(reinterpret_cast<bf16_t*>(p) + i) = w;
  }
}
__device__ __forceinline__ float4 f4(const float* p, int64_t i) { return *reinterpret_cast<const float4*>(p + i); }
__device__ __forceinline__ float sq4(float4 v) { return v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w; }

// ------------------------------------------------------------------------------------------------ embedding
__global__ void __launch_bounds__(NT) embed_pos_kernel(float* out, const void* embed, const void* pos, bool f32,
                                                      const int64_t* ids, const int64_t* positions, int W) {
  const int64_t t = blockIdx.x;
  const int64_t e0 = ids[t] * W, p0 = positions[t] * W;
  if (W % 4 == 0 && al16(embed) && al16(pos) && al16(out)) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      const float4 a = ld4(embed, e0 + c, f32), b = ld4(pos, p0 + c, f32);
      *reinterpret_cast<float4*>(out + t * W + c) = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += NT) out[t * W + c] = ldv(embed, e0 + c, f32) + ldv(pos, p0 + c, f32);
}

// ------------------------------------------------------------------------------------- norms around sublayers
// The row is staged in LDS (fp32) between the passes, so global memory is read once and written once per tensor.
__global__ void __launch_bounds__(NT) post_pre_norm_kernel(PostPreNormArgs a) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int W = a.W;
  float* rr = a.resid + t * W;
  const int64_t y0 = t * a.ystride;
  const bool vec = W % 4 == 0 && a.ystride % 4 == 0 && al16(a.y) && al16(a.resid) &&
                   (a.ybias == nullptr || al16(a.ybias)) && al16(a.w_post) && (a.w_pre == nullptr || al16(a.w_pre)) &&
                   (a.h == nullptr || al16(a.h));
  float ss = 0.f;
  if (vec) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      float4 v = ld4(a.y, y0 + c, a.y_f32);
      if (a.ybias != nullptr) {
        const float4 b = ld4(a.ybias, c, a.y_f32);
        v = make_float4(v.x + b.x, v.y + b.y, v.z + b.z, v.w + b.w);
      }
      *reinterpret_cast<float4*>(row + c) = v;
      ss += sq4(v);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) {
      float v = ldv(a.y, y0 + c, a.y_f32);
      if (a.ybias != nullptr) v += ldv(a.ybias, c, a.y_f32);
      row[c] = v;
      ss += v * v;
    }
  }
  ss = block_sum<NT>(ss, red);
  const float rs = 1.0f / sqrtf(ss / (float)W + a.eps);
  float s2 = 0.f;
  if (vec) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      const float4 v = f4(row, c), g = f4(a.w_post, c), x = f4(rr, c);
      const float4 o = make_float4(x.x + v.x * rs * g.x, x.y + v.y * rs * g.y, x.z + v.z * rs * g.z, x.w + v.w * rs * g.w);
      *reinterpret_cast<float4*>(rr + c) = o;
      *reinterpret_cast<float4*>(row + c) = o;
      s2 += sq4(o);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) {
      const float o = rr[c] + row[c] * rs * a.w_post[c];
      rr[c] = o;
      row[c] = o;
      s2 += o * o;
    }
  }
  if (a.h == nullptr) return;
  s2 = block_sum<NT>(s2, red);
  const float r2 = 1.0f / sqrtf(s2 / (float)W + a.eps);
  if (vec) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      const float4 v = f4(row, c), g = f4(a.w_pre, c);
      st4(a.h, t * W + c, a.h_f32, make_float4(v.x * r2 * g.x, v.y * r2 * g.y, v.z * r2 * g.z, v.w * r2 * g.w));
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) stv(a.h, t * W + c, a.h_f32, row[c] * r2 * a.w_pre[c]);
  }
}

constexpr int MAX_DEPTH = 128;   // planes averaged by one launch (their weights sit in LDS)

__global__ void __launch_bounds__(NT) depth_avg_norm_kernel(DepthAvgArgs a) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  __shared__ float red[NT / 64];
  __shared__ float dws[MAX_DEPTH];
  const int64_t t = blockIdx.x;
  const int W = a.W, n = a.n;
  if (a.dw != nullptr)
    for (int j = threadIdx.x; j < n; j += NT) dws[j] = a.dw[j];
  float* last = a.planes + (int64_t)(n - 1) * a.plane_stride + t * W;
  float* dst = a.planes + (int64_t)n * a.plane_stride + t * W;
  const bool vec = W % 4 == 0 && a.plane_stride % 4 == 0 && al16(a.planes) &&
                   (a.y == nullptr || (a.ystride % 4 == 0 && al16(a.y) && al16(a.w_post) &&
                                       (a.ybias == nullptr || al16(a.ybias)))) &&
                   (a.h == nullptr || (al16(a.h) && al16(a.w_pre)));
  float rs = 0.f;
  if (a.y != nullptr) {
    const int64_t y0 = t * a.ystride;
    float ss = 0.f;
    if (vec) {
      for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
        float4 v = ld4(a.y, y0 + c, a.y_f32);
        if (a.ybias != nullptr) {
          const float4 b = ld4(a.ybias, c, a.y_f32);
          v = make_float4(v.x + b.x, v.y + b.y, v.z + b.z, v.w + b.w);
        }
        *reinterpret_cast<float4*>(row + c) = v;
        ss += sq4(v);
      }
    } else {
      for (int c = threadIdx.x; c < W; c += NT) {
        float v = ldv(a.y, y0 + c, a.y_f32);
        if (a.ybias != nullptr) v += ldv(a.ybias, c, a.y_f32);
        row[c] = v;
        ss += v * v;
      }
    }
    ss = block_sum<NT>(ss, red);
    rs = 1.0f / sqrtf(ss / (float)W + a.eps);
  } else {
    __syncthreads();   // dws
  }
  float s2 = 0.f;
  if (vec) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      float4 x = f4(last, c);
      if (a.y != nullptr) {
        const float4 v = f4(row, c), g = f4(a.w_post, c);
        x = make_float4(x.x + v.x * rs * g.x, x.y + v.y * rs * g.y, x.z + v.z * rs * g.z, x.w + v.w * rs * g.w);
        *reinterpret_cast<float4*>(last + c) = x;
      }
      if (a.dw != nullptr) {
        const float wl = dws[n - 1];
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int j = 0; j < n - 1; ++j) {
          const float4 p = f4(a.planes + (int64_t)j * a.plane_stride + t * W, c);
          const float wj = dws[j];
          acc.x += wj * p.x;
          acc.y += wj * p.y;
          acc.z += wj * p.z;
          acc.w += wj * p.w;
        }
        x = make_float4(acc.x + wl * x.x, acc.y + wl * x.y, acc.z + wl * x.z, acc.w + wl * x.w);
      }
      *reinterpret_cast<float4*>(dst + c) = x;
      *reinterpret_cast<float4*>(row + c) = x;
      s2 += sq4(x);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) {
      float x = last[c];
      if (a.y != nullptr) {
        x += row[c] * rs * a.w_post[c];
        last[c] = x;
      }
      if (a.dw != nullptr) {
        float acc = 0.f;
        for (int j = 0; j < n - 1; ++j) acc += dws[j] * a.planes[(int64_t)j * a.plane_stride + t * W + c];
        x = acc + dws[n - 1] * x;
      }
      dst[c] = x;
      row[c] = x;
      s2 += x * x;
    }
  }
  if (a.h == nullptr) return;
  s2 = block_sum<NT>(s2, red);
  const float r2 = 1.0f / sqrtf(s2 / (float)W + a.eps);
  if (vec) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * NT) {
      const float4 v = f4(row, c), g = f4(a.w_pre, c);
      st4(a.h, t * W + c, a.h_f32, make_float4(v.x * r2 * g.x, v.y * r2 * g.y, v.z * r2 * g.z, v.w * r2 * g.w));
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) stv(a.h, t * W + c, a.h_f32, row[c] * r2 * a.w_pre[c]);
  }
}

// ------------------------------------------------------------------------------------------- elementwise
// grid (column tiles, rows): no division per element; bf16 rows of a multiple of 8 columns move 16 bytes per access
__global__ void __launch_bounds__(NT) bias_relu2_kernel(void* out, const void* z, const void* b, bool f32, int n) {
  const int64_t r0 = (int64_t)blockIdx.y * n;
  if (!f32 && n % 8 == 0 && al16(out) && al16(z) && al16(b)) {
    const int c = 8 * (blockIdx.x * NT + threadIdx.x);
    if (c >= n) return;
    float v[8], bb[8];
    unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(z) + r0 + c), v);
    unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(b) + c), bb);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float x = fmaxf(rnd(v[e] + bb[e], false), 0.f);
      v[e] = x * x;
    }
    *reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(out) + r0 + c) = pack8(v);
    return;
  }
  for (int e = 0; e < 8; ++e) {
    const int c = 8 * blockIdx.x * NT + e * NT + threadIdx.x;
    if (c < n) {
      const float x = fmaxf(rnd(ldv(z, r0 + c, f32) + ldv(b, c, f32), f32), 0.f);
      stv(out, r0 + c, f32, x * x);
    }
  }
}

__global__ void __launch_bounds__(NT) tanh_cap_kernel(float* out, const void* z, bool f32, float cap, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * NT;
  const float inv = 1.0f / cap;
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < total; i += stride)
    out[i] = cap * tanhf(ldv(z, i, f32) * inv);
}

__global__ void __launch_bounds__(NT) head_gate_kernel(void* out, const void* o, const void* g, int64_t gstride,
                                                      bool f32, int T, int H, int v) {
  extern __shared__ float gates[];   // [H]: the token's gates, one sigmoid per head
  const int64_t t = blockIdx.x;
  for (int h = threadIdx.x; h < H; h += NT) gates[h] = sigmoidf(ldv(g, t * gstride + h, f32));
  __syncthreads();
  if (v % 4 == 0 && al16(out) && al16(o)) {
    for (int e = 4 * threadIdx.x; e < H * v; e += 4 * NT) {
      const int h = e / v, c = e - h * v;
      const float gate = gates[h];
      const float4 x = ld4(o, ((int64_t)h * T + t) * v + c, f32);
      st4(out, t * H * v + e, f32, make_float4(x.x * gate, x.y * gate, x.z * gate, x.w * gate));
    }
    return;
  }
  for (int e = threadIdx.x; e < H * v; e += NT) {
    const int h = e / v, c = e % v;
    stv(out, t * H * v + e, f32, ldv(o, ((int64_t)h * T + t) * v + c, f32) * gates[h]);
  }
}

__global__ void __launch_bounds__(NT) norm_sigmoid_gate_kernel(void* out, const float* o, const void* g,
                                                              int64_t gstride, bool f32, const float* w, float eps,
                                                              int n) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const bool vec = n % 4 == 0 && gstride % 4 == 0 && al16(out) && al16(o) && al16(g) && al16(w);
  float ss = 0.f;
  if (vec) {
    for (int c = 4 * threadIdx.x; c < n; c += 4 * NT) ss += sq4(f4(o, t * n + c));
  } else {
    for (int c = threadIdx.x; c < n; c += NT) {
      const float x = o[t * n + c];
      ss += x * x;
    }
  }
  ss = block_sum<NT>(ss, red);
  const float rs = 1.0f / sqrtf(ss / (float)n + eps);
  if (vec) {
    for (int c = 4 * threadIdx.x; c < n; c += 4 * NT) {
      const float4 x = f4(o, t * n + c), ww = f4(w, c), gg = ld4(g, t * gstride + c, f32);
      st4(out, t * n + c, f32,
          make_float4(x.x * rs * ww.x * sigmoidf(gg.x), x.y * rs * ww.y * sigmoidf(gg.y),
                      x.z * rs * ww.z * sigmoidf(gg.z), x.w * rs * ww.w * sigmoidf(gg.w)));
    }
    return;
  }
  for (int c = threadIdx.x; c < n; c += NT)
    stv(out, t * n + c, f32, o[t * n + c] * rs * w[c] * sigmoidf(ldv(g, t * gstride + c, f32)));
}

// ------------------------------------------------------------------------------------------ linear attention
constexpr int TB = 16;  // tokens staged per trip

// One workgroup per (sequence, head). The state S [dim, vdim] lives in registers for the whole step: column j is
// split over the 4 lanes of a quad, lane `part` holding rows [part * DP, (part + 1) * DP). A token costs each lane
// 2 * DP multiply-adds and one quad reduction; q and k come from LDS as float4 broadcasts.
template <int DP>
__global__ void __launch_bounds__(1024) lightning_attn_kernel(LightningArgs a, RaggedRows r) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int DPAD = 4 * DP;
  const int d = a.dim, dv = a.vdim, H = a.heads;
  float* qs = sm;                  // [TB][DPAD], zero beyond dim
  float* ks = qs + TB * DPAD;      // [TB][DPAD]
  float* vs = ks + TB * DPAD;      // [TB][dv]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, nthr = blockDim.x;
  const int j = tid >> 2, part = tid & 3;
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  const bool fresh = r.positions[q0] <= 0;
  const float decay = a.decay[h];
  float* st = a.state + ((int64_t)r.state_slots[s] * H + h) * d * dv;
  float S[DP];
#pragma unroll
  for (int i = 0; i < DP; ++i) {
    const int row = part * DP + i;
    S[i] = (!fresh && row < d && j < dv) ? st[(int64_t)row * dv + j] : 0.f;
  }
  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    __syncthreads();
    for (int e = tid; e < nb * DPAD; e += nthr) {
      const int tt = e / DPAD, c = e % DPAD;
      const int64_t base = (int64_t)(q0 + t0 + tt) * a.xstride + h * d + c;
      qs[e] = c < d ? rnd(siluf(ldv(a.x, base + a.qoff, a.f32)), a.f32) : 0.f;
      ks[e] = c < d ? rnd(siluf(ldv(a.x, base + a.koff, a.f32)), a.f32) : 0.f;
    }
    for (int e = tid; e < nb * dv; e += nthr) {
      const int tt = e / dv, c = e % dv;
      vs[e] = rnd(siluf(ldv(a.x, (int64_t)(q0 + t0 + tt) * a.xstride + a.voff + h * dv + c, a.f32)), a.f32);
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float4* kt = reinterpret_cast<const float4*>(ks + tt * DPAD + part * DP);
      const float4* qt = reinterpret_cast<const float4*>(qs + tt * DPAD + part * DP);
      const float vj = j < dv ? vs[tt * dv + j] : 0.f;
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < DP / 4; ++i) {
        const float4 k4 = kt[i], q4 = qt[i];
        S[4 * i] = S[4 * i] * decay + k4.x * vj;
        S[4 * i + 1] = S[4 * i + 1] * decay + k4.y * vj;
        S[4 * i + 2] = S[4 * i + 2] * decay + k4.z * vj;
        S[4 * i + 3] = S[4 * i + 3] * decay + k4.w * vj;
        o0 += S[4 * i] * q4.x + S[4 * i + 2] * q4.z;
        o1 += S[4 * i + 1] * q4.y + S[4 * i + 3] * q4.w;
      }
      float o = o0 + o1;
      o += __shfl_xor(o, 1, 64);
      o += __shfl_xor(o, 2, 64);
      if (part == 0 && j < dv) a.out[((int64_t)(q0 + t0 + tt) * H + h) * dv + j] = o;
    }
  }
  if (j < dv) {
#pragma unroll
    for (int i = 0; i < DP; ++i) {
      const int row = part * DP + i;
      if (row < d) st[(int64_t)row * dv + j] = S[i];
    }
  }
}

template <int DP> hipError_t launch_lightning_dp(const LightningArgs& a, RaggedRows r, hipStream_t s) {
  const int threads = (4 * a.vdim + 63) / 64 * 64;
  const size_t smem = (size_t)(2 * TB * 4 * DP + TB * a.vdim) * sizeof(float);
  hipLaunchKernelGGL(lightning_attn_kernel<DP>, dim3(a.heads, r.num_seqs), dim3(threads), smem, s, a, r);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_embed_pos(float* out, const void* embed, const void* pos, bool f32, const int64_t* ids,
                            const int64_t* positions, int T, int W, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (W <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(embed_pos_kernel, dim3(T), dim3(NT), 0, s, out, embed, pos, f32, ids, positions, W);
  return hipGetLastError();
}

hipError_t launch_post_pre_norm(const PostPreNormArgs& a, hipStream_t s) {
  if (a.T == 0) return hipSuccess;
  if (a.W <= 0 || a.W > 16384 || (a.h != nullptr && a.w_pre == nullptr)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(post_pre_norm_kernel, dim3(a.T), dim3(NT), (size_t)a.W * sizeof(float), s, a);
  return hipGetLastError();
}

hipError_t launch_depth_avg_norm(const DepthAvgArgs& a, hipStream_t s) {
  if (a.T == 0) return hipSuccess;
  if (a.W <= 0 || a.W > 16384 || a.n < 1 || a.n > MAX_DEPTH || (a.h != nullptr && a.w_pre == nullptr) ||
      (a.y != nullptr && a.w_post == nullptr))
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(depth_avg_norm_kernel, dim3(a.T), dim3(NT), (size_t)a.W * sizeof(float), s, a);
  return hipGetLastError();
}

hipError_t launch_bias_relu2(void* out, const void* z, const void* b, bool f32, int rows, int n, hipStream_t s) {
  if (rows == 0) return hipSuccess;
  if (n <= 0) return hipErrorInvalidValue;
  // rows ride in grid.y (at most 65535 per launch)
  for (int r = 0; r < rows; r += 65535) {
    const int nr = rows - r < 65535 ? rows - r : 65535;
    const size_t off = (size_t)r * n * (f32 ? 4 : 2);
    hipLaunchKernelGGL(bias_relu2_kernel, dim3((unsigned)((n + 8 * NT - 1) / (8 * NT)), (unsigned)nr), dim3(NT), 0, s,
                       static_cast<char*>(out) + off, static_cast<const char*>(z) + off, b, f32, n);
  }
  return hipGetLastError();
}

hipError_t launch_tanh_cap(float* out, const void* z, bool f32, float cap, int64_t total, hipStream_t s) {
  if (total == 0) return hipSuccess;
  if (!(cap > 0.f)) return hipErrorInvalidValue;
  const int64_t blocks = (total + NT - 1) / NT;
  hipLaunchKernelGGL(tanh_cap_kernel, dim3((unsigned)(blocks < 8192 ? blocks : 8192)), dim3(NT), 0, s, out, z, f32,
                     cap, total);
  return hipGetLastError();
}

hipError_t launch_head_gate(void* out, const void* o, const void* g, int64_t gstride, bool f32, int T, int H, int v,
                            hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (H <= 0 || H > 8192 || v <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(head_gate_kernel, dim3(T), dim3(NT), (size_t)H * sizeof(float), s, out, o, g, gstride, f32, T, H,
                     v);
  return hipGetLastError();
}

hipError_t launch_norm_sigmoid_gate(void* out, const float* o, const void* g, int64_t gstride, bool f32,
                                    const float* w, float eps, int T, int n, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (n <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(norm_sigmoid_gate_kernel, dim3(T), dim3(NT), 0, s, out, o, g, gstride, f32, w, eps, n);
  return hipGetLastError();
}

hipError_t launch_lightning_attn(const LightningArgs& a, RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || r.total_rows == 0) return hipSuccess;
  if (a.heads < 1 || a.dim < 1 || a.dim > 128 || a.vdim < 1 || a.vdim > 256 || r.positions == nullptr ||
      r.state_slots == nullptr)
    return hipErrorInvalidValue;
  if (a.dim <= 16) return launch_lightning_dp<4>(a, r, s);
  if (a.dim <= 32) return launch_lightning_dp<8>(a, r, s);
  if (a.dim <= 64) return launch_lightning_dp<16>(a, r, s);
  return launch_lightning_dp<32>(a, r, s);
}

}  // namespace die
