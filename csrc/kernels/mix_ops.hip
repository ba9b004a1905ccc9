// Dtype-generic elementwise / normalisation / routing kernels (gfx950). Storage is bf16 or fp32, selected per
// tensor at run time; every value is widened to fp32 on load and all arithmetic (sums of squares, norms,
// sigmoids, router dot products, the residual sum) is fp32. One workgroup per row; rows of any width.
//
//   rms_norm_ext          y = x / sqrt(mean(x^2) + eps) * (w | 1 + w)
//   post_norm_residual    resid(fp32) += rmsnorm(y) * (w | 1 + w); optional bf16 copy of the new residual
//   gated_act             silu(g) * u, or the clamped variant g' * sigmoid(alpha g') * (u' + 1)
//   route_sigmoid_topk    router logits (fp32), sigmoid scores, top-K without renormalisation
//   gather_scaled         expert input rows scaled by their routing weight
//   combine_sum           per-token sum of its experts' outputs (+ a shared expert), fp32
//   latent_kv_write       compressed-KV cache row: normalised latent | rotated shared key part
#include "common.h"
#include "mix_launchers.h"

namespace die {

namespace {

__device__ __forceinline__ float ldv(const void* p, int64_t i, bool f32) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void stv(void* p, int64_t i, bool f32, float v) {
  if (f32)
    reinterpret_cast<float*>(p)[i] = v;
  else
    reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

constexpr int NT = 256;

__device__ __forceinline__ float row_rs(const void* x, int64_t base, bool f32, int n, float eps, float* red) {
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += NT) {
    const float v = ldv(x, base + c, f32);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  return 1.0f / sqrtf(ss / (float)n + eps);
}

__global__ void __launch_bounds__(NT) rms_norm_ext_kernel(void* out, int64_t ostride, bool out_f32, const void* x,
                                                         int64_t xstride, bool in_f32, const void* w, bool w_f32,
                                                         bool unit, float eps, int n) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  const float rs = row_rs(x, r * xstride, in_f32, n, eps, red);
  for (int c = threadIdx.x; c < n; c += NT) {
    float g = w ? ldv(w, c, w_f32) : 1.0f;
    if (unit) g += 1.0f;
    stv(out, r * ostride + c, out_f32, ldv(x, r * xstride + c, in_f32) * rs * g);
  }
}

__device__ __forceinline__ bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

__global__ void __launch_bounds__(NT) post_norm_residual_kernel(float* resid, void* act, const void* y,
                                                               int64_t ystride, bool y_f32, const void* w, bool w_f32,
                                                               bool unit, float eps, float mult, int n) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  // bf16 rows of a multiple of 8 columns: 16-byte loads and stores, 8 columns per thread and trip
  if (!y_f32 && !w_f32 && n % 8 == 0 && ystride % 8 == 0 && aligned16(y) && aligned16(w) && aligned16(resid) &&
      (act == nullptr || aligned16(act))) {
    const uint4* yr = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(y) + r * ystride);
    float ss = 0.f;
    for (int c = threadIdx.x; c < n / 8; c += NT) {
      float f[8];
      unpack8(yr[c], f);
#pragma unroll
      for (int q = 0; q < 8; ++q) ss += f[q] * f[q];
    }
    ss = block_sum<NT>(ss, red);
    const float rs = mult / sqrtf(ss / (float)n + eps);
    float4* rr = reinterpret_cast<float4*>(resid + r * n);
    for (int c = threadIdx.x; c < n / 8; c += NT) {
      float f[8], g[8];
      unpack8(yr[c], f);
      unpack8(reinterpret_cast<const uint4*>(w)[c], g);
      float4 a0 = rr[2 * c], a1 = rr[2 * c + 1];
      float o[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] += f[q] * rs * (unit ? g[q] + 1.0f : g[q]);
      rr[2 * c] = make_float4(o[0], o[1], o[2], o[3]);
      rr[2 * c + 1] = make_float4(o[4], o[5], o[6], o[7]);
      if (act) reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(act) + r * n)[c] = pack8(o);
    }
    return;
  }
  const float rs = mult * row_rs(y, r * ystride, y_f32, n, eps, red);
  for (int c = threadIdx.x; c < n; c += NT) {
    float g = w ? ldv(w, c, w_f32) : 1.0f;
    if (unit) g += 1.0f;
    const float v = resid[r * n + c] + ldv(y, r * ystride + c, y_f32) * rs * g;
    resid[r * n + c] = v;
    if (act) reinterpret_cast<bf16_t*>(act)[r * n + c] = f2bf(v);
  }
}

__device__ __forceinline__ float gate1(float g, float u, int kind, float limit, float alpha) {
  if (kind == 0) return g / (1.0f + expf(-g)) * u;
  if (kind == 2) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

__global__ void __launch_bounds__(NT) gated_act_kernel(void* out, const void* gu, bool f32, int f, int kind,
                                                      float limit, float alpha) {
  const int64_t r = blockIdx.x;
  if (!f32 && f % 8 == 0 && aligned16(gu) && aligned16(out)) {
    const uint4* gp = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(gu) + r * 2 * f);
    const uint4* up = gp + f / 8;
    uint4* op = reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(out) + r * f);
    for (int c = threadIdx.x; c < f / 8; c += NT) {
      float g[8], u[8], o[8];
      unpack8(gp[c], g);
      unpack8(up[c], u);
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] = gate1(g[q], u[q], kind, limit, alpha);
      op[c] = pack8(o);
    }
    return;
  }
  for (int c = threadIdx.x; c < f; c += NT)
    stv(out, r * f + c, f32, gate1(ldv(gu, r * 2 * f + c, f32), ldv(gu, r * 2 * f + f + c, f32), kind, limit, alpha));
}

constexpr int ROUTE_E_MAX = 256;

// One workgroup per token: wave v computes the logits of experts v, v + 4, ...; thread 0 selects.
__global__ void __launch_bounds__(NT) route_sigmoid_topk_kernel(float* w_out, int* id_out, const void* x,
                                                               int64_t xstride, bool x_f32, const void* wr,
                                                               bool wr_f32, int H, int E, int K) {
  __shared__ float z[ROUTE_E_MAX];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // 16-byte loads where both rows allow them (bf16 x and router: 8 elements per lane and trip, independent trips)
  const bool vec = !x_f32 && !wr_f32 && H % 8 == 0 && xstride % 8 == 0 &&
                   (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(wr) & 15) == 0;
  for (int e = wave; e < E; e += NT / 64) {
    float a = 0.f;
    if (vec) {
      const uint4* xr = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(x) + (int64_t)t * xstride);
      const uint4* wp = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(wr) + (int64_t)e * H);
      for (int c = lane; c < H / 8; c += 64) {
        float xf[8], wf[8];
        unpack8(xr[c], xf);
        unpack8(wp[c], wf);
#pragma unroll
        for (int q = 0; q < 8; ++q) a += xf[q] * wf[q];
      }
    } else {
      for (int c = lane; c < H; c += 64)
        a += ldv(x, (int64_t)t * xstride + c, x_f32) * ldv(wr, (int64_t)e * H + c, wr_f32);
    }
    a = wave_sum(a);
    if (lane == 0) z[e] = a;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  for (int k = 0; k < K; ++k) {
    int bi = -1;
    float bv = 0.f;
    for (int e = 0; e < E; ++e) {
      const float v = z[e];
      if (v != v || v == -INFINITY) continue;  // taken (marked below) or unusable
      if (bi < 0 || v > bv) {
        bv = v;
        bi = e;
      }
    }
    if (bi < 0) bi = 0;
    w_out[(int64_t)t * K + k] = 1.0f / (1.0f + expf(-bv));
    id_out[(int64_t)t * K + k] = bi;
    z[bi] = -INFINITY;
  }
}

// Selection alone, from logits already computed (a library fp32 GEMM for prompt-sized steps): one thread per token.
__global__ void __launch_bounds__(NT) topk_sigmoid_kernel(float* w_out, int* id_out, const float* z, int T, int E,
                                                         int K) {
  const int t = blockIdx.x * NT + threadIdx.x;
  if (t >= T) return;
  const float* zr = z + (int64_t)t * E;
  uint64_t taken[ROUTE_E_MAX / 64] = {0, 0, 0, 0};
  for (int k = 0; k < K; ++k) {
    int bi = -1;
    float bv = 0.f;
    for (int e = 0; e < E; ++e) {
      const float v = zr[e];
      if (v != v || ((taken[e >> 6] >> (e & 63)) & 1ull)) continue;
      if (bi < 0 || v > bv) {
        bv = v;
        bi = e;
      }
    }
    if (bi < 0) bi = 0;
    taken[bi >> 6] |= 1ull << (bi & 63);
    w_out[(int64_t)t * K + k] = 1.0f / (1.0f + expf(-bv));
    id_out[(int64_t)t * K + k] = bi;
  }
}

__global__ void __launch_bounds__(NT) gather_scaled_kernel(void* xs, const void* x, bool f32, const int* sorted,
                                                          const float* w, int K, int H) {
  const int64_t j = blockIdx.x;
  const int flat = sorted ? sorted[j] : (int)j;
  const int64_t t = flat / K;
  const float wk = w ? w[flat] : 1.0f;
  if (!f32 && H % 8 == 0 && aligned16(x) && aligned16(xs)) {
    const uint4* xp = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(x) + t * H);
    uint4* op = reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(xs) + j * H);
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float v[8];
      unpack8(xp[c], v);
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] *= wk;
      op[c] = pack8(v);
    }
    return;
  }
  for (int c = threadIdx.x; c < H; c += NT) stv(xs, j * H + c, f32, wk * ldv(x, t * H + c, f32));
}

__global__ void __launch_bounds__(NT) combine_sum_kernel(float* out, const void* ys, bool f32, const int* pos,
                                                        const void* extra, int K, int H) {
  const int64_t t = blockIdx.x;
  if (!f32 && H % 8 == 0 && aligned16(ys) && aligned16(out) && (extra == nullptr || aligned16(extra))) {
    const bf16_t* yb = reinterpret_cast<const bf16_t*>(ys);
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (extra) unpack8(reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(extra) + t * H)[c], a);
      for (int k = 0; k < K; ++k) {
        const int64_t j = pos ? pos[t * K + k] : t * K + k;
        float v[8];
        unpack8(reinterpret_cast<const uint4*>(yb + j * H)[c], v);
#pragma unroll
        for (int q = 0; q < 8; ++q) a[q] += v[q];
      }
      float4* op = reinterpret_cast<float4*>(out + t * H);
      op[2 * c] = make_float4(a[0], a[1], a[2], a[3]);
      op[2 * c + 1] = make_float4(a[4], a[5], a[6], a[7]);
    }
    return;
  }
  for (int c = threadIdx.x; c < H; c += NT) {
    float a = extra ? ldv(extra, t * H + c, f32) : 0.f;
    for (int k = 0; k < K; ++k) {
      const int64_t j = pos ? pos[t * K + k] : t * K + k;
      a += ldv(ys, j * H + c, f32);
    }
    out[t * H + c] = a;
  }
}

// Softmax-scored selection of one token from its logits z[0 .. E): the K largest softmax(z) + corr (lowest index on
// ties); weights = the chosen scores without corr, over their sum + 1e-20. `sc` [E] is scratch (LDS or registers'
// spill), left holding the scores.
__device__ __forceinline__ void softmax_select(const float* z, float* sc, const float* corr, int E, int K, float* w_out,
                                               int* id_out) {
  float mx = -INFINITY;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, z[e]);
  float den = 0.f;
  for (int e = 0; e < E; ++e) {
    sc[e] = expf(z[e] - mx);
    den += sc[e];
  }
  const float inv = 1.0f / den;
  for (int e = 0; e < E; ++e) sc[e] *= inv;
  uint64_t taken[ROUTE_E_MAX / 64] = {0, 0, 0, 0};
  float sum = 0.f;
  for (int k = 0; k < K; ++k) {
    int bi = -1;
    float bv = 0.f;
    for (int e = 0; e < E; ++e) {
      const float v = sc[e] + (corr ? corr[e] : 0.f);
      if (v != v || ((taken[e >> 6] >> (e & 63)) & 1ull)) continue;
      if (bi < 0 || v > bv) {
        bv = v;
        bi = e;
      }
    }
    if (bi < 0) bi = 0;
    taken[bi >> 6] |= 1ull << (bi & 63);
    w_out[k] = sc[bi];
    id_out[k] = bi;
    sum += sc[bi];
  }
  const float rn = 1.0f / (sum + 1e-20f);
  for (int k = 0; k < K; ++k) w_out[k] *= rn;
}

// One workgroup per token: wave v computes the logits of rows v, v + 4, ... of the router (E choices, then an
// optional gate row); thread 0 selects.
__global__ void __launch_bounds__(NT) route_softmax_topk_kernel(float* w_out, int* id_out, float* gate_out,
                                                               const void* x, int64_t xstride, bool x_f32,
                                                               const void* wr, bool wr_f32, const float* corr, int H,
                                                               int E, int K) {
  __shared__ float z[ROUTE_E_MAX + 1];
  __shared__ float sc[ROUTE_E_MAX];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rows = E + (gate_out ? 1 : 0);
  const bool vec = !x_f32 && !wr_f32 && H % 8 == 0 && xstride % 8 == 0 &&
                   (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(wr) & 15) == 0;
  for (int e = wave; e < rows; e += NT / 64) {
    float a = 0.f;
    if (vec) {
      const uint4* xr = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(x) + (int64_t)t * xstride);
      const uint4* wp = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(wr) + (int64_t)e * H);
      for (int c = lane; c < H / 8; c += 64) {
        float xf[8], wf[8];
        unpack8(xr[c], xf);
        unpack8(wp[c], wf);
#pragma unroll
        for (int q = 0; q < 8; ++q) a += xf[q] * wf[q];
      }
    } else {
      for (int c = lane; c < H; c += 64)
        a += ldv(x, (int64_t)t * xstride + c, x_f32) * ldv(wr, (int64_t)e * H + c, wr_f32);
    }
    a = wave_sum(a);
    if (lane == 0) z[e] = a;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  softmax_select(z, sc, corr, E, K, w_out + (int64_t)t * K, id_out + (int64_t)t * K);
  if (gate_out) gate_out[t] = 1.0f / (1.0f + expf(-z[E]));
}

// Selection alone, from logits already computed (a library fp32 GEMM for prompt-sized steps): one thread per token,
// its scores in a slice of LDS.
constexpr int SEL_NT = 64;
__global__ void __launch_bounds__(SEL_NT) topk_softmax_corrected_kernel(float* w_out, int* id_out, float* gate_out,
                                                                       const float* z, int zstride, const float* corr,
                                                                       int T, int E, int K) {
  extern __shared__ float scs[];   // [SEL_NT][E]
  const int t = blockIdx.x * SEL_NT + threadIdx.x;
  if (t >= T) return;
  const float* zr = z + (int64_t)t * zstride;
  softmax_select(zr, scs + threadIdx.x * E, corr, E, K, w_out + (int64_t)t * K, id_out + (int64_t)t * K);
  if (gate_out) gate_out[t] = 1.0f / (1.0f + expf(-zr[E]));
}

// The weighted sum of a token's experts: sum_k wk[t, k] * (ids[t, k] < E ? ys[pos[t, k]] : x[t]) + gate[t] * extra[t]
// (an id >= E names an identity expert, whose output is the token's input). out != nullptr: the sum as fp32.
// resid != nullptr: resid[t] += mult * rmsnorm(sum) * (w | 1 + w) and act[t] (optional, the activation type) =
// resid[t]; the sum is staged in LDS between its statistics and the update.
__global__ void __launch_bounds__(NT) combine_weighted_kernel(float* out, float* resid, void* act, const void* ys,
                                                             bool f32, const int* pos, const void* x, const float* wk,
                                                             const int* ids, int E, const void* extra,
                                                             const float* gate, int K, int H, const void* w, bool w_f32,
                                                             bool unit, float eps, float mult) {
  extern __shared__ __attribute__((aligned(16))) float acc[];   // [H]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const float gt = extra ? (gate ? gate[t] : 1.0f) : 0.f;
  float ss = 0.f;
  const bool vec = !f32 && H % 8 == 0 && aligned16(ys) && aligned16(x) && (extra == nullptr || aligned16(extra));
  if (vec) {
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (extra) {
        unpack8(reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(extra) + t * H)[c], a);
#pragma unroll
        for (int q = 0; q < 8; ++q) a[q] *= gt;
      }
      for (int k = 0; k < K; ++k) {
        const float wt = wk[t * K + k];
        const bool ident = ids[t * K + k] >= E;
        const int64_t j = pos ? pos[t * K + k] : t * K + k;
        const bf16_t* src = ident ? reinterpret_cast<const bf16_t*>(x) + t * H : reinterpret_cast<const bf16_t*>(ys) + j * H;
        float v[8];
        unpack8(reinterpret_cast<const uint4*>(src)[c], v);
#pragma unroll
        for (int q = 0; q < 8; ++q) a[q] += wt * v[q];
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) ss += a[q] * a[q];
      *reinterpret_cast<float4*>(acc + 8 * c) = make_float4(a[0], a[1], a[2], a[3]);
      *reinterpret_cast<float4*>(acc + 8 * c + 4) = make_float4(a[4], a[5], a[6], a[7]);
    }
  } else {
    for (int c = threadIdx.x; c < H; c += NT) {
      float a = extra ? gt * ldv(extra, t * H + c, f32) : 0.f;
      for (int k = 0; k < K; ++k) {
        const bool ident = ids[t * K + k] >= E;
        const int64_t j = pos ? pos[t * K + k] : t * K + k;
        a += wk[t * K + k] * (ident ? ldv(x, t * H + c, f32) : ldv(ys, j * H + c, f32));
      }
      acc[c] = a;
      ss += a * a;
    }
  }
  if (out != nullptr) {
    __syncthreads();
    for (int c = threadIdx.x; c < H; c += NT) out[t * H + c] = acc[c];
  }
  if (resid == nullptr) return;
  ss = block_sum<NT>(ss, red);
  const float rs = mult / sqrtf(ss / (float)H + eps);
  if (vec && !w_f32 && aligned16(w) && aligned16(resid) && (act == nullptr || aligned16(act))) {
    float4* rr = reinterpret_cast<float4*>(resid + t * H);
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float g[8];
      unpack8(reinterpret_cast<const uint4*>(w)[c], g);
      const float4 u0 = *reinterpret_cast<const float4*>(acc + 8 * c), u1 = *reinterpret_cast<const float4*>(acc + 8 * c + 4);
      const float u[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
      const float4 r0 = rr[2 * c], r1 = rr[2 * c + 1];
      float o[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] += u[q] * rs * (unit ? g[q] + 1.0f : g[q]);
      rr[2 * c] = make_float4(o[0], o[1], o[2], o[3]);
      rr[2 * c + 1] = make_float4(o[4], o[5], o[6], o[7]);
      if (act) reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(act) + t * H)[c] = pack8(o);
    }
    return;
  }
  for (int c = threadIdx.x; c < H; c += NT) {
    float g = ldv(w, c, w_f32);
    if (unit) g += 1.0f;
    const float v = resid[t * H + c] + acc[c] * rs * g;
    resid[t * H + c] = v;
    if (act) stv(act, t * H + c, f32, v);
  }
}

__device__ __forceinline__ void kv_write_row(void* cache, const void* kv, int64_t kvstride, bool f32, const void* w,
                                             bool w_f32, const int64_t* positions, const int64_t* slots,
                                             const LatentShape& sh, float eps, int64_t t, float* red) {
  const int64_t slot = slots[t];
  if (slot < 0) return;  // uniform per workgroup
  const int64_t src = t * kvstride, dst = slot * (int64_t)(sh.rank + sh.rot_dim);
  const float rs = row_rs(kv, src, f32, sh.rank, eps, red);
  for (int c = threadIdx.x; c < sh.rank; c += NT)
    stv(cache, dst + c, f32, ldv(kv, src + c, f32) * rs * (w ? ldv(w, c, w_f32) : 1.0f));
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < sh.rot_dim / 2 + (sh.rot_dim & 1); i += NT) {
    const int c0 = 2 * i;
    const float u = ldv(kv, src + sh.rank + c0, f32);
    if (c0 + 1 >= sh.rot_dim) {
      stv(cache, dst + sh.rank + c0, f32, u);
      continue;
    }
    const float v = ldv(kv, src + sh.rank + c0 + 1, f32);
    if (i < sh.rot_pairs) {
      float sn, cs;
      sincosf(p * sh.inv_freq[i], &sn, &cs);
      stv(cache, dst + sh.rank + c0, f32, u * cs - v * sn);
      stv(cache, dst + sh.rank + c0 + 1, f32, v * cs + u * sn);
    } else {
      stv(cache, dst + sh.rank + c0, f32, u);
      stv(cache, dst + sh.rank + c0 + 1, f32, v);
    }
  }
}

__global__ void __launch_bounds__(NT) latent_kv_write_kernel(void* cache, const void* kv, int64_t kvstride, bool f32,
                                                            const void* w, bool w_f32, const int64_t* positions,
                                                            const int64_t* slots, LatentShape sh, float eps) {
  __shared__ float red[NT / 64];
  kv_write_row(cache, kv, kvstride, f32, w, w_f32, positions, slots, sh, eps, blockIdx.x, red);
}

// Both consumers of the fused down-projection p = [query latent | kv latent | shared rotary key] in one launch:
// blockIdx.y == 0 norms the query latent (plain weight) into cq, blockIdx.y == 1 writes the cache row.
__global__ void __launch_bounds__(NT) latent_qkv_prep_kernel(void* cq, const void* p, int64_t pstride, bool f32,
                                                            int q_rank, const void* wq, const void* wkv, bool w_f32,
                                                            void* cache, const int64_t* positions,
                                                            const int64_t* slots, LatentShape sh, float eps) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  if (blockIdx.y == 0) {
    const float rs = row_rs(p, t * pstride, f32, q_rank, eps, red);
    for (int c = threadIdx.x; c < q_rank; c += NT)
      stv(cq, t * q_rank + c, f32, ldv(p, t * pstride + c, f32) * rs * ldv(wq, c, w_f32));
  } else {
    const char* kv = reinterpret_cast<const char*>(p) + (size_t)q_rank * (f32 ? 4 : 2);
    kv_write_row(cache, kv, pstride, f32, wkv, w_f32, positions, slots, sh, eps, t, red);
  }
}

// resid[t] (fp32) += rmsnorm(sum_k ys[pos[t, k]] + extra[t]) * (w | 1 + w); act[t] (optional, bf16) = resid[t].
// The expert sum is formed twice (statistics, then the update) instead of round-tripping through memory.
__global__ void __launch_bounds__(NT) combine_post_norm_kernel(float* resid, void* act, const void* ys, bool f32,
                                                              const int* pos, const void* extra, int K, int H,
                                                              const void* w, bool w_f32, bool unit, float eps) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  if (!f32 && !w_f32 && H % 8 == 0 && aligned16(ys) && aligned16(resid) && aligned16(w) &&
      (extra == nullptr || aligned16(extra)) && (act == nullptr || aligned16(act))) {
    const bf16_t* yb = reinterpret_cast<const bf16_t*>(ys);
    auto sum8 = [&](int c, float* a) {
#pragma unroll
      for (int q = 0; q < 8; ++q) a[q] = 0.f;
      if (extra) unpack8(reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(extra) + t * H)[c], a);
      for (int k = 0; k < K; ++k) {
        float v[8];
        unpack8(reinterpret_cast<const uint4*>(yb + (int64_t)(pos ? pos[t * K + k] : t * K + k) * H)[c], v);
#pragma unroll
        for (int q = 0; q < 8; ++q) a[q] += v[q];
      }
    };
    float ss = 0.f;
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float a[8];
      sum8(c, a);
#pragma unroll
      for (int q = 0; q < 8; ++q) ss += a[q] * a[q];
    }
    ss = block_sum<NT>(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)H + eps);
    float4* rr = reinterpret_cast<float4*>(resid + t * H);
    for (int c = threadIdx.x; c < H / 8; c += NT) {
      float a[8], g[8];
      sum8(c, a);
      unpack8(reinterpret_cast<const uint4*>(w)[c], g);
      const float4 r0 = rr[2 * c], r1 = rr[2 * c + 1];
      float o[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] += a[q] * rs * (unit ? g[q] + 1.0f : g[q]);
      rr[2 * c] = make_float4(o[0], o[1], o[2], o[3]);
      rr[2 * c + 1] = make_float4(o[4], o[5], o[6], o[7]);
      if (act) reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(act) + t * H)[c] = pack8(o);
    }
    return;
  }
  auto sum_at = [&](int c) {
    float a = extra ? ldv(extra, t * H + c, f32) : 0.f;
    for (int k = 0; k < K; ++k) a += ldv(ys, (int64_t)(pos ? pos[t * K + k] : t * K + k) * H + c, f32);
    return a;
  };
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += NT) {
    const float a = sum_at(c);
    ss += a * a;
  }
  ss = block_sum<NT>(ss, red);
  const float rs = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += NT) {
    float g = ldv(w, c, w_f32);
    if (unit) g += 1.0f;
    const float v = resid[t * H + c] + sum_at(c) * rs * g;
    resid[t * H + c] = v;
    if (act) reinterpret_cast<bf16_t*>(act)[t * H + c] = f2bf(v);
  }
}

}  // namespace

hipError_t launch_rms_norm_ext(void* out, int64_t ostride, bool out_f32, const void* x, int64_t xstride, bool in_f32,
                               const void* w, bool w_f32, bool unit_offset, float eps, int rows, int n,
                               hipStream_t s) {
  if (rows == 0) return hipSuccess;
  if (n <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(rms_norm_ext_kernel, dim3(rows), dim3(NT), 0, s, out, ostride, out_f32, x, xstride, in_f32, w,
                     w_f32, unit_offset, eps, n);
  return hipGetLastError();
}

hipError_t launch_post_norm_residual(float* resid, void* act, const void* y, int64_t ystride, bool y_f32,
                                     const void* w, bool w_f32, bool unit_offset, float eps, float mult, int rows,
                                     int n, hipStream_t s) {
  if (rows == 0) return hipSuccess;
  if (n <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(post_norm_residual_kernel, dim3(rows), dim3(NT), 0, s, resid, act, y, ystride, y_f32, w, w_f32,
                     unit_offset, eps, mult, n);
  return hipGetLastError();
}

hipError_t launch_gated_act(void* out, const void* gu, bool f32, int rows, int f, int kind, float limit, float alpha,
                            hipStream_t s) {
  if (rows == 0) return hipSuccess;
  if (f <= 0 || kind < 0 || kind > 2) return hipErrorInvalidValue;
  hipLaunchKernelGGL(gated_act_kernel, dim3(rows), dim3(NT), 0, s, out, gu, f32, f, kind, limit, alpha);
  return hipGetLastError();
}

hipError_t launch_route_sigmoid_topk(float* w, int* ids, const void* x, int64_t xstride, bool x_f32, const void* wr,
                                     bool wr_f32, int T, int H, int E, int K, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > ROUTE_E_MAX || K < 1 || K > E) return hipErrorInvalidValue;
  hipLaunchKernelGGL(route_sigmoid_topk_kernel, dim3(T), dim3(NT), 0, s, w, ids, x, xstride, x_f32, wr, wr_f32, H, E,
                     K);
  return hipGetLastError();
}

hipError_t launch_topk_sigmoid(float* w, int* ids, const float* z, int T, int E, int K, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > ROUTE_E_MAX || K < 1 || K > E) return hipErrorInvalidValue;
  hipLaunchKernelGGL(topk_sigmoid_kernel, dim3((T + NT - 1) / NT), dim3(NT), 0, s, w, ids, z, T, E, K);
  return hipGetLastError();
}

hipError_t launch_route_softmax_topk(float* w, int* ids, float* gate, const void* x, int64_t xstride, bool x_f32,
                                     const void* wr, bool wr_f32, const float* corr, int T, int H, int E, int K,
                                     hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > ROUTE_E_MAX || K < 1 || K > E) return hipErrorInvalidValue;
  hipLaunchKernelGGL(route_softmax_topk_kernel, dim3(T), dim3(NT), 0, s, w, ids, gate, x, xstride, x_f32, wr, wr_f32,
                     corr, H, E, K);
  return hipGetLastError();
}

hipError_t launch_topk_softmax_corrected(float* w, int* ids, float* gate, const float* z, int zstride,
                                         const float* corr, int T, int E, int K, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > ROUTE_E_MAX || K < 1 || K > E || zstride < E + (gate ? 1 : 0)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(topk_softmax_corrected_kernel, dim3((T + SEL_NT - 1) / SEL_NT), dim3(SEL_NT),
                     (size_t)SEL_NT * E * sizeof(float), s, w, ids, gate, z, zstride, corr, T, E, K);
  return hipGetLastError();
}

hipError_t launch_combine_weighted(float* out, float* resid, void* act, const void* ys, bool f32, const int* pos,
                                   const void* x, const float* wk, const int* ids, int E, const void* extra,
                                   const float* gate, int T, int K, int H, const void* w, bool w_f32, bool unit_offset,
                                   float eps, float mult, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (H <= 0 || H > 16384 || K < 1 || (out == nullptr && resid == nullptr) || (resid != nullptr && w == nullptr))
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(combine_weighted_kernel, dim3(T), dim3(NT), (size_t)H * sizeof(float), s, out, resid, act, ys, f32,
                     pos, x, wk, ids, E, extra, gate, K, H, w, w_f32, unit_offset, eps, mult);
  return hipGetLastError();
}

hipError_t launch_gather_scaled(void* xs, const void* x, bool f32, const int* sorted, const float* w, int n, int K,
                                int H, hipStream_t s) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(gather_scaled_kernel, dim3(n), dim3(NT), 0, s, xs, x, f32, sorted, w, K, H);
  return hipGetLastError();
}

hipError_t launch_combine_sum(float* out, const void* ys, bool f32, const int* pos, const void* extra, int T, int K,
                              int H, hipStream_t s) {
  if (T == 0) return hipSuccess;
  hipLaunchKernelGGL(combine_sum_kernel, dim3(T), dim3(NT), 0, s, out, ys, f32, pos, extra, K, H);
  return hipGetLastError();
}

hipError_t launch_latent_qkv_prep(void* cq, const void* p, int64_t pstride, bool f32, int q_rank, const void* wq,
                                  const void* wkv, bool w_f32, void* cache, const int64_t* positions,
                                  const int64_t* slots, int T, LatentShape sh, float eps, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (q_rank <= 0 || sh.rank <= 0 || sh.rot_dim < 0 || sh.rot_pairs * 2 > sh.rot_dim) return hipErrorInvalidValue;
  hipLaunchKernelGGL(latent_qkv_prep_kernel, dim3(T, 2), dim3(NT), 0, s, cq, p, pstride, f32, q_rank, wq, wkv, w_f32,
                     cache, positions, slots, sh, eps);
  return hipGetLastError();
}

hipError_t launch_combine_post_norm(float* resid, void* act, const void* ys, bool f32, const int* pos,
                                    const void* extra, int T, int K, int H, const void* w, bool w_f32,
                                    bool unit_offset, float eps, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (H <= 0 || K < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(combine_post_norm_kernel, dim3(T), dim3(NT), 0, s, resid, act, ys, f32, pos, extra, K, H, w, w_f32,
                     unit_offset, eps);
  return hipGetLastError();
}

hipError_t launch_latent_kv_write(void* cache, const void* kv, int64_t kvstride, bool f32, const void* w, bool w_f32,
                                  const int64_t* positions, const int64_t* slots, int T, LatentShape sh, float eps,
                                  hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (sh.rank <= 0 || sh.rot_dim < 0 || sh.rot_pairs * 2 > sh.rot_dim) return hipErrorInvalidValue;
  hipLaunchKernelGGL(latent_kv_write_kernel, dim3(T), dim3(NT), 0, s, cache, kv, kvstride, f32, w, w_f32, positions,
                     slots, sh, eps);
  return hipGetLastError();
}

}  // namespace die
