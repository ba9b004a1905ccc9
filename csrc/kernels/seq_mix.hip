// Kernels for models that carry per-sequence state besides the paged KV cache (gfx950). Storage of activations
// is bf16 or fp32 (a run-time flag), arithmetic is fp32; recurrent state, residual streams, decays, gates of the
// recurrence and unit norms are fp32 in both modes.
//
//   embed_hash          token embedding * scale + hashed bigram embedding -> S equal fp32 residual streams
//   store_last_token    the step's last token of every sequence -> state (the next step's "previous token")
//   stream_mix_norm     streams <- mix^T streams + out * y, and the next sublayer's input rmsnorm(in . streams) * g
//   poly_norm_act       c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3
//   delta_prep          short conv + SiLU of q/k/v, unit q/k, beta and decay of the gated delta rule
//   conv_state_update   the convolution's trailing inputs -> state
//   gated_delta         the recurrence itself, one workgroup per (sequence, head), the state in registers (a
//                       column per lane quad)
//   qkv_prep            q/k norm, rotate-half rotary, value norm / value mixing, paged cache write
#include "common.h"
#include "seq_launchers.h"

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
// the value as the activation dtype would hold it
__device__ __forceinline__ float rnd(float v, bool f32) { return f32 ? v : bf2f(f2bf(v)); }
__device__ __forceinline__ float siluf(float z) { return z / (1.0f + expf(-z)); }

constexpr int NT = 256;

__device__ __forceinline__ bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
__device__ __forceinline__ bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; }
// 4 consecutive values (element index i a multiple of 4, the address 8- or 16-byte aligned)
__device__ __forceinline__ float4 ld4(const void* p, int64_t i, bool f32) {
  if (f32) return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
  const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const bf16_t*>(p) + i);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                     __uint_as_float(w.y & 0xffff0000u));
}
__device__ __forceinline__ void st4(void* p, int64_t i, bool f32, float4 v, float sc) {
  if (f32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + i) = make_float4(v.x * sc, v.y * sc, v.z * sc, v.w * sc);
  } else {
    uint2 w;
    w.x = pack2(v.x * sc, v.y * sc);
    w.y = pack2(v.z * sc, v.w * sc);
    *reinterpret_cast<uint2*>(reinterpret_cast<bf16_t*>(p) + i) = w;
  }
}

// sequence of a row: the largest s with cu_q[s] <= row (cu_q == nullptr: the row itself)
__device__ __forceinline__ int seq_of_row(const int* cu_q, int num_seqs, int row) {
  if (cu_q == nullptr) return row;
  int lo = 0, hi = num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= row)
      lo = mid;
    else
      hi = mid - 1;
  }
  return lo;
}

__global__ void __launch_bounds__(NT) embed_hash_kernel(float* streams, int S, int W, const void* embed,
                                                       const void* bigram, bool f32, const int64_t* ids,
                                                       RaggedRows r, int64_t* prev_tok, float scale,
                                                       int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  const int row = blockIdx.x;
  const int64_t tok = ids[row];
  int64_t brow = -1;
  if (bigram != nullptr) {
    const int64_t p = r.positions[row];
    if (p <= 0) {
      brow = buckets;
    } else {
      const int s = seq_of_row(r.cu_q, r.num_seqs, row);
      const int first = r.cu_q ? r.cu_q[s] : s;
      const int64_t prev = row > first ? ids[row - 1] : prev_tok[r.state_slots[s]];
      brow = (prev * mul_prev + tok * mul_cur) % buckets;
    }
    if (r.cu_q == nullptr) {
      // one row per sequence: this workgroup is the slot's only reader, so it also stores the new last token
      __syncthreads();
      if (threadIdx.x == 0) prev_tok[r.state_slots[row]] = tok;
    }
  }
  float* out = streams + (int64_t)row * S * W;
  for (int c = threadIdx.x; c < W; c += NT) {
    float x = ldv(embed, tok * W + c, f32) * scale;
    if (brow >= 0) x += ldv(bigram, brow * W + c, f32);
    for (int s = 0; s < S; ++s) out[(int64_t)s * W + c] = x;
  }
}

__global__ void store_last_token_kernel(int64_t* prev_tok, const int64_t* ids, RaggedRows r) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= r.num_seqs) return;
  const int last = r.cu_q ? r.cu_q[s + 1] - 1 : s;
  if (r.cu_q && last < r.cu_q[s]) return;
  prev_tok[r.state_slots[s]] = ids[last];
}

constexpr int SMAX = 8;

__global__ void __launch_bounds__(NT) stream_mix_norm_kernel(StreamMixArgs a) {
  __shared__ float red[NT / 64];
  __shared__ float sm[SMAX * SMAX + 2 * SMAX];
  const int S = a.S, W = a.W;
  float* mixw = sm;
  float* outw = sm + SMAX * SMAX;
  float* inw = outw + SMAX;
  if (threadIdx.x < S * S) mixw[threadIdx.x] = a.mix ? a.mix[threadIdx.x] : (threadIdx.x / S == threadIdx.x % S);
  if (threadIdx.x < S) {
    outw[threadIdx.x] = a.outw ? a.outw[threadIdx.x] : 1.0f;
    inw[threadIdx.x] = a.inw ? a.inw[threadIdx.x] : 1.0f;
  }
  __syncthreads();
  const int64_t t = blockIdx.x;
  float* xs = a.streams + t * S * W;
  float ss = 0.f;
  // rows of a multiple of 4 columns: 16-byte accesses, 4 columns per thread and trip; the first KEEP trips keep
  // their u = in . x in registers for the second pass (widths up to 4 * KEEP * NT), later ones re-read the streams
  const bool y_ok = a.y1 == nullptr || (a.ys1 % 4 == 0 && aligned8(a.y1) && (a.y2 == nullptr || (a.ys2 % 4 == 0 && aligned8(a.y2))));
  if (W % 4 == 0 && aligned16(a.streams) && y_ok && (a.h == nullptr || aligned16(a.h))) {
    constexpr int KEEP = 8;
    const int W4 = W / 4;
    float4 ukeep[KEEP];
    auto trip = [&](int c4) -> float4 {
      float4 x[SMAX];
#pragma unroll
      for (int s = 0; s < SMAX; ++s)
        if (s < S) x[s] = reinterpret_cast<const float4*>(xs + (int64_t)s * W)[c4];
      float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
      if (a.y1 != nullptr) {
        float4 y = ld4(a.y1, t * a.ys1 + 4 * c4, a.y_f32);
        y.x *= a.a1, y.y *= a.a1, y.z *= a.a1, y.w *= a.a1;
        if (a.y2 != nullptr) {
          const float4 y2 = ld4(a.y2, t * a.ys2 + 4 * c4, a.y_f32);
          y.x += a.a2 * y2.x, y.y += a.a2 * y2.y, y.z += a.a2 * y2.z, y.w += a.a2 * y2.w;
        }
#pragma unroll
        for (int to = 0; to < SMAX; ++to) {
          if (to < S) {
            const float ow = outw[to];
            float4 n = make_float4(ow * y.x, ow * y.y, ow * y.z, ow * y.w);
#pragma unroll
            for (int s = 0; s < SMAX; ++s) {
              if (s < S) {
                const float m = mixw[s * S + to];
                n.x += m * x[s].x, n.y += m * x[s].y, n.z += m * x[s].z, n.w += m * x[s].w;
              }
            }
            reinterpret_cast<float4*>(xs + (int64_t)to * W)[c4] = n;
            const float iw = inw[to];
            u.x += iw * n.x, u.y += iw * n.y, u.z += iw * n.z, u.w += iw * n.w;
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
          if (s < S) {
            const float iw = inw[s];
            u.x += iw * x[s].x, u.y += iw * x[s].y, u.z += iw * x[s].z, u.w += iw * x[s].w;
          }
        }
      }
      ss += u.x * u.x + u.y * u.y + u.z * u.z + u.w * u.w;
      return u;
    };
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c4 = it * NT + threadIdx.x;
      if (c4 < W4) ukeep[it] = trip(c4);
    }
    for (int c4 = KEEP * NT + threadIdx.x; c4 < W4; c4 += NT) trip(c4);
    if (a.h == nullptr) return;
    ss = block_sum<NT>(ss, red);
    const float rs = a.gain[0] / sqrtf(ss / (float)W + a.eps);
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c4 = it * NT + threadIdx.x;
      if (c4 < W4) st4(a.h, t * W + 4 * c4, a.h_f32, ukeep[it], rs);
    }
    for (int c4 = KEEP * NT + threadIdx.x; c4 < W4; c4 += NT) {
      float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int s = 0; s < SMAX; ++s) {
        if (s < S) {
          const float4 x = reinterpret_cast<const float4*>(xs + (int64_t)s * W)[c4];  // this thread's own writes
          const float iw = inw[s];
          u.x += iw * x.x, u.y += iw * x.y, u.z += iw * x.z, u.w += iw * x.w;
        }
      }
      st4(a.h, t * W + 4 * c4, a.h_f32, u, rs);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += NT) {
    float x[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) x[s] = s < S ? xs[(int64_t)s * W + c] : 0.f;
    float u = 0.f;
    if (a.y1 != nullptr) {
      float y = a.a1 * ldv(a.y1, t * a.ys1 + c, a.y_f32);
      if (a.y2 != nullptr) y += a.a2 * ldv(a.y2, t * a.ys2 + c, a.y_f32);
#pragma unroll
      for (int to = 0; to < SMAX; ++to) {
        if (to < S) {
          float n = outw[to] * y;
#pragma unroll
          for (int s = 0; s < SMAX; ++s)
            if (s < S) n += mixw[s * S + to] * x[s];
          xs[(int64_t)to * W + c] = n;
          u += inw[to] * n;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SMAX; ++s)
        if (s < S) u += inw[s] * x[s];
    }
    ss += u * u;
  }
  if (a.h == nullptr) return;
  ss = block_sum<NT>(ss, red);
  const float rs = a.gain[0] / sqrtf(ss / (float)W + a.eps);
  for (int c = threadIdx.x; c < W; c += NT) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < SMAX; ++s)
      if (s < S) u += inw[s] * xs[(int64_t)s * W + c];  // this thread's own writes
    stv(a.h, t * W + c, a.h_f32, u * rs);
  }
}

__global__ void __launch_bounds__(NT) poly_norm_act_kernel(void* out, const void* z, int64_t zstride, bool f32,
                                                          const float* coef, float eps, int n) {
  __shared__ float red[NT / 64];
  const int64_t r = blockIdx.x;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  // bf16 rows of a multiple of 8 columns: 16-byte accesses; the first KEEP trips stay in registers between the two
  // passes (rows up to 8 * KEEP * NT wide are read once), wider rows re-read the rest
  constexpr int KEEP = 8;
  if (!f32 && n % 8 == 0 && zstride % 8 == 0 && aligned16(z) && aligned16(out)) {
    const uint4* zr = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(z) + r * zstride);
    const int n8 = n / 8;
    uint4 keep[KEEP];
    auto sums = [&](const uint4& v) {
      float f[8];
      unpack8(v, f);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float v2 = f[q] * f[q];
        s2 += v2;
        s4 += v2 * v2;
        s6 += v2 * v2 * v2;
      }
    };
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c8 = it * NT + threadIdx.x;
      if (c8 < n8) {
        keep[it] = zr[c8];
        sums(keep[it]);
      }
    }
    for (int c8 = KEEP * NT + threadIdx.x; c8 < n8; c8 += NT) sums(zr[c8]);
    s2 = block_sum<NT>(s2, red);
    s4 = block_sum<NT>(s4, red);
    s6 = block_sum<NT>(s6, red);
    const float r1 = coef[0] / sqrtf(s2 / (float)n + eps), r2 = coef[1] / sqrtf(s4 / (float)n + eps),
                r3 = coef[2] / sqrtf(s6 / (float)n + eps), c3 = coef[3];
    uint4* orow = reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(out) + r * n);
    auto apply = [&](const uint4& v) -> uint4 {
      float f[8];
      unpack8(v, f);
#pragma unroll
      for (int q = 0; q < 8; ++q) f[q] = f[q] * r1 + f[q] * f[q] * r2 + f[q] * f[q] * f[q] * r3 + c3;
      return pack8(f);
    };
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c8 = it * NT + threadIdx.x;
      if (c8 < n8) orow[c8] = apply(keep[it]);
    }
    for (int c8 = KEEP * NT + threadIdx.x; c8 < n8; c8 += NT) orow[c8] = apply(zr[c8]);
    return;
  }
  for (int c = threadIdx.x; c < n; c += NT) {
    const float v = ldv(z, r * zstride + c, f32);
    const float v2 = v * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v2 * v2 * v2;
  }
  s2 = block_sum<NT>(s2, red);
  s4 = block_sum<NT>(s4, red);
  s6 = block_sum<NT>(s6, red);
  const float r1 = coef[0] / sqrtf(s2 / (float)n + eps), r2 = coef[1] / sqrtf(s4 / (float)n + eps),
              r3 = coef[2] / sqrtf(s6 / (float)n + eps), c3 = coef[3];
  for (int c = threadIdx.x; c < n; c += NT) {
    const float v = ldv(z, r * zstride + c, f32);
    stv(out, r * n + c, f32, v * r1 + v * v * r2 + v * v * v * r3 + c3);
  }
}

// ------------------------------------------------------------------------------------------ gated delta rule
constexpr int TAPS_MAX = 16;

__global__ void __launch_bounds__(NT) delta_prep_kernel(float* qkv32, float* bg, const void* x, const void* b,
                                                       const void* a, int64_t xstride, bool f32, const float* conv_w,
                                                       const float* conv_wt, float* conv_state, const float* A_log,
                                                       const float* dt_bias, DeltaShape sh, RaggedRows r) {
  extern __shared__ __attribute__((aligned(16))) float vals[];  // [C]
  const int row = blockIdx.x;
  const int s = seq_of_row(r.cu_q, r.num_seqs, row);
  const int first = r.cu_q ? r.cu_q[s] : s;
  const int i = row - first;
  const int64_t p = r.positions[row];
  const int C = sh.channels(), taps = sh.taps;
  float* st = conv_state + (int64_t)r.state_slots[s] * (taps - 1) * C;
  // bf16 steps with the weights also given tap-major ([taps, C]): 8 channels per thread and trip, 16-byte loads of
  // inputs, weights and state (a decode row is then two dependent trips per thread instead of C / 256)
  const bool wide = conv_wt != nullptr && !f32 && C % 8 == 0 && xstride % 8 == 0 && aligned16(x);
  for (int c8 = threadIdx.x; wide && c8 < C / 8; c8 += NT) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (p - back < 0) continue;
      const int src = i - back;
      float xv[8];
      if (src >= 0) {
        unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(x) + (int64_t)(row - back) * xstride + 8 * c8), xv);
      } else {
        const float4* sp = reinterpret_cast<const float4*>(st + (int64_t)(taps - 1 + src) * C + 8 * c8);
        const float4 s0 = sp[0], s1 = sp[1];
        xv[0] = s0.x, xv[1] = s0.y, xv[2] = s0.z, xv[3] = s0.w, xv[4] = s1.x, xv[5] = s1.y, xv[6] = s1.z, xv[7] = s1.w;
      }

      const float4* wp = reinterpret_cast<const float4*>(conv_wt + (int64_t)j * C + 8 * c8);
      const float4 w0 = wp[0], w1 = wp[1];
      acc[0] += w0.x * xv[0], acc[1] += w0.y * xv[1], acc[2] += w0.z * xv[2], acc[3] += w0.w * xv[3];
      acc[4] += w1.x * xv[4], acc[5] += w1.y * xv[5], acc[6] += w1.z * xv[6], acc[7] += w1.w * xv[7];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) vals[8 * c8 + e] = rnd(siluf(rnd(acc[e], false)), false);
    if (r.cu_q == nullptr) {
      // one row per sequence: this thread is the only reader of its channels' tail, so it shifts it here: state
      // row k takes row k + 1 (zeros where that lies before the sequence's start), the last one the row's input
      const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k = 0; k + 1 < taps - 1; ++k) {
        const bool live = p - (taps - 2 - k) >= 0;
        float4* dp = reinterpret_cast<float4*>(st + (int64_t)k * C + 8 * c8);
        const float4* sp = reinterpret_cast<const float4*>(st + (int64_t)(k + 1) * C + 8 * c8);
        const float4 t0 = sp[0], t1 = sp[1];
        dp[0] = live ? t0 : zero;
        dp[1] = live ? t1 : zero;
      }
      if (taps > 1) {
        float xv[8];
        unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(x) + (int64_t)row * xstride + 8 * c8), xv);
        float4* dp = reinterpret_cast<float4*>(st + (int64_t)(taps - 2) * C + 8 * c8);
        dp[0] = make_float4(xv[0], xv[1], xv[2], xv[3]);
        dp[1] = make_float4(xv[4], xv[5], xv[6], xv[7]);
      }
    }
  }
  for (int c = threadIdx.x; !wide && c < C; c += NT) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (p - back < 0) continue;
      const int src = i - back;
      const float xv = src >= 0 ? ldv(x, (int64_t)(row - back) * xstride + c, f32) : st[(int64_t)(taps - 1 + src) * C + c];
      acc += conv_w[(int64_t)c * taps + j] * xv;
    }
    vals[c] = rnd(siluf(rnd(acc, f32)), f32);
    if (r.cu_q == nullptr) {
      // one row per sequence: this thread is the only reader of its channel's tail, so it shifts it here
      for (int k = 0; k + 1 < taps - 1; ++k)
        st[(int64_t)k * C + c] = p - (taps - 2 - k) >= 0 ? st[(int64_t)(k + 1) * C + c] : 0.f;
      if (taps > 1) st[(int64_t)(taps - 2) * C + c] = ldv(x, (int64_t)row * xstride + c, f32);
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int G = sh.kv_heads, d = sh.dim;
  for (int hh = wave; hh < 2 * G; hh += NT / 64) {
    float* v = vals + hh * d;
    float ss = 0.f;
    for (int c = lane; c < d; c += 64) ss += v[c] * v[c];
    ss = wave_sum(ss);
    float sc = 1.0f / sqrtf(ss + 1e-6f);
    if (hh < G) sc *= 1.0f / sqrtf((float)d);
    for (int c = lane; c < d; c += 64) v[c] *= sc;
  }
  __syncthreads();
  if (C % 4 == 0) {
    float4* dst = reinterpret_cast<float4*>(qkv32 + (int64_t)row * C);
    for (int c4 = threadIdx.x; c4 < C / 4; c4 += NT) dst[c4] = reinterpret_cast<const float4*>(vals)[c4];
  } else {
    for (int c = threadIdx.x; c < C; c += NT) qkv32[(int64_t)row * C + c] = vals[c];
  }
  const int H = sh.heads;
  for (int h = threadIdx.x; h < H; h += NT) {
    const float bv = ldv(b, (int64_t)row * xstride + h, f32);
    const float av = ldv(a, (int64_t)row * xstride + h, f32) + dt_bias[h];
    const float sp = av > 20.f ? av : log1pf(expf(av));
    bg[(int64_t)row * 2 * H + h] = 1.0f / (1.0f + expf(-bv));
    bg[(int64_t)row * 2 * H + H + h] = expf(-expf(A_log[h]) * sp);
  }
}

__global__ void __launch_bounds__(NT) conv_state_update_kernel(float* conv_state, const void* x, int64_t xstride,
                                                              bool f32, DeltaShape sh, RaggedRows r) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * NT + threadIdx.x;
  const int C = sh.channels(), taps = sh.taps;
  if (c >= C) return;
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  const int64_t p0 = r.positions[q0];
  float* st = conv_state + (int64_t)r.state_slots[s] * (taps - 1) * C;
  float old[TAPS_MAX];
#pragma unroll
  for (int k = 0; k < TAPS_MAX; ++k) old[k] = k < taps - 1 ? st[(int64_t)k * C + c] : 0.f;
  for (int k = 0; k < taps - 1; ++k) {
    const int idx = L - 1 - (taps - 2 - k);  // row of the step that lands in place k
    float v = 0.f;
    if (idx >= 0) {
      v = ldv(x, (int64_t)(q0 + idx) * xstride + c, f32);
    } else if (p0 + idx >= 0) {
      const int ok = taps - 1 + idx;
#pragma unroll
      for (int m = 0; m < TAPS_MAX; ++m)
        if (m == ok) v = old[m];
    }
    st[(int64_t)k * C + c] = v;
  }
}

constexpr int TB = 16;  // tokens staged per trip

// One workgroup per (sequence, head). The state S [dim, vdim] lives in registers for the whole step: column j is
// split over the 4 lanes of a quad, lane `part` holding rows [part * DP, (part + 1) * DP) — so a token costs each
// lane 3 * DP multiply-adds and two quad reductions (S^T k and S^T q), with q and k read from LDS as float4
// broadcasts, and 4 * vdim lanes work on one head. Tokens are staged TB at a time; the read-outs of a trip are
// normed and gated afterwards, one wave per token.
template <int DP>
__global__ void __launch_bounds__(1024) gated_delta_kernel(void* out, const float* qkv32, const float* bg,
                                                          const void* gate, int64_t gstride, bool f32,
                                                          const float* norm_w, float eps, float* state, DeltaShape sh,
                                                          RaggedRows r) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int DPAD = 4 * DP;
  const int d = sh.dim, dv = sh.vdim, H = sh.heads, G = sh.kv_heads, C = sh.channels();
  float* qs = sm;                  // [TB][DPAD], zero beyond dim
  float* ks = qs + TB * DPAD;      // [TB][DPAD]
  float* vs = ks + TB * DPAD;      // [TB][dv]
  float* os = vs + TB * dv;        // [TB][dv]
  float* bs = os + TB * dv;        // [TB] beta
  float* gs = bs + TB;             // [TB] decay
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, nthr = blockDim.x;
  const int j = tid >> 2, part = tid & 3;
  const int kh = h / (H / G);
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  const bool fresh = r.positions[q0] <= 0;
  float* st = state + ((int64_t)r.state_slots[s] * H + h) * d * dv;
  float S[DP];
#pragma unroll
  for (int i = 0; i < DP; ++i) {
    const int row = part * DP + i;
    S[i] = (!fresh && row < d && j < dv) ? st[(int64_t)row * dv + j] : 0.f;
  }
  const int lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    __syncthreads();
    for (int e = tid; e < nb * DPAD; e += nthr) {
      const int tt = e / DPAD, c = e % DPAD;
      const float* row = qkv32 + (int64_t)(q0 + t0 + tt) * C;
      qs[e] = c < d ? row[kh * d + c] : 0.f;
      ks[e] = c < d ? row[G * d + kh * d + c] : 0.f;
    }
    for (int e = tid; e < nb * dv; e += nthr) {
      const int tt = e / dv, c = e % dv;
      vs[e] = qkv32[(int64_t)(q0 + t0 + tt) * C + 2 * G * d + h * dv + c];
    }
    if (tid < nb) {
      bs[tid] = bg[(int64_t)(q0 + t0 + tid) * 2 * H + h];
      gs[tid] = bg[(int64_t)(q0 + t0 + tid) * 2 * H + H + h];
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float g = gs[tt], beta = bs[tt];
      const float4* kt = reinterpret_cast<const float4*>(ks + tt * DPAD + part * DP);
      const float4* qt = reinterpret_cast<const float4*>(qs + tt * DPAD + part * DP);
      float kreg[DP];
      float d0 = 0.f, d1 = 0.f;
#pragma unroll
      for (int i = 0; i < DP / 4; ++i) {
        const float4 k4 = kt[i];
        kreg[4 * i] = k4.x;
        kreg[4 * i + 1] = k4.y;
        kreg[4 * i + 2] = k4.z;
        kreg[4 * i + 3] = k4.w;
        S[4 * i] *= g;
        S[4 * i + 1] *= g;
        S[4 * i + 2] *= g;
        S[4 * i + 3] *= g;
        d0 += S[4 * i] * k4.x + S[4 * i + 2] * k4.z;
        d1 += S[4 * i + 1] * k4.y + S[4 * i + 3] * k4.w;
      }
      float dot = d0 + d1;
      dot += __shfl_xor(dot, 1, 64);
      dot += __shfl_xor(dot, 2, 64);
      const float u = beta * ((j < dv ? vs[tt * dv + j] : 0.f) - dot);
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < DP / 4; ++i) {
        const float4 q4 = qt[i];
        S[4 * i] += kreg[4 * i] * u;
        S[4 * i + 1] += kreg[4 * i + 1] * u;
        S[4 * i + 2] += kreg[4 * i + 2] * u;
        S[4 * i + 3] += kreg[4 * i + 3] * u;
        o0 += S[4 * i] * q4.x + S[4 * i + 2] * q4.z;
        o1 += S[4 * i + 1] * q4.y + S[4 * i + 3] * q4.w;
      }
      float o = o0 + o1;
      o += __shfl_xor(o, 1, 64);
      o += __shfl_xor(o, 2, 64);
      if (part == 0 && j < dv) os[tt * dv + j] = o;
    }
    __syncthreads();
    for (int tt = wave; tt < nb; tt += nwaves) {
      float ss = 0.f;
      for (int c = lane; c < dv; c += 64) ss += os[tt * dv + c] * os[tt * dv + c];
      ss = wave_sum(ss);
      const float rs = 1.0f / sqrtf(ss / (float)dv + eps);
      const int64_t row = q0 + t0 + tt;
      for (int c = lane; c < dv; c += 64) {
        const float gt = ldv(gate, row * gstride + h * dv + c, f32);
        stv(out, (row * H + h) * dv + c, f32, os[tt * dv + c] * rs * norm_w[c] * siluf(gt));
      }
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

// --------------------------------------------------------------------------------------------------- qkv prep
__global__ void __launch_bounds__(NT) qkv_prep_kernel(QkvPrepArgs a) {
  extern __shared__ float sm[];
  __shared__ float red[NT / 64];
  const int H = a.heads, G = a.kv_heads, d = a.dim, dv = a.vdim;
  const int nq = H * d, nk = G * d, nv = G * dv;
  float* qv = sm;
  float* kv = qv + nq;
  float* vv = kv + nk;
  const int64_t t = blockIdx.x;
  const bool f32 = a.f32;
  float sq = 0.f, sk = 0.f;
  float lam = 0.f;
  if (a.v_lambda != nullptr) lam = a.v_lambda[0];
  // bf16 with head sizes that are multiples of 8: 16-byte loads and stores, 8 values per thread and trip
  const bool v_is_k = a.v == nullptr;   // values = keys as projected
  const bool wide = !f32 && d % 8 == 0 && dv % 8 == 0 && a.xstride % 8 == 0 && aligned16(a.q) && aligned16(a.k) &&
                    aligned16(a.v) && aligned16(a.q_out) && aligned16(a.cache) &&
                    (a.v_first == nullptr || (a.vfstride % 8 == 0 && aligned16(a.v_first)));
  if (wide) {
    const bf16_t* qp = reinterpret_cast<const bf16_t*>(a.q) + t * a.xstride;
    const bf16_t* kp = reinterpret_cast<const bf16_t*>(a.k) + t * a.xstride;
    const bf16_t* vp = reinterpret_cast<const bf16_t*>(a.v) + t * a.xstride;
    for (int c8 = threadIdx.x; c8 < (v_is_k ? nq + nk : nq + nk + nv) / 8; c8 += NT) {
      const int c = 8 * c8;
      float f[8];
      if (c < nq) {
        unpack8(*reinterpret_cast<const uint4*>(qp + c), f);
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += f[e] * f[e];
      } else if (c < nq + nk) {
        unpack8(*reinterpret_cast<const uint4*>(kp + c - nq), f);
#pragma unroll
        for (int e = 0; e < 8; ++e) sk += f[e] * f[e];
      } else {
        unpack8(*reinterpret_cast<const uint4*>(vp + c - nq - nk), f);
        if (a.v_lambda != nullptr) {
          float g8[8];
          unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(a.v_first) + t * a.vfstride + c - nq - nk), g8);
#pragma unroll
          for (int e = 0; e < 8; ++e) f[e] = (1.0f - lam) * f[e] + lam * g8[e];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[c + e] = f[e];   // qv, kv and vv are adjacent
    }
  } else {
    for (int c = threadIdx.x; c < nq; c += NT) {
      const float x = ldv(a.q, t * a.xstride + c, f32);
      qv[c] = x;
      sq += x * x;
    }
    for (int c = threadIdx.x; c < nk; c += NT) {
      const float x = ldv(a.k, t * a.xstride + c, f32);
      kv[c] = x;
      sk += x * x;
    }
    for (int c = threadIdx.x; c < (v_is_k ? 0 : nv); c += NT) {
      float x = ldv(a.v, t * a.xstride + c, f32);
      if (a.v_lambda != nullptr) x = (1.0f - lam) * x + lam * ldv(a.v_first, t * a.vfstride + c, f32);
      vv[c] = x;
    }
  }
  const bool per_head = a.q_norm != nullptr && a.head_norm;
  auto rotate = [&]() {
    const int half = a.rot_dims / 2;
    const float p = (float)a.positions[t];
    for (int e = threadIdx.x; e < (H + G) * half; e += NT) {
      const int hd = e / half, i = e % half;
      float* base = hd < H ? qv + hd * d : kv + (hd - H) * d;
      float sn, cs;
      sincosf(p * a.inv_freq[i], &sn, &cs);
      const float u = base[i], v = base[i + half];
      base[i] = u * cs - v * sn;
      base[i + half] = v * cs + u * sn;
    }
  };
  const bool rot_first = per_head && a.norm_after_rot;
  if (a.rot_dims > 0 && rot_first) {
    __syncthreads();   // every thread's loads are in LDS
    rotate();
  }
  float qm = 1.0f;   // query temperature
  if (a.q_temp_coef != 0.f) {
    const int64_t p = a.positions[t];
    qm = 1.0f + a.q_temp_coef * logf((float)((p + 1) / a.q_temp_every) + 1.0f);
  }
  if (v_is_k && !per_head) {
    __syncthreads();
    for (int c = threadIdx.x; c < nk; c += NT) vv[c] = kv[c];
  }
  if (per_head) {
    // 16 lanes per head, 16 heads at a time: sum of squares, then one pass that also keeps the raw key as the value
    // (values taken from the keys) and folds the query temperature into the q heads' factor
    __syncthreads();
    const int grp = threadIdx.x >> 4, gl = threadIdx.x & 15;
    for (int hd = grp; hd < H + G; hd += NT / 16) {
      float* base = hd < H ? qv + hd * d : kv + (hd - H) * d;
      const float* w = hd < H ? a.q_norm : a.k_norm;
      float* raw = (v_is_k && hd >= H) ? vv + (hd - H) * d : nullptr;
      float ss = 0.f;
      for (int c = gl; c < d; c += 16) ss += base[c] * base[c];
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      float rs = 1.0f / sqrtf(ss / (float)d + a.eps);
      if (hd < H) rs *= qm;
      for (int c = gl; c < d; c += 16) {
        const float x = base[c];
        if (raw != nullptr) raw[c] = x;
        base[c] = x * rs * w[c];
      }
    }
  } else if (a.q_norm != nullptr) {
    sq = block_sum<NT>(sq, red);   // (a barrier: every thread's loads are in LDS)
    sk = block_sum<NT>(sk, red);
    const float rq = 1.0f / sqrtf(sq / (float)nq + a.eps), rk = 1.0f / sqrtf(sk / (float)nk + a.eps);
    for (int c = threadIdx.x; c < nq; c += NT) qv[c] *= rq * a.q_norm[c];
    for (int c = threadIdx.x; c < nk; c += NT) kv[c] *= rk * a.k_norm[c];
  }
  __syncthreads();
  if (a.q_temp_coef != 0.f && !per_head) {
    for (int c = threadIdx.x; c < nq; c += NT) qv[c] *= qm;
    __syncthreads();
  }
  if (a.rot_dims > 0 && !rot_first) rotate();
  if (a.v_unit) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int g = wave; g < G; g += NT / 64) {
      float ss = 0.f;
      for (int c = lane; c < dv; c += 64) ss += vv[g * dv + c] * vv[g * dv + c];
      ss = wave_sum(ss);
      const float rs = 1.0f / sqrtf(ss / (float)dv + a.eps);
      for (int c = lane; c < dv; c += 64) vv[g * dv + c] *= rs;
    }
  }
  __syncthreads();
  const int64_t slot = a.slots[t];
  // the block's interior is head-major: [G][block_size][K | V]
  const int64_t blk = slot / a.block_size, off = slot % a.block_size;
  if (wide) {
    bf16_t* qo = reinterpret_cast<bf16_t*>(a.q_out) + t * nq;
    for (int c8 = threadIdx.x; c8 < nq / 8; c8 += NT) *reinterpret_cast<uint4*>(qo + 8 * c8) = pack8(qv + 8 * c8);
    if (slot < 0) return;
    bf16_t* cb = reinterpret_cast<bf16_t*>(a.cache);
    for (int c8 = threadIdx.x; c8 < (nk + nv) / 8; c8 += NT) {
      const int c = 8 * c8;
      const int g = c < nk ? c / d : (c - nk) / dv;
      const int e = c < nk ? c % d : d + (c - nk) % dv;
      *reinterpret_cast<uint4*>(cb + ((blk * G + g) * a.block_size + off) * (int64_t)(d + dv) + e) = pack8(kv + c);
    }
    return;
  }
  for (int c = threadIdx.x; c < nq; c += NT) stv(a.q_out, t * nq + c, f32, qv[c]);
  if (slot < 0) return;
  for (int c = threadIdx.x; c < nk + nv; c += NT) {
    const int g = c < nk ? c / d : (c - nk) / dv;
    const int e = c < nk ? c % d : d + (c - nk) % dv;
    stv(a.cache, ((blk * G + g) * a.block_size + off) * (int64_t)(d + dv) + e, f32, kv[c]);  // kv and vv are adjacent
  }
}

bool rows_ok(const RaggedRows& r) { return r.positions != nullptr && r.state_slots != nullptr && r.num_seqs >= 0; }

}  // namespace

hipError_t launch_embed_hash(float* streams, int S, int W, const void* embed, const void* bigram, bool f32,
                             const int64_t* ids, RaggedRows r, int64_t* prev_tok, float scale, int64_t buckets,
                             int64_t mul_prev, int64_t mul_cur, hipStream_t s) {
  if (r.total_rows == 0) return hipSuccess;
  if (S < 1 || W < 1 || (bigram != nullptr && (buckets < 1 || prev_tok == nullptr || !rows_ok(r))))
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(embed_hash_kernel, dim3(r.total_rows), dim3(NT), 0, s, streams, S, W, embed, bigram, f32, ids, r,
                     prev_tok, scale, buckets, mul_prev, mul_cur);
  return hipGetLastError();
}

hipError_t launch_store_last_token(int64_t* prev_tok, const int64_t* ids, RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || r.cu_q == nullptr) return hipSuccess;  // one row per sequence: embed_hash stored it
  if (!rows_ok(r)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(store_last_token_kernel, dim3((r.num_seqs + 63) / 64), dim3(64), 0, s, prev_tok, ids, r);
  return hipGetLastError();
}

hipError_t launch_stream_mix_norm(const StreamMixArgs& a, hipStream_t s) {
  if (a.T == 0) return hipSuccess;
  if (a.S < 1 || a.S > SMAX || a.W < 1 || (a.h != nullptr && a.gain == nullptr)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(stream_mix_norm_kernel, dim3(a.T), dim3(NT), 0, s, a);
  return hipGetLastError();
}

hipError_t launch_poly_norm_act(void* out, const void* z, int64_t zstride, bool f32, const float* coef, float eps,
                                int rows, int n, hipStream_t s) {
  if (rows == 0) return hipSuccess;
  if (n < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(poly_norm_act_kernel, dim3(rows), dim3(NT), 0, s, out, z, zstride, f32, coef, eps, n);
  return hipGetLastError();
}

static bool delta_ok(const DeltaShape& sh) {
  return sh.heads >= 1 && sh.kv_heads >= 1 && sh.heads % sh.kv_heads == 0 && sh.dim >= 1 && sh.dim <= 256 &&
         sh.vdim >= 1 && sh.vdim <= 256 && sh.taps >= 1 && sh.taps <= TAPS_MAX;
}

hipError_t launch_delta_prep(float* qkv32, float* bg, const void* x, const void* b, const void* a, int64_t xstride,
                             bool f32, const float* conv_w, const float* conv_wt, float* conv_state,
                             const float* A_log, const float* dt_bias, DeltaShape sh, RaggedRows r, hipStream_t s) {
  if (r.total_rows == 0) return hipSuccess;
  if (!delta_ok(sh) || !rows_ok(r)) return hipErrorInvalidValue;
  const size_t lds = sizeof(float) * sh.channels();
  if (lds > 150 * 1024) return hipErrorInvalidValue;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(delta_prep_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(delta_prep_kernel, dim3(r.total_rows), dim3(NT), lds, s, qkv32, bg, x, b, a, xstride, f32, conv_w,
                     conv_wt, conv_state, A_log, dt_bias, sh, r);
  return hipGetLastError();
}

hipError_t launch_conv_state_update(float* conv_state, const void* x, int64_t xstride, bool f32, DeltaShape sh,
                                    RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || sh.taps <= 1 || r.cu_q == nullptr) return hipSuccess;  // one row each: delta_prep did it
  if (!delta_ok(sh) || !rows_ok(r)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(conv_state_update_kernel, dim3((sh.channels() + NT - 1) / NT, r.num_seqs), dim3(NT), 0, s,
                     conv_state, x, xstride, f32, sh, r);
  return hipGetLastError();
}

template <int DP>
static hipError_t launch_gd(void* out, const float* qkv32, const float* bg, const void* gate, int64_t gstride, bool f32,
                            const float* norm_w, float eps, float* state, DeltaShape sh, RaggedRows r, hipStream_t s) {
  const int nthr = (4 * sh.vdim + 63) / 64 * 64;
  const size_t lds = sizeof(float) * (TB * (2 * 4 * DP + 2 * sh.vdim) + 2 * TB);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gated_delta_kernel<DP>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(gated_delta_kernel<DP>, dim3(sh.heads, r.num_seqs), dim3(nthr), lds, s, out, qkv32, bg, gate,
                     gstride, f32, norm_w, eps, state, sh, r);
  return hipGetLastError();
}

hipError_t launch_gated_delta(void* out, const float* qkv32, const float* bg, const void* gate, int64_t gstride,
                              bool f32, const float* norm_w, float eps, float* state, DeltaShape sh, RaggedRows r,
                              hipStream_t s) {
  if (r.num_seqs == 0 || r.total_rows == 0) return hipSuccess;
  if (!delta_ok(sh) || !rows_ok(r)) return hipErrorInvalidValue;
  // rows of the state per lane of a quad: dim / 4, rounded up to a multiple of 4
  if (sh.dim <= 16) return launch_gd<4>(out, qkv32, bg, gate, gstride, f32, norm_w, eps, state, sh, r, s);
  if (sh.dim <= 32) return launch_gd<8>(out, qkv32, bg, gate, gstride, f32, norm_w, eps, state, sh, r, s);
  if (sh.dim <= 64) return launch_gd<16>(out, qkv32, bg, gate, gstride, f32, norm_w, eps, state, sh, r, s);
  if (sh.dim <= 128) return launch_gd<32>(out, qkv32, bg, gate, gstride, f32, norm_w, eps, state, sh, r, s);
  return launch_gd<64>(out, qkv32, bg, gate, gstride, f32, norm_w, eps, state, sh, r, s);
}

hipError_t launch_qkv_prep(const QkvPrepArgs& a, hipStream_t s) {
  if (a.T == 0) return hipSuccess;
  if (a.heads < 1 || a.kv_heads < 1 || a.heads % a.kv_heads != 0 || a.dim < 1 || a.vdim < 1 || a.rot_dims < 0 ||
      a.rot_dims > a.dim || (a.rot_dims & 1) || a.block_size < 1 || (a.rot_dims > 0 && a.inv_freq == nullptr) ||
      ((a.q_norm == nullptr) != (a.k_norm == nullptr)) || (a.v_lambda != nullptr && a.v_first == nullptr) ||
      (a.v == nullptr && (a.vdim != a.dim || a.v_lambda != nullptr)) || (a.head_norm && a.q_norm == nullptr) ||
      (a.q_temp_coef != 0.f && a.q_temp_every < 1))
    return hipErrorInvalidValue;
  const size_t lds = sizeof(float) * ((size_t)a.heads * a.dim + (size_t)a.kv_heads * (a.dim + a.vdim));
  if (lds > 150 * 1024) return hipErrorInvalidValue;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_prep_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(qkv_prep_kernel, dim3(a.T), dim3(NT), lds, s, a);
  return hipGetLastError();
}

}  // namespace die
