// Kernels for recurrent mixers whose state is a vector per channel or a matrix per head (gfx950). Storage of
// activations is bf16 or fp32 (a run-time flag), arithmetic is fp32; gates, decays, step sizes, their softplus /
// exponentials / logarithms, unit norms, recurrent state and the residual are fp32 in both modes.
//
//   embed_scaled              token vector * constant -> fp32 residual (+ its activation copy)
//   conv_silu                 short causal convolution with bias + SiLU, history from the state slot; optionally
//                             the per-head (decay, step size) of a scalar-decay state-space layer
//   conv_tail_update          the convolution's trailing inputs -> state
//   selective_scan            S[c, :] <- exp(d A[c, :]) S[c, :] + d x B; y = S[c, :] . C + D x; y * silu(z): a
//                             channel's states in the registers of 1 - 4 lanes for the whole step
//   exp_gate_scan             log-space input / forget gates under a running maximum: a wave-wide scan over tokens
//   gated_linear_attn         S <- a S + b k v^T, o = S^T q: one workgroup per (sequence, head, block of columns), the
//                             state in registers (a column per lane quad); the normaliser n <- a n + b k with its
//                             read-out n . q rides on the first wave
//   head_norm_gate            o / (max(|n . q|, floor) + 1e-6), per-head RMS norm, weight, sigmoid gate
//   skip_gate_group_norm      (o + D x) * silu(z), RMS norm in equal parts of the row, weight
//   pair_post_norm_residual   resid += mult * rms((rms(y1) w1 + rms(y2) w2) / 2) * (1 + w)
#include "common.h"
#include "rec_launchers.h"

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
// the same with the storage type known at compile time: no branch around the load, so a run of loads stays in flight
// together (behind a run-time branch each load is waited for before the next one issues)
template <bool F32> __device__ __forceinline__ float ldt(const void* p, int64_t i) {
  if constexpr (F32)
    return reinterpret_cast<const float*>(p)[i];
  else
    return bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
// the value as the activation dtype would hold it
__device__ __forceinline__ float rnd(float v, bool f32) { return f32 ? v : bf2f(f2bf(v)); }
__device__ __forceinline__ float siluf(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

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

// ------------------------------------------------------------------------------------------------ embedding
__global__ void __launch_bounds__(NT) embed_scaled_kernel(float* resid, void* act, const void* embed, bool f32,
                                                         const int64_t* ids, float scale, int W) {
  const int64_t t = blockIdx.x;
  const int64_t e0 = ids[t] * W;
  if (!f32 && W % 8 == 0 && al16(embed) && al16(resid) && (act == nullptr || al16(act))) {
    const uint4* ep = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(embed) + e0);
    float4* rp = reinterpret_cast<float4*>(resid + t * W);
    for (int c = threadIdx.x; c < W / 8; c += NT) {
      float f[8];
      unpack8(ep[c], f);
#pragma unroll
      for (int q = 0; q < 8; ++q) f[q] *= scale;
      rp[2 * c] = make_float4(f[0], f[1], f[2], f[3]);
      rp[2 * c + 1] = make_float4(f[4], f[5], f[6], f[7]);
      if (act) reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(act) + t * W)[c] = pack8(f);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = ldv(embed, e0 + c, f32) * scale;
    resid[t * W + c] = v;
    if (act) stv(act, t * W + c, f32, v);
  }
}

// ---------------------------------------------------------------------------------------------- convolution
constexpr int TAPS_MAX = 16;

// One workgroup per row. bf16 steps with tap-major weights: 8 channels per thread and trip, 16-byte loads of
// inputs, weights and state.
__global__ void __launch_bounds__(NT) conv_silu_kernel(ConvSiluArgs a, RaggedRows r) {
  const int row = blockIdx.x;
  const int s = seq_of_row(r.cu_q, r.num_seqs, row);
  const int first = r.cu_q ? r.cu_q[s] : s;
  const int i = row - first;
  const int64_t p = r.positions[row];
  const int C = a.C, taps = a.taps;
  const bool f32 = a.f32;
  float* st = a.conv_state + (int64_t)r.state_slots[s] * (taps - 1) * C;
  const bool wide = a.wt != nullptr && !f32 && C % 8 == 0 && a.xstride % 8 == 0 && al16(a.x) && al16(a.y);
  for (int c8 = threadIdx.x; wide && c8 < C / 8; c8 += NT) {
    float acc[8];
    if (a.bias) {
      const float4 b0 = *reinterpret_cast<const float4*>(a.bias + 8 * c8), b1 = *reinterpret_cast<const float4*>(a.bias + 8 * c8 + 4);
      acc[0] = b0.x, acc[1] = b0.y, acc[2] = b0.z, acc[3] = b0.w, acc[4] = b1.x, acc[5] = b1.y, acc[6] = b1.z, acc[7] = b1.w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    }
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (p - back < 0) continue;
      const int src = i - back;
      float xv[8];
      if (src >= 0) {
        unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(a.x) + (int64_t)(row - back) * a.xstride + 8 * c8), xv);
      } else {
        const float4* sp = reinterpret_cast<const float4*>(st + (int64_t)(taps - 1 + src) * C + 8 * c8);
        const float4 s0 = sp[0], s1 = sp[1];
        xv[0] = s0.x, xv[1] = s0.y, xv[2] = s0.z, xv[3] = s0.w, xv[4] = s1.x, xv[5] = s1.y, xv[6] = s1.z, xv[7] = s1.w;
      }
      const float4* wp = reinterpret_cast<const float4*>(a.wt + (int64_t)j * C + 8 * c8);
      const float4 w0 = wp[0], w1 = wp[1];
      acc[0] += w0.x * xv[0], acc[1] += w0.y * xv[1], acc[2] += w0.z * xv[2], acc[3] += w0.w * xv[3];
      acc[4] += w1.x * xv[4], acc[5] += w1.y * xv[5], acc[6] += w1.z * xv[6], acc[7] += w1.w * xv[7];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = siluf(rnd(acc[e], false));
    reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(a.y) + (int64_t)row * C)[c8] = pack8(acc);
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
        unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(a.x) + (int64_t)row * a.xstride + 8 * c8), xv);
        float4* dp = reinterpret_cast<float4*>(st + (int64_t)(taps - 2) * C + 8 * c8);
        dp[0] = make_float4(xv[0], xv[1], xv[2], xv[3]);
        dp[1] = make_float4(xv[4], xv[5], xv[6], xv[7]);
      }
    }
  }
  for (int c = threadIdx.x; !wide && c < C; c += NT) {
    float acc = a.bias ? a.bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (p - back < 0) continue;
      const int src = i - back;
      const float xv = src >= 0 ? ldv(a.x, (int64_t)(row - back) * a.xstride + c, f32) : st[(int64_t)(taps - 1 + src) * C + c];
      acc += a.w[(int64_t)c * taps + j] * xv;
    }
    stv(a.y, (int64_t)row * C + c, f32, siluf(rnd(acc, f32)));
    if (r.cu_q == nullptr) {
      for (int k = 0; k + 1 < taps - 1; ++k)
        st[(int64_t)k * C + c] = p - (taps - 2 - k) >= 0 ? st[(int64_t)(k + 1) * C + c] : 0.f;
      if (taps > 1) st[(int64_t)(taps - 2) * C + c] = ldv(a.x, (int64_t)row * a.xstride + c, f32);
    }
  }
  if (a.dt != nullptr) {
    for (int h = threadIdx.x; h < a.H; h += NT) {
      const float d = softplusf(ldv(a.dt, (int64_t)row * a.xstride + h, f32) + a.dt_bias[h]);
      a.ab[((int64_t)row * a.H + h) * 2] = expf(-expf(a.A_log[h]) * d);
      a.ab[((int64_t)row * a.H + h) * 2 + 1] = d;
    }
  }
}

__global__ void __launch_bounds__(NT) conv_tail_update_kernel(float* conv_state, const void* x, int64_t xstride,
                                                             bool f32, int C, int taps, RaggedRows r) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * NT + threadIdx.x;
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

// ------------------------------------------------------------------------------------------- selective scan
constexpr int TB = 16;   // tokens staged per trip
constexpr int SCH = 256; // threads per workgroup of the scan

// softplus in bf16 steps: hardware exponential and logarithm (v_exp_f32 / v_log_f32), a series where 1 + e^z rounds
template <bool FAST> __device__ __forceinline__ float step_size(float z) {
  if constexpr (FAST) {
    const float e = __expf(-fabsf(z));
    const float l = e < 9.765625e-4f ? e - 0.5f * e * e : __logf(1.0f + e);
    return fmaxf(z, 0.f) + l;
  } else {
    return softplusf(z);
  }
}
// silu(z): bf16 steps use the hardware's exponential and reciprocal
template <bool FAST> __device__ __forceinline__ float gate_of(float z) {
  if constexpr (FAST)
    return z * __builtin_amdgcn_rcpf(1.0f + __expf(-z));
  else
    return siluf(z);
}
// exp(d * A): fp32 steps use expf; bf16 steps fold log2(e) into A once and use the hardware's 2^x
template <bool FAST> __device__ __forceinline__ float decay_of(float d, float a) {
  if constexpr (FAST)
    return __builtin_amdgcn_exp2f(d * a);
  else
    return expf(d * a);
}

// One workgroup per (block of channels, sequence). A channel's N states are split over LPC lanes (NP each) and stay
// in registers for the whole step; a token costs a lane NP exponentials and 3 NP multiply-adds, plus a reduction
// over the LPC lanes. B_t and C_t of TB tokens are staged in LDS per trip and read as float4 broadcasts; every lane
// loads its channel's x, step size and z of the trip into registers up front, so their latencies overlap.
template <int NP, int LPC, bool FAST>
__global__ void __launch_bounds__(SCH) selective_scan_kernel(SelectiveScanArgs a, RaggedRows r) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int NPAD = NP * LPC, CH = SCH / LPC;
  float* Bs = sm;                     // [TB][NPAD], zero beyond N
  float* Cs = Bs + TB * NPAD;         // [TB][NPAD]
  const int s = blockIdx.y, tid = threadIdx.x;
  const int cl = tid / LPC, part = tid % LPC;
  const int c = blockIdx.x * CH + cl;
  const int I = a.I, N = a.N;
  const bool f32 = a.f32;
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  const bool fresh = r.positions[q0] <= 0;
  const bool live = c < I;
  const int cc = live ? c : 0;
  float* st = a.state + ((int64_t)r.state_slots[s] * I + cc) * N;
  const float* Ap = a.A + (int64_t)cc * N;
  float S[NP], A[NP];
  constexpr float LOG2E = 1.4426950408889634f;
  if (N % 4 == 0) {
#pragma unroll
    for (int i = 0; i < NP / 4; ++i) {
      const int n = part * NP + 4 * i;
      const bool ok = live && n < N;
      const float4 z4 = make_float4(0.f, 0.f, 0.f, 0.f);
      const float4 sv = (ok && !fresh) ? *reinterpret_cast<const float4*>(st + n) : z4;
      const float4 av = ok ? *reinterpret_cast<const float4*>(Ap + n) : z4;
      S[4 * i] = sv.x, S[4 * i + 1] = sv.y, S[4 * i + 2] = sv.z, S[4 * i + 3] = sv.w;
      A[4 * i] = av.x, A[4 * i + 1] = av.y, A[4 * i + 2] = av.z, A[4 * i + 3] = av.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int n = part * NP + i;
      const bool ok = live && n < N;
      S[i] = (ok && !fresh) ? st[n] : 0.f;
      A[i] = ok ? Ap[n] : 0.f;
    }
  }
  if (FAST) {
#pragma unroll
    for (int i = 0; i < NP; ++i) A[i] *= LOG2E;
  }
  const float Dc = a.D[cc], dtb = a.dt_bias[cc];
  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    __syncthreads();
    for (int e = tid; e < nb * NPAD; e += SCH) {
      const int tt = e / NPAD, n = e % NPAD;
      const int64_t base = (int64_t)(q0 + t0 + tt) * a.bcstride;
      Bs[e] = n < N ? ldt<!FAST>(a.bc, base + a.boff + n) : 0.f;
      Cs[e] = n < N ? ldt<!FAST>(a.bc, base + a.coff + n) : 0.f;
    }
    float xr[TB], dr[TB], zr[TB];
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      const int64_t row = q0 + t0 + (tt < nb ? tt : 0);
      xr[tt] = ldt<!FAST>(a.x, row * a.xstride + cc);
      dr[tt] = ldt<!FAST>(a.dt, row * a.dtstride + cc);
      zr[tt] = ldt<!FAST>(a.z, row * a.zstride + cc);
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      if (tt < nb) {
        const float x = xr[tt], d = step_size<FAST>(dr[tt] + dtb);
        const float dx = d * x;
        const float4* Bt = reinterpret_cast<const float4*>(Bs + tt * NPAD + part * NP);
        const float4* Ct = reinterpret_cast<const float4*>(Cs + tt * NPAD + part * NP);
        float y0 = 0.f, y1 = 0.f;
#pragma unroll
        for (int i = 0; i < NP / 4; ++i) {
          const float4 b4 = Bt[i], c4 = Ct[i];
          S[4 * i] = decay_of<FAST>(d, A[4 * i]) * S[4 * i] + dx * b4.x;
          S[4 * i + 1] = decay_of<FAST>(d, A[4 * i + 1]) * S[4 * i + 1] + dx * b4.y;
          S[4 * i + 2] = decay_of<FAST>(d, A[4 * i + 2]) * S[4 * i + 2] + dx * b4.z;
          S[4 * i + 3] = decay_of<FAST>(d, A[4 * i + 3]) * S[4 * i + 3] + dx * b4.w;
          y0 += S[4 * i] * c4.x + S[4 * i + 2] * c4.z;
          y1 += S[4 * i + 1] * c4.y + S[4 * i + 3] * c4.w;
        }
        float y = y0 + y1;
        if (LPC > 1) y += __shfl_xor(y, 1, 64);
        if (LPC > 2) y += __shfl_xor(y, 2, 64);
        if (part == 0 && live) stv(a.out, (int64_t)(q0 + t0 + tt) * I + c, f32, (y + Dc * x) * gate_of<FAST>(zr[tt]));
      }
    }
  }
  if (live) {
    if (N % 4 == 0) {
#pragma unroll
      for (int i = 0; i < NP / 4; ++i) {
        const int n = part * NP + 4 * i;
        if (n < N) *reinterpret_cast<float4*>(st + n) = make_float4(S[4 * i], S[4 * i + 1], S[4 * i + 2], S[4 * i + 3]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int n = part * NP + i;
        if (n < N) st[n] = S[i];
      }
    }
  }
}

template <int NP, int LPC> hipError_t launch_scan_one(const SelectiveScanArgs& a, RaggedRows r, hipStream_t s) {
  constexpr int CH = SCH / LPC;
  const size_t smem = (size_t)TB * 2 * NP * LPC * sizeof(float);
  const dim3 grid((a.I + CH - 1) / CH, r.num_seqs);
  if (a.f32)
    hipLaunchKernelGGL((selective_scan_kernel<NP, LPC, false>), grid, dim3(SCH), smem, s, a, r);
  else
    hipLaunchKernelGGL((selective_scan_kernel<NP, LPC, true>), grid, dim3(SCH), smem, s, a, r);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------ gate scan
// One wave per (head, sequence); 64 tokens per trip, one per lane. A token is the map m -> max(m + f, i); two maps
// compose to (f1 + f2, max(i1 + f2, i2)), so an inclusive wave scan gives every token's running maximum.
__global__ void __launch_bounds__(64) exp_gate_scan_kernel(float* abe, const void* x, int64_t xstride, int ioff,
                                                          int foff, bool f32, const float* i_bias,
                                                          const float* f_bias, float cap, float* m_state, int H,
                                                          RaggedRows r) {
  const int h = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  float* mp = m_state + (int64_t)r.state_slots[s] * H + h;
  float m_in = r.positions[q0] <= 0 ? 0.f : *mp;
  const float ib = i_bias[h], fb = f_bias[h], icap = 1.0f / cap;
  for (int t0 = 0; t0 < L; t0 += 64) {
    const int nb = min(64, L - t0);
    const bool ok = lane < nb;
    const int64_t row = q0 + t0 + (ok ? lane : 0);
    const float ig = cap * tanhf((ldv(x, row * xstride + ioff + h, f32) + ib) * icap);
    const float fz = cap * tanhf((ldv(x, row * xstride + foff + h, f32) + fb) * icap);
    // logsigmoid(z) = min(z, 0) - log1p(exp(-|z|))
    const float fg = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));
    float F = ok ? fg : 0.f, Im = ok ? ig : -INFINITY;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float Fp = __shfl_up(F, off, 64), Ip = __shfl_up(Im, off, 64);
      if (lane >= off) {
        Im = fmaxf(Ip + F, Im);
        F = Fp + F;
      }
    }
    const float m = fmaxf(m_in + F, Im);
    float mprev = __shfl_up(m, 1, 64);
    if (lane == 0) mprev = m_in;
    if (ok) {
      float* o = abe + ((int64_t)row * H + h) * 3;
      o[0] = expf(fg + mprev - m);
      o[1] = expf(ig - m);
      o[2] = expf(-m);
    }
    m_in = __shfl(m, nb - 1, 64);
  }
  if (lane == 0) *mp = m_in;
}

// ---------------------------------------------------------------------------------------- matrix recurrence
// One workgroup per (head, sequence, block of VC columns). The state lives in registers for the whole step: column j
// is split over the 4 lanes of a quad, lane `part` holding rows [part * DP, (part + 1) * DP). A token costs each lane
// 2 * DP multiply-adds and one quad reduction; q (scaled) and k come from LDS as float4 broadcasts, b scales the
// value. The normaliser n <- a n + b k (a vector of `dim` rows, RP per lane) is carried by the first wave of column
// block 0, which runs a trip's tokens over the staged k and q once more after its columns and reduces the TB dot
// products n . q over its lanes. (As a column of its own the normaliser would add a ninth wave to workgroups of 512
// threads; measured, that ran 1.8x slower than the kernel without it, and a one-wave launch beside it 1.7x.)
template <int DP, bool F32>
__global__ void __launch_bounds__(1024) gated_linear_attn_kernel(GatedLinearArgs a, RaggedRows r, int VC) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int DPAD = 4 * DP;
  const int d = a.dim, dv = a.vdim, H = a.heads;
  float* qs = sm;                  // [TB][DPAD], zero beyond dim
  float* ks = qs + TB * DPAD;      // [TB][DPAD]
  float* vs = ks + TB * DPAD;      // [TB][VC]
  float* as = vs + TB * VC;        // [TB][2]: a, b
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, nthr = blockDim.x;
  const int v0 = blockIdx.z * VC;
  const int ncol = min(VC, dv - v0);
  const int j = tid >> 2, part = tid & 3;
  const int g = h / (H / a.groups);
  const int q0 = r.cu_q ? r.cu_q[s] : s;
  const int L = r.cu_q ? r.cu_q[s + 1] - q0 : 1;
  if (L <= 0) return;
  const bool fresh = r.positions[q0] <= 0;
  float* st = a.state + ((int64_t)r.state_slots[s] * H + h) * (int64_t)d * dv + v0 + j;
  float S[DP];
#pragma unroll
  for (int i = 0; i < DP; ++i) {
    const int row = part * DP + i;
    S[i] = (!fresh && row < d && j < ncol) ? st[(int64_t)row * dv] : 0.f;
  }
  constexpr int RP = DPAD > 64 ? DPAD / 64 : 1;
  const bool norm = a.n_state != nullptr && blockIdx.z == 0 && tid < 64;   // wave-uniform
  float* nst = norm ? a.n_state + ((int64_t)r.state_slots[s] * H + h) * d : nullptr;
  float nv[RP];
#pragma unroll
  for (int i = 0; i < RP; ++i) nv[i] = (norm && !fresh && tid + 64 * i < d) ? nst[tid + 64 * i] : 0.f;
  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    __syncthreads();
    for (int e = tid; e < nb * DPAD; e += nthr) {
      const int tt = e / DPAD, c = e % DPAD;
      const int64_t base = (int64_t)(q0 + t0 + tt) * a.xstride + g * d + c;
      qs[e] = c < d ? ldt<F32>(a.x, base + a.qoff) * a.qscale : 0.f;
      ks[e] = c < d ? ldt<F32>(a.x, base + a.koff) : 0.f;
    }
    for (int e = tid; e < nb * VC; e += nthr) {
      const int tt = e / VC, c = e % VC;
      vs[e] = c < ncol ? ldt<F32>(a.x, (int64_t)(q0 + t0 + tt) * a.xstride + a.voff + h * dv + v0 + c) : 0.f;
    }
    for (int e = tid; e < 2 * nb; e += nthr) as[e] = a.ab[((int64_t)(q0 + t0 + (e >> 1)) * H + h) * a.abw + (e & 1)];
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float4* kt = reinterpret_cast<const float4*>(ks + tt * DPAD + part * DP);
      const float4* qt = reinterpret_cast<const float4*>(qs + tt * DPAD + part * DP);
      const float2 ab = *reinterpret_cast<const float2*>(as + 2 * tt);
      const float vj = (j < ncol ? vs[tt * VC + j] : 0.f) * ab.y;
      const float dec = ab.x;
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < DP / 4; ++i) {
        const float4 k4 = kt[i], q4 = qt[i];
        S[4 * i] = S[4 * i] * dec + k4.x * vj;
        S[4 * i + 1] = S[4 * i + 1] * dec + k4.y * vj;
        S[4 * i + 2] = S[4 * i + 2] * dec + k4.z * vj;
        S[4 * i + 3] = S[4 * i + 3] * dec + k4.w * vj;
        o0 += S[4 * i] * q4.x + S[4 * i + 2] * q4.z;
        o1 += S[4 * i + 1] * q4.y + S[4 * i + 3] * q4.w;
      }
      float o = o0 + o1;
      o += __shfl_xor(o, 1, 64);
      o += __shfl_xor(o, 2, 64);
      if (part == 0 && j < ncol) a.out[((int64_t)(q0 + t0 + tt) * H + h) * dv + v0 + j] = o;
    }
    if (norm) {
      float p[TB];
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) {
        float acc = 0.f;
        if (tt < nb) {
          const float2 ab = *reinterpret_cast<const float2*>(as + 2 * tt);
#pragma unroll
          for (int i = 0; i < RP; ++i) {
            const int row = tid + 64 * i;
            if (row < DPAD) {
              nv[i] = nv[i] * ab.x + ab.y * ks[tt * DPAD + row];
              acc += nv[i] * qs[tt * DPAD + row];
            }
          }
        }
        p[tt] = xor32_sum(acc);
      }
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) {
        float v = p[tt];
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (tid == 0 && tt < nb) a.nq[(int64_t)(q0 + t0 + tt) * H + h] = v;
      }
    }
  }
  if (j < ncol) {
#pragma unroll
    for (int i = 0; i < DP; ++i) {
      const int row = part * DP + i;
      if (row < d) st[(int64_t)row * dv] = S[i];
    }
  }
  if (norm) {
#pragma unroll
    for (int i = 0; i < RP; ++i)
      if (tid + 64 * i < d) nst[tid + 64 * i] = nv[i];
  }
}

template <int DP, bool F32> hipError_t launch_gla_dp(const GatedLinearArgs& a, RaggedRows r, hipStream_t s) {
  const int VC = a.vdim < 128 ? a.vdim : 128;
  const int nvc = (a.vdim + VC - 1) / VC;
  const int threads = (4 * VC + 63) / 64 * 64;
  const size_t smem = (size_t)(2 * TB * 4 * DP + TB * VC + 2 * TB) * sizeof(float);
  hipLaunchKernelGGL((gated_linear_attn_kernel<DP, F32>), dim3(a.heads, r.num_seqs, nvc), dim3(threads), smem, s, a, r,
                     VC);
  return hipGetLastError();
}
template <int DP> hipError_t launch_gla_dp(const GatedLinearArgs& a, RaggedRows r, hipStream_t s) {
  return a.f32 ? launch_gla_dp<DP, true>(a, r, s) : launch_gla_dp<DP, false>(a, r, s);
}

// ------------------------------------------------------------------------------------------------ epilogues
// 4 consecutive activations (element index a multiple of 4, 8- / 16-byte aligned address)
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

// One workgroup per token; 16 lanes per head, 16 heads at a time. vec: head sizes and strides that are multiples of
// 4 with aligned bases, 4 values per lane and trip.
__global__ void __launch_bounds__(NT) head_norm_gate_kernel(void* out, const float* o, const float* nq,
                                                           const float* abe, const void* g, int64_t gstride, bool f32,
                                                           const float* w, int H, int dv, float eps, bool vec) {
  const int64_t t = blockIdx.x;
  const int gl = threadIdx.x & 15, grp = threadIdx.x >> 4;
  for (int h = grp; h < H; h += NT / 16) {
    const float den = fmaxf(fabsf(nq[t * H + h]), abe[(t * H + h) * 3 + 2]) + 1e-6f;
    const float inv = 1.0f / den;
    const float* oh = o + (t * H + h) * dv;
    float ss = 0.f;
    if (vec) {
      for (int c = 4 * gl; c < dv; c += 64) {
        const float4 u = f4(oh, c);
        ss += (u.x * u.x + u.y * u.y + u.z * u.z + u.w * u.w) * inv * inv;
      }
    } else {
      for (int c = gl; c < dv; c += 16) {
        const float u = oh[c] * inv;
        ss += u * u;
      }
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float rsn = inv / sqrtf(ss / (float)dv + eps);
    if (vec) {
      for (int c = 4 * gl; c < dv; c += 64) {
        const float4 u = f4(oh, c), ww = f4(w, h * dv + c), gt = ld4(g, t * gstride + h * dv + c, f32);
        st4(out, (t * H + h) * dv + c, f32,
            make_float4(u.x * rsn * ww.x * sigmoidf(gt.x), u.y * rsn * ww.y * sigmoidf(gt.y),
                        u.z * rsn * ww.z * sigmoidf(gt.z), u.w * rsn * ww.w * sigmoidf(gt.w)));
      }
    } else {
      for (int c = gl; c < dv; c += 16) {
        const float gt = ldv(g, t * gstride + h * dv + c, f32);
        stv(out, (t * H + h) * dv + c, f32, oh[c] * rsn * w[h * dv + c] * sigmoidf(gt));
      }
    }
  }
}

// One workgroup per (token, part of the row); the gated row is staged in LDS between its statistics and the store.
__global__ void __launch_bounds__(NT) skip_gate_group_norm_kernel(void* out, const float* o, const void* x,
                                                                 int64_t xstride, const float* D, const void* z,
                                                                 int64_t zstride, bool f32, const float* w, int n,
                                                                 int dv, int pw, float eps, bool vec) {
  extern __shared__ __attribute__((aligned(16))) float ys[];   // [pw]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * pw;
  float ss = 0.f;
  if (vec) {
    for (int c = 4 * threadIdx.x; c < pw; c += 4 * NT) {
      const int col = c0 + c;
      const float4 ov = f4(o, t * n + col), xv = ld4(x, t * xstride + col, f32), zv = ld4(z, t * zstride + col, f32);
      const float dh = D[col / dv];
      const float4 y = make_float4((ov.x + dh * xv.x) * siluf(zv.x), (ov.y + dh * xv.y) * siluf(zv.y),
                                   (ov.z + dh * xv.z) * siluf(zv.z), (ov.w + dh * xv.w) * siluf(zv.w));
      *reinterpret_cast<float4*>(ys + c) = y;
      ss += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
    }
  } else {
    for (int c = threadIdx.x; c < pw; c += NT) {
      const int col = c0 + c;
      const float xv = ldv(x, t * xstride + col, f32), zv = ldv(z, t * zstride + col, f32);
      const float y = (o[t * n + col] + D[col / dv] * xv) * siluf(zv);
      ys[c] = y;
      ss += y * y;
    }
  }
  ss = block_sum<NT>(ss, red);
  const float rsn = 1.0f / sqrtf(ss / (float)pw + eps);
  if (vec) {
    for (int c = 4 * threadIdx.x; c < pw; c += 4 * NT) {
      const float4 y = *reinterpret_cast<const float4*>(ys + c), ww = f4(w, c0 + c);
      st4(out, t * n + c0 + c, f32, make_float4(y.x * rsn * ww.x, y.y * rsn * ww.y, y.z * rsn * ww.z, y.w * rsn * ww.w));
    }
    return;
  }
  for (int c = threadIdx.x; c < pw; c += NT) stv(out, t * n + c0 + c, f32, ys[c] * rsn * w[c0 + c]);
}

// One workgroup per row; the averaged row is staged in LDS between its statistics and the update. bf16 rows of a
// multiple of 8 columns: 16-byte loads and stores, 8 columns per thread and trip.
__global__ void __launch_bounds__(NT) pair_post_norm_residual_kernel(float* resid, void* act, const void* y1,
                                                                    int64_t ys1, const float* w1, const void* y2,
                                                                    int64_t ys2, const float* w2, bool f32,
                                                                    const void* w, float mult, float eps, int W) {
  extern __shared__ __attribute__((aligned(16))) float u[];   // [W]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  if (!f32 && W % 8 == 0 && ys1 % 8 == 0 && ys2 % 8 == 0 && al16(y1) && al16(y2) && al16(w) && al16(resid) &&
      (act == nullptr || al16(act))) {
    const uint4* p1 = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(y1) + t * ys1);
    const uint4* p2 = reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(y2) + t * ys2);
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < W / 8; c += NT) {
      float a8[8], b8[8];
      unpack8(p1[c], a8);
      unpack8(p2[c], b8);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        s1 += a8[q] * a8[q];
        s2 += b8[q] * b8[q];
      }
    }
    s1 = block_sum<NT>(s1, red);
    s2 = block_sum<NT>(s2, red);
    const float r1 = 0.5f / sqrtf(s1 / (float)W + eps), r2 = 0.5f / sqrtf(s2 / (float)W + eps);
    float su = 0.f;
    for (int c = threadIdx.x; c < W / 8; c += NT) {
      float a8[8], b8[8];
      unpack8(p1[c], a8);
      unpack8(p2[c], b8);
      const float4 wa0 = f4(w1, 8 * c), wa1 = f4(w1, 8 * c + 4), wb0 = f4(w2, 8 * c), wb1 = f4(w2, 8 * c + 4);
      const float wa[8] = {wa0.x, wa0.y, wa0.z, wa0.w, wa1.x, wa1.y, wa1.z, wa1.w};
      const float wb[8] = {wb0.x, wb0.y, wb0.z, wb0.w, wb1.x, wb1.y, wb1.z, wb1.w};
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        v[q] = a8[q] * r1 * wa[q] + b8[q] * r2 * wb[q];
        su += v[q] * v[q];
      }
      *reinterpret_cast<float4*>(u + 8 * c) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(u + 8 * c + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
    su = block_sum<NT>(su, red);
    const float ru = mult / sqrtf(su / (float)W + eps);
    float4* rr = reinterpret_cast<float4*>(resid + t * W);
    for (int c = threadIdx.x; c < W / 8; c += NT) {
      float g8[8];
      unpack8(reinterpret_cast<const uint4*>(w)[c], g8);
      const float4 u0 = *reinterpret_cast<const float4*>(u + 8 * c), u1 = *reinterpret_cast<const float4*>(u + 8 * c + 4);
      const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
      const float4 a0 = rr[2 * c], a1 = rr[2 * c + 1];
      float o8[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) o8[q] += uv[q] * ru * (1.0f + g8[q]);
      rr[2 * c] = make_float4(o8[0], o8[1], o8[2], o8[3]);
      rr[2 * c + 1] = make_float4(o8[4], o8[5], o8[6], o8[7]);
      if (act) reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(act) + t * W)[c] = pack8(o8);
    }
    return;
  }
  float s1 = 0.f, s2 = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float a = ldv(y1, t * ys1 + c, f32), b = ldv(y2, t * ys2 + c, f32);
    s1 += a * a;
    s2 += b * b;
  }
  s1 = block_sum<NT>(s1, red);
  s2 = block_sum<NT>(s2, red);
  const float r1 = 0.5f / sqrtf(s1 / (float)W + eps), r2 = 0.5f / sqrtf(s2 / (float)W + eps);
  float su = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = ldv(y1, t * ys1 + c, f32) * r1 * w1[c] + ldv(y2, t * ys2 + c, f32) * r2 * w2[c];
    u[c] = v;
    su += v * v;
  }
  su = block_sum<NT>(su, red);
  const float ru = mult / sqrtf(su / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = resid[t * W + c] + u[c] * ru * (1.0f + ldv(w, c, f32));
    resid[t * W + c] = v;
    if (act) stv(act, t * W + c, f32, v);
  }
}

bool rows_ok(const RaggedRows& r) { return r.positions != nullptr && r.state_slots != nullptr && r.num_seqs >= 0; }

}  // namespace

hipError_t launch_embed_scaled(float* resid, void* act, const void* embed, bool f32, const int64_t* ids, float scale,
                               int T, int W, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (W <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(embed_scaled_kernel, dim3(T), dim3(NT), 0, s, resid, act, embed, f32, ids, scale, W);
  return hipGetLastError();
}

hipError_t launch_conv_silu(const ConvSiluArgs& a, RaggedRows r, hipStream_t s) {
  if (r.total_rows == 0) return hipSuccess;
  if (!rows_ok(r) || a.C <= 0 || a.taps < 1 || a.taps > TAPS_MAX || (a.dt != nullptr && (a.H < 1 || a.ab == nullptr)))
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(conv_silu_kernel, dim3(r.total_rows), dim3(NT), 0, s, a, r);
  return hipGetLastError();
}

hipError_t launch_conv_tail_update(float* conv_state, const void* x, int64_t xstride, bool f32, int C, int taps,
                                   RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || taps <= 1) return hipSuccess;
  if (!rows_ok(r) || C <= 0 || taps > TAPS_MAX) return hipErrorInvalidValue;
  if (r.cu_q == nullptr) return hipSuccess;  // conv_silu moved the row's input
  hipLaunchKernelGGL(conv_tail_update_kernel, dim3((C + NT - 1) / NT, r.num_seqs), dim3(NT), 0, s, conv_state, x,
                     xstride, f32, C, taps, r);
  return hipGetLastError();
}

hipError_t launch_selective_scan(const SelectiveScanArgs& a, RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || r.total_rows == 0) return hipSuccess;
  if (!rows_ok(r) || a.I < 1 || a.N < 1 || a.N > 256) return hipErrorInvalidValue;
  if (a.N <= 4) return launch_scan_one<4, 1>(a, r, s);
  if (a.N <= 8) return launch_scan_one<8, 1>(a, r, s);
  if (a.N <= 16) return launch_scan_one<16, 1>(a, r, s);
  if (a.N <= 32) return launch_scan_one<16, 2>(a, r, s);
  if (a.N <= 64) return launch_scan_one<16, 4>(a, r, s);
  if (a.N <= 128) return launch_scan_one<32, 4>(a, r, s);
  return launch_scan_one<64, 4>(a, r, s);
}

hipError_t launch_exp_gate_scan(float* abe, const void* x, int64_t xstride, int ioff, int foff, bool f32,
                                const float* i_bias, const float* f_bias, float cap, float* m_state, int H,
                                RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || r.total_rows == 0) return hipSuccess;
  if (!rows_ok(r) || H < 1 || !(cap > 0.f)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(exp_gate_scan_kernel, dim3(H, r.num_seqs), dim3(64), 0, s, abe, x, xstride, ioff, foff, f32,
                     i_bias, f_bias, cap, m_state, H, r);
  return hipGetLastError();
}

hipError_t launch_gated_linear_attn(const GatedLinearArgs& a, RaggedRows r, hipStream_t s) {
  if (r.num_seqs == 0 || r.total_rows == 0) return hipSuccess;
  if (!rows_ok(r) || a.heads < 1 || a.groups < 1 || a.heads % a.groups || a.dim < 1 || a.dim > 256 || a.vdim < 1 ||
      a.abw < 2 || (a.n_state != nullptr) != (a.nq != nullptr))
    return hipErrorInvalidValue;
  if (a.dim <= 16) return launch_gla_dp<4>(a, r, s);
  if (a.dim <= 32) return launch_gla_dp<8>(a, r, s);
  if (a.dim <= 64) return launch_gla_dp<16>(a, r, s);
  if (a.dim <= 128) return launch_gla_dp<32>(a, r, s);
  return launch_gla_dp<64>(a, r, s);
}

hipError_t launch_head_norm_gate(void* out, const float* o, const float* nq, const float* abe, const void* g,
                                 int64_t gstride, bool f32, const float* w, int T, int H, int vdim, float eps,
                                 hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (H < 1 || vdim < 1) return hipErrorInvalidValue;
  const bool vec = vdim % 4 == 0 && gstride % 4 == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(o) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  hipLaunchKernelGGL(head_norm_gate_kernel, dim3(T), dim3(NT), 0, s, out, o, nq, abe, g, gstride, f32, w, H, vdim, eps,
                     vec);
  return hipGetLastError();
}

hipError_t launch_skip_gate_group_norm(void* out, const float* o, const void* x, int64_t xstride, const float* D,
                                       const void* z, int64_t zstride, bool f32, const float* w, int T, int H, int vdim,
                                       int parts, float eps, hipStream_t s) {
  if (T == 0) return hipSuccess;
  const int n = H * vdim;
  if (H < 1 || vdim < 1 || parts < 1 || parts > 65535 || n % parts || n / parts > 16384) return hipErrorInvalidValue;
  auto a16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec = vdim % 4 == 0 && (n / parts) % 4 == 0 && xstride % 4 == 0 && zstride % 4 == 0 && a16(o) && a16(x) &&
                   a16(z) && a16(w) && a16(out);
  hipLaunchKernelGGL(skip_gate_group_norm_kernel, dim3(T, parts), dim3(NT), (size_t)(n / parts) * sizeof(float), s,
                     out, o, x, xstride, D, z, zstride, f32, w, n, vdim, n / parts, eps, vec);
  return hipGetLastError();
}

hipError_t launch_pair_post_norm_residual(float* resid, void* act, const void* y1, int64_t ys1, const float* w1,
                                          const void* y2, int64_t ys2, const float* w2, bool f32, const void* w,
                                          float mult, float eps, int T, int W, hipStream_t s) {
  if (T == 0) return hipSuccess;
  if (W <= 0 || W > 16384) return hipErrorInvalidValue;
  hipLaunchKernelGGL(pair_post_norm_residual_kernel, dim3(T), dim3(NT), (size_t)W * sizeof(float), s, resid, act, y1,
                     ys1, w1, y2, ys2, w2, f32, w, mult, eps, W);
  return hipGetLastError();
}

}  // namespace die
