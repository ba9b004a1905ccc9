// Grouped-query softmax attention over a paged cache, for prompt portions and single decode tokens alike. A cache
// block holds block_size tokens head-major: [G][block_size][K: dim | V: vdim], so the keys and values that one
// key/value head reads from a block are one contiguous piece of memory. A query at position p of its sequence sees the cached positions j <= p
// with p - j < window (window 0: all of them); its score is (q . k_j) * scale + bias[min(p - j, bias_rows - 1), h]
// (bias optional); the softmax denominator holds one more per-head term exp(sink_h) that belongs to no position
// (the running maximum starts at the sink, the running sum at 1). Query and value widths may differ.
//
// Scores, softmax weights and the weighted sum are fp32; storage of q / cache / out is bf16 or fp32.
//
// FMA form (any shape, both storage types): a workgroup of 4 waves owns 4 * RPW rows (a row = one token and one
// of the H / G query heads of ONE key/value head), stages tiles of BK keys and values once in LDS as fp32 (odd row
// stride) and shares them between its rows. Lanes split (key, slice of dim) for the scores, value columns for the
// weighted sum. The matrix-core form for bf16 follows it below.
#include "common.h"
#include "seq_launchers.h"

namespace die {

namespace {

constexpr int WAVES = 4;

template <bool F32> __device__ __forceinline__ float ldt(const void* p, int64_t i) {
  if constexpr (F32)
    return reinterpret_cast<const float*>(p)[i];
  else
    return bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}
template <bool F32> __device__ __forceinline__ void stt(void* p, int64_t i, float v) {
  if constexpr (F32)
    reinterpret_cast<float*>(p)[i] = v;
  else
    reinterpret_cast<bf16_t*>(p)[i] = f2bf(v);
}

// tanh through one v_exp_f32 and one reciprocal: 1 - 2 / (2^(2 x log2 e) + 1); exact limits at +-inf
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.885390081777927f);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

template <int BK, int CC, int RPW, bool F32>
__global__ void __launch_bounds__(256) sink_attn_kernel(SinkAttnArgs a, int QS, int KS, int VS) {
  constexpr int RW = RPW * WAVES;
  extern __shared__ float smem[];
  float* qs = smem;                 // [RW][QS]
  float* ks = qs + RW * QS;         // [BK][KS]
  float* vs = ks + BK * KS;         // [BK][VS]
  float* ps = vs + BK * VS;         // [RW][BK]
  const int s = blockIdx.y, g = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.heads, G = a.kv_heads, QPG = H / G, D = a.dim, DV = a.vdim;
  const int roww = D + DV;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * QPG, row0 = blockIdx.x * RW;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + RW, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / QPG], p_last = (int)a.positions[q0 + last_row / QPG];
  const int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int jhi = min(p_last, ctx - 1);

  for (int r = wave; r < RW; r += WAVES) {
    const int row = row0 + r;
    const bool ok = row < nrows;
    const int64_t t = q0 + (ok ? row / QPG : 0);
    const int h = g * QPG + (ok ? row % QPG : 0);
    for (int d = lane; d < QS; d += 64) qs[r * QS + d] = (ok && d < D) ? ldt<F32>(a.q, (t * H + h) * D + d) : 0.f;
  }

  int prow[RPW], hrow[RPW];
  bool rok[RPW];
  float m[RPW], l[RPW], o[RPW][CC];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int row = row0 + wave * RPW + i;
    rok[i] = row < nrows;
    prow[i] = rok[i] ? (int)a.positions[q0 + row / QPG] : -1;
    hrow[i] = g * QPG + (rok[i] ? row % QPG : 0);
    const bool has_sink = a.sink != nullptr && rok[i];
    m[i] = has_sink ? a.sink[hrow[i]] : -1e30f;
    l[i] = has_sink ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < CC; ++c) o[i][c] = 0.f;
  }

  constexpr int NP = 64 / BK;
  const int key = lane % BK, part = lane / BK;
  const int dlen = (D + NP - 1) / NP, d0 = part * dlen, d1 = min(D, d0 + dlen);
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;

  for (int j0 = jlo; j0 <= jhi; j0 += BK) {
    __syncthreads();
    for (int k = wave; k < BK; k += WAVES) {
      const int j = j0 + k;
      const bool in = j <= jhi;
      const int64_t rowp =
          in ? (((int64_t)bt[j / a.block_size] * G + g) * a.block_size + j % a.block_size) * roww : 0;
      for (int d = lane; d < D; d += 64) ks[k * KS + d] = in ? ldt<F32>(a.cache, rowp + d) : 0.f;
      for (int d = lane; d < DV; d += 64) vs[k * VS + d] = in ? ldt<F32>(a.cache, rowp + D + d) : 0.f;
    }
    __syncthreads();
    float acc[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) acc[i] = 0.f;
    for (int d = d0; d < d1; ++d) {
      const float kv = ks[key * KS + d];
#pragma unroll
      for (int i = 0; i < RPW; ++i) acc[i] += qs[(wave * RPW + i) * QS + d] * kv;
    }
    const int j = j0 + key;
    float alpha[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      float sc = acc[i];
#pragma unroll
      for (int off = BK; off < 64; off <<= 1) sc += __shfl_xor(sc, off, 64);
      const int n = prow[i] - j;
      const bool valid = rok[i] && j <= jhi && n >= 0 && (a.window <= 0 || n < a.window);
      sc *= a.scale;
      if (a.softcap > 0.f) sc = a.softcap * tanhf(sc / a.softcap);
      if (valid && a.slopes != nullptr) sc -= a.slopes[hrow[i]] * (float)n;
      if (valid && a.bias != nullptr) sc += a.bias[(int64_t)min(n, a.bias_rows - 1) * H + hrow[i]];
      sc = valid ? sc : -INFINITY;
      const float mn = fmaxf(m[i], wave_max(sc));
      const float pe = valid ? expf(sc - mn) : 0.f;
      const float psum = wave_sum(part == 0 ? pe : 0.f);
      alpha[i] = expf(m[i] - mn);
      l[i] = l[i] * alpha[i] + psum;
      m[i] = mn;
      if (part == 0) ps[(wave * RPW + i) * BK + key] = pe;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
#pragma unroll
      for (int c = 0; c < CC; ++c) o[i][c] *= alpha[i];
    }
    for (int k = 0; k < BK; ++k) {
      float vc[CC];
#pragma unroll
      for (int c = 0; c < CC; ++c) vc[c] = (lane + 64 * c < DV) ? vs[k * VS + lane + 64 * c] : 0.f;
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const float pk = ps[(wave * RPW + i) * BK + k];
#pragma unroll
        for (int c = 0; c < CC; ++c) o[i][c] += pk * vc[c];
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (!rok[i]) continue;
    const int row = row0 + wave * RPW + i;
    const int64_t t = q0 + row / QPG;
    const float inv = l[i] > 0.f ? 1.0f / l[i] : 0.f;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c;
      if (col < DV) stt<F32>(a.out, (t * H + hrow[i]) * DV + col, o[i][c] * inv);
    }
  }
}

inline int odd(int x) { return x | 1; }

template <int BK, int CC, int RPW, bool F32> hipError_t launch_one(const SinkAttnArgs& a, hipStream_t s) {
  constexpr int RW = RPW * WAVES;
  const int QS = odd(a.dim), KS = odd(a.dim), VS = odd(a.vdim);
  const size_t lds = sizeof(float) * ((size_t)RW * QS + (size_t)BK * KS + (size_t)BK * VS + (size_t)RW * BK);
  if (lds > 150 * 1024) return hipErrorInvalidValue;
  auto kern = sink_attn_kernel<BK, CC, RPW, F32>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    if (e != hipSuccess) return e;
  }
  const int qpg = a.heads / a.kv_heads;
  const int tiles = (a.max_q * qpg + RW - 1) / RW;
  hipLaunchKernelGGL(kern, dim3(tiles, a.num_seqs, a.kv_heads), dim3(256), lds, s, a, QS, KS, VS);
  return hipGetLastError();
}

template <int BK, int RPW, bool F32> hipError_t launch_cc(const SinkAttnArgs& a, hipStream_t s) {
  if (a.vdim <= 64) return launch_one<BK, 1, RPW, F32>(a, s);
  if (a.vdim <= 128) return launch_one<BK, 2, RPW, F32>(a, s);
  if (a.vdim <= 256) return launch_one<BK, 4, RPW, F32>(a, s);
  return hipErrorInvalidValue;
}

template <bool F32> hipError_t launch_fma(const SinkAttnArgs& a, hipStream_t s) {
  const int qpg = a.heads / a.kv_heads;
  // few rows per (sequence, key/value head): one row per wave, smaller key tiles
  if (a.max_q * qpg <= 4) return launch_cc<32, 1, F32>(a, s);
  if (a.dim + a.vdim > 384) return launch_cc<32, 4, F32>(a, s);
  return launch_cc<64, 4, F32>(a, s);
}

// ---------------------------------------------------------------------------------------------------
// bf16 on the matrix cores (v_mfma_f32_32x32x16_bf16), for dim % 16 == 0, dim <= 128, vdim % 32 == 0, vdim <= 128.
// Workgroup = NW waves x 32 rows of one (sequence, key/value head); NW = 1 for steps of few rows (decode). Per tile
// of 32 keys, staged once in LDS as rows [K_g | V_g] (the next tile's global loads in flight meanwhile):
//   S^T[key][q] = K Q^T        A = K rows from LDS, B = Q rows from LDS      (dim / 16 MFMAs)
//   online softmax per query column (a lane pair owns a query), fp32 scores and weights in log2 units, the bias
//   per distance added before, the running max seeded with the sink; P is rounded to bf16 only as MFMA operand
//   O^T[d][q] += V^T P^T      A = the value columns of the same tile read transposed (ds_read_tr16_b64),
//                              B = P^T straight from the score accumulator   (2 * vdim / 32 MFMAs)
// Split keys (decode over long contexts): split z takes keys [jlo + z * chunk, + chunk) and writes its
// unnormalised O, running max and sum to a workspace; sink_attn_merge_kernel combines them. The sink enters
// split 0 only.
constexpr int MKT = 32;
constexpr int BT_LDS_MAX = 2048;
typedef __attribute__((address_space(3))) short4_t lds_short4;
typedef __attribute__((ext_vector_type(8))) short short8_t;

template <int NDB, int NW, int NKC>
__global__ void __launch_bounds__(64 * NW) sink_attn_mfma_kernel(SinkAttnArgs a, int KP, int QP, int QR, int BTC,
                                                                float* ws_o, float* ws_ml, int nsplit, int chunk) {
  constexpr int ROWS = 32 * NW, NT = 64 * NW;
  constexpr int NPF = (MKT * (4 * NDB + NKC) + NT - 1) / NT;  // 16-byte chunks of a key tile per thread
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  // QR query rows are staged: all ROWS of a prompt-sized step; for steps of few rows (NW = 1) only the rows there
  // can be plus one zero row that every further query column reads, which keeps the workgroup's LDS small enough
  // for two waves per SIMD
  bf16_t* qs = reinterpret_cast<bf16_t*>(smem_raw);          // [QR][QP]
  bf16_t* ks = qs + QR * QP;                                  // [MKT][KP] = [K_g | V_g]
  int bx = blockIdx.x, by = blockIdx.y;
  {
    // XCD k (workgroups are dealt round-robin by linear id) takes a contiguous eighth of the sequence-major tile
    // list, so one sequence's cache rows stay in one L2
    const unsigned total = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
    if (total % 8 == 0) {
      const unsigned nl = (lin % 8) * (total / 8) + lin / 8;
      bx = (int)(nl % gridDim.x);
      by = (int)(nl / gridDim.x);
    }
  }
  const int H = a.heads, G = a.kv_heads, QPG = H / G, D = a.dim, DV = a.vdim;
  const int s = by, g = blockIdx.z % G, z = blockIdx.z / G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tid = threadIdx.x;
  const int roww = D + DV;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * QPG, row0 = bx * ROWS;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + ROWS, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / QPG], p_last = (int)a.positions[q0 + last_row / QPG];
  int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  int jhi = min(p_last, ctx - 1);
  if (nsplit > 1) {
    jlo += z * chunk;
    jhi = min(jhi, jlo + chunk - 1);
  }
  const bf16_t* qg = reinterpret_cast<const bf16_t*>(a.q);
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(a.cache);
  const int qcol = lane & 31, hh = lane >> 5;
  const int myrow = row0 + wave * 32 + qcol;
  const bool rok = myrow < nrows;
  const int myh = g * QPG + (rok ? myrow % QPG : 0);
  const int64_t orow = rok ? (int64_t)(q0 + myrow / QPG) * H + myh : 0;
  const int64_t wrows = (int64_t)a.total_q * H;
  if (jlo > jhi) {  // an empty split (uniform over the workgroup): it only reports that it holds nothing
    if (nsplit > 1 && rok && hh == 0) {
      ws_ml[((int64_t)z * wrows + orow) * 2] = -1e30f;
      ws_ml[((int64_t)z * wrows + orow) * 2 + 1] = 0.f;
    }
    return;
  }

  const int lch = D / 8;
  for (int idx = tid; idx < QR * lch; idx += NT) {
    const int r = idx / lch, c = idx % lch, row = row0 + r;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < nrows) {
      const int64_t t = q0 + row / QPG;
      v = *reinterpret_cast<const uint4*>(qg + (t * H + g * QPG + row % QPG) * D + 8 * c);
    }
    *reinterpret_cast<uint4*>(qs + r * QP + 8 * c) = v;
  }

  const bool wave_live = row0 + wave * 32 < nrows;
  const int prow = rok ? (int)a.positions[q0 + myrow / QPG] : -1;
  constexpr float LOG2E = 1.4426950408889634f;
  const float sl2 = a.scale * LOG2E;
  const bool shaped = a.softcap > 0.f || a.slopes != nullptr;
  const float capl2 = a.softcap * LOG2E, s_over_cap = a.softcap > 0.f ? a.scale / a.softcap : 0.f;
  const float cap_m2 = -2.0f * capl2, s2_over_cap = s_over_cap * 2.885390081777927f;
  const float slope2 = a.slopes != nullptr ? a.slopes[myh] * LOG2E : 0.f;
  const bool has_sink = a.sink != nullptr && rok && z == 0;
  float m = has_sink ? a.sink[myh] * LOG2E : -1e30f;
  float l = has_sink ? 1.0f : 0.0f;
  f32x16_t o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;

  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;
  const int kch = (D + DV) / 8, nkk = D / 16;
  int* btl = reinterpret_cast<int*>(ks + MKT * KP);
  const int b_lo = jlo / a.block_size, nbt = jhi / a.block_size - b_lo + 1;
  const bool bt_lds = nbt <= BTC;
  if (bt_lds)
    for (int u = tid; u < nbt; u += NT) btl[u] = bt[b_lo + u];
  uint4 pf[NPF];
  // chunk idx = tid + u * NT of a tile is (key k, 16-byte piece c) = (idx / kch, idx % kch): one division per
  // thread, then steps of (NT / kch, NT % kch); a block size that is a power of two divides by shifting
  const int k_first = tid / kch, c_first = tid - k_first * kch, k_step = NT / kch, c_step = NT - k_step * kch;
  const int bs_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
  auto fetch = [&](int j0, bool lds) {
    int k = k_first, c = c_first;
#pragma unroll
    for (int u = 0; u < NPF; ++u) {
      const int j = j0 + k;
      pf[u] = make_uint4(0, 0, 0, 0);
      if (k < MKT && j <= jhi) {
        const int jb = bs_shift >= 0 ? j >> bs_shift : j / a.block_size;
        const int64_t blk = lds ? btl[jb - b_lo] : bt[jb];
        const int64_t rowp = ((blk * G + g) * a.block_size + (j - jb * a.block_size)) * roww;
        pf[u] = *reinterpret_cast<const uint4*>(cache + rowp + 8 * c);
      }
      k += k_step;
      c += c_step;
      if (c >= kch) {
        c -= kch;
        ++k;
      }
    }
  };
  fetch(jlo, false);
  const int pitchB = KP * 2;
  const int g16 = lane >> 4, i16 = lane & 15;
  const char* vbase = reinterpret_cast<const char*>(ks) + (4 * hh + (i16 >> 2)) * pitchB +
                      (D + 16 * (g16 & 1) + 4 * (i16 & 3)) * 2;
  const float* bias = a.bias ? a.bias + myh : nullptr;
  // distances from bias_rows - 1 on share the table's last row: a lane whose 16 keys of a tile all lie that far
  // back adds that one value without looking anything up
  const float bias_far = bias ? bias[(int64_t)(a.bias_rows - 1) * H] * LOG2E : 0.f;
  // a tile is interior for a wave when every one of its 32 x 32 (key, row) pairs is visible: no masking then
  const int wrow_first = row0 + wave * 32, wrow_last = wrow_first + 31;
  const bool wave_full = wrow_last < nrows;
  const int pw_first = wave_full ? (int)a.positions[q0 + wrow_first / QPG] : 0;
  const int pw_last = wave_full ? (int)a.positions[q0 + wrow_last / QPG] : 0;
  for (int j0 = jlo; j0 <= jhi; j0 += MKT) {
    __syncthreads();  // every wave is done with the previous tile (first: the queries are being written)
    {
      int k = k_first, c = c_first;
#pragma unroll
      for (int u = 0; u < NPF; ++u) {
        if (k < MKT) *reinterpret_cast<uint4*>(ks + k * KP + 8 * c) = pf[u];
        k += k_step;
        c += c_step;
        if (c >= kch) {
          c -= kch;
          ++k;
        }
      }
    }
    __syncthreads();
    if (j0 + MKT <= jhi) fetch(j0 + MKT, bt_lds);  // in flight while this tile is computed
    if (!wave_live) continue;
    f32x16_t sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    const bf16_t* ka = ks + qcol * KP + 8 * hh;
    const bf16_t* qb = qs + min(wave * 32 + qcol, QR - 1) * QP + 8 * hh;
    for (int kk = 0; kk < nkk; ++kk) {
      const bf16x8_t af = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(ka + 16 * kk));
      const bf16x8_t bfr = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(qb + 16 * kk));
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bfr, sc, 0, 0, 0);
    }
    float mx = -INFINITY;
    const bool interior = wave_full && j0 + MKT - 1 <= min(pw_first, jhi) &&
                          (a.window <= 0 || pw_last - j0 < a.window);
    if (shaped) {
      // capped scores and / or a linear distance penalty: cap * tanh(s * scale / cap) - slope * n, in log2 units.
      // tanh = 1 - 2 / (2^(2 x log2 e) + 1), so the capped score is one multiply-add of the reciprocal; the
      // distance of score r is that of score 0 minus a constant
      const float nf0 = (float)(prow - j0 - 4 * hh);
      if (interior && bias == nullptr) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float nf = nf0 - (float)((r & 3) + 8 * (r >> 2));
          float v;
          if (a.softcap > 0.f)
            v = fmaf(cap_m2, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(sc[r] * s2_over_cap) + 1.0f), capl2);
          else
            v = sc[r] * sl2;
          v = fmaf(-slope2, nf, v);
          sc[r] = v;
          mx = fmaxf(mx, v);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = j0 + (r & 3) + 8 * (r >> 2) + 4 * hh;
          const int n = prow - j;
          const bool valid = interior || (rok && j <= jhi && n >= 0 && (a.window <= 0 || n < a.window));
          float v = a.softcap > 0.f ? capl2 * fast_tanh(sc[r] * s_over_cap) : sc[r] * sl2;
          v -= slope2 * (float)n;
          if (bias != nullptr && valid) v += bias[(int64_t)min(n, a.bias_rows - 1) * H] * LOG2E;
          v = valid ? v : -INFINITY;
          sc[r] = v;
          mx = fmaxf(mx, v);
        }
      }
    } else if (interior) {
      const bool far = bias == nullptr || prow - (j0 + 27 + 4 * hh) >= a.bias_rows - 1;
      if (far) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float v = sc[r] * sl2 + bias_far;
          sc[r] = v;
          mx = fmaxf(mx, v);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = prow - (j0 + (r & 3) + 8 * (r >> 2) + 4 * hh);
          const float v = sc[r] * sl2 + bias[(int64_t)min(n, a.bias_rows - 1) * H] * LOG2E;
          sc[r] = v;
          mx = fmaxf(mx, v);
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = j0 + (r & 3) + 8 * (r >> 2) + 4 * hh;
        const int n = prow - j;
        const bool valid = rok && j <= jhi && n >= 0 && (a.window <= 0 || n < a.window);
        float v = sc[r] * sl2;
        if (bias != nullptr && valid) v += bias[(int64_t)min(n, a.bias_rows - 1) * H] * LOG2E;
        v = valid ? v : -INFINITY;
        sc[r] = v;
        mx = fmaxf(mx, v);
      }
    }
    mx = xor32_max(mx);
    const float mn = fmaxf(m, mx);
    const float alpha = __builtin_amdgcn_exp2f(m - mn);   // v_exp_f32: arguments are <= 0 or -inf here
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pe = __builtin_amdgcn_exp2f(sc[r] - mn);
      sc[r] = pe;
      sum += pe;
    }
    sum = xor32_sum(sum);
    l = l * alpha + sum;
    m = mn;
    bf16x8_t pfr[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      uint4 w;
      w.x = pack2(sc[8 * s2 + 0], sc[8 * s2 + 1]);
      w.y = pack2(sc[8 * s2 + 2], sc[8 * s2 + 3]);
      w.z = pack2(sc[8 * s2 + 4], sc[8 * s2 + 5]);
      w.w = pack2(sc[8 * s2 + 6], sc[8 * s2 + 7]);
      pfr[s2] = __builtin_bit_cast(bf16x8_t, w);
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (alpha != 1.0f) {
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const char* a0 = vbase + (16 * s2) * pitchB + 64 * db;
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(a0));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(a0 + 8 * pitchB));
        const short8_t a8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a8), pfr[s2], o[db], 0, 0, 0);
      }
    }
  }
  if (!rok) return;
  if (nsplit > 1) {
    float* wo = ws_o + ((int64_t)z * wrows + orow) * DV;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<float4*>(wo + 32 * db + 8 * q4 + 4 * hh) =
            make_float4(o[db][4 * q4], o[db][4 * q4 + 1], o[db][4 * q4 + 2], o[db][4 * q4 + 3]);
    if (hh == 0) {
      ws_ml[((int64_t)z * wrows + orow) * 2] = m;
      ws_ml[((int64_t)z * wrows + orow) * 2 + 1] = l;
    }
    return;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  bf16_t* op = reinterpret_cast<bf16_t*>(a.out) + orow * DV;
#pragma unroll
  for (int db = 0; db < NDB; ++db) {
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      uint2 w;
      w.x = pack2(o[db][4 * q4 + 0] * inv, o[db][4 * q4 + 1] * inv);
      w.y = pack2(o[db][4 * q4 + 2] * inv, o[db][4 * q4 + 3] * inv);
      *reinterpret_cast<uint2*>(op + 32 * db + 8 * q4 + 4 * hh) = w;
    }
  }
}


// ---------------------------------------------------------------------------------------------------
// Decode steps (one query token per sequence) in bf16, dim % 8 == 0 <= 128, vdim % 8 == 0 <= 128, at most 8 query
// heads per key/value head: no matrix cores and no staging of keys in LDS. A workgroup of 256 threads owns one
// (sequence, key/value head, split of the keys) and walks its keys 128 at a time:
//   scores   LK lanes share a key (16 bytes of it each, the query's matching 8 dims in registers), 256 / LK keys
//            per pass, all passes' loads issued before the first is used; a shuffle reduction per row
//   softmax  one wave per query row over the 128 scores in LDS (log2 units, running max and sum across trips,
//            the sink seeds split 0)
//   values   16 lanes share a value row, 16 keys per pass, loads issued before the softmax; each thread keeps
//            R x 8 output columns and the 16 key groups are summed through LDS at the end
// Splits write unnormalised sums + (max, sum) to the workspace and sink_attn_merge_kernel combines them.
constexpr int DCH = 128;   // keys per trip

template <int R, int LK>
__global__ void __launch_bounds__(256) sink_attn_decode_kernel(SinkAttnArgs a, float* ws_o, float* ws_ml, int nsplit,
                                                              int chunk) {
  constexpr int NG = 256 / LK, NPK = DCH / NG, NPV = DCH / 16;
  extern __shared__ __attribute__((aligned(16))) float dsm[];
  float* sc = dsm;                       // [R][DCH] scores, then weights
  float* ml = sc + R * DCH;              // [R][3]: running max, running sum, this trip's rescale
  float* red = ml + R * 4;               // [16][R][DV]
  __shared__ int btl[DCH / 1 + 2];       // block-table entries of the trip (at most one per key)
  const int z = blockIdx.x, s = blockIdx.y, g = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = a.heads, G = a.kv_heads, QPG = H / G, D = a.dim, DV = a.vdim, roww = D + DV;
  const int p = (int)a.positions[s];
  const int ctx = a.ctx_lens[s];
  int jlo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  int jhi = min(p, ctx - 1);
  if (nsplit > 1) {
    jlo += z * chunk;
    jhi = min(jhi, jlo + chunk - 1);
  }
  const int64_t wrows = (int64_t)a.total_q * H;
  if (jlo > jhi) {   // an empty split: it only reports that it holds nothing
    if (nsplit > 1 && tid < QPG) {
      const int64_t orow = (int64_t)s * H + g * QPG + tid;
      ws_ml[((int64_t)z * wrows + orow) * 2] = -1e30f;
      ws_ml[((int64_t)z * wrows + orow) * 2 + 1] = 0.f;
    }
    return;
  }
  constexpr float LOG2E = 1.4426950408889634f;
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(a.cache);
  const bf16_t* qg = reinterpret_cast<const bf16_t*>(a.q);
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;
  const int kl = tid % LK, kg = tid / LK;      // score phase: my 8 dims of the key, my key group
  const int vl = tid & 15, vg = tid >> 4;      // value phase: my 8 columns, my key group
  float qf[R][8];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float f[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < QPG && 8 * kl < D) unpack8(*reinterpret_cast<const uint4*>(qg + ((int64_t)s * H + g * QPG + r) * D + 8 * kl), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[r][e] = f[e] * (a.softcap > 0.f ? a.scale / a.softcap : a.scale * LOG2E);
  }
  if (tid < R) {
    const bool has_sink = a.sink != nullptr && tid < QPG && z == 0;
    ml[tid * 4] = has_sink ? a.sink[g * QPG + tid] * LOG2E : -1e30f;
    ml[tid * 4 + 1] = has_sink ? 1.0f : 0.0f;
  }
  float acc[R][8];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;

  for (int j0 = jlo; j0 <= jhi; j0 += DCH) {
    const int b_lo = j0 / a.block_size;
    __syncthreads();   // the previous trip's weights and block-table entries are no longer read
    {
      const int nb = min(jhi, j0 + DCH - 1) / a.block_size - b_lo + 1;
      if (tid < nb) btl[tid] = bt[b_lo + tid];
    }
    __syncthreads();
    uint4 kq[NPK], vq[NPV];
#pragma unroll
    for (int u = 0; u < NPK; ++u) {
      const int j = j0 + u * NG + kg;
      kq[u] = make_uint4(0, 0, 0, 0);
      if (j <= jhi && 8 * kl < D) {
        const int jb = j / a.block_size;
        kq[u] = *reinterpret_cast<const uint4*>(
            cache + (((int64_t)btl[jb - b_lo] * G + g) * a.block_size + (j - jb * a.block_size)) * roww + 8 * kl);
      }
    }
#pragma unroll
    for (int u = 0; u < NPV; ++u) {
      const int j = j0 + u * 16 + vg;
      vq[u] = make_uint4(0, 0, 0, 0);
      if (j <= jhi && 8 * vl < DV) {
        const int jb = j / a.block_size;
        vq[u] = *reinterpret_cast<const uint4*>(
            cache + (((int64_t)btl[jb - b_lo] * G + g) * a.block_size + (j - jb * a.block_size)) * roww + D + 8 * vl);
      }
    }
#pragma unroll
    for (int u = 0; u < NPK; ++u) {
      float f[8];
      unpack8(kq[u], f);
      const int jj = u * NG + kg, j = j0 + jj;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) d += qf[r][e] * f[e];
#pragma unroll
        for (int off = 1; off < LK; off <<= 1) d += __shfl_xor(d, off, 64);
        if (kl == 0) {
          const int n = p - j;
          const bool valid = r < QPG && j <= jhi && n >= 0;
          if (a.softcap > 0.f) d = a.softcap * LOG2E * fast_tanh(d);
          if (valid && a.slopes != nullptr) d -= a.slopes[g * QPG + r] * LOG2E * (float)n;
          if (valid && a.bias != nullptr) d += a.bias[(int64_t)min(n, a.bias_rows - 1) * H + g * QPG + r] * LOG2E;
          sc[r * DCH + jj] = valid ? d : -INFINITY;
        }
      }
    }
    __syncthreads();
    for (int r = wave; r < R; r += 4) {
      const float v0 = sc[r * DCH + lane], v1 = sc[r * DCH + 64 + lane];
      const float m0 = ml[r * 4], l0 = ml[r * 4 + 1];
      const float mn = fmaxf(m0, wave_max(fmaxf(v0, v1)));
      const float p0 = __builtin_amdgcn_exp2f(v0 - mn), p1 = __builtin_amdgcn_exp2f(v1 - mn);
      const float alpha = __builtin_amdgcn_exp2f(m0 - mn);
      const float sum = wave_sum(p0 + p1);
      sc[r * DCH + lane] = p0;
      sc[r * DCH + 64 + lane] = p1;
      if (lane == 0) {
        ml[r * 4] = mn;
        ml[r * 4 + 1] = l0 * alpha + sum;
        ml[r * 4 + 2] = alpha;
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float alpha = ml[r * 4 + 2];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][e] *= alpha;
    }
#pragma unroll
    for (int u = 0; u < NPV; ++u) {
      float f[8];
      unpack8(vq[u], f);
      const int jj = u * 16 + vg;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float pw = sc[r * DCH + jj];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] += pw * f[e];
      }
    }
  }
  // sum the 16 key groups
  if (8 * vl < DV) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float* dst = red + ((int64_t)vg * R + r) * DV + 8 * vl;
      *reinterpret_cast<float4*>(dst) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
      *reinterpret_cast<float4*>(dst + 4) = make_float4(acc[r][4], acc[r][5], acc[r][6], acc[r][7]);
    }
  }
  __syncthreads();
  for (int idx = tid; idx < QPG * DV; idx += 256) {
    const int r = idx / DV, c = idx % DV;
    float o = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) o += red[((int64_t)k * R + r) * DV + c];
    const int64_t orow = (int64_t)s * H + g * QPG + r;
    if (nsplit > 1) {
      ws_o[((int64_t)z * wrows + orow) * DV + c] = o;
      if (c == 0) {
        ws_ml[((int64_t)z * wrows + orow) * 2] = ml[r * 4];
        ws_ml[((int64_t)z * wrows + orow) * 2 + 1] = ml[r * 4 + 1];
      }
    } else {
      const float l = ml[r * 4 + 1];
      reinterpret_cast<bf16_t*>(a.out)[orow * DV + c] = f2bf(l > 0.f ? o / l : 0.f);
    }
  }
}

// out[row] = sum_z O_z 2^(m_z - m*) / sum_z l_z 2^(m_z - m*), m* = max_z m_z (running maxima in log2 units).
__global__ void __launch_bounds__(128) sink_attn_merge_kernel(bf16_t* out, const float* ws_o, const float* ws_ml,
                                                              int nsplit, int64_t rows, int DV) {
  __shared__ float wz[128];   // a split's weight 2^(m_z - m*) / sum (nsplit <= 128)
  const int64_t row = blockIdx.x;
  const int z = threadIdx.x;
  const float mz = z < nsplit ? ws_ml[((int64_t)z * rows + row) * 2] : -1e30f;
  const float lz = z < nsplit ? ws_ml[((int64_t)z * rows + row) * 2 + 1] : 0.f;
  float mstar = wave_max(mz);
  __shared__ float red2[4];
  if ((threadIdx.x & 63) == 0) red2[threadIdx.x >> 6] = mstar;
  __syncthreads();
  mstar = fmaxf(red2[0], red2[1]);
  const float w = lz > 0.f ? exp2f(mz - mstar) : 0.f;
  float lsum = wave_sum(lz * w);
  if ((threadIdx.x & 63) == 0) red2[2 + (threadIdx.x >> 6)] = lsum;
  __syncthreads();
  lsum = red2[2] + red2[3];
  wz[z] = lsum > 0.f ? w / lsum : 0.f;
  __syncthreads();
  for (int c = threadIdx.x; c < DV; c += 128) {
    float acc = 0.f;
    for (int k = 0; k < nsplit; ++k) {
      const float wk = wz[k];
      if (wk != 0.f) acc += ws_o[((int64_t)k * rows + row) * DV + c] * wk;
    }
    out[row * DV + c] = f2bf(acc);
  }
}

template <int NDB, int NW, int NKC> hipError_t launch_mfma(const SinkAttnArgs& a, hipStream_t s) {
  auto* fn = sink_attn_mfma_kernel<NDB, NW, NKC>;
  const int kp = a.dim + a.vdim + 8, qp = a.dim + 8;
  const int qpg0 = a.heads / a.kv_heads;
  const int qr = NW == 1 ? min(32, a.max_q * qpg0 + 1) : 32 * NW;
  const int nsp = a.ws_o != nullptr ? max(1, a.nsplit) : 1;
  // block-table entries staged per workgroup: its key range's (else they are read from global memory)
  const int btc = min(BT_LDS_MAX, (nsp > 1 ? a.chunk / a.block_size + 2 : a.bt_stride) + 1);
  const size_t lds = sizeof(bf16_t) * ((size_t)qr * qp + (size_t)MKT * kp) + sizeof(int) * btc;
  if (lds > 150 * 1024) return hipErrorInvalidValue;
  if (lds > 48 * 1024) {  // only then: the limit is raised per function, and a raised limit is not free
    static size_t raised = 0;
    if (lds > raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds);
      if (e != hipSuccess) return e;
      raised = lds;
    }
  }
  const int qpg = a.heads / a.kv_heads;
  const int nsplit = a.ws_o != nullptr ? max(1, a.nsplit) : 1;
  const dim3 grid((unsigned)(((int64_t)a.max_q * qpg + 32 * NW - 1) / (32 * NW)), (unsigned)a.num_seqs,
                  (unsigned)(a.kv_heads * nsplit));
  hipLaunchKernelGGL(fn, grid, dim3(64 * NW), lds, s, a, kp, qp, qr, btc, a.ws_o, a.ws_ml, nsplit, a.chunk);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || nsplit <= 1) return e;
  hipLaunchKernelGGL(sink_attn_merge_kernel, dim3((unsigned)((int64_t)a.heads * a.total_q)), dim3(128), 0, s,
                     reinterpret_cast<bf16_t*>(a.out), a.ws_o, a.ws_ml, nsplit, (int64_t)a.heads * a.total_q, a.vdim);
  return hipGetLastError();
}

template <int NW, int NKC> hipError_t launch_mfma_ndb(const SinkAttnArgs& a, hipStream_t s) {
  switch (a.vdim / 32) {
    case 1: return launch_mfma<1, NW, NKC>(a, s);
    case 2: return launch_mfma<2, NW, NKC>(a, s);
    case 3: return launch_mfma<3, NW, NKC>(a, s);
    case 4: return launch_mfma<4, NW, NKC>(a, s);
  }
  return hipErrorInvalidValue;
}

template <int NW> hipError_t launch_mfma_nw(const SinkAttnArgs& a, hipStream_t s) {
  return a.dim <= 64 ? launch_mfma_ndb<NW, 8>(a, s) : launch_mfma_ndb<NW, 16>(a, s);
}

template <int R, int LK> hipError_t launch_decode_one(const SinkAttnArgs& a, hipStream_t s) {
  auto* fn = sink_attn_decode_kernel<R, LK>;
  const size_t lds = sizeof(float) * ((size_t)R * DCH + (size_t)R * 4 + (size_t)16 * R * a.vdim);
  if (lds > 48 * 1024) {
    static size_t raised = 0;
    if (lds > raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds);
      if (e != hipSuccess) return e;
      raised = lds;
    }
  }
  const int nsplit = a.ws_o != nullptr ? max(1, a.nsplit) : 1;
  hipLaunchKernelGGL(fn, dim3(nsplit, a.num_seqs, a.kv_heads), dim3(256), lds, s, a, a.ws_o, a.ws_ml, nsplit, a.chunk);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || nsplit <= 1) return e;
  hipLaunchKernelGGL(sink_attn_merge_kernel, dim3((unsigned)((int64_t)a.heads * a.total_q)), dim3(128), 0, s,
                     reinterpret_cast<bf16_t*>(a.out), a.ws_o, a.ws_ml, nsplit, (int64_t)a.heads * a.total_q, a.vdim);
  return hipGetLastError();
}

template <int LK> hipError_t launch_decode_r(const SinkAttnArgs& a, hipStream_t s) {
  const int qpg = a.heads / a.kv_heads;
  if (qpg <= 1) return launch_decode_one<1, LK>(a, s);
  if (qpg <= 2) return launch_decode_one<2, LK>(a, s);
  if (qpg <= 4) return launch_decode_one<4, LK>(a, s);
  return launch_decode_one<8, LK>(a, s);
}

inline bool decode_ok(const SinkAttnArgs& a) {
  return !a.f32 && a.cu_q == nullptr && a.max_q == 1 && a.heads / a.kv_heads <= 8 && a.dim % 8 == 0 && a.dim <= 128 &&
         a.vdim % 8 == 0 && a.vdim <= 128 && (reinterpret_cast<uintptr_t>(a.q) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.cache) & 15) == 0 && (a.nsplit <= 1 || a.nsplit <= 128);
}

inline bool mfma_ok(const SinkAttnArgs& a) {
  return !a.f32 && a.dim % 16 == 0 && a.dim <= 128 && a.vdim % 32 == 0 && a.vdim <= 128 &&
         (reinterpret_cast<uintptr_t>(a.q) & 15) == 0 && (reinterpret_cast<uintptr_t>(a.cache) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.out) & 7) == 0;
}

}  // namespace

bool sink_attn_uses_mfma(const SinkAttnArgs& a) { return a.impl != 1 && mfma_ok(a); }
bool sink_attn_uses_decode(const SinkAttnArgs& a) { return a.impl == 0 && decode_ok(a); }

hipError_t launch_sink_attn(const SinkAttnArgs& a, hipStream_t s) {
  if (a.num_seqs == 0 || a.total_q == 0) return hipSuccess;
  if (a.heads < 1 || a.kv_heads < 1 || a.heads % a.kv_heads != 0 || a.dim < 1 || a.dim > 512 || a.vdim < 1 ||
      a.vdim > 256 || a.block_size < 1 || a.max_q < 1 || (a.bias != nullptr && a.bias_rows < 1))
    return hipErrorInvalidValue;
  if (sink_attn_uses_decode(a)) return a.dim <= 64 ? launch_decode_r<8>(a, s) : launch_decode_r<16>(a, s);
  if (sink_attn_uses_mfma(a)) {
    const int qpg = a.heads / a.kv_heads;
    return a.max_q * qpg <= 32 ? launch_mfma_nw<1>(a, s) : launch_mfma_nw<4>(a, s);
  }
  if (a.impl == 2) return hipErrorInvalidValue;
  return a.f32 ? launch_fma<true>(a, s) : launch_fma<false>(a, s);
}

}  // namespace die
