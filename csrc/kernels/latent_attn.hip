// Latent (compressed-KV) attention over the paged latent cache, in its absorbed form: every head's query
// is first projected into the latent space (q_lat = W_uk^T q_nope, a batched GEMM outside this file), so
// all heads of a token score against the SAME cached row [latent | rotated shared key part] and the output
// is the weighted sum of the latent rows (W_uv is applied afterwards). One kernel serves prompt chunks and
// single decode tokens: a row is a (token, head) pair, its keys are the cache positions j <= p inside the
// sliding window, and the softmax denominator may hold a per-head sink term exp(sink_h) attached to no position
// (running max starts at the sink, running sum at 1).
//
// Scores, softmax weights and the weighted sum are fp32 (FMA); storage of q / cache / out is bf16 or fp32.
// Workgroup = 4 waves x 4 rows. A tile of BK keys is staged once in LDS as fp32 (row stride odd: a lane per
// key reads conflict-free; a lane per column too) and shared by the 16 rows. Lanes split (key, part of the
// score dimension); the rotary part of q is rotated while it is loaded.
#include "common.h"
#include "mix_launchers.h"

namespace die {

namespace {

constexpr int RPW = 4, WAVES = 4, RW = RPW * WAVES;

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

template <int BK, int CC, bool F32>
__global__ void __launch_bounds__(256) latent_attn_kernel(LatentAttnArgs a, int QS, int KS) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [RW][QS]
  float* ks = qs + RW * QS;         // [BK][KS]
  float* ps = ks + BK * KS;         // [WAVES][RPW][BK]
  const int s = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.heads, R = a.sh.rank, Dk = a.sh.rank + a.sh.rot_dim;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * H, row0 = blockIdx.x * RW;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + RW, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / H], p_last = (int)a.positions[q0 + last_row / H];
  const int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int jhi = min(p_last, ctx - 1);

  // queries -> LDS (fp32), the rotary part rotated by the row's position
  for (int r = wave; r < RW; r += WAVES) {
    const int row = row0 + r;
    const bool ok = row < nrows;
    const int tl = ok ? row / H : 0, h = ok ? row % H : 0;
    const int64_t t = q0 + tl;
    const float p = ok ? (float)a.positions[t] : 0.f;
    const int64_t ql = ((int64_t)h * a.total_q + t) * R;
    const int64_t qr = t * a.q_stride + (int64_t)h * a.q_hstride;
    for (int d = lane; d < QS; d += 64) {
      float v = 0.f;
      if (ok && d < R) {
        v = ldt<F32>(a.q_lat, ql + d);
      } else if (ok && d < Dk) {
        const int dd = d - R, i = dd >> 1;
        if (i < a.sh.rot_pairs) {
          const float u = ldt<F32>(a.q_rot, qr + 2 * i), w = ldt<F32>(a.q_rot, qr + 2 * i + 1);
          float sn, cs;
          sincosf(p * a.sh.inv_freq[i], &sn, &cs);
          v = (dd & 1) ? w * cs + u * sn : u * cs - w * sn;
        } else {
          v = ldt<F32>(a.q_rot, qr + dd);
        }
      }
      qs[r * QS + d] = v;
    }
  }

  int prow[RPW];
  bool rok[RPW];
  float m[RPW], l[RPW], o[RPW][CC];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int row = row0 + wave * RPW + i;
    rok[i] = row < nrows;
    prow[i] = rok[i] ? (int)a.positions[q0 + row / H] : -1;
    const bool has_sink = a.sink != nullptr && rok[i];
    m[i] = has_sink ? a.sink[row % H] : -1e30f;
    l[i] = has_sink ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < CC; ++c) o[i][c] = 0.f;
  }

  constexpr int NP = 64 / BK;
  const int key = lane % BK, part = lane / BK;
  const int dlen = (Dk + NP - 1) / NP, d0 = part * dlen, d1 = min(Dk, d0 + dlen);
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;

  for (int j0 = jlo; j0 <= jhi; j0 += BK) {
    __syncthreads();  // the previous tile (and, first, the queries) are no longer / now in LDS
    for (int k = wave; k < BK; k += WAVES) {
      const int j = j0 + k;
      const bool in = j <= jhi;
      const int64_t rowp = in ? ((int64_t)bt[j / a.block_size] * a.block_size + j % a.block_size) * Dk : 0;
      for (int d = lane; d < Dk; d += 64) ks[k * KS + d] = in ? ldt<F32>(a.cache, rowp + d) : 0.f;
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
      const bool valid = rok[i] && j <= jhi && j <= prow[i] && (a.window <= 0 || prow[i] - j < a.window);
      sc = valid ? sc * a.scale : -INFINITY;
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
      float kvc[CC];
#pragma unroll
      for (int c = 0; c < CC; ++c) kvc[c] = (lane + 64 * c < R) ? ks[k * KS + lane + 64 * c] : 0.f;
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const float pk = ps[(wave * RPW + i) * BK + k];
#pragma unroll
        for (int c = 0; c < CC; ++c) o[i][c] += pk * kvc[c];
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (!rok[i]) continue;
    const int row = row0 + wave * RPW + i;
    const int64_t t = q0 + row / H;
    const int h = row % H;
    const float inv = l[i] > 0.f ? 1.0f / l[i] : 0.f;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c;
      if (col < R) stt<F32>(a.out, ((int64_t)h * a.total_q + t) * R + col, o[i][c] * inv);
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 on the matrix cores (v_mfma_f32_32x32x16_bf16), for rank % 32 == 0, rank <= 256, rot_dim % 16 == 0,
// rot_dim <= 128. Workgroup = NW waves x 32 rows (NW = 1 for steps of few rows per sequence: decode). Per
// tile of 32 keys, staged once in LDS row-major ([key][Dk], the next tile's global loads in flight meanwhile):
//   S^T[key][q] = K Q^T        A = K rows from LDS, B = Q rows from LDS      (Dk / 16 MFMAs)
//   online softmax per query column (one lane pair owns a query: no cross-lane traffic beyond xor 32),
//   fp32 scores and weights, running max seeded with the sink; P is rounded to bf16 only as the MFMA operand
//   O^T[d][q] += V^T P^T      A = the latent columns of the same tile, read transposed (ds_read_tr16_b64),
//                              B = P^T straight from the score accumulator  (2 * rank / 32 MFMAs)
// Split keys (grid.z = nsplit > 1; decode over long contexts): split z takes keys [jlo + z * chunk, + chunk),
// writes its unnormalised O, running max and sum to a workspace, and latent_attn_merge_kernel combines them;
// the sink enters split 0 only.
constexpr int MKT = 32;
constexpr int BT_LDS_MAX = 2048;  // block-table entries staged per workgroup (else read from global memory)
typedef __attribute__((address_space(3))) short4_t lds_short4;
typedef __attribute__((ext_vector_type(8))) short short8_t;

template <int NDB, int NW>
__global__ void __launch_bounds__(64 * NW) latent_attn_mfma_kernel(LatentAttnArgs a, int KP) {
  constexpr int ROWS = 32 * NW, NT = 64 * NW;
  constexpr int NPF = (MKT * (4 * NDB + 16) + NT - 1) / NT;  // 16-byte chunks of a key tile per thread (rot_dim <= 128)
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  bf16_t* qs = reinterpret_cast<bf16_t*>(smem_raw);          // [ROWS][KP]
  bf16_t* ks = qs + ROWS * KP;                                // [MKT][KP]
  // unsplit steps: XCD k (workgroups are dealt round-robin by linear id) takes a contiguous eighth of the
  // sequence-major tile list, so one sequence's cache rows stay in one L2
  int bx = blockIdx.x, by = blockIdx.y;
  if (gridDim.z == 1) {
    const unsigned total = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
    if (total % 8 == 0) {
      const unsigned nl = (lin % 8) * (total / 8) + lin / 8;
      bx = (int)(nl % gridDim.x);
      by = (int)(nl / gridDim.x);
    }
  }
  const int s = by, z = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tid = threadIdx.x;
  const int H = a.heads, R = a.sh.rank, Dk = a.sh.rank + a.sh.rot_dim;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * H, row0 = bx * ROWS;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + ROWS, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / H], p_last = (int)a.positions[q0 + last_row / H];
  int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  int jhi = min(p_last, ctx - 1);
  if (a.nsplit > 1) {
    jlo += z * a.chunk;
    jhi = min(jhi, jlo + a.chunk - 1);
  }
  const bf16_t* qlat = reinterpret_cast<const bf16_t*>(a.q_lat);
  const bf16_t* qrot = reinterpret_cast<const bf16_t*>(a.q_rot);
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(a.cache);
  const int qcol = lane & 31, hh = lane >> 5;
  const int myrow = row0 + wave * 32 + qcol;
  const bool rok = myrow < nrows;
  const int64_t orow = rok ? (int64_t)(myrow % H) * a.total_q + (q0 + myrow / H) : 0;
  if (jlo > jhi) {  // an empty split (uniform over the workgroup): it only reports that it holds nothing
    if (a.nsplit > 1 && rok && hh == 0) {
      a.ws_ml[((int64_t)z * a.heads * a.total_q + orow) * 2] = -1e30f;
      a.ws_ml[((int64_t)z * a.heads * a.total_q + orow) * 2 + 1] = 0.f;
    }
    return;
  }

  // queries -> LDS: the latent part as 16-byte copies, the rotary part rotated in fp32
  const int lch = R / 8;
  for (int idx = tid; idx < ROWS * lch; idx += NT) {
    const int r = idx / lch, c = idx % lch, row = row0 + r;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < nrows) {
      const int64_t t = q0 + row / H;
      v = *reinterpret_cast<const uint4*>(qlat + ((int64_t)(row % H) * a.total_q + t) * R + 8 * c);
    }
    *reinterpret_cast<uint4*>(qs + r * KP + 8 * c) = v;
  }
  // one thread per interleaved pair (an odd last element passes unchanged); bf16 operands: the fast sin / cos
  const int npair = (a.sh.rot_dim + 1) / 2;
  for (int idx = tid; idx < ROWS * npair; idx += NT) {
    const int r = idx / npair, i = idx % npair, row = row0 + r;
    const bool two = 2 * i + 1 < a.sh.rot_dim;
    float v0 = 0.f, v1 = 0.f;
    if (row < nrows) {
      const int64_t t = q0 + row / H;
      const int64_t qr = t * a.q_stride + (int64_t)(row % H) * a.q_hstride;
      const float u = bf2f(qrot[qr + 2 * i]), w = two ? bf2f(qrot[qr + 2 * i + 1]) : 0.f;
      v0 = u;
      v1 = w;
      if (i < a.sh.rot_pairs) {
        float sn, cs;
        __sincosf((float)a.positions[t] * a.sh.inv_freq[i], &sn, &cs);
        v0 = u * cs - w * sn;
        v1 = w * cs + u * sn;
      }
    }
    qs[r * KP + R + 2 * i] = f2bf(v0);
    if (two) qs[r * KP + R + 2 * i + 1] = f2bf(v1);
  }

  const bool wave_live = row0 + wave * 32 < nrows;
  const int prow = rok ? (int)a.positions[q0 + myrow / H] : -1;
  constexpr float LOG2E = 1.4426950408889634f;
  const float sl2 = a.scale * LOG2E;
  const bool has_sink = a.sink != nullptr && rok && z == 0;
  float m = has_sink ? a.sink[myrow % H] * LOG2E : -1e30f;
  float l = has_sink ? 1.0f : 0.0f;
  f32x16_t o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;

  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;
  const int kch = Dk / 8, nkk = Dk / 16, nchunks = MKT * kch;
  // block-table entries of this workgroup's key range in LDS (visible after the loop's first barrier; the first
  // tile's loads read the table from global memory)
  int* btl = reinterpret_cast<int*>(ks + MKT * KP);
  const int b_lo = jlo / a.block_size, nbt = jhi / a.block_size - b_lo + 1;
  const bool bt_lds = nbt <= BT_LDS_MAX;
  if (bt_lds)
    for (int u = tid; u < nbt; u += NT) btl[u] = bt[b_lo + u];
  uint4 pf[NPF];
  auto fetch = [&](int j0, bool lds) {
#pragma unroll
    for (int u = 0; u < NPF; ++u) {
      const int idx = tid + u * NT;
      const int k = idx / kch, c = idx % kch, j = j0 + k;
      pf[u] = make_uint4(0, 0, 0, 0);
      if (idx < nchunks && j <= jhi) {
        const int jb = j / a.block_size;
        const int64_t blk = lds ? btl[jb - b_lo] : bt[jb];
        pf[u] = *reinterpret_cast<const uint4*>(cache + (blk * a.block_size + (j - jb * a.block_size)) * Dk + 8 * c);
      }
    }
  };
  fetch(jlo, false);
  const int pitchB = KP * 2;
  const int g16 = lane >> 4, i16 = lane & 15;
  const char* vbase = reinterpret_cast<const char*>(ks) + (4 * hh + (i16 >> 2)) * pitchB +
                      (16 * (g16 & 1) + 4 * (i16 & 3)) * 2;
  for (int j0 = jlo; j0 <= jhi; j0 += MKT) {
    __syncthreads();  // every wave is done with the previous tile (first: the queries are being written)
#pragma unroll
    for (int u = 0; u < NPF; ++u) {
      const int idx = tid + u * NT;
      if (idx < nchunks) *reinterpret_cast<uint4*>(ks + (idx / kch) * KP + 8 * (idx % kch)) = pf[u];
    }
    __syncthreads();
    if (j0 + MKT <= jhi) fetch(j0 + MKT, bt_lds);  // in flight while this tile is computed
    if (!wave_live) continue;
    f32x16_t sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
    const bf16_t* ka = ks + qcol * KP + 8 * hh;
    const bf16_t* qb = qs + (wave * 32 + qcol) * KP + 8 * hh;
    for (int kk = 0; kk < nkk; ++kk) {
      const bf16x8_t af = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(ka + 16 * kk));
      const bf16x8_t bfr = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(qb + 16 * kk));
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bfr, sc, 0, 0, 0);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = j0 + (r & 3) + 8 * (r >> 2) + 4 * hh;
      const bool valid = rok && j <= jhi && j <= prow && (a.window <= 0 || prow - j < a.window);
      const float v = valid ? sc[r] * sl2 : -INFINITY;
      sc[r] = v;
      mx = fmaxf(mx, v);
    }
    mx = xor32_max(mx);
    const float mn = fmaxf(m, mx);
    const float alpha = exp2f(m - mn);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pe = exp2f(sc[r] - mn);
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
  if (a.nsplit > 1) {
    float* wo = a.ws_o + ((int64_t)z * a.heads * a.total_q + orow) * R;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<float4*>(wo + 32 * db + 8 * g + 4 * hh) =
            make_float4(o[db][4 * g], o[db][4 * g + 1], o[db][4 * g + 2], o[db][4 * g + 3]);
    if (hh == 0) {
      a.ws_ml[((int64_t)z * a.heads * a.total_q + orow) * 2] = m;
      a.ws_ml[((int64_t)z * a.heads * a.total_q + orow) * 2 + 1] = l;
    }
    return;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  bf16_t* op = reinterpret_cast<bf16_t*>(a.out) + orow * R;
#pragma unroll
  for (int db = 0; db < NDB; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 w;
      w.x = pack2(o[db][4 * g + 0] * inv, o[db][4 * g + 1] * inv);
      w.y = pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
      *reinterpret_cast<uint2*>(op + 32 * db + 8 * g + 4 * hh) = w;
    }
  }
}

// out[row] = sum_z O_z 2^(m_z - m*) / sum_z l_z 2^(m_z - m*), m* = max_z m_z (running maxima in log2 units).
__global__ void __launch_bounds__(256) latent_attn_merge_kernel(bf16_t* out, const float* ws_o, const float* ws_ml,
                                                                int nsplit, int64_t rows, int R) {
  const int64_t row = blockIdx.x;
  float mstar = -1e30f;
  for (int z = 0; z < nsplit; ++z) mstar = fmaxf(mstar, ws_ml[((int64_t)z * rows + row) * 2]);
  float lsum = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float lz = ws_ml[((int64_t)z * rows + row) * 2 + 1];
    if (lz > 0.f) lsum += lz * exp2f(ws_ml[((int64_t)z * rows + row) * 2] - mstar);
  }
  const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
  for (int c = threadIdx.x; c < R; c += 256) {
    float acc = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float lz = ws_ml[((int64_t)z * rows + row) * 2 + 1];
      if (lz > 0.f) acc += ws_o[((int64_t)z * rows + row) * R + c] * exp2f(ws_ml[((int64_t)z * rows + row) * 2] - mstar);
    }
    out[row * R + c] = f2bf(acc * inv);
  }
}

inline size_t mfma_lds_bytes(int kp, int nw) {
  return sizeof(bf16_t) * (size_t)(32 * nw + MKT) * kp + sizeof(int) * BT_LDS_MAX;
}

template <int NDB, int NW> hipError_t launch_mfma(const LatentAttnArgs& a, hipStream_t s) {
  static bool attr_set = false;
  auto* fn = latent_attn_mfma_kernel<NDB, NW>;
  const int kp = a.sh.rank + a.sh.rot_dim + 8;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       144 * 1024);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const dim3 grid((unsigned)(((int64_t)a.max_q * a.heads + 32 * NW - 1) / (32 * NW)), (unsigned)a.num_seqs,
                  (unsigned)max(1, a.nsplit));
  hipLaunchKernelGGL(fn, grid, dim3(64 * NW), mfma_lds_bytes(kp, NW), s, a, kp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || a.nsplit <= 1) return e;
  hipLaunchKernelGGL(latent_attn_merge_kernel, dim3((unsigned)((int64_t)a.heads * a.total_q)), dim3(256), 0, s,
                     reinterpret_cast<bf16_t*>(a.out), a.ws_o, a.ws_ml, a.nsplit, (int64_t)a.heads * a.total_q,
                     a.sh.rank);
  return hipGetLastError();
}

inline bool mfma_ok(const LatentAttnArgs& a) {
  const int r = a.sh.rank;
  return !a.f32 && r % 32 == 0 && r <= 256 && a.sh.rot_dim % 16 == 0 && a.sh.rot_dim <= 128 &&
         (reinterpret_cast<uintptr_t>(a.q_lat) & 15) == 0 && (reinterpret_cast<uintptr_t>(a.cache) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.out) & 7) == 0;
}

template <int NW> hipError_t launch_mfma_ndb(const LatentAttnArgs& a, hipStream_t s) {
  switch (a.sh.rank / 32) {
    case 1: return launch_mfma<1, NW>(a, s);
    case 2: return launch_mfma<2, NW>(a, s);
    case 3: return launch_mfma<3, NW>(a, s);
    case 4: return launch_mfma<4, NW>(a, s);
    case 5: return launch_mfma<5, NW>(a, s);
    case 6: return launch_mfma<6, NW>(a, s);
    case 7: return launch_mfma<7, NW>(a, s);
    case 8: return launch_mfma<8, NW>(a, s);
  }
  return hipErrorInvalidValue;
}

// Prompt-sized steps at the common rotary widths (rot_dim = 16 * NROT, NROT = 0: no rotary part): the same algorithm with every wave's
// query fragments held in registers (loaded straight from global memory, the rotary part rotated on the way;
// no query tile in LDS, so the per-tile LDS traffic is the key tile alone) and the key tile double-buffered
// (one barrier per tile: the next tile's registers are stored into the other buffer after this tile's MFMAs).
template <int NDB, int NROT>
__global__ void __launch_bounds__(256) latent_attn_mfma_rq_kernel(LatentAttnArgs a, int KP) {
  constexpr int NT = 256, NKK = 2 * NDB + NROT, KCH = 4 * NDB + 2 * NROT, NCH = MKT * KCH;
  constexpr int NPF = (NCH + NT - 1) / NT;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  bf16_t* ks0 = reinterpret_cast<bf16_t*>(smem_raw);          // 2 x [MKT][KP]
  // Workgroups are dealt to the 8 XCDs round-robin by their linear id, and each XCD has its own L2: renumber so
  // that XCD k runs a contiguous eighth of the (sequence-major) tile list — the row tiles of one sequence share
  // that sequence's cache rows in ONE L2 instead of streaming every sequence through all eight
  int bx = blockIdx.x, by = blockIdx.y;
  {
    const unsigned total = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
    if (total % 8 == 0) {
      const unsigned nl = (lin % 8) * (total / 8) + lin / 8;
      bx = (int)(nl % gridDim.x);
      by = (int)(nl / gridDim.x);
    }
  }
  const int s = by, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tid = threadIdx.x;
  const int H = a.heads;
  constexpr int R = 32 * NDB, Dk = R + 16 * NROT;
  const int q0 = a.cu_q ? a.cu_q[s] : s;
  const int nq = a.cu_q ? a.cu_q[s + 1] - q0 : 1;
  const int nrows = nq * H, row0 = bx * 128;
  if (row0 >= nrows) return;
  const int ctx = a.ctx_lens[s];
  const int last_row = min(row0 + 128, nrows) - 1;
  const int p_first = (int)a.positions[q0 + row0 / H], p_last = (int)a.positions[q0 + last_row / H];
  const int jlo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int jhi = min(p_last, ctx - 1);
  const bf16_t* qlat = reinterpret_cast<const bf16_t*>(a.q_lat);
  const bf16_t* qrot = reinterpret_cast<const bf16_t*>(a.q_rot);
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(a.cache);
  const int qcol = lane & 31, hh = lane >> 5;
  const int myrow = row0 + wave * 32 + qcol;
  const bool rok = myrow < nrows;
  const bool wave_live = row0 + wave * 32 < nrows;
  const int64_t tq = rok ? q0 + myrow / H : 0;
  const int hq = rok ? myrow % H : 0;
  const int64_t orow = (int64_t)hq * a.total_q + tq;
  const int prow = rok ? (int)a.positions[tq] : -1;
  const int wrow_lo = row0 + wave * 32;
  const bool all_rows = wrow_lo + 31 < nrows;
  const int pw_min = wave_live ? (int)a.positions[q0 + wrow_lo / H] : 0;
  const int pw_max = wave_live ? (int)a.positions[q0 + min(wrow_lo + 31, nrows - 1) / H] : 0;

  // this lane's query fragments: qf[kk] = Q[row][16 kk + 8 hh .. + 8]
  bf16x8_t qf[NKK];
#pragma unroll
  for (int kk = 0; kk < 2 * NDB; ++kk) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (rok) v = *reinterpret_cast<const uint4*>(qlat + orow * R + 16 * kk + 8 * hh);
    qf[kk] = __builtin_bit_cast(bf16x8_t, v);
  }
#pragma unroll
  for (int kr = 0; kr < NROT; ++kr) {
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = 0.f;
    if (rok) {
      const bf16_t* qp = qrot + tq * a.q_stride + (int64_t)hq * a.q_hstride + 16 * kr + 8 * hh;
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        const int i = (16 * kr + 8 * hh) / 2 + pr;
        const float u = bf2f(qp[2 * pr]), w = bf2f(qp[2 * pr + 1]);
        if (i < a.sh.rot_pairs) {
          float sn, cs;
          __sincosf((float)prow * a.sh.inv_freq[i], &sn, &cs);
          f[2 * pr] = u * cs - w * sn;
          f[2 * pr + 1] = w * cs + u * sn;
        } else {
          f[2 * pr] = u;
          f[2 * pr + 1] = w;
        }
      }
    }
    qf[2 * NDB + kr] = __builtin_bit_cast(bf16x8_t, pack8(f));
  }

  constexpr float LOG2E = 1.4426950408889634f;
  const float sl2 = a.scale * LOG2E;
  const bool has_sink = a.sink != nullptr && rok;
  float m = has_sink ? a.sink[hq] * LOG2E : -1e30f;
  float l = has_sink ? 1.0f : 0.0f;
  f32x16_t o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;

  // the block-table entries of this workgroup's key range, staged in LDS: a key tile's loads then depend on an
  // LDS read, not on a second global round trip
  const int* bt = a.block_tables + (int64_t)s * a.bt_stride;
  int* btl = reinterpret_cast<int*>(ks0 + 2 * MKT * KP);
  const int b_lo = jlo / a.block_size, nbt = jhi / a.block_size - b_lo + 1;
  const bool bt_lds = nbt <= BT_LDS_MAX;
  if (bt_lds) {
    for (int u = tid; u < nbt; u += NT) btl[u] = bt[b_lo + u];
    __syncthreads();
  }
  uint4 pf[NPF];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int u = 0; u < NPF; ++u) {
      const int idx = tid + u * NT;
      const int k = idx / KCH, c = idx % KCH, j = j0 + k;
      pf[u] = make_uint4(0, 0, 0, 0);
      if (idx < NCH && j <= jhi) {
        const int jb = j / a.block_size;
        const int64_t blk = bt_lds ? btl[jb - b_lo] : bt[jb];
        pf[u] = *reinterpret_cast<const uint4*>(cache + (blk * a.block_size + (j - jb * a.block_size)) * Dk + 8 * c);
      }
    }
  };
  auto stash = [&](bf16_t* ks) {
#pragma unroll
    for (int u = 0; u < NPF; ++u) {
      const int idx = tid + u * NT;
      if (idx < NCH) *reinterpret_cast<uint4*>(ks + (idx / KCH) * KP + 8 * (idx % KCH)) = pf[u];
    }
  };
  fetch(jlo);
  stash(ks0);
  if (jlo + MKT <= jhi) fetch(jlo + MKT);
  const int pitchB = KP * 2;
  const int g16 = lane >> 4, i16 = lane & 15;
  const int voff = (4 * hh + (i16 >> 2)) * pitchB + (16 * (g16 & 1) + 4 * (i16 & 3)) * 2;
  int cur = 0;
  for (int j0 = jlo; j0 <= jhi; j0 += MKT, cur ^= 1) {
    __syncthreads();  // tile j0 is complete in buffer cur; every wave has left the other buffer
    bf16_t* ks = ks0 + cur * (MKT * KP);
    if (wave_live) {
      f32x16_t sc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 0.f;
      const bf16_t* ka = ks + qcol * KP + 8 * hh;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        const bf16x8_t af = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(ka + 16 * kk));
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, qf[kk], sc, 0, 0, 0);
      }
      float mx = -INFINITY;
      // interior tiles (every key visible to every row of the wave) skip the per-score mask
      if (all_rows && j0 + MKT - 1 <= min(pw_min, jhi) && (a.window <= 0 || pw_max - j0 < a.window)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sc[r] *= sl2;
          mx = fmaxf(mx, sc[r]);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = j0 + (r & 3) + 8 * (r >> 2) + 4 * hh;
          const bool valid = rok && j <= jhi && j <= prow && (a.window <= 0 || prow - j < a.window);
          const float v = valid ? sc[r] * sl2 : -INFINITY;
          sc[r] = v;
          mx = fmaxf(mx, v);
        }
      }
      mx = xor32_max(mx);
      const float mn = fmaxf(m, mx);
      const float alpha = __builtin_amdgcn_exp2f(m - mn);
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
      const char* vbase = reinterpret_cast<const char*>(ks) + voff;
      const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0;  // wave-uniform: most tiles keep the max
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        if (rescale) {
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
    if (j0 + MKT <= jhi) {
      stash(ks0 + (cur ^ 1) * (MKT * KP));           // tile j0 + 32 (fetched one iteration ago) -> the other buffer
      if (j0 + 2 * MKT <= jhi) fetch(j0 + 2 * MKT);  // in flight during the next tile's MFMAs
    }
  }
  if (!rok) return;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  bf16_t* op = reinterpret_cast<bf16_t*>(a.out) + orow * R;
#pragma unroll
  for (int db = 0; db < NDB; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 w;
      w.x = pack2(o[db][4 * g + 0] * inv, o[db][4 * g + 1] * inv);
      w.y = pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
      *reinterpret_cast<uint2*>(op + 32 * db + 8 * g + 4 * hh) = w;
    }
  }
}

template <int NDB, int NROT> hipError_t launch_mfma_rq(const LatentAttnArgs& a, hipStream_t s) {
  static bool attr_set = false;
  auto* fn = latent_attn_mfma_rq_kernel<NDB, NROT>;
  const int kp = a.sh.rank + a.sh.rot_dim + 8;
  const size_t lds = sizeof(bf16_t) * (size_t)2 * MKT * kp + sizeof(int) * BT_LDS_MAX;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       64 * 1024);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const dim3 grid((unsigned)(((int64_t)a.max_q * a.heads + 127) / 128), (unsigned)a.num_seqs);
  hipLaunchKernelGGL(fn, grid, dim3(256), lds, s, a, kp);
  return hipGetLastError();
}

// the register-query kernel exists for rank in {64, 128, 256} x rot_dim in {0, 16, 32, 64}; unsplit steps only
inline bool mfma_rq_ok(const LatentAttnArgs& a) {
  const int r = a.sh.rank, t = a.sh.rot_dim;
  return a.nsplit <= 1 && (int64_t)a.max_q * a.heads > 32 && (r == 64 || r == 128 || r == 256) &&
         (t == 0 || t == 16 || t == 32 || t == 64);
}

template <int NDB> hipError_t launch_mfma_rq_rot(const LatentAttnArgs& a, hipStream_t s) {
  switch (a.sh.rot_dim) {
    case 0: return launch_mfma_rq<NDB, 0>(a, s);   // no rotary part: latents without positions
    case 16: return launch_mfma_rq<NDB, 1>(a, s);
    case 32: return launch_mfma_rq<NDB, 2>(a, s);
    case 64: return launch_mfma_rq<NDB, 4>(a, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_mfma_rq_any(const LatentAttnArgs& a, hipStream_t s) {
  switch (a.sh.rank) {
    case 64: return launch_mfma_rq_rot<2>(a, s);
    case 128: return launch_mfma_rq_rot<4>(a, s);
    case 256: return launch_mfma_rq_rot<8>(a, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_mfma_any(const LatentAttnArgs& a, hipStream_t s) {
  if (a.impl != 3 && mfma_rq_ok(a)) return launch_mfma_rq_any(a, s);
  // one wave per workgroup when a sequence brings at most 32 rows (decode steps): small LDS, many workgroups
  return (int64_t)a.max_q * a.heads <= 32 ? launch_mfma_ndb<1>(a, s) : launch_mfma_ndb<4>(a, s);
}

constexpr int LDS_MAX = 128 * 1024;

inline size_t lds_bytes(int bk, int qs, int ksd) { return sizeof(float) * ((size_t)RW * qs + (size_t)bk * ksd + (size_t)RW * bk); }

template <int BK, int CC, bool F32>
hipError_t launch_one(const LatentAttnArgs& a, int qs, int ksd, dim3 grid, hipStream_t s) {
  static bool attr_set = false;  // once per instantiation; hipFuncSetAttribute is not a stream operation
  auto* fn = latent_attn_kernel<BK, CC, F32>;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       LDS_MAX);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(fn, grid, dim3(256), lds_bytes(BK, qs, ksd), s, a, qs, ksd);
  return hipGetLastError();
}

template <int BK, bool F32>
hipError_t launch_cc(const LatentAttnArgs& a, int qs, int ksd, dim3 grid, hipStream_t s) {
  const int r = a.sh.rank;
  if (r <= 128) return launch_one<BK, 2, F32>(a, qs, ksd, grid, s);
  if (r <= 512) return launch_one<BK, 8, F32>(a, qs, ksd, grid, s);
  if (r <= 1024) return launch_one<BK, 16, F32>(a, qs, ksd, grid, s);
  return hipErrorInvalidValue;
}

template <bool F32> hipError_t launch_bk(const LatentAttnArgs& a, hipStream_t s) {
  const int dk = a.sh.rank + a.sh.rot_dim;
  const int qs = (dk + 3) & ~3, ksd = dk | 1;
  const dim3 grid((unsigned)(((int64_t)a.max_q * a.heads + RW - 1) / RW), (unsigned)a.num_seqs);
  if (lds_bytes(64, qs, ksd) <= 64 * 1024) return launch_cc<64, F32>(a, qs, ksd, grid, s);
  if (lds_bytes(32, qs, ksd) <= LDS_MAX) return launch_cc<32, F32>(a, qs, ksd, grid, s);
  if (lds_bytes(16, qs, ksd) <= LDS_MAX) return launch_cc<16, F32>(a, qs, ksd, grid, s);
  return hipErrorInvalidValue;
}

}  // namespace

bool latent_attn_uses_mfma(const LatentAttnArgs& a) { return a.impl != 1 && mfma_ok(a); }

hipError_t launch_latent_attn(const LatentAttnArgs& a, hipStream_t s) {
  if (a.num_seqs == 0 || a.total_q == 0) return hipSuccess;
  if (a.heads < 1 || a.sh.rank < 1 || a.sh.rot_dim < 0 || a.sh.rot_pairs * 2 > a.sh.rot_dim || a.block_size < 1 ||
      a.max_q < 1)
    return hipErrorInvalidValue;
  if (a.impl != 1 && mfma_ok(a)) return launch_mfma_any(a, s);
  if (a.impl >= 2) return hipErrorInvalidValue;  // the matrix-core form was demanded and does not apply
  return a.f32 ? launch_bk<true>(a, s) : launch_bk<false>(a, s);
}

}  // namespace die
