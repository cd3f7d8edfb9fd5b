// Latent attention over a paged cache that holds, per token, one row [latent c (kv_rank) | rotated key part (rot_dim)]
// shared by all heads.  Queries arrive in absorbed form: for head h the first kv_rank numbers are W_uk[h]^T q_unrotated
// (so that their product with c equals q_unrotated . (W_uk[h] c)), the last rot_dim are the rotated query part.  The
// kernel returns sum_j p_j c_j per head; the caller applies W_uv[h] afterwards.  Every head of a token reads the same
// key rows, so a workgroup stages a tile of them in LDS once and serves all its heads from it.
//
//   nv_latent_kv_store : RMS norm of the latent, rotation of the shared key part, store into the token's cache row
//   nv_latent_q_rope   : rotation of the per-head query parts into the absorbed-query buffer
//   nv_latent_attn     : sliding-window softmax attention, one workgroup per (token, group of heads)
//   nv_latent_gather, nv_latent_expand, nv_latent_q_rows : the pieces of the EXPANDED form that long prompt portions
//                        take: the step's requests' cache rows gathered in order, keys and values of every head written
//                        out from their up-projections, whole query rows; ordinary paged attention reads the result
//
// Rotation: dimension i pairs with i + dims/2 ("rotate half"), or with `interleaved` dimension 2i with 2i + 1; the angle
// is position * inv_freq[i] in fp32, and both cosine and sine are multiplied by `mscale` (the caller folds frequency
// scaling into inv_freq and mscale).
#include "anyt.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_store_kernel(const float* __restrict__ kv, int64_t kv_rs,
                                                              const T* __restrict__ norm_w,
                                                              const int64_t* __restrict__ positions,
                                                              const float* __restrict__ inv_freq, float mscale,
                                                              const int32_t* __restrict__ slot_mapping,
                                                              T* __restrict__ cache, int rank, int rot_dim, int rot_dims,
                                                              float eps, int interleaved) {
  __shared__ float red[32];
  const int64_t t = blockIdx.x;
  const int32_t slot = slot_mapping[t];
  const float* row = kv + t * kv_rs;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) ss += row[j] * row[j];
  ss = block_sum(ss, red);
  if (slot < 0) return;
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  T* dst = cache + (int64_t)slot * (rank + rot_dim);
  for (int j = threadIdx.x; j < rank; j += blockDim.x) st_f32<T>(dst + j, row[j] * inv * ld_f32<T>(norm_w + j));
  const float pos = (float)positions[t];
  const int half = rot_dims / 2;
  for (int j = threadIdx.x; j < rot_dim; j += blockDim.x) {
    float v = row[rank + j];
    if (j < rot_dims) {
      const bool first = interleaved ? (j & 1) == 0 : j < half;
      const int i = interleaved ? j >> 1 : (first ? j : j - half);
      const float a = pos * inv_freq[i];
      const float cs = cosf(a) * mscale, sn = sinf(a) * mscale;
      const float other = row[rank + (interleaved ? j ^ 1 : (first ? j + half : j - half))];
      v = first ? v * cs - other * sn : v * cs + other * sn;
    }
    st_f32<T>(dst + rank + j, v);
  }
}

// q [tokens, H * (dim + rot_dim)] in storage type -> qa[t, h, rank .. rank + rot_dim) fp32, rotated
template <typename T>
__global__ __launch_bounds__(256) void latent_q_rope_kernel(const T* __restrict__ q, int64_t q_rs,
                                                            const int64_t* __restrict__ positions,
                                                            const float* __restrict__ inv_freq, float mscale,
                                                            float* __restrict__ qa, int H, int dim, int rot_dim,
                                                            int rot_dims, int rank, int interleaved, int copy_front,
                                                            float factor) {
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = rot_dims / 2;
  if (copy_front)          // the unrotated numbers in front of the rotated ones (rank == dim): a whole query row
    for (int idx = threadIdx.x; idx < H * dim; idx += blockDim.x) {
      const int h = idx / dim, j = idx % dim;
      qa[(t * H + h) * (rank + rot_dim) + j] = ld_f32<T>(q + t * q_rs + (int64_t)h * (dim + rot_dim) + j) * factor;
    }
  for (int idx = threadIdx.x; idx < H * rot_dim; idx += blockDim.x) {
    const int h = idx / rot_dim, j = idx % rot_dim;
    const T* src = q + t * q_rs + (int64_t)h * (dim + rot_dim) + dim;
    float v = ld_f32<T>(src + j);
    if (j < rot_dims) {
      const bool first = interleaved ? (j & 1) == 0 : j < half;
      const int i = interleaved ? j >> 1 : (first ? j : j - half);
      const float a = pos * inv_freq[i];
      const float cs = cosf(a) * mscale, sn = sinf(a) * mscale;
      const float other = ld_f32<T>(src + (interleaved ? j ^ 1 : (first ? j + half : j - half)));
      v = first ? v * cs - other * sn : v * cs + other * sn;
    }
    qa[(t * H + h) * (rank + rot_dim) + rank + j] = v * factor;
  }
}

// The cache rows of every request of a step, in order of position, into one buffer: request b's row j goes to row
// cu_k[b] + j (cu_k: starts padded to whole blocks; rows past the request's end are zero).
template <typename T>
__global__ __launch_bounds__(256) void latent_gather_kernel(const T* __restrict__ cache, const int32_t* __restrict__ tables,
                                                            int table_cols, const int32_t* __restrict__ cu_k,
                                                            const int32_t* __restrict__ cu_q,
                                                            const int32_t* __restrict__ past, int B, int block_size,
                                                            int Dk, T* __restrict__ out) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= cu_k[B]) return;
  const int lane = threadIdx.x & 63;
  int b = 0;
  while (b + 1 < B && row >= cu_k[b + 1]) ++b;
  const int j = (int)(row - cu_k[b]);
  const int len = past[b] + cu_q[b + 1] - cu_q[b];
  T* dst = out + row * Dk;
  if (j >= len) {
    for (int e = lane; e < Dk; e += 64) dst[e] = (T)0.0f;
    return;
  }
  const T* src = cache + ((int64_t)tables[(int64_t)b * table_cols + j / block_size] * block_size + j % block_size) * Dk;
  for (int e = lane; e < Dk; e += 64) dst[e] = src[e];
}

// Expanded key/value rows [k: H * (dim + rot_dim) | v: H * vdim] from the up-projections kv [rows, H * dim | H * vdim]
// and the gathered cache rows c [rows, rank + rot_dim]: head h's key is [W_uk[h] c | the shared rotated part].
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_kernel(const T* __restrict__ kv, const T* __restrict__ c,
                                                            T* __restrict__ out, int H, int dim, int rot_dim, int vdim,
                                                            int rank) {
  const int64_t row = blockIdx.x;
  const int dk = dim + rot_dim, kw = H * dk, vw = H * vdim;
  const T* kvr = kv + row * (H * dim + vw);
  const T* rot = c + row * (rank + rot_dim) + rank;
  T* dst = out + row * (kw + vw);
  for (int i = threadIdx.x; i < kw; i += blockDim.x) {
    const int h = i / dk, e = i % dk;
    dst[i] = e < dim ? kvr[h * dim + e] : rot[e - dim];
  }
  for (int i = threadIdx.x; i < vw; i += blockDim.x) dst[kw + i] = kvr[H * dim + i];
}

struct AttnArgs {
  const float* qa;         // [tokens, H, rank + rot_dim]
  const void* cache;       // [rows, rank + rot_dim]
  const int32_t* tables;   // [B, table_cols]
  int table_cols;
  const int32_t* cu_q;     // [B + 1]
  const int32_t* past;     // [B]
  const int32_t* seq_of;   // [tokens] request index of each token
  void* out;               // [tokens, H, rank]
  int H, rank, rot_dim, block_size, window, HC, TK;
  float scale;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_kernel(AttnArgs p) {
  extern __shared__ float lds[];
  const int Dk = p.rank + p.rot_dim, Dp = Dk + 1;
  const int HC = p.HC, TK = p.TK;
  float* sq = lds;                    // [HC][Dk]
  float* skey = sq + HC * Dk;         // [TK][Dp]
  float* sc = skey + TK * Dp;         // [HC][TK]
  float* acc = sc + HC * TK;          // [HC][rank]
  float* sm = acc + HC * p.rank;      // [HC] running maximum
  float* sl = sm + HC;                // [HC] running sum
  float* scorr = sl + HC;             // [HC]
  const int t = blockIdx.y, h0 = blockIdx.x * HC;
  const int nh = min(HC, p.H - h0);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int b = p.seq_of[t];
  const int pos = p.past[b] + (t - p.cu_q[b]);
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int32_t* table = p.tables + (int64_t)b * p.table_cols;
  const T* cache = reinterpret_cast<const T*>(p.cache);

  for (int i = tid; i < nh * Dk; i += 256) sq[i] = p.qa[((int64_t)t * p.H + h0) * Dk + i];
  for (int i = tid; i < nh * p.rank; i += 256) acc[i] = 0.0f;
  if (tid < nh) {
    sm[tid] = -INFINITY;
    sl[tid] = 0.0f;
  }
  __syncthreads();
  for (int j0 = lo; j0 <= pos; j0 += TK) {
    const int nk = min(TK, pos + 1 - j0);
    for (int i = tid; i < nk * Dk; i += 256) {
      const int j = i / Dk, e = i % Dk;
      const int kp = j0 + j;
      const int64_t row = (int64_t)table[kp / p.block_size] * p.block_size + kp % p.block_size;
      skey[j * Dp + e] = ld_f32<T>(cache + row * Dk + e);
    }
    __syncthreads();
    for (int i = tid; i < nh * TK; i += 256) {
      const int h = i / TK, j = i % TK;
      float s = -INFINITY;
      if (j < nk) {
        s = 0.0f;
        const float* qv = sq + h * Dk;
        const float* kv = skey + j * Dp;
        for (int e = 0; e < Dk; ++e) s += qv[e] * kv[e];
        s *= p.scale;
      }
      sc[h * TK + j] = s;
    }
    __syncthreads();
    for (int h = wv; h < nh; h += 4) {
      float m = -INFINITY;
      for (int j = lane; j < TK; j += 64) m = fmaxf(m, sc[h * TK + j]);
      m = wave_max(m);
      const float m_old = sm[h];
      const float m_new = fmaxf(m_old, m);
      float sum = 0.0f;
      for (int j = lane; j < TK; j += 64) {
        const float e = (j < nk) ? expf(sc[h * TK + j] - m_new) : 0.0f;
        sc[h * TK + j] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float corr = expf(m_old - m_new);   // exp(-inf) = 0 at the first tile
        scorr[h] = corr;
        sm[h] = m_new;
        sl[h] = sl[h] * corr + sum;
      }
    }
    __syncthreads();
    for (int i = tid; i < nh * p.rank; i += 256) {
      const int h = i / p.rank, e = i % p.rank;
      float a = acc[i] * scorr[h];
      const float* pv = sc + h * TK;
      for (int j = 0; j < nk; ++j) a += pv[j] * skey[j * Dp + e];
      acc[i] = a;
    }
    __syncthreads();
  }
  T* out = reinterpret_cast<T*>(p.out);
  for (int i = tid; i < nh * p.rank; i += 256) {
    const int h = i / p.rank;
    st_f32<T>(out + ((int64_t)t * p.H + h0) * p.rank + i, acc[i] / sl[h]);
  }
}


// ---- the same attention on the matrix cores (bf16 cache) ----
// A workgroup owns 16 query rows: TQ consecutive tokens of one request times HQ heads (HQ * TQ = 16), which all read
// the same key rows.  Per tile of 64 keys: the rows are staged in LDS twice (row-major for S = Q K^T, transposed for
// O += P V), wavefront w computes the scores of keys 16 w .. 16 w + 15, the softmax statistics are updated by
// 16 threads per row, and every wavefront accumulates its share of the output columns.  Scores, maxima, sums and the
// rescaling are fp32.  Queries and softmax weights enter the MFMAs as the sum of two bf16 numbers (value = hi + lo,
// two MFMAs), so neither is rounded to 8 bits of mantissa; the cached rows are bf16 as stored.
// KEYS rows per tile: 64, or 32 where 64 would not fit the LDS beside wide latents (then two wavefronts compute scores)

struct MfmaAttnArgs {
  AttnArgs a;
  int B, HQ, TQ, Dkp;
  int ksplit;              // workgroups that share a tile's keys (blockIdx.z), each walking every ksplit-th key tile;
  float* partial;          // > 1: their unnormalised shares go to [tokens, H, ksplit, rank + 2] (then maximum and sum)
};

template <int NTILE, int KEYS>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(MfmaAttnArgs q) {
  constexpr int ATT_KEYS = KEYS, ATT_PST = KEYS + 8, ATT_SST = KEYS + 4, KPT = KEYS / 16;
  extern __shared__ u32x4 lds_raw[];
  const AttnArgs& p = q.a;
  const int Dk = p.rank + p.rot_dim, R = p.rank, Dq = q.Dkp + 8;
  bf16_t* sQhi = reinterpret_cast<bf16_t*>(lds_raw);
  bf16_t* sQlo = sQhi + 16 * Dq;
  bf16_t* sK = sQlo + 16 * Dq;
  bf16_t* sVt = sK + ATT_KEYS * Dq;
  bf16_t* sPhi = sVt + R * ATT_PST;
  bf16_t* sPlo = sPhi + 16 * ATT_PST;
  float* sS = reinterpret_cast<float*>(sPlo + 16 * ATT_PST);
  float* sm = sS + 2 * 16 * ATT_SST;      // two score tiles: the second holds the other feature half (32-key tiles)
  float* sl = sm + 16;
  float* scorr = sl + 16;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, c = lane & 15, g = lane >> 4;

  // which request and which of its tokens this tile covers
  int b = 0, before = 0, tstart = 0, tcount = 0;
  for (; b < q.B; ++b) {
    const int len = p.cu_q[b + 1] - p.cu_q[b];
    const int tiles = (len + q.TQ - 1) / q.TQ;
    if ((int)blockIdx.y < before + tiles) {
      tstart = p.cu_q[b] + ((int)blockIdx.y - before) * q.TQ;
      tcount = min(q.TQ, p.cu_q[b + 1] - tstart);
      break;
    }
    before += tiles;
  }
  if (b == q.B) return;
  const int h0 = blockIdx.x * q.HQ;
  const int pos0 = p.past[b] + (tstart - p.cu_q[b]);
  const int kmax = pos0 + tcount - 1;
  const int kmin = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int32_t* table = p.tables + (int64_t)b * p.table_cols;
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(p.cache);

  for (int i = tid; i < ATT_KEYS * Dq; i += 256) sK[i] = (bf16_t)0.0f;       // the padding columns stay zero
  for (int i = tid; i < 16 * Dq; i += 256) {
    const int r = i / Dq, f = i % Dq;
    const int tq = r / q.HQ, hh = h0 + r % q.HQ;
    float v = 0.0f;
    if (tq < tcount && hh < p.H && f < Dk) v = p.qa[((int64_t)(tstart + tq) * p.H + hh) * Dk + f];
    const bf16_t hi = (bf16_t)v;
    sQhi[i] = hi;
    sQlo[i] = (bf16_t)(v - (float)hi);
  }
  if (tid < 16) {
    sm[tid] = -INFINITY;
    sl[tid] = 0.0f;
  }
  f32x4 O[NTILE];
#pragma unroll
  for (int n = 0; n < NTILE; ++n) O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the row this thread serves in the softmax step
  const int srow = tid >> 4, skq = tid & 15;
  const int s_tq = srow / q.HQ, s_hh = h0 + srow % q.HQ;
  const bool s_valid = s_tq < tcount && s_hh < p.H;
  const int s_pos = pos0 + s_tq;
  const int s_lo = p.window > 0 ? max(0, s_pos - p.window + 1) : 0;
  const int chunks = Dk / 8;
  __syncthreads();

  // Key rows travel memory -> registers -> LDS; the loads of the NEXT tile are issued before this tile is multiplied,
  // so their latency hides behind the MFMAs.  Consecutive threads take consecutive keys (conflict-free transposed
  // stores).  NCH bounds the 16-byte pieces per thread and tile (the launcher checks it).
  constexpr int NCH = 10;
  const int pieces = ATT_KEYS * chunks;
  u32x4 stage[NCH];
  auto fetch_tile = [&](int j0) {
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
      const int i = tid + u * 256;
      const int key = i % ATT_KEYS, f8 = i / ATT_KEYS;
      const int kp = j0 + key;
      stage[u] = u32x4{0u, 0u, 0u, 0u};
      if (i < pieces && kp <= kmax) {
        const int64_t row = (int64_t)table[kp / p.block_size] * p.block_size + kp % p.block_size;
        stage[u] = *reinterpret_cast<const u32x4*>(cache + row * Dk + f8 * 8);
      }
    }
  };
  const int kstep = q.ksplit * ATT_KEYS;
  fetch_tile(kmin + (int)blockIdx.z * ATT_KEYS);
  for (int j0 = kmin + (int)blockIdx.z * ATT_KEYS; j0 <= kmax; j0 += kstep) {
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
      const int i = tid + u * 256;
      const int key = i % ATT_KEYS, f8 = i / ATT_KEYS;
      if (i >= pieces) continue;
      *reinterpret_cast<u32x4*>(sK + key * Dq + f8 * 8) = stage[u];
      if (f8 * 8 < R) {
        const uint16_t* e16 = reinterpret_cast<const uint16_t*>(&stage[u]);
        uint16_t* dst = reinterpret_cast<uint16_t*>(sVt) + (f8 * 8) * ATT_PST + key;
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e * ATT_PST] = e16[e];
      }
    }
    __syncthreads();
    if (j0 + kstep <= kmax) fetch_tile(j0 + kstep);
    // S = Q K^T: with 64 keys wavefront w takes keys 16 w ..; with 32 keys the wavefront pairs (0, 1) and (2, 3) take
    // the two halves of the feature dimension and their partial scores are summed in the softmax step
    {
      constexpr int KW = ATT_KEYS / 16;             // wavefronts one pass over the keys needs
      constexpr int PARTS = 4 / KW;                 // feature ranges (1 or 2)
      const int kw = wv % KW, part = wv / KW;
      const int steps = q.Dkp / 32;
      const int f_lo = (steps * part) / PARTS * 32, f_hi = (steps * (part + 1)) / PARTS * 32;
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* krow = sK + (16 * kw + c) * Dq + 8 * g;
      const bf16_t* qhi = sQhi + c * Dq + 8 * g;
      const bf16_t* qlo = sQlo + c * Dq + 8 * g;
      for (int ks = f_lo; ks < f_hi; ks += 32) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(krow + ks);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(qhi + ks), kf, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(qlo + ks), kf, acc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) sS[part * 16 * ATT_SST + (4 * g + r) * ATT_SST + 16 * kw + c] = acc[r] * p.scale;
    }
    __syncthreads();
    // softmax statistics: 16 threads per row, KEYS / 16 keys each
    {
      float sv[KPT], m = -INFINITY;
#pragma unroll
      for (int e = 0; e < KPT; ++e) {
        const int kp = j0 + KPT * skq + e;
        const bool ok = s_valid && kp >= s_lo && kp <= s_pos;
        sv[e] = -INFINITY;
        if (ok) {
          sv[e] = sS[srow * ATT_SST + KPT * skq + e];
          if constexpr (ATT_KEYS == 32) sv[e] += sS[16 * ATT_SST + srow * ATT_SST + KPT * skq + e];
        }
        m = fmaxf(m, sv[e]);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
      const float m_old = sm[srow];
      const float m_new = fmaxf(m_old, m);
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < KPT; ++e) {
        const float pe = (sv[e] == -INFINITY) ? 0.0f : expf(sv[e] - m_new);
        sum += pe;
        const bf16_t hi = (bf16_t)pe;
        sPhi[srow * ATT_PST + KPT * skq + e] = hi;
        sPlo[srow * ATT_PST + KPT * skq + e] = (bf16_t)(pe - (float)hi);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
      if (skq == 0) {
        const float corr = (m_new == -INFINITY) ? 1.0f : expf(m_old - m_new);
        scorr[srow] = corr;
        sm[srow] = m_new;
        sl[srow] = sl[srow] * corr + sum;
      }
    }
    __syncthreads();
    // O = O * corr + P V for this wavefront's output columns
#pragma unroll
    for (int n = 0; n < NTILE; ++n) {
      const int col0 = 16 * (wv * NTILE + n);
      if (col0 < R) {
#pragma unroll
        for (int r = 0; r < 4; ++r) O[n][r] *= scorr[4 * g + r];
#pragma unroll
        for (int ks = 0; ks < ATT_KEYS; ks += 32) {
          const bf16x8 vf = *reinterpret_cast<const bf16x8*>(sVt + (col0 + c) * ATT_PST + ks + 8 * g);
          O[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              *reinterpret_cast<const bf16x8*>(sPhi + c * ATT_PST + ks + 8 * g), vf, O[n], 0, 0, 0);
          O[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              *reinterpret_cast<const bf16x8*>(sPlo + c * ATT_PST + ks + 8 * g), vf, O[n], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
  bf16_t* out = reinterpret_cast<bf16_t*>(p.out);
  if (q.ksplit > 1) {          // another launch joins the shares
    const int PW = R + 2;
#pragma unroll
    for (int n = 0; n < NTILE; ++n) {
      const int col = 16 * (wv * NTILE + n) + c;
      if (col >= R) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 4 * g + r;
        const int tq = row / q.HQ, hh = h0 + row % q.HQ;
        if (tq < tcount && hh < p.H)
          q.partial[(((int64_t)(tstart + tq) * p.H + hh) * q.ksplit + blockIdx.z) * PW + col] = O[n][r];
      }
    }
    if (tid < 16) {
      const int tq = tid / q.HQ, hh = h0 + tid % q.HQ;
      if (tq < tcount && hh < p.H) {
        float* dst = q.partial + (((int64_t)(tstart + tq) * p.H + hh) * q.ksplit + blockIdx.z) * PW + R;
        dst[0] = sm[tid];
        dst[1] = sl[tid];
      }
    }
    return;
  }
#pragma unroll
  for (int n = 0; n < NTILE; ++n) {
    const int col = 16 * (wv * NTILE + n) + c;
    if (col >= R) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * g + r;
      const int tq = row / q.HQ, hh = h0 + row % q.HQ;
      if (tq < tcount && hh < p.H) out[((int64_t)(tstart + tq) * p.H + hh) * R + col] = (bf16_t)(O[n][r] / sl[row]);
    }
  }
}

// joins the shares of the ksplit (at most 32) workgroups that walked one (token, head)'s keys: one workgroup per row,
// the shares' weights exp(m_z - m) / l first, then every thread sums its columns over the shares
__global__ __launch_bounds__(256) void latent_attn_join_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                                                               int ksplit, int R) {
  __shared__ float wz[32];
  const int64_t row = blockIdx.x;
  const int PW = R + 2;
  const float* src = partial + row * ksplit * PW;
  if (threadIdx.x < 64) {
    const int z = threadIdx.x;
    const float mz = z < ksplit ? src[z * PW + R] : -INFINITY;
    const float lz = z < ksplit ? src[z * PW + R + 1] : 0.0f;
    const float m = wave_max(mz);
    const float f = mz == -INFINITY ? 0.0f : __expf(mz - m);
    const float l = wave_sum(lz * f);
    if (z < 32) wz[z] = f / l;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < R; e += 256) {
    float o = 0.0f;
#pragma unroll 8
    for (int z = 0; z < ksplit; ++z) o += src[z * PW + e] * wz[z];
    out[row * R + e] = (bf16_t)o;
  }
}

template <int NTILE, int KEYS>
hipError_t launch_mfma_attn(const MfmaAttnArgs& q, dim3 grid, size_t lds, hipStream_t s) {
  static size_t allowed = 64 * 1024;
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_mfma_kernel<NTILE, KEYS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    allowed = lds;
  }
  latent_attn_mfma_kernel<NTILE, KEYS><<<grid, dim3(256), lds, s>>>(q);
  return hipSuccess;
}

}  // namespace

extern "C" int nv_latent_kv_store(const float* kv, int64_t kv_row_stride, const void* norm_w, const int64_t* positions,
                                  const float* inv_freq, float mscale, const int32_t* slot_mapping, void* cache,
                                  int64_t tokens, int rank, int rot_dim, int rot_dims, int interleaved, float eps,
                                  int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(kv && norm_w && positions && inv_freq && slot_mapping && cache, "nv_latent_kv_store: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_kv_store: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && rank > 0 && rot_dim >= 0 && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0,
               "nv_latent_kv_store: bad shape rank=%d rot_dim=%d rot_dims=%d", rank, rot_dim, rot_dims);
  if (tokens == 0) return NV_OK;
  NV_DISPATCH_T(dtype, latent_kv_store_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           kv, kv_row_stride, (const T*)norm_w, positions, inv_freq, mscale, slot_mapping, (T*)cache,
                           rank, rot_dim, rot_dims, eps, interleaved));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_latent_q_rope(const void* q, int64_t q_row_stride, const int64_t* positions, const float* inv_freq,
                                float mscale, float* qa, int64_t tokens, int heads, int dim, int rot_dim, int rot_dims,
                                int interleaved, int rank, int dtype, nv_stream_t stream) {
  return nv_latent_q_rows(q, q_row_stride, positions, inv_freq, mscale, qa, tokens, heads, dim, rot_dim, rot_dims,
                          interleaved, rank, 0, 1.0f, dtype, stream);
}

extern "C" int nv_latent_q_rows(const void* q, int64_t q_row_stride, const int64_t* positions, const float* inv_freq,
                                float mscale, float* qa, int64_t tokens, int heads, int dim, int rot_dim, int rot_dims,
                                int interleaved, int rank, int copy_front, float factor, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(!copy_front || rank == dim, "nv_latent_q_rows: whole query rows have the unrotated numbers in front");
  NV_CHECK_ARG(q && positions && inv_freq && qa, "nv_latent_q_rope: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_q_rope: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && heads > 0 && dim >= 0 && rot_dim >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0 && rank > 0,
               "nv_latent_q_rope: bad shape");
  if (tokens == 0 || (rot_dim == 0 && !copy_front)) return NV_OK;
  NV_DISPATCH_T(dtype, latent_q_rope_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           (const T*)q, q_row_stride, positions, inv_freq, mscale, qa, heads, dim, rot_dim, rot_dims, rank,
                           interleaved, copy_front, factor));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

// Workgroups that share one decoded token's keys: enough to put about 256 workgroups on the chip, at most 32.  A
// function of the launch shape alone (not of the contexts), so a captured launch stays valid as contexts grow.
static int latent_attn_key_splits(int64_t tokens, int heads) {
  const int64_t groups = tokens * ((heads + 15) / 16);
  int k = 1;
  while (k < 32 && groups * k * 2 <= 512) k *= 2;
  return k;
}

extern "C" size_t nv_latent_attn_workspace_bytes(int64_t tokens, int max_q, int heads, int rank) {
  if (max_q != 1 || tokens <= 0) return 0;
  const int k = latent_attn_key_splits(tokens, heads);
  return k > 1 ? (size_t)tokens * heads * k * (rank + 2) * sizeof(float) : 0;
}

extern "C" int nv_latent_attn(const float* qa, const void* cache, const int32_t* block_tables, int table_cols,
                              const int32_t* cu_q, const int32_t* past_lens, const int32_t* seq_of_token, void* out,
                              int64_t tokens, int num_seqs, int heads, int rank, int rot_dim, int block_size, int window, float scale,
                              int dtype, nv_stream_t stream) {
  return nv_latent_attn_split(qa, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, tokens, num_seqs,
                              heads, rank, rot_dim, block_size, window, scale, 0, nullptr, 0, dtype, stream);
}

extern "C" int nv_latent_attn_split(const float* qa, const void* cache, const int32_t* block_tables, int table_cols,
                                    const int32_t* cu_q, const int32_t* past_lens, const int32_t* seq_of_token, void* out,
                                    int64_t tokens, int num_seqs, int heads, int rank, int rot_dim, int block_size,
                                    int window, float scale, int max_q, void* workspace, size_t workspace_bytes, int dtype,
                                    nv_stream_t stream) {
  NV_CHECK_ARG(qa && cache && block_tables && cu_q && past_lens && seq_of_token && out, "nv_latent_attn: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_attn: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && tokens <= 65535 * 1024 && heads > 0 && rank > 0 && rot_dim >= 0 && block_size > 0 && table_cols > 0,
               "nv_latent_attn: bad shape");
  if (tokens == 0) return NV_OK;
  NV_CHECK_ARG(tokens <= 65535, "nv_latent_attn: %lld tokens exceed one launch", (long long)tokens);
  const int Dk = rank + rot_dim;
  // bf16 caches whose rows split into 16-byte pieces go to the matrix cores
  if (dtype == NV_BF16 && Dk % 8 == 0 && rank % 16 == 0 && rank <= 512 && num_seqs > 0) {
    int HQ = 1;
    while (HQ < heads && HQ < 16) HQ *= 2;
    MfmaAttnArgs q{{qa, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, heads, rank, rot_dim,
                    block_size, window, 0, 0, scale},
                   num_seqs, HQ, 16 / HQ, ((Dk + 31) / 32) * 32, 1, reinterpret_cast<float*>(workspace)};
    // one token per request: several workgroups share its keys, when the caller brought room for their shares
    if (max_q == 1 && workspace) {
      const int k = latent_attn_key_splits(tokens, heads);
      if (k > 1 && workspace_bytes >= (size_t)tokens * heads * k * (rank + 2) * sizeof(float)) q.ksplit = k;
    }
    const int Dq = q.Dkp + 8;
    auto lds_for = [&](int keys) {
      return (size_t)(2 * 16 * Dq + keys * Dq + rank * (keys + 8) + 2 * 16 * (keys + 8)) * 2 + (size_t)(2 * 16 * (keys + 4) + 48) * 4;
    };
    const int keys = lds_for(64) <= 150 * 1024 ? 64 : 32;
    const size_t lds = lds_for(keys);
    if (lds <= 150 * 1024 && keys * (Dk / 8) <= 10 * 256) {
      const int64_t tiles = tokens / q.TQ + num_seqs;        // at most: every request may end in a partial tile
      NV_CHECK_ARG(tiles <= 65535, "nv_latent_attn: %lld tiles exceed one launch", (long long)tiles);
      dim3 grid((unsigned)((heads + HQ - 1) / HQ), (unsigned)tiles, (unsigned)q.ksplit);
      const int ntile = (rank / 16 + 3) / 4;
      hipStream_t st = (hipStream_t)stream;
      hipError_t e;
      if (keys == 64)
        e = ntile <= 2 ? launch_mfma_attn<2, 64>(q, grid, lds, st) : ntile <= 4 ? launch_mfma_attn<4, 64>(q, grid, lds, st)
                                                                                 : launch_mfma_attn<8, 64>(q, grid, lds, st);
      else
        e = launch_mfma_attn<8, 32>(q, grid, lds, st);
      if (e != hipSuccess) {
        nv_set_error("nv_latent_attn: %s", hipGetErrorString(e));
        return NV_ERR_LAUNCH;
      }
      NV_CHECK_LAUNCH();
      if (q.ksplit > 1) {
        const int64_t rows = tokens * heads;
        latent_attn_join_kernel<<<dim3((unsigned)rows), dim3(256), 0, st>>>(q.partial, reinterpret_cast<bf16_t*>(out),
                                                                            q.ksplit, rank);
        NV_CHECK_LAUNCH();
      }
      return NV_OK;
    }
  }
  // LDS plan: as many heads per workgroup as fit beside a key tile of 64 (then 32, 16, 8) rows
  const size_t budget = 64 * 1024;
  int TK = 64, HC = heads;
  auto need = [&](int hc, int tk) {
    return (size_t)(hc * Dk + tk * (Dk + 1) + hc * tk + hc * rank + 3 * hc) * sizeof(float);
  };
  while (TK > 8 && need(1, TK) > budget) TK /= 2;
  NV_CHECK_ARG(need(1, TK) <= budget, "nv_latent_attn: rows of %d numbers do not fit the LDS plan", Dk);
  while (HC > 1 && need(HC, TK) > budget) HC = (HC + 1) / 2;
  AttnArgs p{qa, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, heads, rank, rot_dim, block_size,
             window, HC, TK, scale};
  dim3 grid((unsigned)((heads + HC - 1) / HC), (unsigned)tokens);
  NV_DISPATCH_T(dtype, latent_attn_kernel<T><<<grid, dim3(256), need(HC, TK), (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_latent_gather(const void* cache, const int32_t* block_tables, int table_cols, const int32_t* cu_k,
                                const int32_t* cu_q, const int32_t* past_lens, int num_seqs, int block_size, int row_width,
                                void* out, int64_t rows, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(cache && block_tables && cu_k && cu_q && past_lens && out, "nv_latent_gather: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_gather: bad dtype %d", dtype);
  NV_CHECK_ARG(num_seqs > 0 && block_size > 0 && row_width > 0 && rows >= 0 && table_cols > 0, "nv_latent_gather: bad shape");
  if (rows == 0) return NV_OK;
  NV_DISPATCH_T(dtype, latent_gather_kernel<T><<<dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream>>>(
                           (const T*)cache, block_tables, table_cols, cu_k, cu_q, past_lens, num_seqs, block_size,
                           row_width, (T*)out));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_latent_expand(const void* kv, const void* c, void* out, int64_t rows, int heads, int dim, int rot_dim,
                                int vdim, int rank, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(kv && c && out, "nv_latent_expand: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_expand: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && heads > 0 && dim > 0 && rot_dim >= 0 && vdim > 0 && rank > 0, "nv_latent_expand: bad shape");
  if (rows == 0) return NV_OK;
  NV_DISPATCH_T(dtype, latent_expand_kernel<T><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
                           (const T*)kv, (const T*)c, (T*)out, heads, dim, rot_dim, vdim, rank));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
