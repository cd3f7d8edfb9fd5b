// Softmax attention over a paged cache with grouped key/value heads, key and value sizes that may differ, and a score
// that is shaped before the softmax:
//     s_ij = cap(q_i . k_j) - slope_h (i - j),   cap(z) = c tanh(z / c) (or z without a cap),
// over the keys 0 <= i - j < window (window 0: every earlier key).  q arrives already normalised and multiplied by its
// scale and per-head temperature (qk_norm_store below), so the kernel's own arithmetic is the dot product, the cap,
// the distance term and the softmax, all in fp32.  Options of a design: no distance term; a sink, one learned logit per
// query head that joins the softmax's denominator without a key or a value; values that ARE the keys (rows [k: G * d]
// only, read twice); a sigmoid output gate from fp32 logits laid out like the output, or one logit per head; chunks, in
// which a query sees the keys j <= i of its own chunk only (floor(i / chunk) == floor(j / chunk), counted from the
// sequence's first position).
//
// qk_norm_store: per token, RMS norm over each query and key head (one weight vector shared by the heads), the query
// scaled by scale * temp[h] and left in fp32, the normalised key and the value written to the token's cache row
// [k: G * d | v: G * dv] in the storage type.  The norms may be absent (null weights: the projection as it is), and
// the query may carry a temperature that grows with the position p: 1 + coef * ln(floor((p + 1) / every) + 1).
// Further options: one root mean square over all heads of q (and of k) with a weight per number; a rotation of the first
// rot_dims numbers of every head after the norm (dimension i with i + rot_dims / 2, angle position * inv_freq[i]); values
// blended with another layer's values of the same token, v <- (1 - lam) v + lam v_first, before they are stored.
//
// window_attn_kernel: a workgroup owns TQ consecutive tokens of the packed batch and one key/value head, i.e. up to
// TQ * (H / G) query rows that read the same keys; tokens of different requests inside the tile are served one request
// after the other.  Keys go through LDS in tiles of TK rows; online softmax per row.
#include "anyt.h"

namespace {

struct QkArgs {
  const float* proj;      // [tokens, proj_rs]: q | k | v at the given column offsets (fp32 projections)
  const void* bias;       // [proj columns] added to the projections (same column offsets), or null
  int64_t proj_rs;
  int q_off, k_off, v_off;
  const void* qn;         // query norm weight: [d] shared by the heads, or [H * d] when norm_whole
  const void* kn;         // [d] or [G * d]
  const void* temp;       // [H] or null
  const int64_t* positions;   // [tokens], read when temp_every > 0 or rot_dims > 0
  float temp_coef;
  int temp_every;         // 0: no position temperature
  const int32_t* slot_mapping;   // [tokens] cache row of each token, -1: none
  void* cache;            // [rows, G * (d + dv)]
  float* q_out;           // [tokens, H * d]
  int H, G, d, dv;
  float scale, eps;
  int norm_whole;         // 1: one root mean square over all H * d query numbers (and over all G * d key numbers)
  const float* inv_freq;  // [rot_dims / 2] rotation frequencies, read when rot_dims > 0
  int rot_dims;           // the first rot_dims numbers of every head are rotated, dimension i with i + rot_dims / 2
  float mscale;           // multiplies cosine and sine
  const float* v_first;   // [tokens, v_first_rs] values to blend in, or null
  int64_t v_first_rs;
  const void* vmix;       // one number lam: v <- (1 - lam) v + lam v_first
};

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_store_kernel(QkArgs p) {
  __shared__ float red[32];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float* row = p.proj + t * p.proj_rs;
  const int64_t slot = p.slot_mapping[t];
  const int cw = p.G * (p.d + p.dv);       // dv 0: the values are the keys, rows hold keys only
  T* crow = slot >= 0 ? reinterpret_cast<T*>(p.cache) + slot * cw : nullptr;
  float pos_temp = 1.0f;
  if (p.temp_every > 0) pos_temp = 1.0f + p.temp_coef * logf((float)((p.positions[t] + 1) / p.temp_every) + 1.0f);
  const T* qn = reinterpret_cast<const T*>(p.qn);
  const T* kn = reinterpret_cast<const T*>(p.kn);
  const T* temp = reinterpret_cast<const T*>(p.temp);
  const T* bias = reinterpret_cast<const T*>(p.bias);
  const int half = p.rot_dims / 2;
  const float pos = p.rot_dims > 0 ? (float)p.positions[t] : 0.0f;
  // cosine and sine of the token's angles once for all heads (rotations over more than 256 numbers evaluate them in place)
  __shared__ float s_cs[128], s_sn[128];
  const bool trig_shared = half > 0 && half <= 128;
  if (trig_shared) {
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const float a = pos * p.inv_freq[i];
      s_cs[i] = cosf(a) * p.mscale;
      s_sn[i] = sinf(a) * p.mscale;
    }
    __syncthreads();
  }
  float inv_q = 1.0f, inv_k = 1.0f;
  if (qn && p.norm_whole) {
    float sq = 0.0f, sk = 0.0f;
    for (int e = threadIdx.x; e < p.H * p.d; e += blockDim.x) {
      const float x = row[p.q_off + e] + (bias ? ld_f32<T>(bias + p.q_off + e) : 0.0f);
      sq += x * x;
    }
    for (int e = threadIdx.x; e < p.G * p.d; e += blockDim.x) {
      const float x = row[p.k_off + e] + (bias ? ld_f32<T>(bias + p.k_off + e) : 0.0f);
      sk += x * x;
    }
    inv_q = 1.0f / sqrtf(block_sum(sq, red) / (float)(p.H * p.d) + p.eps);
    inv_k = 1.0f / sqrtf(block_sum(sk, red) / (float)(p.G * p.d) + p.eps);
  }
  for (int v = wv; v < p.H + p.G; v += nw) {
    const bool is_q = v < p.H;
    const int hv = is_q ? v : v - p.H;
    const int col = is_q ? p.q_off + hv * p.d : p.k_off + hv * p.d;
    const float* src = row + col;
    float inv = is_q ? inv_q : inv_k;
    if (qn && !p.norm_whole) {
      float ss = 0.0f;
      for (int e = lane; e < p.d; e += 64) {
        const float x = src[e] + (bias ? ld_f32<T>(bias + col + e) : 0.0f);
        ss += x * x;
      }
      ss = wave_sum(ss);
      inv = 1.0f / sqrtf(ss / (float)p.d + p.eps);
    }
    const T* nw_ = is_q ? qn : kn;
    if (nw_ && p.norm_whole) nw_ += hv * p.d;
    auto normed = [&](int e) {
      const float x = src[e] + (bias ? ld_f32<T>(bias + col + e) : 0.0f);
      return x * inv * (nw_ ? ld_f32<T>(nw_ + e) : 1.0f);
    };
    auto value = [&](int e) {      // normalised, then rotated
      float x = normed(e);
      if (e < p.rot_dims) {
        const bool first = e < half;
        const int fi = first ? e : e - half;
        float cs, sn;
        if (trig_shared) {
          cs = s_cs[fi];
          sn = s_sn[fi];
        } else {
          const float a = pos * p.inv_freq[fi];
          cs = cosf(a) * p.mscale;
          sn = sinf(a) * p.mscale;
        }
        const float other = normed(first ? e + half : e - half);
        x = first ? x * cs - other * sn : x * cs + other * sn;
      }
      return x;
    };
    if (is_q) {
      const float f = p.scale * (temp ? ld_f32<T>(temp + v) : 1.0f) * pos_temp;
      for (int e = lane; e < p.d; e += 64) p.q_out[t * p.H * p.d + v * p.d + e] = value(e) * f;
    } else if (crow) {
      for (int e = lane; e < p.d; e += 64) st_f32<T>(crow + hv * p.d + e, value(e));
    }
  }
  if (crow && p.dv > 0) {
    const float lam = p.v_first ? ld_f32<T>(reinterpret_cast<const T*>(p.vmix)) : 0.0f;
    for (int e = threadIdx.x; e < p.G * p.dv; e += blockDim.x) {
      float x = row[p.v_off + e] + (bias ? ld_f32<T>(bias + p.v_off + e) : 0.0f);
      if (p.v_first) x = (1.0f - lam) * x + lam * p.v_first[t * p.v_first_rs + e];
      st_f32<T>(crow + p.G * p.d + e, x);
    }
  }
}

struct WAttnArgs {
  const float* q;          // [tokens, H * d]
  const void* cache;       // [rows, G * (d + dv)]
  const int32_t* tables;   // [B, table_cols]
  int table_cols;
  const int32_t* cu_q;     // [B + 1]
  const int32_t* past;     // [B]
  const int32_t* seq_of;   // [tokens]
  void* out;               // [tokens, out_rs]: head h at columns h * dv
  int64_t out_rs;
  int64_t tokens;
  int H, G, d, dv, block_size, window, TQ, TK;
  float softcap, out_scale;
  int cw, v_col;           // numbers per cache row; column where the values of key/value head 0 begin (0: the keys)
  int slope_on;            // the distance term 2^(-8 (h + 1) / H) (i - j)
  const void* sink;        // [H] logits that join the denominator, or null
  const float* gate;       // [tokens, gate_rs] logits whose sigmoid multiplies the output (head h at h * dv), or null
  int64_t gate_rs;
  int gate_head;           // 1: one logit per head (head h at column h)
  int chunk;               // > 0: a query sees only the keys of its own chunk, floor(i / chunk) == floor(j / chunk)
  int ksplit;              // SPLIT only: workgroups that share a token's keys (blockIdx.z); > 1: results go to `partial`
  float* partial;          // [tokens, H, ksplit, dv + 2]: unnormalised output, then maximum and sum
};

// (factor for the accumulated values, denominator) once the walk over the keys is over: the sink joins the sum
__device__ __forceinline__ void close_softmax(float m, float l, bool has_sink, float sink, float& f, float& den) {
  if (!has_sink) {
    f = 1.0f;
    den = l;
    return;
  }
  const float top = fmaxf(m, sink);
  f = m == -INFINITY ? 0.0f : expf(m - top);
  den = l * f + expf(sink - top);
}

template <typename T>
__global__ __launch_bounds__(256) void window_attn_kernel(WAttnArgs p) {
  extern __shared__ float lds[];
  const int R = p.H / p.G, d = p.d, dv = p.dv, TK = p.TK, dp = d + 1;
  const int maxrows = p.TQ * R;
  float* sq = lds;                       // [rows][d]
  float* sk = sq + maxrows * d;          // [TK][d + 1]
  float* sv = sk + TK * dp;              // [TK][dv]
  float* sc = sv + TK * dv;              // [rows][TK]
  float* acc = sc + maxrows * TK;        // [rows][dv]
  float* sm = acc + maxrows * dv;        // [rows] running maximum
  float* sl = sm + maxrows;              // [rows] running sum
  float* scorr = sl + maxrows;           // [rows]
  const int g = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int64_t t_begin = (int64_t)blockIdx.x * p.TQ;
  const int64_t t_end = min(p.tokens, t_begin + p.TQ);
  const T* cache = reinterpret_cast<const T*>(p.cache);
  const int cw = p.cw;
  T* out = reinterpret_cast<T*>(p.out);
  const T* sink = reinterpret_cast<const T*>(p.sink);

  for (int64_t ts = t_begin; ts < t_end;) {
    const int b = p.seq_of[ts];
    const int64_t te = min(t_end, (int64_t)p.cu_q[b + 1]);
    const int nq = (int)(te - ts), rows = nq * R;
    const int p0 = p.past[b] + (int)(ts - p.cu_q[b]);
    const int32_t* table = p.tables + (int64_t)b * p.table_cols;
    for (int i = tid; i < rows * d; i += 256) {
      const int rr = i / d, e = i % d;
      sq[i] = p.q[(ts + rr / R) * p.H * d + (g * R + rr % R) * d + e];
    }
    for (int i = tid; i < rows * dv; i += 256) acc[i] = 0.0f;
    if (tid < rows) {
      sm[tid] = -INFINITY;
      sl[tid] = 0.0f;
    }
    __syncthreads();
    int lo = p.window > 0 ? max(0, p0 - p.window + 1) : 0;
    if (p.chunk > 0) lo = max(lo, p0 / p.chunk * p.chunk);      // the tile's first token has the earliest chunk
    const int hi = p0 + nq - 1;
    for (int j0 = lo; j0 <= hi; j0 += TK) {
      const int nk = min(TK, hi + 1 - j0);
      for (int i = tid; i < nk * (d + dv); i += 256) {
        const int j = i / (d + dv), e = i % (d + dv);
        const int kp = j0 + j;
        const int64_t crow = (int64_t)table[kp / p.block_size] * p.block_size + kp % p.block_size;
        if (e < d) sk[j * dp + e] = ld_f32<T>(cache + crow * cw + g * d + e);
        else sv[j * dv + e - d] = ld_f32<T>(cache + crow * cw + p.v_col + g * dv + e - d);
      }
      __syncthreads();
      for (int i = tid; i < rows * TK; i += 256) {
        const int rr = i / TK, j = i % TK;
        const int pos = p0 + rr / R, kp = j0 + j;
        float s = -INFINITY;
        if (j < nk && kp <= pos && (p.window <= 0 || pos - kp < p.window) && (p.chunk <= 0 || kp >= pos / p.chunk * p.chunk)) {
          s = 0.0f;
          const float* qv = sq + rr * d;
          const float* kv = sk + j * dp;
          for (int e = 0; e < d; ++e) s += qv[e] * kv[e];
          if (p.softcap > 0.0f) s = p.softcap * tanhf(s / p.softcap);
          const int h = g * R + rr % R;
          if (p.slope_on) s -= exp2f(-8.0f * (float)(h + 1) / (float)p.H) * (float)(pos - kp);
        }
        sc[i] = s;
      }
      __syncthreads();
      for (int rr = wv; rr < rows; rr += 4) {
        float m = -INFINITY;
        for (int j = lane; j < TK; j += 64) m = fmaxf(m, sc[rr * TK + j]);
        m = wave_max(m);
        const float m_old = sm[rr];
        const float m_new = fmaxf(m_old, m);
        float sum = 0.0f;
        for (int j = lane; j < TK; j += 64) {
          const float s = sc[rr * TK + j];
          const float e = s == -INFINITY ? 0.0f : expf(s - m_new);
          sc[rr * TK + j] = e;
          sum += e;
        }
        sum = wave_sum(sum);
        if (lane == 0) {
          const float corr = m_new == -INFINITY ? 1.0f : expf(m_old - m_new);   // exp(-inf) = 0 at the first tile
          scorr[rr] = corr;
          sm[rr] = m_new;
          sl[rr] = sl[rr] * corr + sum;
        }
      }
      __syncthreads();
      for (int i = tid; i < rows * dv; i += 256) {
        const int rr = i / dv, e = i % dv;
        float a = acc[i] * scorr[rr];
        const float* pv = sc + rr * TK;
        for (int j = 0; j < nk; ++j) a += pv[j] * sv[j * dv + e];
        acc[i] = a;
      }
      __syncthreads();
    }
    for (int i = tid; i < rows * dv; i += 256) {
      const int rr = i / dv, e = i % dv, h = g * R + rr % R;
      float f, den;
      close_softmax(sm[rr], sl[rr], sink != nullptr, sink ? ld_f32<T>(sink + h) : 0.0f, f, den);
      float v = acc[i] * f / den * p.out_scale;
      if (p.gate) v *= sigmoid_f32(p.gate[(ts + rr / R) * p.gate_rs + (p.gate_head ? h : h * dv + e)]);
      st_f32<T>(out + (ts + rr / R) * p.out_rs + h * dv + e, v);
    }
    __syncthreads();
    ts = te;
  }
}

// ---- the same attention on the matrix cores (bf16 cache) ----
// A workgroup of four wavefronts owns up to 64 query rows, 16 per wavefront: TQ consecutive tokens times the R heads
// that share key/value head g.  Per tile of 64 keys the K rows are staged row-major and the V rows transposed (both
// bf16, zero-filled past the last key); every wavefront computes S = Q K^T for its rows with the queries held as
// register fragments, shapes and masks the scores in the accumulator layout (a lane owns four rows of one key column),
// keeps running maxima and sums per row with 16-lane reductions, passes P through a private LDS patch to turn it into an
// A operand, and accumulates O += P V.  Scores, maxima, sums and rescaling are fp32; Q and P enter the MFMAs as bf16.
//
// SPLIT (steps of one token per request, at most 16 heads per key head): the four wavefronts hold the SAME rows and
// walk different key tiles, each with its own staging area and no workgroup barrier inside the walk; their partial
// (maximum, sum, output) triples meet in LDS at the end.  A decoded token's window is thus read four tiles at a time.
constexpr int MA_KEYS = 64, MA_VST = MA_KEYS + 8, MA_PST = MA_KEYS + 8;

constexpr size_t ma_stage_bytes(int ks, int ct) {     // one staging area: K tile, transposed V tile
  return ((size_t)MA_KEYS * (ks * 32 + 8) + (size_t)ct * 16 * MA_VST) * 2;
}
constexpr size_t ma_lds_bytes(int ks, int ct, bool split) {
  return split ? 4 * (ma_stage_bytes(ks, ct) + 16 * MA_PST * 2) : ma_stage_bytes(ks, ct) + 4 * 16 * MA_PST * 2;
}

// EXT: chunks and the gate of one logit per head are compiled in; launches that use neither take the kernel without them
template <int KS, int CT, bool SPLIT, bool EXT>
__global__ __launch_bounds__(256) void window_attn_mfma_kernel(WAttnArgs p) {
  constexpr int DK = KS * 32, KST = DK + 8, DVP = CT * 16;
  constexpr int STAGE = (int)(ma_stage_bytes(KS, CT) / 2);                 // bf16 elements of one staging area
  extern __shared__ u32x4 lds_raw[];
  __shared__ int64_t sRowAll[SPLIT ? 4 : 1][MA_KEYS];
  const int R = p.H / p.G, d = p.d, dv = p.dv;
  const int g = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int lc = lane & 15, lg = lane >> 4;
  bf16_t* base = reinterpret_cast<bf16_t*>(lds_raw);
  bf16_t* sK = base + (SPLIT ? wv * STAGE : 0);              // [64][KST]
  bf16_t* sVt = sK + MA_KEYS * KST;                          // [DVP][MA_VST]
  bf16_t* sPw = base + (SPLIT ? 4 : 1) * STAGE + wv * 16 * MA_PST;   // [16][MA_PST] of this wavefront
  int64_t* sRow = sRowAll[SPLIT ? wv : 0];
  constexpr int ST = SPLIT ? 64 : 256;                                    // threads that stage a tile together
  constexpr int NKC = MA_KEYS * (DK / 8) / ST, NVC = MA_KEYS * (DVP / 8) / ST;   // 16-byte pieces per thread
  const int stid = SPLIT ? lane : tid;
  const int row0 = SPLIT ? 0 : wv * 16;                                   // first query row of this wavefront
  auto sync = [&]() {
    if constexpr (SPLIT) {      // the area is private to this wavefront: its own LDS accesses complete in order
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
      __syncthreads();
    }
  };
  const int64_t t_begin = (int64_t)blockIdx.x * p.TQ;
  const int64_t t_end = min(p.tokens, t_begin + p.TQ);
  const bf16_t* cache = reinterpret_cast<const bf16_t*>(p.cache);
  const int cw = p.cw;
  bf16_t* out = reinterpret_cast<bf16_t*>(p.out);
  const bf16_t* sink = reinterpret_cast<const bf16_t*>(p.sink);

  for (int64_t ts = t_begin; ts < t_end;) {
    const int b = p.seq_of[ts];
    const int64_t te = min(t_end, (int64_t)p.cu_q[b + 1]);
    const int nq = (int)(te - ts), rows = nq * R;
    const int p0 = p.past[b] + (int)(ts - p.cu_q[b]);
    const int32_t* table = p.tables + (int64_t)b * p.table_cols;
    const bool wave_on = row0 < rows;
    // query fragments of this wavefront's 16 rows (A operand: lane holds row lc, features 8 lg .. 8 lg + 7 of each step)
    bf16x8 qf[KS];
    {
      const int rr = row0 + lc;
      const bool ok = rr < rows;
      const float* qrow = ok ? p.q + ((ts + rr / R) * p.H + g * R + rr % R) * d : nullptr;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int e = ks * 32 + lg * 8 + i;
          qf[ks][i] = (bf16_t)((ok && e < d) ? qrow[e] : 0.0f);
        }
      }
    }
    // the four accumulator rows of this lane
    int pos[4], kmin[EXT ? 4 : 1];      // kmin: first key of the row's chunk
    float slope[4], m_run[4], l_run[4];
    bool valid[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int rr = row0 + lg * 4 + r;
      valid[r] = rr < rows;
      pos[r] = p0 + rr / R;
      if constexpr (EXT) kmin[r] = p.chunk > 0 ? pos[r] / p.chunk * p.chunk : 0;
      slope[r] = p.slope_on ? exp2f(-8.0f * (float)(g * R + rr % R + 1) / (float)p.H) : 0.0f;
      m_run[r] = -INFINITY;
      l_run[r] = 0.0f;
    }
    f32x4 acc_o[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc_o[ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const int wpos_lo = p0 + row0 / R, wpos_hi = p0 + min(rows - 1, row0 + 15) / R;

    const int lo_w = p.window > 0 ? max(0, p0 - p.window + 1) : 0;
    // the tile's first token has the earliest chunk
    const int lo = (EXT && p.chunk > 0) ? max(lo_w, p0 / p.chunk * p.chunk) : lo_w, hi = p0 + nq - 1;
    const int walkers = SPLIT ? 4 * p.ksplit : 1;          // wavefronts (of all workgroups) that share this token's keys
    for (int j0 = lo + (SPLIT ? ((int)blockIdx.z * 4 + wv) * MA_KEYS : 0); j0 <= hi; j0 += walkers * MA_KEYS) {
      if (stid < MA_KEYS) {
        const int kp = j0 + stid;
        sRow[stid] = kp <= hi ? (int64_t)table[kp / p.block_size] * p.block_size + kp % p.block_size : -1;
      }
      sync();
      // all of a thread's loads are issued before the first LDS store: one round trip to memory per tile
      u32x4 kreg[NKC], vreg[NVC];
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = stid + i * ST, key = c / (DK / 8), part = c % (DK / 8);
        const int64_t row = sRow[key];
        kreg[i] = u32x4{0u, 0u, 0u, 0u};
        if (row >= 0 && part * 8 < d) kreg[i] = *reinterpret_cast<const u32x4*>(cache + row * cw + g * d + part * 8);
      }
#pragma unroll
      for (int i = 0; i < NVC; ++i) {
        const int c = stid + i * ST, key = c % MA_KEYS, part = c / MA_KEYS;
        const int64_t row = sRow[key];
        vreg[i] = u32x4{0u, 0u, 0u, 0u};
        if (row >= 0 && part * 8 < dv)
          vreg[i] = *reinterpret_cast<const u32x4*>(cache + row * cw + p.v_col + g * dv + part * 8);
      }
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = stid + i * ST, key = c / (DK / 8), part = c % (DK / 8);
        *reinterpret_cast<u32x4*>(sK + key * KST + part * 8) = kreg[i];
      }
#pragma unroll
      for (int i = 0; i < NVC; ++i) {
        const int c = stid + i * ST, key = c % MA_KEYS, part = c / MA_KEYS;
        uint16_t* dst = reinterpret_cast<uint16_t*>(sVt) + (part * 8) * MA_VST + key;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          dst[(2 * w) * MA_VST] = (uint16_t)(vreg[i][w] & 0xffffu);
          dst[(2 * w + 1) * MA_VST] = (uint16_t)(vreg[i][w] >> 16);
        }
      }
      sync();
      // keys this wavefront's rows can see: [wpos_lo - window + 1, wpos_hi]
      bool need = wave_on && j0 <= wpos_hi && (p.window <= 0 || j0 + MA_KEYS - 1 > wpos_lo - p.window);
      if constexpr (EXT) need = need && (p.chunk <= 0 || j0 + MA_KEYS - 1 >= wpos_lo / p.chunk * p.chunk);
      if (need) {
        f32x4 acc_s[4];
#pragma unroll
        for (int sub = 0; sub < 4; ++sub) {
          acc_s[sub] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + (sub * 16 + lc) * KST + ks * 32 + lg * 8);
            acc_s[sub] = mfma16(qf[ks], kf, acc_s[sub]);
          }
        }
        float corr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float mt = -INFINITY;
#pragma unroll
          for (int sub = 0; sub < 4; ++sub) {
            const int kp = j0 + sub * 16 + lc;
            const int dist = pos[r] - kp;
            float sc = acc_s[sub][r];
            if (p.softcap > 0.0f) sc = p.softcap * tanhf(sc / p.softcap);
            sc -= slope[r] * (float)dist;
            bool vis = valid[r] && dist >= 0 && (p.window <= 0 || dist < p.window);
            if constexpr (EXT) vis = vis && kp >= kmin[r];
            sc = vis ? sc : -INFINITY;
            acc_s[sub][r] = sc;
            mt = fmaxf(mt, sc);
          }
#pragma unroll
          for (int o = 1; o < 16; o <<= 1) mt = fmaxf(mt, __shfl_xor(mt, o, 64));
          const float m_new = fmaxf(m_run[r], mt);
          corr[r] = m_new == -INFINITY ? 1.0f : __expf(m_run[r] - m_new);
          float sum = 0.0f;
#pragma unroll
          for (int sub = 0; sub < 4; ++sub) {
            const float sc = acc_s[sub][r];
            const float e = sc == -INFINITY ? 0.0f : __expf(sc - m_new);
            sum += e;
            sPw[(lg * 4 + r) * MA_PST + sub * 16 + lc] = (bf16_t)e;
          }
#pragma unroll
          for (int o = 1; o < 16; o <<= 1) sum += __shfl_xor(sum, o, 64);
          l_run[r] = l_run[r] * corr[r] + sum;
          m_run[r] = m_new;
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc_o[ct][r] *= corr[r];
        // the patch is private to this wavefront: its own LDS accesses complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int ks = 0; ks < MA_KEYS / 32; ++ks) {
          const bf16x8 pf = *reinterpret_cast<const bf16x8*>(sPw + lc * MA_PST + ks * 32 + lg * 8);
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) {
            const bf16x8 vf = *reinterpret_cast<const bf16x8*>(sVt + (ct * 16 + lc) * MA_VST + ks * 32 + lg * 8);
            acc_o[ct] = mfma16(pf, vf, acc_o[ct]);
          }
        }
      }
      sync();
    }
    if constexpr (SPLIT) {
      // partial results of the four wavefronts: rows of DVP outputs, the maximum and the sum, in each one's V area
      constexpr int PW = DVP + 2;
      float* part = reinterpret_cast<float*>(sVt);
      static_assert((size_t)16 * PW * 4 <= (size_t)DVP * MA_VST * 2, "partials fit the V area");
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) part[(lg * 4 + r) * PW + ct * 16 + lc] = acc_o[ct][r];
        if (lc == 0) {
          part[(lg * 4 + r) * PW + DVP] = m_run[r];
          part[(lg * 4 + r) * PW + DVP + 1] = l_run[r];
        }
      }
      __syncthreads();
      for (int idx = tid; idx < 16 * DVP; idx += 256) {
        const int rr = idx / DVP, e = idx % DVP;
        if (rr >= rows || e >= dv) continue;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w)
          m = fmaxf(m, reinterpret_cast<const float*>(base + w * STAGE + MA_KEYS * KST)[rr * PW + DVP]);
        float l = 0.0f, o = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float* pw = reinterpret_cast<const float*>(base + w * STAGE + MA_KEYS * KST);
          const float mw = pw[rr * PW + DVP];
          const float f = mw == -INFINITY ? 0.0f : __expf(mw - m);
          l += pw[rr * PW + DVP + 1] * f;
          o += pw[rr * PW + e] * f;
        }
        const int h = g * R + rr % R;
        if (p.ksplit > 1) {      // another launch joins the workgroups' shares (and the sink, and the gate)
          float* dst = p.partial + (((ts + rr / R) * p.H + h) * p.ksplit + blockIdx.z) * (dv + 2);
          dst[e] = o;
          if (e == 0) {
            dst[dv] = m;
            dst[dv + 1] = l;
          }
          continue;
        }
        float f, den;
        close_softmax(m, l, sink != nullptr, sink ? ld_f32<bf16_t>(sink + h) : 0.0f, f, den);
        float v = o * f * p.out_scale / den;
        if (p.gate) v *= sigmoid_f32(p.gate[(ts + rr / R) * p.gate_rs + ((EXT && p.gate_head) ? h : h * dv + e)]);
        out[(ts + rr / R) * p.out_rs + h * dv + e] = (bf16_t)v;
      }
      __syncthreads();
    } else if (wave_on) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rr = row0 + lg * 4 + r;
        if (!valid[r]) continue;
        const int h = g * R + rr % R;
        float fs, den;
        close_softmax(m_run[r], l_run[r], sink != nullptr, sink ? ld_f32<bf16_t>(sink + h) : 0.0f, fs, den);
        const float f = p.out_scale * fs / den;
        bf16_t* orow = out + (ts + rr / R) * p.out_rs + h * dv;
        const float* grow = p.gate ? p.gate + (ts + rr / R) * p.gate_rs + ((EXT && p.gate_head) ? h : h * dv) : nullptr;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const int e = ct * 16 + lc;
          if (e < dv) orow[e] = (bf16_t)(acc_o[ct][r] * f * (grow ? sigmoid_f32(grow[(EXT && p.gate_head) ? 0 : e]) : 1.0f));
        }
      }
    }
    ts = te;
  }
}

// joins the shares of the ksplit workgroups that walked one token's keys: one wavefront per (token, head)
__global__ __launch_bounds__(256) void window_attn_join_kernel(WAttnArgs p) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.tokens * p.H) return;
  const int lane = threadIdx.x & 63, dv = p.dv, h = (int)(row % p.H);
  const int64_t t = row / p.H;
  const float* src = p.partial + row * p.ksplit * (dv + 2);
  // all maxima and sums first (at most 8 shares: the loads go out together), then one weight per share
  float mz[8], wz[8];
  float m = -INFINITY, l = 0.0f;
#pragma unroll
  for (int z = 0; z < 8; ++z) {
    mz[z] = z < p.ksplit ? src[z * (dv + 2) + dv] : -INFINITY;
    wz[z] = z < p.ksplit ? src[z * (dv + 2) + dv + 1] : 0.0f;
    m = fmaxf(m, mz[z]);
  }
#pragma unroll
  for (int z = 0; z < 8; ++z) {
    const float f = mz[z] == -INFINITY ? 0.0f : __expf(mz[z] - m);
    l += wz[z] * f;
    wz[z] = f;
  }
  const bf16_t* sink = reinterpret_cast<const bf16_t*>(p.sink);
  float f, den;
  close_softmax(m, l, sink != nullptr, sink ? ld_f32<bf16_t>(sink + h) : 0.0f, f, den);
  bf16_t* out = reinterpret_cast<bf16_t*>(p.out) + t * p.out_rs + h * dv;
  for (int e = lane; e < dv; e += 64) {
    float o = 0.0f;
#pragma unroll
    for (int z = 0; z < 8; ++z)
      if (z < p.ksplit) o += src[z * (dv + 2) + e] * wz[z];
    float v = o * f * p.out_scale / den;
    if (p.gate) v *= sigmoid_f32(p.gate[t * p.gate_rs + (p.gate_head ? h : h * dv + e)]);
    out[e] = (bf16_t)v;
  }
}

template <int KS, int CT, bool SPLIT, bool EXT>
hipError_t launch_window_mfma4(const WAttnArgs& p, dim3 grid, hipStream_t s) {
  constexpr size_t lds = ma_lds_bytes(KS, CT, SPLIT);
  static size_t allowed = 64 * 1024;
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&window_attn_mfma_kernel<KS, CT, SPLIT, EXT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    allowed = lds;
  }
  window_attn_mfma_kernel<KS, CT, SPLIT, EXT><<<grid, dim3(256), lds, s>>>(p);
  return hipGetLastError();
}

template <int KS, int CT, bool SPLIT>
hipError_t launch_window_mfma3(const WAttnArgs& p, dim3 grid, hipStream_t s) {
  if (p.chunk > 0 || (p.gate && p.gate_head)) return launch_window_mfma4<KS, CT, SPLIT, true>(p, grid, s);
  return launch_window_mfma4<KS, CT, SPLIT, false>(p, grid, s);
}

template <int KS, int CT>
hipError_t launch_window_mfma2(const WAttnArgs& p, bool split, dim3 grid, hipStream_t s) {
  if constexpr (ma_lds_bytes(KS, CT, true) <= 156 * 1024) {
    if (split) return launch_window_mfma3<KS, CT, true>(p, grid, s);
  }
  return launch_window_mfma3<KS, CT, false>(p, grid, s);
}

template <int KS>
hipError_t launch_window_mfma(const WAttnArgs& p, int ct, bool split, dim3 grid, hipStream_t s) {
  switch (ct) {
    case 2: return launch_window_mfma2<KS, 2>(p, split, grid, s);
    case 4: return launch_window_mfma2<KS, 4>(p, split, grid, s);
    case 8: return launch_window_mfma2<KS, 8>(p, split, grid, s);
    default: return launch_window_mfma2<KS, 16>(p, split, grid, s);
  }
}

}  // namespace

// Workgroups that share one decoded token's keys: enough to put about 256 workgroups on the chip, at most 8.  A
// function of the launch shape alone (not of the contexts), so a captured launch stays valid as contexts grow.
static int window_attn_key_splits(int64_t tokens, int kv_heads) {
  const int64_t groups = tokens * kv_heads;
  int k = 1;
  while (k < 8 && groups * k * 2 <= 256) k *= 2;
  return k;
}

extern "C" size_t nv_paged_softmax_attn_workspace_bytes(int64_t tokens, int max_q, int heads, int kv_heads, int vdim) {
  if (max_q > 1 || tokens <= 0 || heads / kv_heads > 16) return 0;
  const int k = window_attn_key_splits(tokens, kv_heads);
  return k > 1 ? (size_t)tokens * heads * k * (vdim + 2) * sizeof(float) : 0;
}

extern "C" int nv_qk_store(const float* proj, const void* bias, int64_t proj_row_stride, int q_off, int k_off, int v_off,
                           const void* q_norm, const void* k_norm, const void* temp, const int64_t* positions,
                           float temp_coef, int temp_every, float scale, float eps, const int32_t* slot_mapping,
                           void* cache, float* q_out, int64_t tokens, int heads, int kv_heads, int dim, int vdim, int dtype,
                           nv_stream_t stream) {
  return nv_qk_rotate_store(proj, bias, proj_row_stride, q_off, k_off, v_off, q_norm, k_norm, 0, temp, positions, temp_coef,
                            temp_every, nullptr, 0, 1.0f, nullptr, 0, nullptr, scale, eps, slot_mapping, cache, q_out,
                            tokens, heads, kv_heads, dim, vdim, dtype, stream);
}

extern "C" int nv_qk_rotate_store(const float* proj, const void* bias, int64_t proj_row_stride, int q_off, int k_off,
                                  int v_off, const void* q_norm, const void* k_norm, int norm_whole, const void* temp,
                                  const int64_t* positions, float temp_coef, int temp_every, const float* inv_freq,
                                  int rot_dims, float mscale, const float* v_first, int64_t v_first_row_stride,
                                  const void* vmix, float scale, float eps, const int32_t* slot_mapping, void* cache,
                                  float* q_out, int64_t tokens, int heads, int kv_heads, int dim, int vdim, int dtype,
                                  nv_stream_t stream) {
  NV_CHECK_ARG(proj && slot_mapping && cache && q_out, "nv_qk_store: null pointer");
  NV_CHECK_ARG((q_norm == nullptr) == (k_norm == nullptr), "nv_qk_store: both norm weights or none");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_qk_store: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim >= 0,
               "nv_qk_store: bad shape");
  NV_CHECK_ARG(temp_every >= 0 && (temp_every == 0 || positions), "nv_qk_store: the position temperature needs positions");
  NV_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim && (rot_dims == 0 || (positions && inv_freq)),
               "nv_qk_store: a rotation over %d of %d numbers needs positions and frequencies", rot_dims, dim);
  NV_CHECK_ARG(!v_first || (vmix && vdim > 0), "nv_qk_store: blending values needs its weight");
  if (tokens == 0) return NV_OK;
  QkArgs p{proj, bias, proj_row_stride, q_off, k_off, v_off, q_norm, k_norm, temp, positions, temp_coef, temp_every,
           slot_mapping, cache, q_out, heads, kv_heads, dim, vdim, scale, eps, norm_whole, inv_freq, rot_dims, mscale,
           v_first, v_first_row_stride, vmix};
  NV_DISPATCH_T(dtype, qk_norm_store_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_qk_norm_store(const float* proj, const void* bias, int64_t proj_row_stride, int q_off, int k_off,
                                int v_off, const void* q_norm, const void* k_norm, const void* temp, float scale, float eps,
                                const int32_t* slot_mapping, void* cache, float* q_out, int64_t tokens, int heads,
                                int kv_heads, int dim, int vdim, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(q_norm && k_norm && vdim > 0, "nv_qk_norm_store: null pointer");
  return nv_qk_store(proj, bias, proj_row_stride, q_off, k_off, v_off, q_norm, k_norm, temp, nullptr, 0.0f, 0, scale, eps,
                     slot_mapping, cache, q_out, tokens, heads, kv_heads, dim, vdim, dtype, stream);
}

extern "C" int nv_window_attn(const float* q, const void* cache, const int32_t* block_tables, int table_cols,
                              const int32_t* cu_q, const int32_t* past_lens, const int32_t* seq_of_token, void* out,
                              int64_t out_row_stride, int64_t tokens, int max_q, int heads, int kv_heads, int dim, int vdim,
                              int block_size, int window, float softcap, float out_scale, int dtype, nv_stream_t stream) {
  return nv_paged_softmax_attn(q, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, out_row_stride,
                               tokens, max_q, heads, kv_heads, dim, vdim, block_size, window, 0, softcap, out_scale, 1, 0,
                               nullptr, nullptr, 0, 0, nullptr, 0, dtype, stream);
}

extern "C" int nv_paged_softmax_attn(const float* q, const void* cache, const int32_t* block_tables, int table_cols,
                                     const int32_t* cu_q, const int32_t* past_lens, const int32_t* seq_of_token, void* out,
                                     int64_t out_row_stride, int64_t tokens, int max_q, int heads, int kv_heads, int dim,
                                     int vdim, int block_size, int window, int chunk, float softcap, float out_scale,
                                     int distance_term, int values_are_keys, const void* sink, const float* gate,
                                     int64_t gate_row_stride, int gate_per_head, void* workspace, size_t workspace_bytes,
                                     int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(q && cache && block_tables && cu_q && past_lens && seq_of_token && out, "nv_window_attn: null pointer");
  NV_CHECK_ARG(!values_are_keys || vdim == dim, "nv_window_attn: values that are the keys have the keys' size");
  const int cw = values_are_keys ? kv_heads * dim : kv_heads * (dim + vdim), v_col = values_are_keys ? 0 : kv_heads * dim;
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_window_attn: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 &&
                   block_size > 0 && window >= 0 && chunk >= 0 && table_cols > 0,
               "nv_window_attn: bad shape");
  if (tokens == 0) return NV_OK;
  const int R = heads / kv_heads;
  // bf16 caches with 16-byte-aligned heads of up to 256 numbers: the matrix-core kernel
  if (dtype == NV_BF16 && dim % 8 == 0 && vdim % 8 == 0 && dim <= 256 && vdim <= 256 && R <= 64 && kv_heads <= 65535 &&
      (uintptr_t)cache % 16 == 0 && cw % 8 == 0 && v_col % 8 == 0 && getenv("NV_WINDOW_ATTN_MFMA_OFF") == nullptr) {
    const int ks = dim <= 64 ? 2 : dim <= 128 ? 4 : 8;
    const int ct = vdim <= 32 ? 2 : vdim <= 64 ? 4 : vdim <= 128 ? 8 : 16;
    if (ma_lds_bytes(ks, ct, false) <= 160 * 1024) {
      // one token per request: the wavefronts split the window (where four staging areas fit the LDS)
      const bool split = max_q <= 1 && R <= 16 && ma_lds_bytes(ks, ct, true) <= 156 * 1024;
      const int TQm = max_q <= 1 ? 1 : 64 / R;
      // ... and with few requests several workgroups do, when the caller brought room for their shares
      int ksplit = split ? window_attn_key_splits(tokens, kv_heads) : 1;
      if (ksplit > 1 && (!workspace || workspace_bytes < (size_t)tokens * heads * ksplit * (vdim + 2) * sizeof(float)))
        ksplit = 1;
      WAttnArgs pm{q, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, out_row_stride, tokens, heads,
                   kv_heads, dim, vdim, block_size, window, TQm, MA_KEYS, softcap, out_scale, cw, v_col, distance_term, sink,
                   gate, gate_row_stride, gate_per_head, chunk, ksplit, reinterpret_cast<float*>(workspace)};
      dim3 gridm((unsigned)((tokens + TQm - 1) / TQm), (unsigned)kv_heads, (unsigned)ksplit);
      hipStream_t st = (hipStream_t)stream;
      const hipError_t e = ks == 2 ? launch_window_mfma<2>(pm, ct, split, gridm, st)
                           : ks == 4 ? launch_window_mfma<4>(pm, ct, split, gridm, st)
                                     : launch_window_mfma<8>(pm, ct, split, gridm, st);
      if (e != hipSuccess) {
        nv_set_error("nv_window_attn: %s", hipGetErrorString(e));
        return NV_ERR_LAUNCH;
      }
      if (ksplit > 1) {
        window_attn_join_kernel<<<dim3((unsigned)((tokens * heads + 3) / 4)), dim3(256), 0, st>>>(pm);
        NV_CHECK_LAUNCH();
      }
      return NV_OK;
    }
  }
  const size_t budget = 64 * 1024;
  auto need = [&](int tq, int tk) {
    const size_t rows = (size_t)tq * R;
    return (rows * dim + (size_t)tk * (dim + 1) + (size_t)tk * vdim + rows * tk + rows * vdim + 3 * rows) * sizeof(float);
  };
  int TQ = max_q <= 1 ? 1 : 16, TK = 64;
  while (TK > 8 && need(1, TK) > budget) TK /= 2;
  NV_CHECK_ARG(need(1, TK) <= budget, "nv_window_attn: heads of %d + %d numbers do not fit the LDS plan", dim, vdim);
  while (TQ > 1 && (need(TQ, TK) > budget || TQ * R > 256)) TQ /= 2;
  NV_CHECK_ARG(R <= 256 && kv_heads <= 65535, "nv_window_attn: %d query heads per key head exceed a workgroup", R);
  const int64_t tiles = (tokens + TQ - 1) / TQ;
  WAttnArgs p{q, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, out_row_stride, tokens, heads,
              kv_heads, dim, vdim, block_size, window, TQ, TK, softcap, out_scale, cw, v_col, distance_term, sink, gate,
              gate_row_stride, gate_per_head, chunk, 1, nullptr};
  dim3 grid((unsigned)tiles, (unsigned)kv_heads);
  NV_DISPATCH_T(dtype, window_attn_kernel<T><<<grid, dim3(256), need(TQ, TK), (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
