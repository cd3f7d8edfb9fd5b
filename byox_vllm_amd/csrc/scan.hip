// Recurrences with an fp32 state per request, and the short causal convolution that feeds them.  All of them walk the
// tokens a step brings for a request in order, starting from the request's slot (or from zero when the request has no
// tokens behind it) and leaving the state there, so a prompt, its portions and single decoded tokens go one way.
//
// causal_conv:  out[t][c] = act(bias[c] + sum_j w[c][j] * x[t - (taps - 1 - j)][c]); the slot keeps the last
//               taps - 1 inputs of every channel.  act 2 adds the token's own input: out = x[t] + conv(x)[t].
// rglru_scan:   a = exp(-c * sigmoid(gr) * softplus(lam)),  S = a S + sqrt(1 - a^2) * sigmoid(gi) * u,
//               out = S * gelu_tanh(y) * out_scale: the real-gated linear recurrent unit of the Griffin block.
// mingru_scan:  z = sigmoid(zl),  S = (1 - z) S + z c(u),  c(u) = u + 1/2 for u >= 0 and sigmoid(u) below,
//               out = S * silu(g): the minimal gated recurrent unit, whose gates read the current token only.
// ssd_scan:     per head, S [N, P]:  S = exp(-exp(A_log) dt) S + dt B x^T,  y = S^T C + D x,  dt = softplus(raw + bias);
//               out = y * silu(z): the selective state-space recurrence of Mamba-2 in its token-by-token form.
#include "anyt.h"

namespace {

constexpr int CONV_MAX_TAPS = 8;

__device__ __forceinline__ float softplus_f32(float z) { return fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z))); }

struct ConvArgs {
  const float* x;         // [tokens, x_rs] inputs (fp32 projections)
  const void* x_bias;     // [C] added to every input before anything else (the slot keeps inputs with it), or null
  int64_t x_rs;
  const void* w;          // [C, taps]
  const void* bias;       // [C] or null
  float* state;           // [slots, taps - 1, C]
  const int32_t* cu_q;
  const int32_t* past;
  const int32_t* slots;
  const int32_t* seq_of;
  float* out_f32;         // [tokens, of_rs] or null
  int64_t of_rs;
  void* out_t;            // [tokens, ot_rs] in the storage type, or null
  int64_t ot_rs;
  int C, taps, act;       // act 0: none, 1: SiLU, 2: none, and the token's own input is added to the result
  int heads_only;         // 1: blockIdx.x counts requests; only the tokens that reach back over a portion's start are served
  int64_t tokens;
};

// One thread per (token, channel).  Only a portion's first taps - 1 tokens need the slot; they are all served by the
// thread of the portion's FIRST token, which afterwards writes the slot's new contents: every access to a slot's
// channel comes from one thread, in program order.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(ConvArgs p) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= p.C) return;
  if (p.heads_only && p.cu_q[blockIdx.x + 1] <= p.cu_q[blockIdx.x]) return;
  const int64_t t = p.heads_only ? p.cu_q[blockIdx.x] : blockIdx.x;
  const int b = p.heads_only ? blockIdx.x : p.seq_of[t];
  const int64_t t0 = p.cu_q[b];
  const int k = (int)(t - t0), taps = p.taps, keep = taps - 1;
  if (k > 0 && k < keep) return;
  const T* w = reinterpret_cast<const T*>(p.w) + (int64_t)c * taps;
  const float bias = p.bias ? ld_f32<T>(reinterpret_cast<const T*>(p.bias) + c) : 0.0f;
  const float xb = p.x_bias ? ld_f32<T>(reinterpret_cast<const T*>(p.x_bias) + c) : 0.0f;
  float wt[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) wt[j] = j < taps ? ld_f32<T>(w + j) : 0.0f;
  auto emit = [&](int64_t tt, float v) {
    if (p.act == 1) v = silu_f32(v);
    if (p.act == 2) v += p.x[tt * p.x_rs + c] + xb;
    if (p.out_f32) p.out_f32[tt * p.of_rs + c] = v;
    if (p.out_t) st_f32<T>(reinterpret_cast<T*>(p.out_t) + tt * p.ot_rs + c, v);
  };
  if (k >= keep) {
    float v = bias;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
      if (j < taps) v += wt[j] * (p.x[(t - (keep - j)) * p.x_rs + c] + xb);
    emit(t, v);
    return;
  }
  // k == 0: the tokens that reach back over the portion's start
  const int n = p.cu_q[b + 1] - (int)t0;
  float* slot = p.state + (int64_t)p.slots[b] * keep * p.C;
  const bool fresh = p.past[b] == 0;
  float st[CONV_MAX_TAPS];
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) st[i] = (i < keep && !fresh) ? slot[(int64_t)i * p.C + c] : 0.0f;
  const int head = min(keep, n);
  for (int kk = 0; kk < head; ++kk) {
    float v = bias;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
      if (j >= taps) continue;
      const int src = kk - (keep - j);
      v += wt[j] * (src >= 0 ? p.x[(t0 + src) * p.x_rs + c] + xb : st[kk + j]);
    }
    emit(t0 + kk, v);
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    if (i >= keep) continue;
    const int src = n - keep + i;
    slot[(int64_t)i * p.C + c] = src >= 0 ? p.x[(t0 + src) * p.x_rs + c] + xb : st[i + n];
  }
}

// The tokens that lie at least taps - 1 rows behind their portion's start need no slot: a thread takes four channels
// and CONV_TT consecutive tokens of the packed batch, keeps the last taps rows in registers and moves 16 bytes per
// access.  (The others, and the slots, are served by causal_conv_kernel with heads_only.)  C % 4 == 0, aligned rows.
constexpr int CONV_TT = 8;

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_rows_kernel(ConvArgs p) {
  const int c4 = blockIdx.y * blockDim.x + threadIdx.x;
  if (c4 * 4 >= p.C) return;
  const int c = c4 * 4, taps = p.taps, keep = taps - 1;
  const int64_t t_begin = (int64_t)blockIdx.x * CONV_TT, t_end = min(p.tokens, t_begin + CONV_TT);
  f32x4 wt[CONV_MAX_TAPS], win[CONV_MAX_TAPS];
  const T* w = reinterpret_cast<const T*>(p.w);
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) wt[j][i] = j < taps ? ld_f32<T>(w + (int64_t)(c + i) * taps + j) : 0.0f;
  f32x4 bias = f32x4{0.f, 0.f, 0.f, 0.f}, xb = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (p.bias) bias[i] = ld_f32<T>(reinterpret_cast<const T*>(p.bias) + c + i);
    if (p.x_bias) xb[i] = ld_f32<T>(reinterpret_cast<const T*>(p.x_bias) + c + i);
  }
  auto row = [&](int64_t tt) {
    f32x4 v = *reinterpret_cast<const f32x4*>(p.x + max(tt, (int64_t)0) * p.x_rs + c);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += xb[i];
    return v;
  };
  // inside the walk win[CONV_MAX_TAPS - 1] is the current token's row and win[CONV_MAX_TAPS - 1 - m] the row m tokens
  // back; before it the window stands one token earlier
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    const int back = CONV_MAX_TAPS - i;
    win[i] = (back >= 1 && back <= keep) ? row(t_begin - back) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int64_t tt = t_begin; tt < t_end; ++tt) {
#pragma unroll
    for (int i = 0; i + 1 < CONV_MAX_TAPS; ++i) win[i] = win[i + 1];
    win[CONV_MAX_TAPS - 1] = row(tt);
    const int b = p.seq_of[tt];
    if ((int)(tt - p.cu_q[b]) < keep) continue;          // reaches back over its portion's start
    f32x4 v = bias;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {            // tap j reads the row keep - j tokens back
      const int idx = CONV_MAX_TAPS - 1 - (keep - j);
      if (j < taps && idx >= 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += wt[j][i] * win[idx][i];
      }
    }
    if (p.act == 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = silu_f32(v[i]);
    }
    if (p.act == 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += win[CONV_MAX_TAPS - 1][i];
    }
    if (p.out_f32) *reinterpret_cast<f32x4*>(p.out_f32 + tt * p.of_rs + c) = v;
    if (p.out_t) {
      T* dst = reinterpret_cast<T*>(p.out_t) + tt * p.ot_rs + c;
#pragma unroll
      for (int i = 0; i < 4; ++i) st_f32<T>(dst + i, v[i]);
    }
  }
}

struct RglruArgs {
  const float* u;         // [tokens, u_rs] convolution output
  int64_t u_rs;
  const float* gates;     // [tokens, g_rs]: per block of bw channels, bw recurrence-gate logits then bw input-gate logits
  int64_t g_rs;
  const float* y;         // [tokens, y_rs] the other branch before its activation
  const void* y_bias;     // [C] added to y first, or null
  int64_t y_rs;
  const void* lam;        // [C]
  float* state;           // [slots, C]
  const int32_t* cu_q;
  const int32_t* past;
  const int32_t* slots;
  void* out;              // [tokens, out_rs]
  int64_t out_rs;
  int C, bw;
  float c, out_scale;
};

// The recurrence S_t = a_t S_(t-1) + b_t is a composition of affine maps, so a request's tokens are cut into RG_CHUNKS
// runs that are walked side by side: thread (channel, run) first folds its run into one map (A, B), the maps of the
// earlier runs applied to the slot's value give the run's incoming state, and a second walk writes the outputs.
// A step of one token per request costs one run's walk; a prompt's walk is RG_CHUNKS times shorter than the prompt.
constexpr int RG_CHUNKS = 16, RG_CH = 64;

// the walk both gated recurrences share: step(t, a, b) gives the token's map S -> a S + b, emit(t, S) writes its output
template <typename Step, typename Emit>
__device__ __forceinline__ void affine_scan(const int32_t* cu_q, const int32_t* past, const int32_t* slots, float* state,
                                            int C, Step step, Emit emit) {
  __shared__ float sA[RG_CHUNKS][RG_CH], sB[RG_CHUNKS][RG_CH];
  const int cx = threadIdx.x, j = threadIdx.y;
  const int ch = blockIdx.x * RG_CH + cx;
  const int b = blockIdx.y;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  if (t1 <= t0) return;
  const bool on = ch < C;
  const int len = (t1 - t0 + RG_CHUNKS - 1) / RG_CHUNKS;
  const int64_t c0 = min((int64_t)t1, (int64_t)t0 + (int64_t)j * len), c1 = min((int64_t)t1, c0 + len);
  float A = 1.0f, B = 0.0f;
  if (on && t1 - t0 > 1) {
    for (int64_t t = c0; t < c1; ++t) {
      float a, inp;
      step(t, a, inp);
      A *= a;
      B = a * B + inp;
    }
  }
  sA[j][cx] = A;
  sB[j][cx] = B;
  __syncthreads();
  if (!on) return;
  float* slot = state + (int64_t)slots[b] * C + ch;
  float S = past[b] == 0 ? 0.0f : *slot;
  if (t1 - t0 > 1)
    for (int jj = 0; jj < j; ++jj) S = sA[jj][cx] * S + sB[jj][cx];
  for (int64_t t = c0; t < c1; ++t) {
    float a, inp;
    step(t, a, inp);
    S = a * S + inp;
    emit(t, S);
  }
  if (c1 == t1 && c1 > c0) *slot = S;      // the run that holds the step's last token
}

template <typename T>
__global__ __launch_bounds__(RG_CHUNKS * RG_CH) void rglru_scan_kernel(RglruArgs p) {
  const int ch = blockIdx.x * RG_CH + threadIdx.x;
  const bool on = ch < p.C;
  const float sp = on ? p.c * softplus_f32(ld_f32<T>(reinterpret_cast<const T*>(p.lam) + ch)) : 0.0f;
  const int gcol = on ? (ch / p.bw) * 2 * p.bw + ch % p.bw : 0;
  const float yb = (on && p.y_bias) ? ld_f32<T>(reinterpret_cast<const T*>(p.y_bias) + ch) : 0.0f;
  T* out = reinterpret_cast<T*>(p.out);
  affine_scan(
      p.cu_q, p.past, p.slots, p.state, p.C,
      [&](int64_t t, float& a, float& inp) {
        const float gr = p.gates[t * p.g_rs + gcol], gi = p.gates[t * p.g_rs + gcol + p.bw];
        const float log_a = -sp * sigmoid_f32(gr);
        a = expf(log_a);
        // sqrt(1 - a^2) through expm1: 1 - exp(2 log a) loses its digits when the decay is close to one
        inp = sqrtf(-expm1f(2.0f * log_a)) * sigmoid_f32(gi) * p.u[t * p.u_rs + ch];
      },
      [&](int64_t t, float S) {
        st_f32<T>(out + t * p.out_rs + ch, S * gelu_tanh_f32(p.y[t * p.y_rs + ch] + yb) * p.out_scale);
      });
}

struct MinGruArgs {
  const float* proj;      // [tokens, proj_rs] fp32 projections: update-gate logits, candidates and output-gate logits
  int64_t proj_rs;
  int z_off, u_off, g_off;   // at these columns, C of each
  const void* z_bias;     // [C] or null
  const void* u_bias;     // [C] or null
  float* state;           // [slots, C]
  const int32_t* cu_q;
  const int32_t* past;
  const int32_t* slots;
  void* out;              // [tokens, out_rs]
  int64_t out_rs;
  int C;
};

template <typename T>
__global__ __launch_bounds__(RG_CHUNKS * RG_CH) void mingru_scan_kernel(MinGruArgs p) {
  const int ch = blockIdx.x * RG_CH + threadIdx.x;
  const bool on = ch < p.C;
  const float zb = (on && p.z_bias) ? ld_f32<T>(reinterpret_cast<const T*>(p.z_bias) + ch) : 0.0f;
  const float ub = (on && p.u_bias) ? ld_f32<T>(reinterpret_cast<const T*>(p.u_bias) + ch) : 0.0f;
  T* out = reinterpret_cast<T*>(p.out);
  affine_scan(
      p.cu_q, p.past, p.slots, p.state, p.C,
      [&](int64_t t, float& a, float& inp) {
        const float* row = p.proj + t * p.proj_rs;
        const float zl = row[p.z_off + ch] + zb, u = row[p.u_off + ch] + ub;
        a = sigmoid_f32(-zl);                      // 1 - sigmoid(zl), without the cancellation
        inp = sigmoid_f32(zl) * (u >= 0.0f ? u + 0.5f : sigmoid_f32(u));
      },
      [&](int64_t t, float S) { st_f32<T>(out + t * p.out_rs + ch, S * silu_f32(p.proj[t * p.proj_rs + p.g_off + ch])); });
}

struct SsdArgs {
  const float* xbc;       // [tokens, xbc_rs]: x (H * P) | B (G * N) | C (G * N), after convolution and activation
  int64_t xbc_rs;
  const float* z;         // [tokens, z_rs] gate, H * P
  int64_t z_rs;
  const float* dt;        // [tokens, dt_rs] raw step sizes, H
  int64_t dt_rs;
  const void* dt_bias;    // [H]
  const void* A_log;      // [H]
  const void* D;          // [H]
  float* state;           // [slots, H, N, P]
  const int32_t* cu_q;
  const int32_t* past;
  const int32_t* slots;
  float* out;             // [tokens, H * P]
  int H, G, N, P, parts;
  // long prompts: runs of run_len tokens are walked side by side (see ssd_scan_kernel)
  float* ws_state;        // [B * H * runs][N * P] state at the end of each run
  float* ws_decay;        // [B * H * runs] product of the run's decays
  int runs, run_len, pass;
};

// One workgroup per (request, head, run); thread (part, v) keeps S[part + parts * i][v], i < DPT, in registers.  Tokens
// are staged `tc` at a time: step sizes and decays first, then dt * B, C and x rows in LDS; the walk over the staged
// tokens needs no barrier (each thread leaves its partial y per token in LDS), the partial sums meet once per stage.
//
// S_t = decay_t S_(t-1) + U_t is an affine map of the state with a scalar factor, so a long prompt is cut into runs
// that are walked side by side.  Pass 1: run 0 starts from the request's slot and is final; every other run starts
// from zero, writes nothing but its end state E_j and the product D_j of its decays.  Pass 2: run j >= 1 starts from
// S = E_0, S <- D_i S + E_i for 0 < i < j, and walks again, now writing its outputs; the run that holds the step's last
// token leaves the state in the slot (nobody reads the slot in pass 2).  runs == 1 is the plain walk.
template <typename T, int DPT>
__global__ __launch_bounds__(1024) void ssd_scan_kernel(SsdArgs p, int tc) {
  extern __shared__ float lds[];
  const int N = p.N, P = p.P, parts = p.parts;
  float* sB = lds;                       // [tc][N] dt * B
  float* sC = sB + tc * N;               // [tc][N]
  float* sx = sC + tc * N;               // [tc][P]
  float* so = sx + tc * P;               // [tc][parts][P]
  float* sdt = so + tc * parts * P;      // [tc]
  float* sdec = sdt + tc;                // [tc]
  const int h = blockIdx.x, b = blockIdx.y;
  const int j = blockIdx.z + (p.pass == 2 ? 1 : 0);
  const int tid = threadIdx.x, bd = blockDim.x;
  const bool active = tid < parts * P;
  const int v = tid % P, part = tid / P;
  const int t0 = p.cu_q[b], t1 = p.cu_q[b + 1];
  const int64_t cb = p.runs > 1 ? (int64_t)t0 + (int64_t)j * p.run_len : t0;
  const int64_t ce = p.runs > 1 ? min((int64_t)t1, cb + p.run_len) : t1;
  if (cb >= ce) return;
  const bool emit = p.pass == 2 || j == 0;
  const int grp = h / (p.H / p.G);
  float* S_g = p.state + ((int64_t)p.slots[b] * p.H + h) * N * P;
  const int64_t wrow = ((int64_t)b * p.H + h) * p.runs;
  const bool fresh = p.past[b] == 0;
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int n = part * DPT + i;
    const bool mine = active && n < N;
    if (j == 0) S[i] = (mine && !fresh) ? S_g[(int64_t)n * P + v] : 0.0f;
    else if (p.pass == 1) S[i] = 0.0f;
    else S[i] = mine ? p.ws_state[wrow * N * P + (int64_t)n * P + v] : 0.0f;
  }
  if (p.pass == 2) {
    for (int r = 1; r < j; ++r) {
      const float Dr = p.ws_decay[wrow + r];
      const float* E = p.ws_state + (wrow + r) * N * P;
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        const int n = part * DPT + i;
        if (active && n < N) S[i] = Dr * S[i] + E[(int64_t)n * P + v];
      }
    }
  }
  const float rate = expf(ld_f32<T>(reinterpret_cast<const T*>(p.A_log) + h));
  const float dtb = ld_f32<T>(reinterpret_cast<const T*>(p.dt_bias) + h);
  const float Dh = ld_f32<T>(reinterpret_cast<const T*>(p.D) + h);
  const int inner = p.H * P;
  const bool vec4 = N % 4 == 0;
  float dt_sum = 0.0f;
  for (int64_t c0 = cb; c0 < ce; c0 += tc) {
    const int nt = (int)min((int64_t)tc, ce - c0);
    if (tid < nt) {
      const float dt = softplus_f32(p.dt[(c0 + tid) * p.dt_rs + h] + dtb);
      sdt[tid] = dt;
      sdec[tid] = expf(-rate * dt);
    }
    __syncthreads();
    for (int i = tid; i < nt * N; i += bd) {
      const int tt = i / N, n = i % N;
      const float* row = p.xbc + (c0 + tt) * p.xbc_rs;
      sB[i] = sdt[tt] * row[inner + grp * N + n];
      sC[i] = row[inner + p.G * N + grp * N + n];
    }
    for (int i = tid; i < nt * P; i += bd) sx[i] = p.xbc[(c0 + i / P) * p.xbc_rs + h * P + i % P];
    __syncthreads();
    if (active) {
      for (int tt = 0; tt < nt; ++tt) {
        const float xv = sx[tt * P + v], decay = sdec[tt];
        const float* Bt = sB + tt * N;
        const float* Ct = sC + tt * N;
        dt_sum += sdt[tt];
        float o = 0.0f;
        if (vec4) {           // four state rows per LDS read (the rows of a thread are consecutive)
#pragma unroll
          for (int i = 0; i < DPT; i += 4) {
            const int n = part * DPT + i;
            if (n < N) {
              const f32x4 b4 = *reinterpret_cast<const f32x4*>(Bt + n), c4 = *reinterpret_cast<const f32x4*>(Ct + n);
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                S[i + e] = decay * S[i + e] + b4[e] * xv;
                o += S[i + e] * c4[e];
              }
            }
          }
        } else {
#pragma unroll
          for (int i = 0; i < DPT; ++i) {
            const int n = part * DPT + i;
            if (n < N) {
              S[i] = decay * S[i] + Bt[n] * xv;
              o += S[i] * Ct[n];
            }
          }
        }
        so[(tt * parts + part) * P + v] = o;
      }
    }
    __syncthreads();
    if (emit) {
      for (int i = tid; i < nt * P; i += bd) {
        const int tt = i / P, e = i % P;
        float y = Dh * sx[i];
        for (int q = 0; q < parts; ++q) y += so[(tt * parts + q) * P + e];
        p.out[(c0 + tt) * inner + h * P + e] = y * silu_f32(p.z[(c0 + tt) * p.z_rs + h * P + e]);
      }
    }
  }
  if (active) {
    const bool to_slot = emit && ce == t1;
    const bool to_ws = p.runs > 1 && p.pass == 1;
    float* E = p.ws_state + (wrow + j) * N * P;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int n = part * DPT + i;
      if (n < N) {
        if (to_slot) S_g[(int64_t)n * P + v] = S[i];
        if (to_ws) E[(int64_t)n * P + v] = S[i];
      }
    }
    if (to_ws && tid == 0) p.ws_decay[wrow + j] = expf(-rate * dt_sum);
  }
}

}  // namespace

extern "C" int nv_causal_conv(const float* x, const void* x_bias, int64_t x_row_stride, const void* w, const void* bias, float* state,
                              const int32_t* cu_q, const int32_t* past_lens, const int32_t* state_slots,
                              const int32_t* seq_of_token, float* out_f32, int64_t out_f32_row_stride, void* out_t,
                              int64_t out_t_row_stride, int64_t tokens, int channels, int taps, int act, int dtype,
                              nv_stream_t stream) {
  return nv_causal_conv_batch(x, x_bias, x_row_stride, w, bias, state, cu_q, past_lens, state_slots, seq_of_token, out_f32,
                              out_f32_row_stride, out_t, out_t_row_stride, tokens, 0, channels, taps, act, dtype, stream);
}

extern "C" int nv_causal_conv_batch(const float* x, const void* x_bias, int64_t x_row_stride, const void* w,
                                    const void* bias, float* state, const int32_t* cu_q, const int32_t* past_lens,
                                    const int32_t* state_slots, const int32_t* seq_of_token, float* out_f32,
                                    int64_t out_f32_row_stride, void* out_t, int64_t out_t_row_stride, int64_t tokens,
                                    int num_seqs, int channels, int taps, int act, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(x && w && (state || taps == 1) && cu_q && past_lens && state_slots && seq_of_token && (out_f32 || out_t),
               "nv_causal_conv: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_causal_conv: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && tokens < (1ll << 31) && channels > 0 && taps >= 1 && taps <= CONV_MAX_TAPS &&
                   act >= 0 && act <= 2,
               "nv_causal_conv: bad shape (taps up to %d)", CONV_MAX_TAPS);
  if (tokens == 0) return NV_OK;
  ConvArgs p{x, x_bias, x_row_stride, w, bias, state, cu_q, past_lens, state_slots, seq_of_token, out_f32, out_f32_row_stride,
             out_t, out_t_row_stride, channels, taps, act, 0, tokens};
  // with the number of requests known: one launch over the requests for the tokens that need the slot, and (where a
  // request brings more tokens than that) one over all rows, four channels and several tokens per thread
  const size_t tsz = dtype == NV_BF16 ? 2 : 4;
  if (num_seqs > 0 && num_seqs <= 65535 && channels % 4 == 0 && x_row_stride % 4 == 0 && (uintptr_t)x % 16 == 0 &&
      (!out_f32 || (out_f32_row_stride % 4 == 0 && (uintptr_t)out_f32 % 16 == 0)) &&
      (!out_t || ((out_t_row_stride * tsz) % 8 == 0 && (uintptr_t)out_t % 8 == 0))) {
    p.heads_only = 1;
    NV_DISPATCH_T(dtype, causal_conv_kernel<T><<<dim3((unsigned)num_seqs, (unsigned)((channels + 255) / 256)), dim3(256), 0,
                                                 (hipStream_t)stream>>>(p));
    NV_CHECK_LAUNCH();
    if (tokens > num_seqs) {
      const int c4 = channels / 4, threads = c4 >= 256 ? 256 : ((c4 + 63) / 64) * 64;
      NV_DISPATCH_T(dtype, causal_conv_rows_kernel<T><<<dim3((unsigned)((tokens + CONV_TT - 1) / CONV_TT),
                                                            (unsigned)((c4 + threads - 1) / threads)),
                                                       dim3(threads), 0, (hipStream_t)stream>>>(p));
      NV_CHECK_LAUNCH();
    }
    return NV_OK;
  }
  NV_DISPATCH_T(dtype, causal_conv_kernel<T><<<dim3((unsigned)tokens, (unsigned)((channels + 255) / 256)), dim3(256), 0,
                                               (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_rglru_scan(const float* u, int64_t u_row_stride, const float* gates, int64_t gates_row_stride,
                             const float* y, const void* y_bias, int64_t y_row_stride, const void* lam, float* state, const int32_t* cu_q,
                             const int32_t* past_lens, const int32_t* state_slots, void* out, int64_t out_row_stride,
                             int num_seqs, int channels, int block_width, float c, float out_scale, int dtype,
                             nv_stream_t stream) {
  NV_CHECK_ARG(u && gates && y && lam && state && cu_q && past_lens && state_slots && out, "nv_rglru_scan: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_rglru_scan: bad dtype %d", dtype);
  NV_CHECK_ARG(num_seqs >= 0 && num_seqs <= 65535 && channels > 0 && block_width > 0 && channels % block_width == 0,
               "nv_rglru_scan: bad shape");
  if (num_seqs == 0) return NV_OK;
  RglruArgs p{u, u_row_stride, gates, gates_row_stride, y, y_bias, y_row_stride, lam, state, cu_q, past_lens, state_slots, out,
              out_row_stride, channels, block_width, c, out_scale};
  NV_DISPATCH_T(dtype, rglru_scan_kernel<T><<<dim3((unsigned)((channels + RG_CH - 1) / RG_CH), (unsigned)num_seqs),
                                              dim3(RG_CH, RG_CHUNKS), 0, (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_mingru_scan(const float* proj, int64_t proj_row_stride, int z_off, int u_off, int g_off,
                              const void* z_bias, const void* u_bias, float* state, const int32_t* cu_q,
                              const int32_t* past_lens, const int32_t* state_slots, void* out, int64_t out_row_stride,
                              int num_seqs, int channels, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(proj && state && cu_q && past_lens && state_slots && out, "nv_mingru_scan: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_mingru_scan: bad dtype %d", dtype);
  NV_CHECK_ARG(num_seqs >= 0 && num_seqs <= 65535 && channels > 0 && z_off >= 0 && u_off >= 0 && g_off >= 0,
               "nv_mingru_scan: bad shape");
  if (num_seqs == 0) return NV_OK;
  MinGruArgs p{proj, proj_row_stride, z_off, u_off, g_off, z_bias, u_bias, state, cu_q, past_lens, state_slots, out,
               out_row_stride, channels};
  NV_DISPATCH_T(dtype, mingru_scan_kernel<T><<<dim3((unsigned)((channels + RG_CH - 1) / RG_CH), (unsigned)num_seqs),
                                               dim3(RG_CH, RG_CHUNKS), 0, (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

// runs a request of max_q tokens is cut into, and their length.  Runs cost every token a second walk, so they pay only
// while (requests x heads) leaves most of the chip idle.
static void ssd_runs(int num_seqs, int heads, int max_q, int* runs, int* run_len) {
  *runs = 1;
  *run_len = max_q > 0 ? max_q : 1;
  if (max_q < 256 || (int64_t)num_seqs * heads >= 128) return;
  int len = 128;
  if ((max_q + len - 1) / len > 64) len = ((max_q + 63) / 64 + 15) / 16 * 16;
  *run_len = len;
  *runs = (max_q + len - 1) / len;
}

extern "C" size_t nv_ssd_scan_workspace_bytes(int num_seqs, int heads, int state_size, int vdim, int max_q) {
  int runs, len;
  ssd_runs(num_seqs, heads, max_q, &runs, &len);
  return runs > 1 ? (size_t)num_seqs * heads * runs * ((size_t)state_size * vdim + 1) * sizeof(float) : 0;
}

extern "C" int nv_ssd_scan(const float* xbc, int64_t xbc_row_stride, const float* z, int64_t z_row_stride, const float* dt,
                           int64_t dt_row_stride, const void* dt_bias, const void* A_log, const void* D, float* state,
                           const int32_t* cu_q, const int32_t* past_lens, const int32_t* state_slots, float* out,
                           int num_seqs, int heads, int groups, int state_size, int vdim, int max_q, void* workspace,
                           size_t workspace_bytes, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(xbc && z && dt && dt_bias && A_log && D && state && cu_q && past_lens && state_slots && out,
               "nv_ssd_scan: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_ssd_scan: bad dtype %d", dtype);
  NV_CHECK_ARG(num_seqs >= 0 && num_seqs <= 65535 && heads > 0 && groups > 0 && heads % groups == 0 && state_size > 0 &&
                   vdim > 0 && vdim <= 1024,
               "nv_ssd_scan: bad shape");
  if (num_seqs == 0) return NV_OK;
  // threads: vdim columns times `parts` slices of the state rows; each thread keeps up to DPT rows of its column
  int parts = 1024 / vdim;
  if (parts > state_size) parts = state_size;
  if (parts > 8) parts = 8;
  const int per = (state_size + parts - 1) / parts;
  NV_CHECK_ARG(per <= 64, "nv_ssd_scan: a state of %d x %d exceeds one workgroup's registers", state_size, vdim);
  int runs, run_len;
  ssd_runs(num_seqs, heads, max_q, &runs, &run_len);
  if (runs > 1) {
    NV_CHECK_ARG(workspace && workspace_bytes >= nv_ssd_scan_workspace_bytes(num_seqs, heads, state_size, vdim, max_q),
                 "nv_ssd_scan: %d runs need a workspace of nv_ssd_scan_workspace_bytes", runs);
  }
  float* ws_state = reinterpret_cast<float*>(workspace);
  float* ws_decay = runs > 1 ? ws_state + (size_t)num_seqs * heads * runs * state_size * vdim : nullptr;
  SsdArgs p{xbc, xbc_row_stride, z, z_row_stride, dt, dt_row_stride, dt_bias, A_log, D, state, cu_q, past_lens,
            state_slots, out, heads, groups, state_size, vdim, parts, ws_state, ws_decay, runs, run_len, 1};
  const int threads = ((parts * vdim + 63) / 64) * 64;
  // tokens per stage: as many as fit 48 KB of LDS, at most 16
  auto need = [&](int tc) { return (size_t)tc * (2 * state_size + vdim + parts * vdim + 2) * sizeof(float); };
  int tc = 16;
  while (tc > 1 && need(tc) > 48 * 1024) tc /= 2;
  NV_CHECK_ARG(need(tc) <= 64 * 1024, "nv_ssd_scan: a token of %d + %d numbers does not fit the LDS", state_size, vdim);
  const size_t lds = need(tc);
  hipStream_t s = (hipStream_t)stream;
  for (int pass = 1; pass <= (runs > 1 ? 2 : 1); ++pass) {
    p.pass = pass;
    dim3 grid((unsigned)heads, (unsigned)num_seqs, (unsigned)(pass == 1 ? runs : runs - 1));
    if (per <= 4) NV_DISPATCH_T(dtype, ssd_scan_kernel<T, 4><<<grid, dim3(threads), lds, s>>>(p, tc));
    else if (per <= 16) NV_DISPATCH_T(dtype, ssd_scan_kernel<T, 16><<<grid, dim3(threads), lds, s>>>(p, tc));
    else NV_DISPATCH_T(dtype, ssd_scan_kernel<T, 64><<<grid, dim3(threads), lds, s>>>(p, tc));
    NV_CHECK_LAUNCH();
  }
  return NV_OK;
}
