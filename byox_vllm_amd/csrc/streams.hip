// Kernels around a residual that is kept as several fp32 streams (hyper-connections): the embedding with sinusoidal
// positions written into every stream, the norm that first folds the previous sublayer's output into the streams and
// then reads their weighted sum, and the token shift that mixes a norm's output with its predecessor's.
//
// Streams are stored [tokens, S, width] in fp32.  A sublayer with parameters in[S], out[S], mix[S, S] reads
// u = sum_s in[s] x_s and, once its output y is known, replaces the streams by x'_t = sum_s mix[s, t] x_s + out[t] y.
// The replacement is carried out by the NEXT norm launch (every norm follows a sublayer), so the streams are read and
// written once per sublayer.  With S = 1, in = out = mix = 1 this is the ordinary residual sum.
#include "anyt.h"

namespace {

constexpr int HC_MAX_STREAMS = 8;

template <typename T>
__global__ __launch_bounds__(256) void embed_sinusoid_kernel(const int64_t* __restrict__ ids,
                                                             const int64_t* __restrict__ positions,
                                                             const T* __restrict__ table,
                                                             const double* __restrict__ inv_freq,
                                                             float* __restrict__ out, int S, int width, int64_t vocab) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;
  const T* row = table + id * width;
  const double pos = (double)positions[t];
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    // the angle is formed and reduced in double: a float angle of a position in the thousands is already off by 1e-4
    const double a = pos * inv_freq[j >> 1];
    const float v = ld_f32<T>(row + j) + (float)((j & 1) ? cos(a) : sin(a));
    for (int s = 0; s < S; ++s) out[(t * S + s) * width + j] = v;
  }
}

struct HcArgs {
  float* x;                // [tokens, S, W]
  const float* delta;      // [tokens, delta_rs] output of the previous sublayer, or null
  int64_t delta_rs;
  const float* hc_prev;    // in[S] | out[S] | mix[S, S] of the previous sublayer (read when delta is given)
  const float* hc_in;      // in[S] of this sublayer; null: plain sum of the streams
  const void* w;           // [W] norm weight
  const int32_t* rows_idx; // gather (the streams are then left as they are)
  void* out;
  int64_t out_rs;
  int S, W, one_plus;
  float eps;
};

template <int V> struct VecOfFloats { typedef float type __attribute__((ext_vector_type(V))); };
template <> struct VecOfFloats<1> { typedef float type; };

// V numbers per thread and step: 4 (16-byte accesses to the streams) when the width and the strides allow it, else 1.
template <typename T, typename TO, int V>
__global__ __launch_bounds__(256) void hc_norm_kernel(HcArgs p) {
  extern __shared__ float su[];      // [W] the weighted sum of the streams
  __shared__ float red[32];
  typedef typename VecOfFloats<V>::type vec;
  const int64_t i = blockIdx.x;
  const int64_t r = p.rows_idx ? p.rows_idx[i] : i;
  const int S = p.S, W = p.W;
  float* xr = p.x + r * S * W;
  const float* po = p.hc_prev ? p.hc_prev + S : nullptr;
  const float* pm = p.hc_prev ? p.hc_prev + 2 * S : nullptr;
  float ss = 0.0f;
  for (int j = threadIdx.x * V; j < W; j += blockDim.x * V) {
    vec xs[HC_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HC_MAX_STREAMS; ++s) xs[s] = s < S ? *reinterpret_cast<const vec*>(xr + (int64_t)s * W + j) : vec(0.0f);
    if (p.delta) {
      const vec y = *reinterpret_cast<const vec*>(p.delta + r * p.delta_rs + j);
      vec nx[HC_MAX_STREAMS];
#pragma unroll
      for (int t = 0; t < HC_MAX_STREAMS; ++t) {
        vec v = vec(0.0f);
        if (t < S) {
          if (pm) {
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s)
              if (s < S) v += pm[s * S + t] * xs[s];
            v += po[t] * y;
          } else {
            v = xs[t] + y;
          }
          if (!p.rows_idx) *reinterpret_cast<vec*>(xr + (int64_t)t * W + j) = v;
        }
        nx[t] = v;
      }
#pragma unroll
      for (int s = 0; s < HC_MAX_STREAMS; ++s) xs[s] = nx[s];
    }
    vec u = vec(0.0f);
#pragma unroll
    for (int s = 0; s < HC_MAX_STREAMS; ++s)
      if (s < S) u += p.hc_in ? p.hc_in[s] * xs[s] : xs[s];
    *reinterpret_cast<vec*>(su + j) = u;
    if constexpr (V == 1) {
      ss += u * u;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) ss += u[e] * u[e];
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  const T* w = reinterpret_cast<const T*>(p.w);
  TO* out = reinterpret_cast<TO*>(p.out) + i * p.out_rs;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    const float g = ld_f32<T>(w + j) + (p.one_plus ? 1.0f : 0.0f);
    st_f32<TO>(out + j, su[j] * inv * g);
  }
}

// out[t] = h[t] + (h[t-1] - h[t]) * mu, with h[t-1] taken from the request's slot at the start of a portion (zeros for
// a request without tokens behind it).  The workgroup of a portion's first token is the only one that reads the slot;
// the same threads then leave the portion's last row there, so no other workgroup's read can meet that write.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const float* __restrict__ h, const T* __restrict__ mu,
                                                          float* __restrict__ state, const int32_t* __restrict__ cu_q,
                                                          const int32_t* __restrict__ past,
                                                          const int32_t* __restrict__ slots,
                                                          const int32_t* __restrict__ seq_of, T* __restrict__ out,
                                                          int W) {
  const int64_t t = blockIdx.x;
  const int b = seq_of[t];
  const bool first = t == cu_q[b];
  const int64_t last = cu_q[b + 1] - 1;
  float* slot = state + (int64_t)slots[b] * W;
  const bool fresh = past[b] == 0;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    const float hv = h[t * W + j];
    float pv;
    if (first) {
      pv = fresh ? 0.0f : slot[j];
      slot[j] = h[last * W + j];
    } else {
      pv = h[(t - 1) * W + j];
    }
    st_f32<T>(out + t * W + j, hv + (pv - hv) * ld_f32<T>(mu + j));
  }
}

// rows of `groups` equal parts, each divided by its own root mean square and multiplied by its slice of w (and, with
// gate logits of the same layout, by their sigmoid)
template <typename T>
__global__ __launch_bounds__(256) void group_rmsnorm_f32_kernel(const float* __restrict__ x, int64_t x_rs,
                                                                const T* __restrict__ w, T* __restrict__ out,
                                                                int64_t out_rs, int groups, int n, float eps,
                                                                const float* __restrict__ gate, int64_t gate_rs) {
  __shared__ float red[32];
  const int64_t t = blockIdx.x / groups;
  const int g = blockIdx.x % groups;
  const float* xr = x + t * x_rs + (int64_t)g * n;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < n; j += blockDim.x) ss += xr[j] * xr[j];
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    float v = xr[j] * inv * ld_f32<T>(w + (int64_t)g * n + j);
    if (gate) v *= sigmoid_f32(gate[t * gate_rs + (int64_t)g * n + j]);
    st_f32<T>(out + t * out_rs + (int64_t)g * n + j, v);
  }
}

// the same for parts of at most 256 numbers: one wavefront per part, four parts per workgroup, no LDS
template <typename T>
__global__ __launch_bounds__(256) void group_rmsnorm_f32_wave_kernel(const float* __restrict__ x, int64_t x_rs,
                                                                     const T* __restrict__ w, T* __restrict__ out,
                                                                     int64_t out_rs, int64_t parts, int groups, int n,
                                                                     float eps, const float* __restrict__ gate,
                                                                     int64_t gate_rs) {
  const int64_t part = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (part >= parts) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = part / groups;
  const int g = (int)(part % groups);
  const float* xr = x + t * x_rs + (int64_t)g * n;
  float v[4], ss = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int j = lane + 64 * i;
    v[i] = j < n ? xr[j] : 0.0f;
    ss += v[i] * v[i];
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int j = lane + 64 * i;
    if (j >= n) continue;
    float y = v[i] * inv * ld_f32<T>(w + (int64_t)g * n + j);
    if (gate) y *= sigmoid_f32(gate[t * gate_rs + (int64_t)g * n + j]);
    st_f32<T>(out + t * out_rs + (int64_t)g * n + j, y);
  }
}

}  // namespace

extern "C" int nv_embed_sinusoid(const int64_t* ids, const int64_t* positions, const void* table, const double* inv_freq,
                                 float* out, int64_t tokens, int streams, int width, int64_t vocab, int dtype,
                                 nv_stream_t stream) {
  NV_CHECK_ARG(ids && positions && table && inv_freq && out, "nv_embed_sinusoid: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_embed_sinusoid: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && width > 0 && vocab > 0 && streams > 0, "nv_embed_sinusoid: bad shape");
  if (tokens == 0) return NV_OK;
  NV_DISPATCH_T(dtype, embed_sinusoid_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           ids, positions, (const T*)table, inv_freq, out, streams, width, vocab));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_hc_norm(float* x, int streams, int width, const float* delta, int64_t delta_row_stride,
                          const float* hc_prev, const float* hc_in, const void* w, int one_plus, float eps,
                          const int32_t* rows_idx, void* out, int64_t out_row_stride, int out_dtype, int64_t rows,
                          int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(x && w && out, "nv_hc_norm: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_hc_norm: bad dtype %d", dtype);
  NV_CHECK_ARG(out_dtype == NV_F32 || out_dtype == dtype, "nv_hc_norm: the output is fp32 or the model's type");
  NV_CHECK_ARG(rows >= 0 && width > 0 && streams >= 1 && streams <= HC_MAX_STREAMS, "nv_hc_norm: bad shape");
  NV_CHECK_ARG((size_t)width * sizeof(float) <= 64 * 1024, "nv_hc_norm: width %d exceeds the LDS row", width);
  if (rows == 0) return NV_OK;
  HcArgs p{x, delta, delta_row_stride, hc_prev, hc_in, w, rows_idx, out, out_row_stride, streams, width, one_plus, eps};
  const size_t lds = (size_t)width * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const bool vec = width % 4 == 0 && (uintptr_t)x % 16 == 0 &&
                   (!delta || ((uintptr_t)delta % 16 == 0 && delta_row_stride % 4 == 0));
  const dim3 g((unsigned)rows), b(256);
  if (vec) {
    if (dtype == NV_F32) hc_norm_kernel<float, float, 4><<<g, b, lds, s>>>(p);
    else if (out_dtype == NV_F32) hc_norm_kernel<bf16_t, float, 4><<<g, b, lds, s>>>(p);
    else hc_norm_kernel<bf16_t, bf16_t, 4><<<g, b, lds, s>>>(p);
  } else {
    if (dtype == NV_F32) hc_norm_kernel<float, float, 1><<<g, b, lds, s>>>(p);
    else if (out_dtype == NV_F32) hc_norm_kernel<bf16_t, float, 1><<<g, b, lds, s>>>(p);
    else hc_norm_kernel<bf16_t, bf16_t, 1><<<g, b, lds, s>>>(p);
  }
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_token_shift(const float* h, const void* mu, float* state, const int32_t* cu_q, const int32_t* past_lens,
                              const int32_t* state_slots, const int32_t* seq_of_token, void* out, int64_t tokens,
                              int width, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(h && mu && state && cu_q && past_lens && state_slots && seq_of_token && out, "nv_token_shift: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_token_shift: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && width > 0, "nv_token_shift: bad shape");
  if (tokens == 0) return NV_OK;
  NV_DISPATCH_T(dtype, token_shift_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           h, (const T*)mu, state, cu_q, past_lens, state_slots, seq_of_token, (T*)out, width));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_group_rmsnorm_f32(const float* x, int64_t x_row_stride, const void* w, void* out, int64_t out_row_stride,
                                    int64_t rows, int groups, int n, float eps, const float* gate,
                                    int64_t gate_row_stride, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(x && w && out, "nv_group_rmsnorm_f32: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_group_rmsnorm_f32: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && n > 0 && groups > 0 && rows * groups < (1ll << 31), "nv_group_rmsnorm_f32: bad shape");
  if (rows == 0) return NV_OK;
  if (n <= 256 && groups > 1) {
    const int64_t parts = rows * groups;
    NV_DISPATCH_T(dtype, group_rmsnorm_f32_wave_kernel<T><<<dim3((unsigned)((parts + 3) / 4)), dim3(256), 0,
                                                            (hipStream_t)stream>>>(
                             x, x_row_stride, (const T*)w, (T*)out, out_row_stride, parts, groups, n, eps, gate,
                             gate_row_stride));
    NV_CHECK_LAUNCH();
    return NV_OK;
  }
  NV_DISPATCH_T(dtype, group_rmsnorm_f32_kernel<T><<<dim3((unsigned)(rows * groups)), dim3(256), 0, (hipStream_t)stream>>>(
                           x, x_row_stride, (const T*)w, (T*)out, out_row_stride, groups, n, eps, gate, gate_row_stride));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
