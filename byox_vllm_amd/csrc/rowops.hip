// Row-wise kernels of models whose residual stream lives in fp32: scaled embedding gather, Dynamic Tanh (an
// element-wise norm with no statistics) fused with the residual add, and RMSNorm of fp32 rows.  Parameters are in the
// model's storage type (bf16 or fp32), arithmetic is fp32, outputs round once to the storage type.
#include "anyt.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                          float* __restrict__ out, int width, int64_t vocab,
                                                          float scale) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;
  const T* row = table + id * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[t * width + i] = ld_f32<T>(row + i) * scale;
}

// v = x[r] + delta[r] (when delta is given; written back to x unless rows are gathered), out[i] = tanh(alpha * v) * w + b
// with r = rows_idx ? rows_idx[i] : i
template <typename T>
__global__ __launch_bounds__(256) void dyt_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                  int64_t delta_rs, const int32_t* __restrict__ rows_idx,
                                                  const float* __restrict__ alpha, const T* __restrict__ w,
                                                  const T* __restrict__ b, T* __restrict__ out, int n) {
  const int64_t i = blockIdx.x;
  const int64_t r = rows_idx ? rows_idx[i] : i;
  const float a = alpha[0];
  float* xr = x + r * n;
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    float v = xr[j];
    if (delta) {
      v += delta[r * delta_rs + j];
      if (!rows_idx) xr[j] = v;
    }
    st_f32<T>(out + i * n + j, tanhf(a * v) * ld_f32<T>(w + j) + ld_f32<T>(b + j));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_f32_kernel(const float* __restrict__ x, int64_t x_rs,
                                                          const T* __restrict__ w, T* __restrict__ out, int64_t out_rs,
                                                          int n, float eps) {
  __shared__ float red[32];
  const int64_t r = blockIdx.x;
  const float* xr = x + r * x_rs;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < n; j += blockDim.x) ss += xr[j] * xr[j];
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int j = threadIdx.x; j < n; j += blockDim.x) st_f32<T>(out + r * out_rs + j, xr[j] * inv * ld_f32<T>(w + j));
}

// Post-norm residual with a gate: x[t] += mult * (g / sqrt(mean(g^2) + eps)) * w, g = (y[t] + y_bias) * sigmoid(gate[t] +
// gate_bias) (no gate: g = y + y_bias; y_bias is the bias a producing product left to its consumer, or null); the new
// row is also written in the storage type for the products that read the residual.  Without y the row is only copied.
template <typename T> struct Pack4;
template <> struct Pack4<float> {
  typedef f32x4 type;
  static __device__ __forceinline__ f32x4 widen(const f32x4& v) { return v; }
  static __device__ __forceinline__ f32x4 narrow(const f32x4& v) { return v; }
};
template <> struct Pack4<bf16_t> {
  typedef uint2 type;
  static __device__ __forceinline__ f32x4 widen(const uint2& v) {
    return f32x4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                 __uint_as_float(v.y & 0xffff0000u)};
  }
  static __device__ __forceinline__ uint2 narrow(const f32x4& v) {
    union { bf16_t h[4]; uint2 u; } r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.h[i] = (bf16_t)v[i];
    return r.u;
  }
};

// The input convolution of the NEXT sublayer, for steps in which row t is request t's only token: every earlier row a
// tap reads is in the request's slot, so the launch that makes the new residual row also hands out x + conv(x) and moves
// the slot on (csrc/scan.hip has the general form).
struct NextConv {
  const void* w;          // [n, taps], or null: no convolution in this launch
  float* state;           // [slots, taps - 1, n]
  const int32_t* slots;   // [rows]
  const int32_t* past;    // [rows] tokens the request holds already (0: the slot's contents do not count)
  void* out;              // [rows, out_rs] in the storage type
  int64_t out_rs;
  int taps;
};
constexpr int NEXT_CONV_MAX_TAPS = 8;

// NV > 0: rows of at most NV * 1024 numbers, a multiple of 4, every pointer 16-byte aligned: a thread keeps its gated
// values in registers between the two passes and moves four numbers per access.  NV == 0: any row.
template <typename T, int NV>
__global__ __launch_bounds__(256) void gated_postnorm_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                 int64_t y_rs, const float* __restrict__ gate,
                                                                 int64_t gate_rs, const T* __restrict__ gate_bias,
                                                                 const T* __restrict__ y_bias, const T* __restrict__ w,
                                                                 T* __restrict__ out_t, int64_t out_rs, int n, float eps,
                                                                 float mult, NextConv cv) {
  __shared__ float red[32];
  typedef typename Pack4<T>::type P;
  const int64_t t = blockIdx.x;
  float* xr = x + t * n;
  if (y == nullptr && (NV == 0 || cv.w == nullptr)) {
    if (out_t)
      for (int j = threadIdx.x; j < n; j += blockDim.x) st_f32<T>(out_t + t * out_rs + j, xr[j]);
    return;
  }
  const float* yr = y + t * y_rs;
  const float* gr = gate ? gate + t * gate_rs : nullptr;
  if constexpr (NV > 0) {
    const int n4 = n >> 2;
    f32x4 g[NV];
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int c = threadIdx.x + k * 256;
      g[k] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (c < n4 && y) {
        f32x4 v = reinterpret_cast<const f32x4*>(yr)[c];
        if (y_bias) {
          const f32x4 b = Pack4<T>::widen(reinterpret_cast<const P*>(y_bias)[c]);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] += b[i];
        }
        if (gr) {
          f32x4 z = reinterpret_cast<const f32x4*>(gr)[c];
          if (gate_bias) {
            const f32x4 b = Pack4<T>::widen(reinterpret_cast<const P*>(gate_bias)[c]);
#pragma unroll
            for (int i = 0; i < 4; ++i) z[i] += b[i];
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] *= sigmoid_f32(z[i]);
        }
        g[k] = v;
#pragma unroll
        for (int i = 0; i < 4; ++i) ss += v[i] * v[i];
      }
    }
    if (y) ss = block_sum(ss, red);
    const float inv = mult / sqrtf(ss / (float)n + eps);
    const int keep = cv.taps - 1;
    float* slot = cv.w ? cv.state + (int64_t)cv.slots[t] * keep * n : nullptr;
    const bool fresh = cv.w && cv.past[t] == 0;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int c = threadIdx.x + k * 256;
      if (c < n4) {
        f32x4 v = reinterpret_cast<f32x4*>(xr)[c];
        if (y) {
          const f32x4 wv = Pack4<T>::widen(reinterpret_cast<const P*>(w)[c]);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] += g[k][i] * inv * wv[i];
          reinterpret_cast<f32x4*>(xr)[c] = v;
        }
        if (out_t) reinterpret_cast<P*>(out_t + t * out_rs)[c] = Pack4<T>::narrow(v);
        if (cv.w) {
          // tap j reads the row keep - j tokens back: slot row j for j < keep, the new row for the last tap
          const T* cw = reinterpret_cast<const T*>(cv.w) + (int64_t)c * 4 * cv.taps;
          f32x4 h = v;
#pragma unroll
          for (int i = 0; i < 4; ++i) h[i] += ld_f32<T>(cw + i * cv.taps + keep) * v[i];
#pragma unroll
          for (int j = 0; j < NEXT_CONV_MAX_TAPS - 1; ++j) {
            if (j >= keep) continue;
            f32x4 old = fresh ? f32x4{0.0f, 0.0f, 0.0f, 0.0f} : reinterpret_cast<const f32x4*>(slot + (int64_t)j * n)[c];
#pragma unroll
            for (int i = 0; i < 4; ++i) h[i] += ld_f32<T>(cw + i * cv.taps + j) * old[i];
            if (j > 0) reinterpret_cast<f32x4*>(slot + (int64_t)(j - 1) * n)[c] = old;      // the slot moves on by one row
          }
          if (keep > 0) reinterpret_cast<f32x4*>(slot + (int64_t)(keep - 1) * n)[c] = v;
          reinterpret_cast<P*>(reinterpret_cast<T*>(cv.out) + t * cv.out_rs)[c] = Pack4<T>::narrow(h);
        }
      }
    }
    return;
  }
  auto gated = [&](int j) {
    float v = yr[j] + (y_bias ? ld_f32<T>(y_bias + j) : 0.0f);
    if (gr) v *= sigmoid_f32(gr[j] + (gate_bias ? ld_f32<T>(gate_bias + j) : 0.0f));
    return v;
  };
  float ss = 0.0f;
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    const float v = gated(j);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = mult / sqrtf(ss / (float)n + eps);
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    const float v = xr[j] + gated(j) * inv * ld_f32<T>(w + j);
    xr[j] = v;
    if (out_t) st_f32<T>(out_t + t * out_rs + j, v);
  }
}

// out[t] = [x[t] | x0[t]] in the storage type; x takes delta first
template <typename T>
__global__ __launch_bounds__(256) void residual_pair_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                            int64_t delta_rs, const float* __restrict__ x0,
                                                            T* __restrict__ out, int n) {
  const int64_t t = blockIdx.x;
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    float v = x[t * n + j];
    if (delta) {
      v += delta[t * delta_rs + j];
      x[t * n + j] = v;
    }
    st_f32<T>(out + t * 2 * n + j, v);
    st_f32<T>(out + t * 2 * n + n + j, x0[t * n + j]);
  }
}

// out[m][j] = act(y[m][j]) * y[m][n + j]: the gated unit's activation over a plain product's [gate | up] rows
template <typename T>
__global__ __launch_bounds__(256) void act_mul_f32_kernel(const float* __restrict__ y, T* __restrict__ out, int64_t total,
                                                          int n, int act, float c) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = i / n;
    const int j = (int)(i - m * n);
    const float g = y[m * 2 * n + j], u = y[m * 2 * n + n + j];
    st_f32<T>(out + i, glu_act(g, u, act, c));
  }
}

// out = f(y): the element-wise epilogue of nv_linear applied to a plain product's fp32 result (same function codes)
template <typename T>
__global__ __launch_bounds__(256) void act_f32_kernel(const float* __restrict__ y, T* __restrict__ out, int64_t total,
                                                      int act, const float* __restrict__ prm, float c,
                                                      const T* __restrict__ bias, int n) {
  const float a = act == 2 ? prm[0] : 0.0f, b = act == 2 ? prm[1] : 0.0f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const float v = y[i] + (bias ? ld_f32<T>(bias + i % n) : 0.0f);
    float r;
    switch (act) {
      case 0: r = silu_f32(v); break;
      case 1: r = gelu_tanh_f32(v); break;
      case 2: r = v > 0.0f ? a * v * v + 0.5f * v : b * (expm1f(v) - v) + 0.5f * v; break;
      default: r = v * c; break;
    }
    st_f32<T>(out + i, r);
  }
}

// Gumbel-max sampling from fp32 logits: argmax_j (l_j / T + g_j) with g_j = -log(-log(u_j)), u_j a hash of (seed, row,
// column); temperature 0 takes the plain argmax.  Ties go to the lowest index.
__device__ __forceinline__ uint32_t mix32(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return (uint32_t)x;
}

__global__ __launch_bounds__(256) void sample_f32_kernel(const float* __restrict__ logits, int64_t rs,
                                                         const float* __restrict__ temperatures,
                                                         int64_t* __restrict__ tokens, int V, uint64_t seed) {
  __shared__ float bv[256];
  __shared__ int bi[256];
  const int row = blockIdx.x;
  const float temp = temperatures[row];
  const float* l = logits + row * rs;
  float best = -INFINITY;
  int arg = V;
  for (int j = threadIdx.x; j < V; j += blockDim.x) {
    float v = l[j];
    if (temp > 0.0f) {
      const uint32_t h = mix32(seed * 0x9E3779B97F4A7C15ULL + ((uint64_t)row << 32) + (uint64_t)j);
      const float u = ((float)(h >> 8) + 0.5f) * (1.0f / 16777216.0f);
      v = v / temp - logf(-logf(u));
    }
    if (v > best || arg == V) {
      best = v;
      arg = j;
    }
  }
  bv[threadIdx.x] = best;
  bi[threadIdx.x] = arg;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      const float v2 = bv[threadIdx.x + o];
      const int i2 = bi[threadIdx.x + o];
      if (i2 < V && (bi[threadIdx.x] >= V || v2 > bv[threadIdx.x] || (v2 == bv[threadIdx.x] && i2 < bi[threadIdx.x]))) {
        bv[threadIdx.x] = v2;
        bi[threadIdx.x] = i2;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) tokens[row] = bi[0];
}

}  // namespace

extern "C" int nv_sample_f32(const float* logits, int64_t row_stride, const float* temperatures, int64_t* tokens, int B,
                             int V, uint64_t seed, nv_stream_t stream) {
  NV_CHECK_ARG(logits && temperatures && tokens, "nv_sample_f32: null pointer");
  NV_CHECK_ARG(B >= 0 && V > 0, "nv_sample_f32: bad shape B=%d V=%d", B, V);
  if (B == 0) return NV_OK;
  sample_f32_kernel<<<dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream>>>(logits, row_stride, temperatures, tokens, V,
                                                                              seed);
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_residual_pair(float* x, const float* delta, int64_t delta_row_stride, const float* x0, void* out,
                                int64_t rows, int n, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(x && x0 && out, "nv_residual_pair: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_residual_pair: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && rows < (1ll << 31) && n > 0, "nv_residual_pair: bad shape");
  if (rows == 0) return NV_OK;
  NV_DISPATCH_T(dtype, residual_pair_kernel<T><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
                           x, delta, delta_row_stride, x0, (T*)out, n));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_act_mul_f32(const float* y, void* out, int64_t rows, int n, int act, float c, int dtype,
                              nv_stream_t stream) {
  NV_CHECK_ARG(y && out, "nv_act_mul_f32: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_act_mul_f32: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && n > 0 && act >= 0 && act <= 2 && (act != 2 || c > 0.0f), "nv_act_mul_f32: bad shape or activation");
  if (rows == 0) return NV_OK;
  const int64_t total = rows * n;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  NV_DISPATCH_T(dtype, act_mul_f32_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
                           y, (T*)out, total, n, act, c));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_act_f32(const float* y, void* out, int64_t total, int act, const float* params, float c, int dtype,
                          nv_stream_t stream) {
  return nv_bias_act_f32(y, nullptr, 1, out, total, act, params, c, dtype, stream);
}

extern "C" int nv_bias_act_f32(const float* y, const void* bias, int n, void* out, int64_t total, int act,
                               const float* params, float c, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(y && out && n > 0, "nv_act_f32: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_act_f32: bad dtype %d", dtype);
  NV_CHECK_ARG(total >= 0 && act >= 0 && act <= 3 && (act != 2 || params), "nv_act_f32: bad shape or activation");
  if (total == 0) return NV_OK;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  NV_DISPATCH_T(dtype, act_f32_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
                           y, (T*)out, total, act, params, c, (const T*)bias, n));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_embed_scale(const int64_t* ids, const void* table, float* out, int64_t tokens, int width, int64_t vocab,
                              float scale, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(ids && table && out, "nv_embed_scale: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_embed_scale: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && width > 0 && vocab > 0, "nv_embed_scale: bad shape");
  if (tokens == 0) return NV_OK;
  NV_DISPATCH_T(dtype, embed_scale_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           ids, (const T*)table, out, width, vocab, scale));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_dyt_norm(float* x, const float* delta, int64_t delta_row_stride, const int32_t* rows_idx,
                           const float* alpha, const void* w, const void* b, void* out, int64_t rows, int n, int dtype,
                           nv_stream_t stream) {
  NV_CHECK_ARG(x && alpha && w && b && out, "nv_dyt_norm: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_dyt_norm: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && n > 0, "nv_dyt_norm: bad shape");
  if (rows == 0) return NV_OK;
  NV_DISPATCH_T(dtype, dyt_kernel<T><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
                           x, delta, delta_row_stride, rows_idx, alpha, (const T*)w, (const T*)b, (T*)out, n));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_rmsnorm_f32(const float* x, int64_t x_row_stride, const void* w, void* out, int64_t out_row_stride,
                              int64_t rows, int n, float eps, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(x && w && out, "nv_rmsnorm_f32: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_rmsnorm_f32: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && n > 0, "nv_rmsnorm_f32: bad shape");
  if (rows == 0) return NV_OK;
  NV_DISPATCH_T(dtype, rmsnorm_f32_kernel<T><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
                           x, x_row_stride, (const T*)w, (T*)out, out_row_stride, n, eps));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_gated_postnorm_add(float* x, const float* y, int64_t y_row_stride, const void* y_bias, const float* gate,
                                     int64_t gate_row_stride, const void* gate_bias, const void* w, void* out,
                                     int64_t out_row_stride, int64_t rows, int n, float eps, float mult, int dtype,
                                     nv_stream_t stream) {
  return nv_gated_postnorm_add_conv(x, y, y_row_stride, y_bias, gate, gate_row_stride, gate_bias, w, out, out_row_stride,
                                    rows, n, eps, mult, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0, dtype, stream);
}

extern "C" int nv_gated_postnorm_add_conv_ok(const void* x, int n, int taps) {
  return n % 4 == 0 && n <= 4096 && ((uintptr_t)x & 15) == 0 && taps >= 1 && taps <= NEXT_CONV_MAX_TAPS;
}

extern "C" int nv_gated_postnorm_add_conv(float* x, const float* y, int64_t y_row_stride, const void* y_bias,
                                          const float* gate, int64_t gate_row_stride, const void* gate_bias, const void* w,
                                          void* out, int64_t out_row_stride, int64_t rows, int n, float eps, float mult,
                                          const void* conv_w, int taps, float* conv_state, const int32_t* state_slots,
                                          const int32_t* past_lens, void* conv_out, int64_t conv_out_row_stride, int dtype,
                                          nv_stream_t stream) {
  NV_CHECK_ARG(x && (y == nullptr || w), "nv_gated_postnorm_add: null pointer");
  NV_CHECK_ARG(y || out || conv_w, "nv_gated_postnorm_add: nothing to do");
  NV_CHECK_ARG(!conv_w || ((conv_state || taps == 1) && state_slots && past_lens && conv_out &&
                           nv_gated_postnorm_add_conv_ok(x, n, taps)),
               "nv_gated_postnorm_add: the fused convolution needs its slots, and rows of a multiple of 4 up to 4096");
  NextConv cv{conv_w, conv_state, state_slots, past_lens, conv_out, conv_out_row_stride, taps};
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_gated_postnorm_add: bad dtype %d", dtype);
  NV_CHECK_ARG(rows >= 0 && n > 0, "nv_gated_postnorm_add: bad shape");
  if (rows == 0) return NV_OK;
  auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = (y || conv_w) && n % 4 == 0 && n <= 4096 && al16(x) && al16(y) && al16(gate) && al16(gate_bias) &&
                   al16(y_bias) && al16(w) && al16(out) && al16(conv_state) && al16(conv_out) && y_row_stride % 4 == 0 &&
                   gate_row_stride % 4 == 0 && out_row_stride % 4 == 0 && conv_out_row_stride % 4 == 0;
  NV_CHECK_ARG(vec || !conv_w, "nv_gated_postnorm_add: the fused convolution needs 16-byte aligned rows");
#define NV_POSTNORM(NVAL)                                                                                              \
  NV_DISPATCH_T(dtype, gated_postnorm_add_kernel<T, NVAL><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>( \
                           x, y, y_row_stride, gate, gate_row_stride, (const T*)gate_bias, (const T*)y_bias,           \
                           (const T*)w, (T*)out, out_row_stride, n, eps, mult, cv))
  if (vec && n <= 1024) NV_POSTNORM(1);
  else if (vec && n <= 2048) NV_POSTNORM(2);
  else if (vec) NV_POSTNORM(4);
  else NV_POSTNORM(0);
#undef NV_POSTNORM
  NV_CHECK_LAUNCH();
  return NV_OK;
}
