// nv_linear: out = epilogue(A W^T + bias) for any shape, in bf16 or true fp32 storage, fp32 accumulation on the matrix
// cores (v_mfma_f32_16x16x32_bf16 / v_mfma_f32_16x16x4_f32).  One entry point covers the shapes the tiled decode GEMM
// (nv_gemm) does not take: K or N that are no multiples of its tiles, fp32 models, batched products with one weight
// per head, grouped products with one weight per expert over gathered rows, and the gated epilogues.
//
// A workgroup owns a 64 x 64 tile of the output: wavefront w the 16 columns n0 + 16 w .. and all four 16-row
// sub-tiles.  Operands go from memory straight into MFMA fragments (both are K-contiguous rows, which is the fragment
// layout: lane (c, g) holds row c, k = k0 + 8 g .. + 8), so there is no LDS stage; the 4 wavefronts re-read the A rows
// through the L1.  D[n][m] is accumulated (the weight fragment is the first operand), which leaves every lane with
// four consecutive output columns.
#include <stdlib.h>

#include "anyt.h"

namespace {

struct LinArgs {
  const void* a;
  int64_t a_rs;
  const int32_t* a_rows;
  const void* w;
  int64_t w_rs;
  const void* bias;
  void* out;
  int64_t out_rs;
  int64_t M;
  int N, K;
  int64_t a_bs, w_bs, out_bs, bias_bs;
  const int32_t* group_off;
  const float* epi_ptr;
  int64_t epi_rs;
  float epi_c;
  int act;
  int vec_a, vec_w;
};

enum { EPI_NONE = 0, EPI_GLU = 1, EPI_SOFTCAP = 2, EPI_ROW_GATE = 3, EPI_ACT = 4 };

// EPI_ACT: an element-wise function of the product.  act 0 SiLU, 1 tanh-form GELU, 2 xIELU with its two positive
// coefficients at epi_ptr (a z^2 + z/2 above zero, b (exp(z) - 1 - z) + z/2 below), 3 multiplication by epi_c.
__device__ __forceinline__ float unary_act(float v, int act, const float* prm, float c) {
  switch (act) {
    case 0: return silu_f32(v);
    case 1: return gelu_tanh_f32(v);
    case 2: return v > 0.0f ? prm[0] * v * v + 0.5f * v : prm[1] * (expm1f(v) - v) + 0.5f * v;
    default: return v * c;
  }
}

template <typename T> struct Frag;
template <> struct Frag<bf16_t> {
  typedef bf16x8 type;
  static constexpr int KS = 32, PER = 8;
};
template <> struct Frag<float> {
  typedef f32x4 type;
  static constexpr int KS = 16, PER = 4;
};

template <typename T>
__device__ __forceinline__ typename Frag<T>::type load_frag(const T* row, int k, int K, bool vec) {
  typedef typename Frag<T>::type F;
  F r;
  if (row == nullptr) {
#pragma unroll
    for (int e = 0; e < Frag<T>::PER; ++e) r[e] = (T)0.0f;
    return r;
  }
  if (vec && k + Frag<T>::PER <= K) return *reinterpret_cast<const F*>(row + k);
#pragma unroll
  for (int e = 0; e < Frag<T>::PER; ++e) r[e] = (k + e < K) ? row[k + e] : (T)0.0f;
  return r;
}

__device__ __forceinline__ f32x4 mma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma(f32x4 a, f32x4 b, f32x4 c) {
  // lane group g supplies k = k0 + 4 g + e in step e: over the four steps the sixteen k of the block are each used once
#pragma unroll
  for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
  return c;
}

template <typename T, typename TO, int EPI>
__global__ __launch_bounds__(256) void linear_kernel(LinArgs p) {
  typedef typename Frag<T>::type F;
  constexpr int KS = Frag<T>::KS, PER = Frag<T>::PER;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int z = blockIdx.z;
  int64_t lo = 0, hi = p.M;
  if (p.group_off) {
    lo = p.group_off[z];
    hi = p.group_off[z + 1];
  }
  const int64_t mbase = lo + (int64_t)blockIdx.y * 64;
  if (mbase >= hi) return;
  const int nsub = (int)((hi - mbase + 15) / 16 < 4 ? (hi - mbase + 15) / 16 : 4);
  const int n0 = blockIdx.x * 64 + wv * 16;
  if (n0 >= p.N) return;

  const T* A = reinterpret_cast<const T*>(p.a) + z * p.a_bs;
  const T* W = reinterpret_cast<const T*>(p.w) + z * p.w_bs;
  const T* wrow = (n0 + c < p.N) ? W + (int64_t)(n0 + c) * p.w_rs : nullptr;
  const T* urow = nullptr;
  if constexpr (EPI == EPI_GLU) urow = (n0 + c < p.N) ? W + (int64_t)(p.N + n0 + c) * p.w_rs : nullptr;
  const T* arow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t s = mbase + 16 * i + c;
    arow[i] = nullptr;
    if (s < hi) arow[i] = A + (int64_t)(p.a_rows ? p.a_rows[s] : s) * p.a_rs;
  }
  f32x4 acc[4], accu[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = accu[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (nsub == 1) {
    // Few rows (decode): the loop would be one dependent weight load per k-step.  UNR k-steps per round: all fragments
    // of a round are requested before the first MFMA waits for one, so the memory latency is paid once per round.
    constexpr int UNR = 4;
    for (int k0 = 0; k0 < p.K; k0 += KS * UNR) {
      F wf[UNR], uf[UNR], xf[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int k = k0 + u * KS + PER * g;
        wf[u] = load_frag<T>(wrow, k, p.K, p.vec_w);
        if constexpr (EPI == EPI_GLU) uf[u] = load_frag<T>(urow, k, p.K, p.vec_w);
        xf[u] = load_frag<T>(arow[0], k, p.K, p.vec_a);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        acc[0] = mma(wf[u], xf[u], acc[0]);
        if constexpr (EPI == EPI_GLU) accu[0] = mma(uf[u], xf[u], accu[0]);
      }
    }
  } else {
    for (int k0 = 0; k0 < p.K; k0 += KS) {
      const int k = k0 + PER * g;
      const F wf = load_frag<T>(wrow, k, p.K, p.vec_w);
      F uf;
      if constexpr (EPI == EPI_GLU) uf = load_frag<T>(urow, k, p.K, p.vec_w);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (i < nsub) {
          const F xf = load_frag<T>(arow[i], k, p.K, p.vec_a);
          acc[i] = mma(wf, xf, acc[i]);
          if constexpr (EPI == EPI_GLU) accu[i] = mma(uf, xf, accu[i]);
        }
      }
    }
  }

  TO* O = reinterpret_cast<TO*>(p.out) + z * p.out_bs;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + z * p.bias_bs : nullptr;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t s = mbase + 16 * i + c;
    if (i >= nsub || s >= hi) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + 4 * g + r;
      if (n >= p.N) continue;
      float v = acc[i][r];
      if (bias) v += ld_f32<T>(bias + n);
      if constexpr (EPI == EPI_GLU) {
        const float u = accu[i][r];
        v = glu_act(v, u, p.act, p.epi_c);
      } else if constexpr (EPI == EPI_SOFTCAP) {
        v = p.epi_c * tanhf(v / p.epi_c);
      } else if constexpr (EPI == EPI_ROW_GATE) {
        v *= sigmoid_f32(p.epi_ptr[s * p.epi_rs + (p.act ? (int64_t)z * p.N + n : z)]);
      } else if constexpr (EPI == EPI_ACT) {
        v = unary_act(v, p.act, p.epi_ptr, p.epi_c);
      }
      st_f32<TO>(O + s * p.out_rs + n, v);
    }
  }
}


// Many rows (prefill, expert groups): a 128 x 128 output tile per workgroup, operands staged through LDS in K-blocks of
// 32 (two buffers: the next block is fetched into registers while the current one is multiplied), wavefront (wm, wn)
// owns 64 x 64 of the tile.  With the gated epilogue the weight tile holds 64 gate rows and their 64 up rows, and a
// wavefront owns 64 x 32 of gate and of up.  bf16 operands whose rows split into 16-byte pieces only.
constexpr int TBM = 128, TBK = 32, TST = 40;    // LDS row stride in elements (80 bytes: 16-byte aligned, spreads banks)

template <typename TO, int EPI>
__global__ __launch_bounds__(256) void linear_tile_kernel(LinArgs p) {
  constexpr bool GLU = EPI == EPI_GLU;
  constexpr int NOUT = GLU ? 64 : 128;          // output columns per workgroup
  constexpr int NJ = GLU ? 2 : 4;               // 16-column sub-tiles per wavefront
  __shared__ __attribute__((aligned(16))) bf16_t sA[2][TBM * TST];
  __shared__ __attribute__((aligned(16))) bf16_t sW[2][TBM * TST];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, g = lane >> 4, wm = wv >> 1, wn = wv & 1;
  const int z = blockIdx.z;
  int64_t lo = 0, hi = p.M;
  if (p.group_off) {
    lo = p.group_off[z];
    hi = p.group_off[z + 1];
  }
  const int64_t mbase = lo + (int64_t)blockIdx.y * TBM;
  if (mbase >= hi) return;
  const int n0 = blockIdx.x * NOUT;
  const bf16_t* A = reinterpret_cast<const bf16_t*>(p.a) + z * p.a_bs;
  const bf16_t* W = reinterpret_cast<const bf16_t*>(p.w) + z * p.w_bs;
  // this thread's two 16-byte pieces of each operand tile: rows r0 and r0 + 64, K offset 8 * ch
  const int r0 = tid >> 2, ch = tid & 3;
  const bf16_t* ap[2];
  const bf16_t* wp[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = r0 + 64 * h;
    const int64_t s = mbase + r;
    ap[h] = s < hi ? A + (int64_t)(p.a_rows ? p.a_rows[s] : s) * p.a_rs + 8 * ch : nullptr;
    int wrow;                                    // weight row behind tile row r
    if constexpr (GLU) wrow = r < 64 ? n0 + r : p.N + n0 + (r - 64);
    else wrow = n0 + r;
    const bool in = GLU ? (n0 + (r & 63) < p.N) : (wrow < p.N);
    wp[h] = in ? W + (int64_t)wrow * p.w_rs + 8 * ch : nullptr;
  }
  auto fetch = [&](const bf16_t* q, int k0) -> u32x4 {
    if (q == nullptr || k0 + 8 * ch + 8 > p.K) {
      u32x4 v = u32x4{0u, 0u, 0u, 0u};
      if (q != nullptr && k0 + 8 * ch < p.K) {      // a K that is no multiple of 32 ends inside this piece
        uint16_t* e = reinterpret_cast<uint16_t*>(&v);
        for (int i = 0; i < 8 && k0 + 8 * ch + i < p.K; ++i) e[i] = reinterpret_cast<const uint16_t*>(q + k0)[i];
      }
      return v;
    }
    return *reinterpret_cast<const u32x4*>(q + k0);
  };
  f32x4 acc[4][NJ], accu[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = accu[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 ra[2], rw[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    ra[h] = fetch(ap[h], 0);
    rw[h] = fetch(wp[h], 0);
  }
  int buf = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    *reinterpret_cast<u32x4*>(&sA[0][(r0 + 64 * h) * TST + 8 * ch]) = ra[h];
    *reinterpret_cast<u32x4*>(&sW[0][(r0 + 64 * h) * TST + 8 * ch]) = rw[h];
  }
  __syncthreads();
  for (int k0 = 0; k0 < p.K; k0 += TBK) {
    const bool more = k0 + TBK < p.K;
    if (more) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        ra[h] = fetch(ap[h], k0 + TBK);
        rw[h] = fetch(wp[h], k0 + TBK);
      }
    }
    bf16x8 af[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const bf16x8*>(&sA[buf][(64 * wm + 16 * i + c) * TST + 8 * g]);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int wr = GLU ? 32 * wn + 16 * j : 64 * wn + 16 * j;
      const bf16x8 wf = *reinterpret_cast<const bf16x8*>(&sW[buf][(wr + c) * TST + 8 * g]);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i][j] = mma(wf, af[i], acc[i][j]);
      if constexpr (GLU) {
        const bf16x8 uf = *reinterpret_cast<const bf16x8*>(&sW[buf][(64 + wr + c) * TST + 8 * g]);
#pragma unroll
        for (int i = 0; i < 4; ++i) accu[i][j] = mma(uf, af[i], accu[i][j]);
      }
    }
    if (more) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        *reinterpret_cast<u32x4*>(&sA[buf ^ 1][(r0 + 64 * h) * TST + 8 * ch]) = ra[h];
        *reinterpret_cast<u32x4*>(&sW[buf ^ 1][(r0 + 64 * h) * TST + 8 * ch]) = rw[h];
      }
    }
    __syncthreads();
    buf ^= 1;
  }

  TO* O = reinterpret_cast<TO*>(p.out) + z * p.out_bs;
  const bf16_t* bias = p.bias ? reinterpret_cast<const bf16_t*>(p.bias) + z * p.bias_bs : nullptr;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t s = mbase + 64 * wm + 16 * i + c;
    if (s >= hi) continue;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + (GLU ? 32 * wn : 64 * wn) + 16 * j + 4 * g + r;
        if (n >= p.N) continue;
        float v = acc[i][j][r];
        if (bias) v += ld_f32<bf16_t>(bias + n);
        if constexpr (GLU) {
          v = glu_act(v, accu[i][j][r], p.act, p.epi_c);
        } else if constexpr (EPI == EPI_SOFTCAP) {
          v = p.epi_c * tanhf(v / p.epi_c);
        } else if constexpr (EPI == EPI_ROW_GATE) {
          v *= sigmoid_f32(p.epi_ptr[s * p.epi_rs + (p.act ? (int64_t)z * p.N + n : z)]);
        } else if constexpr (EPI == EPI_ACT) {
          v = unary_act(v, p.act, p.epi_ptr, p.epi_c);
        }
        st_f32<TO>(O + s * p.out_rs + n, v);
      }
    }
  }
}

template <typename TO>
int launch_tile(const LinArgs& p, int epi, int batch, hipStream_t s) {
  const unsigned my = (unsigned)((p.M + TBM - 1) / TBM);
  if (epi == EPI_GLU) linear_tile_kernel<TO, EPI_GLU><<<dim3((p.N + 63) / 64, my, batch), dim3(256), 0, s>>>(p);
  else if (epi == EPI_NONE) linear_tile_kernel<TO, EPI_NONE><<<dim3((p.N + 127) / 128, my, batch), dim3(256), 0, s>>>(p);
  else if (epi == EPI_SOFTCAP) linear_tile_kernel<TO, EPI_SOFTCAP><<<dim3((p.N + 127) / 128, my, batch), dim3(256), 0, s>>>(p);
  else if (epi == EPI_ACT) linear_tile_kernel<TO, EPI_ACT><<<dim3((p.N + 127) / 128, my, batch), dim3(256), 0, s>>>(p);
  else linear_tile_kernel<TO, EPI_ROW_GATE><<<dim3((p.N + 127) / 128, my, batch), dim3(256), 0, s>>>(p);
  return 0;
}


// Up to 64 rows per (group of) product: the launch is bound by how many weight loads are in flight, so the four
// wavefronts of a workgroup share ONE 16-column tile and split K between them (four times the workgroups of the
// general kernel, a quarter of the dependent rounds each); the partial sums meet in LDS and wavefront 0 finishes.
// NSUB = 16-row sub-tiles (1: at most 16 rows, 4: at most 64).
template <typename T, typename TO, int EPI, int NSUB>
__global__ __launch_bounds__(256) void linear_fewrow_kernel(LinArgs p) {
  typedef typename Frag<T>::type F;
  constexpr int KS = Frag<T>::KS, PER = Frag<T>::PER, UNR = 4;
  constexpr bool GLU = EPI == EPI_GLU;
  __shared__ float part[GLU ? 2 : 1][4][NSUB][256];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int z = blockIdx.z;
  int64_t lo = 0, hi = p.M;
  if (p.group_off) {
    lo = p.group_off[z];
    hi = p.group_off[z + 1];
  }
  if (lo >= hi) return;
  const int nsub = (int)((hi - lo + 15) / 16 < NSUB ? (hi - lo + 15) / 16 : NSUB);
  const int n0 = blockIdx.x * 16;
  const T* A = reinterpret_cast<const T*>(p.a) + z * p.a_bs;
  const T* W = reinterpret_cast<const T*>(p.w) + z * p.w_bs;
  const T* wrow = (n0 + c < p.N) ? W + (int64_t)(n0 + c) * p.w_rs : nullptr;
  const T* urow = nullptr;
  if constexpr (GLU) urow = (n0 + c < p.N) ? W + (int64_t)(p.N + n0 + c) * p.w_rs : nullptr;
  const T* arow[NSUB];
#pragma unroll
  for (int i = 0; i < NSUB; ++i) {
    const int64_t s = lo + 16 * i + c;
    arow[i] = s < hi ? A + (int64_t)(p.a_rows ? p.a_rows[s] : s) * p.a_rs : nullptr;
  }
  // this wavefront's share of K, in whole rounds
  const int round = KS * UNR;
  const int rounds = (p.K + round - 1) / round;
  const int k_lo = ((rounds * wv) / 4) * round, k_hi = min(p.K, ((rounds * (wv + 1)) / 4) * round);
  f32x4 acc[NSUB], accu[NSUB];
#pragma unroll
  for (int i = 0; i < NSUB; ++i) acc[i] = accu[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = k_lo; k0 < k_hi; k0 += round) {
    F wf[UNR], uf[UNR], xf[NSUB][UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int k = k0 + u * KS + PER * g;
      wf[u] = load_frag<T>(wrow, k, k_hi, p.vec_w);
      if constexpr (GLU) uf[u] = load_frag<T>(urow, k, k_hi, p.vec_w);
#pragma unroll
      for (int i = 0; i < NSUB; ++i)
        if (i < nsub) xf[i][u] = load_frag<T>(arow[i], k, k_hi, p.vec_a);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
#pragma unroll
      for (int i = 0; i < NSUB; ++i) {
        if (i < nsub) {
          acc[i] = mma(wf[u], xf[i][u], acc[i]);
          if constexpr (GLU) accu[i] = mma(uf[u], xf[i][u], accu[i]);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NSUB; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      part[0][wv][i][4 * lane + r] = acc[i][r];
      if constexpr (GLU) part[1][wv][i][4 * lane + r] = accu[i][r];
    }
  }
  __syncthreads();
  if (wv != 0) return;
  TO* O = reinterpret_cast<TO*>(p.out) + z * p.out_bs;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + z * p.bias_bs : nullptr;
#pragma unroll
  for (int i = 0; i < NSUB; ++i) {
    const int64_t s = lo + 16 * i + c;
    if (i >= nsub || s >= hi) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + 4 * g + r;
      if (n >= p.N) continue;
      const int e = 4 * lane + r;
      float v = part[0][0][i][e] + part[0][1][i][e] + part[0][2][i][e] + part[0][3][i][e];
      if (bias) v += ld_f32<T>(bias + n);
      if constexpr (GLU) {
        const float u = part[1][0][i][e] + part[1][1][i][e] + part[1][2][i][e] + part[1][3][i][e];
        v = glu_act(v, u, p.act, p.epi_c);
      } else if constexpr (EPI == EPI_SOFTCAP) {
        v = p.epi_c * tanhf(v / p.epi_c);
      } else if constexpr (EPI == EPI_ROW_GATE) {
        v *= sigmoid_f32(p.epi_ptr[s * p.epi_rs + (p.act ? (int64_t)z * p.N + n : z)]);
      } else if constexpr (EPI == EPI_ACT) {
        v = unary_act(v, p.act, p.epi_ptr, p.epi_c);
      }
      st_f32<TO>(O + s * p.out_rs + n, v);
    }
  }
}

template <typename T, typename TO, int NSUB>
int launch_fewrow(const LinArgs& p, int epi, dim3 grid, hipStream_t s) {
  switch (epi) {
    case EPI_NONE: linear_fewrow_kernel<T, TO, EPI_NONE, NSUB><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_GLU: linear_fewrow_kernel<T, TO, EPI_GLU, NSUB><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_SOFTCAP: linear_fewrow_kernel<T, TO, EPI_SOFTCAP, NSUB><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_ACT: linear_fewrow_kernel<T, TO, EPI_ACT, NSUB><<<grid, dim3(256), 0, s>>>(p); break;
    default: linear_fewrow_kernel<T, TO, EPI_ROW_GATE, NSUB><<<grid, dim3(256), 0, s>>>(p); break;
  }
  return 0;
}

template <int NSUB>
void launch_fewrow_any(const LinArgs& p, int epi, dim3 grid, int dtype, int out_dtype, hipStream_t s) {
  if (dtype == NV_BF16) {
    if (out_dtype == NV_BF16) launch_fewrow<bf16_t, bf16_t, NSUB>(p, epi, grid, s);
    else launch_fewrow<bf16_t, float, NSUB>(p, epi, grid, s);
  } else {
    if (out_dtype == NV_BF16) launch_fewrow<float, bf16_t, NSUB>(p, epi, grid, s);
    else launch_fewrow<float, float, NSUB>(p, epi, grid, s);
  }
}

template <typename T, typename TO>
int launch_epi(const LinArgs& p, int epi, dim3 grid, hipStream_t s) {
  switch (epi) {
    case EPI_NONE: linear_kernel<T, TO, EPI_NONE><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_GLU: linear_kernel<T, TO, EPI_GLU><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_SOFTCAP: linear_kernel<T, TO, EPI_SOFTCAP><<<grid, dim3(256), 0, s>>>(p); break;
    case EPI_ACT: linear_kernel<T, TO, EPI_ACT><<<grid, dim3(256), 0, s>>>(p); break;
    default: linear_kernel<T, TO, EPI_ROW_GATE><<<grid, dim3(256), 0, s>>>(p); break;
  }
  return 0;
}

}  // namespace

extern "C" int nv_linear(const void* a, int64_t a_row_stride, const int32_t* a_rows, const void* w, int64_t w_row_stride,
                         const void* bias, void* out, int64_t out_row_stride, int out_dtype, int64_t M, int N, int K,
                         int batch, int64_t a_batch_stride, int64_t w_batch_stride, int64_t out_batch_stride,
                         int64_t bias_batch_stride, const int32_t* group_offsets, int epilogue, int act,
                         const float* epi_ptr, int64_t epi_row_stride, float epi_const, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(a && w && out, "nv_linear: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_linear: dtype %d is neither bf16 nor fp32", dtype);
  NV_CHECK_ARG(out_dtype == NV_BF16 || out_dtype == NV_F32, "nv_linear: bad output dtype %d", out_dtype);
  NV_CHECK_ARG(M >= 0 && N > 0 && K > 0 && batch > 0 && batch <= 65535, "nv_linear: bad shape M=%lld N=%d K=%d batch=%d",
               (long long)M, N, K, batch);
  NV_CHECK_ARG(epilogue >= EPI_NONE && epilogue <= EPI_ACT, "nv_linear: bad epilogue %d", epilogue);
  NV_CHECK_ARG(epilogue != EPI_ACT || (act >= 0 && act <= 3 && (act != 2 || epi_ptr)), "nv_linear: bad activation %d", act);
  NV_CHECK_ARG(epilogue != EPI_ROW_GATE || epi_ptr, "nv_linear: the row-gate epilogue needs its gate rows");
  NV_CHECK_ARG(epilogue != EPI_SOFTCAP || epi_const > 0.0f, "nv_linear: the soft cap must be positive");
  if (M == 0) return NV_OK;
  const int64_t mtiles = (M + 63) / 64;
  NV_CHECK_ARG(mtiles <= 65535, "nv_linear: %lld rows exceed one launch", (long long)M);
  const size_t esz = dtype == NV_BF16 ? 2 : 4;
  const int per = dtype == NV_BF16 ? 8 : 4;
  LinArgs p{a, a_row_stride, a_rows, w, w_row_stride, bias, out, out_row_stride, M, N, K, a_batch_stride,
            w_batch_stride, out_batch_stride, bias_batch_stride, group_offsets, epi_ptr, epi_row_stride, epi_const, act,
            0, 0};
  p.vec_a = (uintptr_t)a % 16 == 0 && a_row_stride % per == 0 && (a_batch_stride * esz) % 16 == 0;
  p.vec_w = (uintptr_t)w % 16 == 0 && w_row_stride % per == 0 && (w_batch_stride * esz) % 16 == 0;
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)mtiles, (unsigned)batch);
  hipStream_t s = (hipStream_t)stream;
  // more than 64 rows of 16-byte-aligned bf16: the LDS-tiled kernel (a group's rows are not known here: M bounds them)
  if (dtype == NV_BF16 && M > 64 && p.vec_a && p.vec_w && K % 8 == 0 && getenv("NV_LINEAR_TILE_OFF") == nullptr) {
    if (out_dtype == NV_BF16) launch_tile<bf16_t>(p, epilogue, batch, s);
    else launch_tile<float>(p, epilogue, batch, s);
    NV_CHECK_LAUNCH();
    return NV_OK;
  }
  // at most 64 rows per product and a K worth splitting: one 16-column tile per workgroup, K split over its wavefronts
  if (M <= 64 && K >= 256 && (N + 15) / 16 <= 1048576) {
    dim3 g16((unsigned)((N + 15) / 16), 1, (unsigned)batch);
    if (M <= 16) launch_fewrow_any<1>(p, epilogue, g16, dtype, out_dtype, s);
    else launch_fewrow_any<4>(p, epilogue, g16, dtype, out_dtype, s);
    NV_CHECK_LAUNCH();
    return NV_OK;
  }
  if (dtype == NV_BF16) {
    if (out_dtype == NV_BF16) launch_epi<bf16_t, bf16_t>(p, epilogue, grid, s);
    else launch_epi<bf16_t, float>(p, epilogue, grid, s);
  } else {
    if (out_dtype == NV_BF16) launch_epi<float, bf16_t>(p, epilogue, grid, s);
    else launch_epi<float, float>(p, epilogue, grid, s);
  }
  NV_CHECK_LAUNCH();
  return NV_OK;
}
