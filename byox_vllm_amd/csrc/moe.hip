// Mixture-of-experts bookkeeping around the grouped products of nv_linear:
//   nv_moe_route   : per token the `top` largest router logits (fp32) and the softmax over just those (mode 0), or
//                    the softmax over all experts, the chosen scores divided by (their sum + 1e-20) (mode 1)
//   nv_moe_sort    : (token, choice) pairs ordered by expert -> group offsets, the token behind every sorted row and
//                    the sorted row of every pair
//   nv_moe_combine : weighted sum of a token's expert rows (+ a sigmoid-gated shared expert)
// The sum over a token's experts runs in the order of its choices, so it does not depend on what else is in the batch.
#include "anyt.h"

namespace {

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int64_t rs, int E, int top,
                                                        int32_t* __restrict__ idx, float* __restrict__ wt, int64_t T_,
                                                        int mode) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T_) return;
  const float* row = logits + t * rs;
  int32_t* ti = idx + t * top;
  float* tw = wt + t * top;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int arg = -1;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int q = 0; q < j; ++q) taken |= ti[q] == e;
      const float v = row[e];
      if (!taken && (arg < 0 || v > best)) {   // ties go to the lower index
        best = v;
        arg = e;
      }
    }
    ti[j] = arg;
    tw[j] = best;
  }
  const float m = tw[0];   // choices come out in descending order
  if (mode == 1) {         // scores of the softmax over every expert, renormalised over the chosen ones
    float all = 0.0f;
    for (int e = 0; e < E; ++e) all += expf(row[e] - m);
    float sum = 0.0f;
    for (int j = 0; j < top; ++j) {
      tw[j] = expf(tw[j] - m) / all;
      sum += tw[j];
    }
    for (int j = 0; j < top; ++j) tw[j] /= sum + 1e-20f;
    return;
  }
  float sum = 0.0f;
  for (int j = 0; j < top; ++j) {
    tw[j] = expf(tw[j] - m);
    sum += tw[j];
  }
  for (int j = 0; j < top; ++j) tw[j] /= sum;
}

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* __restrict__ idx, int64_t pairs, int E,
                                                        int32_t* __restrict__ offsets, int32_t* __restrict__ sorted_token,
                                                        int32_t* __restrict__ slot_of, int top) {
  extern __shared__ int32_t cnt[];   // [E] counts, then cursors
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int n = cnt[e];
      offsets[e] = run;
      cnt[e] = run;
      run += n;
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int slot = atomicAdd(&cnt[idx[i]], 1);
    sorted_token[slot] = (int32_t)(i / top);
    slot_of[i] = slot;
  }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ slot_of,
                                                          const float* __restrict__ wt, int top,
                                                          const float* __restrict__ shared, const float* __restrict__ sg,
                                                          int64_t sg_rs, float* __restrict__ out, int width) {
  const int64_t t = blockIdx.x;
  const float gate = !shared ? 0.0f : sg ? sigmoid_f32(sg[t * sg_rs]) : 1.0f;   // no gate logits: a plain addend
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float a = 0.0f;
    for (int j = 0; j < top; ++j) a += wt[t * top + j] * y[(int64_t)slot_of[t * top + j] * width + c];
    if (shared) a += gate * shared[t * width + c];
    out[t * width + c] = a;
  }
}

}  // namespace

extern "C" int nv_moe_route(const float* logits, int64_t row_stride, int32_t* idx, float* weights, int64_t tokens,
                            int experts, int top, int mode, nv_stream_t stream) {
  NV_CHECK_ARG(logits && idx && weights, "nv_moe_route: null pointer");
  NV_CHECK_ARG(mode == 0 || mode == 1, "nv_moe_route: bad mode %d", mode);
  NV_CHECK_ARG(tokens >= 0 && experts > 0 && top > 0 && top <= experts, "nv_moe_route: bad shape experts=%d top=%d",
               experts, top);
  if (tokens == 0) return NV_OK;
  moe_route_kernel<<<dim3((unsigned)((tokens + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
      logits, row_stride, experts, top, idx, weights, tokens, mode);
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_moe_sort(const int32_t* idx, int64_t tokens, int experts, int top, int32_t* offsets,
                           int32_t* sorted_token, int32_t* slot_of, nv_stream_t stream) {
  NV_CHECK_ARG(idx && offsets && sorted_token && slot_of, "nv_moe_sort: null pointer");
  NV_CHECK_ARG(tokens >= 0 && experts > 0 && experts <= 8192 && top > 0, "nv_moe_sort: bad shape");
  moe_sort_kernel<<<dim3(1), dim3(1024), (size_t)experts * sizeof(int32_t), (hipStream_t)stream>>>(
      idx, tokens * top, experts, offsets, sorted_token, slot_of, top);
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_moe_combine(const float* y, const int32_t* slot_of, const float* weights, int top, const float* shared,
                              const float* shared_gate, int64_t shared_gate_stride, float* out, int64_t tokens,
                              int width, nv_stream_t stream) {
  NV_CHECK_ARG(y && slot_of && weights && out, "nv_moe_combine: null pointer");
  NV_CHECK_ARG(tokens >= 0 && top > 0 && width > 0, "nv_moe_combine: bad shape");
  if (tokens == 0) return NV_OK;
  moe_combine_kernel<<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(y, slot_of, weights, top, shared,
                                                                                   shared_gate, shared_gate_stride, out,
                                                                                   width);
  NV_CHECK_LAUNCH();
  return NV_OK;
}
