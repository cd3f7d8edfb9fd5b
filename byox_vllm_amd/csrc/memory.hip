// Matrix memories with one decay per head and token: a per-head state S [dim, vdim] in fp32,
//   S_t = keep_t S_(t-1) + take_t k_t v_t^T,   o_t = S_t^T q_t,
// in two forms.
//   MEM_CONST  (lightning attention): keep_t = decay[h], a constant of the head, take_t = 1; q, k, v may pass through
//              SiLU first; o_t leaves as it is.
//   MEM_EXPGATE (the matrix memory of xLSTM): log gates i_t = cap tanh(zi / cap) and f_t = logsigmoid(cap tanh(zf / cap))
//              from one logit each per head, a running maximum m_t = max(f_t + m_(t-1), i_t) that starts at 0,
//              keep_t = exp(f_t + m_(t-1) - m_t), take_t = exp(i_t - m_t); a normaliser n_t = keep_t n_(t-1) + take_t k_t
//              runs beside S, and o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
// A request's slot holds, per head, S (dim x vdim), then in the second form n (dim) and m (1) once per slice of 64 value
// columns.  One workgroup owns one (request, head, slice of 64 state columns) triple - columns are independent of each
// other, so slices need nothing from each other but each keeps its own copy of the normaliser and the maximum; launches
// of many requests give a workgroup all slices of a head instead - and walks the request's tokens of this step in order, starting from the slot (or from zero when
// the request has no tokens behind it) and leaving the state there: a prompt portion, the next portion and single
// decoded tokens all go through this one kernel (states that do not fit a workgroup's registers: a slow general kernel
// that keeps the state in its slot).  The results are fp32 rows; the norm and gate that follow them span
// heads or not, depending on the design, and run in nv_group_rmsnorm_f32.
//
// Thread (cs, v) keeps the entries S[cs * DC .. cs * DC + DC - 1][v] of state column v of its slice in registers (the key channels
// of a column are split over CS threads; their partial o_t meet in LDS once per chunk of tokens).  Tokens are staged
// sixteen at a time: k and q rows in LDS (padded to DMAX with zeros), the thread's own v values in registers; the gates
// of the chunk are a scalar recurrence that one thread walks while the others stage.  Thread d < dim also carries n[d];
// the sixteen n . q meet through wavefront sums.
#include "anyt.h"

namespace {

enum { MEM_CONST = 0, MEM_EXPGATE = 1 };
constexpr int MM_TC = 16;

struct MemArgs {
  const float* proj;     // [tokens, proj_rs]: q | k | v (and the gate logits zi | zf, one per head) at column offsets
  int64_t proj_rs;
  int q_off, k_off, v_off, i_off, f_off;
  const void* bias;      // [proj columns] in the storage type, added to the gate logits; or null
  const float* decay;    // [H] (MEM_CONST)
  float* state;          // [slots, H, per_head]
  const int32_t* cu_q;   // [B + 1] token ranges of the requests in this step
  const int32_t* past;   // [B] tokens each request already holds
  const int32_t* slots;  // [B] state slot of each request
  float* out;            // [tokens, out_rs]: head h at columns h * vdim
  int64_t out_rs;
  int H, dim, vdim, per_head, silu;
  float q_scale, cap;
};

__device__ __forceinline__ float maybe_silu(float z, int on) { return on ? silu_f32(z) : z; }

constexpr int MEM_SLICE = 64;      // state columns that share one copy of n | m

template <typename T, int DMAX, int CS, int MODE>
__global__ __launch_bounds__(256) void matrix_memory_kernel(MemArgs p) {
  constexpr int DC = DMAX / CS;
  extern __shared__ float4 lds4[];
  float* lds = reinterpret_cast<float*>(lds4);
  const int vd = p.vdim;
  // the workgroup covers vdp state columns (a multiple of 64: one slice, or several when the launch has workgroups enough)
  const int tid = threadIdx.x, nthr = blockDim.x, vdp = nthr / CS, nwt = nthr >> 6;
  float* sk = lds;                       // [TC][DMAX]
  float* sq = sk + MM_TC * DMAX;         // [TC][DMAX]
  float* sg = sq + MM_TC * DMAX;         // [3][TC] keep, take, exp(-m)
  float* sred = sg + 3 * MM_TC;          // [TC][wavefronts] partial n . q
  float* so = sred + MM_TC * nwt;        // [CS][TC][vdp] partial outputs (CS > 1)
  const int h = blockIdx.x, b = blockIdx.y;
  const int vl = tid % vdp, cs = tid / vdp;          // column inside the slice, split of the key channels
  const int v = blockIdx.z * vdp + vl;
  const int cb = cs * DC;
  const bool active = v < vd;
  const int col = active ? v : 0;
  const int t0 = p.cu_q[b], t1 = p.cu_q[b + 1];
  if (t1 <= t0) return;
  float* S_g = p.state + ((int64_t)p.slots[b] * p.H + h) * p.per_head;
  const int copy0 = blockIdx.z * (vdp / MEM_SLICE);                     // first of the n | m copies this workgroup owns
  const int ncopies = min(vdp / MEM_SLICE, (vd + MEM_SLICE - 1) / MEM_SLICE - copy0);
  float* n_g = S_g + (int64_t)p.dim * vd + (int64_t)copy0 * (p.dim + 1);
  const bool fresh = p.past[b] == 0;
  float S[DC];
#pragma unroll
  for (int i = 0; i < DC; ++i) S[i] = (active && cb + i < p.dim && !fresh) ? S_g[(int64_t)(cb + i) * vd + v] : 0.0f;
  const bool has_n = MODE == MEM_EXPGATE && tid < p.dim;
  float nreg = (has_n && !fresh) ? n_g[tid] : 0.0f;
  float m_run = (MODE == MEM_EXPGATE && tid == 0 && !fresh) ? n_g[p.dim] : 0.0f;   // walked by thread 0 only
  const float decay = MODE == MEM_CONST ? p.decay[h] : 0.0f;
  const T* bias = reinterpret_cast<const T*>(p.bias);
  for (int c0 = t0; c0 < t1; c0 += MM_TC) {
    const int nt = min(MM_TC, t1 - c0);
    float vreg[MM_TC];
#pragma unroll
    for (int j = 0; j < MM_TC; ++j) {
      vreg[j] = 0.0f;
      if (j < nt) vreg[j] = maybe_silu(p.proj[(int64_t)(c0 + j) * p.proj_rs + p.v_off + h * vd + col], p.silu);
    }
    __syncthreads();                     // the previous chunk's rows are no longer read
    for (int base = tid * 4; base < nt * DMAX; base += nthr * 4) {
      const int j = base / DMAX, i = base % DMAX;          // DMAX is a multiple of 4: the four share a token
      float k4[4], q4[4];
      const float* row = p.proj + (int64_t)(c0 + j) * p.proj_rs;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool in = i + e < p.dim;
        const int ch = h * p.dim + (in ? i + e : 0);
        k4[e] = in ? maybe_silu(row[p.k_off + ch], p.silu) : 0.0f;
        q4[e] = in ? maybe_silu(row[p.q_off + ch], p.silu) * p.q_scale : 0.0f;
      }
      *reinterpret_cast<float4*>(sk + base) = make_float4(k4[0], k4[1], k4[2], k4[3]);
      *reinterpret_cast<float4*>(sq + base) = make_float4(q4[0], q4[1], q4[2], q4[3]);
    }
    // the chunk's gates are a scalar chain: one thread walks it while the others stage
    if (MODE == MEM_EXPGATE && tid == 0) {
      for (int j = 0; j < nt; ++j) {
        const float* row = p.proj + (int64_t)(c0 + j) * p.proj_rs;
        float zi = row[p.i_off + h], zf = row[p.f_off + h];
        if (bias) {
          zi += ld_f32<T>(bias + p.i_off + h);
          zf += ld_f32<T>(bias + p.f_off + h);
        }
        const float ig = p.cap * tanhf(zi / p.cap);
        const float fg = log_sigmoid_f32(p.cap * tanhf(zf / p.cap));
        const float m_new = fmaxf(fg + m_run, ig);
        sg[j] = expf(fg + m_run - m_new);
        sg[MM_TC + j] = expf(ig - m_new);
        sg[2 * MM_TC + j] = expf(-m_new);
        m_run = m_new;
      }
    }
    __syncthreads();
    float o[MM_TC], pn[MM_TC];
#pragma unroll
    for (int j = 0; j < MM_TC; ++j) {
      float acc0 = 0.0f, acc1 = 0.0f;
      pn[j] = 0.0f;
      if (j < nt) {
        const float keep = MODE == MEM_CONST ? decay : sg[j];
        const float take = MODE == MEM_CONST ? 1.0f : sg[MM_TC + j];
        const float vv = vreg[j] * take;
        const float4* k4 = reinterpret_cast<const float4*>(sk + j * DMAX + cb);
        const float4* q4 = reinterpret_cast<const float4*>(sq + j * DMAX + cb);
#pragma unroll
        for (int i = 0; i < DC / 4; ++i) {
          const float4 k = k4[i], q = q4[i];
          S[4 * i + 0] = keep * S[4 * i + 0] + k.x * vv;
          S[4 * i + 1] = keep * S[4 * i + 1] + k.y * vv;
          S[4 * i + 2] = keep * S[4 * i + 2] + k.z * vv;
          S[4 * i + 3] = keep * S[4 * i + 3] + k.w * vv;
          acc0 += S[4 * i + 0] * q.x;
          acc1 += S[4 * i + 1] * q.y;
          acc0 += S[4 * i + 2] * q.z;
          acc1 += S[4 * i + 3] * q.w;
        }
        if (has_n) {
          nreg = keep * nreg + take * sk[j * DMAX + tid];
          pn[j] = nreg * sq[j * DMAX + tid];
        }
      }
      o[j] = acc0 + acc1;
    }
    if constexpr (CS > 1) {
#pragma unroll
      for (int j = 0; j < MM_TC; ++j) so[(cs * MM_TC + j) * vdp + vl] = o[j];
    }
    if constexpr (MODE == MEM_EXPGATE) {
#pragma unroll
      for (int j = 0; j < MM_TC; ++j) {
        const float s = wave_sum(pn[j]);
        if ((tid & 63) == 0) sred[j * nwt + (tid >> 6)] = s;
      }
    }
    if constexpr (CS > 1 || MODE == MEM_EXPGATE) __syncthreads();
    if (cs == 0 && active) {
#pragma unroll
      for (int j = 0; j < MM_TC; ++j) {
        if (j < nt) {
          float r = o[j];
          if constexpr (CS > 1) {
            r = 0.0f;
#pragma unroll
            for (int q = 0; q < CS; ++q) r += so[(q * MM_TC + j) * vdp + vl];
          }
          if constexpr (MODE == MEM_EXPGATE) {
            float nq = 0.0f;
            for (int w = 0; w < nwt; ++w) nq += sred[j * nwt + w];
            r /= fmaxf(fabsf(nq), sg[2 * MM_TC + j]) + 1e-6f;
          }
          p.out[(int64_t)(c0 + j) * p.out_rs + h * vd + v] = r;
        }
      }
    }
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < DC; ++i)
      if (cb + i < p.dim) S_g[(int64_t)(cb + i) * vd + v] = S[i];
  }
  for (int c = 0; c < ncopies; ++c) {
    if (has_n) n_g[c * (p.dim + 1) + tid] = nreg;
    if (MODE == MEM_EXPGATE && tid == 0) n_g[c * (p.dim + 1) + p.dim] = m_run;
  }
}

// States too large for a workgroup's registers: the state stays in its slot (fp32, through the caches) and is read and
// written once per token; thread v owns column v, so no two threads touch the same entry.  Slow and general.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void matrix_memory_generic_kernel(MemArgs p) {
  extern __shared__ float4 lds4[];
  float* sk = reinterpret_cast<float*>(lds4);   // [dim]
  float* sq = sk + p.dim;                       // [dim]
  float* sg = sq + p.dim;                       // keep, take, exp(-m), then 32 floats for sums
  float* red = sg + 4;
  const int vd = p.vdim, tid = threadIdx.x, nthr = blockDim.x;
  const int h = blockIdx.x, b = blockIdx.y;
  const int t0 = p.cu_q[b], t1 = p.cu_q[b + 1];
  if (t1 <= t0) return;
  float* S_g = p.state + ((int64_t)p.slots[b] * p.H + h) * p.per_head;
  float* n_g = S_g + (int64_t)p.dim * vd;           // copies of n | m, one per 64 value columns, all kept equal
  const int copies = (vd + MEM_SLICE - 1) / MEM_SLICE;
  if (p.past[b] == 0)
    for (int i = tid; i < p.per_head; i += nthr) S_g[i] = 0.0f;
  float m_run = (MODE == MEM_EXPGATE && tid == 0 && p.past[b] != 0) ? n_g[p.dim] : 0.0f;
  const float decay = MODE == MEM_CONST ? p.decay[h] : 0.0f;
  const T* bias = reinterpret_cast<const T*>(p.bias);
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const float* row = p.proj + (int64_t)t * p.proj_rs;
    for (int i = tid; i < p.dim; i += nthr) {
      sk[i] = maybe_silu(row[p.k_off + h * p.dim + i], p.silu);
      sq[i] = maybe_silu(row[p.q_off + h * p.dim + i], p.silu) * p.q_scale;
    }
    if (tid == 0) {
      if constexpr (MODE == MEM_EXPGATE) {
        float zi = row[p.i_off + h], zf = row[p.f_off + h];
        if (bias) {
          zi += ld_f32<T>(bias + p.i_off + h);
          zf += ld_f32<T>(bias + p.f_off + h);
        }
        const float ig = p.cap * tanhf(zi / p.cap);
        const float fg = log_sigmoid_f32(p.cap * tanhf(zf / p.cap));
        const float m_new = fmaxf(fg + m_run, ig);
        sg[0] = expf(fg + m_run - m_new);
        sg[1] = expf(ig - m_new);
        sg[2] = expf(-m_new);
        m_run = m_new;
      } else {
        sg[0] = decay;
        sg[1] = 1.0f;
        sg[2] = 0.0f;
      }
    }
    __syncthreads();
    const float keep = sg[0], take = sg[1];
    float den = 1.0f;
    if constexpr (MODE == MEM_EXPGATE) {
      float pn = 0.0f;
      for (int i = tid; i < p.dim; i += nthr) {
        const float n = keep * n_g[i] + take * sk[i];
        for (int c = 0; c < copies; ++c) n_g[c * (p.dim + 1) + i] = n;
        pn += n * sq[i];
      }
      den = fmaxf(fabsf(block_sum(pn, red)), sg[2]) + 1e-6f;
    }
    for (int v = tid; v < vd; v += nthr) {
      const float vv = maybe_silu(row[p.v_off + h * vd + v], p.silu) * take;
      float acc = 0.0f;
      for (int i = 0; i < p.dim; ++i) {
        const float sv = keep * S_g[(int64_t)i * vd + v] + sk[i] * vv;
        S_g[(int64_t)i * vd + v] = sv;
        acc += sv * sq[i];
      }
      p.out[(int64_t)t * p.out_rs + h * vd + v] = acc / den;
    }
    __syncthreads();   // sk / sq / sg are rewritten by the next token
  }
  if (MODE == MEM_EXPGATE && tid == 0)
    for (int c = 0; c < copies; ++c) n_g[c * (p.dim + 1) + p.dim] = m_run;
}

template <typename T, int DMAX, int CS>
void launch_mem_mode(const MemArgs& p, int mode, dim3 grid, int threads, size_t lds, hipStream_t s) {
  if (mode == MEM_CONST) matrix_memory_kernel<T, DMAX, CS, MEM_CONST><<<grid, dim3(threads), lds, s>>>(p);
  else matrix_memory_kernel<T, DMAX, CS, MEM_EXPGATE><<<grid, dim3(threads), lds, s>>>(p);
}

template <typename T, int DMAX>
void launch_mem_cs(const MemArgs& p, int mode, int cs, dim3 grid, int threads, size_t lds, hipStream_t s) {
  if constexpr (DMAX >= 64) {
    if (cs == 4) return launch_mem_mode<T, DMAX, 4>(p, mode, grid, threads, lds, s);
  }
  if constexpr (DMAX >= 32 && DMAX <= 128) {
    if (cs == 2) return launch_mem_mode<T, DMAX, 2>(p, mode, grid, threads, lds, s);
  }
  if constexpr (DMAX <= 64) launch_mem_mode<T, DMAX, 1>(p, mode, grid, threads, lds, s);
}

template <typename T>
void launch_mem(const MemArgs& p, int mode, int dmax, int cs, dim3 grid, int threads, size_t lds, hipStream_t s) {
  switch (dmax) {
    case 16: return launch_mem_cs<T, 16>(p, mode, cs, grid, threads, lds, s);
    case 32: return launch_mem_cs<T, 32>(p, mode, cs, grid, threads, lds, s);
    case 64: return launch_mem_cs<T, 64>(p, mode, cs, grid, threads, lds, s);
    case 128: return launch_mem_cs<T, 128>(p, mode, cs, grid, threads, lds, s);
    default: return launch_mem_cs<T, 256>(p, mode, cs, grid, threads, lds, s);
  }
}

}  // namespace

extern "C" int64_t nv_matrix_memory_state_size(int mode, int dim, int vdim) {
  return (int64_t)dim * vdim + (mode == MEM_EXPGATE ? (int64_t)((vdim + MEM_SLICE - 1) / MEM_SLICE) * (dim + 1) : 0);
}

extern "C" int nv_matrix_memory(const float* proj, int64_t proj_row_stride, int q_off, int k_off, int v_off, int i_off,
                                int f_off, const void* bias, const float* decay, float* state, const int32_t* cu_q,
                                const int32_t* past_lens, const int32_t* state_slots, float* out, int64_t out_row_stride,
                                int num_seqs, int heads, int dim, int vdim, int mode, int silu, float q_scale, float cap,
                                int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(proj && state && cu_q && past_lens && state_slots && out, "nv_matrix_memory: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_matrix_memory: bad dtype %d", dtype);
  NV_CHECK_ARG(mode == MEM_CONST || mode == MEM_EXPGATE, "nv_matrix_memory: bad mode %d", mode);
  NV_CHECK_ARG(mode != MEM_CONST || decay, "nv_matrix_memory: constant decays are missing");
  NV_CHECK_ARG(mode != MEM_EXPGATE || cap > 0.0f, "nv_matrix_memory: the gate cap must be positive");
  NV_CHECK_ARG(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && num_seqs >= 0 && num_seqs <= 65535,
               "nv_matrix_memory: bad shape heads=%d dim=%d vdim=%d seqs=%d", heads, dim, vdim, num_seqs);
  if (num_seqs == 0) return NV_OK;
  int dmax = 16;
  while (dmax < dim) dmax *= 2;
  // One workgroup per slice of 64 state columns, the key channels of a column split over as many threads as leave each
  // at least 16 of them ...
  int slices = (vdim + MEM_SLICE - 1) / MEM_SLICE, cs = dmax >= 64 ? 4 : dmax / 16, vdp = MEM_SLICE;
  // ... unless the launch fills the chip anyway (many requests): then one workgroup walks all columns, if that fits 256
  // threads with at most 64 state registers each (shared staging and fewer, fuller workgroups win there)
  if (slices > 1 && (int64_t)heads * num_seqs >= 512) {
    const int vround = slices * MEM_SLICE;
    int cu = 1;
    while (cu < 4 && vround * cu * 2 <= 256 && dmax / (cu * 2) >= 16) cu *= 2;
    if (vround * cu <= 256 && dmax / cu <= 64 && vround * cu >= dim) {
      cs = cu;
      vdp = vround;
      slices = 1;
    }
  }
  const int threads = vdp * cs;
  MemArgs p{proj, proj_row_stride, q_off, k_off, v_off, i_off, f_off, bias, decay, state, cu_q, past_lens, state_slots,
            out, out_row_stride, heads, dim, vdim, (int)nv_matrix_memory_state_size(mode, dim, vdim), silu, q_scale, cap};
  if (dmax > 256 || slices > 65535 || getenv("NV_MATRIX_MEMORY_GENERIC") != nullptr) {
    const size_t glds = ((size_t)2 * dim + 4 + 32) * sizeof(float);
    NV_CHECK_ARG(glds <= 64 * 1024, "nv_matrix_memory: keys of %d numbers exceed the LDS", dim);
    dim3 grid(heads, num_seqs);
    if (mode == MEM_CONST) {
      NV_DISPATCH_T(dtype, matrix_memory_generic_kernel<T, MEM_CONST><<<grid, dim3(256), glds, (hipStream_t)stream>>>(p));
    } else {
      NV_DISPATCH_T(dtype, matrix_memory_generic_kernel<T, MEM_EXPGATE><<<grid, dim3(256), glds, (hipStream_t)stream>>>(p));
    }
    NV_CHECK_LAUNCH();
    return NV_OK;
  }
  const size_t lds =
      (size_t)(MM_TC * 2 * dmax + 3 * MM_TC + MM_TC * (threads / 64) + (cs > 1 ? cs * MM_TC * vdp : 0)) * sizeof(float);
  NV_CHECK_ARG(lds <= 64 * 1024 && threads <= 256, "nv_matrix_memory: launch plan out of range");
  NV_DISPATCH_T(dtype, launch_mem<T>(p, mode, dmax, cs, dim3(heads, num_seqs, slices), threads, lds, (hipStream_t)stream));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
