// Row kernels of the residual stream for models with per-sequence carried state and a depth-mixed stream:
//
//   embed_rows       x = table[token] (also the first entry of the layer history)
//   token_shift      h = x + (x_prev - x) * mu: x_prev is the row above inside a step's run of tokens, the
//                    sequence's carried row (state slot) at the start of a run, zeros at position 0
//   add_layer_norm   x += layer_norm(delta) * w  (mean / variance / sum in fp32), optionally saving the rows that
//                    become a sequence's carried state, appending the result to the layer history and replacing
//                    x by the history's weighted sum, and writing the activation-dtype copy the next GEMM reads
//   layer_norm       plain layer norm of gathered rows (the model's last norm)
//
// One 256-thread workgroup per row; columns strided over the threads (coalesced), any width.  The statistics
// are two block reductions over the delta row (mean, then the squared deviations), so the variance is the
// mean of squared deviations exactly as defined, not E[x^2] - E[x]^2.
#include "common.h"
#include "latent_launchers.h"

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void embed_rows_kernel(const int* __restrict__ ids, const int* __restrict__ src,
                                                        const int* __restrict__ prev, const T* __restrict__ table,
                                                        float* __restrict__ x, float* __restrict__ hist0, int d) {
  const int row = blockIdx.x;
  const int sr = src ? src[row] : -1;
  const long long tok = sr >= 0 ? prev[sr] : ids[row];
  const T* t = table + tok * d;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = (float)t[c];
    x[(long long)row * d + c] = v;
    hist0[(long long)row * d + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void token_shift_kernel(const float* __restrict__ x, const T* __restrict__ mu,
                                                         const int* __restrict__ prev_row,
                                                         const float* __restrict__ state, long long state_stride,
                                                         T* __restrict__ h, int d) {
  const int row = blockIdx.x;
  const int pr = prev_row[row];
  const float* p = pr >= 0 ? x + (long long)pr * d : (pr == -1 ? nullptr : state + (long long)(-(pr + 2)) * state_stride);
  for (int c = threadIdx.x; c < d; c += NT) {
    const float xv = x[(long long)row * d + c];
    const float pv = p ? p[c] : 0.f;
    h[(long long)row * d + c] = (T)(xv + (pv - xv) * (float)mu[c]);
  }
}

// EPT > 0: the row's delta, x and weight are read once into registers (d <= NT * EPT), all loads in flight together;
// EPT == 0: any width, the delta row is re-read for each pass (it stays in L1 / L2).
template <typename T, typename TD, int EPT>
__global__ __launch_bounds__(NT) void add_layer_norm_kernel(const TD* __restrict__ delta, const T* __restrict__ w,
                                                            float eps, float* __restrict__ x,
                                                            const int* __restrict__ save, float* __restrict__ state,
                                                            long long state_stride, float* __restrict__ hist,
                                                            long long hist_stride, const float* __restrict__ coef,
                                                            int hist_idx, T* __restrict__ out_act, int d) {
  __shared__ float scratch[NT / 64];
  const int row = blockIdx.x;
  const TD* dr = delta + (long long)row * d;
  float* xr = x + (long long)row * d;
  constexpr int NR = EPT > 0 ? EPT : 1;
  float dv[NR], xv[NR], wv[NR];
  float sum = 0.f;
  if constexpr (EPT > 0) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int c = threadIdx.x + i * NT;
      const bool in = c < d;
      dv[i] = in ? (float)dr[c] : 0.f;
      xv[i] = in ? xr[c] : 0.f;
      wv[i] = in ? (float)w[c] : 0.f;
      sum += dv[i];
    }
  } else {
    for (int c = threadIdx.x; c < d; c += NT) sum += (float)dr[c];
  }
  const float mean = block_sum<NT>(sum, scratch) / (float)d;
  float sq = 0.f;
  if constexpr (EPT > 0) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const float v = threadIdx.x + i * NT < d ? dv[i] - mean : 0.f;
      sq += v * v;
    }
  } else {
    for (int c = threadIdx.x; c < d; c += NT) {
      const float v = (float)dr[c] - mean;
      sq += v * v;
    }
  }
  const float rstd = 1.f / sqrtf(block_sum<NT>(sq, scratch) / (float)d + eps);
  const int sv = save ? save[row] : -1;
  auto finish = [&](int c, float dl, float xo, float wc) {
    const long long o = (long long)row * d + c;
    if (sv >= 0) state[(long long)sv * state_stride + c] = xo;
    float xn = xo + (dl - mean) * rstd * wc;
    if (hist) {
      hist[(long long)hist_idx * hist_stride + o] = xn;
      float m = coef[hist_idx] * xn;
      for (int j = 0; j < hist_idx; ++j) m += coef[j] * hist[(long long)j * hist_stride + o];
      xn = m;
    }
    x[o] = xn;
    if (out_act) out_act[o] = (T)xn;
  };
  if constexpr (EPT > 0) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < d) finish(c, dv[i], xv[i], wv[i]);
    }
  } else {
    for (int c = threadIdx.x; c < d; c += NT) finish(c, (float)dr[c], xr[c], (float)w[c]);
  }
}

// Four consecutive columns per thread and pass (d % 4 == 0, d <= NT * 4 * G): 8- / 16-byte accesses for the
// bandwidth-bound prompt-sized launches; the same arithmetic in the same order per element as the scalar kernel.
template <typename V>
SYM_DEV void ld4(const V* p, float* f);
template <>
SYM_DEV void ld4<float>(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
template <>
SYM_DEV void ld4<bf16>(const bf16* p, float* f) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = (float)v[i];
}
SYM_DEV void st4(float* p, const float* f) { *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]); }
SYM_DEV void st4(bf16* p, const float* f) {
  bf16x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = (bf16)f[i];
  *reinterpret_cast<bf16x4*>(p) = v;
}

template <typename T, typename TD, int G>
__global__ __launch_bounds__(NT) void add_layer_norm_vec_kernel(const TD* __restrict__ delta, const T* __restrict__ w,
                                                                float eps, float* __restrict__ x,
                                                                const int* __restrict__ save, float* __restrict__ state,
                                                                long long state_stride, float* __restrict__ hist,
                                                                long long hist_stride, const float* __restrict__ coef,
                                                                int hist_idx, T* __restrict__ out_act, int d) {
  __shared__ float scratch[NT / 64];
  const int row = blockIdx.x;
  const long long rb = (long long)row * d;
  float dv[G][4], xv[G][4], wv[G][4];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < G; ++i) {
    const int c = (threadIdx.x + i * NT) * 4;
    if (c < d) {
      ld4<TD>(delta + rb + c, dv[i]);
      ld4<float>(x + rb + c, xv[i]);
      ld4<T>(w + c, wv[i]);
#pragma unroll
      for (int j = 0; j < 4; ++j) sum += dv[i][j];
    }
  }
  const float mean = block_sum<NT>(sum, scratch) / (float)d;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < G; ++i)
    if ((threadIdx.x + i * NT) * 4 < d) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = dv[i][j] - mean;
        sq += v * v;
      }
    }
  const float rstd = 1.f / sqrtf(block_sum<NT>(sq, scratch) / (float)d + eps);
  const int sv = save ? save[row] : -1;
#pragma unroll
  for (int i = 0; i < G; ++i) {
    const int c = (threadIdx.x + i * NT) * 4;
    if (c >= d) continue;
    if (sv >= 0) st4(state + (long long)sv * state_stride + c, xv[i]);
    float xn[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xn[j] = xv[i][j] + (dv[i][j] - mean) * rstd * wv[i][j];
    if (hist) {
      st4(hist + (long long)hist_idx * hist_stride + rb + c, xn);
      const float ci = coef[hist_idx];
#pragma unroll
      for (int j = 0; j < 4; ++j) xn[j] *= ci;
      for (int k = 0; k < hist_idx; ++k) {
        float hv[4];
        ld4<float>(hist + (long long)k * hist_stride + rb + c, hv);
        const float ck = coef[k];
#pragma unroll
        for (int j = 0; j < 4; ++j) xn[j] += ck * hv[j];
      }
    }
    st4(x + rb + c, xn);
    if (out_act) st4(out_act + rb + c, xn);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void layer_norm_kernel(const float* __restrict__ x, const long long* __restrict__ rows,
                                                        const T* __restrict__ w, float eps, T* __restrict__ out, int d) {
  __shared__ float scratch[NT / 64];
  const int i = blockIdx.x;
  const float* xr = x + (rows ? rows[i] : (long long)i) * d;
  float sum = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) sum += xr[c];
  const float mean = block_sum<NT>(sum, scratch) / (float)d;
  float sq = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = xr[c] - mean;
    sq += v * v;
  }
  const float rstd = 1.f / sqrtf(block_sum<NT>(sq, scratch) / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) out[(long long)i * d + c] = (T)((xr[c] - mean) * rstd * (float)w[c]);
}

}  // namespace

void launch_embed_rows(const int* ids, const int* src, const int* prev, const void* table, float* x, float* hist0,
                       int T, int d, int f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    embed_rows_kernel<float><<<T, NT, 0, s>>>(ids, src, prev, (const float*)table, x, hist0, d);
  else
    embed_rows_kernel<bf16><<<T, NT, 0, s>>>(ids, src, prev, (const bf16*)table, x, hist0, d);
}

void launch_token_shift(const float* x, const void* mu, const int* prev_row, const float* state, long long state_stride,
                        void* h, int T, int d, int f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    token_shift_kernel<float><<<T, NT, 0, s>>>(x, (const float*)mu, prev_row, state, state_stride, (float*)h, d);
  else
    token_shift_kernel<bf16><<<T, NT, 0, s>>>(x, (const bf16*)mu, prev_row, state, state_stride, (bf16*)h, d);
}

template <typename T, typename TD>
void add_layer_norm_pick(const void* delta, const void* w, float eps, float* x, const int* save, float* state,
                         long long state_stride, float* hist, long long hist_stride, const float* coef, int hist_idx,
                         void* out_act, int T_, int d, hipStream_t s) {
#define SYM_ALN(EPT)                                                                                                   \
  add_layer_norm_kernel<T, TD, EPT><<<T_, NT, 0, s>>>((const TD*)delta, (const T*)w, eps, x, save, state, state_stride, \
                                                      hist, hist_stride, coef, hist_idx, (T*)out_act, d)
#define SYM_ALNV(G)                                                                                                   \
  add_layer_norm_vec_kernel<T, TD, G><<<T_, NT, 0, s>>>((const TD*)delta, (const T*)w, eps, x, save, state,            \
                                                        state_stride, hist, hist_stride, coef, hist_idx, (T*)out_act, d)
  if (d % 4 == 0 && state_stride % 4 == 0 && d <= NT * 32) {
    if (d <= NT * 8) SYM_ALNV(2);
    else if (d <= NT * 16) SYM_ALNV(4);
    else SYM_ALNV(8);
    return;
  }
  if (d <= NT * 4) SYM_ALN(4);
  else if (d <= NT * 8) SYM_ALN(8);
  else if (d <= NT * 16) SYM_ALN(16);
  else if (d <= NT * 32) SYM_ALN(32);
  else SYM_ALN(0);
#undef SYM_ALN
#undef SYM_ALNV
}

void launch_add_layer_norm(const void* delta, int delta_f32, const void* w, float eps, float* x, const int* save,
                           float* state, long long state_stride, float* hist, long long hist_stride, const float* coef,
                           int hist_idx, void* out_act, int T, int d, int f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    add_layer_norm_pick<float, float>(delta, w, eps, x, save, state, state_stride, hist, hist_stride, coef, hist_idx,
                                      out_act, T, d, s);
  else if (delta_f32)
    add_layer_norm_pick<bf16, float>(delta, w, eps, x, save, state, state_stride, hist, hist_stride, coef, hist_idx,
                                     out_act, T, d, s);
  else
    add_layer_norm_pick<bf16, bf16>(delta, w, eps, x, save, state, state_stride, hist, hist_stride, coef, hist_idx,
                                    out_act, T, d, s);
}

void launch_layer_norm(const float* x, const long long* rows, const void* w, float eps, void* out, int n, int d,
                       int f32, hipStream_t s) {
  if (n <= 0) return;
  if (f32)
    layer_norm_kernel<float><<<n, NT, 0, s>>>(x, rows, (const float*)w, eps, (float*)out, d);
  else
    layer_norm_kernel<bf16><<<n, NT, 0, s>>>(x, rows, (const bf16*)w, eps, (bf16*)out, d);
}
