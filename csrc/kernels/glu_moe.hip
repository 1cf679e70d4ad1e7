// Feed-forward pieces for clamped gated units, dense or routed by sigmoid scores:
//
//   clamped_glu      y = g' * sigmoid(alpha * g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)
//   sigmoid_topk     router: scores = sigmoid(x . Wr[e]) in fp32, the k largest with their scores (not renormalised)
//   expert_offsets   per-expert segment bounds of the routed rows (one workgroup: LDS histogram + scan)
//   scatter_scaled   routed rows into their expert's segment, multiplied by the router weight (the weight scales
//                    the expert's INPUT; the clamps make the expert non-linear in it, so it cannot move to the output)
//   grouped_linear   y = xs @ W[e]^T over the expert segments, bounds read from device memory (no host sync);
//                    64 x 64 tiles through LDS with fp32 accumulation, any N / K -- the all-shapes, both-dtypes
//                    grouped GEMM (bf16 shapes that tile for the MFMA grouped kernels run on those instead)
//   gather_sum       per token: the sum of its experts' output rows (+ the shared expert's), fp32
#include "common.h"
#include "latent_launchers.h"

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, long long n,
                                                         int F, float limit, float alpha) {
  const long long i = (long long)blockIdx.x * NT + threadIdx.x;
  if (i >= n) return;
  const long long r = i / F;
  const int c = (int)(i - r * F);
  const float g = fminf((float)gu[r * 2 * F + c], limit);
  const float u = fminf(fmaxf((float)gu[r * 2 * F + F + c], -limit), limit);
  out[i] = (T)(g / (1.f + expf(-alpha * g)) * (u + 1.f));
}

// bf16, F % 8 == 0: eight columns per thread, 16-byte loads and stores (prompt-sized launches are bandwidth-bound)
__global__ __launch_bounds__(NT) void clamped_glu_vec_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out,
                                                             long long nvec, int F, float limit, float alpha) {
  const long long i = (long long)blockIdx.x * NT + threadIdx.x;
  if (i >= nvec) return;
  const int fv = F >> 3;
  const long long r = i / fv;
  const int c = (int)(i - r * fv) * 8;
  float g[8], u[8], y[8];
  load8(gu + r * 2 * F + c, g);
  load8(gu + r * 2 * F + F + c, u);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float gj = fminf(g[j], limit);
    const float uj = fminf(fmaxf(u[j], -limit), limit);
    y[j] = gj / (1.f + __expf(-alpha * gj)) * (uj + 1.f);
  }
  store8(out + r * F + c, y);
}

constexpr int MAX_EXPERTS = 1024;

template <typename T>
__global__ __launch_bounds__(NT) void sigmoid_topk_kernel(const T* __restrict__ x, const T* __restrict__ Wr, int d, int E,
                                                          int k, int* __restrict__ ids, float* __restrict__ w) {
  extern __shared__ float xs[];  // d floats
  __shared__ float score[MAX_EXPERTS];
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < d; c += NT) xs[c] = (float)x[(long long)row * d + c];
  __syncthreads();
  for (int e = wave; e < E; e += NT / 64) {
    const T* wr = Wr + (long long)e * d;
    float s = 0.f;
    if constexpr (sizeof(T) == 2) {
      if ((d & 7) == 0) {
        // 16-byte loads, four in flight per lane (a plain strided loop waits for every load in turn)
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        int c = lane * 8;
        for (; c + 3 * 512 < d; c += 4 * 512) {
          float f[4][8];
#pragma unroll
          for (int u = 0; u < 4; ++u) load8(reinterpret_cast<const bf16*>(wr) + c + u * 512, f[u]);
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[u] += xs[c + u * 512 + i] * f[u][i];
        }
        for (; c < d; c += 512) {
          float f[8];
          load8(reinterpret_cast<const bf16*>(wr) + c, f);
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[0] += xs[c + i] * f[i];
        }
        s = (acc[0] + acc[1]) + (acc[2] + acc[3]);
      } else {
        for (int c = lane; c < d; c += 64) s += xs[c] * (float)wr[c];
      }
    } else {
#pragma unroll 4
      for (int c = lane; c < d; c += 64) s += xs[c] * (float)wr[c];
    }
    s = wave_sum(s);
    if (lane == 0) score[e] = 1.f / (1.f + expf(-s));
  }
  __syncthreads();
  if (wave != 0) return;
  for (int j = 0; j < k; ++j) {
    float best = -1.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (score[e] > best) best = score[e], bi = e;  // strided scan keeps the lowest index among equals per lane
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) best = ob, bi = oi;
    }
    if (lane == 0) {
      ids[row * k + j] = bi;
      w[row * k + j] = best;
      score[bi] = -2.f;
    }
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
  }
}

__global__ __launch_bounds__(1024) void expert_offsets_kernel(const int* __restrict__ ids, int R, int E,
                                                              int* __restrict__ offsets, int* __restrict__ cursor) {
  __shared__ int cnt[MAX_EXPERTS];
  for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int a = threadIdx.x; a < R; a += 1024) atomicAdd(&cnt[ids[a]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      acc += cnt[e];
    }
    offsets[E] = acc;
  }
  for (int e = threadIdx.x; e < E; e += 1024) cursor[e] = 0;
}

template <typename T>
__global__ __launch_bounds__(NT) void scatter_scaled_kernel(const T* __restrict__ x, const int* __restrict__ ids,
                                                            const float* __restrict__ w, int k, int d,
                                                            const int* __restrict__ offsets, int* __restrict__ cursor,
                                                            T* __restrict__ xs, int* __restrict__ dst) {
  __shared__ int pos;
  const int a = blockIdx.x;
  if (threadIdx.x == 0) {
    const int e = ids[a];
    pos = offsets[e] + atomicAdd(&cursor[e], 1);
    dst[a] = pos;
  }
  __syncthreads();
  const float wa = w[a];
  const T* xr = x + (long long)(a / k) * d;
  T* o = xs + (long long)pos * d;
  for (int c = threadIdx.x; c < d; c += NT) o[c] = (T)(wa * (float)xr[c]);
}

constexpr int BM = 64, BN = 64, BK = 16;

// grid: (ceil(N / BN), ceil(R / BM) + E): the y slots enumerate the row tiles of every expert segment (a segment of
// n rows has ceil(n / BM) of them; at most ceil(R / BM) + E in all); a workgroup finds its (expert, tile) by walking
// the offsets, surplus slots exit before any barrier.
template <typename T>
__global__ __launch_bounds__(NT) void grouped_linear_kernel(const T* __restrict__ xs, const T* __restrict__ W,
                                                            const int* __restrict__ offsets, int E, int N, int K,
                                                            T* __restrict__ y) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Bs[BK][BN + 4];
  int slot = blockIdx.y, e = 0, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    const int a = offsets[e], b = offsets[e + 1];
    const int tiles = (b - a + BM - 1) / BM;
    if (slot < tiles) {
      r0 = a + slot * BM;
      r1 = b;
      break;
    }
    slot -= tiles;
  }
  if (e >= E) return;
  const int n0 = blockIdx.x * BN;
  const T* We = W + (long long)e * N * K;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int i = threadIdx.x; i < BM * BK; i += NT) {
      const int m = i / BK, kk = i - m * BK;
      const int r = r0 + m, c = k0 + kk;
      As[kk][m] = (r < r1 && c < K) ? (float)xs[(long long)r * K + c] : 0.f;
    }
    for (int i = threadIdx.x; i < BN * BK; i += NT) {
      const int n = i / BK, kk = i - n * BK;
      const int c = k0 + kk;
      Bs[kk][n] = (n0 + n < N && c < K) ? (float)We[(long long)(n0 + n) * K + c] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i], bv[i] = Bs[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty * 4 + i;
    if (r >= r1) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) y[(long long)r * N + n] = (T)acc[i][j];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void gather_sum_kernel(const T* __restrict__ y, const int* __restrict__ dst, int k,
                                                        const T* __restrict__ extra, float* __restrict__ out, int d) {
  __shared__ int rows[64];
  const int t = blockIdx.x;
  for (int j = threadIdx.x; j < k && j < 64; j += NT) rows[j] = dst[t * k + j];
  __syncthreads();
#pragma unroll 4
  for (int c = threadIdx.x; c < d; c += NT) {
    float s = extra ? (float)extra[(long long)t * d + c] : 0.f;
    for (int j = 0; j < k; ++j) s += (float)y[(long long)(j < 64 ? rows[j] : dst[t * k + j]) * d + c];
    out[(long long)t * d + c] = s;
  }
}

}  // namespace

void launch_clamped_glu(const void* gu, void* out, int R, int F, float limit, float alpha, int f32, hipStream_t s) {
  const long long n = (long long)R * F;
  if (n <= 0) return;
  if (!f32 && F % 8 == 0) {
    const long long nvec = n / 8;
    clamped_glu_vec_kernel<<<(unsigned)((nvec + NT - 1) / NT), NT, 0, s>>>((const bf16*)gu, (bf16*)out, nvec, F, limit,
                                                                         alpha);
    return;
  }
  const unsigned grid = (unsigned)((n + NT - 1) / NT);
  if (f32) clamped_glu_kernel<float><<<grid, NT, 0, s>>>((const float*)gu, (float*)out, n, F, limit, alpha);
  else clamped_glu_kernel<bf16><<<grid, NT, 0, s>>>((const bf16*)gu, (bf16*)out, n, F, limit, alpha);
}

void launch_sigmoid_topk(const void* x, const void* Wr, int T, int d, int E, int k, int* ids, float* w, int f32,
                         hipStream_t s) {
  if (T <= 0) return;
  const size_t lds = (size_t)d * sizeof(float);
  if (f32) sigmoid_topk_kernel<float><<<T, NT, lds, s>>>((const float*)x, (const float*)Wr, d, E, k, ids, w);
  else sigmoid_topk_kernel<bf16><<<T, NT, lds, s>>>((const bf16*)x, (const bf16*)Wr, d, E, k, ids, w);
}

void launch_expert_offsets(const int* ids, int R, int E, int* offsets, int* cursor, hipStream_t s) {
  expert_offsets_kernel<<<1, 1024, 0, s>>>(ids, R, E, offsets, cursor);
}

void launch_scatter_scaled(const void* x, const int* ids, const float* w, int k, int R, int d, const int* offsets,
                           int* cursor, void* xs, int* dst, int f32, hipStream_t s) {
  if (R <= 0) return;
  if (f32)
    scatter_scaled_kernel<float><<<R, NT, 0, s>>>((const float*)x, ids, w, k, d, offsets, cursor, (float*)xs, dst);
  else
    scatter_scaled_kernel<bf16><<<R, NT, 0, s>>>((const bf16*)x, ids, w, k, d, offsets, cursor, (bf16*)xs, dst);
}

void launch_grouped_linear(const void* xs, const void* W, const int* offsets, int E, int R, int N, int K, void* y,
                           int f32, hipStream_t s) {
  if (R <= 0) return;
  dim3 grid((N + BN - 1) / BN, (R + BM - 1) / BM + E);
  if (f32) grouped_linear_kernel<float><<<grid, NT, 0, s>>>((const float*)xs, (const float*)W, offsets, E, N, K, (float*)y);
  else grouped_linear_kernel<bf16><<<grid, NT, 0, s>>>((const bf16*)xs, (const bf16*)W, offsets, E, N, K, (bf16*)y);
}

void launch_gather_sum(const void* y, const int* dst, int k, const void* extra, float* out, int T, int d, int f32,
                       hipStream_t s) {
  if (T <= 0) return;
  if (f32) gather_sum_kernel<float><<<T, NT, 0, s>>>((const float*)y, dst, k, (const float*)extra, out, d);
  else gather_sum_kernel<bf16><<<T, NT, 0, s>>>((const bf16*)y, dst, k, (const bf16*)extra, out, d);
}
