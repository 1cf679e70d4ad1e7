// Sliding-window softmax attention with grouped key / value heads over a paged cache, with an optional per-head
// sigmoid output gate.
//
// Row r (position p of sequence row_seq[r]) sees positions max(0, p - window + 1) .. p; query head h reads key / value
// head h / (H / G).  Key and value head sizes are independent (dk, dv).  Scores, softmax statistics, weights and the
// weighted sum are fp32.
//
// window_attn_wave_kernel: one wave per (row, head), every shape, bf16 or fp32.  The window is walked in tiles of 64
// keys: each lane scores one key (the query sits in LDS as fp32, the key row is read in 16-byte pieces where the
// head size allows), the wave forms the tile's running max / sum, then the lanes switch to value columns and add
// the tile's weighted value rows (weights broadcast from LDS, value rows read coalesced).
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int MAX_VCOLS = 8;  // value columns per lane: dv <= 512

template <typename T>
SYM_DEV float dot_row(const T* __restrict__ k, const float* __restrict__ q, int dk);

template <>
SYM_DEV float dot_row<bf16>(const bf16* __restrict__ k, const float* __restrict__ q, int dk) {
  float acc = 0.f;
  int e = 0;
  if ((dk & 7) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0) {
    for (; e < dk; e += 8) {
      float f[8];
      load8(k + e, f);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc += f[i] * q[e + i];
    }
  }
  for (; e < dk; ++e) acc += (float)k[e] * q[e];
  return acc;
}

template <>
SYM_DEV float dot_row<float>(const float* __restrict__ k, const float* __restrict__ q, int dk) {
  float acc = 0.f;
  int e = 0;
  if ((dk & 3) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0) {
    for (; e < dk; e += 4) {
      const float4 f = *reinterpret_cast<const float4*>(k + e);
      acc += f.x * q[e] + f.y * q[e + 1] + f.z * q[e + 2] + f.w * q[e + 3];
    }
  }
  for (; e < dk; ++e) acc += k[e] * q[e];
  return acc;
}

// grid (H, T), 64 threads.  Dynamic LDS: (dk + 64) floats.
template <typename T>
__global__ __launch_bounds__(64) void window_attn_wave_kernel(WindowAttnArgs a) {
  extern __shared__ float lds[];
  float* qs = lds;            // [dk]
  float* ps = lds + a.dk;     // [64]
  const int h = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
  const int g = h / (a.H / a.G);
  const int p = a.positions[row];
  const int j0 = max(0, p - a.window + 1);
  const int* bt = a.block_tables + (long long)a.row_seq[row] * a.max_blocks;
  const T* q = reinterpret_cast<const T*>(a.q) + ((long long)row * a.H + h) * a.dk;
  for (int e = lane; e < a.dk; e += 64) qs[e] = (float)q[e] * a.scale;
  __syncthreads();
  const T* kc = reinterpret_cast<const T*>(a.k_cache);
  const T* vc = reinterpret_cast<const T*>(a.v_cache);
  float acc[MAX_VCOLS];
#pragma unroll
  for (int i = 0; i < MAX_VCOLS; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int t0 = j0; t0 <= p; t0 += 64) {
    const int j = t0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const long long slot = (long long)bt[j / a.BS] * a.BS + j % a.BS;
      s = dot_row<T>(kc + (slot * a.G + g) * a.dk, qs, a.dk);
    }
    const float mt = fmaxf(m, wave_max(s));
    const float w = j <= p ? expf(s - mt) : 0.f;
    const float corr = expf(m - mt);          // first tile: exp(-inf) = 0 on an all-zero accumulator
    l = l * corr + wave_sum(w);
    m = mt;
    __syncthreads();                          // the previous tile's weights have been read
    ps[lane] = w;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAX_VCOLS; ++i) acc[i] *= corr;
    const int nt = min(64, p - t0 + 1);
    for (int jj = 0; jj < nt; ++jj) {
      const int jk = t0 + jj;
      const long long slot = (long long)bt[jk / a.BS] * a.BS + jk % a.BS;
      const T* vr = vc + (slot * a.G + g) * a.dv;
      const float pw = ps[jj];
#pragma unroll
      for (int i = 0; i < MAX_VCOLS; ++i) {
        const int c = lane + 64 * i;
        if (c < a.dv) acc[i] += pw * (float)vr[c];
      }
    }
  }
  float gate = 1.f;
  if (a.gate) {
    const float gv = (float)reinterpret_cast<const T*>(a.gate)[(long long)row * a.ldg + h];
    gate = 1.f / (1.f + expf(-gv));
  }
  const float inv = gate / l;
  T* o = reinterpret_cast<T*>(a.out) + ((long long)row * a.H + h) * a.dv;
#pragma unroll
  for (int i = 0; i < MAX_VCOLS; ++i) {
    const int c = lane + 64 * i;
    if (c < a.dv) o[c] = (T)(acc[i] * inv);
  }
}

}  // namespace

int launch_window_attn(const WindowAttnArgs& a, int f32, int impl, hipStream_t s) {
  if (a.T <= 0) return 0;
  dim3 grid(a.H, a.T);
  const size_t lds = (size_t)(a.dk + 64) * sizeof(float);
  if (f32)
    window_attn_wave_kernel<float><<<grid, 64, lds, s>>>(a);
  else
    window_attn_wave_kernel<bf16><<<grid, 64, lds, s>>>(a);
  return 0;
}
