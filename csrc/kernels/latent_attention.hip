// Attention over a cached low-rank latent (one shared "key/value head" for all query heads).
//
// The cache holds, per token, the normalised latent c [kv_rank] followed by one rotated key part k_r [rot]
// shared by every head.  With the per-head up-projections folded into the query and the output,
//
//     score(t, j, h) = (W_uk[h]^T q_nope[t, h]) . c[j] + q_rot[t, h] . k_r[j]          (times the scale)
//     out(t, h)      = W_uv[h] . sum_j softmax_j(score)(t, j, h) c[j]
//
// so the attention kernel is multi-query attention whose key row is the whole cache row [kv_rank + rot] and whose
// value row is its first kv_rank entries: every cache row is read once for all heads, and nothing but the cache
// row is ever materialised per token.
//
//   latent_prep   per token: RMS-norm the query latent; RMS-norm the kv latent and rotate the shared key part into
//                 the token's cache row (statistics and angles in fp32)
//   rope_pairs    interleaved-pair rotary (dimension 2i with 2i + 1) of a strided [T][H][rot] slice
//   latent_attn   causal softmax attention over the paged latent cache; scores, weights and accumulators fp32
#include "common.h"
#include "latent_launchers.h"

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void latent_prep_kernel(LatentPrepArgs a) {
  __shared__ float scratch[NT / 64];
  const int row = blockIdx.x;
  const T* z = (const T*)a.z + (long long)row * a.nz;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.q_rank; c += NT) {
    const float v = (float)z[c];
    ss += v * v;
  }
  const float rq = 1.f / sqrtf(block_sum<NT>(ss, scratch) / (float)a.q_rank + a.eps);
  T* cq = (T*)a.cq + (long long)row * a.q_rank;
  const T* wq = (const T*)a.wq;
  for (int c = threadIdx.x; c < a.q_rank; c += NT) cq[c] = (T)((float)z[c] * rq * (float)wq[c]);
  if (a.kv_rank == 0) return;
  const int slot = a.slots[row];
  const T* zk = z + a.q_rank;
  ss = 0.f;
  for (int c = threadIdx.x; c < a.kv_rank; c += NT) {
    const float v = (float)zk[c];
    ss += v * v;
  }
  const float rk = 1.f / sqrtf(block_sum<NT>(ss, scratch) / (float)a.kv_rank + a.eps);
  if (slot < 0) return;
  T* out = (T*)a.cache + (long long)slot * (a.kv_rank + a.rot);
  const T* wkv = (const T*)a.wkv;
  for (int c = threadIdx.x; c < a.kv_rank; c += NT) out[c] = (T)((float)zk[c] * rk * (float)wkv[c]);
  const float* cs = a.rope + (long long)a.positions[row] * a.rot;
  for (int i = threadIdx.x; i < a.rot / 2; i += NT) {
    const float u = (float)zk[a.kv_rank + 2 * i], v = (float)zk[a.kv_rank + 2 * i + 1];
    const float co = cs[2 * i], si = cs[2 * i + 1];
    out[a.kv_rank + 2 * i] = (T)(u * co - v * si);
    out[a.kv_rank + 2 * i + 1] = (T)(v * co + u * si);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void rope_pairs_kernel(const T* __restrict__ src, long long s_t, long long s_h,
                                                        T* __restrict__ dst, long long d_t, long long d_h,
                                                        const int* __restrict__ positions,
                                                        const float* __restrict__ rope, int H, int rot) {
  const int row = blockIdx.x;
  const float* cs = rope + (long long)positions[row] * rot;
  const int half = rot / 2;
  for (int i = threadIdx.x; i < H * half; i += NT) {
    const int h = i / half, p = i - h * half;
    const T* s = src + row * s_t + h * s_h + 2 * p;
    T* o = dst + row * d_t + h * d_h + 2 * p;
    const float u = (float)s[0], v = (float)s[1];
    const float co = cs[2 * p], si = cs[2 * p + 1];
    o[0] = (T)(u * co - v * si);
    o[1] = (T)(v * co + u * si);
  }
}

// fp32 dot of a query held in LDS with one cache row (16-byte loads when the row length allows)
SYM_DEV float dot_row(const float* q, const bf16* r, int n) {
  float s = 0.f;
  if ((n & 7) == 0) {
    for (int c = 0; c < n; c += 8) {
      float f[8];
      load8(r + c, f);
#pragma unroll
      for (int i = 0; i < 8; ++i) s += q[c + i] * f[i];
    }
  } else {
    for (int c = 0; c < n; ++c) s += q[c] * (float)r[c];
  }
  return s;
}

SYM_DEV float dot_row(const float* q, const float* r, int n) {
  float s = 0.f;
  if ((n & 3) == 0) {
    for (int c = 0; c < n; c += 4) {
      const float4 f = *reinterpret_cast<const float4*>(r + c);
      s += q[c] * f.x + q[c + 1] * f.y + q[c + 2] * f.z + q[c + 3] * f.w;
    }
  } else {
    for (int c = 0; c < n; ++c) s += q[c] * r[c];
  }
  return s;
}

constexpr int PART = 256;  // keys per split-KV partition of the decode form

// One wave per (query row, head, key partition).  Each lane scores one key of a 64-key tile (the query in LDS, the
// cache row streamed), the tile's softmax statistics are wave reductions, and the weighted sum of the latents
// keeps kv_rank / 64 accumulators per lane (coalesced row reads, the weight broadcast by a lane read).
// parts == 1: the normalised output goes to `out`; otherwise unnormalised partials + (max, sum) go to part_o /
// part_ml and latent_attn_merge_kernel combines them.
template <typename T, int MAXR>
__global__ __launch_bounds__(64) void latent_attn_wave_kernel(LatentAttnArgs a) {
  extern __shared__ float qs[];
  const int row = blockIdx.x, h = blockIdx.y, part = blockIdx.z;
  const int lane = threadIdx.x;
  const int nkeys = a.positions[row] + 1;
  const int k0 = a.parts > 1 ? part * PART : 0;
  const int k1 = a.parts > 1 ? min(nkeys, k0 + PART) : nkeys;
  const T* q = (const T*)a.q + ((long long)row * a.H + h) * a.Dk;
  for (int c = lane; c < a.Dk; c += 64) qs[c] = (float)q[c];
  __syncthreads();
  const int* bt = a.block_tables + (long long)a.row_seq[row] * a.max_blocks;
  const T* cache = (const T*)a.cache;
  float m = -INFINITY, l = 0.f;
  float o[MAXR];
#pragma unroll
  for (int i = 0; i < MAXR; ++i) o[i] = 0.f;
  for (int base = k0; base < k1; base += 64) {
    const int key = base + lane;
    const bool valid = key < k1;
    int crow = 0;
    float s = -INFINITY;
    if (valid) {
      crow = bt[key / a.BS] * a.BS + key % a.BS;
      s = dot_row(qs, cache + (long long)crow * a.Dk, a.Dk) * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < MAXR; ++i) o[i] *= alpha;
    const int n = min(64, k1 - base);
    for (int j = 0; j < n; ++j) {
      const float pj = __shfl(p, j, 64);
      const T* r = cache + (long long)__shfl(crow, j, 64) * a.Dk;
#pragma unroll
      for (int i = 0; i < MAXR; ++i) {
        const int c = lane + 64 * i;
        if (c < a.kv_rank) o[i] += pj * (float)r[c];
      }
    }
    m = m_new;
  }
  if (a.parts == 1) {
    T* out = (T*)a.out + ((long long)row * a.H + h) * a.kv_rank;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int c = lane + 64 * i;
      if (c < a.kv_rank) out[c] = (T)(o[i] * inv);
    }
  } else {
    const long long pi = ((long long)row * a.H + h) * a.parts + part;
    float* po = a.part_o + pi * a.kv_rank;
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int c = lane + 64 * i;
      if (c < a.kv_rank) po[c] = o[i];
    }
    if (lane == 0) {
      a.part_ml[2 * pi] = m;  // -inf, 0 for a partition past the row's keys
      a.part_ml[2 * pi + 1] = l;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(64) void latent_attn_merge_kernel(LatentAttnArgs a) {
  const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const long long p0 = ((long long)row * a.H + h) * a.parts;
  const int np = min(a.parts, (a.positions[row] + PART) / PART);  // partitions that hold keys of this row
  float m = -INFINITY;
  for (int p = 0; p < np; ++p) m = fmaxf(m, a.part_ml[2 * (p0 + p)]);
  float l = 0.f;
  for (int p = 0; p < np; ++p) l += a.part_ml[2 * (p0 + p) + 1] * expf(a.part_ml[2 * (p0 + p)] - m);
  T* out = (T*)a.out + ((long long)row * a.H + h) * a.kv_rank;
  for (int c = lane; c < a.kv_rank; c += 64) {
    float acc = 0.f;
    for (int p = 0; p < np; ++p) acc += a.part_o[(p0 + p) * a.kv_rank + c] * expf(a.part_ml[2 * (p0 + p)] - m);
    out[c] = (T)(acc / l);
  }
}

template <typename T>
void attn_dispatch(const LatentAttnArgs& a, hipStream_t s) {
  dim3 grid(a.T, a.H, a.parts);
  const size_t lds = (size_t)a.Dk * sizeof(float);
  const int nr = (a.kv_rank + 63) / 64;
  if (nr <= 1) latent_attn_wave_kernel<T, 1><<<grid, 64, lds, s>>>(a);
  else if (nr <= 2) latent_attn_wave_kernel<T, 2><<<grid, 64, lds, s>>>(a);
  else if (nr <= 4) latent_attn_wave_kernel<T, 4><<<grid, 64, lds, s>>>(a);
  else latent_attn_wave_kernel<T, 8><<<grid, 64, lds, s>>>(a);
  if (a.parts > 1) latent_attn_merge_kernel<T><<<dim3(a.T, a.H), 64, 0, s>>>(a);
}

}  // namespace

int latent_attn_part_tokens() { return PART; }

void launch_latent_prep(const LatentPrepArgs& a, int T, int f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32) latent_prep_kernel<float><<<T, NT, 0, s>>>(a);
  else latent_prep_kernel<bf16><<<T, NT, 0, s>>>(a);
}

void launch_rope_pairs(const void* src, long long s_t, long long s_h, void* dst, long long d_t, long long d_h,
                       const int* positions, const float* rope, int T, int H, int rot, int f32, hipStream_t s) {
  if (T <= 0 || rot <= 0) return;
  if (f32)
    rope_pairs_kernel<float><<<T, NT, 0, s>>>((const float*)src, s_t, s_h, (float*)dst, d_t, d_h, positions, rope, H, rot);
  else
    rope_pairs_kernel<bf16><<<T, NT, 0, s>>>((const bf16*)src, s_t, s_h, (bf16*)dst, d_t, d_h, positions, rope, H, rot);
}

void launch_latent_attn(const LatentAttnArgs& a, int f32, hipStream_t s) {
  if (a.T <= 0) return;
  if (f32) attn_dispatch<float>(a, s);
  else attn_dispatch<bf16>(a, s);
}
