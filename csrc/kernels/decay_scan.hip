// Linear recurrence with decaying matrix state, the common core of gated linear attention and state-space layers:
//
//     S_t = diag(a_t) S_(t-1) + b_t k_t v_t^T          S [N x P] fp32 per (sequence, head)
//     o_t = S_t^T (q_scale q_t) (+ skip_h v_t)
//
// mode 0 (channel gate): a_t[n] = sigmoid(dz_t[n] + dbias[n])^(1 / tau) = exp(logsigmoid(.) / tau), b_t = 1
// mode 1 (step size):    b_t = softplus(dz_t + dbias[h]), a_t = exp(-exp(rate[h]) b_t) for every n
//
// The state walks token by token in fp32, in the same order however a prompt is cut into steps, so a position's
// output does not depend on the cut.  A run of rows (one sequence's tokens of this step) starts from its state slot
// (or zero at position 0) and ends in it.
//
// Work split: grid (P / 64 column tiles, heads, runs), 256 threads.  Wave w owns 16 value columns; inside a wave the
// lanes are 16 columns x 4 slices of the key channels, so a lane keeps N / 4 state entries of one column in
// registers and a token's output is a 4-lane sum (two cross-lane adds).  The per-token vectors that all columns
// share (q, k, the decays) are staged through LDS for CH tokens at a time by the whole workgroup, with the
// transcendental part of the decay evaluated once per (token, channel) there.
#include "common.h"
#include "hybrid_launchers.h"

namespace {

constexpr int NT = 256;
constexpr int CH = 8;       // tokens staged per round
constexpr int PCOLS = 16;   // value columns per wave
constexpr int SLICES = 4;   // key-channel slices per column (lanes)

SYM_DEV float softplus_exact(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

template <typename T, int MODE, int NPL>  // NPL: state entries per lane (>= ceil(N / 4))
__global__ __launch_bounds__(NT) void decay_scan_kernel(DecayScanArgs a) {
  extern __shared__ float lds[];
  const int N = a.N, P = a.P;
  const int npad = NPL * SLICES;
  float* qS = lds;                    // [CH][npad]
  float* kS = qS + CH * npad;         // [CH][npad]
  float* aS = kS + CH * npad;         // [CH][npad] (mode 0) or [CH] (mode 1)
  float* bS = aS + (MODE == 0 ? CH * npad : CH);  // [CH] (mode 1)
  const int h = blockIdx.y, run = blockIdx.z;
  const int s0 = a.cu_q ? a.cu_q[run] : run, s1 = a.cu_q ? a.cu_q[run + 1] : run + 1;
  if (s1 <= s0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pc = lane & (PCOLS - 1), ns = lane >> 4;
  const int p = blockIdx.x * (PCOLS * (NT / 64)) + wave * PCOLS + pc;
  const bool pin = p < P;
  const int n0 = ns * NPL;
  const int grp = h / a.hpg;
  const int pr = a.prev_row[s0];
  const int sv = a.save_slot[s1 - 1];
  float S[NPL];
  if (pr <= -2 && pin) {
    const float* st = a.state + (long long)(-(pr + 2)) * a.state_stride + (long long)h * N * P + p;
#pragma unroll
    for (int i = 0; i < NPL; ++i) S[i] = n0 + i < N ? st[(long long)(n0 + i) * P] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < NPL; ++i) S[i] = 0.f;
  }
  const T* q = reinterpret_cast<const T*>(a.q) + (long long)grp * N;
  const T* k = reinterpret_cast<const T*>(a.k) + (long long)grp * N;
  const T* v = reinterpret_cast<const T*>(a.v) + (long long)h * P + p;
  const T* dz = reinterpret_cast<const T*>(a.dz);
  const float skip = a.skip ? a.skip[h] : 0.f;
  const float inv_tau = MODE == 0 ? 1.f / a.tau : 0.f;
  const float rate = MODE == 1 ? expf(a.rate[h]) : 0.f;
  for (int t0 = s0; t0 < s1; t0 += CH) {
    const int nt = min(CH, s1 - t0);
    __syncthreads();   // the previous round's vectors have been used
    for (int i = threadIdx.x; i < nt * npad; i += NT) {
      const int tt = i / npad, n = i - tt * npad;
      const long long r = t0 + tt;
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (n < N) {
        qv = (float)q[r * a.ldq + n] * a.q_scale;
        kv = (float)k[r * a.ldk + n];
        if (MODE == 0) {
          const float z = (float)dz[r * a.ldd + (long long)h * N + n] + a.dbias[(long long)h * N + n];
          av = expf(-softplus_exact(-z) * inv_tau);   // logsigmoid(z) = -softplus(-z)
        }
      }
      qS[i] = qv;
      kS[i] = kv;
      if (MODE == 0) aS[i] = av;
    }
    if (MODE == 1 && threadIdx.x < nt) {
      const long long r = t0 + threadIdx.x;
      const float b = softplus_exact((float)dz[r * a.ldd + h] + a.dbias[h]);
      bS[threadIdx.x] = b;
      aS[threadIdx.x] = expf(-rate * b);
    }
    float vr[CH];
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) vr[tt] = (tt < nt && pin) ? (float)v[(long long)(t0 + tt) * a.ldv] : 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      if (tt < nt) {
        const float* qr = qS + tt * npad + n0;
        const float* kr = kS + tt * npad + n0;
        float u = vr[tt], o = 0.f;
        if (MODE == 1) {
          u *= bS[tt];
          const float at = aS[tt];
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            S[i] = at * S[i] + kr[i] * u;
            o += S[i] * qr[i];
          }
        } else {
          const float* ar = aS + tt * npad + n0;
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            S[i] = ar[i] * S[i] + kr[i] * u;
            o += S[i] * qr[i];
          }
        }
        o += __shfl_xor(o, 16, 64);
        o += __shfl_xor(o, 32, 64);
        if (ns == 0 && pin) a.out[((long long)(t0 + tt) * a.H + h) * P + p] = o + skip * vr[tt];
      }
    }
  }
  if (sv >= 0 && pin) {
    float* st = a.state + (long long)sv * a.state_stride + (long long)h * N * P + p;
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (n0 + i < N) st[(long long)(n0 + i) * P] = S[i];
  }
}

template <typename T, int MODE>
void launch_mode(const DecayScanArgs& a, hipStream_t s) {
  const int cols = PCOLS * (NT / 64);
  dim3 grid((a.P + cols - 1) / cols, a.H, a.runs);
  const int need = (a.N + SLICES - 1) / SLICES;
  auto lds = [&](int npl) {
    const int npad = npl * SLICES;
    return (size_t)(CH * npad * 2 + (MODE == 0 ? CH * npad : 2 * CH)) * sizeof(float);
  };
  if (need <= 4) decay_scan_kernel<T, MODE, 4><<<grid, NT, lds(4), s>>>(a);
  else if (need <= 8) decay_scan_kernel<T, MODE, 8><<<grid, NT, lds(8), s>>>(a);
  else if (need <= 16) decay_scan_kernel<T, MODE, 16><<<grid, NT, lds(16), s>>>(a);
  else if (need <= 32) decay_scan_kernel<T, MODE, 32><<<grid, NT, lds(32), s>>>(a);
  else decay_scan_kernel<T, MODE, 64><<<grid, NT, lds(64), s>>>(a);   // N <= 256 (checked by the op layer)
}

}  // namespace

void launch_decay_scan(const DecayScanArgs& a, int f32, hipStream_t s) {
  if (a.runs <= 0 || a.T <= 0) return;
  if (f32) {
    if (a.mode == 0) launch_mode<float, 0>(a, s);
    else launch_mode<float, 1>(a, s);
  } else {
    if (a.mode == 0) launch_mode<bf16, 0>(a, s);
    else launch_mode<bf16, 1>(a, s);
  }
}
