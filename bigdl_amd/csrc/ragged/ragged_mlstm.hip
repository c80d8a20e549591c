// mLSTM on the ragged engine: the scalar part of the recurrence (gates, running maximum) and the per-head output
// norm with its gate.  The matrix memory itself is the scan of ragged_ops.hip with three gate arrays.
//
// Per head, with log gates i_t, f_t:   m_t = max(f_t + m_(t-1), i_t),
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,  n_t = a_t n_(t-1) + b_t k_t,  a_t = e^(f_t + m_(t-1) - m_t),  b_t = e^(i_t - m_t),
//   o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + floor).
// Only m is a chain from token to token, and a cheap one (an add and a maximum): mlstm_gates_kernel evaluates the gates of
// 64 tokens side by side, walks the chain over them from LDS, and leaves a_t, b_t and e^(-m_t) per (token, head).
// mlstm_expand_kernel turns them into the scan's arrays qf = q_t, ff = a_t (repeated over the rows), gf = b_t k_t; the
// scan carries n as one more column of S whose value is the constant 1, so its output's last column is n_t . q_t, and
// head_norm_gate_kernel divides by the denominator.  Everything here is float whatever the activation type of the
// projections is; exponentials, tanh and logarithms are the full-precision library functions.
#include "ragged_common.h"

using namespace ragged;

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One wavefront per (head, sequence).  mstate: [slots, H].
template <typename T>
__global__ __launch_bounds__(64) void mlstm_gates_kernel(const T* __restrict__ P, int64_t ldp, int i0,
                                                         const float* __restrict__ gate_bias, float cap, float m_start,
                                                         float* __restrict__ mstate, float* __restrict__ a, float* __restrict__ b,
                                                         float* __restrict__ em, int H, Batch bt) {
  __shared__ float sl[64], sf[64];
  const int h = blockIdx.x, sq = blockIdx.y, lane = threadIdx.x;
  const int start = bt.seq_start[sq], n = bt.seq_start[sq + 1] - start, past = bt.seq_past[sq], slot = bt.seq_slot[sq];
  const float bi = gate_bias[h], bf = gate_bias[H + h];
  float m = past > 0 ? mstate[(int64_t)slot * H + h] : m_start;
  for (int j0 = 0; j0 < n; j0 += 64) {
    const int i = j0 + lane;
    const bool live = i < n;
    float li = 0.f, lf = 0.f;
    if (live) {
      const T* row = P + (int64_t)(start + i) * ldp + i0;
      li = cap * tanhf((to_f(row[h]) + bi) / cap);
      lf = log_sigmoid(cap * tanhf((to_f(row[H + h]) + bf) / cap));
    }
    __syncthreads();
    sl[lane] = li;
    sf[lane] = lf;
    __syncthreads();
    const int cnt = n - j0 < 64 ? n - j0 : 64;
    float before = m, after = m;
#pragma unroll 8
    for (int j = 0; j < 64; ++j) {
      const float m2 = j < cnt ? fmaxf(sf[j] + m, sl[j]) : m;
      if (j == lane) { before = m; after = m2; }
      m = m2;
    }
    if (live) {
      const int64_t o = (int64_t)(start + i) * H + h;
      a[o] = expf(lf + before - after);
      b[o] = expf(li - after);
      em[o] = expf(-after);
    }
  }
  if (lane == 0) mstate[(int64_t)slot * H + h] = m;
}

extern "C" int ragged_mlstm_gates(const void* P, int64_t ldp, int i0, const float* gate_bias, float cap, float m_start,
                                  float* mstate, float* a, float* b, float* em, int H, Batch bt, int dtype, hipStream_t st) {
  if (bt.B <= 0 || H <= 0 || !(cap > 0.f) || !mstate || !gate_bias) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((mlstm_gates_kernel<T>), dim3(H, bt.B), dim3(64), 0, st, (const T*)P, ldp, i0, gate_bias,
                                            cap, m_start, mstate, a, b, em, H, bt))
  return RAGGED_LAUNCH_OK();
}

// qf = q * dim^(-1/2), ff = a (one number per token and head, repeated), gf = b * k: float [T, H d] each
template <typename T>
__global__ __launch_bounds__(256) void mlstm_expand_kernel(const T* __restrict__ P, int64_t ldp, int q0, int k0,
                                                           const float* __restrict__ a, const float* __restrict__ b,
                                                           float* __restrict__ qf, float* __restrict__ ff, float* __restrict__ gf,
                                                           int64_t rows, int H, int d, float qs) {
  const int64_t n = rows * H * d;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / (H * d);
    const int c = (int)(i % (H * d)), h = c / d;
    qf[i] = to_f(P[t * ldp + q0 + c]) * qs;
    ff[i] = a[t * H + h];
    gf[i] = b[t * H + h] * to_f(P[t * ldp + k0 + c]);
  }
}

extern "C" int ragged_mlstm_expand(const void* P, int64_t ldp, int q0, int k0, const float* a, const float* b, float* qf, float* ff,
                                   float* gf, int64_t rows, int H, int d, int dtype, hipStream_t st) {
  if (rows <= 0 || H <= 0 || d <= 0) return -1;
  const int64_t n = rows * H * d;
  const unsigned grid = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  const float qs = 1.0f / sqrtf((float)d);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((mlstm_expand_kernel<T>), dim3(grid), dim3(256), 0, st, (const T*)P, ldp, q0, k0, a, b, qf,
                                            ff, gf, rows, H, d, qs))
  return RAGGED_LAUNCH_OK();
}

// out[t, h, :] = u / rms(u) * w[h, :] * sigmoid(gate logits of row t, columns g0 + h * vd ...), u = o[t, h, :vd], or with
// `em`: u = o[t, h, :vd] / (max(|o[t, h, vd]|, em[t, h]) + floor).  o has ldo floats per (row, head).  `scale` multiplies the
// result (a mixer that is one of two summed side by side carries its weight here).  One wavefront per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const T* __restrict__ P, int64_t ldp, int g0, T* __restrict__ out,
                                                             int64_t items, int H, int vd, float eps, int ldo,
                                                             const float* __restrict__ em, float den_floor, float scale) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (item >= items) return;
  const int64_t t = item / H;
  const int h = (int)(item % H);
  const float* row = o + item * ldo;
  const float inv = em ? 1.0f / (fmaxf(fabsf(row[vd]), em[item]) + den_floor) : 1.0f;
  float ss = 0.f;
  for (int c = lane; c < vd; c += 64) { const float v = row[c] * inv; ss += v * v; }
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)vd + eps);
  for (int c = lane; c < vd; c += 64) {
    float v = row[c] * inv * r * w[h * vd + c] * scale;
    if (P) v *= 1.0f / (1.0f + expf(-to_f(P[t * ldp + g0 + h * vd + c])));
    out[item * vd + c] = from_f<T>(v);
  }
}

extern "C" int ragged_head_norm_gate(const float* o, const float* w, const void* P, int64_t ldp, int g0, void* out, int64_t rows,
                                     int H, int vd, float eps, int ldo, const float* em, float den_floor, float scale, int dtype,
                                     hipStream_t st) {
  if (rows <= 0 || H <= 0 || vd <= 0 || rows * H > 0x7fffffff || ldo < vd + (em ? 1 : 0)) return -1;
  const int64_t items = rows * H;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((head_norm_gate_kernel<T>), dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, o, w,
                                            (const T*)P, ldp, g0, (T*)out, items, H, vd, eps, ldo, em, den_floor, scale))
  return RAGGED_LAUNCH_OK();
}
