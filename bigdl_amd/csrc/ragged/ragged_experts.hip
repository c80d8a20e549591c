// Routed experts of the ragged engine: the router (32-bit softmax scores, group-limited choice of the best experts) and
// the row-wise expert products that serve single decoded tokens and short portions, where every (row, chosen expert) pair
// reads its expert's weights once.  Long portions run their experts as dense library products over rows sorted by expert
// (models/ragged_engine.py); they share the router and the activation kernel with this path.
#include "ragged_common.h"

using namespace ragged;

constexpr int MOE_MAX_E = 512;      // experts
constexpr int MOE_SLOTS = MOE_MAX_E / 64;

// Scores s = softmax(W_r x) over all experts (score_fn 0) or sigmoid(W_r x) per expert (score_fn 1), in float (x may be
// the bfloat16 rounding of the normed stream).  Experts form `groups` equal runs of neighbours; a group's score is the sum
// of its `group_top` (1 or 2) best experts' scores; the `top` best experts of the `keep` best groups are chosen, best
// first, with weight s * scale, or (renorm) s / (sum of the chosen s + 1e-20) * scale.  Ties go to the lower lane.
// One workgroup of four wavefronts per row: the wavefronts share the router's rows, wavefront 0 chooses.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ x, int64_t ldx, const float* __restrict__ wr,
                                                        int* __restrict__ idx, float* __restrict__ wts, int D, int E, int groups,
                                                        int keep, int top, float scale, int score_fn, int group_top, int renorm) {
  __shared__ float z[MOE_MAX_E];
  __shared__ float gbest[64];
  extern __shared__ __attribute__((aligned(16))) float xs[];       // the row as floats
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* xr = x + (int64_t)t * ldx;
  for (int c = threadIdx.x; c < D; c += 256) xs[c] = to_f(xr[c]);
  __syncthreads();
  // two experts per wavefront and pass, 16 bytes of each router row per lane: eight loads in flight
  const bool v4 = (D & 3) == 0;
  for (int e0 = 2 * wave; e0 < E; e0 += 8) {
    const int e1 = e0 + 1 < E ? e0 + 1 : e0;
    const float* w0 = wr + (int64_t)e0 * D;
    const float* w1 = wr + (int64_t)e1 * D;
    float a0 = 0.f, a1 = 0.f;
    if (v4) {
      for (int c = 4 * lane; c < D; c += 1024) {
        float4 p[4], q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int cc = c + 256 * u < D ? c + 256 * u : c;
          p[u] = *reinterpret_cast<const float4*>(w0 + cc);
          q[u] = *reinterpret_cast<const float4*>(w1 + cc);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c + 256 * u < D) {
            const float4 xv = *reinterpret_cast<const float4*>(xs + c + 256 * u);
            a0 += p[u].x * xv.x + p[u].y * xv.y + p[u].z * xv.z + p[u].w * xv.w;
            a1 += q[u].x * xv.x + q[u].y * xv.y + q[u].z * xv.z + q[u].w * xv.w;
          }
      }
    } else {
      for (int c = lane; c < D; c += 64) { a0 += w0[c] * xs[c]; a1 += w1[c] * xs[c]; }
    }
    a0 = wave_sum(a0);
    a1 = wave_sum(a1);
    if (lane == 0) { z[e0] = a0; z[e1] = a1; }
  }
  __syncthreads();
  if (wave != 0) return;
  float s[MOE_SLOTS];
  if (score_fn == 1) {
#pragma unroll
    for (int k = 0; k < MOE_SLOTS; ++k) {
      const int e = lane + 64 * k;
      s[k] = e < E ? 1.0f / (1.0f + expf(-z[e])) : 0.f;
      if (e < E) z[e] = s[k];
    }
  } else {
    float mx = -1e30f;
#pragma unroll
    for (int k = 0; k < MOE_SLOTS; ++k) {
      const int e = lane + 64 * k;
      s[k] = e < E ? z[e] : -1e30f;
      mx = fmaxf(mx, s[k]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < MOE_SLOTS; ++k) {
      const int e = lane + 64 * k;
      s[k] = e < E ? expf(s[k] - mx) : 0.f;
      sum += s[k];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int k = 0; k < MOE_SLOTS; ++k) {
      const int e = lane + 64 * k;
      s[k] = s[k] / sum;
      if (e < E) z[e] = s[k];
    }
  }
  // (a wavefront's LDS requests are served in order: the scores written above are what is read below)
  const int gsz = E / groups;
  if (groups > 1 && keep < groups) {
    float g = -1.f;
    if (lane < groups) {
      float second = 0.f;                                   // (scores are not negative: a group of one adds nothing)
      for (int j = 0; j < gsz; ++j) {
        const float v = z[lane * gsz + j];
        if (v > g) { second = g > 0.f ? g : 0.f; g = v; }
        else if (v > second) second = v;
      }
      if (group_top == 2) g += second;
    }
    bool kept = false;
    for (int it = 0; it < keep; ++it) {
      const float best = wave_max(kept ? -1.f : g);
      const unsigned long long who = __ballot(!kept && g == best && lane < groups);
      if (lane == __ffsll((long long)who) - 1) kept = true;
    }
    gbest[lane] = kept ? 1.f : 0.f;
#pragma unroll
    for (int k = 0; k < MOE_SLOTS; ++k) {
      const int e = lane + 64 * k;
      if (e < E && gbest[e / gsz] == 0.f) s[k] = -1.f;
    }
  }
#pragma unroll
  for (int k = 0; k < MOE_SLOTS; ++k)
    if (lane + 64 * k >= E) s[k] = -1.f;
  float total = 0.f, kept_w = 0.f;                         // lane `it` keeps the score of the it-th choice (top <= 64 with renorm)
  for (int it = 0; it < top; ++it) {
    float mine = s[0];
    int at = 0;
#pragma unroll
    for (int k = 1; k < MOE_SLOTS; ++k)
      if (s[k] > mine) { mine = s[k]; at = k; }
    const float best = wave_max(mine);
    const unsigned long long who = __ballot(mine == best);
    total += best;
    if (lane == (it & 63)) kept_w = best;
    if (lane == __ffsll((long long)who) - 1) {
      idx[(int64_t)t * top + it] = lane + 64 * at;
      if (!renorm) wts[(int64_t)t * top + it] = best * scale;
#pragma unroll
      for (int k = 0; k < MOE_SLOTS; ++k)
        if (k == at) s[k] = -2.f;
    }
  }
  if (renorm && lane < top) wts[(int64_t)t * top + lane] = kept_w / (total + 1e-20f) * scale;
}

extern "C" int ragged_moe_route(const void* x, int64_t ldx, const float* wr, int* idx, float* wts, int64_t rows, int D, int E,
                                int groups, int keep, int top, float scale, int score_fn, int group_top, int renorm, int dtype,
                                hipStream_t st) {
  if (score_fn < 0 || score_fn > 1 || group_top < 1 || group_top > 2 || (renorm && top > 64)) return -1;
  if (rows <= 0 || rows > 0x7fffffff || D <= 0 || D > 12288 || E <= 0 || E > MOE_MAX_E || groups <= 0 || groups > 64 || E % groups) return -1;
  if (keep <= 0 || keep > groups || top <= 0 || top > keep * (E / groups)) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((moe_route_kernel<T>), dim3((unsigned)rows), dim3(256), D * sizeof(float), st, (const T*)x, ldx, wr, idx,
                                            wts, D, E, groups, keep, top, scale, score_fn, group_top, renorm))
  return RAGGED_LAUNCH_OK();
}

// relu(a)^2, elementwise
template <typename T>
__global__ __launch_bounds__(256) void relu2_kernel(const T* __restrict__ a, T* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float v = fmaxf(to_f(a[i]), 0.f);
    out[i] = from_f<T>(v * v);
  }
}

extern "C" int ragged_relu2(const void* a, void* out, int64_t n, int dtype, hipStream_t st) {
  if (n <= 0) return -1;
  const unsigned grid = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((relu2_kernel<T>), dim3(grid), dim3(256), 0, st, (const T*)a, (T*)out, n))
  return RAGGED_LAUNCH_OK();
}

// ---- row-wise expert products.  dot of a weight row with a vector held in LDS as floats, lanes striding 16 bytes
template <typename T> struct WVec;
template <> struct WVec<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const uint4& u, float* o) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <> struct WVec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const uint4& u, float* o) {
    o[0] = __uint_as_float(u.x); o[1] = __uint_as_float(u.y); o[2] = __uint_as_float(u.z); o[3] = __uint_as_float(u.w);
  }
};

// partial dot products of R weight rows (row r at w + r * K) with xs[0 .. K), this lane's share; K % N == 0 and rows
// 16-byte aligned when vec
template <typename T, int R>
__device__ __forceinline__ void rows_dot(const T* __restrict__ w, int64_t K, int nrows, const float* xs, bool vec, int lane,
                                         float (&acc)[R]) {
  constexpr int N = WVec<T>::N;
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  if (vec) {
    // four strides of every row requested before the first is used: 4 R loads of 16 bytes in flight per lane
    constexpr int UN = 4;
    for (int c0 = lane * N; c0 < K; c0 += UN * 64 * N) {
      uint4 raw[UN][R];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int c = c0 + u * 64 * N < K ? c0 + u * 64 * N : c0;
#pragma unroll
        for (int r = 0; r < R; ++r)
          raw[u][r] = *reinterpret_cast<const uint4*>(w + (int64_t)(r < nrows ? r : nrows - 1) * K + c);
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int c = c0 + u * 64 * N;
        if (c < K) {
#pragma unroll
          for (int r = 0; r < R; ++r) {
            float wv[N];
            WVec<T>::unpack(raw[u][r], wv);
#pragma unroll
            for (int e = 0; e < N; ++e) acc[r] += wv[e] * xs[c + e];
          }
        }
      }
    }
  } else {
    for (int c = lane; c < K; c += 64)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += to_f(w[(int64_t)(r < nrows ? r : nrows - 1) * K + c]) * xs[c];
  }
}

constexpr int MOE_RW = 4;           // weight rows per wavefront and pass

// ACT 0: A[(t, j), f] = relu(W_up[idx[t, j]][f, :] . x[t, :])^2.  ACT 1 (gated experts): W_up holds 2 ff rows per expert, the
// gate row and the up row of inner channel f next to each other (rows 2 f, 2 f + 1), and A[(t, j), f] = silu(gate) * up.
// Grid (rows * top, blocks of 4 * MOE_RW weight rows); `ff` counts the weight rows of an expert.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void moe_rows_up_kernel(const T* __restrict__ x, int64_t ldx, const int* __restrict__ idx,
                                                          const T* __restrict__ w_up, T* __restrict__ A, int D, int ff, int top,
                                                          int vec) {
  extern __shared__ __attribute__((aligned(16))) float xs[];
  const int pair = blockIdx.x, t = pair / top;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int c = threadIdx.x; c < D; c += 256) xs[c] = to_f(x[(int64_t)t * ldx + c]);
  __syncthreads();
  const int f0 = (blockIdx.y * 4 + wave) * MOE_RW;
  if (f0 >= ff) return;
  const int nrows = ff - f0 < MOE_RW ? ff - f0 : MOE_RW;
  const T* w = w_up + ((int64_t)idx[pair] * ff + f0) * D;
  float acc[MOE_RW];
  rows_dot<T, MOE_RW>(w, D, nrows, xs, vec != 0, lane, acc);
#pragma unroll
  for (int r = 0; r < MOE_RW; ++r) acc[r] = wave_sum(acc[r]);
  if (ACT == 1) {
#pragma unroll
    for (int r = 0; r < MOE_RW; r += 2)
      if (lane == 0 && r + 1 < nrows)
        A[(int64_t)pair * (ff / 2) + (f0 + r) / 2] = from_f<T>(acc[r] / (1.0f + expf(-acc[r])) * acc[r + 1]);
  } else {
#pragma unroll
    for (int r = 0; r < MOE_RW; ++r) {
      const float v = fmaxf(acc[r], 0.f);
      if (lane == 0 && r < nrows) A[(int64_t)pair * ff + f0 + r] = from_f<T>(v * v);
    }
  }
}

// y[t, c] = base[t, c] + sum_j wts[t, j] * W_down[idx[t, j]][c, :] . A[(t, j), :].  Grid (rows, blocks of 4 * MOE_RW channels).
template <typename T>
__global__ __launch_bounds__(256) void moe_rows_down_kernel(const T* __restrict__ A, const int* __restrict__ idx,
                                                            const float* __restrict__ wts, const T* __restrict__ w_dn,
                                                            const T* __restrict__ base, T* __restrict__ y, int D, int ff, int top,
                                                            int vec) {
  extern __shared__ __attribute__((aligned(16))) float as[];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c0 = (blockIdx.y * 4 + wave) * MOE_RW;
  const int nrows = c0 < D ? (D - c0 < MOE_RW ? D - c0 : MOE_RW) : 0;
  float tot[MOE_RW];
#pragma unroll
  for (int r = 0; r < MOE_RW; ++r) tot[r] = 0.f;
  for (int j = 0; j < top; ++j) {
    __syncthreads();
    for (int c = threadIdx.x; c < ff; c += 256) as[c] = to_f(A[((int64_t)t * top + j) * ff + c]);
    __syncthreads();
    if (nrows > 0) {
      const T* w = w_dn + ((int64_t)idx[(int64_t)t * top + j] * D + c0) * ff;
      float acc[MOE_RW];
      rows_dot<T, MOE_RW>(w, ff, nrows, as, vec != 0, lane, acc);
      const float wt = wts[(int64_t)t * top + j];
#pragma unroll
      for (int r = 0; r < MOE_RW; ++r) tot[r] += wt * wave_sum(acc[r]);
    }
  }
  if (lane == 0)
#pragma unroll
    for (int r = 0; r < MOE_RW; ++r)
      if (r < nrows) {
        const int64_t o = (int64_t)t * D + c0 + r;
        y[o] = from_f<T>(tot[r] + (base ? to_f(base[o]) : 0.f));
      }
}

// act 0: two-matrix experts with relu^2; act 1: gated experts, w_up [E, 2 ff, D] with (gate, up) rows next to each other
extern "C" int ragged_moe_rows(const void* x, int64_t ldx, const int* idx, const float* wts, const void* w_up, const void* w_dn,
                               const void* base, void* A, void* y, int64_t rows, int D, int ff, int top, int act, int dtype,
                               hipStream_t st) {
  if (rows <= 0 || D <= 0 || ff <= 0 || top <= 0 || rows * top > 0x7fffffff || D > 12288 || ff > 12288) return -1;
  if (act < 0 || act > 1) return -1;
  const int per = 4 * MOE_RW;
  const int wrows = act == 1 ? 2 * ff : ff;
  RAGGED_DISPATCH(dtype,
    const int vu = D % WVec<T>::N == 0; const int vd = ff % WVec<T>::N == 0;
    if (act == 1)
      hipLaunchKernelGGL((moe_rows_up_kernel<T, 1>), dim3((unsigned)(rows * top), (wrows + per - 1) / per), dim3(256), D * sizeof(float),
                         st, (const T*)x, ldx, idx, (const T*)w_up, (T*)A, D, wrows, top, vu);
    else
      hipLaunchKernelGGL((moe_rows_up_kernel<T, 0>), dim3((unsigned)(rows * top), (ff + per - 1) / per), dim3(256), D * sizeof(float), st,
                         (const T*)x, ldx, idx, (const T*)w_up, (T*)A, D, ff, top, vu);
    hipLaunchKernelGGL((moe_rows_down_kernel<T>), dim3((unsigned)rows, (D + per - 1) / per), dim3(256), ff * sizeof(float), st,
                       (const T*)A, idx, wts, (const T*)w_dn, (const T*)base, (T*)y, D, ff, top, vd))
  return RAGGED_LAUNCH_OK();
}

// y[t, :] = base[t, :] + sum_j wts[t, j] * ys[place[t, j], :]: the experts' outputs, computed on rows sorted by expert,
// brought back to their rows (every row sums its own terms in the order of its choices).
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T* __restrict__ ys, const int* __restrict__ place,
                                                          const float* __restrict__ wts, const T* __restrict__ base,
                                                          T* __restrict__ y, int D, int top) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < D; c += 256) {
    float acc = base ? to_f(base[t * D + c]) : 0.f;
    for (int j = 0; j < top; ++j) acc += wts[t * top + j] * to_f(ys[(int64_t)place[t * top + j] * D + c]);
    y[t * D + c] = from_f<T>(acc);
  }
}

extern "C" int ragged_moe_combine(const void* ys, const int* place, const float* wts, const void* base, void* y, int64_t rows, int D,
                                  int top, int dtype, hipStream_t st) {
  if (rows <= 0 || rows > 0x7fffffff || D <= 0 || top <= 0) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((moe_combine_kernel<T>), dim3((unsigned)rows), dim3(256), 0, st, (const T*)ys, place, wts,
                                            (const T*)base, (T*)y, D, top))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Long portions: the experts' products over rows sorted by expert, one launch for all experts (bfloat16, matrix cores).
// moe_tile_map_kernel cuts every expert's run of rows [seg[e], seg[e + 1]) into tiles of 64 rows; the product kernel's
// workgroup (tile, block of 256 output channels) computes out^T = W_e X^T with v_mfma_f32_16x16x32_bf16, wavefront w all 64
// rows against channels 64 w .. 64 w + 63: a lane holds one row and four neighbouring output channels of each 16 x 16
// block, so a row's results are stored 8 bytes at a time.  K runs in steps of 64 channels: the step's weight tile
// [256][64] and activation tile [64][64] are read by the whole workgroup in 128-byte row pieces into registers while the
// previous step's matrix instructions run, stored to the other of two LDS buffers, and read back as fragments (both
// operands are K-contiguous, so a fragment is one 16-byte LDS read); one barrier per step.
// src_row: the activation row behind every sorted place (null: the place itself).  ACT = 1: relu(.)^2 on the way out.
// ACT = 2: the N output channels are (gate, up) pairs of N / 2 inner channels, out[row, c] = silu(gate_c) * up_c (a lane's
// four neighbouring channels are two whole pairs; the output rows are N / 2 long).
typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));
union MoeFrag {
  moe_bf16x8 v;
  uint4 q;
};

constexpr int MG_ROWS = 64;       // rows of a tile
constexpr int MG_NB = 4;          // 16-channel blocks of a wavefront: a workgroup covers 256 output channels

__global__ __launch_bounds__(512) void moe_tile_map_kernel(const int* __restrict__ seg, int E, int* __restrict__ tile_e,
                                                           int* __restrict__ tile_r0, int* __restrict__ ntiles, int max_tiles) {
  __shared__ int first[MOE_MAX_E + 1];
  const int e = threadIdx.x;
  const int len = e < E ? seg[e + 1] - seg[e] : 0;
  const int cnt = (len + MG_ROWS - 1) / MG_ROWS;
  first[e + 1 <= MOE_MAX_E ? e + 1 : MOE_MAX_E] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    first[0] = 0;
    for (int i = 1; i <= E; ++i) first[i] += first[i - 1];
    *ntiles = first[E] < max_tiles ? first[E] : max_tiles;
  }
  __syncthreads();
  if (e < E)
    for (int j = 0; j < cnt; ++j)
      if (first[e] + j < max_tiles) {
        tile_e[first[e] + j] = e;
        tile_r0[first[e] + j] = seg[e] + j * MG_ROWS;
      }
}

constexpr int MG_K = 32;          // channels of a K step
constexpr int MG_LD = MG_K + 8;   // LDS row stride in elements: rows stay 16-byte aligned and neighbouring rows shift banks
constexpr int MG_N = 64 * MG_NB;  // output channels of a workgroup

template <int ACT>
__global__ __launch_bounds__(256) void moe_grouped_gemm_kernel(const bf16* __restrict__ X, int64_t ldx, const int* __restrict__ src_row,
                                                               const bf16* __restrict__ W, bf16* __restrict__ out,
                                                               const int* __restrict__ seg, const int* __restrict__ tile_e,
                                                               const int* __restrict__ tile_r0, const int* __restrict__ ntiles,
                                                               int N, int K) {
  extern __shared__ __attribute__((aligned(16))) uint16_t tiles[];   // 2 x { W [MG_N][MG_LD], X [MG_ROWS][MG_LD] }
  const int tile = blockIdx.x;
  if (tile >= *ntiles) return;                             // (the whole workgroup leaves: no barrier is left waiting)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int lq = lane & 15, g4 = lane >> 4;
  const int e = tile_e[tile], r0 = tile_r0[tile], rend = seg[e + 1];
  const int nw = blockIdx.y * MG_N;                        // the workgroup's first output channel
  constexpr int RB = MG_ROWS / 16, BUF = (MG_N + MG_ROWS) * MG_LD;
  constexpr int PPR = MG_K / 8;                            // 16-byte pieces of a tile row
  constexpr int WP = MG_N * PPR / 256, XP = MG_ROWS * PPR / 256;   // pieces per thread
  // loaders: piece p of a tile = (row p / 8, channels 8 (p % 8) ..): eight neighbouring threads read 128 bytes of a row
  const bf16* wsrc[WP];
  const bf16* xsrc[XP];
#pragma unroll
  for (int u = 0; u < WP; ++u) {
    const int n = nw + (tid + 256 * u) / PPR;
    wsrc[u] = n < N ? W + ((int64_t)e * N + n) * K : nullptr;
  }
#pragma unroll
  for (int u = 0; u < XP; ++u) {
    const int row = r0 + (tid + 256 * u) / PPR;
    const int place = row < rend ? row : r0;
    xsrc[u] = X + (int64_t)(src_row ? src_row[place] : place) * ldx;
  }
  const int pc = 8 * (tid % PPR);
  uint4 wreg[WP], xreg[XP];
  auto gload = [&](int k0) {
    const int k = k0 + pc;
#pragma unroll
    for (int u = 0; u < WP; ++u)
      wreg[u] = (wsrc[u] && k < K) ? *reinterpret_cast<const uint4*>(wsrc[u] + k) : uint4{0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < XP; ++u) xreg[u] = k < K ? *reinterpret_cast<const uint4*>(xsrc[u] + k) : uint4{0, 0, 0, 0};
  };
  auto lstore = [&](uint16_t* buf) {
#pragma unroll
    for (int u = 0; u < WP; ++u) *reinterpret_cast<uint4*>(buf + ((tid + 256 * u) / PPR) * MG_LD + pc) = wreg[u];
#pragma unroll
    for (int u = 0; u < XP; ++u) *reinterpret_cast<uint4*>(buf + (MG_N + (tid + 256 * u) / PPR) * MG_LD + pc) = xreg[u];
  };
  moe_f32x4 acc[RB][MG_NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int nb = 0; nb < MG_NB; ++nb) acc[rb][nb] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
  gload(0);
  lstore(tiles);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < K; k0 += MG_K) {
    const bool more = k0 + MG_K < K;
    if (more) gload(k0 + MG_K);                            // in flight during this step's matrix instructions
    const uint16_t* wt = tiles + cur * BUF + (64 * wave) * MG_LD;
    const uint16_t* xt = tiles + cur * BUF + MG_N * MG_LD;
#pragma unroll
    for (int ks = 0; ks < MG_K / 32; ++ks) {
      MoeFrag xf[RB], wf[MG_NB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) xf[rb].q = *reinterpret_cast<const uint4*>(xt + (16 * rb + lq) * MG_LD + 32 * ks + 8 * g4);
#pragma unroll
      for (int nb = 0; nb < MG_NB; ++nb) wf[nb].q = *reinterpret_cast<const uint4*>(wt + (16 * nb + lq) * MG_LD + 32 * ks + 8 * g4);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int nb = 0; nb < MG_NB; ++nb)
          acc[rb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nb].v, xf[rb].v, acc[rb][nb], 0, 0, 0);
    }
    if (more) lstore(tiles + (cur ^ 1) * BUF);             // (its last readers passed the barrier of the step before)
    __syncthreads();
    cur ^= 1;
  }
  const int n0 = nw + 64 * wave;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = r0 + 16 * rb + lq;
    if (row >= rend) continue;
    bf16* orow = out + (ACT == 2 ? (int64_t)row * (N / 2) + n0 / 2 : (int64_t)row * N + n0);
#pragma unroll
    for (int nb = 0; nb < MG_NB; ++nb) {
      const int n = 16 * nb + 4 * g4;
      if (n0 + n < N) {                                    // N is a multiple of 16: four channels are in or out together
        if (ACT == 2) {
          const float g0 = acc[rb][nb][0], g1 = acc[rb][nb][2];
          const float a0 = g0 / (1.0f + __expf(-g0)) * acc[rb][nb][1], a1 = g1 / (1.0f + __expf(-g1)) * acc[rb][nb][3];
          *reinterpret_cast<uint32_t*>(orow + n / 2) = (uint32_t)from_f<bf16>(a0).b | ((uint32_t)from_f<bf16>(a1).b << 16);
          continue;
        }
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i] = acc[rb][nb][i];
          if (ACT == 1) { v[i] = fmaxf(v[i], 0.f); v[i] *= v[i]; }
        }
        uint2 w;
        w.x = (uint32_t)from_f<bf16>(v[0]).b | ((uint32_t)from_f<bf16>(v[1]).b << 16);
        w.y = (uint32_t)from_f<bf16>(v[2]).b | ((uint32_t)from_f<bf16>(v[3]).b << 16);
        *reinterpret_cast<uint2*>(orow + n) = w;
      }
    }
  }
}

// 1 when the grouped product serves these sizes (bfloat16 only)
extern "C" int ragged_moe_grouped_ok(int N, int K, int E) { return N % 16 == 0 && K % 8 == 0 && E <= MOE_MAX_E; }

extern "C" int ragged_moe_tile_map(const int* seg, int E, int* tile_e, int* tile_r0, int* ntiles, int max_tiles, hipStream_t st) {
  if (E <= 0 || E > MOE_MAX_E || max_tiles <= 0) return -1;
  hipLaunchKernelGGL(moe_tile_map_kernel, dim3(1), dim3(512), 0, st, seg, E, tile_e, tile_r0, ntiles, max_tiles);
  return RAGGED_LAUNCH_OK();
}

// out[place, :N] = act(X[src_row[place], :K] . W[expert of the place][:N, :K]^T) for all sorted places
extern "C" int ragged_moe_grouped_gemm(const void* X, int64_t ldx, const int* src_row, const void* W, void* out, const int* seg,
                                       const int* tile_e, const int* tile_r0, const int* ntiles, int max_tiles, int N, int K, int E,
                                       int act, hipStream_t st) {
  if (max_tiles <= 0 || !ragged_moe_grouped_ok(N, K, E) || N <= 0 || K <= 0 || ldx < K || ldx % 8) return -1;
  const dim3 grid(max_tiles, (N + MG_N - 1) / MG_N);
  const size_t lds = 2 * (size_t)(MG_N + MG_ROWS) * MG_LD * sizeof(uint16_t);
  static bool raised = false;                               // two tiles above 64 KB: the limit is raised once per kernel
  if (!raised) {
    if (hipFuncSetAttribute((const void*)moe_grouped_gemm_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||
        hipFuncSetAttribute((const void*)moe_grouped_gemm_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||
        hipFuncSetAttribute((const void*)moe_grouped_gemm_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return -3;
    raised = true;
  }
  if (act < 0 || act > 2) return -1;
  if (act == 2)
    hipLaunchKernelGGL((moe_grouped_gemm_kernel<2>), grid, dim3(256), lds, st, (const bf16*)X, ldx, src_row, (const bf16*)W, (bf16*)out,
                       seg, tile_e, tile_r0, ntiles, N, K);
  else if (act == 1)
    hipLaunchKernelGGL((moe_grouped_gemm_kernel<1>), grid, dim3(256), lds, st, (const bf16*)X, ldx, src_row, (const bf16*)W, (bf16*)out,
                       seg, tile_e, tile_r0, ntiles, N, K);
  else
    hipLaunchKernelGGL((moe_grouped_gemm_kernel<0>), grid, dim3(256), lds, st, (const bf16*)X, ldx, src_row, (const bf16*)W, (bf16*)out,
                       seg, tile_e, tile_r0, ntiles, N, K);
  return RAGGED_LAUNCH_OK();
}
