// Row-wise kernels of the ragged engine: residual sum + grouped RMS norm, short causal convolution with per-sequence
// state + per-head norm + rotary + paged append, clamped gated activation, HGRN2 gates / scan / output norm, the stream
// updates of the sandwich, parallel and sequential pre-norm blocks (the last over several copies of the stream),
// embedding rows, activations of dense feed-forwards, gates per channel.
// gfx950, wave64.  Everything that the engine keeps in 32 bits (residual, norms, angles, gates, recurrent state) is
// float here whatever the activation type T is.
#include "ragged_common.h"

using namespace ragged;

// ---------------------------------------------------------------------------------------------------------------
// x <- w * groupnorm(alpha * x + y): the vector is cut into `groups` equal parts, each divided by its own root mean
// square (eps inside the root).  One workgroup per (row, group).  x float in place; xa: the same values as T for the
// matrix product that reads them next.  y may be null (a plain norm).  x_out may differ from x (the final norm).
template <typename T>
__global__ __launch_bounds__(256) void sum_group_norm_kernel(const float* __restrict__ x, const T* __restrict__ y,
                                                             const float* __restrict__ w, float* __restrict__ x_out,
                                                             T* __restrict__ xa, int D, int groups, float alpha, float eps) {
  const int row = blockIdx.x / groups, g = blockIdx.x % groups, dg = D / groups;
  const int64_t base = (int64_t)row * D + (int64_t)g * dg;
  __shared__ float red[4];
  float ss = 0.f;
  for (int c = threadIdx.x; c < dg; c += 256) {
    float v = alpha * x[base + c] + (y ? to_f(y[base + c]) : 0.f);
    ss += v * v;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float r = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)dg + eps);
  for (int c = threadIdx.x; c < dg; c += 256) {
    float v = alpha * x[base + c] + (y ? to_f(y[base + c]) : 0.f);
    v = v * r * w[g * dg + c];
    if (x_out) x_out[base + c] = v;
    if (xa) xa[base + c] = from_f<T>(v);
  }
}

extern "C" int ragged_sum_group_norm(const float* x, const void* y, const float* w, float* x_out, void* xa, int64_t rows,
                                     int D, int groups, float alpha, float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || D <= 0 || groups <= 0 || D % groups || rows * groups > 0x7fffffff) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((sum_group_norm_kernel<T>), dim3((unsigned)(rows * groups)), dim3(256), 0, st, x,
                                            (const T*)y, w, x_out, (T*)xa, D, groups, alpha, eps))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Sandwich form: x <- x + w_post * rmsnorm(y), then (w_next given) xa = w_next * rmsnorm(x) for the product that reads
// the stream next.  One workgroup per row; x float in place, y and xa of type T.  Each thread re-reads only what it
// wrote itself, so the passes need no barrier beyond those of the two sums.
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// NV > 0: rows of at most 256 NV channels, each thread keeps its NV sums in registers (every operand is read once);
// NV = 0: any width, the passes re-read what they need.
template <typename T, int NV>
__global__ __launch_bounds__(256) void post_norm_add_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                            const float* __restrict__ w_post, const float* __restrict__ w_next,
                                                            T* __restrict__ xa, int D, float eps) {
  __shared__ float red[8];
  const int64_t base = (int64_t)blockIdx.x * D;
  if (NV > 0) {
    float yv[NV > 0 ? NV : 1], xv[NV > 0 ? NV : 1], wp[NV > 0 ? NV : 1], wn[NV > 0 ? NV : 1];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int c = threadIdx.x + 256 * u;
      const bool ok = c < D;
      yv[u] = ok ? to_f(y[base + c]) : 0.f;
      xv[u] = ok ? x[base + c] : 0.f;
      wp[u] = ok ? w_post[c] : 0.f;
      wn[u] = (ok && xa) ? w_next[c] : 0.f;
      ss += yv[u] * yv[u];
    }
    const float r1 = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
    ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int c = threadIdx.x + 256 * u;
      xv[u] += yv[u] * r1 * wp[u];
      if (c < D) x[base + c] = xv[u];
      ss += xv[u] * xv[u];
    }
    if (!xa) return;
    const float r2 = 1.0f / sqrtf(block_sum_256(ss, red + 4) / (float)D + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int c = threadIdx.x + 256 * u;
      if (c < D) xa[base + c] = from_f<T>(xv[u] * r2 * wn[u]);
    }
    return;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < D; c += 256) { const float v = to_f(y[base + c]); ss += v * v; }
  const float r1 = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
  ss = 0.f;
  for (int c = threadIdx.x; c < D; c += 256) {
    const float v = x[base + c] + to_f(y[base + c]) * r1 * w_post[c];
    x[base + c] = v;
    ss += v * v;
  }
  if (!xa) return;
  const float r2 = 1.0f / sqrtf(block_sum_256(ss, red + 4) / (float)D + eps);
  for (int c = threadIdx.x; c < D; c += 256) xa[base + c] = from_f<T>(x[base + c] * r2 * w_next[c]);
}

extern "C" int ragged_post_norm_add(float* x, const void* y, const float* w_post, const float* w_next, void* xa, int64_t rows,
                                    int D, float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || D <= 0 || rows > 0x7fffffff || !x || !y || !w_post || (xa && !w_next)) return -1;
  RAGGED_DISPATCH(dtype,
    if (D <= 1024) hipLaunchKernelGGL((post_norm_add_kernel<T, 4>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y, w_post,
                                      w_next, (T*)xa, D, eps);
    else if (D <= 4096) hipLaunchKernelGGL((post_norm_add_kernel<T, 16>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y,
                                           w_post, w_next, (T*)xa, D, eps);
    else hipLaunchKernelGGL((post_norm_add_kernel<T, 0>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y, w_post, w_next,
                            (T*)xa, D, eps))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Short causal convolution over time per channel, then (optionally) RMS norm over groups of `gsize` channels with a
// weight shared by all groups, then (optionally) rotation of the first `rot` channels of each group (pairs i, i + rot/2,
// cosine and sine of the row's angles from a table made once per step), then a store into a dense float buffer or into
// cache pages.
struct ConvHeadArgs {
  const void* P;          // [T, ldp] projections of this step
  int64_t ldp;
  int col0;               // first column of this segment in P
  const float* cw;        // [C, taps] taps of the whole convolved region, or null (no convolution)
  int taps, C, ch0;       // ch0: this segment's first channel inside the convolved region
  const void* state;      // [slots, taps - 1, C]: the last taps - 1 projected rows of every sequence
  int ngroups, gsize;
  const float* normw;     // [gsize] or null
  float eps;
  int rot;                // 0: no rotation
  const float* cossin;    // [T, rot / 2, 2]: cos and sin of position * frequency for every row of the batch
  float* out_dense;       // [T, ngroups * gsize] or null
  void* pages;            // [num_pages, heads, PAGE, rowlen]
  int rowlen, heads;
  int norm_n;             // leading channels of a group that the norm covers (0: all of them)
  int rot0;               // first rotated channel of a group
  int interleaved;        // 1: the pairs are neighbours (2 i, 2 i + 1) instead of (i, i + rot / 2)
};

template <typename T>
__global__ __launch_bounds__(256) void conv_head_kernel(ConvHeadArgs a, Batch bt) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  const bool live = item < (int64_t)bt.T * a.ngroups;
  float* buf = smem + wave * a.gsize;
  int t = 0, grp = 0, b = 0, pos = 0, past = 0, slot = 0;
  if (live) {
    t = (int)(item / a.ngroups);
    grp = (int)(item % a.ngroups);
    b = bt.tok_seq[t];
    pos = bt.tok_pos[t];
    past = bt.seq_past[b];
    slot = bt.seq_slot[b];
  }
  const T* P = (const T*)a.P;
  const T* S = (const T*)a.state;
  const int nn = a.norm_n > 0 ? a.norm_n : a.gsize;
  float ss = 0.f;
  if (live) {
    for (int c = lane; c < a.gsize; c += 64) {
      const int f = grp * a.gsize + c;           // channel inside the segment
      float v;
      if (a.cw) {
        const int ch = a.ch0 + f;
        v = 0.f;
        for (int j = 0; j < a.taps; ++j) {
          const int back = a.taps - 1 - j, pp = pos - back;
          float u = 0.f;
          if (pp >= past) u = to_f(P[(int64_t)(t - back) * a.ldp + a.col0 + f]);
          else if (pp >= 0) u = to_f(S[((int64_t)slot * (a.taps - 1) + (pp - past + a.taps - 1)) * a.C + ch]);
          v += a.cw[(int64_t)ch * a.taps + j] * u;
        }
      } else {
        v = to_f(P[(int64_t)t * a.ldp + a.col0 + f]);
      }
      buf[c] = v;
      if (c < nn) ss += v * v;
    }
  }
  if (a.normw) {
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)nn + a.eps);
    if (live)
      for (int c = lane; c < nn; c += 64) buf[c] = buf[c] * r * a.normw[c];
  }
  __syncthreads();
  if (!live) return;
  const int half = a.rot >> 1;
  for (int c = lane; c < a.gsize; c += 64) {
    float v = buf[c];
    const int rc = c - a.rot0;
    if (rc >= 0 && rc < a.rot) {
      const bool first = a.interleaved ? !(rc & 1) : rc < half;
      const int i = a.interleaved ? rc >> 1 : (first ? rc : rc - half), step = a.interleaved ? 1 : half;
      const float2 tr = *reinterpret_cast<const float2*>(a.cossin + ((int64_t)t * half + i) * 2);
      const float cs = tr.x, sn = tr.y;
      v = first ? buf[c] * cs - buf[c + step] * sn : buf[c] * cs + buf[c - step] * sn;
    }
    const int f = grp * a.gsize + c;
    if (a.out_dense) {
      a.out_dense[(int64_t)t * a.ngroups * a.gsize + f] = v;
    } else {
      const int head = f / a.rowlen, off = f % a.rowlen;
      const int page = bt.pages[(int64_t)b * bt.max_pages + pos / PAGE];
      ((T*)a.pages)[(((int64_t)page * a.heads + head) * PAGE + (pos % PAGE)) * a.rowlen + off] = from_f<T>(v);
    }
  }
}

extern "C" int ragged_conv_head(ConvHeadArgs a, Batch bt, int dtype, hipStream_t st) {
  if (bt.T <= 0 || a.ngroups <= 0 || a.gsize <= 0 || a.gsize > 2048) return -1;
  if (a.cw && (a.taps < 1 || a.taps > 16 || (a.taps > 1 && !a.state))) return -1;
  if (a.rot < 0 || (a.rot & 1) || a.rot0 < 0 || a.rot0 + a.rot > a.gsize || (a.rot && !a.cossin)) return -1;
  if (a.norm_n < 0 || a.norm_n > a.gsize) return -1;
  if (!a.out_dense && (!a.pages || a.rowlen <= 0 || (a.ngroups * a.gsize) % a.rowlen || a.heads * a.rowlen != a.ngroups * a.gsize))
    return -1;
  const int64_t items = (int64_t)bt.T * a.ngroups;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((conv_head_kernel<T>), dim3((unsigned)((items + 3) / 4)), dim3(256),
                                            4 * a.gsize * sizeof(float), st, a, bt))
  return RAGGED_LAUNCH_OK();
}

// The convolution's state after a step: projected rows of positions past + n - (taps - 1) .. past + n - 1 (zeros before
// the sequence's start).  One thread per (sequence, channel) reads all it needs before it writes.
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ P, int64_t ldp, int col0, T* __restrict__ state,
                                                         int taps, int C, Batch bt) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)bt.B * C) return;
  const int b = (int)(id / C), ch = (int)(id % C);
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b], slot = bt.seq_slot[b];
  const int keep = taps - 1;
  T vals[15];
  for (int k = 0; k < keep; ++k) {
    const int pp = past + n - keep + k;
    T v = from_f<T>(0.f);
    if (pp >= past) v = P[(int64_t)(start + pp - past) * ldp + col0 + ch];
    else if (pp >= 0) v = state[((int64_t)slot * keep + (pp - past + keep)) * C + ch];
    vals[k] = v;
  }
  for (int k = 0; k < keep; ++k) state[((int64_t)slot * keep + k) * C + ch] = vals[k];
}

extern "C" int ragged_conv_state(const void* P, int64_t ldp, int col0, void* state, int taps, int C, Batch bt, int dtype,
                                 hipStream_t st) {
  if (bt.B <= 0 || C <= 0 || taps < 2 || taps > 16) return -1;
  const int64_t n = (int64_t)bt.B * C;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((conv_state_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                                            (const T*)P, ldp, col0, (T*)state, taps, C, bt))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Clamped gated unit: g = min(gate, limit), u = clamp(up, -limit, limit), y = g * sigmoid(slope * g) * (u + 1).
// GU holds [gate | up] per row.
template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ GU, T* __restrict__ out, int64_t rows, int F,
                                                          float limit, float slope) {
  const int64_t n = rows * F;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / F, c = i % F;
    float g = fminf(to_f(GU[r * 2 * F + c]), limit);
    float u = fminf(fmaxf(to_f(GU[r * 2 * F + F + c]), -limit), limit);
    out[i] = from_f<T>(g * sigmoidf_(slope * g) * (u + 1.0f));
  }
}

extern "C" int ragged_clamped_glu(const void* GU, void* out, int64_t rows, int F, float limit, float slope, int dtype,
                                  hipStream_t st) {
  if (rows <= 0 || F <= 0) return -1;
  const int64_t n = rows * F;
  const unsigned grid = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((clamped_glu_kernel<T>), dim3(grid), dim3(256), 0, st, (const T*)GU, (T*)out, rows, F,
                                            limit, slope))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// HGRN2.  Gates: q = silu(q_proj), f = lower + (1 - lower) * sigmoid(f_proj + bias), both float [T, HD].
template <typename T>
__global__ __launch_bounds__(256) void hgrn2_gates_kernel(const T* __restrict__ P, int64_t ldp, int q0, int f0,
                                                          const float* __restrict__ fb, const float* __restrict__ lower,
                                                          float* __restrict__ qf, float* __restrict__ ff, int64_t rows, int HD) {
  const int64_t n = rows * HD;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / HD;
    const int c = (int)(i % HD);
    const float q = to_f(P[r * ldp + q0 + c]);
    qf[i] = q * sigmoidf_(q);
    const float l = lower[c];
    ff[i] = l + (1.0f - l) * sigmoidf_(to_f(P[r * ldp + f0 + c]) + fb[c]);
  }
}

extern "C" int ragged_hgrn2_gates(const void* P, int64_t ldp, int q0, int f0, const float* fb, const float* lower, float* qf,
                                  float* ff, int64_t rows, int HD, int dtype, hipStream_t st) {
  if (rows <= 0 || HD <= 0) return -1;
  const int64_t n = rows * HD;
  const unsigned grid = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((hgrn2_gates_kernel<T>), dim3(grid), dim3(256), 0, st, (const T*)P, ldp, q0, f0, fb,
                                            lower, qf, ff, rows, HD))
  return RAGGED_LAUNCH_OK();
}

// Scan: per head S <- diag(f_t) S + (1 - f_t) v_t^T, o_t = S^T q_t, S float [d, vd] per (slot, head).
// A wavefront owns 64 / R columns of S; R neighbouring lanes share a column, lane r of them holds rows 32 r .. 32 r + 31
// in registers (R = d / 32 rounded up to a power of two; rows past d carry q = 0, f = 1 and stay zero), so the only
// cross-lane step of a token is the sum of R partial dot products (DPP moves).  A workgroup is four such wavefronts.
// Gates and queries of a block of TB tokens are brought into LDS by the whole workgroup with coalesced loads while the
// previous block is being scanned (register look-ahead, two LDS buffers); a step reads its 32 gates and 32 queries
// back as 16-byte broadcasts with no condition around them, so all reads of a step are in flight together.
// Grid: (column blocks, heads, sequences).
constexpr int HG_DR = 32;
constexpr int HG_SEG = HG_DR + 4;   // LDS floats per lane group and token (padding shifts the banks between groups)
constexpr int HG_TBR = 64;          // TB * R <= this
// pvd: value columns per head in P.  pvd = vd - 1: the state's last column takes a constant 1 as its value, so that it
// carries n <- f n + g and the output's last column is n . q (the normaliser of an mLSTM head).
// GIN: the input's weights come from a third array, S <- diag(f_t) S + g_t v_t^T (mLSTM hands in f = its decay
// repeated over the rows and g = its input gate times the key); otherwise g = 1 - f.
template <typename T, bool GIN>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(const float* __restrict__ qf, const float* __restrict__ ff,
                                                         const float* __restrict__ gf,
                                                         const T* __restrict__ P, int64_t ldp, int v0, float* __restrict__ state,
                                                         float* __restrict__ out, int H, int d, int vd, int pvd, int R, int TB, Batch bt) {
  constexpr int NA = GIN ? 3 : 2;
  constexpr int HG_PRE = NA * HG_TBR * HG_DR / 256;
  extern __shared__ __attribute__((aligned(16))) float smem[];   // 2 x { q[TB][R][SEG], f[TB][R][SEG], (g,) v[TB][wcols] }
  const int b = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int cols = 64 / R, wcols = 4 * cols;
  const int r = lane % R, lc = wave * cols + lane / R;     // column inside the workgroup's block
  const int col = blockIdx.x * wcols + lc;
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b], slot = bt.seq_slot[b];
  const bool colok = col < vd;
  const int row0 = r * HG_DR;
  const int HD = H * d;
  const int qsz = TB * R * HG_SEG;                         // floats of q (and of f) in a buffer
  const int bufsz = NA * qsz + TB * wcols;
  float S[HG_DR];
  float* sp = state + (((int64_t)slot * H + h) * d) * vd;
  {
    const int cc = colok ? col : vd - 1;
#pragma unroll
    for (int k = 0; k < HG_DR; ++k) {
      const int row = row0 + k;
      const float v = sp[(int64_t)(row < d ? row : d - 1) * vd + cc];    // no condition around the load
      S[k] = (past > 0 && colok && row < d) ? v : 0.f;
    }
  }
  float pre[HG_PRE], prev[4];
  const int nel = TB * R * HG_DR;                          // q (or f) elements of a block, padded rows included
  auto fetch = [&](int i0) {                               // block of tokens i0 .. i0 + TB - 1 into registers
#pragma unroll
    for (int u = 0; u < HG_PRE; ++u) {
      const int e = tid + 256 * u;
      const int which = e / nel, rem = e - which * nel;
      const int tk = rem / (R * HG_DR), row = rem % (R * HG_DR);
      float v = which == 1 ? 1.f : 0.f;                    // padding: f = 1, q = 0, g = 0
      if (e < NA * nel && row < d && i0 + tk < n)
        v = (which == 0 ? qf : which == 1 ? ff : gf)[(int64_t)(start + i0 + tk) * HD + h * d + row];
      pre[u] = v;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + 256 * u;
      float v = 0.f;
      if (e < TB * wcols) {
        const int tk = e / wcols, c = blockIdx.x * wcols + e % wcols;
        if (i0 + tk < n && c < vd) v = c < pvd ? to_f(P[(int64_t)(start + i0 + tk) * ldp + v0 + h * pvd + c]) : 1.f;
      }
      prev[u] = v;
    }
  };
  auto stash = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < HG_PRE; ++u) {
      const int e = tid + 256 * u;
      if (e < NA * nel) {
        const int which = e / nel, rem = e - which * nel;
        const int tk = rem / (R * HG_DR), row = rem % (R * HG_DR);
        buf[which * qsz + (tk * R + row / HG_DR) * HG_SEG + row % HG_DR] = pre[u];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + 256 * u;
      if (e < TB * wcols) buf[NA * qsz + e] = prev[u];
    }
  };
  if (n > 0) { fetch(0); stash(smem); }
  __syncthreads();
  int cur = 0;
  for (int i0 = 0; i0 < n; i0 += TB) {
    const bool more = i0 + TB < n;
    if (more) fetch(i0 + TB);
    const float* buf = smem + cur * bufsz;
    const int nt = n - i0 < TB ? n - i0 : TB;
    for (int tk = 0; tk < nt; ++tk) {
      const float4* q4 = reinterpret_cast<const float4*>(buf + (tk * R + r) * HG_SEG);
      const float4* f4 = reinterpret_cast<const float4*>(buf + qsz + (tk * R + r) * HG_SEG);
      const float4* g4 = reinterpret_cast<const float4*>(buf + (NA - 1) * qsz + (tk * R + r) * HG_SEG);
      float qv[HG_DR], fv[HG_DR], gv[HG_DR];
#pragma unroll
      for (int k = 0; k < HG_DR / 4; ++k) {
        const float4 a = q4[k], c = f4[k];
        qv[4 * k] = a.x; qv[4 * k + 1] = a.y; qv[4 * k + 2] = a.z; qv[4 * k + 3] = a.w;
        fv[4 * k] = c.x; fv[4 * k + 1] = c.y; fv[4 * k + 2] = c.z; fv[4 * k + 3] = c.w;
        if (GIN) {
          const float4 e = g4[k];
          gv[4 * k] = e.x; gv[4 * k + 1] = e.y; gv[4 * k + 2] = e.z; gv[4 * k + 3] = e.w;
        } else {
          gv[4 * k] = 1.0f - c.x; gv[4 * k + 1] = 1.0f - c.y; gv[4 * k + 2] = 1.0f - c.z; gv[4 * k + 3] = 1.0f - c.w;
        }
      }
      const float v = buf[NA * qsz + tk * wcols + lc];
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < HG_DR; ++k) {
        S[k] = fv[k] * S[k] + gv[k] * v;
        acc[k & 3] += S[k] * qv[k];
      }
      const float tot = group_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), R);
      if (r == 0 && colok) out[(int64_t)(start + i0 + tk) * (H * vd) + h * vd + col] = tot;
    }
    if (more) stash(smem + (cur ^ 1) * bufsz);
    __syncthreads();
    cur ^= 1;
  }
#pragma unroll
  for (int k = 0; k < HG_DR; ++k) {
    const int row = row0 + k;
    if (colok && row < d) sp[(int64_t)row * vd + col] = S[k];
  }
}

// gf null: the input's weight is 1 - f (HGRN2); otherwise the third gate array
extern "C" int ragged_hgrn2_scan(const float* qf, const float* ff, const float* gf, const void* P, int64_t ldp, int v0,
                                 float* state, float* out, int H, int d, int vd, int ones_col, Batch bt, int dtype,
                                 hipStream_t st) {
  if (bt.B <= 0 || H <= 0 || d <= 0 || vd <= (ones_col ? 1 : 0) || d > HG_DR * 64) return -1;
  const int pvd = ones_col ? vd - 1 : vd;
  int R = 1;
  while (R * HG_DR < d) R <<= 1;
  const int wcols = 4 * (64 / R);
  int TB = HG_TBR / R < 16 ? HG_TBR / R : 16;
  if (TB * wcols > 4 * 256) TB = 4 * 256 / wcols;           // the value look-ahead holds 4 floats per thread
  const int na = gf ? 3 : 2;
  const size_t sm = 2 * (size_t)(na * TB * R * HG_SEG + TB * wcols) * sizeof(float);
  const dim3 grid((vd + wcols - 1) / wcols, H, bt.B);
  RAGGED_DISPATCH(dtype,
    if (gf) hipLaunchKernelGGL((hgrn2_scan_kernel<T, true>), grid, dim3(256), sm, st, qf, ff, gf, (const T*)P, ldp, v0, state, out,
                               H, d, vd, pvd, R, TB, bt);
    else hipLaunchKernelGGL((hgrn2_scan_kernel<T, false>), grid, dim3(256), sm, st, qf, ff, gf, (const T*)P, ldp, v0, state, out,
                            H, d, vd, pvd, R, TB, bt))
  return RAGGED_LAUNCH_OK();
}

// Long portions: the scan is cut into chunks that run side by side.  Every chunk is scanned from a zero state (its
// local end state L_c), the product D_c of its gates is taken per row, the true state at every chunk's start follows
// from S_(c+1) = diag(D_c) S_c + L_c, and the chunks are scanned again from those states for the outputs.  Nothing is
// divided, so small gate products only fade a contribution out.  The scans are hgrn2_scan_kernel over a batch whose
// "sequences" are the chunks and whose "slots" are rows of a scratch state array.
__global__ __launch_bounds__(256) void hgrn2_chunk_decay_kernel(const float* __restrict__ ff, const int* __restrict__ cstart,
                                                                float* __restrict__ decay, int HD) {
  const int c = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
  if (ch >= HD) return;
  float p = 1.f;
  for (int t = cstart[c]; t < cstart[c + 1]; ++t) p *= ff[(int64_t)t * HD + ch];
  decay[(int64_t)c * HD + ch] = p;
}

// one thread per state element of a real sequence; cfirst[b] .. cfirst[b + 1] - 1 are its chunks
__global__ __launch_bounds__(256) void hgrn2_chunk_combine_kernel(const float* __restrict__ state, const float* __restrict__ local,
                                                                  const float* __restrict__ decay, float* __restrict__ begin,
                                                                  const int* __restrict__ cfirst, const int* __restrict__ seq_past,
                                                                  const int* __restrict__ seq_slot, int H, int d, int vd) {
  const int b = blockIdx.y;
  const int64_t E = (int64_t)H * d * vd, e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= E) return;
  const int hrow = (int)(e / vd);                          // h * d + row
  float S = seq_past[b] > 0 ? state[(int64_t)seq_slot[b] * E + e] : 0.f;
  for (int c = cfirst[b]; c < cfirst[b + 1]; ++c) {
    begin[(int64_t)c * E + e] = S;
    S = decay[(int64_t)c * H * d + hrow] * S + local[(int64_t)c * E + e];
  }
}

extern "C" int ragged_hgrn2_chunk_decay(const float* ff, const int* cstart, float* decay, int n_chunks, int HD, hipStream_t st) {
  if (n_chunks <= 0 || HD <= 0) return -1;
  hipLaunchKernelGGL(hgrn2_chunk_decay_kernel, dim3(n_chunks, (HD + 255) / 256), dim3(256), 0, st, ff, cstart, decay, HD);
  return RAGGED_LAUNCH_OK();
}

extern "C" int ragged_hgrn2_chunk_combine(const float* state, const float* local, const float* decay, float* begin,
                                          const int* cfirst, const int* seq_past, const int* seq_slot, int B, int H, int d, int vd,
                                          hipStream_t st) {
  if (B <= 0 || H <= 0 || d <= 0 || vd <= 0) return -1;
  const int64_t E = (int64_t)H * d * vd;
  hipLaunchKernelGGL(hgrn2_chunk_combine_kernel, dim3((unsigned)((E + 255) / 256), B), dim3(256), 0, st, state, local, decay, begin,
                     cfirst, seq_past, seq_slot, H, d, vd);
  return RAGGED_LAUNCH_OK();
}

// RMS norm over rows of `n` floats with a weight (or none), output of type T.  One wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void row_norm_kernel(const float* __restrict__ x, const float* __restrict__ w, T* __restrict__ out,
                                                       int64_t rows, int n, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  float ss = 0.f;
  for (int c = lane; c < n; c += 64) { const float v = x[row * n + c]; ss += v * v; }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)n + eps);
  for (int c = lane; c < n; c += 64) out[row * n + c] = from_f<T>(x[row * n + c] * r * (w ? w[c] : 1.0f));
}

extern "C" int ragged_row_norm(const float* x, const float* w, void* out, int64_t rows, int n, float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || n <= 0) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((row_norm_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, x, w, (T*)out,
                                            rows, n, eps))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Embedding rows as the float stream: x[t] = scale * table[ids[t]] (+ table2[ids2[t]]), summed in float.  The second
// table serves embeddings of token pairs (a row chosen by a hash of the previous and the current token).
template <typename T>
__global__ __launch_bounds__(256) void embed_rows_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                         const int64_t* __restrict__ ids2, const T* __restrict__ table2,
                                                         float scale, float* __restrict__ x, int D) {
  const int64_t t = blockIdx.x;
  const T* r1 = table + ids[t] * D;
  const T* r2 = table2 ? table2 + ids2[t] * D : nullptr;
  for (int c = threadIdx.x; c < D; c += 256) {
    float v = to_f(r1[c]) * scale;
    if (r2) v += to_f(r2[c]);
    x[t * D + c] = v;
  }
}

extern "C" int ragged_embed_rows(const int64_t* ids, const void* table, const int64_t* ids2, const void* table2, float scale,
                                 float* x, int64_t rows, int D, int dtype, hipStream_t st) {
  if (rows <= 0 || rows > 0x7fffffff || D <= 0 || !ids || !table || !x || (table2 && !ids2)) return -1;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((embed_rows_kernel<T>), dim3((unsigned)rows), dim3(256), 0, st, ids, (const T*)table, ids2,
                                            (const T*)table2, scale, x, D))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Pre-norm form: x <- x + y1 (+ y2) on the float stream, then (w_next given) xa = w_next * rmsnorm(x) for the products
// that read the stream next.  y2 serves blocks whose mixer and feed-forward read the same normed input and are summed
// into the stream together.  One workgroup per row; NV as in post_norm_add_kernel.
template <typename T, int NV>
__global__ __launch_bounds__(256) void add_norm_kernel(float* __restrict__ x, const T* __restrict__ y1, const T* __restrict__ y2,
                                                       const float* __restrict__ w_next, T* __restrict__ xa, int D, float eps) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * D;
  if (NV > 0) {
    float xv[NV > 0 ? NV : 1], wn[NV > 0 ? NV : 1];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int c = threadIdx.x + 256 * u;
      const bool ok = c < D;
      float v = ok ? x[base + c] : 0.f;
      float s = (ok && y1) ? to_f(y1[base + c]) : 0.f;
      if (ok && y2) s += to_f(y2[base + c]);
      v += s;
      wn[u] = (ok && xa) ? w_next[c] : 0.f;
      if (ok && (y1 || y2)) x[base + c] = v;
      xv[u] = v;
      ss += v * v;
    }
    if (!xa) return;
    const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int c = threadIdx.x + 256 * u;
      if (c < D) xa[base + c] = from_f<T>(xv[u] * r * wn[u]);
    }
    return;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < D; c += 256) {
    float s = y1 ? to_f(y1[base + c]) : 0.f;
    if (y2) s += to_f(y2[base + c]);
    const float v = x[base + c] + s;
    if (y1 || y2) x[base + c] = v;
    ss += v * v;
  }
  if (!xa) return;
  const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
  for (int c = threadIdx.x; c < D; c += 256) xa[base + c] = from_f<T>(x[base + c] * r * w_next[c]);
}

extern "C" int ragged_add_norm(float* x, const void* y1, const void* y2, const float* w_next, void* xa, int64_t rows, int D,
                               float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || D <= 0 || rows > 0x7fffffff || !x || (xa && !w_next) || (y2 && !y1)) return -1;
  RAGGED_DISPATCH(dtype,
    if (D <= 1024) hipLaunchKernelGGL((add_norm_kernel<T, 4>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y1, (const T*)y2,
                                      w_next, (T*)xa, D, eps);
    else if (D <= 4096) hipLaunchKernelGGL((add_norm_kernel<T, 16>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y1,
                                           (const T*)y2, w_next, (T*)xa, D, eps);
    else hipLaunchKernelGGL((add_norm_kernel<T, 0>), dim3((unsigned)rows), dim3(256), 0, st, x, (const T*)y1, (const T*)y2, w_next,
                            (T*)xa, D, eps))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Activations of a feed-forward's inner channels.  act_cols: out[r, c] = act(P[r, col0 + c]), c < n, with
// kind 0: gelu through erf, 0.5 z (1 + erf(z / sqrt 2));  1: gelu through tanh, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)));
// 2: relu(z)^2;  3: a unit with two curvatures (p0, p1 >= 0 are handed in): p0 z^2 + z / 2 right of zero,
// (1/2 + p1) (e^z - 1 - z) + z / 2 left of it (both branches and their slopes meet at 0);  4: tanh(z).
// glu_pairs: the inner channels come as neighbouring (gate, up) pairs, out[r, c] = silu(P[r, 2 c]) * P[r, 2 c + 1].
__device__ __forceinline__ float act_value(float z, int kind, float p0, float p1) {
  if (kind == 3) return z > 0.f ? p0 * z * z + 0.5f * z : (0.5f + p1) * (expm1f(z) - z) + 0.5f * z;
  if (kind == 4) return tanhf(z);
  if (kind == 0) return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
  if (kind == 1) return 0.5f * z * (1.0f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
  const float v = fmaxf(z, 0.f);
  return v * v;
}

// grid (blocks of 256 pieces of a row, rows); VEC: a thread takes 16 bytes of a row (rows and the first column are
// 16-byte aligned, n a multiple of the piece), otherwise one element
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void act_cols_kernel(const T* __restrict__ P, int64_t ldp, int col0, T* __restrict__ out, int n,
                                                       int kind, float p0, float p1) {
  constexpr int N = VEC ? 16 / (int)sizeof(T) : 1;
  const int64_t r = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * N;
  if (c >= n) return;
  const T* src = P + r * ldp + col0 + c;
  T* dst = out + r * n + c;
  if (VEC) {
    union { uint4 q; T e[N]; } v;
    v.q = *reinterpret_cast<const uint4*>(src);
#pragma unroll
    for (int i = 0; i < N; ++i) v.e[i] = from_f<T>(act_value(to_f(v.e[i]), kind, p0, p1));
    *reinterpret_cast<uint4*>(dst) = v.q;
  } else {
    dst[0] = from_f<T>(act_value(to_f(src[0]), kind, p0, p1));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void glu_pairs_kernel(const T* __restrict__ P, int64_t ldp, T* __restrict__ out, int64_t rows, int n) {
  const int64_t total = rows * n;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / n;
    const int c = (int)(i % n);
    const float g = to_f(P[r * ldp + 2 * c]), u = to_f(P[r * ldp + 2 * c + 1]);
    out[i] = from_f<T>(g / (1.0f + expf(-g)) * u);
  }
}

extern "C" int ragged_act_cols(const void* P, int64_t ldp, int col0, void* out, int64_t rows, int n, int kind, float p0, float p1,
                               int dtype, hipStream_t st) {
  if (rows <= 0 || rows > 65535LL * 65535LL || n <= 0 || col0 < 0 || ldp < col0 + n || kind < 0 || kind > 4) return -1;
  RAGGED_DISPATCH(dtype,
    constexpr int N = 16 / (int)sizeof(T);
    const bool vec = n % N == 0 && ldp % N == 0 && col0 % N == 0 && ((uintptr_t)P % 16) == 0 && ((uintptr_t)out % 16) == 0;
    // (the grid's second dimension holds at most 65535 rows: more rows go in several launches)
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
      const unsigned nr = (unsigned)(rows - r0 < 65535 ? rows - r0 : 65535);
      const T* src = (const T*)P + r0 * ldp;
      T* dst = (T*)out + r0 * n;
      if (vec) hipLaunchKernelGGL((act_cols_kernel<T, true>), dim3((n / N + 255) / 256, nr), dim3(256), 0, st, src, ldp, col0, dst, n, kind,
                                  p0, p1);
      else hipLaunchKernelGGL((act_cols_kernel<T, false>), dim3((n + 255) / 256, nr), dim3(256), 0, st, src, ldp, col0, dst, n, kind, p0, p1);
    })
  return RAGGED_LAUNCH_OK();
}

extern "C" int ragged_glu_pairs(const void* P, int64_t ldp, void* out, int64_t rows, int n, int dtype, hipStream_t st) {
  if (rows <= 0 || n <= 0 || ldp < 2 * n) return -1;
  const int64_t blocks = (rows * n + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 16384 ? blocks : 16384);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((glu_pairs_kernel<T>), dim3(grid), dim3(256), 0, st, (const T*)P, ldp, (T*)out, rows, n))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Pre-norm blocks over a stream that is kept in S copies X[row][s][D] (S = 1: the ordinary residual stream).  One call
// sits between two sublayers:
//   y given:    X'[t] = sum_s mix[s][t] X[s] + out[t] * y      for all t from the old copies (prev = [in | out | mix])
//   nin given:  u = sum_s nin[s] X'[s];  u_out <- u (float);  xa <- w_next * u / sqrt(mean(u^2) + eps)
// so the write-back of one sublayer, the read-out of the next and its norm pass over a row once.  One workgroup per row.
// NV > 0: rows of at most 256 NV channels, u stays in registers; NV = 0: any width, u is made again for the second pass.
constexpr int HC_MAX = 8;

// SS: the number of copies as a compile-time constant (1 .. 4), or HC_MAX for any S up to that many (loops of HC_MAX
// steps with the steps past S switched off): either way the copies of a channel and the coefficients live in registers.
template <typename T, int NV, int SS>
__global__ __launch_bounds__(256) void hc_step_kernel(float* __restrict__ X, const T* __restrict__ y, const float* __restrict__ prev,
                                                      const float* __restrict__ nin, const float* __restrict__ w_next,
                                                      T* __restrict__ xa, float* __restrict__ u_out, int S, int D, float eps) {
  __shared__ float red[4];
  float cin[SS], cout[SS], cmix[SS][SS];                   // cmix[from][to]
#pragma unroll
  for (int s = 0; s < SS; ++s) {
    const bool ok = s < S;
    cin[s] = (nin && ok) ? nin[s] : 0.f;
    cout[s] = (y && ok) ? prev[S + s] : 0.f;
#pragma unroll
    for (int t = 0; t < SS; ++t) cmix[s][t] = (y && ok && t < S) ? prev[2 * S + s * S + t] : 0.f;
  }
  const int64_t row = blockIdx.x;
  float* xr = X + row * S * D;
  // the copies of one channel: update from the old values, return what the next sublayer reads
  auto channel = [&](int c) {
    float old[SS], u = 0.f;
#pragma unroll
    for (int s = 0; s < SS; ++s) old[s] = s < S ? xr[(int64_t)s * D + c] : 0.f;
    if (y) {
      const float yv = to_f(y[row * D + c]);
#pragma unroll
      for (int t = 0; t < SS; ++t) {
        float v = cout[t] * yv;
#pragma unroll
        for (int s = 0; s < SS; ++s) v += cmix[s][t] * old[s];
        if (t < S) xr[(int64_t)t * D + c] = v;
        u += cin[t] * v;
      }
    } else {
#pragma unroll
      for (int s = 0; s < SS; ++s) u += cin[s] * old[s];
    }
    return u;
  };
  if (NV > 0) {
    float uv[NV > 0 ? NV : 1], ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int c = threadIdx.x + 256 * k;
      uv[k] = c < D ? channel(c) : 0.f;
      ss += uv[k] * uv[k];
      if (u_out && c < D) u_out[row * D + c] = uv[k];
    }
    if (!xa) return;
    const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int c = threadIdx.x + 256 * k;
      if (c < D) xa[row * D + c] = from_f<T>(uv[k] * r * w_next[c]);
    }
    return;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < D; c += 256) {
    const float u = channel(c);
    ss += u * u;
    if (u_out) u_out[row * D + c] = u;
  }
  if (!xa) return;
  const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)D + eps);
  for (int c = threadIdx.x; c < D; c += 256) {       // (each thread re-reads the copies it has written itself)
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < SS; ++s) u += s < S ? cin[s] * xr[(int64_t)s * D + c] : 0.f;
    xa[row * D + c] = from_f<T>(u * r * w_next[c]);
  }
}

template <typename T, int SS>
static void launch_hc(float* X, const void* y, const float* prev, const float* nin, const float* w_next, void* xa, float* u_out,
                      int64_t rows, int S, int D, float eps, hipStream_t st) {
  if (D <= 1024) hipLaunchKernelGGL((hc_step_kernel<T, 4, SS>), dim3((unsigned)rows), dim3(256), 0, st, X, (const T*)y, prev, nin,
                                    w_next, (T*)xa, u_out, S, D, eps);
  else if (D <= 4096 && SS <= 4) hipLaunchKernelGGL((hc_step_kernel<T, 16, SS>), dim3((unsigned)rows), dim3(256), 0, st, X, (const T*)y,
                                                    prev, nin, w_next, (T*)xa, u_out, S, D, eps);
  else hipLaunchKernelGGL((hc_step_kernel<T, 0, SS>), dim3((unsigned)rows), dim3(256), 0, st, X, (const T*)y, prev, nin, w_next,
                          (T*)xa, u_out, S, D, eps);
}

extern "C" int ragged_hc_step(float* X, const void* y, const float* prev, const float* nin, const float* w_next, void* xa,
                              float* u_out, int64_t rows, int S, int D, float eps, int dtype, hipStream_t st) {
  if (rows <= 0 || rows > 0x7fffffff || D <= 0 || S <= 0 || S > HC_MAX || !X || (y && !prev) || (xa && (!w_next || !nin)) ||
      (u_out && !nin)) return -1;
  RAGGED_DISPATCH(dtype,
    if (S == 1) launch_hc<T, 1>(X, y, prev, nin, w_next, xa, u_out, rows, S, D, eps, st);
    else if (S == 2) launch_hc<T, 2>(X, y, prev, nin, w_next, xa, u_out, rows, S, D, eps, st);
    else if (S == 3) launch_hc<T, 3>(X, y, prev, nin, w_next, xa, u_out, rows, S, D, eps, st);
    else if (S == 4) launch_hc<T, 4>(X, y, prev, nin, w_next, xa, u_out, rows, S, D, eps, st);
    else launch_hc<T, HC_MAX>(X, y, prev, nin, w_next, xa, u_out, rows, S, D, eps, st))
  return RAGGED_LAUNCH_OK();
}

// out[r, c] = scale * o[r, c] * sigmoid(P[r, g0 + c]), c < n: a gate per channel on float head outputs, rounded once
template <typename T>
__global__ __launch_bounds__(256) void gate_cols_kernel(const float* __restrict__ o, const T* __restrict__ P, int64_t ldp, int g0,
                                                        T* __restrict__ out, int64_t rows, int n, float scale) {
  const int64_t total = rows * n;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / n;
    const int c = (int)(i % n);
    out[i] = from_f<T>(scale * o[i] * sigmoidf_(to_f(P[r * ldp + g0 + c])));
  }
}

extern "C" int ragged_gate_cols(const float* o, const void* P, int64_t ldp, int g0, void* out, int64_t rows, int n, float scale,
                                int dtype, hipStream_t st) {
  if (rows <= 0 || n <= 0 || g0 < 0 || ldp < g0 + n) return -1;
  const int64_t blocks = (rows * n + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 16384 ? blocks : 16384);
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((gate_cols_kernel<T>), dim3(grid), dim3(256), 0, st, o, (const T*)P, ldp, g0, (T*)out, rows,
                                            n, scale))
  return RAGGED_LAUNCH_OK();
}
