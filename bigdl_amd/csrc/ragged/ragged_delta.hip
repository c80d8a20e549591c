// Generalised delta rule of the ragged engine: a matrix state per head that decays per key channel, forgets along the
// direction of the unit key and then takes the new key / value pair,
//     S_t = diag(w_t) S_(t-1) - (a_t * n_t) (n_t^T S_(t-1)) + k_t v_t^T,     o_t = S_t^T r_t,     n = k / sqrt(|k|^2 + tiny)
// with both terms reading the old state.  S float [d, vd] per (slot, head).  Everything but the projections themselves
// (decay, removal rate, unit key, state, outputs) is float whatever the activation type T is.
#include "ragged_common.h"

using namespace ragged;

// ---------------------------------------------------------------------------------------------------------------
// The scan's five arrays from this step's projections, float [rows, H d] each:
//   rf = r,  wf = exp(-rate * sigmoid(decay logits + w0)),  nf = n,  bf = sigmoid(a logits + ab) * n,  kf = k
// r, k and the a logits are columns of P (type T); the decay logits come from a second small product and are float.
// One wavefront per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void delta_gates_kernel(const T* __restrict__ P, int64_t ldp, int r0, int k0, int a0,
                                                          const float* __restrict__ wl, const float* __restrict__ w0,
                                                          const float* __restrict__ ab, float rate, float tiny,
                                                          float* __restrict__ rf, float* __restrict__ wf, float* __restrict__ nf,
                                                          float* __restrict__ bf, float* __restrict__ kf, int64_t items, int H, int d) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (item >= items) return;
  const int64_t t = item / H;
  const int h = (int)(item % H);
  const T* row = P + t * ldp;
  float ss = 0.f;
  for (int c = lane; c < d; c += 64) { const float k = to_f(row[k0 + h * d + c]); ss += k * k; }
  const float inv = 1.0f / sqrtf(wave_sum(ss) + tiny);
  for (int c = lane; c < d; c += 64) {
    const int ch = h * d + c;
    const int64_t o = t * (int64_t)(H * d) + ch;
    const float k = to_f(row[k0 + ch]), n = k * inv;
    const float sw = 1.0f / (1.0f + expf(-(wl[o] + w0[ch])));
    const float sa = 1.0f / (1.0f + expf(-(to_f(row[a0 + ch]) + ab[ch])));
    rf[o] = to_f(row[r0 + ch]);
    wf[o] = expf(-rate * sw);
    nf[o] = n;
    bf[o] = sa * n;
    kf[o] = k;
  }
}

extern "C" int ragged_delta_gates(const void* P, int64_t ldp, int r0, int k0, int a0, const float* wl, const float* w0,
                                  const float* ab, float rate, float tiny, float* rf, float* wf, float* nf, float* bf, float* kf,
                                  int64_t rows, int H, int d, int dtype, hipStream_t st) {
  if (rows <= 0 || H <= 0 || d <= 0 || rows * H > 0x7fffffff || r0 < 0 || k0 < 0 || a0 < 0) return -1;
  const int64_t items = rows * H;
  RAGGED_DISPATCH(dtype, hipLaunchKernelGGL((delta_gates_kernel<T>), dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, (const T*)P,
                                            ldp, r0, k0, a0, wl, w0, ab, rate, tiny, rf, wf, nf, bf, kf, items, H, d))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// The scan.  Columns of S are independent: column j follows s <- w * s - b (n . s) + k v_j, and its output is r . s.
// A wavefront owns 64 / R columns; R neighbouring lanes share a column, lane r of them holds rows 32 r .. 32 r + 31 in
// registers (R = d / 32 rounded up to a power of two; rows past d carry w = 1 and zeros and stay zero), so a token costs
// two cross-lane sums of R partial products (DPP moves): n . s before the update, r . s after it.  A workgroup is NW such
// wavefronts (as many as the state has columns for, at most four: a wavefront without columns would still read all five
// arrays).  The five arrays of a block of TB tokens are brought into LDS by the whole workgroup with coalesced loads
// while the previous block is scanned (register look-ahead, two LDS buffers) and read back as 16-byte broadcasts.
// Grid: (column blocks, heads, sequences).  `values` = 0: v is taken as 0 (the state only decays and forgets: from an
// identity state this yields a chunk's transition matrix).
constexpr int DL_DR = 32;
constexpr int DL_SEG = DL_DR + 4;   // LDS floats per lane group and token (padding shifts the banks between groups)
constexpr int DL_TBR = 32;          // TB * R <= this
constexpr int DL_NA = 5;

template <typename T, int NW>
__global__ __launch_bounds__(64 * NW) void delta_scan_kernel(const float* __restrict__ rf, const float* __restrict__ wf,
                                                         const float* __restrict__ nf, const float* __restrict__ bf,
                                                         const float* __restrict__ kf, const T* __restrict__ P, int64_t ldp, int v0,
                                                         float* __restrict__ state, float* __restrict__ out, int H, int d, int vd,
                                                         int R, int TB, int values, Batch bt) {
  constexpr int NT = 64 * NW, DL_PRE = DL_NA * DL_TBR * DL_DR / NT;
  extern __shared__ __attribute__((aligned(16))) float smem[];   // 2 x { r, w, n, b, k: [TB][R][SEG] each, v[TB][wcols] }
  const int b = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int cols = 64 / R, wcols = NW * cols;
  const int r = lane % R, lc = wave * cols + lane / R;     // column inside the workgroup's block
  const int col = blockIdx.x * wcols + lc;
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b], slot = bt.seq_slot[b];
  const bool colok = col < vd;
  const int row0 = r * DL_DR;
  const int HD = H * d;
  const int qsz = TB * R * DL_SEG;                         // floats of one array in a buffer
  const int bufsz = DL_NA * qsz + TB * wcols;
  float S[DL_DR];
  float* sp = state + (((int64_t)slot * H + h) * d) * vd;
  {
    const int cc = colok ? col : vd - 1;
#pragma unroll
    for (int k = 0; k < DL_DR; ++k) {
      const int row = row0 + k;
      const float v = sp[(int64_t)(row < d ? row : d - 1) * vd + cc];    // no condition around the load
      S[k] = (past > 0 && colok && row < d) ? v : 0.f;
    }
  }
  float pre[DL_PRE], prev[4];
  // element e of a block = (token tk, array, row): tokens are the slowest index, so a block of few tokens (a single
  // decoded one) ends the loops early; R * 32 is a power of two (lr = its logarithm) and 5 a constant, so no step divides
  const int lr = 31 - __clz(R * DL_DR), rows = R * DL_DR;
  auto fetch = [&](int i0) {                               // block of tokens i0 .. i0 + TB - 1 into registers
    const int live = (n - i0 < TB ? n - i0 : TB) * DL_NA * rows;
#pragma unroll
    for (int u = 0; u < DL_PRE; ++u) {
      if (NT * u >= live) break;
      const int e = tid + NT * u;
      const int ta = e >> lr, row = e & (rows - 1);
      const int tk = ta / DL_NA, which = ta - tk * DL_NA;
      float v = which == 1 ? 1.f : 0.f;                    // padding: w = 1, everything else 0
      if (e < live && row < d) {
        const float* src = which == 0 ? rf : which == 1 ? wf : which == 2 ? nf : which == 3 ? bf : kf;
        v = src[(int64_t)(start + i0 + tk) * HD + h * d + row];
      }
      pre[u] = v;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + NT * u;
      float v = 0.f;
      if (e < TB * wcols && values) {
        const int tk = e / wcols, c = blockIdx.x * wcols + e % wcols;
        if (i0 + tk < n && c < vd) v = to_f(P[(int64_t)(start + i0 + tk) * ldp + v0 + h * vd + c]);
      }
      prev[u] = v;
    }
  };
  auto stash = [&](float* buf, int i0) {
    const int live = (n - i0 < TB ? n - i0 : TB) * DL_NA * rows;
#pragma unroll
    for (int u = 0; u < DL_PRE; ++u) {
      if (NT * u >= live) break;
      const int e = tid + NT * u;
      if (e < live) {
        const int ta = e >> lr, row = e & (rows - 1);
        const int tk = ta / DL_NA, which = ta - tk * DL_NA;
        buf[which * qsz + (tk * R + (row >> 5)) * DL_SEG + (row & 31)] = pre[u];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + NT * u;
      if (e < TB * wcols) buf[DL_NA * qsz + e] = prev[u];
    }
  };
  if (n > 0) { fetch(0); stash(smem, 0); }
  __syncthreads();
  int cur = 0;
  for (int i0 = 0; i0 < n; i0 += TB) {
    const bool more = i0 + TB < n;
    if (more) fetch(i0 + TB);
    const float* buf = smem + cur * bufsz;
    const int nt = n - i0 < TB ? n - i0 : TB;
    for (int tk = 0; tk < nt; ++tk) {
      const int seg = (tk * R + r) * DL_SEG;
      const float4* r4 = reinterpret_cast<const float4*>(buf + seg);
      const float4* w4 = reinterpret_cast<const float4*>(buf + qsz + seg);
      const float4* n4 = reinterpret_cast<const float4*>(buf + 2 * qsz + seg);
      const float4* b4 = reinterpret_cast<const float4*>(buf + 3 * qsz + seg);
      const float4* k4 = reinterpret_cast<const float4*>(buf + 4 * qsz + seg);
      const float v = buf[DL_NA * qsz + tk * wcols + lc];
      // n . s over the old state
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < DL_DR / 4; ++k) {
        const float4 a = n4[k];
        acc[0] += S[4 * k] * a.x; acc[1] += S[4 * k + 1] * a.y; acc[2] += S[4 * k + 2] * a.z; acc[3] += S[4 * k + 3] * a.w;
      }
      const float dot = group_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), R);
      acc[0] = acc[1] = acc[2] = acc[3] = 0.f;
#pragma unroll
      for (int k = 0; k < DL_DR / 4; ++k) {
        const float4 w = w4[k], bb = b4[k], kk = k4[k], q = r4[k];
        S[4 * k] = w.x * S[4 * k] - bb.x * dot + kk.x * v;
        S[4 * k + 1] = w.y * S[4 * k + 1] - bb.y * dot + kk.y * v;
        S[4 * k + 2] = w.z * S[4 * k + 2] - bb.z * dot + kk.z * v;
        S[4 * k + 3] = w.w * S[4 * k + 3] - bb.w * dot + kk.w * v;
        acc[0] += S[4 * k] * q.x; acc[1] += S[4 * k + 1] * q.y; acc[2] += S[4 * k + 2] * q.z; acc[3] += S[4 * k + 3] * q.w;
      }
      const float tot = group_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), R);
      if (out && r == 0 && colok) out[(int64_t)(start + i0 + tk) * (H * vd) + h * vd + col] = tot;
    }
    if (more) stash(smem + (cur ^ 1) * bufsz, i0 + TB);
    __syncthreads();
    cur ^= 1;
  }
#pragma unroll
  for (int k = 0; k < DL_DR; ++k) {
    const int row = row0 + k;
    if (colok && row < d) sp[(int64_t)row * vd + col] = S[k];
  }
}

// out may be null (only the end states are wanted); values = 0: the value columns of P are not read and count as 0
extern "C" int ragged_delta_scan(const float* rf, const float* wf, const float* nf, const float* bf, const float* kf, const void* P,
                                 int64_t ldp, int v0, float* state, float* out, int H, int d, int vd, int values, Batch bt,
                                 int dtype, hipStream_t st) {
  if (bt.B <= 0 || H <= 0 || d <= 0 || vd <= 0 || d > DL_DR * 32 || (values && !P)) return -1;
  int R = 1;
  while (R * DL_DR < d) R <<= 1;
  const int nw = vd <= 2 * (64 / R) ? 2 : 4;                // wavefronts of a workgroup: no more than the columns ask for
  const int wcols = nw * (64 / R);
  int TB = DL_TBR / R < 16 ? DL_TBR / R : 16;
  if (TB * wcols > 4 * 64 * nw) TB = 4 * 64 * nw / wcols;   // the value look-ahead holds 4 floats per thread
  if (TB < 1) return -1;
  const size_t sm = 2 * (size_t)(DL_NA * TB * R * DL_SEG + TB * wcols) * sizeof(float);
  const dim3 grid((vd + wcols - 1) / wcols, H, bt.B);
  RAGGED_DISPATCH(dtype,
    if (nw == 2) hipLaunchKernelGGL((delta_scan_kernel<T, 2>), grid, dim3(128), sm, st, rf, wf, nf, bf, kf, (const T*)P, ldp, v0, state,
                                    out, H, d, vd, R, TB, values, bt);
    else hipLaunchKernelGGL((delta_scan_kernel<T, 4>), grid, dim3(256), sm, st, rf, wf, nf, bf, kf, (const T*)P, ldp, v0, state, out,
                            H, d, vd, R, TB, values, bt))
  return RAGGED_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------------------------
// Long portions are cut into chunks that are scanned side by side.  A chunk maps the state at its start linearly,
// S_end = A_c S_start + L_c (A_c [d, d] per head: the chunk scanned without inputs from the identity; L_c: the chunk
// scanned from zero).  This kernel walks a sequence's chunks one after the other: begin[c] <- S, S <- A_c S + L_c, and
// leaves the last S in the sequence's slot.  A workgroup holds 16 columns of S in LDS; thread (i0, j) makes rows
// i0, i0 + 16, ... of column j.  Grid: (column blocks, heads, sequences); cfirst[b] .. cfirst[b + 1] - 1 are b's chunks.
constexpr int DC_COLS = 16;
constexpr int DC_LDS_D = 120;                              // up to this many rows a chunk's A is staged in LDS
constexpr int DC_APRE = (DC_LDS_D * DC_LDS_D + 255) / 256;
constexpr int DC_LPRE = (DC_LDS_D + 15) / 16;              // rows of a column that a thread makes

// LDSA: A_c is brought into LDS by the whole workgroup (coalesced) and A_c and the thread's elements of L_c are requested
// one chunk ahead into registers, so a chunk's step waits for no memory; otherwise every thread reads its rows of A_c and
// its elements of L_c from memory as it goes.
template <bool LDSA>
__global__ __launch_bounds__(256) void delta_chain_kernel(float* __restrict__ state, const float* __restrict__ local,
                                                          const float* __restrict__ trans, float* __restrict__ begin,
                                                          const int* __restrict__ cfirst, const int* __restrict__ seq_past,
                                                          const int* __restrict__ seq_slot, int H, int d, int vd) {
  extern __shared__ __attribute__((aligned(16))) float smem[];   // two buffers [d][DC_COLS], then A [d][d + 1]
  const int b = blockIdx.z, h = blockIdx.y;
  const int j = threadIdx.x % DC_COLS, i0 = threadIdx.x / DC_COLS, col = blockIdx.x * DC_COLS + j;
  const bool colok = col < vd;
  const int cc = colok ? col : vd - 1;
  float* cur = smem;
  float* nxt = smem + d * DC_COLS;
  float* As = smem + 2 * d * DC_COLS;
  const int lda = d + 1;
  float* sp = state + ((int64_t)seq_slot[b] * H + h) * d * vd;
  const bool old = seq_past[b] > 0;
  for (int i = i0; i < d; i += 256 / DC_COLS) cur[i * DC_COLS + j] = old ? sp[(int64_t)i * vd + cc] : 0.f;
  const int c0 = cfirst[b], c1 = cfirst[b + 1];
  float apre[LDSA ? DC_APRE : 1], lpre[LDSA ? DC_LPRE : 1], lcur[LDSA ? DC_LPRE : 1];
  auto fetch = [&](int c) {
    const float* A = trans + ((int64_t)c * H + h) * d * d;
    const float* L = local + ((int64_t)c * H + h) * d * vd;
#pragma unroll
    for (int u = 0; u < DC_APRE; ++u) {
      if (256 * u >= d * d) break;
      const int e = threadIdx.x + 256 * u;
      apre[u] = e < d * d ? A[e] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < DC_LPRE; ++u) {
      const int i = i0 + 16 * u;
      lpre[u] = i < d ? L[(int64_t)i * vd + cc] : 0.f;
    }
  };
  const int step_r = 256 / d, step_c = 256 % d;
  if (LDSA && c0 < c1) fetch(c0);
  __syncthreads();
  for (int c = c0; c < c1; ++c) {
    const float* A = trans + ((int64_t)c * H + h) * d * d;
    const float* L = local + ((int64_t)c * H + h) * d * vd;
    float* B = begin + ((int64_t)c * H + h) * d * vd;
    if (LDSA) {
      int ar_ = threadIdx.x / d, ac_ = threadIdx.x % d;      // element e = threadIdx.x + 256 u of A sits at (e / d, e % d)
#pragma unroll
      for (int u = 0; u < DC_APRE; ++u) {
        if (256 * u >= d * d) break;
        if (ar_ < d) As[ar_ * lda + ac_] = apre[u];
        ar_ += step_r;
        ac_ += step_c;
        if (ac_ >= d) { ac_ -= d; ++ar_; }
      }
#pragma unroll
      for (int u = 0; u < DC_LPRE; ++u) lcur[u] = lpre[u];
      __syncthreads();
      if (c + 1 < c1) fetch(c + 1);
    }
#pragma unroll 1
    for (int i = i0, u = 0; i < d; i += 256 / DC_COLS, ++u) {
      if (colok) B[(int64_t)i * vd + col] = cur[i * DC_COLS + j];
      float first = 0.f;
      if (LDSA) {
#pragma unroll
        for (int uu = 0; uu < DC_LPRE; ++uu) first = uu == u ? lcur[uu] : first;     // (a register, not an indexed array)
      } else {
        first = L[(int64_t)i * vd + cc];
      }
      float acc[4] = {first, 0.f, 0.f, 0.f};
      const float* ar = LDSA ? As + i * lda : A + (int64_t)i * d;
      int l = 0;
      for (; l + 4 <= d; l += 4) {
        acc[0] += ar[l] * cur[l * DC_COLS + j];
        acc[1] += ar[l + 1] * cur[(l + 1) * DC_COLS + j];
        acc[2] += ar[l + 2] * cur[(l + 2) * DC_COLS + j];
        acc[3] += ar[l + 3] * cur[(l + 3) * DC_COLS + j];
      }
      for (; l < d; ++l) acc[0] += ar[l] * cur[l * DC_COLS + j];
      nxt[i * DC_COLS + j] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    }
    __syncthreads();
    float* t = cur; cur = nxt; nxt = t;
  }
  for (int i = i0; i < d; i += 256 / DC_COLS)
    if (colok) sp[(int64_t)i * vd + col] = cur[i * DC_COLS + j];
}

extern "C" int ragged_delta_chain_ok(int d) { return d > 0 && d <= 384; }

extern "C" int ragged_delta_chain(float* state, const float* local, const float* trans, float* begin, const int* cfirst,
                                  const int* seq_past, const int* seq_slot, int B, int H, int d, int vd, hipStream_t st) {
  if (B <= 0 || H <= 0 || vd <= 0 || !ragged_delta_chain_ok(d)) return -1;
  const dim3 grid((vd + DC_COLS - 1) / DC_COLS, H, B);
  if (d <= DC_LDS_D) {
    const size_t sm = (2 * (size_t)d * DC_COLS + (size_t)d * (d + 1)) * sizeof(float);
    hipLaunchKernelGGL(delta_chain_kernel<true>, grid, dim3(256), sm, st, state, local, trans, begin, cfirst, seq_past, seq_slot, H, d, vd);
  } else {
    const size_t sm = 2 * (size_t)d * DC_COLS * sizeof(float);
    hipLaunchKernelGGL(delta_chain_kernel<false>, grid, dim3(256), sm, st, state, local, trans, begin, cfirst, seq_past, seq_slot, H, d, vd);
  }
  return RAGGED_LAUNCH_OK();
}
