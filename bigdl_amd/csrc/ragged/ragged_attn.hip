// Paged attention of the ragged engine: causal sliding window that also keeps the first tokens and / or a mask of blocks
// counted from the sequence's start, soft-capped scores, one or two score maps per head over shared values
// (differential attention), per-head output norm and sigmoid gate (per head or per channel) in the epilogue.
//
// paged_attn_kernel (this file): one workgroup serves one (token row, query head).  A cache page holds 64 keys, one per
// lane, so the scores of a page are one register per map and the softmax statistics are wavefront reductions; values
// are read with lanes over channels.  A wavefront's life is a chain of dependent memory round trips (page id, keys,
// rounds of values), so the workgroup is up to 16 wavefronts that take every 16th visible page -- one or two pages
// each at a window of 1024 -- and merge their partial results through LDS.  It serves single decoded tokens and short portions in both activation types, and everything
// in float32; long bfloat16 prompt portions go to the MFMA kernel in ragged_attn_mfma.hip.
#include "ragged_attn.h"

using namespace ragged;

constexpr int MAX_VRP = 4;   // pairs of value channels per lane and 128 channels: vd <= 512

template <typename T> struct Vec;
template <> struct Vec<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16* p, float* o) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void load2(const bf16* p, float& a, float& b) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(p);
    a = __uint_as_float(u << 16);
    b = __uint_as_float(u & 0xffff0000u);
  }
};
template <> struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const float4 u = *reinterpret_cast<const float4*>(p);
    o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
  }
  static __device__ __forceinline__ void load2(const float* p, float& a, float& b) {
    const float2 u = *reinterpret_cast<const float2*>(p);
    a = u.x; b = u.y;
  }
};

// VEC: keys 16 bytes at a time (d a multiple of 8 halves / 4 floats) and values two channels at a time (vd even).
// REP > 1 and the row-spanning key fetch need VEC.
template <typename T, int MAPS, bool VEC, int VRP, int REP>
__global__ __launch_bounds__(512) void paged_attn_kernel(AttnArgs a, Batch bt, int coal) {
  constexpr int U = 32 / VRP;                         // keys per round of value loads
  constexpr int N = Vec<T>::N;
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int hgroups = a.H / REP;
  const int item = blockIdx.x;
  const int t = a.rows ? a.rows[item / hgroups] : item / hgroups, h0 = (item % hgroups) * REP;
  const int b = bt.tok_seq[t], i = bt.tok_pos[t];
  const int g = h0 / (a.H / a.G);
  const int qd = MAPS * a.d;
  const int vdp = (a.vd + 1) & ~1;
  const int pstride = 2 * MAPS + MAPS * vdp;          // one head's partial result: m[MAPS] l[MAPS] acc[MAPS][vdp]
  const int wstride = REP * pstride > REP * MAPS * PAGE ? REP * pstride : REP * MAPS * PAGE;
  float* qs = smem;                                   // [REP][qd]
  float* mine = smem + ((REP * qd + 3) & ~3) + wave * wstride;      // scores of a page, later this wavefront's partials
  for (int c = threadIdx.x; c < REP * qd; c += blockDim.x) qs[c] = a.q[((int64_t)t * a.H + h0) * qd + c];
  __syncthreads();

  const int lo_raw = low_key(i, a.window, a.chunk);
  const int lo = lo_raw > 0 ? lo_raw : 0;
  const int keep = a.window > 0 ? a.keep_first : 0;
  const T* K = (const T*)a.kpages;
  const T* V = (const T*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;
  // visible pages: those of the kept first tokens that lie before the window's first page, then the window's
  const int pl = lo / PAGE, last = i / PAGE;
  const int kept_pages = (keep + PAGE - 1) / PAGE < pl ? (keep + PAGE - 1) / PAGE : pl;
  const int npg = kept_pages + last - pl + 1;

  // row-spanning key fetch: a row is cpr pieces of 16 bytes, a load instruction covers 64 / cpr keys
  const int cpr = qd / N, cpm = cpr / MAPS;
  const int ks = coal ? lane / cpr : 0, ch = coal ? lane % cpr : 0;
  float qreg[REP][N];
  if (VEC && coal) {
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int e = 0; e < N; ++e) qreg[r][e] = qs[r * qd + ch * N + e];
  }

  float m[REP][MAPS], l[REP][MAPS], acc[REP][MAPS][VRP][2];
#pragma unroll
  for (int r = 0; r < REP; ++r)
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      m[r][mp] = -1e30f;
      l[r][mp] = 0.f;
#pragma unroll
      for (int v = 0; v < VRP; ++v) acc[r][mp][v][0] = acc[r][mp][v][1] = 0.f;
    }
  for (int o = wave; o < npg; o += nw) {
    const int pg = o < kept_pages ? o : pl + (o - kept_pages);
    const int page = pages[pg];
    const int kp = pg * PAGE + lane;
    const bool vis = kp <= i && (kp >= lo || kp < keep);
    const T* kpage = K + (((int64_t)page * a.G + g) * PAGE) * qd;
    // values: lanes over channel pairs (lanes past vd re-read the last pair; their sums are never stored), keys past
    // the query are read from the page's last valid row and weigh 0
    const int nk = i - pg * PAGE + 1 < PAGE ? i - pg * PAGE + 1 : PAGE;
    const T* vbase = V + (((int64_t)page * a.G + g) * PAGE) * a.ldv;
    float va[U][VRP][2], vb[U][VRP][2];
    auto load_values = [&](float (&dst)[U][VRP][2], int j0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = j0 + u < nk ? j0 + u : nk - 1;
#pragma unroll
        for (int v = 0; v < VRP; ++v) {
          const int c = 2 * lane + 128 * v;
          if (VEC) {
            Vec<T>::load2(vbase + (int64_t)j * a.ldv + (c < a.vd ? c : a.vd - 2), dst[u][v][0], dst[u][v][1]);
          } else {
            dst[u][v][0] = to_f(vbase[(int64_t)j * a.ldv + (c < a.vd ? c : a.vd - 1)]);
            dst[u][v][1] = to_f(vbase[(int64_t)j * a.ldv + (c + 1 < a.vd ? c + 1 : a.vd - 1)]);
          }
        }
      }
    };
    load_values(va, 0);                               // in flight during the scores
    float s[REP][MAPS];
    if (VEC && coal) {
      const int kpi = 64 / cpr;                       // keys per load instruction
      constexpr int KG = 16;                          // load instructions in flight before the first is used
      for (int u0 = 0; u0 < cpr; u0 += KG) {
        float kv[KG][N];
#pragma unroll
        for (int uu = 0; uu < KG; ++uu) {
          const int u = u0 + uu < cpr ? u0 + uu : cpr - 1;
          Vec<T>::load(kpage + (int64_t)(u * kpi + ks) * qd + ch * N, kv[uu]);
        }
#pragma unroll
        for (int uu = 0; uu < KG; ++uu) {
          if (u0 + uu < cpr) {
            float part[REP];
#pragma unroll
            for (int r = 0; r < REP; ++r) {
              part[r] = 0.f;
#pragma unroll
              for (int e = 0; e < N; ++e) part[r] += qreg[r][e] * kv[uu][e];
            }
#pragma unroll
            for (int r = 0; r < REP; ++r) part[r] = group_sum(part[r], cpm);
            if (ch % cpm == 0) {
#pragma unroll
              for (int r = 0; r < REP; ++r) mine[(r * MAPS + ch / cpm) * PAGE + (u0 + uu) * kpi + ks] = part[r];
            }
          }
        }
      }
      // (the wavefront reads what its own lanes wrote: LDS serves a wavefront's requests in order)
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) s[r][mp] = mine[(r * MAPS + mp) * PAGE + lane] * a.scale;
    } else {
      const T* krow = kpage + (int64_t)lane * qd;
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) s[r][mp] = 0.f;
      if (vis) {
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) {
          const T* kr = krow + mp * a.d;
          if (VEC) {
            for (int c = 0; c < a.d; c += N) {
              float kv[N];
              Vec<T>::load(kr + c, kv);
#pragma unroll
              for (int r = 0; r < REP; ++r)
#pragma unroll
                for (int e = 0; e < N; ++e) s[r][mp] += qs[r * qd + mp * a.d + c + e] * kv[e];
            }
          } else {
            for (int c = 0; c < a.d; ++c) {
              const float kvv = to_f(kr[c]);
#pragma unroll
              for (int r = 0; r < REP; ++r) s[r][mp] += qs[r * qd + mp * a.d + c] * kvv;
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) s[r][mp] *= a.scale;
    }
    if (a.slopes) {
      const float dist = (float)(i - kp);
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) s[r][mp] -= a.slopes[h0 + r] * dist;
    }
    if (a.softcap > 0.f) {
      const float inv_cap = 1.0f / a.softcap;
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) s[r][mp] = a.softcap * tanhf(s[r][mp] * inv_cap);
    }
    if (U < nk) load_values(vb, U);
    // softmax statistics of all heads and maps side by side (their cross-lane steps overlap)
    float p[REP][MAPS], mx[REP][MAPS], sm[REP][MAPS];
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) mx[r][mp] = wave_max(vis ? s[r][mp] : -1e30f);
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) {
        mx[r][mp] = fmaxf(m[r][mp], mx[r][mp]);
        p[r][mp] = vis ? __expf(s[r][mp] - mx[r][mp]) : 0.f;
      }
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) sm[r][mp] = wave_sum(p[r][mp]);
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) {
        const float corr = __expf(m[r][mp] - mx[r][mp]);
        l[r][mp] = l[r][mp] * corr + sm[r][mp];
        m[r][mp] = mx[r][mp];
#pragma unroll
        for (int v = 0; v < VRP; ++v) { acc[r][mp][v][0] *= corr; acc[r][mp][v][1] *= corr; }
      }
    // weights times values, U keys per round: round 0 was requested before the scores, round 1 before the softmax
    // (into the registers the keys have left), so a page exposes one memory round trip
    auto weigh = [&](float (&src)[U][VRP][2], int j0) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < REP; ++r)
#pragma unroll
          for (int mp = 0; mp < MAPS; ++mp) {
            const float pj = lane_value(p[r][mp], (j0 + u) & 63);
#pragma unroll
            for (int v = 0; v < VRP; ++v) { acc[r][mp][v][0] += pj * src[u][v][0]; acc[r][mp][v][1] += pj * src[u][v][1]; }
          }
    };
    weigh(va, 0);
    if (U < nk) weigh(vb, U);
    for (int j0 = 2 * U; j0 < nk; j0 += U) {
      load_values(va, j0);
      weigh(va, j0);
    }
  }
  // merge the wavefronts' partial results: wavefront r of the first REP finishes head h0 + r
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    float* pr = mine + r * pstride;
    if (lane == 0) {
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) { pr[mp] = m[r][mp]; pr[MAPS + mp] = l[r][mp]; }
    }
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
      for (int v = 0; v < VRP; ++v) {
        const int c = 2 * lane + 128 * v;
        if (c < vdp) { pr[2 * MAPS + mp * vdp + c] = acc[r][mp][v][0]; pr[2 * MAPS + mp * vdp + c + 1] = acc[r][mp][v][1]; }
      }
  }
  __syncthreads();
  const float* part0 = smem + ((REP * qd + 3) & ~3);
  for (int r = wave; r < REP; r += nw) {
    const int h = h0 + r;
    float o[VRP][2], ss = 0.f;
#pragma unroll
    for (int v = 0; v < VRP; ++v) o[v][0] = o[v][1] = 0.f;
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      float M = -1e30f, L = 0.f, w[8];
      for (int wv = 0; wv < nw; ++wv) M = fmaxf(M, part0[wv * wstride + r * pstride + mp]);
      const float sink_score = a.sinks ? a.sinks[h] : a.sink_score;
      if (a.sink) M = fmaxf(M, sink_score);
      for (int wv = 0; wv < nw; ++wv) {
        w[wv] = __expf(part0[wv * wstride + r * pstride + mp] - M);
        L += w[wv] * part0[wv * wstride + r * pstride + MAPS + mp];
      }
      if (a.sink) L += __expf(sink_score - M);
      const float coef = (mp == 0 ? 1.0f : -a.lambda) / L;
#pragma unroll
      for (int v = 0; v < VRP; ++v) {
        const int c = 2 * lane + 128 * v;
        if (c < vdp) {
          float s0 = 0.f, s1 = 0.f;
          for (int wv = 0; wv < nw; ++wv) {
            s0 += w[wv] * part0[wv * wstride + r * pstride + 2 * MAPS + mp * vdp + c];
            s1 += w[wv] * part0[wv * wstride + r * pstride + 2 * MAPS + mp * vdp + c + 1];
          }
          o[v][0] += coef * s0;
          o[v][1] += coef * s1;
        }
      }
    }
#pragma unroll
    for (int v = 0; v < VRP; ++v) {
      const int c = 2 * lane + 128 * v;
      if (c >= a.vd) o[v][0] = 0.f;
      if (c + 1 >= a.vd) o[v][1] = 0.f;
      ss += o[v][0] * o[v][0] + o[v][1] * o[v][1];
    }
    float f = a.out_scale;
    if (a.out_norm) f *= 1.0f / sqrtf(wave_sum(ss) / (float)a.vd + a.eps);
    if (a.gate && !a.gate_wide) f *= sigmoidf_(to_f(((const T*)a.gate)[(int64_t)t * a.ldg + a.gate0 + h]));
    T* orow = (T*)a.out + (int64_t)t * a.H * a.vd + (int64_t)h * a.vd;
    const T* grow = (const T*)a.gate + (int64_t)t * a.ldg + a.gate0 + (int64_t)h * a.vd;     // (read only with gate_wide)
#pragma unroll
    for (int v = 0; v < VRP; ++v) {
      const int c = 2 * lane + 128 * v;
      float f0 = f, f1 = f;
      if (a.gate_wide) {
        if (c < a.vd) f0 *= sigmoidf_(to_f(grow[c]));
        if (c + 1 < a.vd) f1 *= sigmoidf_(to_f(grow[c + 1]));
      }
      if (c < a.vd) orow[c] = from_f<T>(o[v][0] * f0);
      if (c + 1 < a.vd) orow[c + 1] = from_f<T>(o[v][1] * f1);
    }
  }
}

template <typename T, int MAPS, bool VEC, int VRP, int REP>
static void launch_one(AttnArgs a, Batch bt, int nrows, int coal, hipStream_t st, int* rc) {
  const int qd = MAPS * a.d, vdp = (a.vd + 1) & ~1;
  const int pstride = 2 * MAPS + MAPS * vdp;
  const int wstride = REP * pstride > REP * MAPS * PAGE ? REP * pstride : REP * MAPS * PAGE;
  // as many wavefronts as a row can have visible pages (longest sequence of the batch), at most 8, fewer if the
  // partial results would not fit 48 KB of LDS
  int nw = 8;
  int most = bt.max_pages;
  if (a.window > 0) most = (a.window + PAGE - 1) / PAGE + 1 + (a.keep_first + PAGE - 1) / PAGE;
  if (a.chunk > 0 && (a.chunk + PAGE - 1) / PAGE + 1 < most) most = (a.chunk + PAGE - 1) / PAGE + 1;
  while (nw > 1 && nw / 2 >= (most < bt.max_pages ? most : bt.max_pages)) nw >>= 1;
  auto lds = [&](int w) { return (size_t)(((REP * qd + 3) & ~3) + w * wstride) * sizeof(float); };
  while (nw > 1 && lds(nw) > 48 * 1024) nw >>= 1;
  if (lds(nw) > 60 * 1024) { *rc = -1; return; }
  const unsigned grid = (unsigned)(nrows * (a.H / REP));
  hipLaunchKernelGGL((paged_attn_kernel<T, MAPS, VEC, VRP, REP>), dim3(grid), dim3(64 * nw), lds(nw), st, a, bt, coal);
}

template <typename T, int MAPS>
static void launch_rows(AttnArgs a, Batch bt, int nrows, hipStream_t st, int* rc) {
  constexpr int N = Vec<T>::N;
  const bool vec = (a.vd % 2 == 0) && (a.d % N == 0) && (a.ldv % 2 == 0);
  const int vrp = a.vd <= 128 ? 1 : a.vd <= 256 ? 2 : 4;
  if (!vec || vrp == 4) {
    if (vrp == 1) launch_one<T, MAPS, false, 1, 1>(a, bt, nrows, 0, st, rc);
    else if (vrp == 2) launch_one<T, MAPS, false, 2, 1>(a, bt, nrows, 0, st, rc);
    else launch_one<T, MAPS, false, 4, 1>(a, bt, nrows, 0, st, rc);
    return;
  }
  const int cpr = MAPS * a.d / N;                                    // 16-byte pieces of a key row
  const int coal = cpr <= 64 && (cpr & (cpr - 1)) == 0 && (cpr / MAPS) >= 1;
  const int share = a.H / a.G;                                       // query heads per key/value head
  if (vrp == 1) {
    if (share % 8 == 0) launch_one<T, MAPS, true, 1, 8>(a, bt, nrows, coal, st, rc);
    else if (share % 4 == 0) launch_one<T, MAPS, true, 1, 4>(a, bt, nrows, coal, st, rc);
    else if (share % 2 == 0) launch_one<T, MAPS, true, 1, 2>(a, bt, nrows, coal, st, rc);
    else launch_one<T, MAPS, true, 1, 1>(a, bt, nrows, coal, st, rc);
  } else {
    if (share % 4 == 0) launch_one<T, MAPS, true, 2, 4>(a, bt, nrows, coal, st, rc);
    else if (share % 2 == 0) launch_one<T, MAPS, true, 2, 2>(a, bt, nrows, coal, st, rc);
    else launch_one<T, MAPS, true, 2, 1>(a, bt, nrows, coal, st, rc);
  }
}

extern "C" int ragged_paged_attn(AttnArgs a, Batch bt, int maps, int dtype, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || a.d <= 0 || a.vd <= 0 || a.vd > 128 * MAX_VRP) return -1;
  if ((maps != 1 && maps != 2) || a.ldv < a.vd || a.chunk < 0 || (a.gate_wide && !a.gate) || (a.sinks && !a.sink)) return -1;
  const int nrows = a.rows ? a.n_rows : bt.T;
  if (nrows <= 0 || (int64_t)nrows * a.H > 0x7fffffff) return -1;
  int rc = 0;
  RAGGED_DISPATCH(dtype,
    if (maps == 2) launch_rows<T, 2>(a, bt, nrows, st, &rc);
    else launch_rows<T, 1>(a, bt, nrows, st, &rc))
  if (rc) return rc;
  return RAGGED_LAUNCH_OK();
}
