// Paged attention for long bfloat16 prompt portions on the matrix cores (v_mfma_f32_16x16x32_bf16), same semantics as
// paged_attn_kernel in ragged_attn.hip.
//
//  * workgroup = 64 consecutive rows of one sequence's portion and one query head; wavefront w owns rows 16 w .. 16 w + 15.
//  * a cache page is the key tile.  Scores are computed transposed, S^T = K Q^T, so that a lane holds ONE query (its
//    column) and 4 keys of each 16-key block: running maximum, normaliser and rescale factor are per-lane scalars
//    (two cross-lane steps join the 4 lanes of a query), and the exponentials are already laid out as the B operand of
//    the second product O^T += V^T P^T, with the keys of a 32-key chunk in the order (4 g + j, 16 + 4 g + j).
//  * K fragments come straight from the page (16 bytes per lane), requested one page ahead; the value tile is transposed into LDS once per page by the whole
//    workgroup (a lane per key, so the 2-byte stores of a wavefront fall into consecutive addresses) from registers
//    that were loaded during the previous page's arithmetic, and read back as A fragments (two 8-byte reads each).
//  * softmax weights stay 32-bit quantities up to the matrix core: each goes through it as two bfloat16 terms, the upper
//    16 bits of p and the upper 16 bits of the exact remainder (2^-16 relative), so the second product loses nothing
//    beyond the values' own 16 bits.
//  * both maps of a differential head share the K page walk and the value tile.
#include "ragged_attn.h"

using namespace ragged;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int MF_DK = 4;     // 32-channel steps of a map: d <= 128
constexpr int MF_NEB = 8;    // 16-channel blocks of the values: vd <= 128
constexpr int MF_LDV = PAGE + 8;

union Frag {
  bf16x8 v;
  uint32_t u[4];
  uint16_t h[8];
  uint4 q;
  uint2 d2[2];
};

__device__ __forceinline__ uint16_t bf_bits(float f) { return from_f<bf16>(f).b; }
// tanh through one exponential and the hardware reciprocal: 1 - 2 / (e^(2x) + 1); absolute error of a few 1e-7, no
// overflow trouble (e^(2x) = inf gives 1, 0 gives -1)
__device__ __forceinline__ float fast_tanh(float x) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * x) + 1.0f); }

template <int MAPS, int DK>
__global__ __launch_bounds__(256) void paged_attn_mfma_kernel(AttnArgs a, Batch bt) {
  __shared__ __attribute__((aligned(16))) uint16_t vt[MF_NEB * 16 * MF_LDV];      // V^T [vd][PAGE (+ pad)]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lq = lane & 15, g4 = lane >> 4;
  const int tile = blockIdx.x / a.H, h = blockIdx.x % a.H;
  const int b = a.tiles[2 * tile], row0 = a.tiles[2 * tile + 1];
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b];
  const int gk = h / (a.H / a.G);
  const int qd = MAPS * a.d;
  const int neb = a.vd / 16;
  const int nrows = n - row0 < 64 ? n - row0 : 64;          // rows of this tile
  const int myrow = row0 + 16 * wave + lq;                  // this lane's query inside the portion
  const bool rowok = 16 * wave + lq < nrows;
  const int qpos = rowok ? past + myrow : -1;
  const int64_t t = start + (rowok ? myrow : row0);

  // queries as B fragments: lane = query lq, channels 32 ks + 8 g4 .. + 7
  Frag qf[MAPS][DK];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      const int ch = 32 * ks + 8 * g4;
#pragma unroll
      for (int e = 0; e < 4; ++e) qf[mp][ks].u[e] = 0;
      if (ch < a.d && rowok) {
        const float* qp = a.q + ((t * a.H + h) * MAPS + mp) * a.d + ch;
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[mp][ks].h[e] = bf_bits(qp[e]);
      }
    }

  const int p_first = past + row0, p_last = past + row0 + nrows - 1;
  const bool win = a.window > 0 || a.chunk > 0;              // some keys at or below a row's position are hidden
  const int keep = a.window > 0 ? a.keep_first : 0;
  const int lo_first = low_key(p_first, a.window, a.chunk);
  const int lo_tile = lo_first > 0 ? lo_first : 0;
  const int pl = lo_tile / PAGE, last = p_last / PAGE;
  const int kept_pages = (keep + PAGE - 1) / PAGE < pl ? (keep + PAGE - 1) / PAGE : pl;
  const int npg = kept_pages + last - pl + 1;
  // what this wavefront's 16 rows can see
  const int w_first = p_first + 16 * wave, w_last = (w_first + 15 < p_last ? w_first + 15 : p_last);
  const int w_lo = low_key(w_first, a.window, a.chunk);      // (the lowest key a row sees never falls as positions grow)
  const int w_lo_last = low_key(w_last, a.window, a.chunk);
  const bool wave_has_rows = 16 * wave < nrows;
  const int my_lo = low_key(qpos, a.window, a.chunk);
  const bool capped = a.softcap > 0.f;
  const float inv_cap = capped ? 1.0f / a.softcap : 0.f;
  const bool biased = a.slopes != nullptr;                   // scores fall with the distance between query and key
  const float slope = biased ? a.slopes[h] : 0.f;

  const bf16* K = (const bf16*)a.kpages;
  const bf16* V = (const bf16*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;

  float m[MAPS], l[MAPS];
  f32x4 O[MAPS][MF_NEB];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    m[mp] = -1e30f;
    l[mp] = 0.f;
#pragma unroll
    for (int eb = 0; eb < MF_NEB; ++eb) O[mp][eb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // value tile of a page: lane = key, wavefront w takes channel groups w, w + 4, ... (8 channels = 16 bytes each)
  Frag vreg[4];
  auto page_of = [&](int o) { return pages[o < kept_pages ? o : pl + (o - kept_pages)]; };
  auto load_values = [&](int page) {
    const bf16* vsrc = V + (((int64_t)page * a.G + gk) * PAGE + lane) * a.ldv;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) vreg[it].q = *reinterpret_cast<const uint4*>(vsrc + e0);
    }
  };
  // K fragments of a page: 16 bytes per lane and (key block, map, 32-channel step), requested one page ahead
  Frag kf[4][MAPS][DK], kfn[4][MAPS][DK];
  auto sees = [&](int o) {
    const int k0 = (o < kept_pages ? o : pl + (o - kept_pages)) * PAGE;
    return wave_has_rows && k0 <= w_last && (k0 + PAGE - 1 >= w_lo || k0 < keep);
  };
  auto load_keys = [&](int page) {
    const bf16* kpage = K + (((int64_t)page * a.G + gk) * PAGE) * qd;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const bf16* krow = kpage + (int64_t)(16 * kb + lq) * qd;
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) {
          const int ch = 32 * ks + 8 * g4;
          kfn[kb][mp][ks].q = ch < a.d ? *reinterpret_cast<const uint4*>(krow + mp * a.d + ch) : uint4{0, 0, 0, 0};
        }
    }
  };
  if (npg > 0) {
    load_values(page_of(0));
    if (sees(0)) load_keys(page_of(0));
  }

  for (int o = 0; o < npg; ++o) {
    const int pg = o < kept_pages ? o : pl + (o - kept_pages);
    const int k0 = pg * PAGE;
    const bool wave_sees = sees(o);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) kf[kb][mp][ks].q = kfn[kb][mp][ks].q;
    // ---- value tile -> LDS, transposed
    __syncthreads();                                         // the previous page's fragments have been read
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) {
#pragma unroll
        for (int u = 0; u < 8; ++u) vt[(e0 + u) * MF_LDV + lane] = vreg[it].h[u];
      }
    }
    __syncthreads();
    if (o + 1 < npg) {                                       // in flight during this page's arithmetic
      load_values(page_of(o + 1));
      if (sees(o + 1)) load_keys(page_of(o + 1));
    }
    if (!wave_sees) continue;

    // ---- S^T = K Q^T for the 4 key blocks of the page
    f32x4 S[MAPS][4];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        S[mp][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
          S[mp][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb][mp][ks].v, qf[mp][ks].v, S[mp][kb], 0, 0, 0);
      }
    // ---- mask, online softmax (per-lane scalars of the lane's query), exponentials as two bfloat16 terms
    Frag phi[MAPS][2], plo[MAPS][2];
    // a page whose 64 keys every row of this wavefront sees needs no mask arithmetic
    const bool inner = k0 + PAGE - 1 <= w_first && (!win || k0 >= w_lo_last || k0 + PAGE - 1 < keep);
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      float mx = -1e30f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float sc = S[mp][kb][i] * a.scale;
          if (biased) sc -= slope * (float)(qpos - (k0 + 16 * kb + 4 * g4 + i));
          if (capped) sc = a.softcap * fast_tanh(sc * inv_cap);
          if (!inner) {
            const int key = k0 + 16 * kb + 4 * g4 + i;
            const bool vis = key <= qpos && (key >= my_lo || key < keep);
            sc = vis ? sc : -1e30f;
          }
          S[mp][kb][i] = sc;
          mx = fmaxf(mx, sc);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mnew = fmaxf(m[mp], mx);
      const float corr = __expf(m[mp] - mnew);
      float sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; i += 2) {
          // masked scores are -1e30: their exponential is 0 unless the row has seen no key yet (mnew = -1e30)
          float p0 = S[mp][kb][i] > -1e29f ? __expf(S[mp][kb][i] - mnew) : 0.f;
          float p1 = S[mp][kb][i + 1] > -1e29f ? __expf(S[mp][kb][i + 1] - mnew) : 0.f;
          sum += p0 + p1;
          // p = hi + lo with hi the upper 16 bits of p (exact remainder) and lo the upper 16 bits of the remainder
          const uint32_t h0 = __float_as_uint(p0) & 0xffff0000u, h1 = __float_as_uint(p1) & 0xffff0000u;
          const uint32_t l0 = __float_as_uint(p0 - __uint_as_float(h0)), l1 = __float_as_uint(p1 - __uint_as_float(h1));
          phi[mp][kb >> 1].u[2 * (kb & 1) + (i >> 1)] = (h0 >> 16) | h1;
          plo[mp][kb >> 1].u[2 * (kb & 1) + (i >> 1)] = (l0 >> 16) | (l1 & 0xffff0000u);
        }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l[mp] = l[mp] * corr + sum;
      m[mp] = mnew;
#pragma unroll
      for (int eb = 0; eb < MF_NEB; ++eb) O[mp][eb] *= corr;
    }
    // ---- O^T += V^T P^T
#pragma unroll
    for (int eb = 0; eb < MF_NEB; ++eb) {
      if (eb < neb) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          Frag vf;
          const uint16_t* vrow = vt + (16 * eb + lq) * MF_LDV + 32 * c + 4 * g4;
          vf.d2[0] = *reinterpret_cast<const uint2*>(vrow);
          vf.d2[1] = *reinterpret_cast<const uint2*>(vrow + 16);
#pragma unroll
          for (int mp = 0; mp < MAPS; ++mp) {
            O[mp][eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, phi[mp][c].v, O[mp][eb], 0, 0, 0);
            O[mp][eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, plo[mp][c].v, O[mp][eb], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!rowok) return;
  // ---- epilogue: combine the maps, per-head norm, gate; the lane holds channels 16 eb + 4 g4 + i of its query
  if (a.sink) {                                              // one more term in every normaliser
    const float sink_score = a.sinks ? a.sinks[h] : a.sink_score;
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      const float mnew = fmaxf(m[mp], sink_score), corr = __expf(m[mp] - mnew);
      l[mp] = l[mp] * corr + __expf(sink_score - mnew);
#pragma unroll
      for (int eb = 0; eb < MF_NEB; ++eb) O[mp][eb] *= corr;
    }
  }
  const float c0 = 1.0f / l[0];
  const float c1 = MAPS == 2 ? a.lambda / l[MAPS - 1] : 0.f;
  float ss = 0.f;
#pragma unroll
  for (int eb = 0; eb < MF_NEB; ++eb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = O[0][eb][i] * c0;
      if (MAPS == 2) v -= O[MAPS - 1][eb][i] * c1;
      if (eb >= neb) v = 0.f;
      O[0][eb][i] = v;
      ss += v * v;
    }
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
  float f = a.out_scale;
  if (a.out_norm) f *= 1.0f / sqrtf(ss / (float)a.vd + a.eps);
  if (a.gate && !a.gate_wide) f *= sigmoidf_(to_f(((const bf16*)a.gate)[t * a.ldg + a.gate0 + h]));
  uint16_t* orow = (uint16_t*)a.out + t * (int64_t)(a.H * a.vd) + (int64_t)h * a.vd;
  const bf16* grow = (const bf16*)a.gate + t * a.ldg + a.gate0 + (int64_t)h * a.vd;        // (read only with gate_wide)
#pragma unroll
  for (int eb = 0; eb < MF_NEB; ++eb)
    if (eb < neb) {
      if (a.gate_wide) {                                     // one gate per channel: 8 bytes of logits per lane and block
        Frag gl;
        gl.d2[0] = *reinterpret_cast<const uint2*>(grow + 16 * eb + 4 * g4);
#pragma unroll
        for (int i = 0; i < 4; ++i) O[0][eb][i] *= sigmoidf_(__uint_as_float((uint32_t)gl.h[i] << 16));
      }
      uint2 w;
      w.x = (uint32_t)bf_bits(O[0][eb][0] * f) | ((uint32_t)bf_bits(O[0][eb][1] * f) << 16);
      w.y = (uint32_t)bf_bits(O[0][eb][2] * f) | ((uint32_t)bf_bits(O[0][eb][3] * f) << 16);
      *reinterpret_cast<uint2*>(orow + 16 * eb + 4 * g4) = w;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Wide rows: key rows of up to 32 DK channels and values of up to 16 NEB channels (one score map), as the latent
// attention has them after its queries are carried into the latent space (keys [latent row | rotated part], values the
// latent row).  Same tile, same transposed scores, same softmax and same two-term weights as above; what differs is
// where the operands live: the output tile alone takes up to 128 registers, so K fragments are not held a page ahead but
// come from memory six 32-channel steps at a time (the four wavefronts of a workgroup read the same page, so three of
// four reads hit the CU's cache), and the value tile's registers are requested one page ahead.
template <int DK, int NEB>
__global__ __launch_bounds__(256) void paged_attn_mfma_wide_kernel(AttnArgs a, Batch bt) {
  extern __shared__ __attribute__((aligned(16))) uint16_t vt[];                   // V^T [16 NEB][PAGE (+ pad)]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lq = lane & 15, g4 = lane >> 4;
  const int tile = blockIdx.x / a.H, h = blockIdx.x % a.H;
  const int b = a.tiles[2 * tile], row0 = a.tiles[2 * tile + 1];
  const int start = bt.seq_start[b], n = bt.seq_start[b + 1] - start, past = bt.seq_past[b];
  const int gk = h / (a.H / a.G);
  const int neb = a.vd / 16;
  const int nrows = n - row0 < 64 ? n - row0 : 64;
  const int myrow = row0 + 16 * wave + lq;
  const bool rowok = 16 * wave + lq < nrows;
  const int qpos = rowok ? past + myrow : -1;
  const int64_t t = start + (rowok ? myrow : row0);

  Frag qf[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    const int ch = 32 * ks + 8 * g4;
#pragma unroll
    for (int e = 0; e < 4; ++e) qf[ks].u[e] = 0;
    if (ch < a.d && rowok) {
      const float* qp = a.q + (t * a.H + h) * a.d + ch;
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks].h[e] = bf_bits(qp[e]);
    }
  }

  const int p_first = past + row0, p_last = past + row0 + nrows - 1;
  const bool win = a.window > 0;
  const int lo_tile = win ? (p_first - a.window + 1 > 0 ? p_first - a.window + 1 : 0) : 0;
  const int pl = lo_tile / PAGE, last = p_last / PAGE;
  const int w_first = p_first + 16 * wave, w_last = (w_first + 15 < p_last ? w_first + 15 : p_last);
  const int w_lo = win ? w_first - a.window + 1 : 0;
  const bool wave_has_rows = 16 * wave < nrows;
  const int my_lo = win ? qpos - a.window + 1 : 0;

  const bf16* K = (const bf16*)a.kpages;
  const bf16* V = (const bf16*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;

  float m = -1e30f, l = 0.f;
  f32x4 O[NEB];
#pragma unroll
  for (int eb = 0; eb < NEB; ++eb) O[eb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this lane's share of a page's value tile (lane = key, wavefront w takes channel groups w, w + 4, ..., 16 bytes each),
  // requested one page ahead so that it is in flight during the current page's arithmetic
  Frag vreg[NEB / 2];
  auto load_values = [&](int page) {
    const bf16* vsrc = V + (((int64_t)page * a.G + gk) * PAGE + lane) * a.ldv;
#pragma unroll
    for (int it = 0; it < NEB / 2; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) vreg[it].q = *reinterpret_cast<const uint4*>(vsrc + e0);
    }
  };
  if (pl <= last) load_values(pages[pl]);

  for (int pg = pl; pg <= last; ++pg) {
    const int page = pages[pg];
    const int k0 = pg * PAGE;
    const bool wave_sees = wave_has_rows && k0 <= w_last && k0 + PAGE - 1 >= w_lo;
    // ---- value tile -> LDS, transposed
    __syncthreads();                                         // the previous page's tile has been read
#pragma unroll
    for (int it = 0; it < NEB / 2; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) {
#pragma unroll
        for (int u = 0; u < 8; ++u) vt[(e0 + u) * MF_LDV + lane] = vreg[it].h[u];
      }
    }
    __syncthreads();
    if (pg < last) load_values(pages[pg + 1]);
    if (!wave_sees) continue;

    // ---- S^T = K Q^T for the 4 key blocks of the page, K fragments from memory KS 32-channel steps at a time
    const bf16* kpage = K + (((int64_t)page * a.G + gk) * PAGE) * a.d;
    f32x4 S[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) S[kb] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int KS = DK % 6 == 0 ? 6 : 5;
#pragma unroll
    for (int ks0 = 0; ks0 < DK; ks0 += KS) {
      Frag kf[4][KS];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int j = 0; j < KS; ++j) {
          const int ch = 32 * (ks0 + j) + 8 * g4;
          kf[kb][j].q = (ks0 + j < DK && ch < a.d) ? *reinterpret_cast<const uint4*>(kpage + (int64_t)(16 * kb + lq) * a.d + ch)
                                                   : uint4{0, 0, 0, 0};
        }
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int j = 0; j < KS; ++j)
          if (ks0 + j < DK) S[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb][j].v, qf[ks0 + j].v, S[kb], 0, 0, 0);
    }
    // ---- mask, online softmax (per-lane scalars of the lane's query), exponentials as two bfloat16 terms
    Frag phi[2], plo[2];
    const bool inner = k0 + PAGE - 1 <= w_first && (!win || k0 >= w_last - a.window + 1);
    float mx = -1e30f;
    if (inner) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          S[kb][i] *= a.scale;
          mx = fmaxf(mx, S[kb][i]);
        }
    } else {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + 16 * kb + 4 * g4 + i;
          const bool vis = key <= qpos && key >= my_lo;
          S[kb][i] = vis ? S[kb][i] * a.scale : -1e30f;
          mx = fmaxf(mx, S[kb][i]);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mnew = fmaxf(m, mx);
    const float corr = __expf(m - mnew);
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 4; i += 2) {
        float p0 = S[kb][i] > -1e29f ? __expf(S[kb][i] - mnew) : 0.f;
        float p1 = S[kb][i + 1] > -1e29f ? __expf(S[kb][i + 1] - mnew) : 0.f;
        sum += p0 + p1;
        const uint32_t h0 = __float_as_uint(p0) & 0xffff0000u, h1 = __float_as_uint(p1) & 0xffff0000u;
        const uint32_t l0 = __float_as_uint(p0 - __uint_as_float(h0)), l1 = __float_as_uint(p1 - __uint_as_float(h1));
        phi[kb >> 1].u[2 * (kb & 1) + (i >> 1)] = (h0 >> 16) | h1;
        plo[kb >> 1].u[2 * (kb & 1) + (i >> 1)] = (l0 >> 16) | (l1 & 0xffff0000u);
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    l = l * corr + sum;
    m = mnew;
#pragma unroll
    for (int eb = 0; eb < NEB; ++eb) O[eb] *= corr;
    // ---- O^T += V^T P^T
#pragma unroll
    for (int eb = 0; eb < NEB; ++eb) {
      if (eb < neb) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          Frag vf;
          const uint16_t* vrow = vt + (16 * eb + lq) * MF_LDV + 32 * c + 4 * g4;
          vf.d2[0] = *reinterpret_cast<const uint2*>(vrow);
          vf.d2[1] = *reinterpret_cast<const uint2*>(vrow + 16);
          O[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, phi[c].v, O[eb], 0, 0, 0);
          O[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, plo[c].v, O[eb], 0, 0, 0);
        }
      }
    }
  }
  if (!rowok) return;
  if (a.sink) {
    const float mnew = fmaxf(m, a.sink_score), corr = __expf(m - mnew);
    l = l * corr + __expf(a.sink_score - mnew);
#pragma unroll
    for (int eb = 0; eb < NEB; ++eb) O[eb] *= corr;
  }
  const float f = a.out_scale / l;
  uint16_t* orow = (uint16_t*)a.out + t * (int64_t)(a.H * a.vd) + (int64_t)h * a.vd;
#pragma unroll
  for (int eb = 0; eb < NEB; ++eb)
    if (eb < neb) {
      uint2 w;
      w.x = (uint32_t)bf_bits(O[eb][0] * f) | ((uint32_t)bf_bits(O[eb][1] * f) << 16);
      w.y = (uint32_t)bf_bits(O[eb][2] * f) | ((uint32_t)bf_bits(O[eb][3] * f) << 16);
      *reinterpret_cast<uint2*>(orow + 16 * eb + 4 * g4) = w;
    }
}

// 1 when the wide kernel serves this layout: one map, no kept first tokens, no output norm, no gate
extern "C" int ragged_paged_attn_mfma_wide_ok(int d, int vd) {
  return d % 8 == 0 && d <= 32 * 18 && vd % 16 == 0 && vd <= 16 * 32;
}

template <int DK, int NEB>
static int launch_wide(AttnArgs a, Batch bt, unsigned grid, hipStream_t st) {
  const size_t lds = (size_t)NEB * 16 * MF_LDV * sizeof(uint16_t);
  static bool raised = false;                                 // tiles above 64 KB need the limit raised once per kernel
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)paged_attn_mfma_wide_kernel<DK, NEB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) return -3;
    raised = true;
  }
  hipLaunchKernelGGL((paged_attn_mfma_wide_kernel<DK, NEB>), dim3(grid), dim3(256), lds, st, a, bt);
  return 0;
}

extern "C" int ragged_paged_attn_mfma_wide(AttnArgs a, Batch bt, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || !ragged_paged_attn_mfma_wide_ok(a.d, a.vd)) return -1;
  if (a.ldv < a.vd || a.ldv % 8 || a.keep_first > 0 || a.out_norm || a.gate || a.chunk > 0 || a.softcap > 0.f || a.sinks || a.slopes) return -1;
  if (!a.tiles || a.n_tiles <= 0 || (int64_t)a.n_tiles * a.H > 0x7fffffff) return -1;
  const unsigned grid = (unsigned)(a.n_tiles * a.H);
  const int dk = (a.d + 31) / 32, neb = a.vd / 16;
  int rc;
  if (dk <= 6 && neb <= 8) rc = launch_wide<6, 8>(a, bt, grid, st);
  else if (dk <= 6 && neb <= 16) rc = launch_wide<6, 16>(a, bt, grid, st);
  else if (dk <= 10 && neb <= 16) rc = launch_wide<10, 16>(a, bt, grid, st);
  else if (dk <= 10) rc = launch_wide<10, 32>(a, bt, grid, st);
  else rc = launch_wide<18, 32>(a, bt, grid, st);
  if (rc) return rc;
  return RAGGED_LAUNCH_OK();
}

// Wide rows, single tokens and short portions: one workgroup serves one token row and 16 query heads that share a
// key/value head -- the heads are the 16 columns of the score tile, so a page's keys are read once for all of them.
// The four wavefronts split a page's keys for the scores (wavefront w: keys 16 w .. 16 w + 15, K fragments straight from
// memory, requested one page ahead) and the value channels for the weighted sum (wavefront w: a quarter of the 16-channel
// blocks); in between, the page's maxima, sums and exponentials (two bfloat16 terms each, already in the layout of the
// second product's operand) cross the wavefronts through LDS.
template <int DK, int NEB>
__global__ __launch_bounds__(256) void paged_attn_mfma_heads_kernel(AttnArgs a, Batch bt) {
  extern __shared__ __attribute__((aligned(16))) uint16_t vt[];                   // V^T [16 NEB][PAGE (+ pad)]
  uint4* pbuf = reinterpret_cast<uint4*>(vt + NEB * 16 * MF_LDV);                 // [4 key blocks][64 lanes]
  float* smax = reinterpret_cast<float*>(pbuf + 256);                             // [4][16]
  float* ssum = smax + 64;                                                        // [4][16]
  constexpr int NE = NEB / 4;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lq = lane & 15, g4 = lane >> 4;
  const int share = a.H / a.G, nblk = (share + 15) / 16;
  const int item = blockIdx.x, ri = item / (a.G * nblk), rem = item % (a.G * nblk);
  const int gk = rem / nblk, blk = rem % nblk;
  const int64_t t = a.rows ? a.rows[ri] : ri;
  const int b = bt.tok_seq[t], qpos = bt.tok_pos[t];
  const bool headok = blk * 16 + lq < share;
  const int h = gk * share + (headok ? blk * 16 + lq : 0);
  const int neb = a.vd / 16;

  Frag qf[DK];
#pragma unroll
  for (int ks = 0; ks < DK; ++ks) {
    const int ch = 32 * ks + 8 * g4;
#pragma unroll
    for (int e = 0; e < 4; ++e) qf[ks].u[e] = 0;
    if (ch < a.d && headok) {
      const float* qp = a.q + (t * a.H + h) * a.d + ch;
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks].h[e] = bf_bits(qp[e]);
    }
  }
  const bool win = a.window > 0;
  const int lo = win ? (qpos - a.window + 1 > 0 ? qpos - a.window + 1 : 0) : 0;
  const int pl = lo / PAGE, last = qpos / PAGE;
  const bf16* K = (const bf16*)a.kpages;
  const bf16* V = (const bf16*)a.vpages;
  const int* pages = bt.pages + (int64_t)b * bt.max_pages;

  float m = -1e30f, l = 0.f;
  f32x4 O[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) O[e] = f32x4{0.f, 0.f, 0.f, 0.f};

  Frag vreg[NEB / 2], kfn[DK];
  auto load_page = [&](int page) {
    const bf16* vsrc = V + (((int64_t)page * a.G + gk) * PAGE + lane) * a.ldv;
#pragma unroll
    for (int it = 0; it < NEB / 2; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) vreg[it].q = *reinterpret_cast<const uint4*>(vsrc + e0);
    }
    const bf16* krow = K + (((int64_t)page * a.G + gk) * PAGE + 16 * wave + lq) * a.d;
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      const int ch = 32 * ks + 8 * g4;
      kfn[ks].q = ch < a.d ? *reinterpret_cast<const uint4*>(krow + ch) : uint4{0, 0, 0, 0};
    }
  };
  load_page(pages[pl]);

  for (int pg = pl; pg <= last; ++pg) {
    const int k0 = pg * PAGE;
    Frag kf[DK];
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) kf[ks].q = kfn[ks].q;
    __syncthreads();                                         // the previous page's tile and exponentials have been read
#pragma unroll
    for (int it = 0; it < NEB / 2; ++it) {
      const int e0 = 8 * (4 * it + wave);
      if (e0 < a.vd) {
#pragma unroll
        for (int u = 0; u < 8; ++u) vt[(e0 + u) * MF_LDV + lane] = vreg[it].h[u];
      }
    }
    if (pg < last) load_page(pages[pg + 1]);
    // ---- scores of this wavefront's 16 keys against the 16 heads
    f32x4 S = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) S = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks].v, qf[ks].v, S, 0, 0, 0);
    float mx = -1e30f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = k0 + 16 * wave + 4 * g4 + i;
      S[i] = (key <= qpos && key >= lo) ? S[i] * a.scale : -1e30f;
      mx = fmaxf(mx, S[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    if (g4 == 0) smax[wave * 16 + lq] = mx;
    __syncthreads();
    const float pm = fmaxf(fmaxf(smax[lq], smax[16 + lq]), fmaxf(smax[32 + lq], smax[48 + lq]));
    const float mnew = fmaxf(m, pm);
    const float corr = __expf(m - mnew);
    float p[4], sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = S[i] > -1e29f ? __expf(S[i] - mnew) : 0.f;
      sum += p[i];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    if (g4 == 0) ssum[wave * 16 + lq] = sum;
    {
      uint32_t hi[4], lw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        hi[i] = __float_as_uint(p[i]) & 0xffff0000u;
        lw[i] = __float_as_uint(p[i] - __uint_as_float(hi[i]));
      }
      pbuf[wave * 64 + lane] = uint4{(hi[0] >> 16) | hi[1], (hi[2] >> 16) | hi[3], (lw[0] >> 16) | (lw[1] & 0xffff0000u),
                                     (lw[2] >> 16) | (lw[3] & 0xffff0000u)};
    }
    __syncthreads();
    l = l * corr + ((ssum[lq] + ssum[16 + lq]) + (ssum[32 + lq] + ssum[48 + lq]));
    m = mnew;
    Frag phi[2], plo[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const uint4 x0 = pbuf[(2 * c) * 64 + lane], x1 = pbuf[(2 * c + 1) * 64 + lane];
      phi[c].u[0] = x0.x; phi[c].u[1] = x0.y; phi[c].u[2] = x1.x; phi[c].u[3] = x1.y;
      plo[c].u[0] = x0.z; plo[c].u[1] = x0.w; plo[c].u[2] = x1.z; plo[c].u[3] = x1.w;
    }
    // ---- this wavefront's value channels
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int eb = wave * NE + e;
      O[e] *= corr;
      if (eb < neb) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          Frag vf;
          const uint16_t* vrow = vt + (16 * eb + lq) * MF_LDV + 32 * c + 4 * g4;
          vf.d2[0] = *reinterpret_cast<const uint2*>(vrow);
          vf.d2[1] = *reinterpret_cast<const uint2*>(vrow + 16);
          O[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, phi[c].v, O[e], 0, 0, 0);
          O[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, plo[c].v, O[e], 0, 0, 0);
        }
      }
    }
  }
  if (!headok) return;
  float corr = 1.0f;
  if (a.sink) {
    const float mnew = fmaxf(m, a.sink_score);
    corr = __expf(m - mnew);
    l = l * corr + __expf(a.sink_score - mnew);
  }
  const float f = a.out_scale * corr / l;
  uint16_t* orow = (uint16_t*)a.out + t * (int64_t)(a.H * a.vd) + (int64_t)h * a.vd;
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int eb = wave * NE + e;
    if (eb < neb) {
      uint2 w;
      w.x = (uint32_t)bf_bits(O[e][0] * f) | ((uint32_t)bf_bits(O[e][1] * f) << 16);
      w.y = (uint32_t)bf_bits(O[e][2] * f) | ((uint32_t)bf_bits(O[e][3] * f) << 16);
      *reinterpret_cast<uint2*>(orow + 16 * eb + 4 * g4) = w;
    }
  }
}

template <int DK, int NEB>
static int launch_heads(AttnArgs a, Batch bt, unsigned grid, hipStream_t st) {
  const size_t lds = (size_t)NEB * 16 * MF_LDV * sizeof(uint16_t) + 256 * sizeof(uint4) + 128 * sizeof(float);
  static bool raised = false;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)paged_attn_mfma_heads_kernel<DK, NEB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) return -3;
    raised = true;
  }
  hipLaunchKernelGGL((paged_attn_mfma_heads_kernel<DK, NEB>), dim3(grid), dim3(256), lds, st, a, bt);
  return 0;
}

// token rows a.rows[0 .. n_rows) (all T rows without a list)
extern "C" int ragged_paged_attn_mfma_heads(AttnArgs a, Batch bt, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || !ragged_paged_attn_mfma_wide_ok(a.d, a.vd)) return -1;
  if (a.ldv < a.vd || a.ldv % 8 || a.keep_first > 0 || a.out_norm || a.gate || a.chunk > 0 || a.softcap > 0.f || a.sinks || a.slopes) return -1;
  const int nrows = a.rows ? a.n_rows : bt.T;
  const int nblk = (a.H / a.G + 15) / 16;
  if (nrows <= 0 || (int64_t)nrows * a.G * nblk > 0x7fffffff) return -1;
  const unsigned grid = (unsigned)(nrows * a.G * nblk);
  const int dk = (a.d + 31) / 32, neb = a.vd / 16;
  int rc;
  if (dk <= 6 && neb <= 8) rc = launch_heads<6, 8>(a, bt, grid, st);
  else if (dk <= 6 && neb <= 16) rc = launch_heads<6, 16>(a, bt, grid, st);
  else if (dk <= 10 && neb <= 16) rc = launch_heads<10, 16>(a, bt, grid, st);
  else if (dk <= 10) rc = launch_heads<10, 32>(a, bt, grid, st);
  else rc = launch_heads<18, 32>(a, bt, grid, st);
  if (rc) return rc;
  return RAGGED_LAUNCH_OK();
}

// 1 when the MFMA kernel serves this head layout (bfloat16 only)
extern "C" int ragged_paged_attn_mfma_ok(int d, int vd) {
  return d % 8 == 0 && d <= 32 * MF_DK && vd % 16 == 0 && vd <= 16 * MF_NEB;
}

template <int MAPS>
static void launch_mfma(AttnArgs a, Batch bt, unsigned grid, hipStream_t st) {
  const int dk = (a.d + 31) / 32;
  if (dk == 1) hipLaunchKernelGGL((paged_attn_mfma_kernel<MAPS, 1>), dim3(grid), dim3(256), 0, st, a, bt);
  else if (dk == 2) hipLaunchKernelGGL((paged_attn_mfma_kernel<MAPS, 2>), dim3(grid), dim3(256), 0, st, a, bt);
  else if (dk == 3) hipLaunchKernelGGL((paged_attn_mfma_kernel<MAPS, 3>), dim3(grid), dim3(256), 0, st, a, bt);
  else hipLaunchKernelGGL((paged_attn_mfma_kernel<MAPS, 4>), dim3(grid), dim3(256), 0, st, a, bt);
}

extern "C" int ragged_paged_attn_mfma(AttnArgs a, Batch bt, int maps, hipStream_t st) {
  if (bt.T <= 0 || a.H <= 0 || a.G <= 0 || a.H % a.G || !ragged_paged_attn_mfma_ok(a.d, a.vd)) return -1;
  if (a.ldv < a.vd || a.ldv % 8) return -1;                  // value rows are read 16 bytes at a time
  // per-channel gate logits are read 8 bytes at a time
  if (a.chunk < 0 || (a.gate_wide && (!a.gate || a.ldg % 4 || a.gate0 % 4)) || (a.sinks && !a.sink)) return -1;
  if ((maps != 1 && maps != 2) || !a.tiles || a.n_tiles <= 0 || (int64_t)a.n_tiles * a.H > 0x7fffffff) return -1;
  const unsigned grid = (unsigned)(a.n_tiles * a.H);
  if (maps == 2) launch_mfma<2>(a, bt, grid, st);
  else launch_mfma<1>(a, bt, grid, st);
  return RAGGED_LAUNCH_OK();
}
