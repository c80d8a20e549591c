// Argument block shared by the two paged attention kernels.
#pragma once
#include "ragged_common.h"

struct AttnArgs {
  const float* q;        // [T, H, MAPS, d]  normed and rotated
  const void* kpages;    // [num_pages, G, PAGE, MAPS * d]
  const void* vpages;    // [num_pages, G, PAGE, vd]
  void* out;             // [T, H * vd]
  const void* gate;      // gate logits: row t, column gate0 + h of a [T, ldg] matrix, or null
  int64_t ldg;
  int gate0;
  int H, G, d, vd;
  int window, keep_first;   // key j is visible from i if j <= i and (i - j < window or j < keep_first); window <= 0: all
                            // (see also chunk below)
  float scale;
  float lambda;          // two maps: o = a1 - lambda * a2
  float out_scale;       // applied after the output norm
  int out_norm;          // divide each head's output by its root mean square
  float eps;
  const int* rows;       // row-wise kernel: the token rows to serve (null: all T rows)
  int n_rows;
  const int* tiles;      // MFMA kernel: [n_tiles][2] = (sequence in the batch, first row of the tile inside its portion)
  int n_tiles;
  int64_t ldv;           // elements between the value rows of neighbouring keys (vd, or the key row's length when the
                         // values are the leading channels of the key rows and vpages == kpages)
  int sink;              // 1: exp(sink_score) joins every row's normaliser (a key that all queries see and that has no value)
  float sink_score;
  int chunk;             // > 0: positions are cut into blocks of this many, counted from the sequence's start, and key j
                         // is visible from i only inside i's block (on top of j <= i and of the window, if any)
  float softcap;         // > 0: scores pass through softcap * tanh(score / softcap) after the scale
  int gate_wide;         // 1: one gate logit per output channel (column gate0 + h * vd + c) instead of one per head
  const float* sinks;    // [H] or null: with `sink`, head h's own sink score instead of sink_score
  const float* slopes;   // [H] or null: slopes[h] * (i - j) is taken off the scaled score of query i and key j (in front of
                         // the cap, if there is one): a bias that grows with the distance
};

namespace ragged {
// the first key position that position `pos` may see (a window's lower edge can be negative: no key is that low)
__device__ __forceinline__ int low_key(int pos, int window, int chunk) {
  int lo = window > 0 ? pos - window + 1 : 0;
  if (chunk > 0) {
    const int c0 = pos >= 0 ? pos - pos % chunk : 0;
    lo = lo > c0 ? lo : c0;
  }
  return lo;
}
}  // namespace ragged
