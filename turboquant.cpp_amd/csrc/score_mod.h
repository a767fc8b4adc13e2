// What a model may do to an attention score between the product of query and key and the softmax, and which
// positions a token may see at all.  Every attention kernel takes the same description:
//
//   cap > 0        score <- cap * tanh(score / cap), after the scale
//   r1, r2         (per query head; null: none) then score <- score - r1[h] * ln(1 + r2[h] * (i - j)) for a query at
//                  position i and a key at position j <= i: a bias by distance
//   chunk > 0      position i sees j only if i / chunk == j / chunk (chunks counted from position 0 of the sequence),
//                  beside j <= i and beside a window, if there is one
//   sink           (per query head; null: none) the softmax's denominator also holds exp(sink[h]): a score that has no
//                  key and no value, is not scaled, capped or biased, and counts once per query.  The kernels start
//                  their running maximum at sink[h] with a denominator of 1 (the joins of decode steps add it once)
//   pb             (per query head; null: none) no softmax: the weight of a visible key is sigmoid(score + pb[h]), and
//                  the weights are not normalised over the keys.  The kernels keep their running maximum at 0, so that
//                  nothing is ever rescaled, and leave the division by the sum out
//   keep > 0       the first `keep` positions of a sequence stay visible to every later token, whatever the window:
//                  position i sees j <= i if j >= reach_lo(i) or j < keep
//
// All of it in float, on both libraries.
#pragma once
#include <hip/hip_runtime.h>

struct ScoreMod {
  float cap;
  const float* r1;
  const float* r2;
  int chunk;
  const float* sink;
  const float* pb;
  int keep;
};

// Tiles of `tile` positions that hold kept first positions, and the tile that follows tile t in a token's reach when
// its window starts in tile `lo_tile`: the kept tiles come first, then the walk jumps to the window's first tile.
__host__ __device__ __forceinline__ int keep_tiles(int keep, int tile) { return keep > 0 ? (keep + tile - 1) / tile : 0; }
__host__ __device__ __forceinline__ int first_tile(int lo_tile, int kept) { return kept > 0 ? 0 : lo_tile; }
__host__ __device__ __forceinline__ int next_tile(int t, int lo_tile, int kept) {
  ++t;
  return (t >= kept && t < lo_tile) ? lo_tile : t;
}
// whether a token at position p whose window starts at lo sees position j
__host__ __device__ __forceinline__ bool sees(int j, int p, int lo, int keep) { return j <= p && (j >= lo || j < keep); }

__device__ __forceinline__ float sigmoid_weight(float s) { return 1.0f / (1.0f + expf(-s)); }

// the first position that a token at position p may see
__host__ __device__ __forceinline__ int reach_lo(int p, int window, int chunk) {
  int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  if (chunk > 0 && p >= 0) {
    const int c = p / chunk * chunk;
    lo = c > lo ? c : lo;
  }
  return lo;
}

__device__ __forceinline__ bool score_mod_on(const ScoreMod& m) { return m.cap > 0.f || m.r1 != nullptr; }

// s: the scaled score; dist = i - j (taken as 0 where the key lies ahead of the query: such a key is masked anyway)
__device__ __forceinline__ float mod_score(float s, float cap, bool biased, float r1, float r2, int dist) {
  if (cap > 0.f) s = cap * tanhf(s / cap);
  if (biased) s -= r1 * log1pf(r2 * (float)(dist > 0 ? dist : 0));
  return s;
}

// The same with the hardware's exponential, logarithm and reciprocal (about 1e-7 absolute on tanh and on the
// logarithm of arguments of this size): for the bfloat16 library, whose probabilities are rounded to 8 bits
// anyway; the float32 library keeps the exact functions above.
__device__ __forceinline__ float mod_score_fast(float s, float cap, bool biased, float r1, float r2, int dist) {
  if (cap > 0.f) {
    // tanh(x) = 1 - 2 / (e^(2x) + 1); x is clamped where tanh is 1 to the last bit, so that e^(2x) stays finite
    const float x = fminf(fmaxf(s * __builtin_amdgcn_rcpf(cap), -15.f), 15.f);
    const float e = __builtin_amdgcn_exp2f(2.8853900817779268f * x);       // e^(2x) = 2^(2 x log2 e)
    s = cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
  }
  // ln(y) = log2(y) ln 2
  if (biased) s -= r1 * (0.6931471805599453f * __builtin_amdgcn_logf(1.0f + r2 * (float)(dist > 0 ? dist : 0)));
  return s;
}
