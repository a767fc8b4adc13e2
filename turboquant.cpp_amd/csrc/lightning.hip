// Linear attention with a constant decay per head ("lightning"), over per-sequence state of fixed size.
//
// Per head, with a state S [D][V] (key channels by value channels) that starts at zero, token by token:
//   S <- decay_h S + k v^T ;  o = S^T q
// with q, k (D per head) and v (V per head) the silu of projections, and nothing else scaled.  The read-outs of all
// heads of a token are then normed together (one root mean square over H V numbers), multiplied by a weight per channel
// and by sigmoid(gate), the gate a projection of its own.  Everything here is float arithmetic on both libraries; the
// products around it are the library's.
//
// Projections P [T][NP] (float): q (H D) | k (H D) | v (H V) | gate (H V), NP >= 2 H D + 2 H V floats apart.
// A sequence's row of state (float): S as [H][D][V].
//
// Two kernels, for prompts and for decoding alike (a decoded token is a run of one):
//   lightning_scan  per (sequence, head, block of value channels): the recurrence over the run's tokens in order, the
//                   state in registers (LN_ROWS key channels of a value channel per lane, the lanes of a value channel
//                   neighbours that add their partial read-outs by shuffles), tokens staged through LDS in chunks with
//                   silu applied as they are staged.  The order of every sum depends on the sizes only, never on how
//                   the sequence was cut into steps or on what else the step holds.
//   lightning_out   per token: the norm over all heads, the weight and the gate, into the activation type.
#include "common.h"

#define LN_ROWS 16        // key channels of a value channel that one lane keeps
#define LN_CHUNK 16       // tokens staged at a time
#define LN_SEG 20         // floats between the rows of two lanes in LDS (16 would put eight lanes on four banks)

__device__ __forceinline__ float ln_silu(float x) { return x / (1.0f + expf(-x)); }

// grid (ceil(V / VB), H, B), block 256; L = lanes per value channel (a power of two, L * LN_ROWS >= D), VB = 256 / L.
template <int L>
__global__ __launch_bounds__(256) void lightning_scan_kernel(const float* __restrict__ P, int64_t ldp,
                                                             const float* __restrict__ decay,
                                                             const int* __restrict__ cu_seqlens,
                                                             const int* __restrict__ slots, float* __restrict__ state,
                                                             int64_t state_stride, int H, int D, int V,
                                                             float* __restrict__ o) {
  constexpr int VB = 256 / L;
  __shared__ float qs[LN_CHUNK][L * LN_SEG], ks[LN_CHUNK][L * LN_SEG], vs[LN_CHUNK][VB];
  const int b = blockIdx.z, h = blockIdx.y, v0 = blockIdx.x * VB;
  const int tid = threadIdx.x, vc = tid / L, j = tid % L;
  const int v = v0 + vc;
  const bool live = v < V;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
  if (n <= 0) return;
  const float lam = decay[h];
  float* srow = state + (size_t)slots[b] * state_stride + (size_t)h * D * V;
  float S[LN_ROWS];
#pragma unroll
  for (int r = 0; r < LN_ROWS; ++r) {
    const int d = j * LN_ROWS + r;
    S[r] = live && d < D ? srow[(size_t)d * V + v] : 0.f;
  }
  const float* q0 = P + (size_t)h * D;
  const float* k0 = P + (size_t)H * D + (size_t)h * D;
  const float* vv0 = P + (size_t)2 * H * D + (size_t)h * V + v0;
  const int nvb = min(VB, V - v0);
  for (int c0 = 0; c0 < n; c0 += LN_CHUNK) {
    const int nc = min(LN_CHUNK, n - c0);
    __syncthreads();
    for (int idx = tid; idx < nc * L * LN_ROWS; idx += 256) {
      const int c = idx / (L * LN_ROWS), d = idx % (L * LN_ROWS);
      const size_t row = (size_t)(t0 + c0 + c) * ldp;
      const int at = (d / LN_ROWS) * LN_SEG + d % LN_ROWS;
      qs[c][at] = d < D ? ln_silu(q0[row + d]) : 0.f;
      ks[c][at] = d < D ? ln_silu(k0[row + d]) : 0.f;
    }
    for (int idx = tid; idx < nc * VB; idx += 256) {
      const int c = idx / VB, i = idx % VB;
      vs[c][i] = i < nvb ? ln_silu(vv0[(size_t)(t0 + c0 + c) * ldp + i]) : 0.f;
    }
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
      const float val = vs[c][vc];
      const float* kr = &ks[c][j * LN_SEG];
      const float* qr = &qs[c][j * LN_SEG];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < LN_ROWS; ++r) {
        S[r] = fmaf(lam, S[r], kr[r] * val);
        acc = fmaf(S[r], qr[r], acc);
      }
#pragma unroll
      for (int off = L / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, TQ_WAVE);
      if (j == 0 && live) o[(size_t)(t0 + c0 + c) * H * V + (size_t)h * V + v] = acc;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < LN_ROWS; ++r) {
      const int d = j * LN_ROWS + r;
      if (d < D) srow[(size_t)d * V + v] = S[r];
    }
  }
}

// P: the step's projections [T][ldp]; decay [H]; cu_seqlens [B + 1], slots [B]: the tokens as one run per sequence;
// state: the rows of all slots, state_stride floats apart; o [T][H V] float.
TQ_API int tq_lightning_scan(const float* P, int64_t ldp, const float* decay, const int* cu_seqlens, const int* slots,
                             float* state, int64_t state_stride, int B, int H, int D, int V, float* o, hipStream_t st) {
  if (B <= 0) return 0;
  if (H < 1 || D < 1 || V < 1 || ldp < (int64_t)2 * H * D + (int64_t)2 * H * V || state_stride < (int64_t)H * D * V)
    return TQ_ERR_BAD_ARG;
  if (D > 16 * LN_ROWS || H > 65535 || B > 65535) return TQ_ERR_UNSUPPORTED;
  int L = 1;
  while (L * LN_ROWS < D) L *= 2;
#define TQ_LN_LAUNCH(LV)                                                                                              \
  hipLaunchKernelGGL(lightning_scan_kernel<LV>, dim3((V + 256 / LV - 1) / (256 / LV), H, B), dim3(256), 0, st, P, ldp, \
                     decay, cu_seqlens, slots, state, state_stride, H, D, V, o)
  switch (L) {
    case 1: TQ_LN_LAUNCH(1); break;
    case 2: TQ_LN_LAUNCH(2); break;
    case 4: TQ_LN_LAUNCH(4); break;
    case 8: TQ_LN_LAUNCH(8); break;
    default: TQ_LN_LAUNCH(16); break;
  }
#undef TQ_LN_LAUNCH
  TQ_LAUNCH_CHECK();
  return 0;
}

// out[t][i] = o[t][i] / sqrt(mean_i(o[t][i]^2) + eps) * w[i] * sigmoid(gate[t][i]) over all N = H V numbers of a token,
// in the activation type; the gate's row of token t at gate + t * ldg.  A workgroup a token.
template <class W>
__global__ __launch_bounds__(256) void lightning_out_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                            int64_t ldg, const W* __restrict__ w, float eps,
                                                            act_t* __restrict__ out, int N) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* row = o + (size_t)t * N;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += 256) ss = fmaf(row[i], row[i], ss);
  ss = block_sum(ss, red);
  const float rs = 1.0f / sqrtf(ss / (float)N + eps);
  const float* g = gate + (size_t)t * ldg;
  for (int i = threadIdx.x; i < N; i += 256)
    out[(size_t)t * N + i] = from_f32<act_t>(row[i] * rs * to_f32(w[i]) * (1.0f / (1.0f + expf(-g[i]))));
}

TQ_API int tq_lightning_out(const float* o, const float* gate, int64_t ldg, const void* w, int wtype, float eps, void* out,
                            int T, int N, hipStream_t st) {
  if (T <= 0) return 0;
  if (N < 1 || ldg < N || !w || !gate) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(lightning_out_kernel<W>, dim3(T), dim3(256), 0, st, o, gate, ldg, (const W*)w, eps, (act_t*)out, N);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}
