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
// Two kernels, for short runs and for decoding (a decoded token is a run of one; long runs: the chunked form below):
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

// ------------------------------------------------------------------------------------------ long runs, in chunks
// The same recurrence over chunks of LC_T tokens on the matrix cores (v_mfma_f32_16x16x4_f32: float operands as they
// are, on both libraries).  With S_c the state before chunk c, n its number of tokens and t, s counted from its start:
//   o_t     = sum_{s <= t} decay^(t - s) (q_t . k_s) v_s  +  decay^(t + 1) S_c^T q_t
//   S_(c+1) = decay^n S_c + L_c,   L_c = sum_s decay^(n - 1 - s) k_s v_s^T
// Three launches: every chunk's L_c (chunks side by side), the states before the chunks (per element of the state, over a
// sequence's chunks in order; the sequence's row of state is read first and written last), every chunk's read-outs.
// Chunks start at the first token that the step brings for a sequence.  Chunk c of sequence b is number
// sum_{b' < b} ceil(n_b' / LC_T) + c in the scratch array, which holds H D V floats a chunk.
#define LC_T 64        // tokens of a chunk
#define LC_V 64        // value channels of a workgroup
#define LC_VLD 80      // floats between two tokens' value channels in LDS

typedef float lc_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int lc_chunk_base(const int* __restrict__ cu_seqlens, int b) {
  int base = 0;
  for (int i = 0; i < b; ++i) base += (cu_seqlens[i + 1] - cu_seqlens[i] + LC_T - 1) / LC_T;
  return base;
}

// A chunk's rows of one projection on their way into LDS: first every load (all in flight together), then the silu and
// the stores.  W numbers a row (WP in LDS, a multiple of 16; zeros behind W and behind the chunk's nc tokens).  VEC: rows
// start at multiples of 16 bytes and W is a multiple of four.
template <int WP, bool VEC>
struct LcRows {
  static constexpr int N = VEC ? LC_T * WP / 4 / 256 : LC_T * WP / 256;
  float x[VEC ? 4 * N : N];
  __device__ __forceinline__ void fetch(const float* __restrict__ src, int64_t ld, int nc, int W, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + 256 * i;
      if (VEC) {
        const int s = idx / (WP / 4), d = 4 * (idx % (WP / 4));
        const float4 v = s < nc && d < W ? *reinterpret_cast<const float4*>(src + (size_t)s * ld + d) : float4{0.f, 0.f, 0.f, 0.f};
        x[4 * i] = v.x, x[4 * i + 1] = v.y, x[4 * i + 2] = v.z, x[4 * i + 3] = v.w;
      } else {
        const int s = idx / WP, d = idx % WP;
        x[i] = s < nc && d < W ? src[(size_t)s * ld + d] : 0.f;
      }
    }
  }
  // dst[s * ld + d] = silu(x) * (wt ? wt[s] : 1)
  __device__ __forceinline__ void store(float* __restrict__ dst, int ld, const float* __restrict__ wt, int tid) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + 256 * i;
      if (VEC) {
        const int s = idx / (WP / 4), d = 4 * (idx % (WP / 4));
        const float w = wt ? wt[s] : 1.f;
        *reinterpret_cast<float4*>(dst + s * ld + d) =
            float4{w * ln_silu(x[4 * i]), w * ln_silu(x[4 * i + 1]), w * ln_silu(x[4 * i + 2]), w * ln_silu(x[4 * i + 3])};
      } else {
        const int s = idx / WP, d = idx % WP;
        dst[s * ld + d] = (wt ? wt[s] : 1.f) * ln_silu(x[i]);
      }
    }
  }
};

// grid (ceil(V / LC_V), H, B * NC), block 256: L_c [D][LC_V columns] = K^T (w . V), a wave to 16 value channels.
template <int ND, bool VEC>
__global__ __launch_bounds__(256) void lightning_chunk_state_kernel(const float* __restrict__ P, int64_t ldp,
                                                                    const float* __restrict__ decay,
                                                                    const int* __restrict__ cu_seqlens, int NC, int cap,
                                                                    int H, int D, int V, float* __restrict__ L) {
  extern __shared__ __align__(16) float lc_lds[];
  constexpr int DP = 16 * ND, KLD = DP + (80 - DP % 64) % 64;
  float* ks = lc_lds;                    // [LC_T][KLD]
  float* vs = ks + LC_T * KLD;           // [LC_T][LC_VLD], each token's values times its weight
  float* wt = vs + LC_T * LC_VLD;        // [LC_T]
  const int b = blockIdx.z / NC, c = blockIdx.z % NC, h = blockIdx.y, v0 = blockIdx.x * LC_V;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
  if (c * LC_T >= n) return;
  const int gi = lc_chunk_base(cu_seqlens, b) + c;
  if (gi >= cap) return;
  const int nc = min(LC_T, n - c * LC_T), tid = threadIdx.x;
  const float lam = decay[h];
  if (tid < LC_T) wt[tid] = tid < nc ? powf(lam, (float)(nc - 1 - tid)) : 0.f;
  const float* k0 = P + (size_t)(t0 + c * LC_T) * ldp + (size_t)H * D + (size_t)h * D;
  const float* vv0 = P + (size_t)(t0 + c * LC_T) * ldp + (size_t)2 * H * D + (size_t)h * V + v0;
  LcRows<DP, VEC> kr_;
  LcRows<LC_V, VEC> vr_;
  kr_.fetch(k0, ldp, nc, D, tid);
  vr_.fetch(vv0, ldp, nc, V - v0, tid);
  kr_.store(ks, KLD, nullptr, tid);
  __syncthreads();
  vr_.store(vs, LC_VLD, wt, tid);
  __syncthreads();
  const int wave = tid / 64, lane = tid % 64, g = lane / 16, r = lane % 16;
  lc_f32x4 acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = lc_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k4 = 0; k4 < LC_T / 4; ++k4) {
    const float bv = vs[(4 * k4 + g) * LC_VLD + 16 * wave + r];
    const float* kr = ks + (4 * k4 + g) * KLD + r;
#pragma unroll
    for (int rt = 0; rt < ND; ++rt) acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(kr[16 * rt], bv, acc[rt], 0, 0, 0);
  }
  const int v = v0 + 16 * wave + r;
  if (v < V) {
    float* out = L + ((size_t)gi * H + h) * D * V + v;
#pragma unroll
    for (int rt = 0; rt < ND; ++rt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 16 * rt + 4 * g + i;
        if (d < D) out[(size_t)d * V] = acc[rt][i];
      }
  }
}

// grid (ceil(D V / 256), H, B), block 256: L_c becomes S_c in place, chunk by chunk; the row of state is advanced.
__global__ __launch_bounds__(256) void lightning_chunk_prefix_kernel(const float* __restrict__ decay,
                                                                     const int* __restrict__ cu_seqlens,
                                                                     const int* __restrict__ slots, float* __restrict__ state,
                                                                     int64_t state_stride, int cap, int H, int D, int V,
                                                                     float* __restrict__ L) {
  const int b = blockIdx.z, h = blockIdx.y;
  const int e = blockIdx.x * 256 + threadIdx.x;
  const int n = cu_seqlens[b + 1] - cu_seqlens[b];
  if (n <= 0 || e >= D * V) return;
  const int base = lc_chunk_base(cu_seqlens, b), chunks = (n + LC_T - 1) / LC_T;
  if (base + chunks > cap) return;
  const float lam = decay[h];
  const float full = powf(lam, (float)LC_T), last = powf(lam, (float)(n - (chunks - 1) * LC_T));
  float* srow = state + (size_t)slots[b] * state_stride + (size_t)h * D * V + e;
  float carry = *srow;
  float* at = L + ((size_t)base * H + h) * D * V + e;
  for (int c = 0; c < chunks; ++c, at += (size_t)H * D * V) {
    const float own = *at;
    *at = carry;
    carry = fmaf(c + 1 < chunks ? full : last, carry, own);
  }
  *srow = carry;
}

// grid (ceil(V / LC_V), H, B * NC), block 256: a chunk's read-outs for LC_V value channels, a wave to 16 tokens.
template <int ND, bool VEC>
__global__ __launch_bounds__(256) void lightning_chunk_out_kernel(const float* __restrict__ P, int64_t ldp,
                                                                  const float* __restrict__ decay,
                                                                  const int* __restrict__ cu_seqlens, int NC, int cap,
                                                                  int H, int D, int V, const float* __restrict__ S,
                                                                  float* __restrict__ o) {
  extern __shared__ __align__(16) float lc_lds[];
  constexpr int DP = 16 * ND, QLD = DP + 4, PLD = LC_T + 4, KROWS = QLD > PLD ? QLD : PLD;
  float* qs = lc_lds;                    // [LC_T][QLD]
  float* ks = qs + LC_T * QLD;           // [LC_T][QLD]; later the weighted scores [LC_T][PLD]
  float* vs = ks + LC_T * KROWS;         // [LC_T][LC_VLD]
  float* pw = vs + LC_T * LC_VLD;        // decay^j, j = 0 .. LC_T
  const int b = blockIdx.z / NC, c = blockIdx.z % NC, h = blockIdx.y, v0 = blockIdx.x * LC_V;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0;
  if (c * LC_T >= n) return;
  const int gi = lc_chunk_base(cu_seqlens, b) + c;
  if (gi >= cap) return;
  const int nc = min(LC_T, n - c * LC_T), tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64, g = lane / 16, r = lane % 16;
  // the state before the chunk, as the last product's operand: asked for first, so that it arrives while the rest is staged
  constexpr int AHEAD = DP / 4 > 32 ? 32 : DP / 4;
  const float* sb = S + ((size_t)gi * H + h) * D * V + v0 + r;
  float sv[AHEAD][4];
#pragma unroll
  for (int k4 = 0; k4 < AHEAD; ++k4)
#pragma unroll
    for (int cv = 0; cv < 4; ++cv)
      sv[k4][cv] = 4 * k4 + g < D && v0 + 16 * cv + r < V ? sb[(size_t)(4 * k4 + g) * V + 16 * cv] : 0.f;
  const float lam = decay[h];
  if (tid <= LC_T) pw[tid] = powf(lam, (float)tid);
  const float* q0 = P + (size_t)(t0 + c * LC_T) * ldp + (size_t)h * D;
  const float* k0 = q0 + (size_t)H * D;
  const float* vv0 = P + (size_t)(t0 + c * LC_T) * ldp + (size_t)2 * H * D + (size_t)h * V + v0;
  {
    LcRows<DP, VEC> qr_, kr_;
    LcRows<LC_V, VEC> vr_;
    qr_.fetch(q0, ldp, nc, D, tid);
    kr_.fetch(k0, ldp, nc, D, tid);
    vr_.fetch(vv0, ldp, nc, V - v0, tid);
    qr_.store(qs, QLD, nullptr, tid);
    kr_.store(ks, QLD, nullptr, tid);
    vr_.store(vs, LC_VLD, nullptr, tid);
  }
  __syncthreads();
  // scores of the wave's 16 tokens against the tokens of the column tiles up to its own
  lc_f32x4 sc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) sc[i] = lc_f32x4{0.f, 0.f, 0.f, 0.f};
  const float* qrow = qs + (16 * wave + r) * QLD + g;
#pragma unroll 4
  for (int k4 = 0; k4 < DP / 4; ++k4) {
    const float a = qrow[4 * k4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
      if (ct <= wave) sc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, ks[(16 * ct + r) * QLD + 4 * k4 + g], sc[ct], 0, 0, 0);
  }
  __syncthreads();                        // every wave has read the keys: their place takes the weighted scores
  float* ps = ks;
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
    if (ct <= wave)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * wave + 4 * g + i, s = 16 * ct + r;
        ps[t * PLD + s] = s <= t ? sc[ct][i] * pw[t - s] : 0.f;
      }
  __syncthreads();
  lc_f32x4 acc[4], far[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = far[i] = lc_f32x4{0.f, 0.f, 0.f, 0.f};
  const float* prow = ps + (16 * wave + r) * PLD + g;
  for (int k4 = 0; k4 < 4 * (wave + 1); ++k4) {
    const float a = prow[4 * k4];
    const float* vr = vs + (4 * k4 + g) * LC_VLD + r;
#pragma unroll
    for (int cv = 0; cv < 4; ++cv) acc[cv] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vr[16 * cv], acc[cv], 0, 0, 0);
  }
  // what the state before the chunk adds: q S, each row times decay^(t + 1)
#pragma unroll
  for (int k4 = 0; k4 < AHEAD; ++k4) {
    const float a = qrow[4 * k4];
#pragma unroll
    for (int cv = 0; cv < 4; ++cv) far[cv] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, sv[k4][cv], far[cv], 0, 0, 0);
  }
#pragma unroll 8
  for (int k4 = AHEAD; k4 < DP / 4; ++k4) {
    const float a = qrow[4 * k4];
    const int d = 4 * k4 + g;
#pragma unroll
    for (int cv = 0; cv < 4; ++cv) {
      const float bv = d < D && v0 + 16 * cv + r < V ? sb[(size_t)d * V + 16 * cv] : 0.f;
      far[cv] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bv, far[cv], 0, 0, 0);
    }
  }
#pragma unroll
  for (int cv = 0; cv < 4; ++cv) {
    const int v = v0 + 16 * cv + r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 16 * wave + 4 * g + i;
      if (t < nc && v < V) o[(size_t)(t0 + c * LC_T + t) * H * V + (size_t)h * V + v] = fmaf(pw[t + 1], far[cv][i], acc[cv][i]);
    }
  }
}

template <int ND, bool VEC>
static int lightning_chunked_launch(const float* P, int64_t ldp, const float* decay, const int* cu_seqlens, const int* slots,
                                    float* state, int64_t state_stride, int B, int NC, int cap, int H, int D, int V,
                                    float* scratch, float* o, hipStream_t st) {
  constexpr int DP = 16 * ND, KLD = DP + (80 - DP % 64) % 64, QLD = DP + 4, KROWS = QLD > LC_T + 4 ? QLD : LC_T + 4;
  const size_t sh_state = ((size_t)LC_T * KLD + (size_t)LC_T * LC_VLD + LC_T) * sizeof(float);
  const size_t sh_out = ((size_t)LC_T * QLD + (size_t)LC_T * KROWS + (size_t)LC_T * LC_VLD + LC_T + 4) * sizeof(float);
  if (sh_state > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)lightning_chunk_state_kernel<ND, VEC>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)sh_state);
  if (sh_out > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)lightning_chunk_out_kernel<ND, VEC>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)sh_out);
  const dim3 grid((V + LC_V - 1) / LC_V, H, B * NC);
  hipLaunchKernelGGL((lightning_chunk_state_kernel<ND, VEC>), grid, dim3(256), sh_state, st, P, ldp, decay, cu_seqlens, NC, cap, H,
                     D, V, scratch);
  hipLaunchKernelGGL(lightning_chunk_prefix_kernel, dim3((D * V + 255) / 256, H, B), dim3(256), 0, st, decay, cu_seqlens, slots,
                     state, state_stride, cap, H, D, V, scratch);
  hipLaunchKernelGGL((lightning_chunk_out_kernel<ND, VEC>), grid, dim3(256), sh_out, st, P, ldp, decay, cu_seqlens, NC, cap, H, D,
                     V, scratch, o);
  TQ_LAUNCH_CHECK();
  return 0;
}

// As tq_lightning_scan, for steps with long runs: max_new is the longest run's number of tokens, scratch holds
// scratch_chunks * H D V floats with scratch_chunks >= sum_b ceil(n_b / 64) (T / 64 + B is always enough).
TQ_API int tq_lightning_chunked(const float* P, int64_t ldp, const float* decay, const int* cu_seqlens, const int* slots,
                                float* state, int64_t state_stride, int B, int H, int D, int V, int max_new, float* scratch,
                                int scratch_chunks, float* o, hipStream_t st) {
  if (B <= 0 || max_new <= 0) return 0;
  if (H < 1 || D < 1 || V < 1 || ldp < (int64_t)2 * H * D + (int64_t)2 * H * V || state_stride < (int64_t)H * D * V ||
      !scratch || scratch_chunks < 1)
    return TQ_ERR_BAD_ARG;
  const int NC = (max_new + LC_T - 1) / LC_T;
  if (D > 256 || H > 65535 || (int64_t)B * NC > 65535 || (int64_t)D * V > (int64_t)256 * 65535) return TQ_ERR_UNSUPPORTED;
  // whole rows of four floats: every row of every head starts at a multiple of 16 bytes
  const bool vec = D % 4 == 0 && V % 4 == 0 && ldp % 4 == 0 && (uintptr_t)P % 16 == 0;
#define TQ_LC(NDV)                                                                                                        \
  return vec ? lightning_chunked_launch<NDV, true>(P, ldp, decay, cu_seqlens, slots, state, state_stride, B, NC,          \
                                                   scratch_chunks, H, D, V, scratch, o, st)                               \
             : lightning_chunked_launch<NDV, false>(P, ldp, decay, cu_seqlens, slots, state, state_stride, B, NC,         \
                                                    scratch_chunks, H, D, V, scratch, o, st)
  if (D <= 16) TQ_LC(1);
  if (D <= 32) TQ_LC(2);
  if (D <= 64) TQ_LC(4);
  if (D <= 128) TQ_LC(8);
  TQ_LC(16);
#undef TQ_LC
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
