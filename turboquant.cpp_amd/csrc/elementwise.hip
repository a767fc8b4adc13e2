// Row-wise kernels: embedding rows, residual sum + RMS norm, rotary position encoding with
// the write of keys and values into cache pages, and the weighted sum of expert outputs.
// All of them are bound by memory traffic; each fuses what would otherwise be a second pass.
#include "common.h"

// ---------------------------------------------------------------- embedding
// x[t, :] = table[tokens[t], :] widened to float; no scaling for this architecture
// (/root/reference/src/engine/tq_transformer.c:2297-2329); `scale` other than 1 multiplies the row, for the
// architectures that scale their embeddings (tq_transformer.c:2332).
template <class W>
__global__ void embed_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                             float* __restrict__ x, int H, float scale) {
  const int t = blockIdx.x;
  const W* row = table + (size_t)tokens[t] * H;
  float* out = x + (size_t)t * H;
  if (scale == 1.0f) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32(row[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32(row[i]) * scale;
  }
}

TQ_API int tq_embed(const int* tokens, const void* table, int wtype, float* x, int T, int H, float scale, hipStream_t st) {
  if (T <= 0) return 0;
  TQ_DISPATCH_W(wtype, { hipLaunchKernelGGL(embed_kernel<W>, dim3(T), dim3(256), 0, st, tokens, (const W*)table, x, H, scale); });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a soft cap on logits
// x <- cap * tanh(x / cap), in place: what a model plan may ask for between the vocabulary product and sampling.
__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// x <- x * scale, then (cap > 0) x <- cap * tanh(x / cap): logits that a model multiplies by a constant before it caps them.
__global__ void scale_softcap_kernel(float* __restrict__ x, int64_t n, float scale, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = x[i] * scale;
  x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

TQ_API int tq_scale_softcap(float* x, int64_t n, float scale, float cap, hipStream_t st) {
  if (n <= 0) return 0;
  if (cap < 0.f) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, n, scale, cap);
  TQ_LAUNCH_CHECK();
  return 0;
}

TQ_API int tq_softcap(float* x, int64_t n, float cap, hipStream_t st) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return TQ_ERR_BAD_ARG;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, n, cap);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- rows by index
// The rows of a sequence's fixed-size state lie at its slot; a step works on the rows of its own sequences.
// gather: dst[i] = src[idx[i]];  scatter: dst[idx[i]] = src[i];  rows of `words` 32-bit words.  grid (rows, chunks).
__global__ void move_rows_kernel(const uint32_t* __restrict__ src, const int* __restrict__ idx, uint32_t* __restrict__ dst,
                                 int64_t words, int scatter) {
  const int64_t row = blockIdx.x, at = idx[row];
  const uint32_t* from = src + (scatter ? row : at) * words;
  uint32_t* to = dst + (scatter ? at : row) * words;
  for (int64_t w = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; w < words; w += (int64_t)gridDim.y * blockDim.x) to[w] = from[w];
}

// src, dst: rows of row_bytes bytes (a multiple of 4); idx [n]: for gather the row of src behind each row of dst, for
// scatter the row of dst that each row of src goes to (every index once).
TQ_API int tq_move_rows(const void* src, const int* idx, void* dst, int n, int64_t row_bytes, int scatter, hipStream_t st) {
  if (n <= 0 || row_bytes <= 0) return 0;
  if (row_bytes % 4 != 0 || n > 65535 * 32768) return TQ_ERR_UNSUPPORTED;
  const int64_t words = row_bytes / 4;
  const int chunks = (int)((words + 1023) / 1024 < 1024 ? (words + 1023) / 1024 : 1024);
  hipLaunchKernelGGL(move_rows_kernel, dim3(n, chunks), dim3(256), 0, st, (const uint32_t*)src, idx, (uint32_t*)dst, words, scatter);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- residual sum + RMS norm
// For row r (token rows[r], or r itself when rows is null):
//   v = x[row] + d[row]                         (the residual sum, in float)
//   x[row] = v                                  (only when rows is null)
//   ss = sum v^2 / H + eps ; out = (v * (1/sqrt(ss))) * w
// Formula and product order of /root/reference/src/engine/tq_ops.c:1373-1410.  What is added, d, is either
//   the partial sums delta[s][row] one after the other, s ascending (each added to v in turn), or, with y set,
//   the experts' outputs that nobody has summed yet, as moe_combine below would:
//   d = sum_j weights[row][j] * y[pair_slot[row][j]] (j ascending) + gate[row] * sum_s delta[s][row].
// The sum of squares is taken in a fixed order that does not depend on the number of rows.
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 load4f(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4f(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
               __uint_as_float(u.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
  uint2 u;
  u.x = (uint32_t)f32_to_bf16(v.x).bits | ((uint32_t)f32_to_bf16(v.y).bits << 16);
  u.y = (uint32_t)f32_to_bf16(v.z).bits | ((uint32_t)f32_to_bf16(v.w).bits << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// A thread takes four consecutive elements at a time when H is a multiple of four (every load is 16 bytes and
// all of a thread's loads can be on their way at once), else one element at a time; what is computed per
// element is the same.
template <class W>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ delta, int S,
                                   size_t delta_stride, const float* __restrict__ y,
                                   const int* __restrict__ pair_slot, const float* __restrict__ weights, int topk,
                                   const float* __restrict__ gate, const W* __restrict__ w, float eps,
                                   const int* __restrict__ rows, act_t* __restrict__ out,
                                   float* __restrict__ out32, int H) {
  extern __shared__ __attribute__((aligned(16))) float v[];       // H floats, then one float per wave
  __shared__ int slot[64];
  __shared__ float wgt[64];
  float* red = v + (H + 3) / 4 * 4;
  const int r = blockIdx.x;
  const int row = rows ? rows[r] : r;
  float* xr = x + (size_t)row * H;
  const float* dr = delta + (size_t)row * H;
  float g = 1.0f;
  if (y) {
    if (threadIdx.x < topk) {      // the token's rows and weights once, not once per element
      slot[threadIdx.x] = pair_slot[(size_t)row * topk + threadIdx.x];
      wgt[threadIdx.x] = weights[(size_t)row * topk + threadIdx.x];
    }
    if (gate) g = gate[row];
    __syncthreads();
  }
  const bool vec = H % 4 == 0;
  float ss = 0.f;
  if (vec) {
#pragma unroll 2
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      // the terms are fetched four at a time and added in their order: the loads of a group are on their way
      // together instead of one after the other
      f32x4 a = load4f(xr + i);
      if (y) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < topk; j += 4) {
          f32x4 t[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (j + u < topk) t[u] = slot[j + u] < 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : load4f(y + (size_t)slot[j + u] * H + i);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (j + u < topk) acc += wgt[j + u] * t[u];
        }
        if (S > 0) {
          f32x4 sh = {0.f, 0.f, 0.f, 0.f};
          for (int s = 0; s < S; s += 4) {
            f32x4 t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
              if (s + u < S) t[u] = load4f(dr + (s + u) * delta_stride + i);
#pragma unroll
            for (int u = 0; u < 4; ++u)
              if (s + u < S) sh += t[u];
          }
          acc += g * sh;
        }
        a += acc;
      } else {
        for (int s = 0; s < S; s += 4) {
          f32x4 t[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s + u < S) t[u] = load4f(dr + (s + u) * delta_stride + i);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s + u < S) a += t[u];
        }
      }
      store4(v + i, a);
      if (!rows) store4(xr + i, a);
      ss += a.x * a.x;
      ss += a.y * a.y;
      ss += a.z * a.z;
      ss += a.w * a.w;
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float a = xr[i];
      if (y) {
        float acc = 0.f;
        for (int j = 0; j < topk; ++j)
          if (slot[j] >= 0) acc += wgt[j] * y[(size_t)slot[j] * H + i];      // (-1: a pair without a row)
        if (S > 0) {
          float sh = 0.f;
          for (int s = 0; s < S; ++s) sh += dr[s * delta_stride + i];
          acc += g * sh;
        }
        a += acc;
      } else {
        for (int s = 0; s < S; ++s) a += dr[s * delta_stride + i];
      }
      v[i] = a;
      if (!rows) xr[i] = a;
      ss += a * a;
    }
  }
  ss = block_sum(ss, red);
  ss = ss / (float)H + eps;
  const float rs = 1.0f / sqrtf(ss);
  if (vec) {
#pragma unroll 2
    for (int i = threadIdx.x * 4; i < H; i += blockDim.x * 4) {
      const f32x4 o = load4f(v + i) * rs * load4f(w + i);
      if (out) store4(out + (size_t)r * H + i, o);
      if (out32) store4(out32 + (size_t)r * H + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float o = v[i] * rs * to_f32(w[i]);
      if (out) out[(size_t)r * H + i] = from_f32<act_t>(o);
      if (out32) out32[(size_t)r * H + i] = o;
    }
  }
}

TQ_API int tq_add_rmsnorm(float* x, const float* delta, int S, int64_t delta_stride, const float* y,
                          const int* pair_slot, const float* weights, int topk, const float* gate, const void* w,
                          int wtype, float eps, const int* rows, int R, void* out, float* out32, int H,
                          hipStream_t st) {
  if (R <= 0) return 0;
  if (y && (topk < 1 || topk > 64 || !pair_slot || !weights)) return TQ_ERR_BAD_ARG;
  // a row of 2,048 and more by 512 threads, so that each takes its four elements in one go and all of a row's loads
  // are on their way at once (a function of H alone: a row's sums do not depend on what else the step holds)
  const int threads = (H % 4 == 0 && H >= 2048) ? 512 : 256;
  const size_t shmem = (size_t)((H + 3) / 4 * 4 + threads / TQ_WAVE) * sizeof(float);
  if (shmem > 150 * 1024) return TQ_ERR_UNSUPPORTED;
  TQ_DISPATCH_W(wtype, {
    if (shmem > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)add_rmsnorm_kernel<W>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    hipLaunchKernelGGL(add_rmsnorm_kernel<W>, dim3(R), dim3(threads), shmem, st, x, delta, S, (size_t)delta_stride, y,
                       pair_slot, weights, topk, gate, (const W*)w, eps, rows, (act_t*)out, out32, H);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// The limit of gated pairs that the next launches of products and of gated_act take (common.h: gated_pair); 0: none.
float tq_pair_limit_host = 0.f;
TQ_API int tq_set_pair_limit(float limit) {
  if (!(limit >= 0.f)) return TQ_ERR_BAD_ARG;
  tq_pair_limit_host = limit;
  return 0;
}

// ---------------------------------------------------------------- the gate of a gated pair, applied afterwards
// out[m][n] = f(gu[m][n]) * gu[m][N + n]: for a pair of products that came out of one plain product over the two
// matrices laid one behind the other (a library's, which has no such epilogue).  gu is float32 with row stride ld.
// (the general form: the gate's rows at g with stride ldg, the other factor's at u with stride ldu; u null: out = f(g)
// alone, an activation behind a plain product; gate < 0: f is the identity, a change of type)
template <bool VEC>
__global__ __launch_bounds__(256) void gated_act_kernel(const float* __restrict__ gp, int64_t ldg, const float* __restrict__ up,
                                                        int64_t ldu, act_t* __restrict__ out, int N, int gate,
                                                        float limit) {
  const float* row = gp + (size_t)blockIdx.y * ldg;
  const float* urow = up ? up + (size_t)blockIdx.y * ldu : nullptr;
  act_t* dst = out + (size_t)blockIdx.y * N;
  if (VEC) {
    const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= N) return;
    f32x4 g = load4f(row + n);
    if (gate >= 0 && urow && limit > 0.f) {
      const f32x4 u = load4f(urow + n);
      g = f32x4{gated_pair(g.x, u.x, gate, limit), gated_pair(g.y, u.y, gate, limit), gated_pair(g.z, u.z, gate, limit),
                gated_pair(g.w, u.w, gate, limit)};
    } else {
      if (gate >= 0) g = f32x4{gate_fn(g.x, gate), gate_fn(g.y, gate), gate_fn(g.z, gate), gate_fn(g.w, gate)};
      if (urow) g *= load4f(urow + n);
    }
    store4(dst + n, g);
  } else {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    float g = row[n];
    if (gate >= 0 && urow && limit > 0.f) {
      g = gated_pair(g, urow[n], gate, limit);
    } else {
      if (gate >= 0) g = gate_fn(g, gate);
      if (urow) g *= urow[n];
    }
    dst[n] = from_f32<act_t>(g);
  }
}

static int launch_gated_act(const float* g, int64_t ldg, const float* u, int64_t ldu, void* out, int M, int N, int gate,
                            hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (gate >= TQ_GATE_COUNT || ldg < N || (u && ldu < N)) return TQ_ERR_BAD_ARG;
  if (M > 65535) return TQ_ERR_UNSUPPORTED;
  const bool vec = N % 4 == 0 && ldg % 4 == 0 && ((uintptr_t)g % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                   (!u || (ldu % 4 == 0 && ((uintptr_t)u % 16) == 0));
  if (vec)
    hipLaunchKernelGGL(gated_act_kernel<true>, dim3((N / 4 + 255) / 256, M), dim3(256), 0, st, g, ldg, u, ldu, (act_t*)out, N, gate,
                       tq_pair_limit_host);
  else
    hipLaunchKernelGGL(gated_act_kernel<false>, dim3((N + 255) / 256, M), dim3(256), 0, st, g, ldg, u, ldu, (act_t*)out, N, gate,
                       tq_pair_limit_host);
  TQ_LAUNCH_CHECK();
  return 0;
}

TQ_API int tq_gated_act(const float* gu, int64_t ld, void* out, int M, int N, int gate, hipStream_t st) {
  if (gate < 0 || ld < 2 * (int64_t)N) return TQ_ERR_BAD_ARG;
  return launch_gated_act(gu, ld, gu + N, ld, out, M, N, gate, st);
}

// out[m][n] = f(g[m][n]) * u[m][n] in the activation type, with rows of g and u at strides of their own; u null:
// f(g) alone; gate < 0: no activation (with u null: the rows of g in the activation type).
TQ_API int tq_act_rows(const float* g, int64_t ldg, const float* u, int64_t ldu, void* out, int M, int N, int gate,
                       hipStream_t st) {
  for (int r = 0; r < M; r += 65535) {          // the grid's y takes 65,535 rows at a time
    const int rows = M - r < 65535 ? M - r : 65535;
    const int rc = launch_gated_act(g + (size_t)r * ldg, ldg, u ? u + (size_t)r * ldu : nullptr, ldu,
                                    (act_t*)out + (size_t)r * N, rows, N, gate, st);
    if (rc) return rc;
  }
  return 0;
}

// out[m][n] = f(gate[m][n]) * o[m][n]: an output gate on rows that are already in the activation type (an attention's
// heads), the gate float with a row stride of its own.  In place if out == o.
__global__ __launch_bounds__(256) void gate_rows_kernel(const act_t* __restrict__ o, const float* __restrict__ gate, int64_t ldg,
                                                        act_t* __restrict__ out, int N, int kind) {
  const int m = blockIdx.y;
  for (int n = blockIdx.x * 256 + threadIdx.x; n < N; n += gridDim.x * 256)
    out[(size_t)m * N + n] = from_f32<act_t>(to_f32(o[(size_t)m * N + n]) * gate_fn(gate[(size_t)m * ldg + n], kind));
}

TQ_API int tq_gate_rows(const void* o, const float* gate, int64_t ldg, void* out, int M, int N, int kind, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (kind < 0 || kind >= TQ_GATE_COUNT || ldg < N) return TQ_ERR_BAD_ARG;
  for (int r = 0; r < M; r += 65535) {
    const int rows = M - r < 65535 ? M - r : 65535;
    hipLaunchKernelGGL(gate_rows_kernel, dim3((N + 1023) / 1024 < 1 ? 1 : (N + 1023) / 1024, rows), dim3(256), 0, st,
                       (const act_t*)o + (size_t)r * N, gate + (size_t)r * ldg, ldg, (act_t*)out + (size_t)r * N, N, kind);
  }
  TQ_LAUNCH_CHECK();
  return 0;
}

// out[m][h hd + i] = f(gate[m][h]) * o[m][h hd + i]: one number per head and token gates the head's whole output.
__global__ __launch_bounds__(256) void gate_heads_kernel(const act_t* __restrict__ o, const float* __restrict__ gate, int64_t ldg,
                                                         act_t* __restrict__ out, int heads, int hd, int kind) {
  const int m = blockIdx.y, N = heads * hd;
  for (int n = blockIdx.x * 256 + threadIdx.x; n < N; n += gridDim.x * 256)
    out[(size_t)m * N + n] = from_f32<act_t>(to_f32(o[(size_t)m * N + n]) * gate_fn(gate[(size_t)m * ldg + n / hd], kind));
}

TQ_API int tq_gate_heads(const void* o, const float* gate, int64_t ldg, void* out, int M, int heads, int hd, int kind,
                         hipStream_t st) {
  if (M <= 0 || heads <= 0 || hd <= 0) return 0;
  if (kind < 0 || kind >= TQ_GATE_COUNT || ldg < heads) return TQ_ERR_BAD_ARG;
  const int N = heads * hd;
  for (int r = 0; r < M; r += 65535) {
    const int rows = M - r < 65535 ? M - r : 65535;
    hipLaunchKernelGGL(gate_heads_kernel, dim3((N + 1023) / 1024 < 1 ? 1 : (N + 1023) / 1024, rows), dim3(256), 0, st,
                       (const act_t*)o + (size_t)r * N, gate + (size_t)r * ldg, ldg, (act_t*)out + (size_t)r * N, heads, hd, kind);
  }
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- RMS norm of a run of columns, written several times
// out[t][c * Rp + i] = in[t][i] / sqrt(mean_i(in[t][i]^2) + eps) * w[i] for i < R, 0 for R <= i < Rp, for the copies
// c = 0 .. copies - 1: the normed latent of an attention that keeps one compressed row per position, laid where the
// cache write expects a key row and a value row (both are that latent), padded to the kernels' width.  A wave a token.
template <class W>
__global__ __launch_bounds__(256) void latent_norm_kernel(const float* __restrict__ in, int64_t ld_in, const W* __restrict__ w,
                                                          float eps, float* __restrict__ out, int64_t ld_out, int copies,
                                                          int R, int Rp, int T) {
  const int t = blockIdx.x * 4 + threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  if (t >= T) return;
  const float* row = in + (size_t)t * ld_in;
  float ss = 0.f;
  for (int i = lane; i < R; i += TQ_WAVE) ss += row[i] * row[i];
  ss = wave_sum(ss);
  const float rs = 1.0f / sqrtf(ss / (float)R + eps);
  for (int i = lane; i < Rp; i += TQ_WAVE) {
    const float v = i < R ? row[i] * rs * to_f32(w[i]) : 0.f;
    for (int c = 0; c < copies; ++c) out[(size_t)t * ld_out + (size_t)c * Rp + i] = v;
  }
}

TQ_API int tq_latent_norm(const float* in, int64_t ld_in, const void* w, int wtype, float eps, float* out, int64_t ld_out,
                          int copies, int R, int Rp, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (R < 1 || Rp < R || copies < 1 || ld_in < R || ld_out < (int64_t)copies * Rp || !w) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(latent_norm_kernel<W>, dim3((T + 3) / 4), dim3(256), 0, st, in, ld_in, (const W*)w, eps, out, ld_out,
                       copies, R, Rp, T);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// The same with `lead` columns that are not normed: in[t][R .. R + lead) pass as they are and come first in every copy,
// out[t][c * Rp + i] = in[t][R + i] for i < lead, the normed in[t][i - lead] for lead <= i < lead + R, 0 up to Rp (a
// latent whose row also carries a part of the key that is rotated later and shared by all heads).  OUT_ACT: the copies
// are written in the activation type (a normed row that feeds the next product).
template <class W, class O>
__global__ __launch_bounds__(256) void lead_norm_kernel(const float* __restrict__ in, int64_t ld_in, const W* __restrict__ w,
                                                        float eps, O* __restrict__ out, int64_t ld_out, int copies, int R,
                                                        int lead, int Rp, int T) {
  const int t = blockIdx.x * 4 + threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  if (t >= T) return;
  const float* row = in + (size_t)t * ld_in;
  float ss = 0.f;
  for (int i = lane; i < R; i += TQ_WAVE) ss += row[i] * row[i];
  ss = wave_sum(ss);
  const float rs = 1.0f / sqrtf(ss / (float)R + eps);
  for (int i = lane; i < Rp; i += TQ_WAVE) {
    const float v = i < lead ? row[R + i] : i < lead + R ? row[i - lead] * rs * to_f32(w[i - lead]) : 0.f;
    for (int c = 0; c < copies; ++c) out[(size_t)t * ld_out + (size_t)c * Rp + i] = from_f32<O>(v);
  }
}

// The same for steps of a few tokens, a workgroup to a token: a wave alone walks a row of several hundred numbers in a
// dozen dependent rounds.
template <class W, class O>
__global__ __launch_bounds__(256) void lead_norm_few_kernel(const float* __restrict__ in, int64_t ld_in, const W* __restrict__ w,
                                                            float eps, O* __restrict__ out, int64_t ld_out, int copies, int R,
                                                            int lead, int Rp) {
  __shared__ float part[256 / TQ_WAVE];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* row = in + (size_t)t * ld_in;
  float ss = 0.f;
  for (int i = tid; i < R; i += 256) ss += row[i] * row[i];
  ss = wave_sum(ss);
  if (tid % TQ_WAVE == 0) part[tid / TQ_WAVE] = ss;
  __syncthreads();
  ss = 0.f;
#pragma unroll
  for (int i = 0; i < 256 / TQ_WAVE; ++i) ss += part[i];
  const float rs = 1.0f / sqrtf(ss / (float)R + eps);
  for (int i = tid; i < Rp; i += 256) {
    const float v = i < lead ? row[R + i] : i < lead + R ? row[i - lead] * rs * to_f32(w[i - lead]) : 0.f;
    for (int c = 0; c < copies; ++c) out[(size_t)t * ld_out + (size_t)c * Rp + i] = from_f32<O>(v);
  }
}

TQ_API int tq_lead_norm(const float* in, int64_t ld_in, const void* w, int wtype, float eps, void* out, int out_is_act,
                        int64_t ld_out, int copies, int R, int lead, int Rp, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (R < 1 || lead < 0 || Rp < R + lead || copies < 1 || ld_in < R + lead || ld_out < (int64_t)copies * Rp || !w)
    return TQ_ERR_BAD_ARG;
  if (T <= 32 && R > 2 * TQ_WAVE) {
    TQ_DISPATCH_W(wtype, {
      if (out_is_act)
        hipLaunchKernelGGL((lead_norm_few_kernel<W, act_t>), dim3(T), dim3(256), 0, st, in, ld_in, (const W*)w, eps,
                           (act_t*)out, ld_out, copies, R, lead, Rp);
      else
        hipLaunchKernelGGL((lead_norm_few_kernel<W, float>), dim3(T), dim3(256), 0, st, in, ld_in, (const W*)w, eps,
                           (float*)out, ld_out, copies, R, lead, Rp);
    });
    TQ_LAUNCH_CHECK();
    return 0;
  }
  TQ_DISPATCH_W(wtype, {
    if (out_is_act)
      hipLaunchKernelGGL((lead_norm_kernel<W, act_t>), dim3((T + 3) / 4), dim3(256), 0, st, in, ld_in, (const W*)w, eps,
                         (act_t*)out, ld_out, copies, R, lead, Rp, T);
    else
      hipLaunchKernelGGL((lead_norm_kernel<W, float>), dim3((T + 3) / 4), dim3(256), 0, st, in, ld_in, (const W*)w, eps,
                         (float*)out, ld_out, copies, R, lead, Rp, T);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- RMS norm of every head of q and k
// qkv[t] holds, in float, nh query heads, then nkv key heads, then nkv value heads of hd each.  Every query head is
// normed over its hd values with the weights wq[hd], every key head with wk[hd] (a null pointer leaves those heads
// as they are), in place: the per-head norm between the product and the rotation of
// /root/reference/src/engine/tq_transformer.c:1111-1124, with the formula of tq_ops.c:1373-1410.  A wave per head.
template <class W>
__global__ __launch_bounds__(256) void head_rmsnorm_kernel(float* __restrict__ qkv, const W* __restrict__ wq,
                                                           const W* __restrict__ wk, float eps, int nh, int nkv, int hd,
                                                           int norm_dim) {
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int head = blockIdx.y * 4 + wave;
  if (head >= nh + nkv) return;
  const W* w = head < nh ? wq : wk;
  if (!w) return;
  float* x = qkv + ((size_t)blockIdx.x * (nh + 2 * nkv) + head) * hd;
  float ss = 0.f;
  for (int i = lane; i < hd; i += TQ_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss) / (float)norm_dim + eps;      // (heads laid out wider than they are hold zeros behind their norm_dim values)
  const float rs = 1.0f / sqrtf(ss);
  for (int i = lane; i < hd; i += TQ_WAVE) x[i] = x[i] * rs * to_f32(w[i]);
}

TQ_API int tq_head_rmsnorm(float* qkv, const void* wq, const void* wk, int wtype, float eps, int T, int nh, int nkv,
                           int hd, int norm_dim, hipStream_t st) {
  if (T <= 0 || (!wq && !wk)) return 0;
  if (nh < 0 || nkv < 0 || hd < 1 || norm_dim < 1 || norm_dim > hd || (nh + nkv + 3) / 4 > 65535) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(head_rmsnorm_kernel<W>, dim3(T, (nh + nkv + 3) / 4), dim3(256), 0, st, qkv, (const W*)wq,
                       (const W*)wk, eps, nh, nkv, hd, norm_dim);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- rotary encoding + cache write
// qkv[t] holds, in float, nh query heads, then nkv key heads, then nkv value heads of hd each.
// Queries and keys are rotated by angle pos * inv_freq[i] (float) on the pair
//   pairing 0 ("half"):        (x[i], x[i + rot/2])   (/root/reference/src/engine/tq_transformer.c:1263-1289)
//   pairing 1 ("interleaved"): (x[2i], x[2i+1])        (/root/reference/src/engine/tq_ops.c:1418-1448)
// as (a, b) <- (a cos - b sin, a sin + b cos); dimensions from rot on pass through.  Rotated queries
// go to q_out; rotated keys and the values go into the page that holds position pos of the token's
// sequence: page = block_table[seq][pos / page_size], row pos % page_size of kv head h.  After the
// layer's own offset (already added to k_pool / v_pool) keys lie [page][kv head][row][hd] and values
// transposed, [page][kv head][hd][row].
// A workgroup of four waves takes `spb` heads of one token (grid (T, ceil(heads / spb))); a wave takes every
// fourth of them and turns pair i of all its heads with one sine and cosine.  write_kv: 0 queries only, 1 keys
// and values, 2 keys only (the values of whole runs of tokens go through v_write_tile_kernel below).
// element i of a bias that the product before did not add; BIAS: 0 none, 1 float32, 2 bfloat16 (a template
// argument, so that the loads of the bias go out beside those of the row and not behind a branch)
template <int BIAS>
__device__ __forceinline__ float bias_elem(const void* bias, size_t i) {
  if (BIAS == 0) return 0.f;
  return BIAS == 1 ? ((const float*)bias)[i] : to_f32(((const bf16_t*)bias)[i]);
}

template <int BIAS>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(const float* __restrict__ qkv, const void* __restrict__ bias,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                     int bt_stride, const float* __restrict__ inv_freq, int pairing, int rot,
                                     act_t* __restrict__ q_out, act_t* __restrict__ k_pool,
                                     act_t* __restrict__ v_pool, int page_size, int64_t page_stride, int nh,
                                     int nkv, int hd, int write_kv, int spb, int64_t ld, float amp) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int heads = nh + 2 * nkv;       // 0..nh-1 query heads, then key heads, then value heads
  const int s0 = blockIdx.y * spb + wave, s1 = min(blockIdx.y * spb + spb, heads);
  if (s0 >= s1) return;
  const int pos = positions[t];
  const float* src_t = qkv + (size_t)t * ld;
  act_t* q_t = q_out + (size_t)t * nh * hd;
  act_t *k_t = nullptr, *v_t = nullptr;      // the token's row of kv head 0 in its page
  if (write_kv && s1 > nh) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    const int row = pos % page_size;
    k_t = k_pool + (size_t)page * page_stride + (size_t)row * hd;
    v_t = v_pool + (size_t)page * page_stride + row;
  }
  const int rot_end = write_kv ? min(s1, nh + nkv) : min(s1, nh);     // heads below this are rotated
  const size_t kv_head_stride = (size_t)page_size * hd;
  const int half = rot / 2;
  for (int i = lane; i < half; i += TQ_WAVE) {
    const float theta = (float)pos * inv_freq[i];
    float sn, cs;
    sincosf(theta, &sn, &cs);
    sn *= amp;      // (an amplitude of 1 changes no bit)
    cs *= amp;
    const int ia = pairing == 0 ? i : 2 * i;
    const int ib = pairing == 0 ? i + half : 2 * i + 1;
    for (int s = s0; s < rot_end; s += 4) {
      const float* src = src_t + (size_t)s * hd;
      act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
      const float a = src[ia] + bias_elem<BIAS>(bias, (size_t)s * hd + ia);
      const float b = src[ib] + bias_elem<BIAS>(bias, (size_t)s * hd + ib);
      dst[ia] = from_f32<act_t>(a * cs - b * sn);
      dst[ib] = from_f32<act_t>(a * sn + b * cs);
    }
  }
  for (int s = s0; s < rot_end; s += 4) {      // dimensions from rot on pass through
    const float* src = src_t + (size_t)s * hd;
    act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
    for (int i = rot + lane; i < hd; i += TQ_WAVE)
      dst[i] = from_f32<act_t>(src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i));
  }
  if (write_kv != 1) return;
  for (int s = s0; s < s1; s += 4) {           // values lie transposed, [hd][row]
    if (s < nh + nkv) continue;
    const float* src = src_t + (size_t)s * hd;
    act_t* col = v_t + (size_t)(s - nh - nkv) * kv_head_stride;
    for (int i = lane; i < hd; i += TQ_WAVE)
      col[(size_t)i * page_size] = from_f32<act_t>(src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i));
  }
}

// The same with a norm behind the rotation: every rotated query and key head is divided by its root mean square over
// its first norm_dim values, x / sqrt(mean(x^2) + eps), no weights (heads laid out wider hold zeros behind them).  A wave
// takes a head at a time: a lane keeps the sines and cosines of its pairs (up to four: heads of up to 512), sums the
// squares of what it has turned, and scales as it stores.
template <int BIAS>
__global__ __launch_bounds__(256) void rope_norm_kv_write_kernel(const float* __restrict__ qkv, const void* __restrict__ bias,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                     int bt_stride, const float* __restrict__ inv_freq, int pairing, int rot,
                                     act_t* __restrict__ q_out, act_t* __restrict__ k_pool,
                                     act_t* __restrict__ v_pool, int page_size, int64_t page_stride, int nh,
                                     int nkv, int hd, int write_kv, int spb, int64_t ld, float amp, float eps,
                                     int norm_dim) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int heads = nh + 2 * nkv;
  const int s0 = blockIdx.y * spb + wave, s1 = min(blockIdx.y * spb + spb, heads);
  if (s0 >= s1) return;
  const int pos = positions[t];
  const float* src_t = qkv + (size_t)t * ld;
  act_t* q_t = q_out + (size_t)t * nh * hd;
  act_t *k_t = nullptr, *v_t = nullptr;
  if (write_kv && s1 > nh) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    const int row = pos % page_size;
    k_t = k_pool + (size_t)page * page_stride + (size_t)row * hd;
    v_t = v_pool + (size_t)page * page_stride + row;
  }
  const int rot_end = write_kv ? min(s1, nh + nkv) : min(s1, nh);
  const size_t kv_head_stride = (size_t)page_size * hd;
  const int half = rot / 2;
  float cs[4], sn[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + TQ_WAVE * j;
    cs[j] = 1.f;
    sn[j] = 0.f;
    if (i < half) {
      sincosf((float)pos * inv_freq[i], &sn[j], &cs[j]);
      sn[j] *= amp;
      cs[j] *= amp;
    }
  }
  for (int s = s0; s < rot_end; s += 4) {
    const float* src = src_t + (size_t)s * hd;
    act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
    float ra[4], rb[4], ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = lane + TQ_WAVE * j;
      ra[j] = rb[j] = 0.f;
      if (i < half) {
        const int ia = pairing == 0 ? i : 2 * i;
        const int ib = pairing == 0 ? i + half : 2 * i + 1;
        const float a = src[ia] + bias_elem<BIAS>(bias, (size_t)s * hd + ia);
        const float b = src[ib] + bias_elem<BIAS>(bias, (size_t)s * hd + ib);
        ra[j] = a * cs[j] - b * sn[j];
        rb[j] = a * sn[j] + b * cs[j];
        ss = fmaf(ra[j], ra[j], ss);
        ss = fmaf(rb[j], rb[j], ss);
      }
    }
    for (int i = rot + lane; i < hd; i += TQ_WAVE) {
      const float v = src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i);
      ss = fmaf(v, v, ss);
    }
    const float rs = 1.0f / sqrtf(wave_sum(ss) / (float)norm_dim + eps);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = lane + TQ_WAVE * j;
      if (i < half) {
        dst[pairing == 0 ? i : 2 * i] = from_f32<act_t>(ra[j] * rs);
        dst[pairing == 0 ? i + half : 2 * i + 1] = from_f32<act_t>(rb[j] * rs);
      }
    }
    for (int i = rot + lane; i < hd; i += TQ_WAVE)
      dst[i] = from_f32<act_t>((src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i)) * rs);
  }
  if (write_kv != 1) return;
  for (int s = s0; s < s1; s += 4) {
    if (s < nh + nkv) continue;
    const float* src = src_t + (size_t)s * hd;
    act_t* col = v_t + (size_t)(s - nh - nkv) * kv_head_stride;
    for (int i = lane; i < hd; i += TQ_WAVE)
      col[(size_t)i * page_size] = from_f32<act_t>(src[i] + bias_elem<BIAS>(bias, (size_t)s * hd + i));
  }
}

// The values of runs of tokens, one run per sequence (tokens cu_seqlens[b] .. of sequence b lie at positions
// start[b] ..): a workgroup takes 64 positions that share a page (grid (chunks, nkv, B)), turns their rows
// [position][hd] into [hd][position] in LDS and writes every dimension's positions 16 bytes at a time, where the
// token-by-token write above would touch a cache line per dimension for two bytes.
#define VT_POS 64
template <int VEC, int BIAS>      // positions per 16-byte store; the bias as in rope_kv_write_kernel
__global__ __launch_bounds__(256) void v_write_tile_kernel(const float* __restrict__ qkv,
                                                           const void* __restrict__ bias,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ slots,
                                                           const int* __restrict__ start,
                                                           const int* __restrict__ block_table, int bt_stride,
                                                           act_t* __restrict__ v_pool, int page_size,
                                                           int64_t page_stride, int nh, int nkv, int hd, int64_t ld) {
  extern __shared__ __attribute__((aligned(16))) unsigned char vt_raw[];
  act_t* ts = (act_t*)vt_raw;                        // [hd][VT_POS + VEC]
  constexpr int TS = VT_POS + VEC;
  const int b = blockIdx.z, h = blockIdx.y;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0, st = start[b];
  const int P0 = (st / VT_POS + blockIdx.x) * VT_POS;
  const int lo = max(P0, st), hi = min(P0 + VT_POS, st + n);
  if (lo >= hi) return;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const float* src0 = qkv + (size_t)(t0 + lo - st) * ld + (size_t)(nh + nkv + h) * hd;      // value row of position lo
  const size_t row_stride = (size_t)ld;
  const size_t bias0 = (size_t)(nh + nkv + h) * hd;      // the bias of this value head
  if (hd % 4 == 0) {        // 16 bytes of a row per thread and turn, all of a thread's loads on their way at once
    const int q4 = hd / 4, total = (hi - lo) * q4;
#pragma unroll 8
    for (int idx = threadIdx.x; idx < total; idx += 256) {
      const int r = idx / q4, d = (idx % q4) * 4;
      const f32x4 v = load4f(src0 + r * row_stride + d);
      act_t* to = ts + d * TS + (lo + r - P0);
      to[0] = from_f32<act_t>(v.x + bias_elem<BIAS>(bias, bias0 + d));
      to[TS] = from_f32<act_t>(v.y + bias_elem<BIAS>(bias, bias0 + d + 1));
      to[2 * TS] = from_f32<act_t>(v.z + bias_elem<BIAS>(bias, bias0 + d + 2));
      to[3 * TS] = from_f32<act_t>(v.w + bias_elem<BIAS>(bias, bias0 + d + 3));
    }
  } else {
    for (int r = wave; r < hi - lo; r += 4)
      for (int d = lane; d < hd; d += TQ_WAVE)
        ts[d * TS + (lo + r - P0)] = from_f32<act_t>(src0[r * row_stride + d] + bias_elem<BIAS>(bias, bias0 + d));
  }
  __syncthreads();
  const int page = block_table[(size_t)slots[b] * bt_stride + P0 / page_size];
  act_t* base = v_pool + (size_t)page * page_stride + (size_t)h * page_size * hd + P0 % page_size;
  constexpr int GROUPS = VT_POS / VEC;
  for (int idx = threadIdx.x; idx < hd * GROUPS; idx += blockDim.x) {
    const int d = idx / GROUPS, g = idx % GROUPS;
    const int p0 = P0 + g * VEC;
    act_t* dst = base + (size_t)d * page_size + g * VEC;
    const act_t* from = ts + d * TS + g * VEC;
    if (p0 >= lo && p0 + VEC <= hi) {
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(from);
    } else {
      for (int j = max(p0, lo) - p0; j < min(p0 + VEC, hi) - p0; ++j) dst[j] = from[j];
    }
  }
}

// cu_seqlens, slots, start (null, or [B + 1], [B], [B] with max_new the longest run): the tokens as runs of
// consecutive positions, one per sequence; given for whole prompts, they let the values go by tiles.
// bias (null, or [(nh + 2 nkv) * hd] of bias_type): added to qkv as it is read, for a product that left it out.
// ld: floats between the rows of two tokens in qkv (at least (nh + 2 nkv) * hd: the rows may be runs of columns of a
// wider product).  amp: a factor on every sine and cosine (1: none).  norm_eps > 0: the rotated query and key heads are
// divided by their root mean square over norm_dim values (rope_norm_kv_write_kernel; heads of up to 512).
TQ_API int tq_rope_kv_write_ex(const float* qkv, int64_t ld, const void* bias, int bias_type, const int* positions,
                               const int* seq_of_token, const int* block_table, int bt_stride, const float* inv_freq,
                               int pairing, int rot, float amp, float norm_eps, int norm_dim, void* q_out, void* k_pool,
                               void* v_pool, int page_size, int64_t page_stride, int T, int nh, int nkv, int hd, int write_kv,
                               const int* cu_seqlens, const int* slots, const int* start, int B, int max_new,
                               hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > hd || (rot & 1) || (pairing != 0 && pairing != 1)) return TQ_ERR_BAD_ARG;
  if (ld < (int64_t)(nh + 2 * nkv) * hd || norm_eps < 0.f) return TQ_ERR_BAD_ARG;
  if (norm_eps > 0.f && (norm_dim < 1 || norm_dim > hd || rot > 512)) return TQ_ERR_BAD_ARG;
  if (bias && bias_type != TQ_F32 && bias_type != TQ_BF16) return TQ_ERR_BAD_ARG;
  constexpr int VEC = 16 / (int)sizeof(act_t);
  const size_t vt_shmem = (size_t)hd * (VT_POS + VEC) * sizeof(act_t);
  const bool tiles = write_kv && cu_seqlens && slots && start && B > 0 && B <= 65535 && nkv <= 65535 && max_new > 8 &&
                     page_size % VT_POS == 0 && vt_shmem <= 64 * 1024;
  if (tiles) write_kv = 2;
  const int heads = nh + 2 * nkv;
  // few tokens: a head per wave, so that the chip sees many small workgroups; many: all heads of a token in one
  int spb = 4;
  while (spb < heads && (int64_t)T * ((heads + spb - 1) / spb) > 4096) spb *= 2;
  if ((heads + spb - 1) / spb > 65535) return TQ_ERR_UNSUPPORTED;
  const int bias_kind = !bias ? 0 : bias_type == TQ_F32 ? 1 : 2;
#define TQ_ROPE_LAUNCH(BIAS)                                                                                          \
  do {                                                                                                                \
    if (norm_eps > 0.f)                                                                                               \
      hipLaunchKernelGGL(rope_norm_kv_write_kernel<BIAS>, dim3(T, (heads + spb - 1) / spb), dim3(256), 0, st, qkv,    \
                         bias, positions, seq_of_token, block_table, bt_stride, inv_freq, pairing, rot,               \
                         (act_t*)q_out, (act_t*)k_pool, (act_t*)v_pool, page_size, page_stride, nh, nkv, hd,          \
                         write_kv, spb, ld, amp, norm_eps, norm_dim);                                                 \
    else                                                                                                              \
      hipLaunchKernelGGL(rope_kv_write_kernel<BIAS>, dim3(T, (heads + spb - 1) / spb), dim3(256), 0, st, qkv, bias,   \
                         positions, seq_of_token, block_table, bt_stride, inv_freq, pairing, rot, (act_t*)q_out,      \
                         (act_t*)k_pool, (act_t*)v_pool, page_size, page_stride, nh, nkv, hd, write_kv, spb, ld,      \
                         amp);                                                                                        \
  } while (0)
  if (bias_kind == 0) TQ_ROPE_LAUNCH(0);
  else if (bias_kind == 1) TQ_ROPE_LAUNCH(1);
  else TQ_ROPE_LAUNCH(2);
#undef TQ_ROPE_LAUNCH
  TQ_LAUNCH_CHECK();
  if (tiles) {
#define TQ_VT_LAUNCH(BIAS)                                                                                            \
  do {                                                                                                                \
    if (vt_shmem > 48 * 1024)                                                                                         \
      (void)hipFuncSetAttribute((const void*)v_write_tile_kernel<VEC, BIAS>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)vt_shmem);                                                                       \
    hipLaunchKernelGGL((v_write_tile_kernel<VEC, BIAS>), dim3((max_new + VT_POS - 1) / VT_POS + 1, nkv, B), dim3(256), \
                       vt_shmem, st, qkv, bias, cu_seqlens, slots, start, block_table, bt_stride, (act_t*)v_pool,     \
                       page_size, page_stride, nh, nkv, hd, ld);                                                      \
  } while (0)
    if (bias_kind == 0) TQ_VT_LAUNCH(0);
    else if (bias_kind == 1) TQ_VT_LAUNCH(1);
    else TQ_VT_LAUNCH(2);
#undef TQ_VT_LAUNCH
    TQ_LAUNCH_CHECK();
  }
  return 0;
}

TQ_API int tq_rope_kv_write(const float* qkv, const void* bias, int bias_type, const int* positions, const int* seq_of_token,
                            const int* block_table, int bt_stride, const float* inv_freq, int pairing, int rot,
                            void* q_out, void* k_pool, void* v_pool, int page_size, int64_t page_stride, int T,
                            int nh, int nkv, int hd, int write_kv, const int* cu_seqlens, const int* slots,
                            const int* start, int B, int max_new, hipStream_t st) {
  return tq_rope_kv_write_ex(qkv, (int64_t)(nh + 2 * nkv) * hd, bias, bias_type, positions, seq_of_token, block_table,
                             bt_stride, inv_freq, pairing, rot, 1.0f, 0.f, hd, q_out, k_pool, v_pool, page_size, page_stride,
                             T, nh, nkv, hd, write_kv, cu_seqlens, slots, start, B, max_new, st);
}

// ---------------------------------------------------------------- sum of expert outputs
// out[t] = sum_j weights[t][j] * y[slot[t][j]]   (j ascending: the order in which experts were selected,
//          /root/reference/src/engine/tq_moe.c:720,864-999)
//        + gate[t] * sum_s shared[s][t]           (shared expert last, tq_moe.c:1005-1058)
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ pair_slot,
                                                          const float* __restrict__ weights, int topk,
                                                          const float* __restrict__ shared, int S, size_t shared_stride,
                                                          const float* __restrict__ gate, float* __restrict__ out, int H) {
  __shared__ int slot[64];
  __shared__ float wgt[64];
  const int t = blockIdx.x;
  if (threadIdx.x < topk) {      // the token's rows and weights once, not once per element
    slot[threadIdx.x] = pair_slot[t * topk + threadIdx.x];
    wgt[threadIdx.x] = weights[t * topk + threadIdx.x];
  }
  __syncthreads();
  const float g = gate ? gate[t] : 1.0f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < topk; ++j)
      if (slot[j] >= 0) acc += wgt[j] * y[(size_t)slot[j] * H + i];      // (-1: a pair without a row)
    if (shared) {
      float sh = 0.f;
      for (int s = 0; s < S; ++s) sh += shared[s * shared_stride + (size_t)t * H + i];
      acc += g * sh;
    }
    out[(size_t)t * H + i] = acc;
  }
}

TQ_API int tq_moe_combine(const float* y, const int* pair_slot, const float* weights, int topk,
                          const float* shared, int S, int64_t shared_stride, const float* gate, float* out, int T,
                          int H, hipStream_t st) {
  if (T <= 0) return 0;
  if (topk < 1 || topk > 64) return TQ_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, pair_slot, weights, topk, shared, S,
                     (size_t)shared_stride, gate, out, H);
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- embedding with a learned position row
// x[t, :] = table[tokens[t], :] * scale + pos_table[positions[t], :], in float: for models that add a learned vector
// per position to the embedded token instead of rotating queries and keys.
template <class W>
__global__ void embed_pos_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                 const W* __restrict__ table, const W* __restrict__ pos_table, float* __restrict__ x,
                                 int H, float scale) {
  const int t = blockIdx.x;
  const W* row = table + (size_t)tokens[t] * H;
  const W* prow = pos_table + (size_t)positions[t] * H;
  float* out = x + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_f32(row[i]) * scale + to_f32(prow[i]);
}

TQ_API int tq_embed_pos(const int* tokens, const int* positions, const void* table, const void* pos_table, int wtype,
                        float* x, int T, int H, float scale, hipStream_t st) {
  if (T <= 0) return 0;
  if (!positions || !pos_table) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(embed_pos_kernel<W>, dim3(T), dim3(256), 0, st, tokens, positions, (const W*)table,
                       (const W*)pos_table, x, H, scale);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- residual sum of a normed part + RMS norm
// For layers that norm a part's output before it joins the stream (a norm before and one after every part):
//   d = what add_rmsnorm would add (partial sums in order, or the experts' weighted rows and the gated dense sums)
//   v = x[row] + (d * (1 / sqrt(mean(d^2) + eps_d))) * wd          (the residual sum, in float)
//   x[row] = v                                                       (only when rows is null)
//   out = (v * (1 / sqrt(mean(v^2) + eps))) * w                      (left out when w is null)
// Both sums of squares run in the fixed order of block_sum over a thread's own elements, whatever the step holds.
template <class W, bool VEC>
__global__ void add_normed_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ delta, int S,
                                          size_t delta_stride, const float* __restrict__ y,
                                          const int* __restrict__ pair_slot, const float* __restrict__ weights,
                                          int topk, const float* __restrict__ gate, const W* __restrict__ wd,
                                          float eps_d, const W* __restrict__ w, float eps,
                                          const int* __restrict__ rows, act_t* __restrict__ out,
                                          float* __restrict__ out32, int H, const float* __restrict__ shift_w,
                                          float* __restrict__ shift_state, const int* __restrict__ shift_slots) {
  extern __shared__ __attribute__((aligned(16))) float v[];       // H floats, then one float per wave
  __shared__ int slot[64];
  __shared__ float wgt[64];
  float* red = v + (H + 3) / 4 * 4;
  const int r = blockIdx.x;
  const int row = rows ? rows[r] : r;
  float* xr = x + (size_t)row * H;
  const float* dr = delta + (size_t)row * H;
  // (shift_state, with w null and every row a sequence of its own: what goes out is the summed row blended with the row
  // that the sequence's slot keeps, a + (kept - a) * shift_w, and the slot then keeps the summed row: the token shift of a
  // decode step, without a launch of its own)
  float* kept = shift_state ? shift_state + (size_t)shift_slots[row] * H : nullptr;
  float g = 1.0f;
  if (y) {
    if (threadIdx.x < topk) {
      slot[threadIdx.x] = pair_slot[(size_t)row * topk + threadIdx.x];
      wgt[threadIdx.x] = weights[(size_t)row * topk + threadIdx.x];
    }
    if (gate) g = gate[row];
    __syncthreads();
  }
  constexpr int N = VEC ? 4 : 1;
  float ss = 0.f;
  for (int i = threadIdx.x * N; i < H; i += blockDim.x * N) {
    float d[N];
#pragma unroll
    for (int u = 0; u < N; ++u) d[u] = 0.f;
    if (y) {
      for (int j = 0; j < topk; ++j) {
        if (slot[j] < 0) continue;        // a pair without a row (an expert that is the identity: its share rides in `delta`)
        const float* yr = y + (size_t)slot[j] * H + i;
        if constexpr (VEC) {
          const f32x4 t = load4f(yr);
          d[0] += wgt[j] * t.x;
          d[1] += wgt[j] * t.y;
          d[2] += wgt[j] * t.z;
          d[3] += wgt[j] * t.w;
        } else {
          d[0] += wgt[j] * yr[0];
        }
      }
      if (S > 0) {
        float sh[N];
#pragma unroll
        for (int u = 0; u < N; ++u) sh[u] = 0.f;
        for (int s = 0; s < S; ++s)
#pragma unroll
          for (int u = 0; u < N; ++u) sh[u] += dr[s * delta_stride + i + u];
#pragma unroll
        for (int u = 0; u < N; ++u) d[u] += g * sh[u];
      }
    } else {
      for (int s = 0; s < S; ++s) {
        if constexpr (VEC) {
          const f32x4 t = load4f(dr + s * delta_stride + i);
          d[0] += t.x;
          d[1] += t.y;
          d[2] += t.z;
          d[3] += t.w;
        } else {
          d[0] += dr[s * delta_stride + i];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < N; ++u) {
      v[i + u] = d[u];
      ss += d[u] * d[u];
    }
  }
  ss = block_sum(ss, red);
  const float rd = 1.0f / sqrtf(ss / (float)H + eps_d);
  float s2 = 0.f;
  for (int i = threadIdx.x * N; i < H; i += blockDim.x * N) {
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const float a = xr[i + u] + (v[i + u] * rd) * to_f32(wd[i + u]);
      v[i + u] = a;
      if (!rows) xr[i + u] = a;
      if (!w && out) {      // the summed stream itself, for a part that reads it un-normed
        float h = a;
        if (kept) {
          h = a + (kept[i + u] - a) * shift_w[i + u];
          kept[i + u] = a;
        }
        out[(size_t)r * H + i + u] = from_f32<act_t>(h);
      }
      s2 += a * a;
    }
  }
  if (!w) return;
  s2 = block_sum(s2, red);
  const float rs = 1.0f / sqrtf(s2 / (float)H + eps);
  for (int i = threadIdx.x * N; i < H; i += blockDim.x * N) {
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const float o = v[i + u] * rs * to_f32(w[i + u]);
      if (out) out[(size_t)r * H + i + u] = from_f32<act_t>(o);
      if (out32) out32[(size_t)r * H + i + u] = o;
    }
  }
}

TQ_API int tq_add_normed_rmsnorm_shift(float* x, const float* delta, int S, int64_t delta_stride, const float* y,
                                       const int* pair_slot, const float* weights, int topk, const float* gate,
                                       const void* wd, float eps_d, const void* w, int wtype, float eps, const int* rows,
                                       int R, void* out, float* out32, int H, const float* shift_w, float* shift_state,
                                       const int* shift_slots, hipStream_t st);

// As tq_add_rmsnorm, with the weights wd and the eps_d of the norm that what is added passes first; w null: the
// stream is summed and nothing is normed (no out32; `out`, if given, receives the summed stream in the activation type).
TQ_API int tq_add_normed_rmsnorm(float* x, const float* delta, int S, int64_t delta_stride, const float* y,
                                 const int* pair_slot, const float* weights, int topk, const float* gate,
                                 const void* wd, float eps_d, const void* w, int wtype, float eps, const int* rows,
                                 int R, void* out, float* out32, int H, hipStream_t st) {
  return tq_add_normed_rmsnorm_shift(x, delta, S, delta_stride, y, pair_slot, weights, topk, gate, wd, eps_d, w, wtype, eps, rows,
                                     R, out, out32, H, nullptr, nullptr, nullptr, st);
}

// The same with a token shift behind the sum (w and rows null, `out` given, every row a sequence of its own whose slot is
// shift_slots[row]): out = a + (shift_state[slot] - a) * shift_w for the summed row a, and shift_state[slot] = a.
TQ_API int tq_add_normed_rmsnorm_shift(float* x, const float* delta, int S, int64_t delta_stride, const float* y,
                                       const int* pair_slot, const float* weights, int topk, const float* gate,
                                       const void* wd, float eps_d, const void* w, int wtype, float eps, const int* rows,
                                       int R, void* out, float* out32, int H, const float* shift_w, float* shift_state,
                                       const int* shift_slots, hipStream_t st) {
  if (R <= 0) return 0;
  if (shift_state && (w || rows || !out || !shift_w || !shift_slots)) return TQ_ERR_BAD_ARG;
  if (!wd || (y && (topk < 1 || topk > 64 || !pair_slot || !weights))) return TQ_ERR_BAD_ARG;
  if (!y && (S < 1 || !delta)) return TQ_ERR_BAD_ARG;
  const int threads = (H % 4 == 0 && H >= 2048) ? 512 : 256;
  const size_t shmem = (size_t)((H + 3) / 4 * 4 + threads / TQ_WAVE) * sizeof(float);
  if (shmem > 150 * 1024) return TQ_ERR_UNSUPPORTED;
  const bool vec = H % 4 == 0;
  TQ_DISPATCH_W(wtype, {
    if (vec) {
      if (shmem > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)add_normed_rmsnorm_kernel<W, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
      hipLaunchKernelGGL((add_normed_rmsnorm_kernel<W, true>), dim3(R), dim3(threads), shmem, st, x, delta, S,
                         (size_t)delta_stride, y, pair_slot, weights, topk, gate, (const W*)wd, eps_d, (const W*)w, eps,
                         rows, (act_t*)out, out32, H, shift_w, shift_state, shift_slots);
    } else {
      if (shmem > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)add_normed_rmsnorm_kernel<W, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
      hipLaunchKernelGGL((add_normed_rmsnorm_kernel<W, false>), dim3(R), dim3(threads), shmem, st, x, delta, S,
                         (size_t)delta_stride, y, pair_slot, weights, topk, gate, (const W*)wd, eps_d, (const W*)w, eps,
                         rows, (act_t*)out, out32, H, shift_w, shift_state, shift_slots);
    }
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- token shift
// What a mixer reads where every token is blended with the token before it: out[t] = x[t] + (x[t-1] - x[t]) * w, x[t-1]
// being the sequence's row before, as it was before any blending: the step's own row t - 1, or for the first token that
// a sequence brings the row that its slot keeps from the step before (zeros for a new sequence).  Afterwards the slot
// keeps the last row that the sequence brought.  The workgroup of a run's first token reads the slot's row and is the
// one that writes it, each thread its own elements, so no other workgroup touches it in between.
template <class W>
__global__ __launch_bounds__(256) void token_shift_kernel(const float* __restrict__ x, const W* __restrict__ w,
                                                          float* __restrict__ state, const int* __restrict__ cu_seqlens,
                                                          const int* __restrict__ slots, int B, act_t* __restrict__ out, int H) {
  const int t = blockIdx.x;
  // the run that holds token t: the last one that starts at or before it (a step of one token per sequence: run t)
  int lo = gridDim.x == (unsigned)B ? t : 0, hi = gridDim.x == (unsigned)B ? t : B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (cu_seqlens[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int first = cu_seqlens[lo], last = cu_seqlens[lo + 1] - 1;
  const float* xr = x + (size_t)t * H;
  if (t != first) {
    const float* xp = xr - H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[(size_t)t * H + i] = from_f32<act_t>(xr[i] + (xp[i] - xr[i]) * to_f32(w[i]));
    return;
  }
  float* sr = state + (size_t)slots[lo] * H;
  const float* xl = x + (size_t)last * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float before = sr[i];
    out[(size_t)t * H + i] = from_f32<act_t>(xr[i] + (before - xr[i]) * to_f32(w[i]));
    sr[i] = xl[i];
  }
}

// x float [T][H]; w [H]; state float [slots][H]; cu_seqlens [B + 1], slots [B]: the step's runs; out [T][H] in the
// activation type.
TQ_API int tq_token_shift(const float* x, const void* w, int wtype, float* state, const int* cu_seqlens, const int* slots,
                          int B, void* out, int T, int H, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || H <= 0) return TQ_ERR_BAD_ARG;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(token_shift_kernel<W>, dim3(T), dim3(256), 0, st, x, (const W*)w, state, cu_seqlens, slots, B,
                       (act_t*)out, H);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- unit values, mixed with another layer's
// Every value head of the float rows v [T][.. heads * hd ..] (row stride ld, head stride hd, a head's first vd numbers
// its values) is divided by its root mean square over vd (eps inside the root, no weights; eps 0: left as it is), in place; with `first`
// (another layer's rows of values, laid out alike with its own strides, already so normed) it then becomes
// (1 - lambda) v + lambda first, lambda read from the device.  A wave takes a head of a token.
template <class W>
__global__ __launch_bounds__(256) void value_norm_mix_kernel(float* __restrict__ v, int64_t ld, int hd, int vd, int heads,
                                                             float eps, const float* __restrict__ first, int64_t ld_first,
                                                             int hd_first, const W* __restrict__ lambda, int T) {
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x / TQ_WAVE) + wave;
  if (item >= (int64_t)T * heads) return;
  const int t = (int)(item / heads), h = (int)(item % heads);
  float* row = v + (size_t)t * ld + (size_t)h * hd;
  float ss = 0.f;
  for (int i = lane; i < vd; i += TQ_WAVE) ss += row[i] * row[i];
  ss = wave_sum(ss);
  const float r = eps > 0.f ? 1.0f / sqrtf(ss / (float)vd + eps) : 1.0f;      // eps 0: the values are mixed as they are
  const float lam = first ? to_f32(lambda[0]) : 0.f;
  const float* fr = first ? first + (size_t)t * ld_first + (size_t)h * hd_first : nullptr;
  for (int i = lane; i < vd; i += TQ_WAVE) {
    float a = row[i] * r;
    if (first) a = (1.0f - lam) * a + lam * fr[i];
    row[i] = a;
  }
}

TQ_API int tq_value_norm_mix(float* v, int64_t ld, int hd, int vd, int heads, float eps, const float* first,
                             int64_t ld_first, int hd_first, const void* lambda, int wtype, int T, hipStream_t st) {
  if (T <= 0 || heads <= 0) return 0;
  if (vd < 1 || vd > hd || (first && (!lambda || vd > hd_first))) return TQ_ERR_BAD_ARG;
  const int64_t items = (int64_t)T * heads;
  TQ_DISPATCH_W(first ? wtype : TQ_F32, {
    hipLaunchKernelGGL(value_norm_mix_kernel<W>, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, v, ld, hd, vd, heads, eps,
                       first, ld_first, hd_first, (const W*)lambda, T);
  });
  TQ_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- head norms, unit values, mix, rotation and cache write in one
// What head_rmsnorm, value_norm_mix and rope_kv_write do one after the other, in one pass over a token's row: a wave takes a
// head.  Query and key heads (qk_eps > 0): x * (1 / sqrt(sum(x^2) / norm_dim + qk_eps)) * w, w = wq or wk (null: heads of
// that kind are left as they are), then the rotation; value heads (v_eps > 0): the head's first vd numbers divided by their
// root mean square, then, with v_first, (1 - lambda) v + lambda v_first.  The values are also written back into qkv as the
// cache holds them: for the tile write of whole runs of tokens that follows (write_kv 2), and for later layers that mix
// them into their own.  The row holds every product's bias already.
template <class W>
__global__ __launch_bounds__(256) void attn_prep_kv_write_kernel(
    float* __restrict__ qkv, int64_t ld, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int bt_stride, const float* __restrict__ inv_freq, int pairing, int rot, float amp,
    const W* __restrict__ wq, const W* __restrict__ wk, float qk_eps, int norm_dim, float v_eps, int vd,
    const float* __restrict__ v_first, int64_t ld_first, int hd_first, const W* __restrict__ lambda,
    act_t* __restrict__ q_out, act_t* __restrict__ k_pool, act_t* __restrict__ v_pool, int page_size, int64_t page_stride,
    int nh, int nkv, int hd, int write_kv, int spb) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TQ_WAVE, lane = threadIdx.x % TQ_WAVE;
  const int heads = nh + 2 * nkv;
  const int s0 = blockIdx.y * spb + wave, s1 = min(blockIdx.y * spb + spb, heads);
  if (s0 >= s1) return;
  const int pos = positions[t];
  float* src_t = qkv + (size_t)t * ld;
  act_t* q_t = q_out + (size_t)t * nh * hd;
  act_t *k_t = nullptr, *v_t = nullptr;
  if (write_kv && s1 > nh) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    const int row = pos % page_size;
    k_t = k_pool + (size_t)page * page_stride + (size_t)row * hd;
    v_t = v_pool + (size_t)page * page_stride + row;
  }
  const int rot_end = write_kv ? min(s1, nh + nkv) : min(s1, nh);
  const size_t kv_head_stride = (size_t)page_size * hd;
  const int half = rot / 2;
  float cs[4], sn[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + TQ_WAVE * j;
    cs[j] = 1.f;
    sn[j] = 0.f;
    if (i < half) {
      sincosf((float)pos * inv_freq[i], &sn[j], &cs[j]);
      sn[j] *= amp;
      cs[j] *= amp;
    }
  }
  for (int s = s0; s < rot_end; s += 4) {
    const float* src = src_t + (size_t)s * hd;
    act_t* dst = s < nh ? q_t + (size_t)s * hd : k_t + (size_t)(s - nh) * kv_head_stride;
    const W* w = qk_eps > 0.f ? (s < nh ? wq : wk) : nullptr;
    float rs = 1.0f;
    if (w) {
      float ss = 0.f;
      for (int i = lane; i < hd; i += TQ_WAVE) ss = fmaf(src[i], src[i], ss);
      rs = 1.0f / sqrtf(wave_sum(ss) / (float)norm_dim + qk_eps);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = lane + TQ_WAVE * j;
      if (i < half) {
        const int ia = pairing == 0 ? i : 2 * i;
        const int ib = pairing == 0 ? i + half : 2 * i + 1;
        float a = src[ia], b = src[ib];
        if (w) {
          a = a * rs * to_f32(w[ia]);
          b = b * rs * to_f32(w[ib]);
        }
        dst[ia] = from_f32<act_t>(a * cs[j] - b * sn[j]);
        dst[ib] = from_f32<act_t>(a * sn[j] + b * cs[j]);
      }
    }
    for (int i = rot + lane; i < hd; i += TQ_WAVE) dst[i] = from_f32<act_t>(w ? src[i] * rs * to_f32(w[i]) : src[i]);
  }
  if (!write_kv) return;
  const float lam = v_first ? to_f32(lambda[0]) : 0.f;
  for (int s = s0; s < s1; s += 4) {
    if (s < nh + nkv) continue;
    const int g = s - nh - nkv;
    float* src = src_t + (size_t)s * hd;
    float r = 1.0f;
    if (v_eps > 0.f) {
      float ss = 0.f;
      for (int i = lane; i < vd; i += TQ_WAVE) ss = fmaf(src[i], src[i], ss);
      r = 1.0f / sqrtf(wave_sum(ss) / (float)vd + v_eps);
    }
    const float* fr = v_first ? v_first + (size_t)t * ld_first + (size_t)g * hd_first : nullptr;
    act_t* col = v_t + (size_t)g * kv_head_stride;
    for (int i = lane; i < hd; i += TQ_WAVE) {
      float a = src[i];
      if (i < vd) {
        a *= r;
        if (fr) a = (1.0f - lam) * a + lam * fr[i];
        src[i] = a;
      }
      if (write_kv == 1) col[(size_t)i * page_size] = from_f32<act_t>(a);
    }
  }
}

// Arguments as tq_rope_kv_write_ex's (no bias: the rows hold it), with wq, wk (null: no norm of those heads), qk_eps,
// norm_dim for the heads' norm before the rotation, v_eps (0: none) and vd for the values' unit norm, and v_first (null:
// none), ld_first, hd_first, lambda for their mix.  hd at most 512 rotated numbers.
TQ_API int tq_attn_prep_kv_write(float* qkv, int64_t ld, const int* positions, const int* seq_of_token, const int* block_table,
                                 int bt_stride, const float* inv_freq, int pairing, int rot, float amp, const void* wq,
                                 const void* wk, int wtype, float qk_eps, int norm_dim, float v_eps, int vd,
                                 const float* v_first, int64_t ld_first, int hd_first, const void* lambda, void* q_out,
                                 void* k_pool, void* v_pool, int page_size, int64_t page_stride, int T, int nh, int nkv,
                                 int hd, int write_kv, const int* cu_seqlens, const int* slots, const int* start, int B,
                                 int max_new, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot % 2 != 0 || rot > hd || rot > 512 || (pairing != 0 && pairing != 1)) return TQ_ERR_BAD_ARG;
  if (ld < (int64_t)(nh + 2 * nkv) * hd || norm_dim < 1 || norm_dim > hd || vd < 1 || vd > hd) return TQ_ERR_BAD_ARG;
  if (v_first && (!lambda || vd > hd_first)) return TQ_ERR_BAD_ARG;
  if (write_kv && (!k_pool || !v_pool)) return TQ_ERR_BAD_ARG;
  constexpr int VEC = 16 / (int)sizeof(act_t);
  const size_t vt_shmem = (size_t)hd * (VT_POS + VEC) * sizeof(act_t);
  const bool tiles = write_kv && cu_seqlens && slots && start && B > 0 && B <= 65535 && nkv <= 65535 && max_new > 8 &&
                     page_size % VT_POS == 0 && vt_shmem <= 64 * 1024;
  if (tiles) write_kv = 2;
  const int heads = nh + 2 * nkv;
  int spb = 4;
  while (spb < heads && (int64_t)T * ((heads + spb - 1) / spb) > 4096) spb *= 2;
  if ((heads + spb - 1) / spb > 65535) return TQ_ERR_UNSUPPORTED;
  TQ_DISPATCH_W(wtype, {
    hipLaunchKernelGGL(attn_prep_kv_write_kernel<W>, dim3(T, (heads + spb - 1) / spb), dim3(256), 0, st, qkv, ld, positions,
                       seq_of_token, block_table, bt_stride, inv_freq, pairing, rot, amp, (const W*)wq, (const W*)wk, qk_eps,
                       norm_dim, v_eps, vd, v_first, ld_first, hd_first, (const W*)lambda, (act_t*)q_out, (act_t*)k_pool,
                       (act_t*)v_pool, page_size, page_stride, nh, nkv, hd, write_kv, spb);
  });
  TQ_LAUNCH_CHECK();
  if (tiles) {
    if (vt_shmem > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)v_write_tile_kernel<VEC, 0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)vt_shmem);
    hipLaunchKernelGGL((v_write_tile_kernel<VEC, 0>), dim3((max_new + VT_POS - 1) / VT_POS + 1, nkv, B), dim3(256), vt_shmem, st,
                       qkv, nullptr, cu_seqlens, slots, start, block_table, bt_stride, (act_t*)v_pool, page_size, page_stride,
                       nh, nkv, hd, ld);
    TQ_LAUNCH_CHECK();
  }
  return 0;
}
