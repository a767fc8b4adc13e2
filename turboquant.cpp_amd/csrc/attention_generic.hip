// Attention of each given token over the cache pages of its sequence, with plain float arithmetic.
//
// Token t of sequence s at position p attends to positions lo..p, lo = max(0, p - window + 1)
// when a window is set (the last `window` positions, the current one included:
// /root/reference/src/engine/tq_transformer.c:1646-1654), else 0.  Query head h reads kv head
// h / (nh / nkv) (tq_transformer.c:1675-1679).  score = (q . k) / sqrt(hd) (:1908-1937), softmax
// over the scores (/root/reference/src/engine/tq_ops.c:1496-1519), output = sum p_j v_j
// (tq_transformer.c:1975-1976).  The softmax is computed chunk by chunk with a running maximum;
// chunks start at multiples of CHUNK positions, so the order of every sum depends only on the
// token's own position.  The same kernel serves whole prompts and single decoded tokens: the cache
// has been written for all tokens of the step before it runs.  In a page, keys lie [kv head][row][hd]
// and values transposed, [kv head][hd][row].
#include "common.h"
#include "score_mod.h"

#define CHUNK 128

__global__ __launch_bounds__(CHUNK) void attention_generic_kernel(
    const act_t* __restrict__ q, const act_t* __restrict__ k_pool, const act_t* __restrict__ v_pool,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int bt_stride, int page_size, int64_t page_stride, int nh, int nkv, int hd, int window, float scale,
    ScoreMod mod, act_t* __restrict__ out) {
  extern __shared__ float sm[];
  float* qs = sm;                       // hd
  float* ps = qs + hd;                  // CHUNK probabilities
  float* red = ps + CHUNK;              // one per wave
  int64_t* head_off = (int64_t*)(red + 4);  // per row of the chunk: offset of its page's block for this kv head
  int* row_in_page = (int*)(head_off + CHUNK);
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int* table = block_table + (size_t)seq_of_token[t] * bt_stride;
  const int lo = reach_lo(pos, window, mod.chunk);
  const bool biased = mod.r1 != nullptr;
  const float r1 = biased ? mod.r1[h] : 0.f, r2 = biased ? mod.r2[h] : 0.f;

  for (int i = tid; i < hd; i += CHUNK) qs[i] = to_f32(q[((size_t)t * nh + h) * hd + i]);
  __syncthreads();

  // each thread owns the output dimensions tid, tid + CHUNK, ... (at most 4: hd <= 512)
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  if (mod.sink) {        // a score without key or value, counted once
    m_run = mod.sink[h];
    l_run = 1.f;
  }
  const bool sig = mod.pb != nullptr;       // weights are sigmoids of the scores and are not normalised
  const float pb = sig ? mod.pb[h] : 0.f;
  if (sig) m_run = 0.f;
  const int kept = keep_tiles(mod.keep, CHUNK), lo_chunk = lo / CHUNK;

  for (int c_i = first_tile(lo_chunk, kept); c_i * CHUNK <= pos; c_i = next_tile(c_i, lo_chunk, kept)) {
    const int base = c_i * CHUNK;
    const int j = base + tid;
    const bool valid = sees(j, pos, lo, mod.keep);
    float sc = -INFINITY;
    int64_t off = 0;
    if (valid) {
      const int page = table[j / page_size];
      off = (int64_t)page * page_stride + (int64_t)kvh * page_size * hd;
      const act_t* kr = k_pool + off + (int64_t)(j % page_size) * hd;   // keys: [row][hd]
      float d = 0.f;
      for (int i = 0; i < hd; ++i) d = fmaf(qs[i], to_f32(kr[i]), d);
      sc = mod_score(d * scale, mod.cap, biased, r1, r2, pos - j);
    }
    head_off[tid] = off;
    row_in_page[tid] = j % page_size;
    const float m_chunk = sig ? 0.f : block_max(sc, red);
    const float m_new = fmaxf(m_run, m_chunk);
    const float p = valid ? (sig ? sigmoid_weight(sc + pb) : expf(sc - m_new)) : 0.f;
    ps[tid] = p;
    const float l_chunk = block_sum(p, red);   // has the barriers that publish ps and the offsets
    const float alpha = m_run == -INFINITY ? 0.f : expf(m_run - m_new);
    l_run = l_run * alpha + l_chunk;
    m_run = m_new;
    const int n_in_chunk = min(CHUNK, pos - base + 1);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int d = tid + c * CHUNK;
      if (d < hd) {
        float a = acc[c] * alpha;
        for (int jj = 0; jj < n_in_chunk; ++jj) {
          const float pj = ps[jj];
          // values: [hd][row]
          if (pj != 0.f) a = fmaf(pj, to_f32(v_pool[head_off[jj] + (int64_t)d * page_size + row_in_page[jj]]), a);
        }
        acc[c] = a;
      }
    }
    __syncthreads();
  }
  const float inv = sig ? 1.0f : 1.0f / l_run;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int d = tid + c * CHUNK;
    if (d < hd) out[((size_t)t * nh + h) * hd + d] = from_f32<act_t>(acc[c] * inv);
  }
}

TQ_API int tq_attention_generic_sig(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                                    const int* seq_of_token, const int* block_table, int bt_stride, int page_size,
                                    int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale,
                                    float softcap, const float* r1, const float* r2, int chunk, const float* sink,
                                    const float* pb, int keep, void* out, hipStream_t st);

// softcap, r1, r2, chunk, sink: what happens to a score before the softmax and the chunks of positions, see score_mod.h
// (0, null, null, 0, null: nothing).
TQ_API int tq_attention_generic_mod(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                                    const int* seq_of_token, const int* block_table, int bt_stride, int page_size,
                                    int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale,
                                    float softcap, const float* r1, const float* r2, int chunk, const float* sink,
                                    void* out, hipStream_t st) {
  return tq_attention_generic_sig(q, k_pool, v_pool, positions, seq_of_token, block_table, bt_stride, page_size,
                                  page_stride, T, nh, nkv, hd, window, scale, softcap, r1, r2, chunk, sink, nullptr, 0,
                                  out, st);
}

// pb, keep: sigmoid weights with a bias per head, and first positions that stay visible (score_mod.h; null, 0: neither).
TQ_API int tq_attention_generic_sig(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                                    const int* seq_of_token, const int* block_table, int bt_stride, int page_size,
                                    int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale,
                                    float softcap, const float* r1, const float* r2, int chunk, const float* sink,
                                    const float* pb, int keep, void* out, hipStream_t st) {
  if (T <= 0) return 0;
  if ((r1 == nullptr) != (r2 == nullptr) || chunk < 0 || softcap < 0.f || keep < 0 || (pb && sink)) return TQ_ERR_BAD_ARG;
  const ScoreMod mod{softcap, r1, r2, chunk, sink, pb, keep};
  if (hd > 4 * CHUNK || nkv <= 0 || nh % nkv != 0) return TQ_ERR_UNSUPPORTED;
  if (nh > 65535) return TQ_ERR_UNSUPPORTED;
  const size_t shmem = (size_t)(hd + CHUNK + 4) * sizeof(float) + CHUNK * (sizeof(int64_t) + sizeof(int));
  hipLaunchKernelGGL(attention_generic_kernel, dim3(T, nh), dim3(CHUNK), shmem, st, (const act_t*)q,
                     (const act_t*)k_pool, (const act_t*)v_pool, positions, seq_of_token, block_table, bt_stride,
                     page_size, page_stride, nh, nkv, hd, window, scale, mod, (act_t*)out);
  TQ_LAUNCH_CHECK();
  return 0;
}

TQ_API int tq_attention_generic(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                                const int* seq_of_token, const int* block_table, int bt_stride, int page_size,
                                int64_t page_stride, int T, int nh, int nkv, int hd, int window, float scale,
                                void* out, hipStream_t st) {
  return tq_attention_generic_mod(q, k_pool, v_pool, positions, seq_of_token, block_table, bt_stride, page_size,
                                  page_stride, T, nh, nkv, hd, window, scale, 0.f, nullptr, nullptr, 0, nullptr, out, st);
}
