// Paged causal attention with float32 arithmetic for any head size, block size,
// head grouping and window: one workgroup per (query row, query head), used for
// prompt portions and decoded tokens alike. It is the true 32-bit path and the
// fallback for shapes the MFMA kernels refuse.
//
// Query row t of sequence s sits at position pos = ctx[s] - n_new[s] + (t - qs[s])
// and reads keys start..pos through the sequence's block table, where start = 0
// or pos - window + 1; query head h reads KV head h / (H / KVH). Scores are
// scale * (q . k); the softmax is the online form over chunks of 256 keys, with
// running maximum, sum and accumulator in float32
// (reference: src/backend/cpu/cpu_backend.cpp:261-319, which walks key by key).
// The chunks start at `start`, so what is computed for a position depends only
// on that position's keys - not on how the tokens were cut into steps, on the
// other sequences of the batch, or on which pages hold the keys.
#include "common.h"

#include <math.h>

#define AT 256  // threads per workgroup = keys per chunk

template <typename TC>
__device__ __forceinline__ float dot_row(const float* __restrict__ q_s, const TC* __restrict__ k, int Dh) {
  float dot = 0.f;
  for (int d = 0; d < Dh; ++d) dot = fmaf(q_s[d], load_as_float(k + d), dot);
  return dot;
}

template <typename TQ, typename TC, typename TO>
__global__ __launch_bounds__(AT) void paged_attention_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache, TO* __restrict__ out,
    const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ seq_of_row, int H, int KVH, int Dh,
    int block_size, int max_blocks, float scale, int window) {
  extern __shared__ float smem[];
  const int groups = Dh >= AT ? 1 : AT / Dh;          // key groups that accumulate P.V side by side
  float* q_s = smem;                                  // [Dh]
  float* p_s = q_s + Dh;                              // [AT]
  float* acc_s = p_s + AT;                            // [groups * Dh]
  float* scratch = acc_s + groups * Dh;               // [16]

  const int t = blockIdx.y;
  const int h = blockIdx.x;
  const int tid = threadIdx.x;
  const int s = seq_of_row[t];
  const int n_new = query_start[s + 1] - query_start[s];
  const int pos = context_lens[s] - n_new + (t - query_start[s]);
  const int start = window > 0 ? max(0, pos - window + 1) : 0;
  const int kvh = h / (H / KVH);
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  const TQ* qr = q + (static_cast<size_t>(t) * H + h) * Dh;
  for (int d = tid; d < Dh; d += AT) q_s[d] = load_as_float(qr + d);
  __syncthreads();

  const bool wide = Dh > AT;                          // each thread then owns dims tid and tid + AT
  const int g = wide ? 0 : tid / Dh;
  const int d0 = wide ? tid : tid % Dh;
  const bool active = wide ? (tid < Dh) : (tid < groups * Dh);

  float m = -INFINITY, l = 0.f, acc0 = 0.f, acc1 = 0.f;
  for (int base = start; base <= pos; base += AT) {
    const int j = base + tid;
    float sc = -INFINITY;
    if (j <= pos) {
      const size_t off =
          ((static_cast<size_t>(table[j / block_size]) * KVH + kvh) * block_size + j % block_size) * Dh;
      sc = scale * dot_row(q_s, k_cache + off, Dh);
    }
    const float cmax = block_max(sc, scratch);
    const float m_new = fmaxf(m, cmax);
    const float corr = expf(m - m_new);               // exp(-inf) = 0 on the first chunk
    const float p = (j <= pos) ? expf(sc - m_new) : 0.f;
    p_s[tid] = p;
    const float csum = block_sum(p, scratch);         // its barriers also publish p_s
    l = l * corr + csum;
    acc0 *= corr;
    acc1 *= corr;
    m = m_new;
    const int nkeys = min(AT, pos - base + 1);
    if (active) {
      for (int jj = g; jj < nkeys; jj += groups) {
        const int j2 = base + jj;
        // values lie transposed inside a page: [page][kv head][dim][offset]
        const TC* vr = v_cache + (static_cast<size_t>(table[j2 / block_size]) * KVH + kvh) * Dh * block_size +
                       j2 % block_size;
        const float pj = p_s[jj];
        acc0 = fmaf(pj, load_as_float(vr + static_cast<size_t>(d0) * block_size), acc0);
        if (wide && d0 + AT < Dh) acc1 = fmaf(pj, load_as_float(vr + static_cast<size_t>(d0 + AT) * block_size), acc1);
      }
    }
    __syncthreads();                                  // p_s is rewritten by the next chunk
  }

  TO* o = out + (static_cast<size_t>(t) * H + h) * Dh;
  if (wide) {
    if (tid < Dh) store_from_float(o + tid, acc0 / l);
    if (tid + AT < Dh) store_from_float(o + tid + AT, acc1 / l);
    return;
  }
  if (active) acc_s[g * Dh + d0] = acc0;
  __syncthreads();
  if (tid < Dh) {
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += acc_s[gg * Dh + tid];
    store_from_float(o + tid, total / l);
  }
}

extern "C" int tie_paged_attention_generic(const void* q, int q_dtype, const void* k_cache, const void* v_cache,
                                           int cache_dtype, void* out, int out_dtype, const int* query_start,
                                           const int* context_lens, const int* block_tables,
                                           const int* seq_of_row, int T, int H, int KVH, int Dh, int block_size,
                                           int max_blocks, float scale, int window, hipStream_t stream) {
  if (T <= 0 || T > 65535 || H <= 0 || KVH <= 0 || H % KVH != 0 || Dh <= 0 || Dh > 2 * AT || block_size <= 0 ||
      max_blocks <= 0)
    return TIE_BAD_ARGUMENT;
  const int groups = Dh >= AT ? 1 : AT / Dh;
  const size_t shared = sizeof(float) * (Dh + AT + groups * Dh + 16);
  const dim3 grid(H, T);
#define LAUNCH(TQ, TC, TO)                                                                                  \
  paged_attention_generic_kernel<TQ, TC, TO><<<grid, AT, shared, stream>>>(                                  \
      static_cast<const TQ*>(q), static_cast<const TC*>(k_cache), static_cast<const TC*>(v_cache),          \
      static_cast<TO*>(out), query_start, context_lens, block_tables, seq_of_row, H, KVH, Dh, block_size,   \
      max_blocks, scale, window)
  if (q_dtype == TIE_F32 && cache_dtype == TIE_F32 && out_dtype == TIE_F32) LAUNCH(float, float, float);
  else if (q_dtype == TIE_BF16 && cache_dtype == TIE_BF16 && out_dtype == TIE_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (q_dtype == TIE_F32 && cache_dtype == TIE_BF16 && out_dtype == TIE_F32) LAUNCH(float, bf16_t, float);
  else if (q_dtype == TIE_F32 && cache_dtype == TIE_F16 && out_dtype == TIE_F32) LAUNCH(float, f16_t, float);
  else return TIE_BAD_ARGUMENT;
#undef LAUNCH
  return tie_launch_status();
}
