// Paged causal attention for prompt portions (several new rows per sequence) on the gfx950 matrix
// cores: bfloat16 queries and cache, float32 softmax. Compiled per head size: -DHEAD_DIM=<multiple of 16>.
//
// It is the decode kernel's scheme with query rows as the MFMA columns. One wave owns a tile of 16
// consecutive new rows of one sequence for up to four (query head, row tile) pairs that share a KV
// head - HC heads of the group times QC row tiles - so every key and value fragment it reads from
// the cache feeds up to four column tiles. Per 32 keys and column tile c:
//
//   S^T[key, row] = K[key, :] . Q_c[row, :]     A = K rows from the cache, B = Q_c (registers)
//   online softmax per row (= per lane column) in float32, causal by position (and windowed)
//   O^T[d, row]  += V^T[d, key] . P^T[key, row]  A = V^T rows (values lie transposed in a page), B = P
//
// Keys come through the block table, so a portion attends to earlier portions and to itself alike;
// the row at new index i of a sequence sits at position ctx - n_new + i. Key tiles are cut at
// multiples of 32 positions, as in the decode kernel, so a position's result does not depend on
// how the prompt was cut into steps.
//
// Formula: src/backend/cpu/cpu_backend.cpp:261-319.
#include "common.h"

#include <math.h>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int DH = HEAD_DIM;
constexpr int KSTEPS = (DH + 31) / 32;
constexpr int DTILES = DH / 16;

union Frag {
  bf16x8_t v;
  uint4 u4;
  uint2 u2[2];
  bf16_t h[8];
};

// items: [num_items][2] = (sequence, index of its first 16-row tile handled here)
template <int HC, int QC>
__global__ __launch_bounds__(TIE_WAVE) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ items, int H, int KVH, int block_size,
    int max_blocks, float scale, int window) {
  constexpr int CT = HC * QC;
  const int lane = threadIdx.x;
  const int col = lane & 15;
  const int quad = lane >> 4;
  const int s = items[blockIdx.x * 2];
  const int tile0 = items[blockIdx.x * 2 + 1];
  const int kvh = blockIdx.y;
  const int G = H / KVH;
  const int head0 = kvh * G + blockIdx.z * HC;       // first query head of this pass
  const int heads_here = min(HC, kvh * G + G - head0);
  const int qs = query_start[s];
  const int n_new = query_start[s + 1] - qs;
  const int ctx = context_lens[s];
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  // Column tile c = (head hc, row tile qc): this lane's row and position in each.
  int row[CT], pos[CT], lo[CT];
  bool valid[CT];
  Frag qf[CT][KSTEPS];
  int pos_last = -1, pos_first = 0x7fffffff;
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hc = c / QC, qc = c % QC;
    const int i = (tile0 + qc) * 16 + col;              // new-row index within the sequence
    valid[c] = i < n_new && hc < heads_here;
    row[c] = qs + i;
    pos[c] = valid[c] ? ctx - n_new + i : -1;
    lo[c] = (window > 0 && valid[c]) ? max(0, pos[c] - window + 1) : 0;
    const bf16_t* qr = q + (static_cast<size_t>(valid[c] ? row[c] : qs) * H + head0 + (valid[c] ? hc : 0)) * DH;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      const int d = st * 32 + quad * 8;
      qf[c][st].u4 = (valid[c] && d < DH) ? *reinterpret_cast<const uint4*>(qr + d) : make_uint4(0, 0, 0, 0);
    }
    if (valid[c]) {
      pos_last = max(pos_last, pos[c]);
      pos_first = min(pos_first, lo[c]);
    }
  }
  // The wave's key range covers every lane's rows.
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    pos_last = max(pos_last, __shfl_xor(pos_last, off, TIE_WAVE));
    pos_first = min(pos_first, __shfl_xor(pos_first, off, TIE_WAVE));
  }
  if (pos_last < 0) return;

  floatx4 acc[CT][DTILES];
  float m[CT], l[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    m[c] = -INFINITY;
    l[c] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) acc[c][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const size_t page_stride = static_cast<size_t>(KVH) * block_size * DH;
  const size_t head_off = static_cast<size_t>(kvh) * block_size * DH;

  for (int tile = pos_first / 32; tile <= pos_last / 32; ++tile) {
    const int base = tile * 32;
    Frag kf[2][KSTEPS];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = min(base + u * 16 + col, pos_last);
      const bf16_t* kr = k_cache + static_cast<size_t>(table[kp / block_size]) * page_stride + head_off +
                         static_cast<size_t>(kp % block_size) * DH;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        const int d = st * 32 + quad * 8;
        kf[u][st].u4 = d < DH ? *reinterpret_cast<const uint4*>(kr + d) : make_uint4(0, 0, 0, 0);
      }
    }
    Frag vf[DTILES];
    {
      const int k0 = min(base + quad * 4, pos_last);
      const int k1 = min(base + 16 + quad * 4, pos_last);
      const bf16_t* v0 = v_cache + static_cast<size_t>(table[k0 / block_size]) * page_stride + head_off +
                         (k0 % block_size) / 4 * 4;
      const bf16_t* v1 = v_cache + static_cast<size_t>(table[k1 / block_size]) * page_stride + head_off +
                         (k1 % block_size) / 4 * 4;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
        const size_t d_off = static_cast<size_t>(dt * 16 + col) * block_size;
        vf[dt].u2[0] = *reinterpret_cast<const uint2*>(v0 + d_off);
        vf[dt].u2[1] = *reinterpret_cast<const uint2*>(v1 + d_off);
      }
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      floatx4 sc[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        sc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st)
          sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][st].v, qf[c][st].v, sc[u], 0, 0, 0);
      }
      float sv[8];
      float tile_max = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int kp = base + u * 16 + quad * 4 + v;
          const float x = (kp <= pos[c] && kp >= lo[c]) ? sc[u][v] * scale : -INFINITY;
          sv[u * 4 + v] = x;
          tile_max = fmaxf(tile_max, x);
        }
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, TIE_WAVE));
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, TIE_WAVE));
      const float m_new = fmaxf(m[c], tile_max);
      const float corr = (m[c] == -INFINITY) ? 0.f : expf(m[c] - m_new);
      Frag pf;
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = (sv[i] == -INFINITY) ? 0.f : expf(sv[i] - m_new);
        psum += p;
        pf.h[i] = float_to_bf16(p);
      }
      l[c] = l[c] * corr + psum;
      m[c] = m_new;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[c][dt][v] *= corr;
        acc[c][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, acc[c][dt], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int c = 0; c < CT; ++c) {
    float total = l[c];
    total += __shfl_xor(total, 16, TIE_WAVE);
    total += __shfl_xor(total, 32, TIE_WAVE);
    if (!valid[c]) continue;
    const int hc = c / QC;
    bf16_t* o = out + (static_cast<size_t>(row[c]) * H + head0 + hc) * DH;
    const float inv = 1.0f / total;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
      Frag r;
#pragma unroll
      for (int v = 0; v < 4; ++v) r.h[v] = float_to_bf16(acc[c][dt][v] * inv);
      *reinterpret_cast<uint2*>(o + dt * 16 + quad * 4) = r.u2[0];
    }
  }
}

// Rows of new tokens one work item covers, for a model with G query heads per KV head.
extern "C" int tie_attention_prefill_rows_per_item(int G) {
  const int hc = G >= 4 ? 4 : G;
  return 16 * (4 / hc >= 1 ? 4 / hc : 1);
}

extern "C" int tie_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                          const int* query_start, const int* context_lens, const int* block_tables,
                                          const int* items, int num_items, int H, int KVH, int block_size,
                                          int max_blocks, float scale, int window, hipStream_t stream) {
  if (num_items <= 0 || H <= 0 || KVH <= 0 || KVH > 65535 || H % KVH != 0 || block_size <= 0 || block_size % 4 != 0 ||
      max_blocks <= 0)
    return TIE_BAD_ARGUMENT;
  const int G = H / KVH;
  const int hc = G >= 4 ? 4 : G;
  const int passes = (G + hc - 1) / hc;
  if (passes > 65535) return TIE_BAD_ARGUMENT;
  const dim3 grid(num_items, KVH, passes);
#define LAUNCH(HC, QC)                                                                                        \
  attention_prefill_kernel<HC, QC><<<grid, TIE_WAVE, 0, stream>>>(                                             \
      static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), \
      static_cast<bf16_t*>(out), query_start, context_lens, block_tables, items, H, KVH, block_size,          \
      max_blocks, scale, window)
  if (hc == 4) LAUNCH(4, 1);
  else if (hc == 3) LAUNCH(3, 1);
  else if (hc == 2) LAUNCH(2, 2);
  else LAUNCH(1, 4);
#undef LAUNCH
  return tie_launch_status();
}
