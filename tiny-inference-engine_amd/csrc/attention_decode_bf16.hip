// Paged attention for decoded tokens (one new row per sequence) on the gfx950 matrix cores,
// bfloat16 queries and cache, float32 softmax. Compiled per head size: -DHEAD_DIM=<multiple of 16>.
//
// One wave handles one (sequence, KV head, split of the keys). The G = H / KVH query heads that
// share the KV head are the 16 columns of the MFMA tiles (columns >= G are zeros), so keys and
// values are read once for the whole group. Per 32 keys:
//
//   S^T[key, g] = K[key, :] . Q[g, :]      A = K rows (16 bytes a lane, straight from the cache),
//                                          B = Q (held in registers)          2 x HEAD_DIM/32 MFMAs
//   online softmax per column g in float32: running maximum, sum, rescale of the accumulator
//   O^T[d, g]  += V^T[d, key] . P^T[key, g]   A = V^T rows (the cache keeps values transposed inside a
//                                          page, so 4 positions of one dimension are 8 bytes),
//                                          B = P, which is exactly what the lane already holds
//                                          from the first product              HEAD_DIM/16 MFMAs
//
// Nothing passes through LDS and no lane ever needs another lane's scores. Splits of the keys
// run as separate waves; a second kernel merges their (maximum, sum, accumulator) triples in a
// fixed order. Keys are always cut at multiples of 32 positions, so what is computed for a
// position does not depend on the batch around it.
//
// Formula: src/backend/cpu/cpu_backend.cpp:261-319 (score = scale * q.k, causal by position,
// online softmax, query head h reads KV head h / (H / KVH)).
#include "common.h"

#include <math.h>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int DH = HEAD_DIM;
constexpr int KSTEPS = (DH + 31) / 32;  // k blocks of the first product
constexpr int DTILES = DH / 16;         // row tiles of the second product

union Frag {
  bf16x8_t v;
  uint4 u4;
  uint2 u2[2];
  bf16_t h[8];
};

__global__ __launch_bounds__(TIE_WAVE) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ seq_ids, int H, int KVH, int block_size,
    int max_blocks, float scale, int window, int nsplit) {
  const int lane = threadIdx.x;
  const int col = lane & 15;   // query head within the group (column of every tile)
  const int quad = lane >> 4;  // 0..3
  const int split = blockIdx.x;
  const int kvh = blockIdx.y;
  const int s = seq_ids ? seq_ids[blockIdx.z] : blockIdx.z;
  const int G = H / KVH;
  const int t = query_start[s];            // the sequence's single new row
  const int pos = context_lens[s] - 1;     // its position; keys start..pos are read
  const int start = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  // Tiles of 32 keys at absolute positions; this split's share of them.
  const int first_tile = start / 32;
  const int num_tiles = pos / 32 + 1;
  const int per_split = (num_tiles - first_tile + nsplit - 1) / nsplit;
  const int tile_begin = first_tile + split * per_split;
  const int tile_end = min(num_tiles, tile_begin + per_split);

  // Q as the B operand: lane (col = g, quad) holds Q[g][step*32 + quad*8 .. +8].
  Frag qf[KSTEPS];
  {
    const bool valid = col < G;
    const bf16_t* qr = q + (static_cast<size_t>(t) * H + static_cast<size_t>(kvh) * G + (valid ? col : 0)) * DH;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      const int d = st * 32 + quad * 8;
      qf[st].u4 = (valid && d < DH) ? *reinterpret_cast<const uint4*>(qr + d) : make_uint4(0, 0, 0, 0);
    }
  }

  floatx4 acc[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const size_t page_stride = static_cast<size_t>(KVH) * block_size * DH;   // elements of one page, K or V
  const size_t head_off = static_cast<size_t>(kvh) * block_size * DH;

  // Fragments of one 32-key tile: keys for the first product (two 16-key sub-tiles), values for the second.
  // Positions are clamped to pos for the address only; what lies beyond pos is masked in the softmax.
  auto load_keys = [&](int base, Frag (&kf)[2][KSTEPS]) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = min(base + u * 16 + col, pos);
      const bf16_t* kr = k_cache + static_cast<size_t>(table[kp / block_size]) * page_stride + head_off +
                         static_cast<size_t>(kp % block_size) * DH;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        const int d = st * 32 + quad * 8;
        kf[u][st].u4 = d < DH ? *reinterpret_cast<const uint4*>(kr + d) : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto load_values = [&](int base, Frag (&vf)[DTILES]) {
    const int k0 = min(base + quad * 4, pos);               // a run of 4 positions inside one page
    const int k1 = min(base + 16 + quad * 4, pos);
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
  };

  // The loads of tile t + 1 are issued before the arithmetic of tile t, so memory latency and the
  // matrix cores overlap.
  Frag kf[2][KSTEPS], vf[DTILES], kf_next[2][KSTEPS], vf_next[DTILES];
  if (tile_begin < tile_end) {
    load_keys(tile_begin * 32, kf_next);
    load_values(tile_begin * 32, vf_next);
  }
  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const int base = tile * 32;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) kf[u][st] = kf_next[u][st];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) vf[dt] = vf_next[dt];
    if (tile + 1 < tile_end) {
      load_keys(base + 32, kf_next);
      load_values(base + 32, vf_next);
    }
    // ---- first product: two 16-key tiles
    floatx4 sc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      sc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st)
        sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][st].v, qf[st].v, sc[u], 0, 0, 0);
    }
    // ---- softmax of this lane's column over its 8 keys, then across the four quads
    float sv[8];
    float tile_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int kp = base + u * 16 + quad * 4 + v;
        const float x = (kp <= pos && kp >= start) ? sc[u][v] * scale : -INFINITY;
        sv[u * 4 + v] = x;
        tile_max = fmaxf(tile_max, x);
      }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, TIE_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, TIE_WAVE));
    const float m_new = fmaxf(m, tile_max);
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    Frag pf;
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = (sv[i] == -INFINITY) ? 0.f : expf(sv[i] - m_new);
      psum += p;
      pf.h[i] = float_to_bf16(p);
    }
    l = l * corr + psum;
    m = m_new;
    // ---- second product
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[dt][v] *= corr;
      acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, acc[dt], 0, 0, 0);
    }
  }

  // The column's sum over all keys of this split.
  l += __shfl_xor(l, 16, TIE_WAVE);
  l += __shfl_xor(l, 32, TIE_WAVE);
  if (col >= G) return;
  const int h = kvh * G + col;
  if (nsplit == 1) {  // no merge needed: normalise and store
    bf16_t* o = out + (static_cast<size_t>(t) * H + h) * DH;
    const float inv = 1.0f / l;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
      for (int v = 0; v < 4; ++v) o[dt * 16 + quad * 4 + v] = float_to_bf16(acc[dt][v] * inv);
    return;
  }
  const size_t slot = (static_cast<size_t>(blockIdx.z) * H + h) * nsplit + split;
  float* po = part_o + slot * DH;
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt)
    *reinterpret_cast<float4*>(po + dt * 16 + quad * 4) = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
  if (quad == 0) {
    part_ml[slot * 2] = m;
    part_ml[slot * 2 + 1] = l;
  }
}

// Merges the splits of one (sequence, query head): m = max m_i, L = sum l_i e^(m_i - m),
// out = sum o_i e^(m_i - m) / L, splits in ascending order. The weights e^(m_i - m) are computed
// once by the first threads and shared through LDS.
#define MERGE_MAX_SPLITS 256
__global__ void attention_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              bf16_t* __restrict__ out, const int* __restrict__ query_start,
                                              const int* __restrict__ seq_ids, int H, int nsplit) {
  __shared__ float weight[MERGE_MAX_SPLITS];
  __shared__ float weighted_sum[MERGE_MAX_SPLITS];
  __shared__ float scratch[16];
  const int h = blockIdx.x;
  const int z = blockIdx.y;
  const int s = seq_ids ? seq_ids[z] : z;
  const int t = query_start[s];
  const size_t slot0 = (static_cast<size_t>(z) * H + h) * nsplit;
  const int i = threadIdx.x;
  const float mi = i < nsplit ? part_ml[(slot0 + i) * 2] : -INFINITY;
  const float li = i < nsplit ? part_ml[(slot0 + i) * 2 + 1] : 0.f;
  const float m = block_max(mi, scratch);
  const float wi = (mi == -INFINITY) ? 0.f : expf(mi - m);
  if (i < nsplit) {
    weight[i] = wi;
    weighted_sum[i] = wi * li;
  }
  __syncthreads();
  float L = 0.f;
  for (int k = 0; k < nsplit; ++k) L += weighted_sum[k];   // ascending order, the same in every thread
  for (int d = threadIdx.x; d < DH; d += blockDim.x) {
    float o = 0.f;
#pragma unroll 8
    for (int k = 0; k < nsplit; ++k) o += part_o[(slot0 + k) * DH + d] * weight[k];
    out[(static_cast<size_t>(t) * H + h) * DH + d] = float_to_bf16(o / L);
  }
}

extern "C" int tie_attention_decode_head_dim() { return DH; }

extern "C" int tie_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                         float* part_o, float* part_ml, const int* query_start,
                                         const int* context_lens, const int* block_tables, const int* seq_ids,
                                         int num_seqs, int H, int KVH, int block_size, int max_blocks, float scale,
                                         int window, int nsplit, hipStream_t stream) {
  if (num_seqs <= 0 || num_seqs > 65535 || H <= 0 || KVH <= 0 || KVH > 65535 || H % KVH != 0 || H / KVH > 16 ||
      block_size <= 0 || block_size % 4 != 0 || max_blocks <= 0 || nsplit <= 0 || nsplit > MERGE_MAX_SPLITS)
    return TIE_BAD_ARGUMENT;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr)) return TIE_BAD_ARGUMENT;
  const dim3 grid(nsplit, KVH, num_seqs);
  attention_decode_kernel<<<grid, TIE_WAVE, 0, stream>>>(
      static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache),
      static_cast<bf16_t*>(out), part_o, part_ml, query_start, context_lens, block_tables, seq_ids, H, KVH,
      block_size, max_blocks, scale, window, nsplit);
  int status = tie_launch_status();
  if (status != TIE_OK || nsplit == 1) return status;
  const int merge_threads = (nsplit > DH ? nsplit : DH) <= 64 ? 64 : ((nsplit > DH ? nsplit : DH) <= 128 ? 128 : 256);
  attention_decode_merge_kernel<<<dim3(H, num_seqs), merge_threads, 0, stream>>>(
      part_o, part_ml, static_cast<bf16_t*>(out), query_start, seq_ids, H, nsplit);
  return tie_launch_status();
}
