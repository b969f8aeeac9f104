// The merge of key splits, shared by the decode and the prefill attention kernels (included after
// DH is defined). A split leaves, per (row, query head), its running maximum in the exponent's units
// (base 2), its sum of weights and its unnormalised accumulator.
#pragma once

// Merges the splits of one (row, query head): m = max m_i, L = sum l_i 2^(m_i - m),
// out = sum o_i 2^(m_i - m) / L, splits in ascending order (the maxima come scaled by
// scale * log2(e), the units of the exponent). The weights 2^(m_i - m) are computed
// once by the first threads and shared through LDS.
#define MERGE_MAX_SPLITS 256
// Where the partial results of workgroup y lie and which output row they become:
//   rows given (prefill: results kept per row of the step)      slot rows[y], output row rows[y];
//   otherwise  (decode: results kept per sequence of the launch) slot y, output row
//                                                                query_start[seq_ids ? seq_ids[y] : y].
__global__ void attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                       bf16_t* __restrict__ out, const int* __restrict__ rows,
                                       const int* __restrict__ query_start, const int* __restrict__ seq_ids,
                                       int H, int nsplit) {
  __shared__ float weight[MERGE_MAX_SPLITS];
  __shared__ float weighted_sum[MERGE_MAX_SPLITS];
  __shared__ float scratch[16];
  const int h = blockIdx.x;
  const int z = rows ? rows[blockIdx.y] : static_cast<int>(blockIdx.y);
  const int t = rows ? z : query_start[seq_ids ? seq_ids[z] : z];
  const size_t slot0 = (static_cast<size_t>(z) * H + h) * nsplit;
  const int i = threadIdx.x;
  const float mi = i < nsplit ? part_ml[(slot0 + i) * 2] : -INFINITY;
  const float li = i < nsplit ? part_ml[(slot0 + i) * 2 + 1] : 0.f;
  const float m = block_max(mi, scratch);
  const float wi = (mi == -INFINITY) ? 0.f : exp2f(mi - m);
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
    for (int k = 0; k < nsplit; ++k) o += part_o[(slot0 + k) * DH + d] * weight[k];   // an empty split wrote zeros
    out[(static_cast<size_t>(t) * H + h) * DH + d] = float_to_bf16(o / L);
  }
}

// Threads of a merge workgroup: enough for one thread per split and per dimension, at most 256.
static inline int attention_merge_threads(int nsplit) {
  const int need = nsplit > DH ? nsplit : DH;
  return need <= 64 ? 64 : (need <= 128 ? 128 : 256);
}
