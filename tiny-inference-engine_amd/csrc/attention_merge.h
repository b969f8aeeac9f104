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
    for (int k = 0; k < nsplit; ++k) {
      // every load is asked for whatever the weight (they are in flight together); a split without weight is
      // empty and may have written nothing, so what came back for it is not used
      const float p = part_o[(slot0 + k) * DH + d];
      o += (weight[k] != 0.f ? p : 0.f) * weight[k];
    }
    out[(static_cast<size_t>(t) * H + h) * DH + d] = float_to_bf16(o / L);
  }
}

// Threads of a merge workgroup: enough for one thread per split and per dimension, at most 256.
static inline int attention_merge_threads(int nsplit) {
  const int need = nsplit > DH ? nsplit : DH;
  return need <= 64 ? 64 : (need <= 128 ? 128 : 256);
}

// The same merge with one wave per (row, query head), for up to 64 splits: lane k holds split k's maximum
// and sum, the weights travel by lane broadcast, no LDS and no barrier; a workgroup of four waves takes four
// pairs. The operations and their order are those of the kernel above, so the results are the same bits.
// Used for up to MERGE_WAVE_SPLITS splits, where thousands of rows (prompt portions) merge faster this way
// (2048 rows in 2 shares: 26 against 46 us; 512 rows in 4 shares: 6 against 14); with 8 or more shares the
// kernel above, with twice the waves, keeps more loads in flight and wins.
#define MERGE_WAVES 4
#define MERGE_WAVE_SPLITS 4
__global__ __launch_bounds__(MERGE_WAVES* TIE_WAVE) void attention_merge_wave_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int* __restrict__ rows, const int* __restrict__ query_start, const int* __restrict__ seq_ids, int H,
    int nsplit, int num_pairs) {
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int pair = blockIdx.x * MERGE_WAVES + threadIdx.x / TIE_WAVE;   // (y, h), h fastest
  if (pair >= num_pairs) return;                                        // whole waves leave
  const int y = pair / H, h = pair % H;
  const int z = rows ? rows[y] : y;
  const int t = rows ? z : query_start[seq_ids ? seq_ids[z] : z];
  const size_t slot0 = (static_cast<size_t>(z) * H + h) * nsplit;
  const float mi = lane < nsplit ? part_ml[(slot0 + lane) * 2] : -INFINITY;
  const float li = lane < nsplit ? part_ml[(slot0 + lane) * 2 + 1] : 0.f;
  const float m = wave_max(mi);
  const float wi = (mi == -INFINITY) ? 0.f : exp2f(mi - m);
  const float wli = wi * li;
  float L = 0.f;
  for (int k = 0; k < nsplit; ++k) L += __shfl(wli, k, TIE_WAVE);       // ascending order
  const float* po = part_o + slot0 * DH;
  bf16_t* o = out + (static_cast<size_t>(t) * H + h) * DH;
  // Every lane walks the loop (the broadcasts read all lanes); lanes beyond the head size read dimension 0
  // and store nothing.
#pragma unroll
  for (int d0 = 0; d0 < DH; d0 += 2 * TIE_WAVE) {
    const int d = d0 + lane * 2;
    const int dr = d < DH ? d : 0;
    float o0 = 0.f, o1 = 0.f;
#pragma unroll 8
    for (int k = 0; k < nsplit; ++k) {
      const float w = __shfl(wi, k, TIE_WAVE);
      const float2 p = *reinterpret_cast<const float2*>(po + static_cast<size_t>(k) * DH + dr);
      o0 += (w != 0.f ? p.x : 0.f) * w;   // a split without weight is empty and may have written nothing
      o1 += (w != 0.f ? p.y : 0.f) * w;
    }
    if (d < DH) *reinterpret_cast<uint32_t*>(o + d) = pack_bf16x2(o0 / L, o1 / L);
  }
}

// Launches the merge of `count` (row or sequence) x H pairs on the kernel that suits the number of splits.
static inline void launch_attention_merge(const float* part_o, const float* part_ml, bf16_t* out, const int* rows,
                                          const int* query_start, const int* seq_ids, int H, int nsplit, int count,
                                          hipStream_t stream) {
  if (nsplit <= MERGE_WAVE_SPLITS) {
    const int pairs = count * H;
    attention_merge_wave_kernel<<<(pairs + MERGE_WAVES - 1) / MERGE_WAVES, MERGE_WAVES * TIE_WAVE, 0, stream>>>(
        part_o, part_ml, out, rows, query_start, seq_ids, H, nsplit, pairs);
  } else {
    attention_merge_kernel<<<dim3(H, count), attention_merge_threads(nsplit), 0, stream>>>(
        part_o, part_ml, out, rows, query_start, seq_ids, H, nsplit);
  }
}
