// Drawing a token from a row of logits with top-k and top-p, on the GPU: one workgroup a row.
//
// The rules are src/sampling/sampler.cpp:35-80: s_i = (l_i - max) * (1 / temperature) in float32; with
// 0 < top_k < V only the top_k most likely stay, in the order (value descending, id ascending); weights
// w_i = exp(s_i) (the maximum maps to 1); with top_p < 1 the smallest prefix of that order whose weight reaches
// top_p * total stays; one uniform number u picks the first candidate at which the running sum exceeds
// u * (what stayed).
//
// No sort. With key_i = bits(s_i), sign cleared (s_i <= 0, so keys ascend as likelihood falls), the order of the
// candidates is the order of the 50-bit numbers c_i = key_i << 19 | i, and all three questions are one: the
// first c at which a running sum (of ones for top-k, of weights for top-p and for the draw) over the candidates
// c_i <= limit reaches a target. That c is found digit by digit from histograms of the sums. The first
// histogram, over the whole row, is by a coarse, even scale (buckets of 1/64 in s, which ascend with the keys);
// the candidates of the bucket it points to are copied to LDS, and the five digits of 10 bits that fix c are
// found there. Once a limit is known and few enough candidates lie within it (top-k at most 8192, or a top-p
// nucleus of that size), they are all copied to LDS and the row is not read again. A bucket that does not fit
// LDS (a row of equal logits) is searched in the row itself, five passes more.
//
// Sums are integers (weights in units of 2^-44, truncated): adding them in any order gives the same bits, so
// the histograms may be filled with atomic additions in LDS and the result is the same in every run. A row of
// 2^19 tokens of weight 1 still fits 64 bits. Against sums in double precision this moves a boundary by at most
// 1e-8 of the total, and weights below 2^-44 of the largest count as nothing.
//
// out[r] = -1 for a row with a NaN, -2 for a row that is all -inf; a +inf logit wins outright (the lowest id).
#include "common.h"

#include <math.h>
#include <stdint.h>

#define SF_THREADS 1024
#define SF_BUCKETS 2048                // of the coarse scale
#define SF_PER_UNIT 64.0f              // of them per unit of s: they cover [0, 32), where the weights are not 0
#define SF_DIGIT 1024                  // 10 bits of c at a time
#define SF_CAP 8192                    // candidates that LDS holds
#define SF_ID_BITS 19
#define SF_UNIT 17592186044416.0f      // 2^44
typedef unsigned long long sf_u64;

enum { SF_TOPK, SF_TOPP, SF_DRAW };

struct SfRow {
  const float* row;
  int V;
  float mx, inv_t;
  bool by_four;             // the row starts on 16 bytes
};
// The candidates: c <= limit; `listed`: they are list[0 .. n), and the row need not be read.
struct SfCandidates {
  sf_u64 limit;
  int n;
  bool listed;
};

__device__ __forceinline__ uint32_t sf_key(const SfRow& r, float v) {
  return __float_as_uint((v - r.mx) * r.inv_t) & 0x7fffffffu;
}
__device__ __forceinline__ sf_u64 sf_number(uint32_t key, int id) {
  return (static_cast<sf_u64>(key) << SF_ID_BITS) | static_cast<uint32_t>(id);
}
// Weight of a key in units of 2^-44 (the key is the scaled logit's bits with the sign cleared: the logit is -key).
__device__ __forceinline__ sf_u64 sf_weight(uint32_t key) {
  return static_cast<sf_u64>(expf(-__uint_as_float(key)) * SF_UNIT);
}
// Never falls as the key grows.
__device__ __forceinline__ int sf_bucket(uint32_t key) {
  const float a = __uint_as_float(key) * SF_PER_UNIT;
  return a >= static_cast<float>(SF_BUCKETS - 1) ? SF_BUCKETS - 1 : static_cast<int>(a);
}

// f(value, id, valid) for every logit of the row, four loads of 16 bytes in flight per thread; every thread
// makes the same number of calls (the surplus with valid = false), so f may use wave-wide operations.
template <typename F>
__device__ __forceinline__ void sf_for_each(const SfRow& r, F f) {
  const int tid = threadIdx.x;
  int done = 0;
  if (r.by_four) {
    const float4* p = reinterpret_cast<const float4*>(r.row);
    const int n4 = r.V >> 2;
    for (int j0 = 0; j0 < n4; j0 += 4 * SF_THREADS) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * SF_THREADS + tid;
        v[u] = j < n4 ? p[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * SF_THREADS + tid;
        const bool ok = j < n4;
        f(v[u].x, 4 * j, ok);
        f(v[u].y, 4 * j + 1, ok);
        f(v[u].z, 4 * j + 2, ok);
        f(v[u].w, 4 * j + 3, ok);
      }
    }
    done = n4 * 4;
  }
  for (int i0 = done; i0 < r.V; i0 += SF_THREADS) {
    const int i = i0 + tid;
    const bool ok = i < r.V;
    f(ok ? r.row[i] : 0.f, i, ok);
  }
}

// Histogram over the row's candidates: by the coarse scale (bucket < 0), or by the digit of c at `shift` among
// those of one coarse bucket whose c matches the digits known.
template <bool COUNT>
__device__ void sf_histogram_of_row(const SfRow& r, sf_u64 limit, int bucket, sf_u64 known, sf_u64 mask, int shift,
                                    sf_u64* hist) {
  for (int b = threadIdx.x; b < SF_BUCKETS; b += SF_THREADS) hist[b] = 0;
  __syncthreads();
  sf_for_each(r, [&](float v, int i, bool ok) {
    const uint32_t key = sf_key(r, v);
    const sf_u64 c = sf_number(key, i);
    const int coarse = sf_bucket(key);
    if (!ok || c > limit) return;
    if (bucket >= 0 && (coarse != bucket || (c & mask) != known)) return;
    const sf_u64 w = COUNT ? 1 : sf_weight(key);
    if (w != 0) atomicAdd(&hist[bucket < 0 ? coarse : static_cast<int>((c >> shift) & (SF_DIGIT - 1))], w);
  });
}

// The same by the digit at `shift` over the candidates in LDS.
template <bool COUNT>
__device__ void sf_histogram_of_list(const sf_u64* list, int n, sf_u64 limit, sf_u64 known, sf_u64 mask, int shift,
                                     sf_u64* hist) {
  for (int b = threadIdx.x; b < SF_DIGIT; b += SF_THREADS) hist[b] = 0;
  __syncthreads();
  for (int j = threadIdx.x; j < n; j += SF_THREADS) {
    const sf_u64 c = list[j];
    if (c > limit || (c & mask) != known) continue;
    const sf_u64 w = COUNT ? 1 : sf_weight(static_cast<uint32_t>(c >> SF_ID_BITS));
    if (w != 0) atomicAdd(&hist[(c >> shift) & (SF_DIGIT - 1)], w);
  }
}

// Copies the row's candidates (of one coarse bucket, or of all with bucket < 0) to LDS, in any order; how many
// there are, also where that is more than LDS holds (then the list is of no use).
__device__ int sf_list_from_row(const SfRow& r, sf_u64 limit, int bucket, sf_u64* list, int* list_n) {
  if (threadIdx.x == 0) *list_n = 0;
  __syncthreads();
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  sf_for_each(r, [&](float v, int i, bool ok) {
    const uint32_t key = sf_key(r, v);
    const sf_u64 c = sf_number(key, i);
    const bool take = ok && c <= limit && (bucket < 0 || sf_bucket(key) == bucket);
    const sf_u64 takers = __ballot(take);
    if (takers == 0) return;
    const int leader = __ffsll(takers) - 1;      // one addition to the counter a wave
    int start = 0;
    if (lane == leader) start = atomicAdd(list_n, __popcll(takers));
    start = __shfl(start, leader);
    if (take) {
      const int at = start + __popcll(takers & ((1ull << lane) - 1));
      if (at < SF_CAP) list[at] = c;
    }
  });
  __syncthreads();
  const int n = *list_n;
  __syncthreads();
  return n;
}

__device__ __forceinline__ sf_u64 sf_target(int mode, sf_u64 total, double x) {
  if (mode == SF_TOPK) return static_cast<sf_u64>(x);
  if (mode == SF_TOPP) {
    const sf_u64 t = static_cast<sf_u64>(ceil(x * static_cast<double>(total)));
    return t < 1 ? 1 : (t > total ? total : t);
  }
  sf_u64 below = static_cast<sf_u64>(x * static_cast<double>(total));     // the first sum that exceeds u * total
  if (below >= total) below = total - 1;
  return below + 1;
}

// The first of `nb` buckets at which base + the running sum reaches the target, and base + the sum before it.
// `decide`: the target is not known yet and follows from the sum of all buckets. Wave 0 does it: a lane sums
// its stretch of buckets, the lanes' sums are scanned, the lane in whose stretch the target falls walks it.
__device__ void sf_find_bucket(const sf_u64* hist, int nb, bool decide, int mode, double x, sf_u64* shared, sf_u64* base,
                               sf_u64* target, int* bucket) {
  __syncthreads();
  if (threadIdx.x < TIE_WAVE) {
    const int lane = threadIdx.x, per = nb / TIE_WAVE;
    sf_u64 mine = 0;
    for (int j = 0; j < per; ++j) mine += hist[lane * per + j];
    sf_u64 upto = mine;
    for (int d = 1; d < TIE_WAVE; d <<= 1) {
      const sf_u64 other = __shfl_up(upto, d);
      if (lane >= d) upto += other;
    }
    const sf_u64 total = __shfl(upto, TIE_WAVE - 1);
    const sf_u64 t = decide ? sf_target(mode, total, x) : *target;
    const sf_u64 reached = __ballot(*base + upto >= t);
    const int who = reached ? __ffsll(reached) - 1 : TIE_WAVE - 1;
    if (lane == who) {
      sf_u64 acc = *base + upto - mine;
      int b = lane * per;
      for (; b < lane * per + per - 1; ++b) {
        if (acc + hist[b] >= t) break;
        acc += hist[b];
      }
      shared[0] = acc;
      shared[1] = static_cast<sf_u64>(b);
      shared[2] = t;
    }
  }
  __syncthreads();
  *base = shared[0];
  *bucket = static_cast<int>(shared[1]);
  *target = shared[2];
  __syncthreads();
}

// The first candidate, in the order of c, at which the running sum of the weights (COUNT: of ones) reaches the
// target: k for SF_TOPK, x = top_p of all for SF_TOPP, just above x = u of all for SF_DRAW. Its c and the sum
// there. All threads call it and all get the result. A list of all candidates in LDS is left as it is; without
// one, the list is overwritten.
template <bool COUNT>
__device__ void sf_search(const SfRow& r, const SfCandidates& cand, int mode, double x, sf_u64* hist, sf_u64* list,
                          int* list_n, sf_u64* shared, sf_u64* found, sf_u64* sum_there) {
  sf_u64 base = 0, target = 0;
  bool decide = true, from_list = cand.listed;
  int n = cand.n, coarse = -1, digit;
  const sf_u64 limit = cand.limit;
  if (!from_list) {
    sf_histogram_of_row<COUNT>(r, limit, -1, 0, 0, 0, hist);
    sf_find_bucket(hist, SF_BUCKETS, true, mode, x, shared, &base, &target, &coarse);
    decide = false;
    n = sf_list_from_row(r, limit, coarse, list, list_n);
    from_list = n <= SF_CAP;
  }
  sf_u64 known = 0, mask = 0;
#pragma unroll 1
  for (int shift = 40; shift >= 0; shift -= 10) {
    if (from_list) sf_histogram_of_list<COUNT>(list, n, limit, known, mask, shift, hist);
    else sf_histogram_of_row<COUNT>(r, limit, coarse, known, mask, shift, hist);
    sf_find_bucket(hist, SF_DIGIT, decide, mode, x, shared, &base, &target, &digit);
    decide = false;
    known |= static_cast<sf_u64>(digit) << shift;
    mask |= static_cast<sf_u64>(SF_DIGIT - 1) << shift;
  }
  *found = known;
  *sum_there = base + (COUNT ? 1 : sf_weight(static_cast<uint32_t>(known >> SF_ID_BITS)));
}

__global__ __launch_bounds__(SF_THREADS) void sample_filtered_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ row_max,
                                                                     const float* __restrict__ inv_temperature,
                                                                     const double* __restrict__ uniform,
                                                                     const double* __restrict__ other_uniform,
                                                                     const int* __restrict__ take_other,
                                                                     int* __restrict__ drew_none,
                                                                     const int* __restrict__ top_k,
                                                                     const float* __restrict__ top_p,
                                                                     const int* __restrict__ rows,
                                                                     int* __restrict__ out, int V) {
  __shared__ sf_u64 hist[SF_BUCKETS];
  __shared__ sf_u64 list[SF_CAP];
  __shared__ sf_u64 shared[4];
  __shared__ float fscratch[16];
  __shared__ int flag_nan, chosen, list_n;
  const int rix = rows ? rows[blockIdx.x] : blockIdx.x, tid = threadIdx.x;
  SfRow r;
  r.row = logits + static_cast<size_t>(rix) * V;
  r.V = V;
  r.by_four = (reinterpret_cast<uintptr_t>(r.row) & 15) == 0;
  r.mx = 0.f;
  r.inv_t = 1.f;
  if (row_max) {
    // The caller looks at the maxima too: a row with a NaN or of -inf is its to report, and where the maximum
    // is +inf the argmax stands; none of them draws.
    r.mx = row_max[rix];
    if (!(r.mx > -INFINITY && r.mx < INFINITY)) {
      if (tid == 0 && drew_none) drew_none[rix] = 1;
      return;
    }
  } else {
    if (tid == 0) {
      flag_nan = 0;
      chosen = V;
    }
    __syncthreads();
    float mx = -INFINITY;
    bool nan = false;
    sf_for_each(r, [&](float v, int, bool ok) {
      if (!ok) return;
      nan |= (v != v);
      mx = fmaxf(mx, v);
    });
    if (nan) flag_nan = 1;
    mx = block_max(mx, fscratch);
    __syncthreads();
    if (tid == 0 && drew_none) drew_none[rix] = !(mx > -INFINITY && mx < INFINITY) || flag_nan;
    if (flag_nan || mx == -INFINITY) {
      if (tid == 0) out[rix] = flag_nan ? -1 : -2;
      return;
    }
    if (mx == INFINITY) {     // the lowest +inf index wins without a draw
      int first = V;
      sf_for_each(r, [&](float v, int i, bool ok) {
        if (ok && v == INFINITY) first = min(first, i);
      });
      if (first < V) atomicMin(&chosen, first);
      __syncthreads();
      if (tid == 0) out[rix] = chosen;
      return;
    }
    r.mx = mx;
  }
  r.inv_t = inv_temperature[rix];
  if (row_max && tid == 0 && drew_none) drew_none[rix] = 0;

  SfCandidates cand;
  cand.limit = ~0ull;
  cand.n = 0;
  cand.listed = false;
  sf_u64 sum, limit;
  const int k = top_k[rix];
  if (k > 0 && k < V) {
    sf_search<true>(r, cand, SF_TOPK, static_cast<double>(k), hist, list, &list_n, shared, &limit, &sum);
    cand.limit = limit;
    if (k <= SF_CAP) {
      cand.n = sf_list_from_row(r, cand.limit, -1, list, &list_n);
      cand.listed = true;
    }
  }
  const float p = top_p[rix];
  if (p < 1.0f) {
    sf_search<false>(r, cand, SF_TOPP, static_cast<double>(p), hist, list, &list_n, shared, &limit, &sum);
    cand.limit = limit;
    if (!cand.listed) {
      cand.n = sf_list_from_row(r, cand.limit, -1, list, &list_n);
      cand.listed = cand.n <= SF_CAP;
    }
  }
  sf_u64 drawn;
  const double u = take_other && take_other[rix] ? other_uniform[rix] : uniform[rix];
  sf_search<false>(r, cand, SF_DRAW, u, hist, list, &list_n, shared, &drawn, &sum);
  if (tid == 0) out[rix] = static_cast<int>(drawn & ((1u << SF_ID_BITS) - 1));
}

// top_k[r] <= 0 or >= V: no top-k; top_p[r] >= 1: no top-p. uniform[r] in [0, 1). The arrays have an entry for
// each of the R rows of `logits`; with `rows` only the `num_rows` rows it lists are drawn, and out[] of the
// others is left as it is. With `row_max` (the rows' maxima) the kernel does not look for them, and leaves out[]
// of a row whose maximum is not finite as it is. `drew_none` (optional): 1 for a row that took no uniform number
// (no finite maximum), else 0. `take_other` (optional): where it is not 0 the row's number is other_uniform[r];
// a caller that queues a step before it has read the one before passes that step's `drew_none` here, and both
// numbers the row's stream may be at.
extern "C" int tie_sample_filtered(const float* logits, const float* row_max, const float* inv_temperature,
                                   const double* uniform, const double* other_uniform, const int* take_other,
                                   int* drew_none, const int* top_k, const float* top_p, const int* rows, int num_rows,
                                   int* out, int R, int V, hipStream_t stream) {
  if (R <= 0 || V <= 0 || V > (1 << SF_ID_BITS) || (rows && (num_rows <= 0 || num_rows > R))) return TIE_BAD_ARGUMENT;
  if (take_other && !other_uniform) return TIE_BAD_ARGUMENT;
  sample_filtered_kernel<<<rows ? num_rows : R, SF_THREADS, 0, stream>>>(logits, row_max, inv_temperature, uniform,
                                                                         other_uniform, take_other, drew_none, top_k,
                                                                         top_p, rows, out, V);
  return tie_launch_status();
}
