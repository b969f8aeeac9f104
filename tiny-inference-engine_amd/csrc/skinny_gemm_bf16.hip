// The decode-time matrix product for gfx950: out[M, N] (+)= x[M, K] . w[N, K]^T for few rows M
// (1..64), bfloat16 operands, float32 accumulation on v_mfma_f32_16x16x32_bf16.
//
// The product is bound by reading w once from HBM, so the kernel is built around that stream:
// a workgroup of four (or eight) waves owns 16 rows of w; the waves split K into contiguous ranges;
// every lane reads 16 bytes of "its" row per MFMA (row = lane % 16, k-chunk = lane / 16), which
// is exactly the B-operand layout, so weights go from memory to the matrix core with no staging.
// The few rows of x are the A operand, read through the caches (they are shared by every
// workgroup); rows beyond M are zeros. The waves' partial sums meet in LDS and are added in a fixed
// order, so the result does not depend on timing. M > 16 runs 2 or 4 row tiles of x against each
// weight fragment.
//
// Requires K % 8 == 0 (16-byte loads); other shapes go to the generic kernel.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define SK_UNROLL 4

__device__ __forceinline__ bf16x8_t load_frag(const bf16_t* p) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  return *reinterpret_cast<const bf16x8_t*>(&v);
}

__device__ __forceinline__ bf16x8_t zero_frag() {
  const uint4 v = make_uint4(0, 0, 0, 0);
  return *reinterpret_cast<const bf16x8_t*>(&v);
}

template <int MT, typename TO, int SK_WAVES>
__global__ __launch_bounds__(SK_WAVES* TIE_WAVE) void skinny_gemm_kernel(const bf16_t* __restrict__ x,
                                                                         const bf16_t* __restrict__ w,
                                                                         TO* __restrict__ out, int M, int N, int K,
                                                                         int accumulate, int gated) {
  __shared__ float red[SK_WAVES][MT][256];
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = threadIdx.x / TIE_WAVE;
  const int r = lane & 15;   // row of the 16-row tile (of w for B, of x for A)
  const int g = lane >> 4;   // which 8-element chunk of the 32-wide k block
  const int n0 = blockIdx.x * 16;

  // Rows beyond N are clamped for the loads; their columns are dropped at the store.
  const bf16_t* wp = w + static_cast<size_t>(min(n0 + r, N - 1)) * K;
  const bf16_t* xp[MT];
  bool xvalid[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    xvalid[mt] = m < M;
    xp[mt] = x + static_cast<size_t>(xvalid[mt] ? m : 0) * K;
  }

  // This wave's k range, in blocks of 32.
  const int kblocks = (K + 31) / 32;
  const int per_wave = (kblocks + SK_WAVES - 1) / SK_WAVES;
  const int kb_begin = wave * per_wave;
  const int kb_end = min(kblocks, kb_begin + per_wave);

  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  int kb = kb_begin;
  // Main loop: SK_UNROLL blocks at a time, all loads issued before the first MFMA.
  for (; kb + SK_UNROLL <= kb_end && (kb + SK_UNROLL) * 32 <= K; kb += SK_UNROLL) {
    bf16x8_t b[SK_UNROLL];
    bf16x8_t a[MT][SK_UNROLL];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = (kb + u) * 32 + g * 8;
      b[u] = load_frag(wp + k);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[mt][u] = xvalid[mt] ? load_frag(xp[mt] + k) : zero_frag();
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt][u], b[u], acc[mt], 0, 0, 0);
  }
  // Remainder, one block at a time; the last block may be partly or wholly beyond K.
  for (; kb < kb_end; ++kb) {
    const int k = kb * 32 + g * 8;
    const bool kvalid = k < K;  // K % 8 == 0: a chunk is whole or absent
    const bf16x8_t b = kvalid ? load_frag(wp + k) : zero_frag();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8_t a = (kvalid && xvalid[mt]) ? load_frag(xp[mt] + k) : zero_frag();
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
    }
  }

  // D layout: lane holds rows (lane / 16) * 4 + v of x, column lane % 16 of w.
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][mt][(g * 4 + v) * 16 + r] = acc[mt][v];
  __syncthreads();

  for (int e = threadIdx.x; e < 256; e += SK_WAVES * TIE_WAVE) {  // 16 x 16 outputs of a tile
    const int c = e & 15;
    const int n = n0 + c;
    if (n >= N) continue;
    if (gated && c >= 8) continue;       // gated: columns 0..7 are gates, 8..15 the ups of the same outputs
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + (e >> 4);
      if (m >= M) continue;
      float sum = red[0][mt][e];
#pragma unroll
      for (int wv = 1; wv < SK_WAVES; ++wv) sum += red[wv][mt][e];
      if (gated) {
        float up = red[0][mt][e + 8];
#pragma unroll
        for (int wv = 1; wv < SK_WAVES; ++wv) up += red[wv][mt][e + 8];
        store_from_float(out + static_cast<size_t>(m) * (N / 2) + blockIdx.x * 8 + c, sum / (1.0f + __expf(-sum)) * up);
        continue;
      }
      TO* o = out + static_cast<size_t>(m) * N + n;
      if (accumulate) sum = load_as_float(o) + sum;
      store_from_float(o, sum);
    }
  }
}

// gated: w holds blocks of 16 rows = 8 gate rows then 8 up rows of the same 8 outputs; out has N / 2 columns
// and receives silu(gate) * up.
extern "C" int tie_skinny_gemm_bf16(const void* x, const void* w, void* out, int out_dtype, int accumulate, int gated,
                                    int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || K % 8 != 0) return TIE_BAD_ARGUMENT;
  if (gated && (accumulate || N % 16 != 0)) return TIE_BAD_ARGUMENT;
  const dim3 grid((N + 15) / 16);
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  // Few workgroups (small N) or long rows: eight waves a workgroup keep more loads in flight.
  const bool wide = grid.x <= 512 || K >= 8192;   // by the shape of w alone: every M sums in the same order
#define LAUNCH(MT, TO, WAVES)                                                                                   \
  skinny_gemm_kernel<MT, TO, WAVES><<<grid, WAVES * TIE_WAVE, 0, stream>>>(                                      \
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<TO*>(out), M, N, K, accumulate, gated)
  if (out_dtype == TIE_F32) {
    if (wide) { if (mt == 1) LAUNCH(1, float, 8); else if (mt == 2) LAUNCH(2, float, 8); else LAUNCH(4, float, 8); }
    else { if (mt == 1) LAUNCH(1, float, 4); else if (mt == 2) LAUNCH(2, float, 4); else LAUNCH(4, float, 4); }
  } else if (out_dtype == TIE_BF16) {
    if (wide) { if (mt == 1) LAUNCH(1, bf16_t, 8); else if (mt == 2) LAUNCH(2, bf16_t, 8); else LAUNCH(4, bf16_t, 8); }
    else { if (mt == 1) LAUNCH(1, bf16_t, 4); else if (mt == 2) LAUNCH(2, bf16_t, 4); else LAUNCH(4, bf16_t, 4); }
  } else {
    return TIE_BAD_ARGUMENT;
  }
#undef LAUNCH
  return tie_launch_status();
}
