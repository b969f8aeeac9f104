// The plain matrix product for gfx950: out[T, N] (+)= x[T, K] . w[N, K]^T with
// float32 multiply-adds on the vector units, for any sizes and any mix of
// float32 / bfloat16 operands. It is the true 32-bit path of every projection
// and the fallback for shapes the MFMA kernels refuse. Each output element is
// summed over k in ascending order by one thread, so a row's result does not
// depend on how many other rows the call holds.
// Reference contraction: src/backend/cpu/cpu_backend.cpp:93-139 (x @ w^T, weights [out, in]).
#include "common.h"

#define GT 64   // output tile is GT x GT
#define GK 16   // k slice staged per iteration

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                           TO* __restrict__ out, int T, int N, int K,
                                                           int accumulate) {
  __shared__ float xs[GK][GT + 4];
  __shared__ float ws[GK][GT + 4];
  const int tid = threadIdx.x;
  const int row0 = blockIdx.y * GT;
  const int col0 = blockIdx.x * GT;
  const int ty = tid / 16, tx = tid % 16;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // Each thread stages 4 consecutive k of one row of each operand.
  const int lr = tid / 4;         // 0..63: row within the tile
  const int lk = (tid % 4) * 4;   // 0,4,8,12: first k within the slice

  for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int xr = row0 + lr;
      const int wr = col0 + lr;
      xs[lk + i][lr] = (xr < T && k < K) ? load_as_float(x + static_cast<size_t>(xr) * K + k) : 0.f;
      ws[lk + i][lr] = (wr < N && k < K) ? load_as_float(w + static_cast<size_t>(wr) * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c >= N) continue;
      TO* o = out + static_cast<size_t>(r) * N + c;
      float v = acc[i][j];
      if (accumulate) v = load_as_float(o) + v;
      store_from_float(o, v);
    }
  }
}

extern "C" int tie_gemm_generic(const void* x, int x_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                                int accumulate, int T, int N, int K, hipStream_t stream) {
  if (T <= 0 || N <= 0 || K <= 0) return TIE_BAD_ARGUMENT;
  if ((x_dtype | w_dtype | out_dtype) & ~1) return TIE_BAD_ARGUMENT;
  const dim3 grid((N + GT - 1) / GT, (T + GT - 1) / GT);
  if (grid.y > 65535) return TIE_BAD_ARGUMENT;
#define LAUNCH(TX, TW, TO)                                                                              \
  gemm_generic_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>(static_cast<const TX*>(x), static_cast<const TW*>(w), \
                                                            static_cast<TO*>(out), T, N, K, accumulate)
  const int key = x_dtype * 4 + w_dtype * 2 + out_dtype;
  switch (key) {
    case 0: LAUNCH(float, float, float); break;
    case 1: LAUNCH(float, float, bf16_t); break;
    case 2: LAUNCH(float, bf16_t, float); break;
    case 3: LAUNCH(float, bf16_t, bf16_t); break;
    case 4: LAUNCH(bf16_t, float, float); break;
    case 5: LAUNCH(bf16_t, float, bf16_t); break;
    case 6: LAUNCH(bf16_t, bf16_t, float); break;
    case 7: LAUNCH(bf16_t, bf16_t, bf16_t); break;
    default: return TIE_BAD_ARGUMENT;
  }
#undef LAUNCH
  return tie_launch_status();
}
