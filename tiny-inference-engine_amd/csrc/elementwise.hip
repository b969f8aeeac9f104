// Row-wise and element-wise kernels for gfx950: embedding gather, RMSNorm,
// SwiGLU, the fused QK-norm + rotary + cache write, dtype casts, and the
// sampling kernels (argmax, temperature). All arithmetic is float32; only
// loads and stores convert. One C entry point per operation.
#include "common.h"
#include "qk_prepare.h"
#include "argmax_static.h"

#include <math.h>
#include <stdio.h>

#include <mutex>

// ---------------------------------------------------------------- embedding
// out[t, :] = float(table[ids[t], :]). Reference: src/backend/cpu/cpu_backend.cpp:51-76.
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int D) {
  const int t = blockIdx.x;
  const TW* row = table + static_cast<size_t>(ids[t]) * D;
  float* o = out + static_cast<size_t>(t) * D;
  if (D % 8 == 0) {  // rows start 16-byte aligned: move 8 elements a thread
    for (int d = threadIdx.x * 8; d < D; d += blockDim.x * 8) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = load_as_float(row + d + i);
      *reinterpret_cast<float4*>(o + d) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(o + d + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
    return;
  }
  for (int d = threadIdx.x; d < D; d += blockDim.x) o[d] = load_as_float(row + d);
}

extern "C" int tie_embed(const void* table, int table_dtype, const int* ids, float* out, int T, int D,
                         hipStream_t stream) {
  if (T <= 0 || D <= 0) return TIE_BAD_ARGUMENT;
  const int threads = D >= 2048 ? 256 : 64;
  if (table_dtype == TIE_F32) {
    embed_kernel<float><<<T, threads, 0, stream>>>(static_cast<const float*>(table), ids, out, D);
  } else if (table_dtype == TIE_BF16) {
    embed_kernel<bf16_t><<<T, threads, 0, stream>>>(static_cast<const bf16_t*>(table), ids, out, D);
  } else {
    return TIE_BAD_ARGUMENT;
  }
  return tie_launch_status();
}

// ------------------------------------------------------------------ RMSNorm
// out[r, i] = (x[src(r), i] * inv) * w[i], inv = 1 / sqrt(mean(x^2) + eps), src(r) = rows ? rows[r] : r.
// Reference: src/backend/cpu/cpu_backend.cpp:141-159 (weight multiplies after normalisation).
template <typename TX, typename TO>
__global__ void rms_norm_kernel(const TX* __restrict__ x, const float* __restrict__ w, float eps,
                                TO* __restrict__ out, const int* __restrict__ rows, int n) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const TX* xr = x + static_cast<size_t>(rows ? rows[r] : r) * n;
  TO* o = out + static_cast<size_t>(r) * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = load_as_float(xr + i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    store_from_float(o + i, (load_as_float(xr + i) * inv) * w[i]);
  }
}

// Float32 rows of up to four float4 a thread (n % 4 == 0) stay in registers between the sum of
// squares and the scaling. With COUNT > 0 the row first receives COUNT planes of partial sums
// (x[r] += p_0[r] + p_1[r] + ..., written back): see the section on partial sums below. All loads
// of a thread are issued before the first use; the kernel is bound by latency, not by bytes.
template <typename TO, int COUNT, int V>
__global__ void rms_norm_row_kernel(float* __restrict__ x, const float* __restrict__ partials, size_t plane_stride,
                                    const float* __restrict__ w, float eps, TO* __restrict__ out,
                                    const int* __restrict__ rows, int n) {
  __shared__ float scratch[16];
  const size_t row = static_cast<size_t>(rows ? rows[blockIdx.x] : blockIdx.x) * n;
  TO* o = out + static_cast<size_t>(blockIdx.x) * n;
  float4 v[V], p[COUNT > 0 ? COUNT : 1][V], wv[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    const bool in = i < n;
    v[j] = in ? *reinterpret_cast<const float4*>(x + row + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    wv[j] = in ? *reinterpret_cast<const float4*>(w + i) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int s = 0; s < COUNT; ++s)
      p[s][j] = in ? *reinterpret_cast<const float4*>(partials + static_cast<size_t>(s) * plane_stride + row + i)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) {
#pragma unroll
    for (int s = 0; s < COUNT; ++s) {
      v[j].x += p[s][j].x;
      v[j].y += p[s][j].y;
      v[j].z += p[s][j].z;
      v[j].w += p[s][j].w;
    }
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    if (COUNT > 0 && i < n) *reinterpret_cast<float4*>(x + row + i) = v[j];
    ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    if (i >= n) continue;
    store_from_float(o + i, (v[j].x * inv) * wv[j].x);
    store_from_float(o + i + 1, (v[j].y * inv) * wv[j].y);
    store_from_float(o + i + 2, (v[j].z * inv) * wv[j].z);
    store_from_float(o + i + 3, (v[j].w * inv) * wv[j].w);
  }
}

template <typename TO, int COUNT>
static void launch_rms_norm_row(float* x, const float* partials, size_t stride, const float* w, float eps, TO* out,
                                const int* rows, int R, int n, hipStream_t stream) {
  // As many threads as the row has float4, up to 1024: measured faster than fewer threads with more loads each.
  const int quads = n / 4;
  if (quads <= 1024) {
    const int threads = (quads + TIE_WAVE - 1) / TIE_WAVE * TIE_WAVE;
    rms_norm_row_kernel<TO, COUNT, 1><<<R, threads, 0, stream>>>(x, partials, stride, w, eps, out, rows, n);
  } else if (quads <= 2048) {
    rms_norm_row_kernel<TO, COUNT, 2><<<R, 1024, 0, stream>>>(x, partials, stride, w, eps, out, rows, n);
  } else {
    rms_norm_row_kernel<TO, COUNT, 4><<<R, 1024, 0, stream>>>(x, partials, stride, w, eps, out, rows, n);
  }
}

extern "C" int tie_rms_norm(const void* x, int x_dtype, const float* w, float eps, void* out, int out_dtype,
                            const int* rows, int R, int n, hipStream_t stream) {
  if (R <= 0 || n <= 0) return TIE_BAD_ARGUMENT;
  if (x_dtype == TIE_F32 && n % 4 == 0 && n <= 16384 && n >= 256) {
    float* xf = static_cast<float*>(const_cast<void*>(x));   // without planes the kernel only reads it
    if (out_dtype == TIE_F32) launch_rms_norm_row<float, 0>(xf, nullptr, 0, w, eps, static_cast<float*>(out), rows, R, n, stream);
    else if (out_dtype == TIE_BF16) launch_rms_norm_row<bf16_t, 0>(xf, nullptr, 0, w, eps, static_cast<bf16_t*>(out), rows, R, n, stream);
    else return TIE_BAD_ARGUMENT;
    return tie_launch_status();
  }
  const int threads = n >= 2048 ? 512 : (n >= 512 ? 256 : 64);
#define LAUNCH(TX, TO)                                                                                   \
  rms_norm_kernel<TX, TO><<<R, threads, 0, stream>>>(static_cast<const TX*>(x), w, eps, static_cast<TO*>(out), \
                                                     rows, n)
  if (x_dtype == TIE_F32 && out_dtype == TIE_F32) LAUNCH(float, float);
  else if (x_dtype == TIE_F32 && out_dtype == TIE_BF16) LAUNCH(float, bf16_t);
  else if (x_dtype == TIE_BF16 && out_dtype == TIE_F32) LAUNCH(bf16_t, float);
  else if (x_dtype == TIE_BF16 && out_dtype == TIE_BF16) LAUNCH(bf16_t, bf16_t);
  else return TIE_BAD_ARGUMENT;
#undef LAUNCH
  return tie_launch_status();
}

// ------------------------------------------------------------------- SwiGLU
// gate_up is [T, 2I] with the gate in columns [0, I) and up in [I, 2I).
// out[t, i] = gate / (1 + exp(-gate)) * up, left to right. Reference: cpu_backend.cpp:195-207.
template <typename TX, typename TO>
__global__ void swiglu_kernel(const TX* __restrict__ gate_up, TO* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const TX* row = gate_up + static_cast<size_t>(t) * 2 * I;
  const float g = load_as_float(row + i);
  const float u = load_as_float(row + I + i);
  store_from_float(out + static_cast<size_t>(t) * I + i, g / (1.0f + expf(-g)) * u);
}

extern "C" int tie_swiglu(const void* gate_up, int in_dtype, void* out, int out_dtype, int T, int I,
                          hipStream_t stream) {
  if (T <= 0 || I <= 0 || T > 65535 * 64) return TIE_BAD_ARGUMENT;
  const dim3 grid((I + 255) / 256, T);
#define LAUNCH(TX, TO) \
  swiglu_kernel<TX, TO><<<grid, 256, 0, stream>>>(static_cast<const TX*>(gate_up), static_cast<TO*>(out), I)
  if (in_dtype == TIE_F32 && out_dtype == TIE_F32) LAUNCH(float, float);
  else if (in_dtype == TIE_F32 && out_dtype == TIE_BF16) LAUNCH(float, bf16_t);
  else if (in_dtype == TIE_BF16 && out_dtype == TIE_BF16) LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == TIE_BF16 && out_dtype == TIE_F32) LAUNCH(bf16_t, float);
  else return TIE_BAD_ARGUMENT;
#undef LAUNCH
  return tie_launch_status();
}

// ------------------------------------------------------------ rows that lack their norm's factor
// rows[m][:] *= 1 / sqrt((squares[m][0] + ... + squares[m][tiles - 1]) / n + eps): the sums of squares come per
// 16-column tile from the product that prepared the rows; lane l adds the tiles l, l + 64, ... in ascending
// order and the lanes meet in a fixed butterfly, as in the products that apply the factor themselves.
template <typename T>
__global__ void scale_rows_kernel(T* __restrict__ rows, int width, const float* __restrict__ squares, int tiles,
                                  float n, float eps) {
  __shared__ float factor;
  const int m = blockIdx.x;
  if (threadIdx.x < TIE_WAVE) {
    float sq = 0.f;
    for (int t = threadIdx.x; t < tiles; t += TIE_WAVE) sq += squares[static_cast<size_t>(m) * tiles + t];
    sq = wave_sum(sq);
    if (threadIdx.x == 0) factor = 1.0f / sqrtf(sq / n + eps);
  }
  __syncthreads();
  T* row = rows + static_cast<size_t>(m) * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) store_from_float(row + i, load_as_float(row + i) * factor);
}

extern "C" int tie_scale_rows(void* rows, int dtype, int M, int width, const float* squares, int tiles, float n,
                              float eps, hipStream_t stream) {
  if (M <= 0 || width <= 0 || tiles <= 0 || !(n > 0.f) || squares == nullptr) return TIE_BAD_ARGUMENT;
  if (dtype == TIE_F32) scale_rows_kernel<float><<<M, 256, 0, stream>>>(static_cast<float*>(rows), width, squares, tiles, n, eps);
  else if (dtype == TIE_BF16) scale_rows_kernel<bf16_t><<<M, 256, 0, stream>>>(static_cast<bf16_t*>(rows), width, squares, tiles, n, eps);
  else return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}

// ------------------------------------------------------------ a projection's bias
// rows[m][n] += bias[n], in float32, stored in the rows' own type: a projection with a bias is its product and
// this (the products' epilogues have no bias term; the reference's projections have none either).
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ rows, const float* __restrict__ bias, size_t count, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  store_from_float(rows + i, load_as_float(rows + i) + bias[i % width]);
}

extern "C" int tie_add_bias(void* rows, int dtype, int M, int width, const float* bias, hipStream_t stream) {
  if (M <= 0 || width <= 0 || rows == nullptr || bias == nullptr) return TIE_BAD_ARGUMENT;
  const size_t count = static_cast<size_t>(M) * width;
  const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
  if (dtype == TIE_F32) add_bias_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<float*>(rows), bias, count, width);
  else if (dtype == TIE_BF16) add_bias_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(rows), bias, count, width);
  else return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}

// ------------------------------------------------------------ tokens the host has not seen
// tokens[i] = previous[sources[i]] where sources[i] >= 0: rows whose token an earlier step's sampling kernel left
// on the device (the host queues this step before it has read that one); the other rows keep the host's token.
__global__ void take_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ sources,
                                   const int* __restrict__ previous, int T, int num_previous) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T) return;
  const int from = sources[i];
  if (from >= 0 && from < num_previous) tokens[i] = previous[from];
}

extern "C" int tie_take_tokens(int* tokens, const int* sources, const int* previous, int T, int num_previous,
                               hipStream_t stream) {
  if (T <= 0 || num_previous <= 0 || tokens == nullptr || sources == nullptr || previous == nullptr)
    return TIE_BAD_ARGUMENT;
  take_tokens_kernel<<<(T + 255) / 256, 256, 0, stream>>>(tokens, sources, previous, T, num_previous);
  return tie_launch_status();
}

// ------------------------------------------------------------ random weights
// Element i of a tensor is a function of (key, i) alone: the 64-bit mix of key + (i + 1) * 0x9E3779B97F4A7C15
// (the SplitMix64 step) gives 52 bits of a uniform number u in (0, 1), and a normal value is the inverse normal
// distribution function of u by Wichura's algorithm AS 241 (PPND16: rational functions, a logarithm and a root
// in the tails). Every operation below is an IEEE double addition, multiplication, division or square root with
// nothing contracted into a fused multiply-add, and the logarithm is a fixed series of such operations, so the
// host (weights/random_init.py, the same steps in numpy) and the GPU draw the same bits.
__device__ __forceinline__ unsigned long long random_mix(unsigned long long key, unsigned long long i) {
  unsigned long long z = key + (i + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ double random_log(double x) {           // x in (0, 1); log(m * 2^e) = 2 atanh((m - 1) / (m + 1)) + e ln 2
#pragma clang fp contract(off)
  int e;
  double m = frexp(x, &e);                         // m in [0.5, 1), exact
  if (m < 0.70710678118654752440) {
    m = m * 2.0;
    e -= 1;
  }
  const double s = (m - 1.0) / (m + 1.0), s2 = s * s;
  double series = 1.0 / 27.0;
  series = series * s2 + 1.0 / 25.0;
  series = series * s2 + 1.0 / 23.0;
  series = series * s2 + 1.0 / 21.0;
  series = series * s2 + 1.0 / 19.0;
  series = series * s2 + 1.0 / 17.0;
  series = series * s2 + 1.0 / 15.0;
  series = series * s2 + 1.0 / 13.0;
  series = series * s2 + 1.0 / 11.0;
  series = series * s2 + 1.0 / 9.0;
  series = series * s2 + 1.0 / 7.0;
  series = series * s2 + 1.0 / 5.0;
  series = series * s2 + 1.0 / 3.0;
  series = series * s2 + 1.0;
  return 2.0 * s * series + static_cast<double>(e) * 0.69314718055994530942;
}

#define RANDOM_POLY(c0, c1, c2, c3, c4, c5, c6, c7, r) \
  ((((((((c7) * (r) + (c6)) * (r) + (c5)) * (r) + (c4)) * (r) + (c3)) * (r) + (c2)) * (r) + (c1)) * (r) + (c0))

__device__ double random_normal_of(double p) {     // AS 241, PPND16
#pragma clang fp contract(off)
  const double q = p - 0.5;
  if (fabs(q) <= 0.425) {
    const double r = 0.180625 - q * q;
    const double num = RANDOM_POLY(3.3871328727963666080, 1.3314166789178437745e2, 1.9715909503065514427e3,
                                   1.3731693765509461125e4, 4.5921953931549871457e4, 6.7265770927008700853e4,
                                   3.3430575583588128105e4, 2.5090809287301226727e3, r);
    const double den = RANDOM_POLY(1.0, 4.2313330701600911252e1, 6.8718700749205790830e2, 5.3941960214247511077e3,
                                   2.1213794301586595867e4, 3.9307895800092710610e4, 2.8729085735721942674e4,
                                   5.2264952788528545610e3, r);
    return q * num / den;
  }
  double r = q < 0.0 ? p : 1.0 - p;
  r = __dsqrt_rn(-random_log(r));
  double v;
  if (r <= 5.0) {
    r = r - 1.6;
    const double num = RANDOM_POLY(1.42343711074968357734, 4.63033784615654529590, 5.76949722146069140550,
                                   3.64784832476320460504, 1.27045825245236838258, 2.41780725177450611770e-1,
                                   2.27238449892691845833e-2, 7.74545014278341407640e-4, r);
    const double den = RANDOM_POLY(1.0, 2.05319162663775882187, 1.67638483018380384940, 6.89767334985100004550e-1,
                                   1.48103976427480074590e-1, 1.51986665636164571966e-2, 5.47593808499534494600e-4,
                                   1.05075007164441684324e-9, r);
    v = num / den;
  } else {
    r = r - 5.0;
    const double num = RANDOM_POLY(6.65790464350110377720, 5.46378491116411436990, 1.78482653991729133580,
                                   2.96560571828504891230e-1, 2.65321895265761230930e-2, 1.24266094738807843860e-3,
                                   2.71155556874348757815e-5, 2.01033439929228813265e-7, r);
    const double den = RANDOM_POLY(1.0, 5.99832206555887937690e-1, 1.36929880922735805310e-1, 1.48753612908506148525e-2,
                                   7.86869131145613259100e-4, 1.84631831751005468180e-5, 1.42151175831644588870e-7,
                                   2.04426310338993978564e-15, r);
    v = num / den;
  }
  return q < 0.0 ? -v : v;
}

// kind 0: scale * normal; kind 1: 1 + scale * (2 u - 1). Rounded once to float32.
__global__ void random_fill_kernel(float* __restrict__ out, size_t n, unsigned long long key, int kind, double scale) {
#pragma clang fp contract(off)
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const double u = (static_cast<double>(random_mix(key, i) >> 12) + 0.5) * 2.2204460492503130808e-16;   // 2^-52
  const double v = kind == 0 ? scale * random_normal_of(u) : 1.0 + scale * (2.0 * u - 1.0);
  out[i] = static_cast<float>(v);
}

extern "C" int tie_random_fill(float* out, long long n, unsigned long long key, int kind, double scale,
                               hipStream_t stream) {
  if (n <= 0 || (kind != 0 && kind != 1) || (n + 255) / 256 > 0x7fffffffLL) return TIE_BAD_ARGUMENT;
  random_fill_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(out, static_cast<size_t>(n), key, kind,
                                                                                   scale);
  return tie_launch_status();
}

// --------------------------------------------------------------------- cast
template <typename TX, typename TO>
__global__ void cast_kernel(const TX* __restrict__ x, TO* __restrict__ out, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) store_from_float(out + i, load_as_float(x + i));
}

extern "C" int tie_cast(const void* x, int in_dtype, void* out, int out_dtype, long long n, hipStream_t stream) {
  if (n <= 0) return TIE_BAD_ARGUMENT;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  if (in_dtype == TIE_F32 && out_dtype == TIE_BF16)
    cast_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const float*>(x), static_cast<bf16_t*>(out), n);
  else if (in_dtype == TIE_BF16 && out_dtype == TIE_F32)
    cast_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<float*>(out), n);
  else
    return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}

// ------------------------------------------------- partial sums (+ RMSNorm)
// A matrix product cut along K leaves `count` planes of partial sums, plane_stride floats apart.
// x[r, i] += p_0[r, i] + p_1[r, i] + ... in plane order (float32, the residual stream), and, with a
// norm weight, out[r, :] = RMSNorm(x[r, :]) * w of the updated row in the same pass: the row is
// read once, and the product's result never makes a round trip of its own through memory.
__device__ __forceinline__ float add_planes(float v, const float* __restrict__ p, size_t plane_stride, int count) {
  for (int s = 0; s < count; ++s) v += p[static_cast<size_t>(s) * plane_stride];
  return v;
}

template <typename TO>
__global__ void add_partials_rms_norm_kernel(float* __restrict__ x, const float* __restrict__ partials,
                                             size_t plane_stride, int count, const float* __restrict__ w, float eps,
                                             TO* __restrict__ out, int n) {
  __shared__ float scratch[16];
  const size_t row = static_cast<size_t>(blockIdx.x) * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = add_planes(x[row + i], partials + row + i, plane_stride, count);
    x[row + i] = v;     // read back below by the thread that wrote it
    ss += v * v;
  }
  if (w == nullptr) return;
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) store_from_float(out + row + i, (x[row + i] * inv) * w[i]);
}

// w (and out) null: only the addition.
extern "C" int tie_add_partials_rms_norm(float* x, const float* partials, long plane_stride, int count, const float* w,
                                         float eps, void* out, int out_dtype, int R, int n, hipStream_t stream) {
  if (R <= 0 || n <= 0 || count <= 0 || plane_stride < static_cast<long>(R) * n || (w != nullptr && out == nullptr))
    return TIE_BAD_ARGUMENT;
  if (w != nullptr && out_dtype != TIE_F32 && out_dtype != TIE_BF16) return TIE_BAD_ARGUMENT;
  const size_t stride = static_cast<size_t>(plane_stride);
  if (w != nullptr && n % 4 == 0 && plane_stride % 4 == 0 && n <= 16384 && n >= 256 && (count <= 4 || count == 8)) {
#define ROW(TO, COUNT) launch_rms_norm_row<TO, COUNT>(x, partials, stride, w, eps, static_cast<TO*>(out), nullptr, R, n, stream)
    if (out_dtype == TIE_F32) {
      if (count == 1) ROW(float, 1); else if (count == 2) ROW(float, 2); else if (count == 3) ROW(float, 3);
      else if (count == 4) ROW(float, 4); else ROW(float, 8);
    } else {
      if (count == 1) ROW(bf16_t, 1); else if (count == 2) ROW(bf16_t, 2); else if (count == 3) ROW(bf16_t, 3);
      else if (count == 4) ROW(bf16_t, 4); else ROW(bf16_t, 8);
    }
#undef ROW
    return tie_launch_status();
  }
  const int threads = n >= 2048 ? 512 : (n >= 512 ? 256 : 64);
  if (w == nullptr || out_dtype == TIE_F32)
    add_partials_rms_norm_kernel<float><<<R, threads, 0, stream>>>(x, partials, stride, count, w, eps,
                                                                   static_cast<float*>(out), n);
  else
    add_partials_rms_norm_kernel<bf16_t><<<R, threads, 0, stream>>>(x, partials, stride, count, w, eps,
                                                                    static_cast<bf16_t*>(out), n);
  return tie_launch_status();
}

// ------------------------------------------ QK-norm + rotary + cache write
// One wave per (token, head slot). Head slots 0..H-1 are query heads, then KVH
// key heads, then KVH value heads of the fused projection row
// qkv[t] = [q (H*Dh) | k (KVH*Dh) | v (KVH*Dh)], in_row elements apart from the next token's.
//   q, k: per-head RMSNorm over Dh with one weight vector shared by all heads,
//         THEN rotate-half rotary: pairs (i, i + Dh/2), angle = float(pos) * inv_freq[i]
//         (reference: src/model/qwen3.cpp:222-225, cpu_backend.cpp:161-193, backend/rope.h:9-13).
//         More generally the first rotary_dim <= Dh dimensions of a head are rotated, as pairs
//         (i, i + rotary_dim/2) or, interleaved, (2i, 2i + 1); the rest only passes the norm.
//   q goes to q_out[t * q_row + h*Dh + d]; k (after norm and rotation) and raw v go to the paged
//   cache with page = slot / block_size, offset = slot % block_size (cpu_backend.cpp:235-259):
//   keys at ((page*KVH + h)*block_size + offset)*Dh + d, one row per position; values transposed
//   inside the page, at ((page*KVH + h)*Dh + d)*block_size + offset, one row per dimension, which
//   is the order in which the attention kernels' matrix cores consume them.
// Norm weights or inv_freq may be null: that step is then skipped. With k_dense set, keys are
// written there (row stride k_row) instead of into the cache; without write_kv and k_dense only
// the query heads are processed. q_out and k_dense may alias qkv (each wave holds its head in
// registers before it writes). The input may come as `planes` partial sums, plane_stride elements
// apart (a product cut along K): they are added in plane order as they are read.
#define TIE_MAX_PAIRS 4  // head_dim <= 512

template <typename TX, typename TQ, typename TC>
__global__ void qk_norm_rope_kv_write_kernel(const TX* qkv, TQ* q_out, const float* __restrict__ q_w,
                                             const float* __restrict__ k_w, float eps,
                                             const float* __restrict__ inv_freq,
                                             const float* __restrict__ angles,
                                             const int* __restrict__ positions, const int* __restrict__ slots,
                                             TC* __restrict__ k_cache, TC* __restrict__ v_cache, TQ* k_dense, int H,
                                             int KVH, int Dh, int block_size, int in_row, int q_row, int k_row,
                                             size_t plane_stride, int planes, int rotary_dim, int interleaved) {
  const int t = blockIdx.y;
  const int slot_index = blockIdx.x;
  const int lane = threadIdx.x;
  const int half = Dh / 2;
  // Pair p < Dh/2 of a head is the elements (e1(p), e2(p)): the rotated pairs first, then the
  // dimensions beyond rotary_dim in two runs (they are not rotated, so how they pair does not matter).
  const int rhalf = rotary_dim / 2;
  auto e1 = [&](int p) { return p < rhalf ? (interleaved ? 2 * p : p) : rotary_dim + (p - rhalf); };
  auto e2 = [&](int p) {
    return p < rhalf ? (interleaved ? 2 * p + 1 : p + rhalf) : rotary_dim + (half - rhalf) + (p - rhalf);
  };
  const TX* in = qkv + static_cast<size_t>(t) * in_row + static_cast<size_t>(slot_index) * Dh;

  const bool is_q = slot_index < H;
  const bool is_k = !is_q && slot_index < H + KVH;

  if (!is_q && !is_k) {  // value head: straight copy into the cache
    const int h = slot_index - H - KVH;
    const int slot = slots[t];
    TC* dst = v_cache + (static_cast<size_t>(slot / block_size) * KVH + h) * Dh * block_size + slot % block_size;
    for (int d = lane; d < Dh; d += TIE_WAVE) store_from_float(dst + static_cast<size_t>(d) * block_size, load_planes(in + d, plane_stride, planes));
    return;
  }

  float x1[TIE_MAX_PAIRS], x2[TIE_MAX_PAIRS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < TIE_MAX_PAIRS; ++i) {
    const int p = lane + i * TIE_WAVE;
    x1[i] = 0.f;
    x2[i] = 0.f;
    if (p < half) {
      x1[i] = load_planes(in + e1(p), plane_stride, planes);
      x2[i] = load_planes(in + e2(p), plane_stride, planes);
      ss += x1[i] * x1[i] + x2[i] * x2[i];
    }
  }
  const float* w = is_q ? q_w : k_w;
  float inv = 1.0f;
  if (w != nullptr) {
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / static_cast<float>(Dh) + eps);
  }
  const float pos = static_cast<float>(positions[t]);

  TQ* dense_dst = nullptr;
  TC* cache_dst = nullptr;
  if (is_q) {
    dense_dst = q_out + static_cast<size_t>(t) * q_row + static_cast<size_t>(slot_index) * Dh;
  } else if (k_dense != nullptr) {
    dense_dst = k_dense + static_cast<size_t>(t) * k_row + static_cast<size_t>(slot_index - H) * Dh;
  } else {
    const int h = slot_index - H;
    const int slot = slots[t];
    cache_dst = k_cache + ((static_cast<size_t>(slot / block_size) * KVH + h) * block_size + slot % block_size) * Dh;
  }
#pragma unroll
  for (int i = 0; i < TIE_MAX_PAIRS; ++i) {
    const int p = lane + i * TIE_WAVE;
    if (p >= half) continue;
    const int d1 = e1(p), d2 = e2(p);
    float a = x1[i], b = x2[i];
    if (w != nullptr) {
      a = (a * inv) * w[d1];
      b = (b * inv) * w[d2];
    }
    float o1 = a, o2 = b;
    if (p >= rhalf) {
      // beyond the rotated dimensions
    } else if (angles != nullptr) {   // cos and sin of this token's angles, computed once for all heads and layers
      const float cs = angles[static_cast<size_t>(t) * rotary_dim + p];
      const float sn = angles[static_cast<size_t>(t) * rotary_dim + rhalf + p];
      o1 = a * cs - b * sn;
      o2 = b * cs + a * sn;
    } else if (inv_freq != nullptr) {
      const float angle = pos * inv_freq[p];
      float sn, cs;
      sincosf(angle, &sn, &cs);
      o1 = a * cs - b * sn;
      o2 = b * cs + a * sn;
    }
    if (dense_dst != nullptr) {
      store_from_float(dense_dst + d1, o1);
      store_from_float(dense_dst + d2, o2);
    } else {
      store_from_float(cache_dst + d1, o1);
      store_from_float(cache_dst + d2, o2);
    }
  }
}

// The values of a portion of tokens into the cache, eight tokens at a time. A page holds a value head transposed
// (one row of block_size positions per dimension), so the kernel above, a token a workgroup, writes 2 bytes here
// and 2 bytes there: 2048 tokens of an 8B layer took 13 us for 8 MB. Here (extra workgroups of the same launch) a thread takes one dimension of eight
// consecutive rows of the step; where their slots are eight consecutive positions of one page, starting at a
// multiple of eight (a portion of a prompt nearly everywhere), it stores them as one 16-byte piece, else one by
// one. The same conversions, the same bits. Caches of 2-byte elements, pages of a multiple of 8 positions.
#define VROWS_THREADS 256
#define VROWS_TOKENS 8

template <typename TX, typename TC>
__device__ __forceinline__ void v_write_rows(const TX* __restrict__ qkv, const int* __restrict__ slots,
                                             TC* __restrict__ v_cache, int T, int KVH, int Dh, int block_size,
                                             int in_row, int v_offset, size_t plane_stride, int planes, int head,
                                             int block_of_groups) {
  static_assert(sizeof(TC) == 2, "eight elements are one 16-byte piece");
  const int groups_a_workgroup = Dh >= VROWS_THREADS ? 1 : VROWS_THREADS / Dh;
  const int group = block_of_groups * groups_a_workgroup + (Dh >= VROWS_THREADS ? 0 : threadIdx.x / Dh);
  const int t0 = group * VROWS_TOKENS;
  if (t0 >= T) return;
  const int n = min(VROWS_TOKENS, T - t0);
  int slot[VROWS_TOKENS];
#pragma unroll
  for (int i = 0; i < VROWS_TOKENS; ++i) slot[i] = slots[min(t0 + i, T - 1)];
  bool together = n == VROWS_TOKENS && slot[0] % VROWS_TOKENS == 0;
#pragma unroll
  for (int i = 1; i < VROWS_TOKENS; ++i) together = together && slot[i] == slot[0] + i;
  for (int d = Dh >= VROWS_THREADS ? threadIdx.x : threadIdx.x % Dh; d < Dh; d += VROWS_THREADS) {
    const TX* in = qkv + static_cast<size_t>(t0) * in_row + v_offset + static_cast<size_t>(head) * Dh + d;
    float v[VROWS_TOKENS];
#pragma unroll
    for (int i = 0; i < VROWS_TOKENS; ++i)
      v[i] = i < n ? load_planes(in + static_cast<size_t>(i) * in_row, plane_stride, planes) : 0.f;
    if (together) {
      TC* dst = v_cache + (static_cast<size_t>(slot[0] / block_size) * KVH + head) * Dh * block_size +
                static_cast<size_t>(d) * block_size + slot[0] % block_size;
      TC piece[VROWS_TOKENS];
#pragma unroll
      for (int i = 0; i < VROWS_TOKENS; ++i) store_from_float(piece + i, v[i]);
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(piece);
    } else {
      for (int i = 0; i < n; ++i) {
        TC* dst = v_cache + (static_cast<size_t>(slot[i] / block_size) * KVH + head) * Dh * block_size +
                  static_cast<size_t>(d) * block_size + slot[i] % block_size;
        store_from_float(dst, v[i]);
      }
    }
  }
}

// The same for head sizes of 32, 64, 128, 256 or 512: a lane takes 4 consecutive elements of a head's
// first half and the 4 they pair with in the second (16-byte loads and stores where the one-wave-a-head
// kernel above moves 4 and 2 bytes), head_dim / 8 lanes share a head, four waves of heads a workgroup.
// The sums of squares meet by shuffles inside the lanes of a head. Whole heads rotated as halves only.
#define QK4_THREADS 256

template <typename TX, typename TQ, typename TC, int LPH>   // LPH: lanes per head = head_dim / 8
__global__ __launch_bounds__(QK4_THREADS) void qk_norm_rope_kv_write4_kernel(
    const TX* qkv, TQ* q_out, const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    const float* __restrict__ inv_freq, const float* __restrict__ angles, const int* __restrict__ positions,
    const int* __restrict__ slots, TC* __restrict__ k_cache, TC* __restrict__ v_cache, TQ* k_dense, int H, int KVH,
    int block_size, int in_row, int q_row, int k_row, size_t plane_stride, int planes, int heads, int tokens,
    int blocks_a_token) {
  constexpr int Dh = LPH * 8, half = LPH * 4;
  // Workgroups 0 .. T x blocks_a_token - 1 take the heads of a token; those behind them, where there are any, the
  // values of groups of tokens (v_write_rows), KVH of them a block of groups.
  const int qk_blocks = tokens * blocks_a_token;
  if (static_cast<int>(blockIdx.x) >= qk_blocks) {
    if constexpr (sizeof(TC) == 2) {
      const int b = blockIdx.x - qk_blocks;
      v_write_rows<TX, TC>(qkv, slots, v_cache, tokens, KVH, Dh, block_size, in_row, (H + KVH) * Dh, plane_stride, planes,
                           b % KVH, b / KVH);
    }
    return;
  }
  const int t = blockIdx.x / blocks_a_token;
  const int slot_index = (blockIdx.x % blocks_a_token) * (QK4_THREADS / LPH) + threadIdx.x / LPH;
  const int p0 = (threadIdx.x % LPH) * 4;
  if (slot_index >= heads) return;             // whole heads leave: the shuffles below stay inside a head
  const TX* in = qkv + static_cast<size_t>(t) * in_row + static_cast<size_t>(slot_index) * Dh;
  const bool is_q = slot_index < H;
  const bool is_k = !is_q && slot_index < H + KVH;
  if (!is_q && !is_k) {
    // Value head: into the cache, transposed inside the page. Neighbouring lanes take neighbouring
    // dimensions, which lie block_size elements apart there: the closest the stores of one token get.
    const int slot = slots[t];
    TC* dst = v_cache + (static_cast<size_t>(slot / block_size) * KVH + (slot_index - H - KVH)) * Dh * block_size +
              slot % block_size;
    const int sub = threadIdx.x % LPH;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = load_planes(in + sub + LPH * i, plane_stride, planes);
#pragma unroll
    for (int i = 0; i < 8; ++i) store_from_float(dst + static_cast<size_t>(sub + LPH * i) * block_size, v[i]);
    return;
  }
  qk_f4_t a = load4_planes(in + p0, plane_stride, planes);
  qk_f4_t b = load4_planes(in + half + p0, plane_stride, planes);

  const float* w = is_q ? q_w : k_w;
  if (w != nullptr) qk_head_norm<LPH>(a, b, w, eps, p0);
  qk_f4_t o1 = a, o2 = b;
  if (angles != nullptr) {
    qk_rotate_by_table<LPH>(a, b, angles + static_cast<size_t>(t) * Dh, p0, o1, o2);
  } else if (inv_freq != nullptr) {
    const float pos = static_cast<float>(positions[t]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float sn, cs;
      sincosf(pos * inv_freq[p0 + i], &sn, &cs);
      o1[i] = a[i] * cs - b[i] * sn;
      o2[i] = b[i] * cs + a[i] * sn;
    }
  }
  if (is_q) {
    TQ* dst = q_out + static_cast<size_t>(t) * q_row + static_cast<size_t>(slot_index) * Dh;
    store4(dst + p0, o1);
    store4(dst + half + p0, o2);
  } else if (k_dense != nullptr) {
    TQ* dst = k_dense + static_cast<size_t>(t) * k_row + static_cast<size_t>(slot_index - H) * Dh;
    store4(dst + p0, o1);
    store4(dst + half + p0, o2);
  } else {
    const int slot = slots[t];
    TC* dst = k_cache + ((static_cast<size_t>(slot / block_size) * KVH + (slot_index - H)) * block_size +
                         slot % block_size) * Dh;
    store4(dst + p0, o1);
    store4(dst + half + p0, o2);
  }
}

// angles[t, 0:Dh/2] = cos(float(positions[t]) * inv_freq[i]), angles[t, Dh/2:Dh] = sin of the same: what
// the kernel below would compute per head and layer, once per step instead.
__global__ void rope_angles_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                   float* __restrict__ angles, int T, int half) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * half) return;
  const int t = i / half, p = i % half;
  float sn, cs;
  sincosf(static_cast<float>(positions[t]) * inv_freq[p], &sn, &cs);
  angles[static_cast<size_t>(t) * 2 * half + p] = cs;
  angles[static_cast<size_t>(t) * 2 * half + half + p] = sn;
}

extern "C" int tie_rope_angles(const int* positions, const float* inv_freq, float* angles, int T, int half,
                               hipStream_t stream) {
  if (T <= 0 || half <= 0) return TIE_BAD_ARGUMENT;
  const long n = static_cast<long>(T) * half;
  rope_angles_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(positions, inv_freq, angles, T, half);
  return tie_launch_status();
}

// angles (optional): the table of tie_rope_angles for these positions ([T, rotary_dim]); then inv_freq is not read.
// rotary_dim: how many leading dimensions of a head are rotated (inv_freq holds rotary_dim / 2 values);
// interleaved: pairs (2i, 2i + 1) instead of (i, i + rotary_dim / 2).
extern "C" int tie_qk_norm_rope_kv_write(const void* qkv, int in_dtype, void* q_out, int q_dtype,
                                         const float* q_w, const float* k_w, float eps, const float* inv_freq,
                                         const float* angles, const int* positions, const int* slots, void* k_cache, void* v_cache,
                                         int cache_dtype, int write_kv, void* k_dense, int T, int H, int KVH,
                                         int Dh, int block_size, int in_row, int q_row, int k_row,
                                         long plane_stride, int planes, int rotary_dim, int interleaved,
                                         hipStream_t stream) {
  if (rotary_dim < 0 || rotary_dim > Dh || rotary_dim % 2 != 0) return TIE_BAD_ARGUMENT;
  if (inv_freq == nullptr && angles == nullptr) {   // no rotation at all
    rotary_dim = 0;
    interleaved = 0;
  }
  if (planes < 1 || (planes > 1 && plane_stride < static_cast<long>(T) * in_row)) return TIE_BAD_ARGUMENT;
  if (T <= 0 || H <= 0 || KVH <= 0 || Dh <= 0 || Dh % 2 != 0 || Dh > 2 * TIE_MAX_PAIRS * TIE_WAVE ||
      block_size <= 0 || T > 65535 || q_row < H * Dh)
    return TIE_BAD_ARGUMENT;
  if (write_kv && (slots == nullptr || k_cache == nullptr || v_cache == nullptr || k_dense != nullptr))
    return TIE_BAD_ARGUMENT;
  const int heads = H + ((write_kv || k_dense != nullptr) ? KVH : 0) + (write_kv ? KVH : 0);
  if (in_row < heads * Dh || (k_dense != nullptr && k_row < KVH * Dh)) return TIE_BAD_ARGUMENT;
  // Head sizes of 32 .. 512 in powers of two, and rows that keep 16-byte pieces aligned: the 4-wide kernel.
  const bool wide = (rotary_dim == 0 || (rotary_dim == Dh && !interleaved)) && (Dh == 32 || Dh == 64 || Dh == 128 || Dh == 256 || Dh == 512) && in_row % 4 == 0 &&
                    q_row % 4 == 0 && k_row % 4 == 0 && plane_stride % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(k_dense) % 16 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(angles) % 16 == 0 && reinterpret_cast<uintptr_t>(q_w) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(k_w) % 16 == 0;
  if (wide) {
    const int lph = Dh / 8;
    // From 32 rows on the values go by workgroups of their own that store eight tokens of a dimension at once.
    const bool values_apart = write_kv && T >= 32 && block_size % VROWS_TOKENS == 0 && cache_dtype != TIE_F32 &&
                              reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
    const int heads_here = values_apart ? heads - KVH : heads;
    const int blocks_a_token = (heads_here + QK4_THREADS / lph - 1) / (QK4_THREADS / lph);
    long blocks = static_cast<long>(T) * blocks_a_token;
    if (values_apart) {
      const int groups = (T + VROWS_TOKENS - 1) / VROWS_TOKENS;
      const int groups_a_workgroup = Dh >= VROWS_THREADS ? 1 : VROWS_THREADS / Dh;
      blocks += static_cast<long>(KVH) * ((groups + groups_a_workgroup - 1) / groups_a_workgroup);
    }
    if (blocks > 0x7fffffffL) return TIE_BAD_ARGUMENT;
    const dim3 grid4(static_cast<unsigned>(blocks));
#define LAUNCH4_L(TX, TQ, TC, LPH)                                                                            \
  qk_norm_rope_kv_write4_kernel<TX, TQ, TC, LPH><<<grid4, QK4_THREADS, 0, stream>>>(                          \
      static_cast<const TX*>(qkv), static_cast<TQ*>(q_out), q_w, k_w, eps, inv_freq, angles, positions, slots, \
      static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), static_cast<TQ*>(k_dense), H, KVH, block_size,   \
      in_row, q_row, k_row, static_cast<size_t>(plane_stride), planes, heads_here, T, blocks_a_token)
#define LAUNCH4(TX, TQ, TC)                         \
  {                                                 \
    if (lph == 4) LAUNCH4_L(TX, TQ, TC, 4);         \
    else if (lph == 8) LAUNCH4_L(TX, TQ, TC, 8);    \
    else if (lph == 16) LAUNCH4_L(TX, TQ, TC, 16);  \
    else if (lph == 32) LAUNCH4_L(TX, TQ, TC, 32);  \
    else LAUNCH4_L(TX, TQ, TC, 64);                 \
  }
    if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_F32) LAUNCH4(float, float, float)
    else if (in_dtype == TIE_F32 && q_dtype == TIE_BF16 && cache_dtype == TIE_BF16) LAUNCH4(float, bf16_t, bf16_t)
    else if (in_dtype == TIE_BF16 && q_dtype == TIE_BF16 && cache_dtype == TIE_BF16) LAUNCH4(bf16_t, bf16_t, bf16_t)
    else if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_BF16) LAUNCH4(float, float, bf16_t)
    else if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_F16) LAUNCH4(float, float, f16_t)
    else return TIE_BAD_ARGUMENT;
#undef LAUNCH4
#undef LAUNCH4_L
    return tie_launch_status();
  }
  const dim3 grid(heads, T);
#define LAUNCH(TX, TQ, TC)                                                                                   \
  qk_norm_rope_kv_write_kernel<TX, TQ, TC><<<grid, TIE_WAVE, 0, stream>>>(                                    \
      static_cast<const TX*>(qkv), static_cast<TQ*>(q_out), q_w, k_w, eps, inv_freq, angles, positions, slots, \
      static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), static_cast<TQ*>(k_dense), H, KVH, Dh,           \
      block_size, in_row, q_row, k_row, static_cast<size_t>(plane_stride), planes, rotary_dim, interleaved)
  if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_F32) LAUNCH(float, float, float);
  else if (in_dtype == TIE_F32 && q_dtype == TIE_BF16 && cache_dtype == TIE_BF16) LAUNCH(float, bf16_t, bf16_t);
  else if (in_dtype == TIE_BF16 && q_dtype == TIE_BF16 && cache_dtype == TIE_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_BF16) LAUNCH(float, float, bf16_t);
  else if (in_dtype == TIE_F32 && q_dtype == TIE_F32 && cache_dtype == TIE_F16) LAUNCH(float, float, f16_t);
  else return TIE_BAD_ARGUMENT;
#undef LAUNCH
  return tie_launch_status();
}

// ------------------------------------------------------------------ argmax
// out[r] = index of the first maximum of logits[r, :] (ties go to the lowest id,
// as std::max_element in src/sampling/sampler.cpp:24); -1 if the row holds a NaN.
// Two stages so that a few long rows still fill the GPU: ARGMAX_CHUNKS workgroups scan a slice of
// a row each, then one wave per row picks among their candidates.
#define ARGMAX_CHUNKS 64

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__global__ void argmax_partial_kernel(const float* __restrict__ logits, float* __restrict__ part_v,
                                      int* __restrict__ part_i, int V) {
  __shared__ float best_v[4];
  __shared__ int best_i[4];
  const int r = blockIdx.y, chunk = blockIdx.x;
  const float* row = logits + static_cast<size_t>(r) * V;
  const int per = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
  const int begin = chunk * per, end = min(V, begin + per);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool nan = false;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float v = row[i];
    nan |= (v != v);
    if (better(v, i, bv, bi)) {
      bv = v;
      bi = i;
    }
  }
  if (nan) {  // a NaN beats everything and is remembered as index -1
    bv = INFINITY;
    bi = -1;
  }
#pragma unroll
  for (int off = TIE_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, TIE_WAVE);
    const int oi = __shfl_xor(bi, off, TIE_WAVE);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  const int lane = threadIdx.x & (TIE_WAVE - 1), wave = threadIdx.x / TIE_WAVE;
  if (lane == 0) {
    best_v[wave] = bv;
    best_i[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < static_cast<int>(blockDim.x) / TIE_WAVE; ++w)
      if (better(best_v[w], best_i[w], bv, bi)) {
        bv = best_v[w];
        bi = best_i[w];
      }
    part_v[r * ARGMAX_CHUNKS + chunk] = bv;
    part_i[r * ARGMAX_CHUNKS + chunk] = bi;
  }
}

__global__ void argmax_final_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i,
                                    int* __restrict__ out, float* __restrict__ max_out) {
  const int r = blockIdx.x;
  float bv = part_v[r * ARGMAX_CHUNKS + threadIdx.x];
  int bi = part_i[r * ARGMAX_CHUNKS + threadIdx.x];
#pragma unroll
  for (int off = TIE_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, TIE_WAVE);
    const int oi = __shfl_xor(bi, off, TIE_WAVE);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if (threadIdx.x == 0) {
    out[r] = bi;
    if (max_out != nullptr) max_out[r] = bv;
  }
}

// part_v / part_i: workspace of R * 64 floats / ints. max_out (optional): the maximum itself, per row.
extern "C" int tie_argmax(const float* logits, int* out, float* max_out, float* part_v, int* part_i, int R, int V,
                          hipStream_t stream) {
  if (R <= 0 || R > 65535 || V <= 0 || part_v == nullptr || part_i == nullptr) return TIE_BAD_ARGUMENT;
  static_assert(ARGMAX_CHUNKS == TIE_WAVE, "the final stage is one wave per row");
  argmax_partial_kernel<<<dim3(ARGMAX_CHUNKS, R), 256, 0, stream>>>(logits, part_v, part_i, V);
  int status = tie_launch_status();
  if (status != TIE_OK) return status;
  argmax_final_kernel<<<R, TIE_WAVE, 0, stream>>>(part_v, part_i, out, max_out);
  return tie_launch_status();
}

// The same two stages with the candidates in a file-scope array instead of a caller's workspace,
// for callers that cannot allocate (declared and described in argmax_static.h). In host code the
// array's name is only a stand-in: its address on a device comes from hipGetSymbolAddress, once per
// device with that device current, and that pointer is what the kernels receive.
// The array carries no `used` attribute: its use by host code below is what makes the compiler export
// the device symbol, which the runtime looks up by name; marked `used` it stays a local symbol and
// loading the library aborts.
#define ARGMAX_STATIC_DEVICES 64
static __device__ __align__(256) unsigned char argmax_static_scratch[TIE_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS *
                                                                      (sizeof(float) + sizeof(int))];
static void* argmax_static_ptr[ARGMAX_STATIC_DEVICES];   // per device: where its copy of the array lies
static std::mutex argmax_static_mutex;

extern "C" int tie_argmax_static(const float* logits, int* out, float* max_out, int R, int V, hipStream_t stream) {
  if (R <= 0 || V <= 0 || logits == nullptr || out == nullptr) return TIE_BAD_ARGUMENT;
  if (R > TIE_ARGMAX_STATIC_MAX_ROWS) {
    fprintf(stderr, "tie_argmax_static: %d rows exceed the %d rows its static scratch array holds\n", R,
            TIE_ARGMAX_STATIC_MAX_ROWS);
    return TIE_EXCEEDS_STATIC_SCRATCH;
  }
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return static_cast<int>(e);
  if (device < 0 || device >= ARGMAX_STATIC_DEVICES) return TIE_BAD_ARGUMENT;
  void* base;
  {
    std::lock_guard<std::mutex> lock(argmax_static_mutex);
    if (argmax_static_ptr[device] == nullptr) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_static_scratch));
      if (e != hipSuccess) return static_cast<int>(e);
      if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
      argmax_static_ptr[device] = p;
    }
    base = argmax_static_ptr[device];
  }
  float* part_v = static_cast<float*>(base);
  int* part_i = reinterpret_cast<int*>(part_v + static_cast<size_t>(TIE_ARGMAX_STATIC_MAX_ROWS) * ARGMAX_CHUNKS);
  return tie_argmax(logits, out, max_out, part_v, part_i, R, V, stream);
}

// ------------------------------------------------------ temperature sampling
// Draws out[r] from softmax(logits[r] * inv_temperature[r]) by inverting the
// cumulative sum in index order with the uniform number uniform[r] in [0, 1):
// weights exp((l - max) * inv_t) in float, sums in double, r = uniform * total,
// first index at which the running remainder turns negative
// (src/sampling/sampler.cpp:35-39,56-60,75-80 without top-k / top-p).
// out[r] = -1 for a row with a NaN, -2 for a row that is all -inf; a +inf logit wins outright.
//
// One workgroup a row, one pass for the sums: the waves own consecutive stretches of the row and read them in
// pieces of 256 logits (four in a row per lane, so the loads are whole lines); the sum of every piece goes to
// LDS. One thread then finds the piece in which u * total falls, walking the waves' sums and then that wave's
// pieces in index order, and a wave reads this one piece again and finds the lane and the logit.
#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / TIE_WAVE)
#define SAMPLE_PIECE (4 * TIE_WAVE)
#define SAMPLE_MAX_PIECES 4096          // rows of up to 2^20 logits

__device__ __forceinline__ double sample_wave_sum(double v) {
  for (int d = TIE_WAVE / 2; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

// Four logits from index i on; beyond the row -inf, which weighs nothing.
__device__ __forceinline__ float4 sample_load4(const float* row, int i, int V, bool by_four) {
  if (by_four && i + 3 < V) return *reinterpret_cast<const float4*>(row + i);
  float4 v;
  v.x = i < V ? row[i] : -INFINITY;
  v.y = i + 1 < V ? row[i + 1] : -INFINITY;
  v.z = i + 2 < V ? row[i + 2] : -INFINITY;
  v.w = i + 3 < V ? row[i + 3] : -INFINITY;
  return v;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ row_max,
                                                                const float* __restrict__ inv_temperature,
                                                                const double* __restrict__ uniform,
                                                                const double* __restrict__ other_uniform,
                                                                const int* __restrict__ take_other,
                                                                int* __restrict__ drew_none,
                                                                const int* __restrict__ rows, int* __restrict__ out,
                                                                int V) {
  __shared__ float fscratch[16];
  __shared__ double piece_sums[SAMPLE_MAX_PIECES];
  __shared__ double wave_sums[SAMPLE_WAVES];
  __shared__ double remainder;
  __shared__ int flag_nan, chosen, owner_piece;
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  const int tid = threadIdx.x, lane = tid & (TIE_WAVE - 1), wave = tid / TIE_WAVE;
  const float* row = logits + static_cast<size_t>(r) * V;
  const bool by_four = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  const int pieces = (V + SAMPLE_PIECE - 1) / SAMPLE_PIECE;
  const int per_wave = (pieces + SAMPLE_WAVES - 1) / SAMPLE_WAVES;
  const int first_piece = wave * per_wave;
  float mx;
  if (row_max) {
    // The caller looks at the maxima too: a row with a NaN or of -inf is its to report, and where the maximum
    // is +inf the argmax stands; none of them draws.
    mx = row_max[r];
    if (tid == 0 && drew_none) drew_none[r] = !(mx > -INFINITY && mx < INFINITY);
    if (!(mx > -INFINITY && mx < INFINITY)) return;
  } else {
    if (tid == 0) {
      flag_nan = 0;
      chosen = V;
    }
    __syncthreads();
    mx = -INFINITY;
    bool nan = false;
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      const float v = row[i];
      nan |= (v != v);
      mx = fmaxf(mx, v);
    }
    if (nan) flag_nan = 1;
    mx = block_max(mx, fscratch);
    __syncthreads();
    if (tid == 0 && drew_none) drew_none[r] = !(mx > -INFINITY && mx < INFINITY) || flag_nan;
    if (flag_nan || mx == -INFINITY) {
      if (tid == 0) out[r] = flag_nan ? -1 : -2;
      return;
    }
    if (mx == INFINITY) {  // the lowest +inf index wins without a draw
      int first = V;
      for (int i = tid; i < V; i += SAMPLE_THREADS)
        if (row[i] == INFINITY) first = min(first, i);
      if (first < V) atomicMin(&chosen, first);
      __syncthreads();
      if (tid == 0) out[r] = chosen;
      return;
    }
  }
  const float inv_t = inv_temperature[r];
  double of_wave = 0.0;
  for (int p0 = 0; p0 < per_wave; p0 += 4) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = sample_load4(row, (first_piece + p0 + u) * SAMPLE_PIECE + 4 * lane, V, by_four);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (p0 + u >= per_wave || first_piece + p0 + u >= pieces) break;
      double mine = static_cast<double>(expf((v[u].x - mx) * inv_t));
      mine += static_cast<double>(expf((v[u].y - mx) * inv_t));
      mine += static_cast<double>(expf((v[u].z - mx) * inv_t));
      mine += static_cast<double>(expf((v[u].w - mx) * inv_t));
      const double piece = sample_wave_sum(mine);
      if (lane == 0) piece_sums[first_piece + p0 + u] = piece;
      of_wave += piece;
    }
  }
  if (lane == 0) wave_sums[wave] = of_wave;
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) total += wave_sums[w];
    double rem = (take_other && take_other[r] ? other_uniform[r] : uniform[r]) * total;
    // The walk over the waves' sums, then over the pieces of the wave it stops in. Their sums were added in
    // other orders than the total, so by a rounding the walk may run past the end of either: then it ended, in
    // exact arithmetic, at the last token that weighs anything (an infinite remainder says so to the lanes).
    bool ran_past = false;
    int w = 0, p;
    for (; w < SAMPLE_WAVES; ++w) {
      if (rem - wave_sums[w] < 0.0) break;
      rem -= wave_sums[w];
    }
    if (w == SAMPLE_WAVES) {
      ran_past = true;
      p = pieces - 1;
    } else {
      p = w * per_wave;                    // the wave weighs more than the remainder: it has pieces
      const int last = min(p + per_wave, pieces) - 1;
      for (; p <= last; ++p) {
        if (rem - piece_sums[p] < 0.0) break;
        rem -= piece_sums[p];
      }
      if (p > last) {
        ran_past = true;
        p = last;
      }
    }
    if (ran_past) {
      while (p > 0 && !(piece_sums[p] > 0.0)) --p;
      rem = INFINITY;
    }
    owner_piece = p;
    remainder = rem;
  }
  __syncthreads();
  if (wave != 0) return;
  const int base = owner_piece * SAMPLE_PIECE + 4 * lane;
  const float4 v = sample_load4(row, base, V, by_four);
  const double w0 = static_cast<double>(expf((v.x - mx) * inv_t)), w1 = static_cast<double>(expf((v.y - mx) * inv_t));
  const double w2 = static_cast<double>(expf((v.z - mx) * inv_t)), w3 = static_cast<double>(expf((v.w - mx) * inv_t));
  const double mine = ((w0 + w1) + w2) + w3;
  double upto = mine;                     // of this lane and the lanes before it
  for (int d = 1; d < TIE_WAVE; d <<= 1) {
    const double other = __shfl_up(upto, d);
    if (lane >= d) upto += other;
  }
  // Only tokens that weigh something can be chosen. The lanes' running sums are added in different orders, so
  // that of a lane behind the last such token may exceed the one before it by a rounding, and rounding may also
  // leave a remainder beyond every lane's sum (this scan adds in another order than the piece's sum): then the
  // piece's last token that weighs anything, where the walk in exact arithmetic ends.
  const bool weighs = mine > 0.0;
  const unsigned long long reached = __ballot(weighs && remainder - upto < 0.0);
  const unsigned long long alive = __ballot(weighs);
  const int who = reached ? __ffsll(reached) - 1 : (alive ? 63 - __clzll(alive) : 0);
  int pick = min(owner_piece * SAMPLE_PIECE + SAMPLE_PIECE, V) - 1;
  if (lane == who && alive) {
    const double w[4] = {w0, w1, w2, w3};
    double rem = remainder - (upto - mine);
    int at = 0;
    bool found = false;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (found || !(w[i] > 0.0)) continue;
      at = i;                              // the last that weighs something, unless the walk ends earlier
      rem -= w[i];
      found = reached != 0 && rem < 0.0;
    }
    pick = base + at;
  }
  if (lane == who) out[r] = pick;
}

// With `rows` only the `num_rows` rows it lists are drawn, and out[] of the others is left as it is. With `row_max`
// (the rows' maxima) the kernel does not look for them, and leaves out[] of a row whose maximum is not finite as
// it is. `drew_none` (optional): 1 for a row that took no uniform number (no finite maximum), else 0.
// `take_other` (optional): where it is not 0 the row's number is other_uniform[r]; a caller that queues a step
// before it has read the one before passes that step's `drew_none` here, and both numbers the row's stream may
// be at.
extern "C" int tie_sample(const float* logits, const float* row_max, const float* inv_temperature, const double* uniform,
                          const double* other_uniform, const int* take_other, int* drew_none, const int* rows,
                          int num_rows, int* out, int R, int V, hipStream_t stream) {
  if (R <= 0 || V <= 0 || (rows && (num_rows <= 0 || num_rows > R))) return TIE_BAD_ARGUMENT;
  if (V > SAMPLE_MAX_PIECES * SAMPLE_PIECE || (take_other && !other_uniform)) return TIE_BAD_ARGUMENT;
  sample_kernel<<<rows ? num_rows : R, SAMPLE_THREADS, 0, stream>>>(logits, row_max, inv_temperature, uniform,
                                                                    other_uniform, take_other, drew_none, rows, out, V);
  return tie_launch_status();
}
