// What the kernels that prepare queries and keys share: sums over planes of partial sums, the per-head RMS
// norm and the rotation by a table of angles for heads whose lanes hold 4 + 4 elements (head_dim / 8 lanes
// a head). The q/k kernel and the decode attention kernel that prepares its own queries both call these, so
// a query is the same bits on either way.
#pragma once

template <typename TX>
__device__ __forceinline__ float load_planes(const TX* p, size_t plane_stride, int planes) {
  // The usual cuts (2, 4, 8) have all their loads in flight together; the sum is formed in plane order in every case.
  if (planes == 2) return load_as_float(p) + load_as_float(p + plane_stride);
  if (planes == 4 || planes == 8) {
    float part[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) part[s] = s < planes ? load_as_float(p + static_cast<size_t>(s) * plane_stride) : 0.f;
    float v = part[0];
#pragma unroll
    for (int s = 1; s < 8; ++s)
      if (s < planes) v += part[s];
    return v;
  }
  float v = load_as_float(p);
  for (int s = 1; s < planes; ++s) v += load_as_float(p + static_cast<size_t>(s) * plane_stride);
  return v;
}

typedef __attribute__((ext_vector_type(4))) float qk_f4_t;

template <typename T>
__device__ __forceinline__ qk_f4_t load4(const T* p);
template <>
__device__ __forceinline__ qk_f4_t load4<float>(const float* p) { return *reinterpret_cast<const qk_f4_t*>(p); }
template <>
__device__ __forceinline__ qk_f4_t load4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return qk_f4_t{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                 __uint_as_float(v.y & 0xffff0000u)};
}
template <typename T>
__device__ __forceinline__ void store4(T* p, qk_f4_t v);
template <>
__device__ __forceinline__ void store4<float>(float* p, qk_f4_t v) { *reinterpret_cast<qk_f4_t*>(p) = v; }
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, qk_f4_t v) {
  uint2 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  *reinterpret_cast<uint2*>(p) = o;
}

template <>
__device__ __forceinline__ void store4<f16_t>(f16_t* p, qk_f4_t v) {
  typedef __attribute__((ext_vector_type(4))) _Float16 qk_h4_t;
  *reinterpret_cast<qk_h4_t*>(p) = __builtin_convertvector(v, qk_h4_t);
}

template <typename TX>
__device__ __forceinline__ qk_f4_t load4_planes(const TX* p, size_t plane_stride, int planes) {
  if (planes == 2) return load4(p) + load4(p + plane_stride);
  if (planes == 4 || planes == 8) {
    qk_f4_t part[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
      part[s] = s < planes ? load4(p + static_cast<size_t>(s) * plane_stride) : qk_f4_t{0.f, 0.f, 0.f, 0.f};
    qk_f4_t v = part[0];
#pragma unroll
    for (int s = 1; s < 8; ++s)
      if (s < planes) v += part[s];
    return v;
  }
  qk_f4_t v = load4(p);
  for (int s = 1; s < planes; ++s) v += load4(p + static_cast<size_t>(s) * plane_stride);
  return v;
}

// RMS norm of one head: lane i of the head's LPH lanes holds elements 4 i .. 4 i + 3 (a) and the four they pair
// with in the second half (b); the sums of squares meet by shuffles inside the head's lanes. All LPH lanes of
// a head call this together. Formula: src/backend/cpu/cpu_backend.cpp:141-159 over one head (src/model/qwen3.cpp:222-223).
template <int LPH>
__device__ __forceinline__ void qk_head_norm(qk_f4_t& a, qk_f4_t& b, const float* __restrict__ w, float eps, int p0) {
  constexpr int Dh = LPH * 8, half = LPH * 4;
  float ss = (a[0] * a[0] + b[0] * b[0]) + (a[1] * a[1] + b[1] * b[1]) + (a[2] * a[2] + b[2] * b[2]) +
             (a[3] * a[3] + b[3] * b[3]);
#pragma unroll
  for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, TIE_WAVE);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(Dh) + eps);
  a = (a * inv) * load4(w + p0);
  b = (b * inv) * load4(w + half + p0);
}

// Rotation of the pairs (i, i + head_dim / 2) by the angles of one token: row = cos of the head_dim / 2 angles,
// then their sines. Formula: src/backend/cpu/cpu_backend.cpp:161-193, src/backend/rope.h:9-13.
template <int LPH>
__device__ __forceinline__ void qk_rotate_by_table(qk_f4_t a, qk_f4_t b, const float* __restrict__ row, int p0,
                                                   qk_f4_t& o1, qk_f4_t& o2) {
  constexpr int half = LPH * 4;
  const qk_f4_t cs = load4(row + p0);
  const qk_f4_t sn = load4(row + half + p0);
  o1 = a * cs - b * sn;
  o2 = b * cs + a * sn;
}
