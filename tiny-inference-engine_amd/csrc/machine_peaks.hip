// What this GPU delivers when nothing but the measured resource is asked of it: a streaming read of memory
// that no cache holds, and matrix instructions fed from registers. A benchmark prices a decode step against the
// first and a prefill step against the second, beside the published peaks; neither is used by the engine itself.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) unsigned int mp_u32x4_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 mp_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mp_floatx16_t;

#define MP_IN_FLIGHT 8     // 16-byte loads a lane has outstanding: 8 KB a wave

// Every wave reads a run of consecutive memory of its own, 1 KB an instruction, MP_IN_FLIGHT instructions
// issued before the first is used; loads are marked non-temporal since nothing is read twice. `sink` is
// written only if the XOR of everything read equals a value it cannot have by accident, so the loads stay.
__global__ __launch_bounds__(256) void stream_read_kernel(const mp_u32x4_t* __restrict__ data, size_t chunks_per_wave,
                                                          unsigned* __restrict__ sink) {
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const size_t wave = static_cast<size_t>(blockIdx.x) * (blockDim.x / TIE_WAVE) + threadIdx.x / TIE_WAVE;
  const mp_u32x4_t* base = data + wave * chunks_per_wave * TIE_WAVE * MP_IN_FLIGHT;
  unsigned acc = 0;
  for (size_t c = 0; c < chunks_per_wave; ++c) {
    mp_u32x4_t v[MP_IN_FLIGHT];
#pragma unroll
    for (int u = 0; u < MP_IN_FLIGHT; ++u)
      v[u] = __builtin_nontemporal_load(base + (c * MP_IN_FLIGHT + u) * TIE_WAVE + lane);
#pragma unroll
    for (int u = 0; u < MP_IN_FLIGHT; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

// Reads the first `bytes` of `data` once (rounded down to whole chunks of 8 KB a wave over all waves); returns
// through *bytes_read how many bytes the launch reads. `workgroups` of four waves each.
extern "C" int tie_stream_read(const void* data, long long bytes, int workgroups, unsigned* sink,
                               long long* bytes_read, hipStream_t stream) {
  if (data == nullptr || sink == nullptr || bytes_read == nullptr || workgroups <= 0 || workgroups > (1 << 20) ||
      (reinterpret_cast<uintptr_t>(data) & 15) != 0)
    return TIE_BAD_ARGUMENT;
  const long long waves = static_cast<long long>(workgroups) * 4;
  const long long chunk = static_cast<long long>(TIE_WAVE) * MP_IN_FLIGHT * 16;
  const long long chunks_per_wave = bytes / (waves * chunk);
  if (chunks_per_wave <= 0) return TIE_BAD_ARGUMENT;
  *bytes_read = chunks_per_wave * waves * chunk;
  stream_read_kernel<<<workgroups, 256, 0, stream>>>(static_cast<const mp_u32x4_t*>(data),
                                                     static_cast<size_t>(chunks_per_wave), sink);
  return tie_launch_status();
}

// Four independent 32 x 32 x 16 bfloat16 matrix instructions a round, operands and accumulators in registers,
// nothing loaded or stored in the loop: the rate the matrix cores reach at the clock the chip sustains.
__global__ __launch_bounds__(256) void mfma_rate_kernel(int rounds, float* __restrict__ sink) {
  mp_bf16x8_t a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(0.001f * static_cast<float>((threadIdx.x + i) % 7));
    b[i] = static_cast<__bf16>(0.002f * static_cast<float>((threadIdx.x + 2 * i) % 5));
  }
  mp_floatx16_t acc0 = {0}, acc1 = {0}, acc2 = {0}, acc3 = {0};
  for (int r = 0; r < rounds; ++r) {
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc1, 0, 0, 0);
    acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc2, 0, 0, 0);
    acc3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc3, 0, 0, 0);
  }
  float total = 0.f;
  for (int i = 0; i < 16; ++i) total += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  if (total == -1.f) sink[0] = total;
}

// Launches `workgroups` x 4 waves of `rounds` x 4 matrix instructions; *flops receives the floating-point
// operations of the launch (2 x 32 x 32 x 16 an instruction).
extern "C" int tie_mfma_rate(int workgroups, int rounds, float* sink, double* flops, hipStream_t stream) {
  if (workgroups <= 0 || workgroups > (1 << 20) || rounds <= 0 || sink == nullptr || flops == nullptr)
    return TIE_BAD_ARGUMENT;
  *flops = static_cast<double>(workgroups) * 4.0 * rounds * 4.0 * (2.0 * 32 * 32 * 16);
  mfma_rate_kernel<<<workgroups, 256, 0, stream>>>(rounds, sink);
  return tie_launch_status();
}
