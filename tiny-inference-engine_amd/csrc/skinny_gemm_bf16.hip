// The decode-time matrix product for gfx950: out[M, N] (+)= x[M, K] . w[N, K]^T for few rows M
// (1..64), bfloat16 operands, float32 accumulation on v_mfma_f32_16x16x32_bf16.
//
// The product is bound by reading w once from HBM, so the kernel is built around that stream.
// A workgroup of four waves owns RT tiles of 16 rows of w and one of `splits` ranges of K; its
// waves split that range into contiguous parts. Every lane reads 16 bytes of "its" row per MFMA
// (row = lane % 16, k-chunk = lane / 16), which is exactly the B-operand layout, so weights go from
// memory to the matrix core with no staging. The few rows of x are the A operand, read through the
// caches (they are shared by every workgroup); rows beyond M are zeros. One x fragment feeds the
// RT weight tiles of the wave, which is what keeps the x traffic below the weight traffic when M
// grows: RT is chosen per launch from M and the number of workgroups that results. The waves'
// partial sums meet in LDS and are added in a fixed order.
//
// With splits > 1 the output is [splits, M, N] float32 partial sums, one plane per range of K, for
// the consumer to add up in plane order (no atomics, no fences: the result is the same in every
// run). How K is cut depends on K, splits and the waves of a workgroup, never on RT or on which rows
// are present; up to 16 rows the caller's splits follow from the weight's shape alone, so a row's sums
// are formed in the same order whatever else is in the batch. From 17 rows on the plan (few_rows_plan)
// may name other ranges for another number of rows: between steps of such sizes a row's sums differ
// by rounding, as they do between this product and the tiled one.
//
// Requires K % 8 == 0 (16-byte loads); other shapes go to the generic kernel.
//
// Two things a decode step's RMS norms would otherwise need kernels of their own for ride in the epilogue
// (SkNorm, up to 16 rows): a product that ends a sub-layer and is not cut along K adds its sums to the residual
// stream x in place, stores bf16(x * w) for the norm that follows (its weight w, the 1 / rms left out) and, per
// row and 16-column tile, the sum of the squares of the new x; the products that read those rows multiply their
// sums by 1 / sqrt(sum of the squares / n + eps), the factor that was left out (every workgroup adds the
// tiles' squares in the same fixed order), which commutes with the product. Sums of squares, the factor and
// the stream stay float32. Not cut along K, a narrow output would leave such a product one workgroup of four
// waves a compute unit; it runs in workgroups of sixteen waves over one tile, or eight over two (producer_shape).
//
// PACKED: w is stored as [N/16][K/32] blocks of 1 KB, block (t, b) holding rows 16 t .. 16 t + 15 over
// k = 32 b .. 32 b + 31 in the order the matrix core takes them: lane l's 16 bytes (row l % 16, k-chunk
// l / 16) at byte 16 l. A wave's load is then 1 KB of consecutive memory and its stream through K one
// contiguous run, which the memory system serves measurably faster than 16 rows' 64-byte pieces
// (6.1 against 5.1 TB/s on a 201 MB weight); read once, the stream is loaded non-temporally.
#include "common.h"

#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define SK_WAVES 4

__device__ __forceinline__ bf16x8_t load_frag(const bf16_t* p) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  return *reinterpret_cast<const bf16x8_t*>(&v);
}

typedef __attribute__((ext_vector_type(4))) unsigned int sk_u32x4_t;

template <bool PACKED>
__device__ __forceinline__ bf16x8_t load_weight_frag(const bf16_t* p) {
  if (PACKED) {
    const sk_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const sk_u32x4_t*>(p));
    return *reinterpret_cast<const bf16x8_t*>(&v);
  }
  return load_frag(p);
}

__device__ __forceinline__ bf16x8_t zero_frag() {
  const uint4 v = make_uint4(0, 0, 0, 0);
  return *reinterpret_cast<const bf16x8_t*>(&v);
}

// What the epilogue does for the RMS norms around a product (all null / zero: nothing).
struct SkNorm {
  // the rows of x are norm inputs without their 1 / rms: sums are multiplied by
  // 1 / sqrt((scale_squares[m][0] + ... + scale_squares[m][scale_tiles - 1]) / scale_n + scale_eps)
  const float* scale_squares;
  int scale_tiles;
  float scale_n, scale_eps;
  // the product ends a sub-layer: out is the residual stream (added to in place); next_x[m][n] = bf16(out * next_w[n])
  // and squares[m][n / 16] = the sum over the tile's 16 columns of out^2 are left for the norm that follows
  const float* next_w;
  bf16_t* next_x;
  float* squares;
};

#define SK_NORM_ROWS 16     // rows the epilogue's norm work takes
#define SK_SCALE_LDS_MAX 32768   // bytes of LDS for the tiles' sums of the rows to be scaled: 16 rows of a width of 8192

typedef __attribute__((address_space(3))) void sk_lds_void_t;
// Fourth word of a raw buffer descriptor on gfx9-family GPUs: 32-bit float data format, destination
// selects x, y, z, w; no swizzle, no stride.
#define SK_RSRC_FLAGS 0x27000

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14; the other counters at their maxima).
template <int N>
__device__ __forceinline__ void rows_wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// The sum of v over the 16 lanes that share lane / 16, in every one of them: four rotations within the row of 16
// (data-parallel primitives of the vector unit, a few cycles each, where a shuffle goes through LDS). Additions
// commute, so the 16 lanes end with the same bits.
__device__ __forceinline__ float sum_of_16_lanes(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}

// The sums of squares a norm left per 16-column tile, [rows][tiles rounded up to 64]: dynamic LDS, present only in
// launches whose sums are to be scaled (SkNorm::scale_squares).
extern __shared__ float sk_scale_parts[];

// MT: 16-row tiles of x; RT: 16-row tiles of w per workgroup; U: k-blocks of 32 in one batch of loads.
template <int MT, int RT, int U, typename TO, bool PACKED, int WAVES = SK_WAVES>
__global__ __launch_bounds__(WAVES* TIE_WAVE) void skinny_gemm_kernel(const bf16_t* __restrict__ x,
                                                                         const bf16_t* __restrict__ w,
                                                                         TO* __restrict__ out, int M, int N, int K,
                                                                         int accumulate, int gated, int per_wave,
                                                                         SkNorm norm) {
  const int tile_group = blockIdx.x, split = blockIdx.y, num_splits = gridDim.y;
  __shared__ float red[WAVES][MT][RT][256];
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = threadIdx.x / TIE_WAVE;
  const bool scaled = norm.scale_squares != nullptr;
  const int scale_chunks = (norm.scale_tiles + TIE_WAVE - 1) / TIE_WAVE;   // 64 tiles an instruction
  if (scaled) {
    // Wave v takes rows v, v + 4, ...: the tiles' sums go from memory straight into LDS, asked for before the
    // first weight and not waited for until the weights are through (a wait here would hold back the weights'
    // loads for a memory latency, in a kernel that lasts a few of them). Tiles beyond the row's end are asked
    // for beyond the buffer's end and arrive as zeros.
    const unsigned bytes = static_cast<unsigned>(min(M, SK_NORM_ROWS)) * norm.scale_tiles * 4u;
    const __amdgpu_buffer_rsrc_t sq_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(norm.scale_squares), 0, static_cast<int>(bytes), SK_RSRC_FLAGS);
    for (int m = wave; m < M && m < SK_NORM_ROWS; m += WAVES)
      for (int j = 0; j < scale_chunks; ++j) {
        const int t = j * TIE_WAVE + lane;
        const unsigned at = t < norm.scale_tiles ? (static_cast<unsigned>(m) * norm.scale_tiles + t) * 4u : bytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(sq_rsrc, (sk_lds_void_t*)(&sk_scale_parts[(m * scale_chunks + j) * TIE_WAVE]),
                                                 4, at, 0, 0, 0);
      }
  }
  const int r = lane & 15;   // row of the 16-row tile (of w for B, of x for A)
  const int g = lane >> 4;   // which 8-element chunk of the 32-wide k block
  const int n0 = tile_group * 16 * RT;

  // The end of a sub-layer: what the epilogue adds to and multiplies by is asked for now, for the same reason.
  // Thread e of the workgroup ends up with row e / 16 % 16, column e % 16 of tile e / 256 (and of the tiles a
  // workgroup's worth of threads further on); no other thread or workgroup touches those elements of the stream.
  constexpr int ENDS = (256 * RT + WAVES * TIE_WAVE - 1) / (WAVES * TIE_WAVE);   // elements a thread ends up with
  float stream_now[ENDS], next_weight[ENDS];
  if constexpr (MT == 1 && std::is_same<TO, float>::value) {
    if (norm.next_x != nullptr) {
#pragma unroll
      for (int i = 0; i < ENDS; ++i) {
        const int e = threadIdx.x + i * WAVES * TIE_WAVE;
        const int m = (e & 255) >> 4, n = n0 + (e >> 8) * 16 + (e & 15);
        const bool inside = e < 256 * RT && m < M && n < N;
        stream_now[i] = inside ? out[static_cast<size_t>(m) * N + n] : 0.f;
        next_weight[i] = inside ? norm.next_w[n] : 0.f;
      }
    }
  }

  // Rows beyond N are clamped for the loads; their columns are dropped at the store. wp[t] points at
  // this lane's 16 bytes of k-block 0; a k-block further on is KB_STRIDE elements further on.
  constexpr int KB_STRIDE = PACKED ? 512 : 32;
  const bf16_t* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (PACKED) wp[t] = w + static_cast<size_t>(min(n0 / 16 + t, (N - 1) / 16)) * (K / 32) * 512 + lane * 8;
    else wp[t] = w + static_cast<size_t>(min(n0 + t * 16 + r, N - 1)) * K + g * 8;
  }
  const bf16_t* xp[MT];
  bool xvalid[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    xvalid[mt] = m < M;
    xp[mt] = x + static_cast<size_t>(xvalid[mt] ? m : 0) * K;
  }

  // This wave's k range, in blocks of 32: part (split, wave) of gridDim.y * WAVES equal parts.
  const int kblocks = (K + 31) / 32;
  const int kb_begin = min(kblocks, (split * WAVES + wave) * per_wave);
  const int kb_end = min(kblocks, kb_begin + per_wave);

  floatx4 acc[MT][RT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  int kb = kb_begin;
  // Main loop: batches of U blocks. The loads of the next batch are issued before the matrix instructions
  // of the current one, so 2 U blocks of every tile are in flight per wave: a workgroup's share of a narrow
  // weight is a few dozen KB, and it is the bytes in flight, not the instruction rate, that its time hangs on.
  const int batches = (min(kb_end, K / 32) - kb_begin) / U;
  if (batches > 0) {
    bf16x8_t b[RT][U], a[MT][U];
    auto load_batch = [&](bf16x8_t (&bb)[RT][U], bf16x8_t (&aa)[MT][U], int at) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = (at + u) * 32 + g * 8;
#pragma unroll
        for (int t = 0; t < RT; ++t) bb[t][u] = load_weight_frag<PACKED>(wp[t] + static_cast<size_t>(at + u) * KB_STRIDE);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) aa[mt][u] = xvalid[mt] ? load_frag(xp[mt] + k) : zero_frag();
      }
    };
    auto multiply = [&](const bf16x8_t (&bb)[RT][U], const bf16x8_t (&aa)[MT][U]) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int t = 0; t < RT; ++t)
            acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aa[mt][u], bb[t][u], acc[mt][t], 0, 0, 0);
    };
    load_batch(b, a, kb);
    for (int i = 1; i < batches; ++i) {
      bf16x8_t nb[RT][U], na[MT][U];
      load_batch(nb, na, kb + U);
      multiply(b, a);
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int t = 0; t < RT; ++t) b[t][u] = nb[t][u];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[mt][u] = na[mt][u];
      }
      kb += U;
    }
    multiply(b, a);
    kb += U;
  }
  // Remainder, one block at a time; the last block may be partly beyond K.
  for (; kb < kb_end; ++kb) {
    const int k = kb * 32 + g * 8;
    const bool kvalid = k < K;  // K % 8 == 0: a chunk is whole or absent
    bf16x8_t a[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a[mt] = (kvalid && xvalid[mt]) ? load_frag(xp[mt] + k) : zero_frag();
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const bf16x8_t b = kvalid ? load_weight_frag<PACKED>(wp[t] + static_cast<size_t>(kb) * KB_STRIDE) : zero_frag();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt], b, acc[mt][t], 0, 0, 0);
    }
  }

  // The tiles' sums have to be there before the barrier below, whichever wave asked for them.
  if (scaled) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // D layout: lane holds rows (lane / 16) * 4 + v of x, column lane % 16 of w.
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave][mt][t][(g * 4 + v) * 16 + r] = acc[mt][t][v];
  __syncthreads();

  const bool partial = num_splits > 1;   // then TO is float and out holds one [M, N] plane per split
  // 1 / rms of the row this thread's elements lie in (thread e: row e / 16 % 16, in every pass of the loops
  // below). The 16 lanes of a row add its tiles j, j + 16, ... each in ascending order, then meet: the same
  // sums in every workgroup of every launch, whatever the batch.
  float row_scale = 1.0f;
  if (scaled) {
    const int m = (static_cast<int>(threadIdx.x) & 255) >> 4, j = threadIdx.x & 15;
    float sq = 0.f;
    if (m < M)
      for (int i = j; i < scale_chunks * TIE_WAVE; i += 16) sq += sk_scale_parts[m * scale_chunks * TIE_WAVE + i];
    sq = sum_of_16_lanes(sq);
    row_scale = 1.0f / sqrtf(sq / norm.scale_n + norm.scale_eps);
  }
  if (norm.next_x != nullptr) {
    // The end of a sub-layer (MT = 1, one plane, float32 out = the residual stream): the 16 lanes that hold a
    // row's 16 columns of a tile stay together for the sum of its squares.
    if constexpr (std::is_same<TO, float>::value) {
#pragma unroll
      for (int i = 0; i < ENDS; ++i) {
        const int e = threadIdx.x + i * WAVES * TIE_WAVE;
        if (e >= 256 * RT) break;            // whole waves at a time: 256 RT is a multiple of the wave
        const int ee = e & 255, t = e >> 8;
        const int c = ee & 15, m = ee >> 4;
        const int n = n0 + t * 16 + c;
        const bool inside = m < M && n < N;
        float sum = red[0][0][t][ee];
#pragma unroll
        for (int wv = 1; wv < WAVES; ++wv) sum += red[wv][0][t][ee];
        float now = 0.f;
        if (inside) {
          if (scaled) sum *= row_scale;
          now = stream_now[i] + sum;
          out[static_cast<size_t>(m) * N + n] = now;
          norm.next_x[static_cast<size_t>(m) * N + n] = float_to_bf16(now * next_weight[i]);
        }
        const float sq = sum_of_16_lanes(now * now);
        if (c == 0 && m < M && n < N) norm.squares[static_cast<size_t>(m) * (N / 16) + n / 16] = sq;
      }
    }
    return;
  }
  for (int e = threadIdx.x; e < 256 * RT * MT; e += WAVES * TIE_WAVE) {
    const int ee = e & 255;            // 16 x 16 outputs of a tile
    const int t = (e >> 8) % RT;
    const int mt = e / (256 * RT);
    const int c = ee & 15;
    const int m = mt * 16 + (ee >> 4);
    const int n = n0 + t * 16 + c;
    if (m >= M || n >= N) continue;
    if (gated && c >= 8) continue;       // gated: columns 0..7 are gates, 8..15 the ups of the same outputs
    float sum = red[0][mt][t][ee];
#pragma unroll
    for (int wv = 1; wv < WAVES; ++wv) sum += red[wv][mt][t][ee];
    if (scaled) sum *= row_scale;
    if (gated) {
      float up = red[0][mt][t][ee + 8];
#pragma unroll
      for (int wv = 1; wv < WAVES; ++wv) up += red[wv][mt][t][ee + 8];
      if (scaled) up *= row_scale;
      store_from_float(out + static_cast<size_t>(m) * (N / 2) + (n0 + t * 16) / 2 + c, sum / (1.0f + __expf(-sum)) * up);
      continue;
    }
    TO* o = out + (static_cast<size_t>(partial ? split : 0) * M + m) * N + n;
    if (accumulate) sum = load_as_float(o) + sum;
    store_from_float(o, sum);
  }
}

// ------------------------------------------------------------------ 17 to 64 rows: x through LDS
// With more than one 16-row tile of x the kernel above spends most of its load instructions on x: every
// weight block of 1 KB needs MT blocks of x, and a compute unit serves a load instruction of a wave in about 65
// cycles whether it comes from HBM or from L2, so at 64 rows (7 loads for 3 KB of weights) the weights stream
// at 3.6 TB/s. Here the WAVES waves of a workgroup walk the SAME range of K, each over its own RT weight
// tiles, and share x: a chunk of U k-blocks of all rows goes from global memory straight into LDS (buffer
// loads with the lds flag; one instruction brings one 16-row block of 32 k, lane l's 16 bytes - row l % 16,
// k-chunk l / 16 - to byte 16 l, which is the order the matrix core takes its A operand) and all waves read
// their fragments from there. Weights still go from memory straight into registers, non-temporally. x then
// costs MT / (WAVES x RT) of the weights' load instructions.
//
// Both streams run DEPTH chunks ahead of the arithmetic, through a ring of DEPTH + 1 LDS buffers and register
// sets, and a step waits only until the NEXT chunk has landed (loads complete in the order they were asked
// for, so that is when at most the loads of the DEPTH - 1 chunks after it are outstanding): the queue of
// loads never runs empty. (Waiting for everything at each chunk's barrier, as a first version did, left a wave
// idle for a memory latency a chunk: gate/up of the 8B shape at 64 rows 54 us, now 42.) What bounds it now is
// x itself: every workgroup reads all of it, 512 KB beside its 785 KB of weights on that shape, and a compute
// unit takes about 38 GB/s.
//
// The sums are the very ones of the kernel above: a plane's range of K is walked in the same four parts
// of per_wave k-blocks, each summed by the matrix core in k order, and the parts are added in their order
// (there: by the reduction through LDS; here: by folding the accumulator into a running total at each
// part's end). A row's result therefore does not depend on which of the two kernels its batch size picks.
// The matrix instructions of one chunk: x from LDS, the weights from registers. A function of its own with
// restrict pointers, so that the compiler knows these LDS reads from the loads into LDS that are in flight
// (otherwise it waits for all of them before the first read).
template <int MT, int RT, int U, bool FULL>
__device__ __forceinline__ void rows_chunk(const bf16_t* __restrict__ xc, const bf16x8_t (&wr)[RT][U],
                                           floatx4 (&acc)[MT][RT], int kb0, int kb_hi, int lane) {
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (FULL || kb0 + u < kb_hi) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const sk_u32x4_t av = *reinterpret_cast<const sk_u32x4_t*>(xc + (u * MT + mt) * 512 + lane * 8);
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&av);
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, wr[t][u], acc[mt][t], 0, 0, 0);
      }
    }
  }
}

// Calls f(integral_constant<int, I>) for I = 0 .. N - 1.
template <int N, int I = 0, typename F>
__device__ __forceinline__ void rows_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    rows_static_for<N, I + 1>(f);
  }
}

// U: k-blocks of a chunk; DEPTH: chunks in flight behind the one at work.
template <int MT, int RT, int WAVES, int U, int DEPTH, typename TO>
__global__ __launch_bounds__(WAVES* TIE_WAVE) void skinny_rows_kernel(const bf16_t* __restrict__ x,
                                                                      const bf16_t* __restrict__ w,
                                                                      TO* __restrict__ out, int M, int N, int K,
                                                                      int accumulate, int gated, int per_wave) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NS = DEPTH + 1;
  constexpr int NX = (U * MT + WAVES - 1) / WAVES;      // blocks of x a wave loads a chunk
  constexpr int PER_CHUNK = NX + RT * U;                // loads a wave issues a chunk
  __shared__ __attribute__((aligned(16))) bf16_t xs[NS][U * MT * 512];
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TIE_WAVE);
  const int tiles = N / 16;
  const int tile0 = (static_cast<int>(blockIdx.x) * WAVES + wave) * RT;
  const int split = blockIdx.y;
  const int kblocks = K / 32;
  const int kb_lo = min(kblocks, split * SK_WAVES * per_wave);
  const int kb_hi = min(kblocks, kb_lo + SK_WAVES * per_wave);

  const bf16_t* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) wp[t] = w + static_cast<size_t>(min(tile0 + t, tiles - 1)) * kblocks * 512 + lane * 8;

  // x as a buffer: rows beyond M lie beyond its end and read as zeros.
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(x), 0, static_cast<int>(static_cast<size_t>(M) * K * 2), SK_RSRC_FLAGS);
  const unsigned lane_off = (static_cast<unsigned>(lane & 15) * K + (lane >> 4) * 8) * 2;   // bytes, within a 16-row block
  const unsigned tile_rows = 16u * K * 2;

  // Chunk c: k-blocks kb_lo + c U and the U - 1 after it. Its loads, into set S of the ring: every wave issues
  // the same number of them whatever the chunk (the waits count instructions): the blocks (u, mt) of x are dealt
  // to the waves in turn, a wave with one block fewer loads one of the others' again, and k-blocks beyond the
  // range are the range's last again (their products are not formed).
  bf16x8_t wr[NS][RT][U];
  auto issue = [&](auto set, int chunk) {
    constexpr int S = decltype(set)::value;
    const int kb0 = kb_lo + chunk * U;
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int b = (i * WAVES + wave) % (U * MT);
      const int u = b / MT, mt = b % MT;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (sk_lds_void_t*)(&xs[S][(u * MT + mt) * 512]), 16,
                                               lane_off + mt * tile_rows, min(kb0 + u, kb_hi - 1) * 64, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
        wr[S][t][u] = load_weight_frag<true>(wp[t] + static_cast<size_t>(min(kb0 + u, kb_hi - 1)) * 512);
  };

  floatx4 acc[MT][RT], total[MT][RT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[mt][t] = total[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  // A part of K has ended: total += part. Parts are whole chunks (the host sees to it), so this stands between
  // two chunks.
  int part_end = kb_lo + per_wave;
  auto fold_at = [&](int kb0) {
    if (kb0 != part_end) return;
    part_end += per_wave;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int v = 0; v < 4; ++v) total[mt][t][v] += acc[mt][t][v];
        acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
  };

  if (kb_lo < kb_hi) {
    const int chunks = (kb_hi - kb_lo + U - 1) / U;
    // DEPTH chunks are in flight behind the one whose products are formed. A step: ask for chunk c + DEPTH
    // (into the set that chunk c - 1 left), form chunk c's products, then wait until chunk c + 1 has landed,
    // which is when at most the loads of the DEPTH - 1 chunks after it are outstanding, and meet the other
    // waves: their blocks of x have landed too, and all have read chunk c's.
    auto step = [&](auto set, auto next_set, int c) {
      issue(next_set, c + DEPTH);
      fold_at(kb_lo + c * U);
      rows_chunk<MT, RT, U, true>(&xs[decltype(set)::value][0], wr[decltype(set)::value], acc, kb_lo + c * U, kb_hi, lane);
      rows_wait_loads<(DEPTH - 1) * PER_CHUNK>();
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    // The range's last chunks, with nothing more to ask for.
    auto last_step = [&](auto set, int c) {
      fold_at(kb_lo + c * U);
      rows_chunk<MT, RT, U, false>(&xs[decltype(set)::value][0], wr[decltype(set)::value], acc, kb_lo + c * U, kb_hi, lane);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    static_assert((DEPTH - 1) * PER_CHUNK < 64, "the wait counts loads with six bits");
    rows_static_for<DEPTH>([&](auto i) { issue(i, decltype(i)::value); });
    rows_wait_loads<(DEPTH - 1) * PER_CHUNK>();
    asm volatile("s_barrier" ::: "memory");
    // The ring's sets are named at compile time, so the steps come in groups of NS.
    int c = 0;
    for (; c + NS - 1 + DEPTH < chunks; c += NS)
      rows_static_for<NS>([&](auto i) {
        constexpr int I = decltype(i)::value;
        step(i, std::integral_constant<int, (I + DEPTH) % NS>{}, c + I);
      });
    // Up to NS - 1 + DEPTH chunks are left; those that still have a chunk DEPTH ahead ask for it.
    rows_static_for<NS - 1 + DEPTH>([&](auto i) {
      constexpr int I = decltype(i)::value;
      if (c + I + DEPTH < chunks) step(std::integral_constant<int, I % NS>{}, std::integral_constant<int, (I + DEPTH) % NS>{}, c + I);
      else if (c + I < chunks) last_step(std::integral_constant<int, I % NS>{}, c + I);
    });
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) total[mt][t][v] += acc[mt][t][v];

  // D layout: lane holds rows (lane / 16) * 4 + v of a 16-row tile of x, column lane % 16 of the weight tile.
  const int c = lane & 15, q4 = (lane >> 4) * 4;
  const bool partial = gridDim.y > 1;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (tile0 + t >= tiles) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = mt * 16 + q4 + v;
        float sum = total[mt][t][v];
        if (gated) {       // columns 0..7 are gates, 8..15 the ups of the same outputs
          const float up = __shfl(sum, (lane & 48) | ((c + 8) & 15), TIE_WAVE);
          if (m < M && c < 8)
            store_from_float(out + static_cast<size_t>(m) * (N / 2) + (tile0 + t) * 8 + c, sum / (1.0f + __expf(-sum)) * up);
          continue;
        }
        if (m >= M) continue;
        TO* o = out + (static_cast<size_t>(partial ? split : 0) * M + m) * N + (tile0 + t) * 16 + c;
        if (accumulate) sum = load_as_float(o) + sum;
        store_from_float(o, sum);
      }
  }
#endif
}

static int compute_units() {
  static int cached = 0;
  if (cached == 0) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
      count = 256;
    cached = count;
  }
  return cached;
}

// Weight tiles per workgroup. More tiles reuse each x fragment more often (x costs about half a
// weight tile's traffic per 16 rows of it) but leave fewer workgroups, which hurts when their number
// is not a multiple of the compute units. Does not change any sum.
static int choose_rt(int M, int N, int splits) {
  if (M <= 4) return 1;
  const int cus = compute_units();
  const int tiles = (N + 15) / 16;
  int best = 1;
  double best_cost = 0;
  for (int rt = 1; rt <= (M > 8 ? 4 : 3); ++rt) {
    const long wgs = static_cast<long>((tiles + rt - 1) / rt) * splits;
    const double fill = static_cast<double>(wgs) / static_cast<double>((wgs + cus - 1) / cus * cus);
    const double cost = (1.0 + 0.5 * (M / 16.0) / rt) / fill;
    if (rt == 1 || cost <= best_cost) {
      best = rt;
      best_cost = cost;
    }
  }
  return best;
}

// Which kernel, how many weight tiles a workgroup and how many ranges of K a product of 17 to 64 rows takes
// (up to 16 rows: the kernel that reads x from memory, choose_rt and tie_skinny_gemm_splits). One score for
// every candidate, the smallest wins:
//
//     (1 + b x (16-row tiles of x) / (weight tiles that share one load of x)) x (1 + 0.15 log2(ranges)) / fill
//
// The first factor is what x costs beside the weights: a wave of the kernel that reads x from memory loads a
// block of x for every `rt` weight blocks (b = 0.4); in the kernel that shares x through LDS a workgroup loads it
// once for its 3, 6 or 8 tiles (b = 0.2, and the whole score x 0.95: its loads never drain). The second is the
// planes' traffic and the shorter runs of K. The third is how full the compute units are: workgroups run in
// rounds of one a compute unit, and a round that is part empty lasts as long as a full one.
// The constants were chosen on sweeps over the four projections of eight shapes (widths 1024 to 8192) at 24 to 64
// rows, every candidate timed together with the kernel that consumes its planes: the choice lies 2.3 % above the
// best candidate on average (the thresholds on three shapes that stood here before: 7.3 %), within 5 % on 105 of
// 128 points, and on the three shapes held out of the choosing (widths 2560, 3072 and 5120 with K of 17408) 2.7 %.
extern "C" int tie_skinny_gemm_splits(int N, int K);

struct FewRowsPlan { int shares_x, tiles, splits; };

static FewRowsPlan few_rows_plan(int M, int N, int K, int gated, int splits_fixed) {
  const int tiles = (N + 15) / 16, kblocks = (K + 31) / 32, cus = compute_units();
  const int by_shape = gated ? 1 : tie_skinny_gemm_splits(N, K);
  FewRowsPlan best = {0, 1, splits_fixed > 0 ? splits_fixed : by_shape};
  double best_score = 0.0;
  auto fill = [&](long wgs) { return static_cast<double>(wgs) / static_cast<double>((wgs + cus - 1) / cus * cus); };
  auto offer = [&](double score, int shares_x, int t, int splits) {
    if (best_score == 0.0 || score < best_score) {
      best = {shares_x, t, splits};
      best_score = score;
    }
  };
  for (int splits = 1; splits <= 8; splits *= 2) {
    if (splits_fixed > 0 ? splits != splits_fixed : (gated && splits > 1)) continue;
    const int per_wave = (kblocks + splits * SK_WAVES - 1) / (splits * SK_WAVES);
    const double cut = 1.0 + 0.15 * log2(static_cast<double>(splits));
    // x from memory: no more ranges than the shape alone asks for, none shorter than four k-blocks a wave
    if (splits_fixed > 0 || splits == 1 || (splits <= by_shape && per_wave >= 4))
      for (int rt = 1; rt <= (M > 8 ? 4 : 3); ++rt)
        offer((1.0 + 0.4 * (M / 16.0) / rt) * cut / fill(static_cast<long>((tiles + rt - 1) / rt) * splits), 0, rt, splits);
    // x through LDS: whole chunks of four k-blocks a wave, ranges of at least 1024 of K
    if (M > 16 && K % 32 == 0 && N % 16 == 0 && per_wave % 4 == 0 && (splits == 1 || K / splits >= 1024)) {
      const int x_tiles = M <= 32 ? 2 : 4;
      for (int per : {3, 6, 8})
        offer(0.95 * (1.0 + 0.2 * x_tiles / per) * cut / fill(static_cast<long>((tiles + per - 1) / per) * splits), 1, per,
              splits);
    }
  }
  return best;
}

// The plan for callers (17 to 64 rows over a packed weight): *shares_x, *tiles as in FewRowsPlan; returns the ranges
// of K (1 for a gated product).
extern "C" int tie_skinny_few_rows_plan(int M, int N, int K, int gated, int* shares_x, int* tiles) {
  if (M <= 16 || M > 64) {
    if (shares_x != nullptr) *shares_x = 0;
    if (tiles != nullptr) *tiles = 0;
    return gated ? 1 : tie_skinny_gemm_splits(N, K);
  }
  const FewRowsPlan plan = few_rows_plan(M, N, K, gated, 0);
  if (shares_x != nullptr) *shares_x = plan.shares_x;
  if (tiles != nullptr) *tiles = plan.tiles;
  return plan.splits;
}

// Ranges of K that a product over w[N, K] is cut into when its caller takes partial sums: weights with
// few rows would otherwise give too few workgroups to keep enough bytes in flight. The smallest power of
// two that makes about four workgroups a compute unit (1024), as long as a wave keeps four k-blocks and
// at most 8; measured on the projections of the 1.7B, 8B and 32B shapes. By the shape of w alone.
extern "C" int tie_skinny_gemm_splits(int N, int K) {
  const int tiles = (N + 15) / 16;
  int splits = 1;
  while (splits < 8 && tiles * splits < 1024 && K / (32 * SK_WAVES * splits * 2) >= 4) splits *= 2;
  return splits;
}

// A product that ends a sub-layer (launch_skinny with SkNorm::next_x) is not cut along K, so a narrow output
// leaves it few workgroups: wider workgroups then keep as many bytes in flight as the planes of a cut product
// would. Sixteen waves over one tile where the tiles leave every compute unit at most one workgroup; eight
// waves over two tiles where pairs of tiles do; else the ordinary four waves. Measured in chains of a layer's
// four products against the same chain with planes and norm kernels (us a layer, planes | this way):
//   4096 wide (256 tiles): 1 row 73.6 | 67.9, 8 rows 79.2 | 73.9, 10 rows 79.3 | 74.0, 12 rows 79.6 | 76.8,
//     14 rows 80.0 | 76.9, 16 rows 80.5 | 80.4 (x comes in groups of four rows);
//   2048 wide (128 tiles): 8 rows 34.6 | 33.3, 10 rows 35.7 | 34.1, 12 rows 35.9 | 35.8, 16 rows 36.9 | 38.0;
//   2560 wide (160 tiles): 8 rows 53.5 | 53.1, 10 rows 55.4 | 55.2, 12 rows 55.7 | 57.0, 16 rows 58.0 | 62.0;
//   5120 wide (320 tiles), K of 8192 and 25600: 1 row 166.7 | 159.4, 4 rows 161.9 | 163.8, 8 rows 174.4 | 178.6;
//   5120 wide, K of 5120 and 17408: 1 row 123.3 | 113.2, 4 rows 119.6 | 117.7, 8 rows 127.8 | 128.9.
// (One tile and sixteen waves over 320 tiles: 193 us at 8 rows; every workgroup reads all of x.)
struct ProducerShape { int rt, u, waves; };
static ProducerShape producer_shape(int N) {
  const int tiles = (N + 15) / 16, cus = compute_units();
  if (tiles <= cus) return {1, 4, 16};
  if (tiles <= 2 * cus) return {2, 4, 8};
  return {0, 0, SK_WAVES};
}

// The most rows for which a product over w[N, K] that ends a sub-layer is worth running with the next norm's
// work in its epilogue instead of as planes that a norm kernel adds (the figures above); 0: never.
extern "C" int tie_skinny_norm_epilogue_rows(int N, int K) {
  if (N % 16 != 0 || K % 32 != 0) return 0;
  const int tiles = N / 16, cus = compute_units();
  if (tiles <= cus) return tiles * 4 > cus * 3 ? 14 : 10;
  if (tiles <= 2 * cus) return 4;
  return 0;
}

// gated: w holds blocks of 16 rows = 8 gate rows then 8 up rows of the same 8 outputs; out has N / 2 columns
// and receives silu(gate) * up.
// splits > 1: out is float32 [splits, M, N], plane s holding the sums over the s-th range of K.
// packed: w is in the blocked layout described at the top (N % 16 == 0 and K % 32 == 0).
static int launch_skinny(const void* x, const void* w, void* out, int out_dtype, int accumulate, int gated, int M,
                         int N, int K, int splits, int packed, int rt, int u, int waves, const SkNorm& norm,
                         hipStream_t stream) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || K % 8 != 0 || splits < 1 || splits > 64) return TIE_BAD_ARGUMENT;
  const bool norm_work = norm.scale_squares != nullptr || norm.next_x != nullptr;
  if (norm_work && M > SK_NORM_ROWS) return TIE_BAD_ARGUMENT;
  if (norm.scale_squares != nullptr && (norm.scale_tiles <= 0 || !(norm.scale_n > 0.f))) return TIE_BAD_ARGUMENT;
  // the tiles' sums of the rows to be scaled wait in LDS, 64 tiles (256 bytes) a load instruction
  const size_t scale_lds = norm.scale_squares == nullptr ? 0 : static_cast<size_t>(M) * ((norm.scale_tiles + 63) / 64) * 256;
  if (scale_lds > SK_SCALE_LDS_MAX) return TIE_BAD_ARGUMENT;
  if (norm.next_x != nullptr && (norm.next_w == nullptr || norm.squares == nullptr || splits != 1 || gated ||
                                 !accumulate || out_dtype != TIE_F32 || N % 16 != 0))
    return TIE_BAD_ARGUMENT;
  if (packed && (N % 16 != 0 || K % 32 != 0)) return TIE_BAD_ARGUMENT;
  if (gated && (accumulate || N % 16 != 0 || splits != 1)) return TIE_BAD_ARGUMENT;
  if (splits > 1 && (accumulate || out_dtype != TIE_F32)) return TIE_BAD_ARGUMENT;
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int forced_rt = rt;
  const bool rows_kernel = u >= 0;          // u < 0: the kernel that reads x from memory, whatever M (tests compare the two)
  const bool rows_forced = u == 1;          // u = 1: the kernel that shares x through LDS, whatever the shape
  if (u < 0) u = u == -1 ? 0 : -u;
  if (u == 1) u = 0;
  const int kblocks = (K + 31) / 32;
  // A product that ends a sub-layer is not cut along K, so a narrow output leaves it one workgroup a compute
  // unit: more waves a workgroup then keep as many bytes in flight as the planes of a cut product would.
  const bool many_waves_fit = norm.next_x != nullptr && packed && rt <= 2 && u >= 0;
  if (waves == 0) {
    waves = SK_WAVES;
    if (many_waves_fit && rt == 0 && u == 0) {
      const ProducerShape by_rule = producer_shape(N);
      rt = by_rule.rt;
      u = by_rule.u;
      waves = by_rule.waves;
    }
  }
  if (waves != SK_WAVES && !(many_waves_fit && (waves == 8 || waves == 16))) return TIE_BAD_ARGUMENT;
  const int per_wave = (kblocks + splits * waves - 1) / (splits * waves);
  // x through LDS (17 to 64 rows over packed weights, x within 32-bit byte offsets). With u = 1, rt is the
  // number of tiles a workgroup takes: up to 3 three waves x one tile, up to 6 three waves x two, else four x two.
  const int tiles = (N + 15) / 16;
  const bool rows_fit = static_cast<size_t>(M) * K * 2 < (1ull << 31);
  const bool whole_chunks = per_wave % 4 == 0;     // the parts of K in which the sums are formed end between chunks
  const bool rows_take = !norm_work && packed && mt > 1 && rows_fit && whole_chunks && K % 32 == 0;
  // 17 to 64 rows, nothing forced: the plan says which kernel and how many tiles a workgroup, for these ranges of K
  FewRowsPlan plan = {0, 0, splits};
  if (mt > 1 && packed && forced_rt == 0 && u == 0 && rows_kernel && !rows_forced && waves == SK_WAVES)
    plan = few_rows_plan(M, N, K, gated, splits);
  const int by_rule = plan.shares_x ? plan.tiles : 0;
  if (rows_take && rows_kernel && (by_rule != 0 || rows_forced)) {
    const int asked = rows_forced && forced_rt != 0 ? forced_rt : (by_rule != 0 ? by_rule : 6);
    const int per_wg = asked <= 3 ? 3 : (asked <= 6 ? 6 : 8);
    const dim3 rgrid((tiles + per_wg - 1) / per_wg, splits);
#define LAUNCH_ROWS(MT, RT, WAVES, U, DEPTH, TO)                                                                \
  skinny_rows_kernel<MT, RT, WAVES, U, DEPTH, TO><<<rgrid, WAVES * TIE_WAVE, 0, stream>>>(                      \
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<TO*>(out), M, N, K, accumulate, \
      gated, per_wave)
#define LAUNCH_ROWS_TO(MT, RT, WAVES, U, DEPTH)                                 \
  if (out_dtype == TIE_F32) LAUNCH_ROWS(MT, RT, WAVES, U, DEPTH, float);       \
  else if (out_dtype == TIE_BF16) LAUNCH_ROWS(MT, RT, WAVES, U, DEPTH, bf16_t); \
  else return TIE_BAD_ARGUMENT
#define LAUNCH_ROWS_MT(MT)                                  \
  if (per_wg == 8) { LAUNCH_ROWS_TO(MT, 2, 4, 4, 3); }      \
  else if (per_wg == 6) { LAUNCH_ROWS_TO(MT, 2, 3, 4, 3); } \
  else { LAUNCH_ROWS_TO(MT, 1, 3, 4, 3); }
    if (mt == 2) { LAUNCH_ROWS_MT(2) } else { LAUNCH_ROWS_MT(4) }
#undef LAUNCH_ROWS_MT
#undef LAUNCH_ROWS_TO
#undef LAUNCH_ROWS
    return tie_launch_status();
  }
  if (waves != SK_WAVES) {
    if (rt == 0) rt = 1;
    const dim3 wgrid(((N + 15) / 16 + rt - 1) / rt, 1);
    if (u == 0) u = waves == 8 ? 8 / rt : 4;
#define LAUNCH_W(RT, U, W)                                                                                      \
  skinny_gemm_kernel<1, RT, U, float, true, W><<<wgrid, W * TIE_WAVE, scale_lds, stream>>>(                     \
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<float*>(out), M, N, K, accumulate, \
      gated, per_wave, norm)
    if (rt == 1 && waves == 8 && u == 8) LAUNCH_W(1, 8, 8);
    else if (rt == 1 && waves == 8 && u == 4) LAUNCH_W(1, 4, 8);
    else if (rt == 1 && waves == 16 && u == 4) LAUNCH_W(1, 4, 16);
    else if (rt == 1 && waves == 16 && u == 2) LAUNCH_W(1, 2, 16);
    else if (rt == 2 && waves == 8 && u == 4) LAUNCH_W(2, 4, 8);
    else if (rt == 2 && waves == 8 && u == 2) LAUNCH_W(2, 2, 8);
    else if (rt == 2 && waves == 16 && u == 4) LAUNCH_W(2, 4, 16);
    else if (rt == 2 && waves == 16 && u == 2) LAUNCH_W(2, 2, 16);
    else return TIE_BAD_ARGUMENT;
#undef LAUNCH_W
    return tie_launch_status();
  }
  if (rows_forced) rt = 0;                  // asked for the other kernel, which does not take this shape: by the rule
  if (rt == 0) rt = (plan.tiles != 0 && !plan.shares_x) ? plan.tiles : choose_rt(M, N, splits);
  if (rt < 1 || rt > 4) return TIE_BAD_ARGUMENT;
  const dim3 grid(((N + 15) / 16 + rt - 1) / rt, splits);
  if (u == 0) {
    // k-blocks a batch of loads (two batches are in flight): 8, 4 or 2 by the registers the tiles leave, and the
    // largest of these that divides a wave's share of K: what is left over a batch is loaded block by block,
    // nothing in flight beside it (a share of 6 k-blocks in batches of 8: 14.3 us where batches of 2 take 10.7).
    // If none divides it, the largest that leaves at least two batches.
    const int most = rt == 1 ? 8 : (rt == 2 ? 4 : 2);
    for (u = most; u > 2 && per_wave % u != 0; u /= 2) {}
    if (per_wave % u != 0)
      for (u = most; u > 2 && 2 * u > per_wave; u /= 2) {}
  }
  if (u != 2 && u != 4 && u != 8) return TIE_BAD_ARGUMENT;
#define LAUNCH_P(MT, RT, U, TO, P)                                                                           \
  skinny_gemm_kernel<MT, RT, U, TO, P><<<grid, SK_WAVES * TIE_WAVE, scale_lds, stream>>>(                     \
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<TO*>(out), M, N, K, accumulate, \
      gated, per_wave, norm)
#define LAUNCH(MT, RT, U, TO)                  \
  {                                            \
    if (packed) LAUNCH_P(MT, RT, U, TO, true); \
    else LAUNCH_P(MT, RT, U, TO, false);       \
  }
#define LAUNCH_U(MT, RT, TO)                               \
  if (u == 2) LAUNCH(MT, RT, 2, TO)                        \
  else if (u == 4) LAUNCH(MT, RT, 4, TO)                   \
  else LAUNCH(MT, RT, 8, TO)
#define LAUNCH_RT(MT, TO)                                  \
  if (rt == 1) { LAUNCH_U(MT, 1, TO) }                     \
  else if (rt == 2) { LAUNCH_U(MT, 2, TO) }                \
  else if (rt == 3) { LAUNCH_U(MT, 3, TO) }                \
  else { LAUNCH_U(MT, 4, TO) }
#define LAUNCH_MT(TO)                                      \
  if (mt == 1) { LAUNCH_RT(1, TO); }                       \
  else if (mt == 2) { LAUNCH_RT(2, TO); }                  \
  else { LAUNCH_RT(4, TO); }
  if (out_dtype == TIE_F32) { LAUNCH_MT(float) }
  else if (out_dtype == TIE_BF16) { LAUNCH_MT(bf16_t) }
  else return TIE_BAD_ARGUMENT;
#undef LAUNCH_MT
#undef LAUNCH_RT
#undef LAUNCH_U
#undef LAUNCH
#undef LAUNCH_P
  return tie_launch_status();
}

extern "C" int tie_skinny_gemm_bf16_with(const void* x, const void* w, void* out, int out_dtype, int accumulate,
                                         int gated, int M, int N, int K, int splits, int packed, int rt, int u,
                                         hipStream_t stream) {
  return launch_skinny(x, w, out, out_dtype, accumulate, gated, M, N, K, splits, packed, rt, u, SK_WAVES, SkNorm{}, stream);
}

extern "C" int tie_skinny_gemm_bf16(const void* x, const void* w, void* out, int out_dtype, int accumulate, int gated,
                                    int M, int N, int K, int splits, int packed, hipStream_t stream) {
  return tie_skinny_gemm_bf16_with(x, w, out, out_dtype, accumulate, gated, M, N, K, splits, packed, 0, 0, stream);
}

// The product with the norms' work in its epilogue (up to 16 rows; see SkNorm and the top of this file).
// scale_squares (or null): [M][scale_tiles] sums of squares of the rows x was made from; the sums are multiplied by
// 1 / sqrt(their total / scale_n + scale_eps). next_x (or null; then accumulate, one plane, float32 out, N % 16 == 0):
// out += sums in place, next_x = bf16(out * next_w), squares[M][N / 16] = sums of out^2 per 16-column tile.
// rt, u, waves: 0 = by the rule (measurements name tiles a workgroup, k-blocks a batch of loads and waves a
// workgroup themselves).
extern "C" int tie_skinny_gemm_bf16_norm(const void* x, const void* w, void* out, int out_dtype, int accumulate,
                                         int gated, int M, int N, int K, int splits, int packed,
                                         const float* scale_squares, int scale_tiles, float scale_n, float scale_eps,
                                         const float* next_w, void* next_x, float* squares, int rt, int u, int waves,
                                         hipStream_t stream) {
  const SkNorm norm = {scale_squares, scale_tiles, scale_n, scale_eps, next_w, static_cast<bf16_t*>(next_x), squares};
  return launch_skinny(x, w, out, out_dtype, accumulate, gated, M, N, K, splits, packed, rt, u, waves, norm, stream);
}
