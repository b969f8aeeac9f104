// The prefill-time matrix product for gfx950: out[M, N] (+)= x[M, K] . w[N, K]^T with bfloat16
// operands and float32 accumulation on v_mfma_f32_32x32x16_bf16.
//
// Both operands are K-contiguous, which is the order the matrix cores consume: a lane's fragment
// is 8 consecutive k of one row (16 bytes). A workgroup of four waves owns a BM x BN tile of the
// output; k advances in slices of 64. Each slice of x and w goes global memory -> registers ->
// LDS (rows padded by 16 bytes so that the 32 rows a fragment read touches fall into different
// banks), with two LDS buffers: while the matrix cores work on one slice, the loads of the next
// are in flight and are written to the other buffer, one barrier per slice. Each wave computes a
// WM x WN sub-tile as (WM/32) x (WN/32) MFMA tiles, reading A fragments (rows of x) and B
// fragments (rows of w) from LDS.
//
// Ragged edges are masked: rows beyond M or N and k beyond K are read as zeros and never stored,
// so any M, N >= 1 and any K with K % 8 == 0 are taken. The accumulation order over k is fixed by
// the tile shape alone, so a row's result does not depend on the other rows of the call.
//
// Workgroups are numbered so that each of the 8 XCDs (which have an L2 each) works on a
// contiguous band of the output and walks it column-tile by column-tile: the weights of a column
// tile are fetched into that L2 once and reused by the row tiles.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define GB_BK 64
#define GB_PAD 8                      // bf16 elements: 16 bytes per staged row
#define GB_STRIDE (GB_BK + GB_PAD)    // elements per staged row
#define GB_THREADS 256
#define GB_XCDS 8

__device__ __forceinline__ bf16x8_t frag_of(uint4 v) { return *reinterpret_cast<const bf16x8_t*>(&v); }

// Loads the 16-byte chunks of a (ROWS x 64) slice that this thread stages: chunk c of row r for
// (r, c) = (t / 8 + 32 i, t % 8). Rows >= limit and k >= K give zeros.
template <int ROWS>
__device__ __forceinline__ void load_slice(const bf16_t* __restrict__ base, int row0, int limit, int K, int k0,
                                           uint4 (&regs)[ROWS / 32]) {
  const int c = threadIdx.x & 7;
  const int r = threadIdx.x >> 3;
  const int k = k0 + c * 8;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    const int row = row0 + r + 32 * i;
    regs[i] = (row < limit && k < K) ? *reinterpret_cast<const uint4*>(base + static_cast<size_t>(row) * K + k)
                                     : make_uint4(0, 0, 0, 0);
  }
}

template <int ROWS>
__device__ __forceinline__ void store_slice(bf16_t* lds, const uint4 (&regs)[ROWS / 32]) {
  const int c = threadIdx.x & 7;
  const int r = threadIdx.x >> 3;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i)
    *reinterpret_cast<uint4*>(lds + (r + 32 * i) * GB_STRIDE + c * 8) = regs[i];
}

// EPI: 0 = store float32, 1 = store bfloat16, 2 = add to float32 output
template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(GB_THREADS) void gemm_bf16_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w, void* __restrict__ outp,
                                                               int M, int N, int K, int tiles_m, int tiles_n) {
  static_assert(WAVES_M * WAVES_N == 4, "four waves a workgroup");
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // sub-tile of one wave
  constexpr int TM = WM / 32, TN = WN / 32;             // MFMA tiles of one wave
  extern __shared__ bf16_t lds[];                       // [2][(BM + BN) * GB_STRIDE]
  constexpr int BUF = (BM + BN) * GB_STRIDE;

  // XCD-aware numbering: hardware deals consecutive workgroups round-robin to the XCDs.
  const int total = tiles_m * tiles_n;
  int id = blockIdx.x;
  {
    const int per_xcd = (total + GB_XCDS - 1) / GB_XCDS;
    const int remapped = (id % GB_XCDS) * per_xcd + id / GB_XCDS;
    // The last XCDs may have one workgroup fewer; fall back to the plain id where the remap would leave the grid.
    id = (total % GB_XCDS == 0) ? remapped : id;
  }
  const int tile_n = id / tiles_m;
  const int tile_m = id % tiles_m;
  const int row0 = tile_m * BM;
  const int col0 = tile_n * BN;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int fr = lane & 31;    // row of a fragment
  const int fk = lane >> 5;    // which 8 of the 16 k of an MFMA step

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[BM / 32], rb[BN / 32];
  const int k_tiles = (K + GB_BK - 1) / GB_BK;
  load_slice<BM>(x, row0, M, K, 0, ra);
  load_slice<BN>(w, col0, N, K, 0, rb);
  store_slice<BM>(lds, ra);
  store_slice<BN>(lds + BM * GB_STRIDE, rb);
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    const bf16_t* cur = lds + (kt & 1) * BUF;
    bf16_t* nxt = lds + ((kt + 1) & 1) * BUF;
    const bool more = kt + 1 < k_tiles;
    if (more) {
      load_slice<BM>(x, row0, M, K, (kt + 1) * GB_BK, ra);
      load_slice<BN>(w, col0, N, K, (kt + 1) * GB_BK, rb);
    }
    const bf16_t* a_base = cur + (wm * WM + fr) * GB_STRIDE + fk * 8;
    const bf16_t* b_base = cur + (BM + wn * WN + fr) * GB_STRIDE + fk * 8;
#pragma unroll
    for (int ks = 0; ks < GB_BK / 16; ++ks) {
      bf16x8_t af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = frag_of(*reinterpret_cast<const uint4*>(a_base + i * 32 * GB_STRIDE + ks * 16));
#pragma unroll
      for (int j = 0; j < TN; ++j) bfr[j] = frag_of(*reinterpret_cast<const uint4*>(b_base + j * 32 * GB_STRIDE + ks * 16));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      store_slice<BM>(nxt, ra);
      store_slice<BN>(nxt + BM * GB_STRIDE, rb);
    }
    __syncthreads();
  }

  // D layout of a 32x32 tile: lane holds column lane % 32 and rows 8 * (v / 4) + (lane / 32) * 4 + v % 4.
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = col0 + wn * WN + j * 32 + fr;
      if (n >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = row0 + wm * WM + i * 32 + 8 * (v / 4) + fk * 4 + (v % 4);
        if (m >= M) continue;
        const size_t o = static_cast<size_t>(m) * N + n;
        if (EPI == 0) static_cast<float*>(outp)[o] = acc[i][j][v];
        else if (EPI == 1) static_cast<bf16_t*>(outp)[o] = float_to_bf16(acc[i][j][v]);
        else static_cast<float*>(outp)[o] += acc[i][j][v];
      }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_gemm(const void* x, const void* w, void* out, int epi, int M, int N, int K, hipStream_t stream) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t shared = sizeof(bf16_t) * 2 * (BM + BN) * GB_STRIDE;
  const dim3 grid(tiles_m * tiles_n);
  // The two staging buffers exceed the 64 KB a kernel may use without asking; gfx950 has 160 KB a CU.
#define LAUNCH(EPI)                                                                                          \
  {                                                                                                          \
    static bool raised = false;                                                                              \
    if (!raised) {                                                                                           \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, EPI>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared)); \
      if (e != hipSuccess) return static_cast<int>(e);                                                       \
      raised = true;                                                                                         \
    }                                                                                                        \
    gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, EPI><<<grid, GB_THREADS, shared, stream>>>(                    \
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), out, M, N, K, tiles_m, tiles_n);       \
  }
  if (epi == 0) LAUNCH(0) else if (epi == 1) LAUNCH(1) else LAUNCH(2)
#undef LAUNCH
  return tie_launch_status();
}

// out_dtype: TIE_F32 or TIE_BF16; accumulate adds into a float32 output. tile: 0 = choose, 1 = 128x128, 2 = 256x128.
extern "C" int tie_gemm_bf16(const void* x, const void* w, void* out, int out_dtype, int accumulate, int M, int N,
                             int K, int tile, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0) return TIE_BAD_ARGUMENT;
  if (accumulate && out_dtype != TIE_F32) return TIE_BAD_ARGUMENT;
  if (out_dtype != TIE_F32 && out_dtype != TIE_BF16) return TIE_BAD_ARGUMENT;
  const int epi = accumulate ? 2 : (out_dtype == TIE_F32 ? 0 : 1);
  if (tile == 0) {
    // The larger tile halves the LDS traffic per flop; take it once it still yields enough workgroups.
    const long big = static_cast<long>((M + 255) / 256) * ((N + 127) / 128);
    tile = big >= 512 ? 2 : 1;
  }
  if (tile == 2) return launch_gemm<256, 128, 2, 2>(x, w, out, epi, M, N, K, stream);
  return launch_gemm<128, 128, 2, 2>(x, w, out, epi, M, N, K, stream);
}
