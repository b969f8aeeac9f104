// The prefill-time matrix product for gfx950: out[M, N] (+)= x[M, K] . w[N, K]^T with bfloat16
// operands and float32 accumulation on v_mfma_f32_32x32x16_bf16.
//
// Both operands are K-contiguous, which is the order the matrix cores consume: a lane's fragment
// is 8 consecutive k of one row (16 bytes). A workgroup of four or eight waves owns a BM x BN tile of
// the output; k advances in slices of BK (32 or 64). Each slice of x and w goes global memory -> registers ->
// LDS (rows padded by 16 bytes so that the 32 rows a fragment read touches fall into different
// banks), with two LDS buffers and two register sets: while the matrix cores work on slice t, slice
// t + 1 is written to the other buffer and the loads of slice t + 2 are in flight, one barrier per slice. Each wave computes a
// WM x WN sub-tile as (WM/32) x (WN/32) MFMA tiles, reading A fragments (rows of x) and B
// fragments (rows of w) from LDS.
//
// Ragged edges are masked: rows beyond M or N and k beyond K are read as zeros and never stored,
// so any M, N >= 1 and any K with K % 8 == 0 are taken. The accumulation order over k is fixed by
// the tile shape alone, so a row's result does not depend on the other rows of the call.
//
// Every workgroup re-reads its operand tiles from the L2, so the 256 x 256 tile (half the bytes per
// flop of 128 x 128) is used wherever it still fills the GPU, and 256 x 128 where only that does.
//
// Workgroups are numbered so that each of the 8 XCDs (which have an L2 each) works on a
// contiguous band of the output and walks it column-tile by column-tile: the weights of a column
// tile are fetched into that L2 once and reused by the row tiles.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define GB_PAD 8                      // bf16 elements: 16 bytes per staged row
#define GB_XCDS 8

__device__ __forceinline__ bf16x8_t frag_of(uint4 v) { return *reinterpret_cast<const bf16x8_t*>(&v); }

// Loads the 16-byte chunks of a (ROWS x BK) slice that this thread stages: chunk c of row r for
// (r, c) = (t / CPR + RPP i, t % CPR) with CPR = BK / 8 chunks a row and RPP = THREADS / CPR rows a
// pass; rows are ld elements apart. Rows >= limit and k >= K give zeros. With FULL the slice lies wholly below K and rows beyond
// the limit are clamped to the last one instead (their products land in outputs that are never
// stored): the loads then sit in straight-line code, which lets the compiler count the loads in
// flight exactly instead of waiting for all of them wherever branches meet.
template <int ROWS, int BK, int THREADS, bool FULL>
__device__ __forceinline__ void load_slice(const bf16_t* __restrict__ base, int row0, int limit, int ld, int K, int k0,
                                           uint4 (&regs)[ROWS * (BK / 8) / THREADS]) {
  constexpr int CPR = BK / 8, RPP = THREADS / CPR;
  const int c = threadIdx.x % CPR;
  const int r = threadIdx.x / CPR;
  const int k = k0 + c * 8;
#pragma unroll
  for (int i = 0; i < ROWS / RPP; ++i) {
    const int row = row0 + r + RPP * i;
    if (FULL)
      regs[i] = *reinterpret_cast<const uint4*>(base + static_cast<size_t>(min(row, limit - 1)) * ld + k);
    else
      regs[i] = (row < limit && k < K) ? *reinterpret_cast<const uint4*>(base + static_cast<size_t>(row) * ld + k)
                                       : make_uint4(0, 0, 0, 0);
  }
}

template <int ROWS, int BK, int THREADS>
__device__ __forceinline__ void store_slice(bf16_t* lds, const uint4 (&regs)[ROWS * (BK / 8) / THREADS]) {
  constexpr int CPR = BK / 8, RPP = THREADS / CPR, STRIDE = BK + GB_PAD;
  const int c = threadIdx.x % CPR;
  const int r = threadIdx.x / CPR;
#pragma unroll
  for (int i = 0; i < ROWS / RPP; ++i)
    *reinterpret_cast<uint4*>(lds + (r + RPP * i) * STRIDE + c * 8) = regs[i];
}

// EPI: 0 = store float32, 1 = store bfloat16, 2 = add to float32 output,
//      3 = gated: columns come in blocks of 16 = 8 gate columns then 8 up columns of the same 8 outputs;
//          out[m, block * 8 + j] = silu(gate_j) * up_j as bfloat16, out has N / 2 columns
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_bf16_kernel(const bf16_t* __restrict__ x_all,
                                                                          const bf16_t* __restrict__ w_all,
                                                                          void* __restrict__ out_all, int M, int N,
                                                                          int K_all, int tiles_m, int tiles_n,
                                                                          int slices_per_split) {
  // blockIdx.y = which range of K this workgroup sums (one range: the whole of K); its result goes to
  // plane blockIdx.y of the output. From here on x, w, K are that range's.
  const int ld = K_all;
  const int k_base = blockIdx.y * slices_per_split * BK;
  const bf16_t* __restrict__ x = x_all + k_base;
  const bf16_t* __restrict__ w = w_all + k_base;
  const int K = min(K_all - k_base, slices_per_split * BK);
  void* __restrict__ outp = gridDim.y > 1 ? static_cast<void*>(static_cast<float*>(out_all) +
                                                                static_cast<size_t>(blockIdx.y) * M * N)
                                          : out_all;
  constexpr int THREADS = WAVES_M * WAVES_N * 64;
  constexpr int GB_STRIDE = BK + GB_PAD;                // elements per staged row
  constexpr int GB_BK = BK;
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

  // Two register sets: while slice kt is multiplied, slice kt + 1 waits in one set to be written to
  // LDS and the loads of slice kt + 2 are in flight into the other.
  uint4 ra[2][BM * (BK / 8) / THREADS], rb[2][BN * (BK / 8) / THREADS];
  const int k_tiles = (K + GB_BK - 1) / GB_BK;
  const int k_full = K / GB_BK;   // slices that lie wholly below K
  load_slice<BM, BK, THREADS, false>(x, row0, M, ld, K, 0, ra[0]);
  load_slice<BN, BK, THREADS, false>(w, col0, N, ld, K, 0, rb[0]);
  store_slice<BM, BK, THREADS>(lds, ra[0]);
  store_slice<BN, BK, THREADS>(lds + BM * GB_STRIDE, rb[0]);
  __syncthreads();
  // Slice 1 is in flight when the loop is entered, as it is whenever the loop comes round.
  if (k_full > 1) {
    load_slice<BM, BK, THREADS, true>(x, row0, M, ld, K, GB_BK, ra[1]);
    load_slice<BN, BK, THREADS, true>(w, col0, N, ld, K, GB_BK, rb[1]);
  } else if (k_tiles > 1) {
    load_slice<BM, BK, THREADS, false>(x, row0, M, ld, K, GB_BK, ra[1]);
    load_slice<BN, BK, THREADS, false>(w, col0, N, ld, K, GB_BK, rb[1]);
  }

  // Fragments of k step s + 1 are read from LDS before the MFMAs of step s are issued, so the
  // matrix cores do not idle through the LDS latency.
  auto compute = [&](const bf16_t* cur) {
    const bf16_t* a_base = cur + (wm * WM + fr) * GB_STRIDE + fk * 8;
    const bf16_t* b_base = cur + (BM + wn * WN + fr) * GB_STRIDE + fk * 8;
    constexpr int STEPS = GB_BK / 16;
    uint4 af[2][TM], bfr[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) af[0][i] = *reinterpret_cast<const uint4*>(a_base + i * 32 * GB_STRIDE);
#pragma unroll
    for (int j = 0; j < TN; ++j) bfr[0][j] = *reinterpret_cast<const uint4*>(b_base + j * 32 * GB_STRIDE);
#pragma unroll
    for (int ks = 0; ks < STEPS; ++ks) {
      const int cur_set = ks & 1, nxt_set = cur_set ^ 1;
      if (ks + 1 < STEPS) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          af[nxt_set][i] = *reinterpret_cast<const uint4*>(a_base + i * 32 * GB_STRIDE + (ks + 1) * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          bfr[nxt_set][j] = *reinterpret_cast<const uint4*>(b_base + j * 32 * GB_STRIDE + (ks + 1) * 16);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_of(af[cur_set][i]), frag_of(bfr[cur_set][j]),
                                                              acc[i][j], 0, 0, 0);
    }
  };

  // Unrolled by two so that the register sets are addressed statically. The steady state runs while
  // the two slices it fetches lie wholly below K: its body has no branches, so the compiler knows
  // how many loads are in flight at every point and lets slice kt + 2 stay in flight while slice
  // kt + 1 is written to LDS. The last slices go through the general code below.
  int kt = 0;
  auto steady_pair = [&](int k) {
    load_slice<BM, BK, THREADS, true>(x, row0, M, ld, K, (k + 2) * GB_BK, ra[0]);
    load_slice<BN, BK, THREADS, true>(w, col0, N, ld, K, (k + 2) * GB_BK, rb[0]);
    compute(lds);
    store_slice<BM, BK, THREADS>(lds + BUF, ra[1]);
    store_slice<BN, BK, THREADS>(lds + BUF + BM * GB_STRIDE, rb[1]);
    __syncthreads();
    load_slice<BM, BK, THREADS, true>(x, row0, M, ld, K, (k + 3) * GB_BK, ra[1]);
    load_slice<BN, BK, THREADS, true>(w, col0, N, ld, K, (k + 3) * GB_BK, rb[1]);
    compute(lds + BUF);
    store_slice<BM, BK, THREADS>(lds, ra[0]);
    store_slice<BN, BK, THREADS>(lds + BM * GB_STRIDE, rb[0]);
    __syncthreads();
  };
  // The compiler counts loads in flight exactly only within straight-line code: where the loop comes
  // round it waits for all of them. Four pairs a round keep that to one slice in eight.
  for (; kt + 9 < k_full; kt += 8) {
    steady_pair(kt);
    steady_pair(kt + 2);
    steady_pair(kt + 4);
    steady_pair(kt + 6);
  }
  for (; kt + 3 < k_full; kt += 2) steady_pair(kt);
  for (; kt < k_tiles; kt += 2) {
    {  // even slice: in LDS buffer 0; slice kt + 1 sits in set 1; fetch kt + 2 into set 0
      if (kt + 2 < k_tiles) {
        load_slice<BM, BK, THREADS, false>(x, row0, M, ld, K, (kt + 2) * GB_BK, ra[0]);
        load_slice<BN, BK, THREADS, false>(w, col0, N, ld, K, (kt + 2) * GB_BK, rb[0]);
      }
      compute(lds);
      if (kt + 1 < k_tiles) {
        store_slice<BM, BK, THREADS>(lds + BUF, ra[1]);
        store_slice<BN, BK, THREADS>(lds + BUF + BM * GB_STRIDE, rb[1]);
      }
      __syncthreads();
    }
    if (kt + 1 < k_tiles) {  // odd slice: in LDS buffer 1; slice kt + 2 sits in set 0; fetch kt + 3 into set 1
      if (kt + 3 < k_tiles) {
        load_slice<BM, BK, THREADS, false>(x, row0, M, ld, K, (kt + 3) * GB_BK, ra[1]);
        load_slice<BN, BK, THREADS, false>(w, col0, N, ld, K, (kt + 3) * GB_BK, rb[1]);
      }
      compute(lds + BUF);
      if (kt + 2 < k_tiles) {
        store_slice<BM, BK, THREADS>(lds, ra[0]);
        store_slice<BN, BK, THREADS>(lds + BM * GB_STRIDE, rb[0]);
      }
      __syncthreads();
    }
  }

  // D layout of a 32x32 tile: lane holds column lane % 32 and rows 8 * (v / 4) + (lane / 32) * 4 + v % 4.
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = col0 + wn * WN + j * 32 + fr;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = row0 + wm * WM + i * 32 + 8 * (v / 4) + fk * 4 + (v % 4);
        if (EPI == 3) {
          // The partner column (gate <-> up) sits 8 lanes away; every lane takes part in the exchange.
          const float mine = acc[i][j][v];
          const float other = __shfl_xor(mine, 8, 64);
          if ((fr & 8) == 0 && n < N && m < M) {
            const float g = mine, u = other;
            const int out_col = (n >> 4) * 8 + (n & 7);
            static_cast<bf16_t*>(outp)[static_cast<size_t>(m) * (N / 2) + out_col] =
                float_to_bf16(g / (1.0f + __expf(-g)) * u);
          }
          continue;
        }
        if (n >= N || m >= M) continue;
        const size_t o = static_cast<size_t>(m) * N + n;
        if (EPI == 0) static_cast<float*>(outp)[o] = acc[i][j][v];
        else if (EPI == 1) static_cast<bf16_t*>(outp)[o] = float_to_bf16(acc[i][j][v]);
        else static_cast<float*>(outp)[o] += acc[i][j][v];
      }
    }
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
static int launch_gemm(const void* x, const void* w, void* out, int epi, int M, int N, int K, int splits,
                       hipStream_t stream) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int k_slices = (K + BK - 1) / BK;
  const int per_split = (k_slices + splits - 1) / splits;
  if ((k_slices + per_split - 1) / per_split != splits) return TIE_BAD_ARGUMENT;   // a range would be empty
  const size_t shared = sizeof(bf16_t) * 2 * (BM + BN) * (BK + GB_PAD);
  const dim3 grid(tiles_m * tiles_n, splits);
  // The two staging buffers may exceed the 64 KB a kernel can use without asking; gfx950 has 160 KB a CU.
#define LAUNCH(EPI)                                                                                          \
  {                                                                                                          \
    static bool raised = false;                                                                              \
    if (!raised) {                                                                                           \
      hipError_t e = hipFuncSetAttribute(                                                                    \
          reinterpret_cast<const void*>(&gemm_bf16_kernel<BM, BN, BK, WAVES_M, WAVES_N, EPI>),               \
          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared));                             \
      if (e != hipSuccess) return static_cast<int>(e);                                                       \
      raised = true;                                                                                         \
    }                                                                                                        \
    gemm_bf16_kernel<BM, BN, BK, WAVES_M, WAVES_N, EPI><<<grid, WAVES_M * WAVES_N * 64, shared, stream>>>(    \
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), out, M, N, K, tiles_m, tiles_n,        \
        per_split);                                                                                          \
  }
  if (epi == 0) LAUNCH(0) else if (epi == 1) LAUNCH(1) else if (epi == 2) LAUNCH(2) else LAUNCH(3)
#undef LAUNCH
  return tie_launch_status();
}

// Ranges of K that a product of M rows over w[N, K] is best cut into when its caller adds planes of
// partial sums: few rows over a narrow weight give too few workgroups otherwise.
extern "C" int tie_gemm_bf16_splits(int M, int N, int K) {
  const long tiles = static_cast<long>((M + 127) / 128) * ((N + 127) / 128);
  if (tiles >= 256) return 1;
  const int k_slices = (K + 63) / 64;
  // 2, 4 or 8 ranges of at least 512 of K each, none of them empty.
  for (int splits = 8; splits >= 2; splits /= 2) {
    if (static_cast<long>(splits) * tiles > 256 && splits > 2) continue;   // more planes cost more than they fill
    if (splits > k_slices / 8) continue;
    const int per = (k_slices + splits - 1) / splits;
    if ((k_slices + per - 1) / per == splits) return splits;
  }
  return 1;
}

// out_dtype: TIE_F32 or TIE_BF16; accumulate adds into a float32 output; gated (bfloat16 output of N / 2
// columns, N % 16 == 0) applies silu(gate) * up to interleaved column blocks.
// splits > 1: out is float32 [splits, M, N], plane s holding the sums over the s-th range of K
// (128x128 tiles; neither accumulate nor gated).
// tile: 0 = choose, 1 = 128x128 (four waves of 64x64), 2 = 256x256 (eight waves of 128x64),
//       3 = 256x128 (eight waves of 64x64).
extern "C" int tie_gemm_bf16(const void* x, const void* w, void* out, int out_dtype, int accumulate, int gated, int M,
                             int N, int K, int tile, int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || splits < 1) return TIE_BAD_ARGUMENT;
  if (accumulate && out_dtype != TIE_F32) return TIE_BAD_ARGUMENT;
  if (out_dtype != TIE_F32 && out_dtype != TIE_BF16) return TIE_BAD_ARGUMENT;
  if (gated && (accumulate || out_dtype != TIE_BF16 || N % 16 != 0)) return TIE_BAD_ARGUMENT;
  if (splits > 1 && (accumulate || gated || out_dtype != TIE_F32)) return TIE_BAD_ARGUMENT;
  const int epi = gated ? 3 : (accumulate ? 2 : (out_dtype == TIE_F32 ? 0 : 1));
  if (splits > 1) tile = 1;
  if (tile == 0) {
    // Larger tiles need fewer operand bytes per flop; take the largest that still gives most CUs a tile.
    const long rows256 = (M + 255) / 256;
    if (rows256 * ((N + 255) / 256) >= 160) tile = 2;
    else if (rows256 * ((N + 127) / 128) >= 192) tile = 3;
    else tile = 1;
  }
  if (tile == 2) return launch_gemm<256, 256, 64, 2, 4>(x, w, out, epi, M, N, K, splits, stream);
  if (tile == 3) return launch_gemm<256, 128, 64, 4, 2>(x, w, out, epi, M, N, K, splits, stream);
  return launch_gemm<128, 128, 64, 2, 2>(x, w, out, epi, M, N, K, splits, stream);
}
