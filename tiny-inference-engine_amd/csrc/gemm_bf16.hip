// The prefill-time matrix product for gfx950: out[M, N] (+)= x[M, K] . w[N, K]^T with bfloat16
// operands and float32 accumulation on v_mfma_f32_32x32x16_bf16.
//
// Two kernels. The one described first stages operand slices through registers and takes every shape
// with K % 8 == 0; the second (further down, gemm_bf16_dma_kernel) loads them from global memory
// straight into LDS, needs K % 32 == 0 and N % 4 == 0, also reads weights in packed blocks, and is
// the one the prefill step runs on. gemm_plan picks between their tiles.
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
#include <type_traits>

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

// ---------------------------------------------------------------------------------------------
// The same product with operand slices going global memory -> LDS directly (buffer loads with the
// lds flag: no registers, no LDS write instructions), for K % 32 == 0 and N % 4 == 0.
//
// A workgroup of four waves (one per SIMD, 512 registers each) owns a 256 x BN tile, BN = 256 or 128; a wave owns
// 128 x BN/2 of it, so that every byte read from LDS feeds twice the flops it does with the 64-wide
// wave tiles above. k advances in slices of 32 through a ring of four LDS stages: while slice t is
// multiplied, slices t+1 and t+2 are landing or landed and the loads of t+2 (its w rows) and t+3 (its x rows) are
// issued, a few between the matrix instructions of each half slice so that neither the texture
// path nor the in-order instruction stream of the one wave backs up. One barrier a slice: it sits
// after the first half's matrix instructions, when the fragments of the second half are in
// registers already, so that the stage is free and the next slice's first fragments can be read
// while the second half multiplies.
//
// A staged row is 64 bytes, unpadded; 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 3), which
// spreads the 32 rows a fragment read touches over the banks. Rows beyond M or N are clamped to the
// last row (their products land in output rows or columns that are never stored). With PW the weight
// comes in packed blocks of 16 rows x 32 k (1 KB in the matrix cores' operand order, as the decode
// product reads it): one load instruction stages one block, and the 16 lanes that LDS serves in a
// cycle read 256 consecutive bytes of it.
//
// The matrix instructions take w's fragment as their first operand: the tile comes out transposed,
// a lane holding 4 consecutive columns of one output row, which it stores as one 8- or 16-byte piece.
typedef __attribute__((ext_vector_type(4))) float floatx4_t;
typedef __attribute__((address_space(3))) void lds_void_t;

#define GD_BK 32
#define GD_STAGES 4
// Fourth word of a raw buffer descriptor on gfx9-family GPUs: 32-bit float data format, destination
// selects x, y, z, w; no swizzle, no stride (the compiler's own default for raw buffers on this target).
#define GD_RSRC_FLAGS 0x27000

// BM: 256, 128 or 64 rows of x a workgroup; the waves are 2 x 2 in every case, a wave covering BM / 2 rows.
template <int BM, int BN, int EPI, bool PW>
__global__ __launch_bounds__(256) void gemm_bf16_dma_kernel(const bf16_t* __restrict__ x_all,
                                                            const bf16_t* __restrict__ w_all,
                                                            void* __restrict__ out_all, int M, int N, int K,
                                                            int tiles_m, int tiles_n, int slices_per_split) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = GD_BK;
  constexpr int TN = BN / 64;                   // 32-column MFMA tiles of a wave
  constexpr int TM = BM / 64;                   // 32-row MFMA tiles of a wave
  constexpr int PA = BM / 64;                   // wave instructions that stage x's rows (16 rows each, 4 waves)
  constexpr int PB = BN / 64;                   // wave instructions that stage w's rows likewise
  static_assert(BM == 256 || BM == 128 || BM == 64, "rows of a tile");
  constexpr int BUF = (BM + BN) * BK;           // elements of one stage
  extern __shared__ bf16_t lds[];

  const int total = tiles_m * tiles_n;
  int id = blockIdx.x;
  {
    const int per_xcd = (total + GB_XCDS - 1) / GB_XCDS;
    const int remapped = (id % GB_XCDS) * per_xcd + id / GB_XCDS;
    id = (total % GB_XCDS == 0) ? remapped : id;
  }
  const int tile_n = id / tiles_m;
  const int tile_m = id % tiles_m;
  const int row0 = tile_m * BM;
  const int col0 = tile_n * BN;
  const int k_begin = blockIdx.y * slices_per_split;                        // in slices
  const int k_tiles = min(slices_per_split, K / BK - k_begin);
  void* outp = EPI == 0 ? static_cast<void*>(static_cast<float*>(out_all) + static_cast<size_t>(blockIdx.y) * M * N)
                        : out_all;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int fr = lane & 31;
  const int fk = lane >> 5;

  // One wave instruction fills 16 rows of 64 bytes: pass p of wave v covers rows 64 p + 16 v + lane / 4.
  // Rows beyond the matrix are clamped to its last one (their products are never stored).
  const int lr = wave * 16 + (lane >> 2);
  const int lchunk = (lane & 3) ^ ((lr >> 1) & 3);
  const unsigned row_bytes = static_cast<unsigned>(K) * 2;
  const int kblocks = K / BK;
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(x_all + static_cast<size_t>(row0) * K + static_cast<size_t>(k_begin) * BK), 0,
      static_cast<int>(min(BM, M - row0) * row_bytes - k_begin * BK * 2), GD_RSRC_FLAGS);
  unsigned a_off[PA], b_off[PB];
#pragma unroll
  for (int p = 0; p < PA; ++p) a_off[p] = min(lr + p * 64, M - 1 - row0) * row_bytes + lchunk * 16;
  // w: rows like x's, or (PW) the packed layout, where the 16 rows x 32 k that one wave instruction
  // stages are one block of 1 KB: block (tile, k-block) at ((tile * kblocks) + k-block) * 1 KB.
  const int tile0 = col0 / 16, last_tile = (N - 1) / 16;
  const bf16_t* b_base = PW ? w_all + (static_cast<size_t>(tile0) * kblocks + k_begin) * 512
                            : w_all + static_cast<size_t>(col0) * K + static_cast<size_t>(k_begin) * BK;
  const unsigned b_bytes = PW ? static_cast<unsigned>(min(BN / 16, last_tile + 1 - tile0)) * kblocks * 1024 - k_begin * 1024
                              : min(BN, N - col0) * row_bytes - k_begin * BK * 2;
  const __amdgpu_buffer_rsrc_t b_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(b_base), 0, static_cast<int>(b_bytes), GD_RSRC_FLAGS);
  unsigned b_tile_off[PB];   // PW: wave-uniform byte offset of this wave's block row
#pragma unroll
  for (int p = 0; p < PB; ++p) {
    b_off[p] = PW ? lane * 16 : min(lr + p * 64, N - 1 - col0) * row_bytes + lchunk * 16;
    b_tile_off[p] = PW ? static_cast<unsigned>(min(p * 4 + wave, last_tile - tile0)) * kblocks * 1024 : 0;
  }

  auto stage = [&](int kt) { return lds + (kt & (GD_STAGES - 1)) * BUF; };
  auto issue_x = [&](int kt) {
    bf16_t* buf = stage(kt);
#pragma unroll
    for (int p = 0; p < PA; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_void_t*)(buf + (p * 64 + wave * 16) * BK), 16, a_off[p],
                                               kt * BK * 2, 0, 0);
  };
  auto issue_w = [&](int kt) {
    bf16_t* buf = stage(kt);
#pragma unroll
    for (int p = 0; p < PB; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_void_t*)(buf + (BM + p * 64 + wave * 16) * BK), 16,
                                               b_off[p], PW ? b_tile_off[p] + kt * 1024 : kt * BK * 2, 0, 0);
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // Fragment addresses. x's stage rows are swizzled (above); w's are too unless packed, where the
  // 16-byte piece of (row r of block t, k-chunk c) sits at t * 1 KB + (16 c + r) * 16 bytes: the 16 lanes
  // that one LDS cycle serves read 256 consecutive bytes.
  const int sw = (fr >> 1) & 3;
  const int koff0 = ((0 + fk) ^ sw) * 8, koff1 = ((2 + fk) ^ sw) * 8;
  const int a_row = (wm * (BM / 2) + fr) * BK;
  const int b_row = PW ? BM * BK + (wn * (BN / 32) + (fr >> 4)) * 512 + (fr & 15) * 8
                       : (BM + wn * (BN / 2) + fr) * BK;

  bf16x8_t fa[2][TM], fb[2][TN];
  auto load_frags = [&](const bf16_t* buf, int ks, int set) {
    const int koff = ks ? koff1 : koff0;
    const int koff_w = PW ? (ks * 2 + fk) * 128 : koff;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[set][i] = *reinterpret_cast<const bf16x8_t*>(buf + a_row + i * 32 * BK + koff);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[set][j] = *reinterpret_cast<const bf16x8_t*>(buf + b_row + j * 32 * BK + koff_w);
  };
  auto mfma_step = [&](int set) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
  };

  // A stage is free once every wave has passed the barrier of the slice that read it, which stands in the
  // middle of that slice (its last fragments are in registers by then). Slice j's x rows are asked for right
  // after the barrier of slice j - 4, into the stage that slice has just left, and its w rows before the barrier
  // of slice j - 3: the loads of two to three slices are in flight at any time (64 to 96 KB a workgroup of 256 x 256), which is what
  // the latency of L2 asks for at a slice every 0.4 us. (One slice less ahead - 32 to 64 KB - the matrix cores
  // waited a third of the time.) The first slices here; the host gives every range of K at least three.
  issue_x(0);
  issue_w(0);
  issue_x(1);
  issue_w(1);
  issue_x(2);
  issue_w(2);
  // s_waitcnt vmcnt(n) [lgkmcnt(0)], then the barrier (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4,
  // lgkmcnt 11:8; a counter at its maximum is not waited for).
  auto wait_barrier = [&](auto loads, auto lds_too) {
    constexpr int n = decltype(loads)::value;
    static_assert(n >= 0 && n < 64, "vmcnt has six bits");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt((n & 15) | ((n >> 4) << 14) | (7 << 4) | ((decltype(lds_too)::value ? 0 : 15) << 8));
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  using One = std::integral_constant<int, PA + PB>;
  using Two = std::integral_constant<int, 2 * (PA + PB)>;
  using None = std::integral_constant<int, 0>;
  // Slice 0 has landed when at most the loads of slices 1 and 2 are outstanding.
  wait_barrier(Two{}, std::false_type{});
  load_frags(stage(0), 0, 0);
  if (3 < k_tiles) issue_x(3);

  // One slice; its first fragments are in set 0 already. STEADY: slices up to kt + 4 exist, so the loads
  // sit in straight-line code and exactly those of slices kt + 2 and kt + 3 may still be in flight at the barrier.
  auto slice = [&](int kt, auto steady_tag) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    load_frags(stage(kt), 1, 1);
    if (STEADY || kt + 3 < k_tiles) issue_w(kt + 3);
    mfma_step(0);
    if (STEADY && BM == 256) {
#pragma unroll
      for (int q = 0; q < (4 + TN) / 2; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, TN / 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
#pragma unroll
      for (int q = 0; q < PB; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    // My share of slice kt + 1 has landed and my reads of this stage are in registers; after the
    // barrier that holds for every wave.
    if (STEADY || kt + 3 < k_tiles) wait_barrier(Two{}, std::true_type{});
    else if (kt + 2 < k_tiles) wait_barrier(One{}, std::true_type{});
    else wait_barrier(None{}, std::true_type{});
    if (STEADY || kt + 1 < k_tiles) load_frags(stage(kt + 1), 0, 0);
    if (STEADY || kt + 4 < k_tiles) issue_x(kt + 4);
    mfma_step(1);
    if (STEADY && BM == 256) {
#pragma unroll
      for (int q = 0; q < (4 + TN) / 2; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, TN / 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  int kt = 0;
  for (; kt + 7 < k_tiles; kt += 4) {
    slice(kt, std::true_type{});
    slice(kt + 1, std::true_type{});
    slice(kt + 2, std::true_type{});
    slice(kt + 3, std::true_type{});
  }
  for (; kt < k_tiles; ++kt) slice(kt, std::false_type{});

  const bool gated_n = EPI == 3;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = row0 + wm * (BM / 2) + i * 32 + fr;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = col0 + wn * (BN / 2) + j * 32 + 8 * g + 4 * fk;
        if (m >= M || n >= N) continue;
        const float v0 = acc[i][j][4 * g], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2],
                    v3 = acc[i][j][4 * g + 3];
        if (gated_n) {
          // Columns 16 b .. 16 b + 7 are gates and 16 b + 8 .. 16 b + 15 the ups of outputs 8 b .. 8 b + 7:
          // register groups g and g + 1 of one lane.
          if (g & 1) continue;
          const float u0 = acc[i][j][4 * g + 4], u1 = acc[i][j][4 * g + 5], u2 = acc[i][j][4 * g + 6],
                      u3 = acc[i][j][4 * g + 7];
          const int out_col = (n >> 4) * 8 + 4 * fk;
          uint2 pk;
          pk.x = pack_bf16x2(v0 / (1.0f + __expf(-v0)) * u0, v1 / (1.0f + __expf(-v1)) * u1);
          pk.y = pack_bf16x2(v2 / (1.0f + __expf(-v2)) * u2, v3 / (1.0f + __expf(-v3)) * u3);
          *reinterpret_cast<uint2*>(static_cast<bf16_t*>(outp) + static_cast<size_t>(m) * (N / 2) + out_col) = pk;
          continue;
        }
        const size_t o = static_cast<size_t>(m) * N + n;
        if (EPI == 0) {
          const floatx4_t r = {v0, v1, v2, v3};
          *reinterpret_cast<floatx4_t*>(static_cast<float*>(outp) + o) = r;
        } else if (EPI == 1) {
          uint2 pk;
          pk.x = pack_bf16x2(v0, v1);
          pk.y = pack_bf16x2(v2, v3);
          *reinterpret_cast<uint2*>(static_cast<bf16_t*>(outp) + o) = pk;
        } else {
          floatx4_t r = *reinterpret_cast<floatx4_t*>(static_cast<float*>(outp) + o);
          r[0] += v0; r[1] += v1; r[2] += v2; r[3] += v3;
          *reinterpret_cast<floatx4_t*>(static_cast<float*>(outp) + o) = r;
        }
      }
    }
  }
#endif
}

template <int BM, int BN, bool PW>
static int launch_gemm_dma(const void* x, const void* w, void* out, int epi, int M, int N, int K, int splits,
                           hipStream_t stream) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int k_slices = K / GD_BK;
  const int per_split = (k_slices + splits - 1) / splits;
  if (k_slices - per_split * (splits - 1) < 3) return TIE_BAD_ARGUMENT;   // the last range would be too short
  const size_t shared = sizeof(bf16_t) * GD_STAGES * (BM + BN) * GD_BK;
  const dim3 grid(tiles_m * tiles_n, splits);
#define LAUNCH(EPI)                                                                                          \
  {                                                                                                          \
    static bool raised = false;                                                                              \
    if (!raised) {                                                                                           \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_bf16_dma_kernel<BM, BN, EPI, PW>),  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared)); \
      if (e != hipSuccess) return static_cast<int>(e);                                                       \
      raised = true;                                                                                         \
    }                                                                                                        \
    gemm_bf16_dma_kernel<BM, BN, EPI, PW><<<grid, 256, shared, stream>>>(                                    \
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), out, M, N, K, tiles_m, tiles_n, per_split); \
  }
  if (epi == 0) LAUNCH(0) else if (epi == 1) LAUNCH(1) else if (epi == 2) LAUNCH(2) else LAUNCH(3)
#undef LAUNCH
  return tie_launch_status();
}

// Whether the direct-to-LDS kernel takes this product: whole slices of 32, at least three per range of K,
// 16-byte aligned rows and 4-column output pieces, and row offsets within a tile that fit 32 bits.
static bool gemm_dma_takes(const void* x, const void* w, const void* out, int N, int K, int splits) {
  if (K % GD_BK != 0 || N % 4 != 0 || K > (1 << 22)) return false;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(w) % 16 ||
      reinterpret_cast<uintptr_t>(out) % 16)
    return false;
  const int k_slices = K / GD_BK;
  const int per_split = (k_slices + splits - 1) / splits;
  return k_slices - per_split * (splits - 1) >= 3;
}

// Which tile, and how many ranges of K (planes of partial sums that the caller adds), a product takes when
// left to choose.
//
// Up to 64 rows over packed weights: a score (below); 65 to 128 rows: few_rows_us. Above that, for shapes the
// straight-to-LDS tiles take: the cheapest of (tile, ranges) by an estimate of the time, whose constants were chosen
// on sweeps over the projections of four shapes (widths 2048, 3072, 4096 and 5120) at 160 to 2048 rows, every
// candidate timed with the kernel that consumes its planes, so that the choice lies as close to the best candidate
// as it can (2.2 % above it on average, 3.6 % with the constants fitted to times of three shapes before):
//   * a compute unit holds one workgroup (two of the 128 x 128 tile), so the workgroups run in rounds of
//     256; a round that is nearly empty lasts as long as a full one, which is what a rule by thresholds
//     gets wrong (768 rows of 256 x 128 tiles over 6144 columns and two ranges: 288 workgroups, two rounds);
//   * a round is a few microseconds of start and end plus its slices of 32 along K at the tile's own pace;
//   * every plane is written once here and read once by its consumer.
// Without the straight-to-LDS tiles (odd K or N) the older tiles and their rule stand.
struct GemmPlan { int tile, splits; };

static int legacy_splits(int M, int N, int K) {
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

struct DmaTile { int id, bm, bn; float start_us, full_us, slice_us; int per_cu; };
// start_us: a round's start and end; full_us: what a round costs more when it fills every compute unit (measured
// for the 256 x 256 and 256 x 192 tiles, whatever the length of K: 256 workgroups of the first start about 11 us
// later than 192);
// slice_us: one slice of 32 along K with the compute unit to itself.
static const DmaTile kDmaTiles[] = {{4, 256, 256, 8.8f, 7.9f, 0.67f, 1}, {10, 256, 192, 5.f, 5.4f, 0.55f, 1},
                                    {5, 256, 128, 6.25f, 0.f, 0.53f, 1}, {6, 128, 256, 6.25f, 1.f, 0.50f, 1},
                                    {7, 128, 128, 3.24f, 1.f, 0.324f, 2}};

static float estimated_us(const DmaTile& t, int M, int N, int K, int ranges) {
  const long wgs = static_cast<long>((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn) * ranges;
  const int k_slices = K / GD_BK;
  const int slices = (k_slices + ranges - 1) / ranges;
  const long slots = 256L * t.per_cu;
  const float pace = t.slice_us * (t.per_cu > 1 && wgs > 256 ? 1.94f : 1.0f);   // two workgroups share the matrix cores
  auto round_us = [&](float fill) {
    const float crowded = fminf(fmaxf((fill - 0.75f) * 4.0f, 0.f), 1.f);
    return t.start_us + t.full_us * crowded + slices * pace;
  };
  float us = static_cast<float>(wgs / slots) * round_us(1.0f);
  if (wgs % slots) us += round_us(static_cast<float>(wgs % slots) / slots);
  const float plane_mb = static_cast<float>(M) * N * 4e-6f;
  return ranges > 1 ? us + ranges * plane_mb * 0.2f : us;   // planes written here, read by the consumer: MB / (TB/s) = us
}

// 65 to 128 rows: a workgroup's pace is set by the bytes it loads a slice of 32 along K, its rows of x and its
// columns of w (about 40 GB/s a compute unit), and all of them together by the weights' bytes (5.5 TB/s);
// workgroups run in rounds of 256. Fitted to sweeps over the projections of the 1.7B, 8B and 32B shapes at 80,
// 96 and 128 rows: 8B gate/up at 128 rows 61 us on 128 x 128 tiles (192 workgroups) against 82 on 128 x 256 (96).
struct FewRowsTile { int id, bm, bn; };
static const FewRowsTile kFewRowsTiles[] = {{6, 128, 256}, {7, 128, 128}, {8, 64, 256}, {9, 64, 128}};

static float few_rows_us(const FewRowsTile& t, int M, int N, int K, int ranges) {
  const long wgs = static_cast<long>((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn) * ranges;
  const int k_slices = K / GD_BK;
  const int slices = (k_slices + ranges - 1) / ranges;
  const float per_slice = static_cast<float>(t.bm + t.bn) * (GD_BK * 2) / 40000.f;
  float us = static_cast<float>((wgs + 255) / 256) * (4.f + slices * per_slice);
  us = fmaxf(us, static_cast<float>(N) * K * 2e-6f / 5.5f);
  if (ranges > 1) us += ranges * static_cast<float>(M) * N * 4e-6f * (1.0f / 6.0f + 1.0f / 5.0f);
  return us;
}

// splits: 0 = free to choose (the caller adds planes), else the number of ranges the caller has fixed (1: none).
static GemmPlan gemm_plan(int M, int N, int K, bool straight_to_lds, int splits, bool packed) {
  const bool may_split = splits == 0;
  if (straight_to_lds && packed && M > 64 && M <= 128) {
    // 65 to 128 rows over packed weights: the weights are read once by few workgroups, so what counts is that
    // one round of workgroups fills the compute units. The cheapest of (tile, ranges) by few_rows_us.
    GemmPlan best = {7, may_split ? 1 : splits};
    float best_us = 0.f;
    for (int r = may_split ? 1 : splits; r <= (may_split ? 8 : splits); r *= 2) {
      if (may_split && r > 1 && K / r < 512) break;
      for (const FewRowsTile& t : kFewRowsTiles) {
        const float us = few_rows_us(t, M, N, K, r);
        if (best_us == 0.f || us < best_us * 0.98f) {       // ties go to fewer planes, then to the larger tile
          best = {t.id, r};
          best_us = us;
        }
      }
    }
    return best;
  }
  if (straight_to_lds && packed && M <= 64) {
    // Up to 64 rows over packed weights: tiles of 64 rows, one workgroup a compute unit, the weights read once. The
    // cheapest (tile, ranges) by a score of three factors: what the 64 rows of x cost beside a tile's columns
    // (1 + 1 / columns' 16-blocks), the planes' traffic and shorter runs of K (1 + 0.25 log2(ranges)), and how
    // full the rounds of 256 workgroups are. The caller's fixed ranges (a gated product: one) are scored alone,
    // with the same result when it hands back what this plan chose. Ranges of at least 512 of K. Over the
    // projections of eight shapes at 48 and 64 rows the choice lies 2.9 % above the best forced (tile, ranges) on
    // average and at most 17 %; the rule by thresholds that stood here gave the 32B shape's QKV (40 tiles of 256
    // columns) eight ranges, 320 workgroups, a second round for 64 of them: 1.7 times the time of four.
    GemmPlan best = {9, may_split ? 1 : splits};
    float best_score = 0.f;
    // a weight so wide that the wider tile alone fills a round (an lm_head) has nothing to balance: the wider tile
    for (int tile = (N + 255) / 256 >= 256 ? 8 : 9; tile >= 8; --tile) {
      const int columns = tile == 8 ? 256 : 128;
      const long across = (N + columns - 1) / columns;
      for (int r = may_split ? 1 : splits; r <= (may_split ? 8 : splits); r *= 2) {
        if (may_split && r > 1 && K / r < 512) break;
        const long wgs = across * r;
        const float fill = static_cast<float>(wgs) / static_cast<float>((wgs + 255) / 256 * 256);
        const float score = (1.0f + 16.0f / columns) * (1.0f + 0.25f * log2f(static_cast<float>(r))) / fill;
        if (best_score == 0.f || score < best_score) {
          best = {tile, r};
          best_score = score;
        }
      }
    }
    return best;
  }
  if (straight_to_lds && M > 128) {
    GemmPlan best = {4, may_split ? 1 : splits};
    float best_us = 0.f;
    const int k_slices = K / GD_BK;
    for (int r = may_split ? 1 : splits; r <= (may_split ? 8 : splits); r *= 2) {
      const int per = (k_slices + r - 1) / r;
      if (may_split && r > 1 && (K / r < 512 || k_slices - per * (r - 1) < 3)) break;
      for (const DmaTile& t : kDmaTiles) {
        const float us = estimated_us(t, M, N, K, r);
        if (best_us == 0.f || us < best_us * 0.98f) {       // ties go to fewer planes, then to the larger tile
          best = {t.id, r};
          best_us = us;
        }
      }
    }
    return best;
  }
  if (may_split) return {1, legacy_splits(M, N, K)};
  if (splits > 1) return {1, splits};
  const long rows256 = (M + 255) / 256;
  const long t256 = rows256 * ((N + 255) / 256), t128 = rows256 * ((N + 127) / 128);
  return {t256 >= 160 ? 2 : (t128 >= 192 ? 3 : 1), 1};
}

static bool straight_to_lds_shape(int N, int K) { return K % GD_BK == 0 && N % 4 == 0 && K <= (1 << 22) && K >= 3 * GD_BK; }

// Whether a product of 33 to 64 rows runs faster here than on the decode product: over packed weights whose
// shape the tiles that load straight into LDS take, unless it is gated and not very wide (measured).
extern "C" int tie_gemm_bf16_wins_few_rows(int M, int N, int K, int packed, int gated) {
  if (M <= 32 || M > 64 || !packed || !straight_to_lds_shape(N, K) || N % 16 != 0 || K < 1024) return 0;
  return gated ? N >= 32768 : 1;
}

// Ranges of K that a product of M rows over w[N, K] is best cut into when its caller adds planes of
// partial sums: few rows over a narrow weight give too few workgroups otherwise.
extern "C" int tie_gemm_bf16_splits(int M, int N, int K, int packed) {
  if (packed && !straight_to_lds_shape(N, K)) return 1;
  return gemm_plan(M, N, K, straight_to_lds_shape(N, K), 0, packed != 0).splits;
}

// The tile a product left to choose runs on (the numbers of tie_gemm_bf16's `tile`), with `splits` ranges of K
// fixed by the caller (1: none) or 0 for the plan's own number; for tests and sweeps.
extern "C" int tie_gemm_bf16_tile(int M, int N, int K, int packed, int splits) {
  return gemm_plan(M, N, K, straight_to_lds_shape(N, K), splits, packed != 0).tile;
}

// out_dtype: TIE_F32 or TIE_BF16; accumulate adds into a float32 output; gated (bfloat16 output of N / 2
// columns, N % 16 == 0) applies silu(gate) * up to interleaved column blocks.
// splits > 1: out is float32 [splits, M, N], plane s holding the sums over the s-th range of K
// (128x128 tiles; neither accumulate nor gated).
// tile: 0 = choose, 1 = 128x128 (four waves of 64x64), 2 = 256x256 (eight waves of 128x64),
//       3 = 256x128 (eight waves of 64x64), 4 = 256x256 and 5 = 256x128 loaded straight into LDS (four
//       waves of 128x128 or 128x64; K % 32 == 0, N % 4 == 0, 16-byte aligned operands, else refused),
//       6 = 128x256, 7 = 128x128, 8 = 64x256, 9 = 64x128 likewise, for fewer rows; 10 = 256x192 likewise, for
//       widths that 256 columns a tile leave with a round of workgroups that does not fill the compute units.
// packed: w is stored in blocks of 16 rows x 32 k, 1 KB each, in the matrix cores' operand order (as the
//       decode product reads it); N % 16 == 0, and only tiles 4 and 5 read it.
extern "C" int tie_gemm_bf16(const void* x, const void* w, void* out, int out_dtype, int accumulate, int gated, int M,
                             int N, int K, int tile, int splits, int packed, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || splits < 1) return TIE_BAD_ARGUMENT;
  if (accumulate && out_dtype != TIE_F32) return TIE_BAD_ARGUMENT;
  if (out_dtype != TIE_F32 && out_dtype != TIE_BF16) return TIE_BAD_ARGUMENT;
  if (gated && (accumulate || out_dtype != TIE_BF16 || N % 16 != 0)) return TIE_BAD_ARGUMENT;
  if (splits > 1 && (accumulate || gated || out_dtype != TIE_F32)) return TIE_BAD_ARGUMENT;
  const int epi = gated ? 3 : (accumulate ? 2 : (out_dtype == TIE_F32 ? 0 : 1));
  const bool straight = gemm_dma_takes(x, w, out, N, K, splits);
  if (packed && (N % 16 != 0 || !straight || (tile != 0 && (tile < 4 || tile > 10)))) return TIE_BAD_ARGUMENT;
  if (tile == 0) {
    tile = gemm_plan(M, N, K, straight, splits, packed != 0).tile;
  } else if (tile < 4 && splits > 1) {
    tile = 1;
  }
  if (tile >= 4 && tile <= 10) {
    if (!straight) return TIE_BAD_ARGUMENT;
#define DMA(BM, BN)                                                                            \
  return packed ? launch_gemm_dma<BM, BN, true>(x, w, out, epi, M, N, K, splits, stream)       \
                : launch_gemm_dma<BM, BN, false>(x, w, out, epi, M, N, K, splits, stream)
    switch (tile) {
      case 4: DMA(256, 256);
      case 5: DMA(256, 128);
      case 6: DMA(128, 256);
      case 7: DMA(128, 128);
      case 8: DMA(64, 256);
      case 9: DMA(64, 128);
      default: DMA(256, 192);
    }
#undef DMA
  }
  if (tile == 2) return launch_gemm<256, 256, 64, 2, 4>(x, w, out, epi, M, N, K, splits, stream);
  if (tile == 3) return launch_gemm<256, 128, 64, 4, 2>(x, w, out, epi, M, N, K, splits, stream);
  return launch_gemm<128, 128, 64, 2, 2>(x, w, out, epi, M, N, K, splits, stream);
}
