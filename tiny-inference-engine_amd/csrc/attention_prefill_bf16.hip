// Paged causal attention for prompt portions (several new rows per sequence) on the gfx950 matrix
// cores: bfloat16 queries and cache, float32 softmax. Compiled per head size: -DHEAD_DIM=<multiple of 16>.
//
// A workgroup of four waves owns up to 128 consecutive new rows of one sequence and up to four
// query heads that share a KV head: wave w takes (head hc, 32-row tile qc) with HC x QC = 4 pairs,
// HC = min(4, heads per KV head). The workgroup walks the keys in tiles of 64 at absolute
// multiples of 64 positions: the four waves together copy the tile's keys ([key][d]) and values
// (transposed, [d][key], as they lie in a page) from the cache into LDS, one tile ahead of the
// arithmetic, and each wave then computes for its 32 rows
//
//   S^T[key, row] = K[key, :] . Q[row, :]        A = K rows from LDS, B = Q (registers), 32x32x16 MFMA
//   online softmax per row (= per lane column) in float32, causal by position (and windowed)
//   O^T[d, row]  += V^T[d, key] . P^T[key, row]   A = V^T rows from LDS, B = P (registers)
//
// so every byte of the cache is read once per workgroup and feeds four (head, row tile) pairs. The
// D layout of S^T hands each lane exactly the probabilities it must supply as B operand of the
// second product when the values' keys are taken in the same order (4 keys, skip 4, 4 keys), so
// probabilities never leave registers.
//
// Keys come through the block table, so a portion attends to earlier portions and to itself alike;
// the row at new index i of a sequence sits at position ctx - n_new + i. Because tiles are cut at
// absolute positions and every row keeps its own running maximum, a position's result does not
// depend on how the prompt was cut into steps or on which rows share its workgroup.
//
// Formula: src/backend/cpu/cpu_backend.cpp:261-319.
#include "common.h"

#include <math.h>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // a native vector: stays in registers
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int DH = HEAD_DIM;
constexpr int KS = DH / 16;            // k-steps of the score product
constexpr int DT = (DH + 31) / 32;     // 32-row tiles of O^T; rows beyond DH are zero
constexpr int KT = 64;                 // keys per tile
constexpr int KROW = DH + 8;           // LDS row of a key, padded: 16-byte reads of 16 lanes hit distinct banks
constexpr int VROW = KT + 8;           // LDS row of one value dimension, padded likewise; its keys are permuted (below)
constexpr int THREADS = 256;
constexpr int K_CHUNKS = KT * DH / 8;          // 16-byte pieces of a key tile
constexpr int V_CHUNKS = DT * 32 * (KT / 8);   // 8-key pieces of a value tile (rows beyond DH are zeros)
constexpr int K_PER_THREAD = (K_CHUNKS + THREADS - 1) / THREADS;
constexpr int V_PER_THREAD = (V_CHUNKS + THREADS - 1) / THREADS;
constexpr int LDS_TILE = KT * KROW + DT * 32 * VROW;   // bf16 elements of one buffer

union Frag {
  bf16x8_t v;
  uint4 u4;
  uint2 u2[2];
  uint32_t w[4];   // pairs of bfloat16; built with pack2 so that fragments stay in registers
};

__device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }

// Reads tile `tile` of the keys and values of one KV head into the registers kreg / vreg of the
// calling kernel. Key positions are clamped into [first, last]: pages before or after the range this
// workgroup may touch are never addressed (their table entries need not be valid); clamped keys are
// masked by position later. A macro, so that the register arrays are plain locals of the kernel.
//
// Addresses are formed in units of 8 bytes from 32-bit numbers (a page's number times the units of a page
// with the 24-bit multiply, which runs at full rate): the address arithmetic of the eight pieces a thread
// copies per tile weighs as much as the softmax when done in 64 bits. The host refuses caches of 32 GB or
// more and pages of 2^24 units or more, which this cannot address.
#define PAGE_OF(kp) ((kp) >> block_shift)
#define OFFSET_OF(kp) ((kp) & (block_size - 1))
// LOAD_PAGES looks up the pages of every piece of a tile this thread copies; LOAD_TILE then reads the
// pieces. Two steps, so that all lookups are in flight together and no data load waits for one:
// the pages of tile t + 2 are looked up while the data of tile t + 1 is on its way.
#define LOAD_PAGES(tile_index)                                                                                     \
  {                                                                                                                \
    const int base_ = (tile_index) * KT;                                                                           \
    _Pragma("unroll") for (int i_ = 0; i_ < K_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      const int kp_ = min(max(base_ + c_ / (DH / 8), wg_first), wg_last);                                          \
      kpage[i_] = (K_CHUNKS % THREADS == 0 || c_ < K_CHUNKS) ? table[PAGE_OF(kp_)] : 0;                            \
    }                                                                                                              \
    _Pragma("unroll") for (int i_ = 0; i_ < V_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      const int kg_ = c_ % (KT / 8);                                                                               \
      const bool live_ = (V_CHUNKS % THREADS == 0 || c_ < V_CHUNKS) && (DH % 32 == 0 || c_ / (KT / 8) < DH);       \
      const int kp0_ = min(max(base_ + kg_ * 8, first_v), last_v);                                                 \
      vpage[i_][0] = live_ ? table[PAGE_OF(kp0_)] : 0;                                                             \
      if (!WIDE) {                                                                                                 \
        const int kp1_ = min(max(base_ + kg_ * 8 + 4, first_v), last_v);                                           \
        vpage[i_][1] = live_ ? table[PAGE_OF(kp1_)] : 0;                                                           \
      }                                                                                                            \
    }                                                                                                              \
  }

#define LOAD_TILE(tile_index)                                                                                      \
  {                                                                                                                \
    const int base_ = (tile_index) * KT;                                                                           \
    _Pragma("unroll") for (int i_ = 0; i_ < K_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      if (K_CHUNKS % THREADS == 0 || c_ < K_CHUNKS) {                                                              \
        const int kp_ = min(max(base_ + c_ / (DH / 8), wg_first), wg_last);                                        \
        const uint32_t unit_ = __umul24(static_cast<uint32_t>(kpage[i_]), page_units) + head_units +               \
                               static_cast<uint32_t>(OFFSET_OF(kp_)) * (DH / 4) + (c_ % (DH / 8)) * 2;             \
        kreg[i_] = *reinterpret_cast<const u32x4_t*>(k_units + unit_);                                             \
      }                                                                                                            \
    }                                                                                                              \
    _Pragma("unroll") for (int i_ = 0; i_ < V_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      const int d_ = c_ / (KT / 8), kg_ = c_ % (KT / 8);                                                           \
      if ((V_CHUNKS % THREADS == 0 || c_ < V_CHUNKS) && (DH % 32 == 0 || d_ < DH)) {                               \
        const int kp0_ = min(max(base_ + kg_ * 8, first_v), last_v);                                               \
        const uint32_t row_ = head_units + static_cast<uint32_t>(d_) * row_units;   /* the same for every tile */  \
        const uint32_t unit0_ = __umul24(static_cast<uint32_t>(vpage[i_][0]), page_units) + row_ +                 \
                                (static_cast<uint32_t>(OFFSET_OF(kp0_)) >> 2);                                     \
        if (WIDE) {                                                                                                \
          vreg[i_] = *reinterpret_cast<const u32x4_t*>(v_units + unit0_);                                          \
        } else {                                                                                                   \
          const int kp1_ = min(max(base_ + kg_ * 8 + 4, first_v), last_v);                                         \
          const uint32_t unit1_ = __umul24(static_cast<uint32_t>(vpage[i_][1]), page_units) + row_ +               \
                                  (static_cast<uint32_t>(OFFSET_OF(kp1_)) >> 2);                                   \
          const u32x2_t h0_ = v_units[unit0_];                                                                     \
          const u32x2_t h1_ = v_units[unit1_];                                                                     \
          vreg[i_] = u32x4_t{h0_.x, h0_.y, h1_.x, h1_.y};                                                          \
        }                                                                                                          \
      } else {                                                                                                     \
        vreg[i_] = u32x4_t{0, 0, 0, 0};                                                                            \
      }                                                                                                            \
    }                                                                                                              \
  }

#define STORE_TILE(k_dst, v_dst)                                                                                   \
  {                                                                                                                \
    _Pragma("unroll") for (int i_ = 0; i_ < K_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      if (K_CHUNKS % THREADS == 0 || c_ < K_CHUNKS)                                                                \
        *reinterpret_cast<u32x4_t*>((k_dst) + (c_ / (DH / 8)) * KROW + (c_ % (DH / 8)) * 8) = kreg[i_];            \
    }                                                                                                              \
    _Pragma("unroll") for (int i_ = 0; i_ < V_PER_THREAD; ++i_) {                                                  \
      const int c_ = threadIdx.x + i_ * THREADS;                                                                   \
      if (V_CHUNKS % THREADS == 0 || c_ < V_CHUNKS) {                                                              \
        /* Within a block of 16 keys the order in LDS is 0-3, 8-11, 4-7, 12-15: the 8 keys a lane supplies to */   \
        /* one matrix instruction (4 keys, skip 4, 4 keys) then lie together and are read as one 16-byte piece. */ \
        const int kg_ = c_ % (KT / 8);                                                                             \
        bf16_t* row_ = (v_dst) + (c_ / (KT / 8)) * VROW + (kg_ / 2) * 16 + (kg_ % 2) * 4;                          \
        *reinterpret_cast<u32x2_t*>(row_) = u32x2_t{vreg[i_].x, vreg[i_].y};                                       \
        *reinterpret_cast<u32x2_t*>(row_ + 8) = u32x2_t{vreg[i_].z, vreg[i_].w};                                   \
      }                                                                                                            \
    }                                                                                                              \
  }

// items: [num_items][2] = (sequence, index of its first new row handled here); the last items run first.
// WIDE: the block size is a multiple of 8, so 8 keys of one value dimension lie together in a page.
template <int HC, int QC, bool WIDE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ items, int num_items, int H, int KVH, int block_size,
    int max_blocks, float scale_log2e, int window, int block_shift, int flip_from, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* lds = reinterpret_cast<bf16_t*>(smem);
  const int wave = threadIdx.x / TIE_WAVE;
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int r32 = lane & 31;
  const int hi = lane >> 5;
  const int hc = wave / QC, qc = wave % QC;
  // Long rows (late in a prompt) first. Where the whole grid is resident at once (two workgroups a CU),
  // the second half of it runs short rows first instead, so that a CU's two workgroups add up alike.
  const bool flipped = static_cast<int>(blockIdx.y + blockIdx.z * gridDim.y) >= flip_from;
  // With nsplit > 1 a workgroup walks only its share of the item's key tiles and leaves partial results.
  const int bx = static_cast<int>(blockIdx.x) / nsplit;
  const int split = static_cast<int>(blockIdx.x) % nsplit;
  const int item = flipped ? bx : num_items - 1 - bx;
  const int s = items[item * 2];
  const int row0 = items[item * 2 + 1];
  const int kvh = blockIdx.y;
  const int G = H / KVH;
  const int head0 = kvh * G + blockIdx.z * HC;
  const int heads_here = min(HC, kvh * G + G - head0);
  const int qs = query_start[s];
  const int n_new = query_start[s + 1] - qs;
  const int ctx = context_lens[s];
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  // The workgroup's rows and the keys any of them may see.
  const int rows_end = min(n_new, row0 + 32 * QC);
  if (rows_end <= row0) return;   // uniform for the workgroup
  const int wg_first = window > 0 ? max(0, ctx - n_new + row0 - window + 1) : 0;
  const int wg_last = ctx - n_new + rows_end - 1;

  // This wave's rows; this lane's row is column r32 of every product.
  const int wave_row0 = row0 + qc * 32;
  const bool wave_active = hc < heads_here && wave_row0 < n_new;
  const int i = wave_row0 + r32;
  const bool valid = wave_active && i < n_new;
  const int pos = valid ? ctx - n_new + i : -1;
  const int lo = (window > 0 && valid) ? max(0, pos - window + 1) : 0;
  const int wave_last = wave_active ? ctx - n_new + min(n_new, wave_row0 + 32) - 1 : -1;
  const int wave_min_pos = ctx - n_new + wave_row0;   // lowest position among the wave's rows

  Frag qf[KS];
  {
    const bf16_t* qr = q + (static_cast<size_t>(qs + (valid ? i : 0)) * H + head0 + (wave_active ? hc : 0)) * DH;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks].u4 = valid ? *reinterpret_cast<const uint4*>(qr + ks * 16 + hi * 8) : make_uint4(0, 0, 0, 0);
  }

  floatx16 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;
  float m = -INFINITY, l = 0.f;

  int tile_begin = wg_first / KT, tile_end = wg_last / KT;       // inclusive
  if (nsplit > 1) {
    const int per = (tile_end - tile_begin + nsplit) / nsplit;   // ceil(count / nsplit)
    tile_begin += split * per;
    tile_end = min(tile_end, tile_begin + per - 1);
  }
  const bool empty = tile_begin > tile_end;                      // uniform: a short row range has fewer tiles than splits
  // In units of 8 bytes (4 elements): a page, this KV head inside a page, one value dimension's keys of a page.
  const uint32_t page_units = static_cast<uint32_t>(KVH) * block_size * (DH / 4);
  const uint32_t head_units = static_cast<uint32_t>(kvh) * block_size * (DH / 4);
  const uint32_t row_units = static_cast<uint32_t>(block_size) / 4;
  const u32x2_t* k_units = reinterpret_cast<const u32x2_t*>(k_cache);
  const u32x2_t* v_units = reinterpret_cast<const u32x2_t*>(v_cache);
  constexpr int VG = WIDE ? 8 : 4;   // keys of one value dimension read in one piece
  const int first_v = wg_first / VG * VG, last_v = wg_last / VG * VG;
  u32x4_t kreg[K_PER_THREAD], vreg[V_PER_THREAD];
  int kpage[K_PER_THREAD], vpage[V_PER_THREAD][WIDE ? 1 : 2];
  if (!empty) {
    LOAD_PAGES(tile_begin);
    LOAD_TILE(tile_begin);
    if (tile_begin < tile_end) LOAD_PAGES(tile_begin + 1);
    STORE_TILE(lds, lds + KT * KROW);
  }
  __syncthreads();

  for (int tile = tile_begin; tile <= tile_end; ++tile) {
    const int buf = (tile - tile_begin) & 1;
    const bf16_t* k_lds = lds + buf * LDS_TILE;
    const bf16_t* v_lds = k_lds + KT * KROW;
    if (tile < tile_end) LOAD_TILE(tile + 1);          // its pages were looked up an iteration ago
    if (tile + 1 < tile_end) LOAD_PAGES(tile + 2);

    const int base = tile * KT;
    if (wave_active && base <= wave_last) {
      floatx16 sc[2];
      const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          Frag a;
          a.u4 = *reinterpret_cast<const uint4*>(k_lds + (u * 32 + r32) * KROW + ks * 16 + hi * 8);
          sc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[ks].v, ks == 0 ? zero : sc[u], 0, 0, 0);
        }
      }
      // Element v of sc[u] is key base + u*32 + 8*(v/4) + hi*4 + v%4 against this lane's row.
      // A tile every row of the wave sees whole needs no mask.
      const bool whole = base + KT - 1 <= wave_min_pos && (window <= 0 || base >= wave_last - window + 1) &&
                         wave_row0 + 32 <= n_new;
      // Scores stay unscaled; scale * log2(e) > 0 enters in the exponent: p = 2^(s*c - m*c), one fma each.
      if (!whole) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int kp = base + u * 32 + 8 * (v / 4) + hi * 4 + (v % 4);
            sc[u][v] = (kp <= pos && kp >= lo) ? sc[u][v] : -INFINITY;
          }
      }
      float tile_max = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 16; ++v) tile_max = fmaxf(tile_max, sc[u][v]);
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, TIE_WAVE));
      const float m_new = fmaxf(m, tile_max);
      const float neg_mc = (m_new == -INFINITY) ? 0.f : -m_new * scale_log2e;
      const float corr = __builtin_amdgcn_exp2f(fmaf(m, scale_log2e, neg_mc));   // m = -inf: 0
      Frag pf[4];
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[j / 2][(j % 2) * 8 + e], scale_log2e, neg_mc));   // masked: 0
          const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[j / 2][(j % 2) * 8 + e + 1], scale_log2e, neg_mc));
          psum += p0;
          psum += p1;
          pf[j].w[e / 2] = pack2(p0, p1);
        }
      l = l * corr + psum;
      if (__any(m_new != m)) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[dt][v] *= corr;
      }
      m = m_new;
      // B operand slot hi*8 + e of 16-key block j holds key j*16 + hi*4 + e%4 + 8*(e/4): V^T lies in that order.
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Frag a;
          a.u4 = *reinterpret_cast<const uint4*>(v_lds + (dt * 32 + r32) * VROW + j * 16 + hi * 8);
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[j].v, acc[dt], 0, 0, 0);
        }
      // The output accumulators are rescaled by ordinary multiplications: keep them in vector
      // registers across iterations rather than in accumulation registers that need copies.
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+v"(acc[dt]));
    }

    if (tile < tile_end) {
      bf16_t* next = lds + (buf ^ 1) * LDS_TILE;   // last read two iterations ago, before the barrier below
      STORE_TILE(next, next + KT * KROW);
    }
    __syncthreads();
  }

  l += __shfl_xor(l, 32, TIE_WAVE);
  if (!valid) return;
  // Element v of acc[dt] is dimension dt*32 + 8*(v/4) + hi*4 + v%4.
  if (nsplit > 1) {   // partial results of this share of the keys, merged by a second kernel
    const size_t slot = (static_cast<size_t>(qs + i) * H + head0 + hc) * nsplit + split;
    float* po = part_o + slot * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int d0 = dt * 32 + 8 * vq + hi * 4;
        if (DH % 32 != 0 && d0 >= DH) continue;
        *reinterpret_cast<float4*>(po + d0) =
            make_float4(acc[dt][vq * 4], acc[dt][vq * 4 + 1], acc[dt][vq * 4 + 2], acc[dt][vq * 4 + 3]);
      }
    if (hi == 0) {
      part_ml[slot * 2] = m * scale_log2e;     // the merge works in the exponent's units (base 2); -inf if empty
      part_ml[slot * 2 + 1] = l;
    }
    return;
  }
  const float inv = 1.0f / l;
  bf16_t* o = out + (static_cast<size_t>(qs + i) * H + head0 + hc) * DH;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int d0 = dt * 32 + 8 * vq + hi * 4;
      if (DH % 32 != 0 && d0 >= DH) continue;
      *reinterpret_cast<uint2*>(o + d0) = make_uint2(pack2(acc[dt][vq * 4] * inv, acc[dt][vq * 4 + 1] * inv),
                                                     pack2(acc[dt][vq * 4 + 2] * inv, acc[dt][vq * 4 + 3] * inv));
    }
}

#include "attention_merge.h"

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

static void shape_for_group(int G, int* hc, int* qc) {
  *hc = G >= 4 ? 4 : G;
  *qc = *hc == 4 || *hc == 3 ? 1 : (*hc == 2 ? 2 : 4);
}

// Rows of new tokens one work item covers, for a model with G query heads per KV head.
extern "C" int tie_attention_prefill_rows_per_item(int G) {
  int hc, qc;
  shape_for_group(G, &hc, &qc);
  return 32 * qc;
}

template <int HC, int QC, bool WIDE>
static int launch_prefill(const dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k_cache,
                          const bf16_t* v_cache, bf16_t* out, const int* query_start, const int* context_lens,
                          const int* block_tables, const int* items, int num_items, int H, int KVH, int block_size,
                          int max_blocks, float scale_log2e, int window, int nsplit, float* part_o, float* part_ml) {
  const int block_shift = __builtin_ctz(block_size);   // block sizes are powers of two here
  // One resident round (at most two workgroups on each of the compute units): see the kernel's item order.
  const long planes = static_cast<long>(grid.y) * grid.z;
  const int flip_from = (nsplit == 1 && planes >= 2 && planes * grid.x <= 2L * compute_units())
                            ? static_cast<int>(planes / 2) : 0x7fffffff;
  constexpr size_t lds_bytes = 2 * static_cast<size_t>(LDS_TILE) * sizeof(bf16_t);
  static bool configured = false;
  if (!configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<HC, QC, WIDE>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (e != hipSuccess) return static_cast<int>(e);
    configured = true;
  }
  attention_prefill_kernel<HC, QC, WIDE><<<grid, THREADS, lds_bytes, stream>>>(
      q, k_cache, v_cache, out, query_start, context_lens, block_tables, items, num_items, H, KVH, block_size,
      max_blocks, scale_log2e, window, block_shift, flip_from, nsplit, part_o, part_ml);
  return tie_launch_status();
}

// nsplit > 1: every item's keys are cut into nsplit shares, one workgroup each; part_o
// [rows][H][nsplit][DH] and part_ml [rows][H][nsplit][2] (rows = all rows of the step) take the
// partial results and a second kernel merges them into out for the num_rows rows of the step.
extern "C" int tie_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                          const int* query_start, const int* context_lens, const int* block_tables,
                                          const int* items, int num_items, int H, int KVH, int block_size,
                                          int max_blocks, float scale, int window, int nsplit, float* part_o,
                                          float* part_ml, const int* merge_rows, int num_merge_rows,
                                          hipStream_t stream) {
  if (num_items <= 0 || H <= 0 || KVH <= 0 || KVH > 65535 || H % KVH != 0 || block_size < 4 ||
      (block_size & (block_size - 1)) != 0 || max_blocks <= 0 || !(scale > 0.f) || nsplit < 1 ||
      nsplit > MERGE_MAX_SPLITS)   // the running maximum is kept on unscaled scores
    return TIE_BAD_ARGUMENT;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr || merge_rows == nullptr || num_merge_rows <= 0 ||
                     num_merge_rows > 65535))
    return TIE_BAD_ARGUMENT;
  const int G = H / KVH;
  int hc, qc;
  shape_for_group(G, &hc, &qc);
  const int passes = (G + hc - 1) / hc;
  if (passes > 65535) return TIE_BAD_ARGUMENT;
  const dim3 grid(num_items * nsplit, KVH, passes);
  const float scale_log2e = scale * 1.44269504088896340736f;
  int status;
#define LAUNCH(HC, QC)                                                                                            \
  status = (block_size % 8 == 0 ? launch_prefill<HC, QC, true> : launch_prefill<HC, QC, false>)(                  \
      grid, stream, static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_cache),                           \
      static_cast<const bf16_t*>(v_cache), static_cast<bf16_t*>(out), query_start, context_lens, block_tables,    \
      items, num_items, H, KVH, block_size, max_blocks, scale_log2e, window, nsplit, part_o, part_ml)
  if (hc == 4) LAUNCH(4, 1);
  else if (hc == 3) LAUNCH(3, 1);
  else if (hc == 2) LAUNCH(2, 2);
  else LAUNCH(1, 4);
#undef LAUNCH
  if (status != TIE_OK || nsplit == 1) return status;
  launch_attention_merge(part_o, part_ml, static_cast<bf16_t*>(out), merge_rows, nullptr, nullptr, H, nsplit,
                         num_merge_rows, stream);
  return tie_launch_status();
}
