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

// ---------------------------------------------------------------------------------------------
// The same attention with the tiles going cache -> LDS directly (buffer loads with the lds flag), for pages
// of 16 positions or more and head sizes 32, 64, 128 and 256.
//
// The kernel above copies a tile through registers: per tile a thread looks up eight pages, forms eight
// addresses, loads eight pieces and writes them to LDS, and that arithmetic is a third of its vector
// instructions. Here a block of 16 keys lies in one page, and wave w stages block w of every tile (64 keys =
// four blocks): it reads the block's page number with a scalar load, makes the block's keys and values a
// buffer each, and issues DH / 32 + DH / 32 load instructions whose per-lane offsets never change; no vector
// arithmetic, no staging registers, no LDS write instructions. One instruction fills 1 KB of consecutive
// LDS (lane l's 16 bytes at byte 16 l), so the layout is made by choosing what each lane fetches:
//
//   keys    [64 rows][DH], unpadded. Row r of a block of 16 holds key pi(r) of the block, pi swapping the
//           second and third group of four (0-3, 8-11, 4-7, 12-15): the score product then leaves a lane the
//           probabilities of 8 consecutive keys, which is the order of the values. 16-byte chunk c of a row
//           sits at chunk c ^ swizzle(row), which spreads the 16 rows that 16 lanes read over the banks.
//   values  [4 blocks][DH rows][16 keys], as they lie in a page; the halves of 8 keys of row d swap when
//           (d / 8) is odd, for the banks.
//
// The next tile's loads are issued before the current tile's arithmetic and land in the other buffer;
// a wave waits for its own loads and then for the workgroup's barrier. Positions are clamped into the range
// the workgroup may touch in steps of 16 (a block is fetched from a page that exists, or the nearest one);
// what lies outside a row's range is masked by position, as above.
constexpr bool DMA_HEAD_DIM = DH == 32 || DH == 64 || DH == 128 || DH == 256;
constexpr int KC = DH / 8;                                      // 16-byte chunks of a key row
constexpr int DMA_LOADS = DH / 32 > 0 ? DH / 32 : 1;            // load instructions a wave issues per tile for keys; as many for values
constexpr int K_SWZ_SHIFT = KC >= 16 ? 0 : (KC == 8 ? 1 : 2);   // rows that share 256 bytes: 1, 2 or 4
constexpr int K_SWZ_MASK = (KC < 16 ? KC : 16) - 1;
constexpr int DMA_TILE = 2 * KT * DH;                           // bf16 elements of one buffer: keys, then values
typedef __attribute__((address_space(3))) void ap_lds_void_t;
// Fourth word of a raw buffer descriptor on gfx9-family GPUs: 32-bit float data format, destination
// selects x, y, z, w; no swizzle, no stride.
#define AP_RSRC_FLAGS 0x27000

__device__ __forceinline__ int key_swizzle(int row) { return (row >> K_SWZ_SHIFT) & K_SWZ_MASK; }
__device__ __forceinline__ int key_of_row16(int r) {
  const int g = r >> 2;
  return ((g == 1 ? 2 : (g == 2 ? 1 : g)) << 2) | (r & 3);
}

// One tile of 64 keys for a wave's 32 rows, from the LDS layout above. A function of its own with pointers that
// are promised not to alias: the compiler, which otherwise makes every LDS read wait for all loads into LDS
// that are in flight (here: the next tile's), then leaves the waiting to the kernel's own wait and barrier.
__device__ __forceinline__ void attend_tile_from_lds(const bf16_t* __restrict__ k_lds, const bf16_t* __restrict__ v_lds,
                                                     const Frag (&qf)[KS], floatx16 (&acc)[DT], float& m, float& l,
                                                     const int (&k_frag)[KS], int v_frag, int base, int pos, int lo,
                                                     int hi, bool whole, float scale_log2e) {
  floatx16 sc[2];
  const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Frag a;
      a.u4 = *reinterpret_cast<const uint4*>(k_lds + u * 32 * DH + k_frag[ks]);
      sc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[ks].v, ks == 0 ? zero : sc[u], 0, 0, 0);
    }
  }
  // Element v of sc[u] is key base + u*32 + 16*(v/8) + hi*8 + v%8 against this lane's row (the rows of a
  // block of 16 hold its keys in the order 0-3, 8-11, 4-7, 12-15).
  if (!whole) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int kp = base + u * 32 + 16 * (v / 8) + hi * 8 + (v % 8);
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
  // B operand slot hi*8 + e of 16-key block j holds key j*16 + hi*8 + e: the order of the values.
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      Frag a;
      a.u4 = *reinterpret_cast<const uint4*>(v_lds + j * 16 * DH + dt * 32 * 16 + v_frag);
      acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[j].v, acc[dt], 0, 0, 0);
    }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+v"(acc[dt]));
}

template <int HC, int QC>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_prefill_dma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ items, int num_items, int H, int KVH, int block_size,
    int max_blocks, float scale_log2e, int window, int block_shift, int flip_from, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* lds = reinterpret_cast<bf16_t*>(smem);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TIE_WAVE);
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int r32 = lane & 31;
  const int hi = lane >> 5;
  const int hc = wave / QC, qc = wave % QC;
  const bool flipped = static_cast<int>(blockIdx.y + blockIdx.z * gridDim.y) >= flip_from;
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

  const int rows_end = min(n_new, row0 + 32 * QC);
  if (rows_end <= row0) return;   // uniform for the workgroup
  const int wg_first = window > 0 ? max(0, ctx - n_new + row0 - window + 1) : 0;
  const int wg_last = ctx - n_new + rows_end - 1;

  const int wave_row0 = row0 + qc * 32;
  const bool wave_active = hc < heads_here && wave_row0 < n_new;
  const int i = wave_row0 + r32;
  const bool valid = wave_active && i < n_new;
  const int pos = valid ? ctx - n_new + i : -1;
  const int lo = (window > 0 && valid) ? max(0, pos - window + 1) : 0;
  const int wave_last = wave_active ? ctx - n_new + min(n_new, wave_row0 + 32) - 1 : -1;
  const int wave_min_pos = ctx - n_new + wave_row0;

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
  const bool empty = tile_begin > tile_end;

  // What each lane fetches with load n of a block, as byte offsets into the block's keys and values.
  unsigned k_voff[DMA_LOADS], v_voff[DMA_LOADS];
#pragma unroll
  for (int n = 0; n < DMA_LOADS; ++n) {
    const int chunk = n * 64 + lane;                       // LDS chunk within the block's 16 rows
    const int r16 = chunk / KC, c_lds = chunk % KC;
    k_voff[n] = static_cast<unsigned>(key_of_row16(r16) * DH * 2 + ((c_lds ^ key_swizzle(r16)) * 16));
    const int slot = n * 64 + lane;                        // LDS slot within the block's DH rows of two halves
    const int d = slot >> 1, half = (slot & 1) ^ ((d >> 3) & 1);
    v_voff[n] = static_cast<unsigned>((d * block_size + half * 8) * 2);
  }
  const int first16 = wg_first & ~15, last16 = wg_last & ~15;
  const size_t page_elems = static_cast<size_t>(KVH) * block_size * DH;
  const size_t head_elems = static_cast<size_t>(kvh) * block_size * DH;
  // The page of block `wave` of tile `tile` (a scalar load), looked up one tile before the block is loaded
  // so that no load waits for it.
  auto page_of_block = [&](int tile) { return table[min(max(tile * KT + wave * 16, first16), last16) >> block_shift]; };
  // Block `wave` of tile `tile`, which lies in `page`, into buffer `buf`.
  auto issue = [&](int tile, int buf, int page) {
    const int p16 = min(max(tile * KT + wave * 16, first16), last16);
    const int off = p16 & (block_size - 1);
    const bf16_t* kb = k_cache + static_cast<size_t>(page) * page_elems + head_elems + static_cast<size_t>(off) * DH;
    const bf16_t* vb = v_cache + static_cast<size_t>(page) * page_elems + head_elems + off;
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(kb), 0, 16 * DH * 2, AP_RSRC_FLAGS);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(vb), 0, (DH * block_size - off) * 2, AP_RSRC_FLAGS);
    bf16_t* kdst = lds + buf * DMA_TILE + wave * 16 * DH;
    bf16_t* vdst = lds + buf * DMA_TILE + KT * DH + wave * 16 * DH;
#pragma unroll
    for (int n = 0; n < DMA_LOADS; ++n)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (ap_lds_void_t*)(kdst + n * 512), 16, k_voff[n], 0, 0, 0);
#pragma unroll
    for (int n = 0; n < DMA_LOADS; ++n)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (ap_lds_void_t*)(vdst + n * 512), 16, v_voff[n], 0, 0, 0);
  };
  // Fragment addresses (elements): a key row's chunk ks * 2 + hi sits at that number ^ the row's swizzle.
  const int swz = key_swizzle(r32);
  int k_frag[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_frag[ks] = r32 * DH + (((ks * 2 + hi) ^ swz) * 8);
  const int v_frag = r32 * 16 + ((hi ^ ((r32 >> 3) & 1)) * 8);

  int next_page = 0;
  if (!empty) {
    issue(tile_begin, 0, page_of_block(tile_begin));
    if (tile_begin < tile_end) next_page = page_of_block(tile_begin + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int tile = tile_begin; tile <= tile_end; ++tile) {
    const int buf = (tile - tile_begin) & 1;
    const bf16_t* k_lds = lds + buf * DMA_TILE;
    const bf16_t* v_lds = k_lds + KT * DH;
    if (tile < tile_end) {
      issue(tile + 1, buf ^ 1, next_page);           // that buffer was last read before the barrier below
      if (tile + 1 < tile_end) next_page = page_of_block(tile + 2);
    }

    const int base = tile * KT;
    if (wave_active && base <= wave_last) {
      const bool whole = base + KT - 1 <= wave_min_pos && (window <= 0 || base >= wave_last - window + 1) &&
                         wave_row0 + 32 <= n_new;
      attend_tile_from_lds(k_lds, v_lds, qf, acc, m, l, k_frag, v_frag, base, pos, lo, hi, whole, scale_log2e);
    }
    // My loads of the next tile have landed and my reads of this one are done; after the barrier that holds
    // for every wave.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
  }

  l += __shfl_xor(l, 32, TIE_WAVE);
  if (!valid) return;
  if (nsplit > 1) {
    const size_t slot = (static_cast<size_t>(qs + i) * H + head0 + hc) * nsplit + split;
    float* po = part_o + slot * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq)
        *reinterpret_cast<float4*>(po + dt * 32 + 8 * vq + hi * 4) =
            make_float4(acc[dt][vq * 4], acc[dt][vq * 4 + 1], acc[dt][vq * 4 + 2], acc[dt][vq * 4 + 3]);
    if (hi == 0) {
      part_ml[slot * 2] = m * scale_log2e;
      part_ml[slot * 2 + 1] = l;
    }
    return;
  }
  const float inv = 1.0f / l;
  bf16_t* o = out + (static_cast<size_t>(qs + i) * H + head0 + hc) * DH;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq)
      *reinterpret_cast<uint2*>(o + dt * 32 + 8 * vq + hi * 4) =
          make_uint2(pack2(acc[dt][vq * 4] * inv, acc[dt][vq * 4 + 1] * inv),
                     pack2(acc[dt][vq * 4 + 2] * inv, acc[dt][vq * 4 + 3] * inv));
#endif
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

template <int HC, int QC>
static int launch_prefill_dma(const dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k_cache,
                              const bf16_t* v_cache, bf16_t* out, const int* query_start, const int* context_lens,
                              const int* block_tables, const int* items, int num_items, int H, int KVH,
                              int block_size, int max_blocks, float scale_log2e, int window, int nsplit,
                              float* part_o, float* part_ml) {
  const int block_shift = __builtin_ctz(block_size);
  const long planes = static_cast<long>(grid.y) * grid.z;
  const int flip_from = (nsplit == 1 && planes >= 2 && planes * grid.x <= 2L * compute_units())
                            ? static_cast<int>(planes / 2) : 0x7fffffff;
  constexpr size_t lds_bytes = 2 * static_cast<size_t>(DMA_TILE) * sizeof(bf16_t);
  static bool configured = false;
  if (!configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_dma_kernel<HC, QC>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (e != hipSuccess) return static_cast<int>(e);
    configured = true;
  }
  attention_prefill_dma_kernel<HC, QC><<<grid, THREADS, lds_bytes, stream>>>(
      q, k_cache, v_cache, out, query_start, context_lens, block_tables, items, num_items, H, KVH, block_size,
      max_blocks, scale_log2e, window, block_shift, flip_from, nsplit, part_o, part_ml);
  return tie_launch_status();
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
// staging: 0 = by the rule, 1 = tiles copied through registers (any page size and head size), 2 = tiles loaded
// straight into LDS (pages of 16 positions or more, head sizes 32, 64, 128, 256; refused otherwise).
extern "C" int tie_attention_prefill_bf16_with(const void* q, const void* k_cache, const void* v_cache, void* out,
                                               const int* query_start, const int* context_lens,
                                               const int* block_tables, const int* items, int num_items, int H,
                                               int KVH, int block_size, int max_blocks, float scale, int window,
                                               int nsplit, float* part_o, float* part_ml, const int* merge_rows,
                                               int num_merge_rows, int staging, hipStream_t stream) {
  if (num_items <= 0 || H <= 0 || KVH <= 0 || KVH > 65535 || H % KVH != 0 || block_size < 4 ||
      (block_size & (block_size - 1)) != 0 || max_blocks <= 0 || !(scale > 0.f) || nsplit < 1 ||
      nsplit > MERGE_MAX_SPLITS)   // the running maximum is kept on unscaled scores
    return TIE_BAD_ARGUMENT;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr || merge_rows == nullptr || num_merge_rows <= 0 ||
                     num_merge_rows > 65535))
    return TIE_BAD_ARGUMENT;
  const bool dma_takes = DMA_HEAD_DIM && block_size >= 16;
  if (staging < 0 || staging > 2 || (staging == 2 && !dma_takes)) return TIE_BAD_ARGUMENT;
  const bool dma = staging == 2 || (staging == 0 && dma_takes);
  const int G = H / KVH;
  int hc, qc;
  shape_for_group(G, &hc, &qc);
  const int passes = (G + hc - 1) / hc;
  if (passes > 65535) return TIE_BAD_ARGUMENT;
  const dim3 grid(num_items * nsplit, KVH, passes);
  const float scale_log2e = scale * 1.44269504088896340736f;
  int status;
#define LAUNCH_DMA(HC, QC)                                                                                        \
  status = launch_prefill_dma<HC, QC>(                                                                            \
      grid, stream, static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_cache),                           \
      static_cast<const bf16_t*>(v_cache), static_cast<bf16_t*>(out), query_start, context_lens, block_tables,    \
      items, num_items, H, KVH, block_size, max_blocks, scale_log2e, window, nsplit, part_o, part_ml)
#define LAUNCH(HC, QC)                                                                                            \
  status = (block_size % 8 == 0 ? launch_prefill<HC, QC, true> : launch_prefill<HC, QC, false>)(                  \
      grid, stream, static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_cache),                           \
      static_cast<const bf16_t*>(v_cache), static_cast<bf16_t*>(out), query_start, context_lens, block_tables,    \
      items, num_items, H, KVH, block_size, max_blocks, scale_log2e, window, nsplit, part_o, part_ml)
  if (dma) {
    if constexpr (DMA_HEAD_DIM) {
      if (hc == 4) LAUNCH_DMA(4, 1);
      else if (hc == 3) LAUNCH_DMA(3, 1);
      else if (hc == 2) LAUNCH_DMA(2, 2);
      else LAUNCH_DMA(1, 4);
    } else {
      return TIE_BAD_ARGUMENT;
    }
  } else if (hc == 4) LAUNCH(4, 1);
  else if (hc == 3) LAUNCH(3, 1);
  else if (hc == 2) LAUNCH(2, 2);
  else LAUNCH(1, 4);
#undef LAUNCH
#undef LAUNCH_DMA
  if (status != TIE_OK || nsplit == 1) return status;
  launch_attention_merge(part_o, part_ml, static_cast<bf16_t*>(out), merge_rows, nullptr, nullptr, H, nsplit,
                         num_merge_rows, stream);
  return tie_launch_status();
}

extern "C" int tie_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                          const int* query_start, const int* context_lens, const int* block_tables,
                                          const int* items, int num_items, int H, int KVH, int block_size,
                                          int max_blocks, float scale, int window, int nsplit, float* part_o,
                                          float* part_ml, const int* merge_rows, int num_merge_rows,
                                          hipStream_t stream) {
  return tie_attention_prefill_bf16_with(q, k_cache, v_cache, out, query_start, context_lens, block_tables, items,
                                         num_items, H, KVH, block_size, max_blocks, scale, window, nsplit, part_o,
                                         part_ml, merge_rows, num_merge_rows, 0, stream);
}
