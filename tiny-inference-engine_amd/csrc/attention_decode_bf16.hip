// Paged attention for decoded tokens (one new row per sequence) on the gfx950 matrix cores,
// bfloat16 queries and cache, float32 softmax. Compiled per head size: -DHEAD_DIM=<multiple of 16>.
//
// One wave handles one (sequence, KV head, split of the keys). The G = H / KVH query heads that
// share the KV head are the 16 columns of the MFMA tiles (columns >= G are zeros), so keys and
// values are read once for the whole group. Per 32 keys:
//
//   S^T[key, g] = K[key, :] . Q[g, :]      A = K rows (16 bytes a lane, straight from the cache),
//                                          B = Q (held in registers)          2 x HEAD_DIM/32 MFMAs
//   online softmax per column g in float32: running maximum, sum, rescale of the accumulator
//   O^T[d, g]  += V^T[d, key] . P^T[key, g]   A = V^T rows (the cache keeps values transposed inside a
//                                          page, so 8 positions of one dimension are 16 bytes),
//                                          B = P, which is exactly what the lane already holds
//                                          from the first product              HEAD_DIM/16 MFMAs
//
// Nothing passes through LDS and no lane ever needs another lane's scores. Splits of the keys
// run as separate waves; a second kernel merges their (maximum, sum, accumulator) triples in a
// fixed order. Keys are always cut at multiples of 32 positions, so what is computed for a
// position does not depend on the batch around it. Block-table lookups run two tiles ahead of the
// arithmetic and the data loads one tile ahead, so neither waits for the other.
//
// Formula: src/backend/cpu/cpu_backend.cpp:261-319 (score = scale * q.k, causal by position,
// online softmax, query head h reads KV head h / (H / KVH)).
#include "common.h"
#include "qk_prepare.h"

#include <math.h>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int DH = HEAD_DIM;
constexpr int KSTEPS = (DH + 31) / 32;  // k blocks of the first product
constexpr int DTILES = DH / 16;         // row tiles of the second product

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // native vectors: fragments stay in registers
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ bf16x8_t frag(u32x4_t v) { return *reinterpret_cast<const bf16x8_t*>(&v); }

// One tile of 32 keys for the 16 columns of a wave: scores, online softmax in float32, values. kf: the keys'
// fragments of the two 16-key sub-tiles, vf: the values' fragments, qf: the queries. Shared by the kernels
// below, so that a position's result does not depend on which of them ran.
__device__ __forceinline__ void attend_tile(const u32x4_t (&kf)[2][KSTEPS], const u32x4_t (&vf)[DTILES],
                                            const u32x4_t (&qf)[KSTEPS], floatx4 (&acc)[DTILES], float& m, float& l,
                                            int base, int start, int pos, int quad, float scale_log2e) {
  // ---- first product: two 16-key sub-tiles
  floatx4 sc[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    sc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st)
      sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag(kf[u][st]), frag(qf[st]), sc[u], 0, 0, 0);
  }
  // ---- softmax of this lane's column over its 8 keys (quad * 8 + u * 4 + v), then across the four quads.
  // Scores stay unscaled; scale * log2(e) > 0 enters in the exponent: p = 2^(s c - m c).
  float sv[8];
  float tile_max = -INFINITY;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int kp = base + quad * 8 + u * 4 + v;
      const float x = (kp <= pos && kp >= start) ? sc[u][v] : -INFINITY;
      sv[u * 4 + v] = x;
      tile_max = fmaxf(tile_max, x);
    }
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, TIE_WAVE));
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, TIE_WAVE));
  const float m_new = fmaxf(m, tile_max);
  const float neg_mc = (m_new == -INFINITY) ? 0.f : -m_new * scale_log2e;
  const float corr = __builtin_amdgcn_exp2f(fmaf(m, scale_log2e, neg_mc));   // m = -inf: 0
  u32x4_t pf;
  float psum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const float p0 = __builtin_amdgcn_exp2f(fmaf(sv[i], scale_log2e, neg_mc));       // masked: 0
    const float p1 = __builtin_amdgcn_exp2f(fmaf(sv[i + 1], scale_log2e, neg_mc));
    psum += p0;
    psum += p1;
    pf[i / 2] = pack_bf16x2(p0, p1);
  }
  l = l * corr + psum;
  m = m_new;
  // ---- second product
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[dt][v] *= corr;
    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag(vf[dt]), frag(pf), acc[dt], 0, 0, 0);
  }
}

// What a wave leaves when its keys are done: the output row itself with one share, else its (maximum, sum,
// accumulator) for the merge. h: the query head of this lane's column, z: the sequence's place in the launch.
__device__ __forceinline__ void store_share(const floatx4 (&acc)[DTILES], float m, float l, bf16_t* __restrict__ out,
                                            float* __restrict__ part_o, float* __restrict__ part_ml, int t, int z,
                                            int h, int H, int quad, int nsplit, int split, float scale_log2e) {
  if (nsplit == 1) {  // no merge needed: normalise and store
    bf16_t* o = out + (static_cast<size_t>(t) * H + h) * DH;
    const float inv = 1.0f / l;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
      *reinterpret_cast<u32x2_t*>(o + dt * 16 + quad * 4) =
          u32x2_t{pack_bf16x2(acc[dt][0] * inv, acc[dt][1] * inv), pack_bf16x2(acc[dt][2] * inv, acc[dt][3] * inv)};
    return;
  }
  const size_t slot = (static_cast<size_t>(z) * H + h) * nsplit + split;
  float* po = part_o + slot * DH;
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt)
    *reinterpret_cast<float4*>(po + dt * 16 + quad * 4) = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
  if (quad == 0) {
    part_ml[slot * 2] = m * scale_log2e;     // the merge works in the exponent's units (base 2)
    part_ml[slot * 2 + 1] = l;
  }
}

// Keys of a 32-key tile are taken in runs of 8: row r of 16-key sub-tile u is key (r / 4) * 8 + u * 4 + r % 4
// of the tile. The scores a lane then holds (rows quad * 4 + v of both sub-tiles) are those of the 8
// consecutive keys quad * 8 .. + 7, which is also how the values of one dimension lie in a page: with
// WIDE (block sizes in steps of 8) a lane reads them in one 16-byte piece.
template <bool WIDE>
__global__ __launch_bounds__(TIE_WAVE) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ seq_ids, int H, int KVH, int block_size,
    int block_shift, int max_blocks, float scale_log2e, int window, int nsplit) {
  const int lane = threadIdx.x;
  const int col = lane & 15;   // query head within the group (column of every tile)
  const int quad = lane >> 4;  // 0..3
  const int split = blockIdx.x;
  const int kvh = blockIdx.y;
  const int s = seq_ids ? seq_ids[blockIdx.z] : blockIdx.z;
  const int G = H / KVH;
  const int t = query_start[s];            // the sequence's single new row
  const int pos = context_lens[s] - 1;     // its position; keys start..pos are read
  const int start = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  // Tiles of 32 keys at absolute positions; this split's share of them.
  const int first_tile = start / 32;
  const int num_tiles = pos / 32 + 1;
  const int per_split = (num_tiles - first_tile + nsplit - 1) / nsplit;
  const int tile_begin = first_tile + split * per_split;
  const int tile_end = min(num_tiles, tile_begin + per_split);

  // Q as the B operand: lane (col = g, quad) holds Q[g][step*32 + quad*8 .. +8].
  u32x4_t qf[KSTEPS];
  {
    const bool valid = col < G;
    const bf16_t* qr = q + (static_cast<size_t>(t) * H + static_cast<size_t>(kvh) * G + (valid ? col : 0)) * DH;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      const int d = st * 32 + quad * 8;
      qf[st] = (valid && d < DH) ? *reinterpret_cast<const u32x4_t*>(qr + d) : u32x4_t{0, 0, 0, 0};
    }
  }

  floatx4 acc[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const size_t page_stride = static_cast<size_t>(KVH) * block_size * DH;   // elements of one page, K or V
  const size_t head_off = static_cast<size_t>(kvh) * block_size * DH;
  // Positions are clamped into [start, pos] for addresses only (pages outside that range may be gone or
  // never have been there); what lies outside is masked in the softmax.
  auto page_of = [&](int kp) { return kp >> block_shift; };          // block sizes are powers of two here
  auto offset_of = [&](int kp) { return kp & (block_size - 1); };
  // This lane's keys of a tile: rows of the two sub-tiles, and the runs of values it reads.
  const int krow0 = (col >> 2) * 8 + (col & 3);        // sub-tile 1: + 4
  constexpr int VG = WIDE ? 8 : 4;

  // Pages first, one tile further ahead than the data, so that no data load waits for a lookup.
  struct Pages { int k[2]; int v[WIDE ? 1 : 2]; };
  auto lookup = [&](int base, Pages& pg) {
#pragma unroll
    for (int u = 0; u < 2; ++u) pg.k[u] = table[page_of(min(max(base + krow0 + u * 4, start), pos))];
#pragma unroll
    for (int j = 0; j < (WIDE ? 1 : 2); ++j)
      pg.v[j] = table[page_of(min(max(base + quad * 8 + j * 4, start / VG * VG), pos / VG * VG))];
  };
  auto load_keys = [&](int base, const Pages& pg, u32x4_t (&kf)[2][KSTEPS]) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = min(max(base + krow0 + u * 4, start), pos);
      const bf16_t* kr = k_cache + static_cast<size_t>(pg.k[u]) * page_stride + head_off +
                         static_cast<size_t>(offset_of(kp)) * DH;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        const int d = st * 32 + quad * 8;
        kf[u][st] = d < DH ? __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kr + d)) : u32x4_t{0, 0, 0, 0};
      }
    }
  };
  auto load_values = [&](int base, const Pages& pg, u32x4_t (&vf)[DTILES]) {
    const bf16_t* vp[WIDE ? 1 : 2];
#pragma unroll
    for (int j = 0; j < (WIDE ? 1 : 2); ++j) {
      const int kp = min(max(base + quad * 8 + j * 4, start / VG * VG), pos / VG * VG);
      vp[j] = v_cache + static_cast<size_t>(pg.v[j]) * page_stride + head_off + offset_of(kp);
    }
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
      const size_t d_off = static_cast<size_t>(dt * 16 + col) * block_size;
      if (WIDE) {
        vf[dt] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vp[0] + d_off));
      } else {
        const u32x2_t h0 = *reinterpret_cast<const u32x2_t*>(vp[0] + d_off);
        const u32x2_t h1 = *reinterpret_cast<const u32x2_t*>(vp[WIDE ? 0 : 1] + d_off);
        vf[dt] = u32x4_t{h0.x, h0.y, h1.x, h1.y};
      }
    }
  };

  // The loads of tile t + 1 are issued before the arithmetic of tile t, so memory latency and the
  // matrix cores overlap; the pages of tile t + 2 are looked up at the same time.
  u32x4_t kf[2][KSTEPS], vf[DTILES], kf_next[2][KSTEPS], vf_next[DTILES];
  Pages pages;
  if (tile_begin < tile_end) {
    lookup(tile_begin * 32, pages);
    load_keys(tile_begin * 32, pages, kf_next);
    load_values(tile_begin * 32, pages, vf_next);
    if (tile_begin + 1 < tile_end) lookup(tile_begin * 32 + 32, pages);
  }
  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const int base = tile * 32;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) kf[u][st] = kf_next[u][st];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) vf[dt] = vf_next[dt];
    if (tile + 1 < tile_end) {
      load_keys(base + 32, pages, kf_next);
      load_values(base + 32, pages, vf_next);
      if (tile + 2 < tile_end) lookup(base + 64, pages);
    }
    attend_tile(kf, vf, qf, acc, m, l, base, start, pos, quad, scale_log2e);
  }

  // The column's sum over all keys of this split.
  l += __shfl_xor(l, 16, TIE_WAVE);
  l += __shfl_xor(l, 32, TIE_WAVE);
  if (col >= G) return;
  store_share(acc, m, l, out, part_o, part_ml, t, blockIdx.z, kvh * G + col, H, quad, nsplit, split, scale_log2e);
}

// The same for pages of 16 positions or more, with DEPTH - 1 tiles in flight behind the one that is computed.
// The kernel above asks for a tile's data after it has waited for the lookup of its pages, and the counter of
// outstanding vector loads runs in order: waiting for a lookup waits for every data load issued before it, so
// a wave never has more than one tile (16 KB at head size 128) on its way and its time is one memory latency
// a tile. Here a half tile of 16 positions lies in one page, so the two page numbers of a tile are the same
// for all lanes and come by scalar loads, which have a counter of their own; the tiles live in a ring of
// DEPTH register sets that is walked with constant indices, so no set is copied (a copy would wait for its
// loads). The arithmetic of a tile and the order of the tiles are those of the kernel above: the same bits.
//
// PREPARE: the kernel makes its queries itself from the projection's planes of partial sums (sum, per-head RMS
// norm, rotation by the step's table of angles: the q/k kernel's own functions, so the same bits), every wave
// those of its KV head's group, through LDS into the operand layout; and the wave whose share holds the
// sequence's newest position first makes that token's key and value and writes them into the cache, waits
// for the stores, and only then reads its tiles. One kernel less a layer; head sizes 32 to 256 in powers of
// two (head_dim / 8 lanes a head).
struct QkSource {
  const float* qkv;        // [planes][rows][in_row] float32: q heads, k heads, v heads of a row
  size_t plane_stride;
  int planes;
  int in_row;
  const float* q_weight;   // per-head norm weights, or null for no norm
  const float* k_weight;
  float eps;
  const float* angles;     // [rows][DH]: cos of the DH / 2 angles, then sin
  int write_kv;            // 0: the cache holds the newest token already (another layer's cache)
};

template <int DEPTH, bool PREPARE>
__global__ __launch_bounds__(TIE_WAVE) void attention_decode_ring_kernel(
    const bf16_t* __restrict__ q, bf16_t* k_cache, bf16_t* v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ query_start, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, const int* __restrict__ seq_ids, int H, int KVH, int block_size,
    int block_shift, int max_blocks, float scale_log2e, int window, int nsplit, const int* __restrict__ share_tiles,
    QkSource src) {
  const int lane = threadIdx.x;
  const int col = lane & 15;
  const int quad = lane >> 4;
  // Workgroups go to the eight XCDs in turn by their number, of which the share is the fastest part: with shares
  // of one length, where the later shares of most sequences are empty, share j is therefore given to another
  // workgroup of the sequence's eight from pair to pair, or a few XCDs would carry all the work.
  const int split = share_tiles != nullptr ? static_cast<int>((blockIdx.x + blockIdx.y + blockIdx.z) % gridDim.x)
                                           : static_cast<int>(blockIdx.x);
  const int kvh = blockIdx.y;
  const int s = seq_ids ? seq_ids[blockIdx.z] : blockIdx.z;
  const int G = H / KVH;
  const int t = query_start[s];
  const int pos = context_lens[s] - 1;
  const int start = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_tables + static_cast<size_t>(s) * max_blocks;

  const int first_tile = start / 32;
  const int num_tiles = pos / 32 + 1;
  // A share is the nsplit-th part of this sequence's tiles, or, where the step names a length for all shares
  // (share_tiles, in tiles; sequences of very different lengths), that many tiles if it is more: a short sequence
  // then fills fewer shares, the others are empty (the merge gives them no weight), and every wave that works
  // walks about as many keys. Whatever the step names, the shares cover the sequence.
  int per_split = (num_tiles - first_tile + nsplit - 1) / nsplit;
  if (share_tiles != nullptr) per_split = max(per_split, *share_tiles);
  const int tile_begin = first_tile + split * per_split;
  const int tile_end = min(num_tiles, tile_begin + per_split);
  if (share_tiles != nullptr && tile_begin >= tile_end) {
    // An empty share leaves at once: a maximum of -inf gives it no weight, and the merge does not read the rest.
    if (quad == 0 && col < G) {
      const size_t slot = (static_cast<size_t>(blockIdx.z) * H + kvh * G + col) * nsplit + split;
      part_ml[slot * 2] = -INFINITY;
      part_ml[slot * 2 + 1] = 0.f;
    }
    return;
  }

  const size_t page_stride = static_cast<size_t>(KVH) * block_size * DH;
  const size_t head_off = static_cast<size_t>(kvh) * block_size * DH;
  u32x4_t qf[KSTEPS];
  // PREPARE: the wave whose share ends the sequence takes the newest token from the projection itself: it makes
  // the token's key and value, sends them to the cache for later steps, keeps them (as the cache will hold
  // them, in bfloat16) in LDS, leaves the newest position out of its last tile and attends to it by itself
  // after the loop. Nothing it reads from the cache was written in this launch.
  const bool takes_newest = PREPARE && src.write_kv && tile_end == num_tiles && tile_begin < tile_end;
  const int last_cached = takes_newest ? pos - 1 : pos;     // the newest position the tiles may show
  __shared__ __attribute__((aligned(16))) bf16_t newest_lds[PREPARE ? 2 * DH : 8];   // key, then value
  if constexpr (PREPARE) {
  } else {
    const bool valid = col < G;
    const bf16_t* qr = q + (static_cast<size_t>(t) * H + static_cast<size_t>(kvh) * G + (valid ? col : 0)) * DH;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      const int d = st * 32 + quad * 8;
      qf[st] = (valid && d < DH) ? *reinterpret_cast<const u32x4_t*>(qr + d) : u32x4_t{0, 0, 0, 0};
    }
  }
  floatx4 acc[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const int krow0 = (col >> 2) * 8 + (col & 3);
  const bool keys_in_upper_half = krow0 >= 16;      // both sub-tiles' rows (krow0, krow0 + 4) lie in one half
  const bool values_in_upper_half = quad >= 2;      // positions quad * 8 .. + 7
  const int in_page = block_size - 1;
  const size_t dim_off = static_cast<size_t>(col) * block_size;

  struct Tile { u32x4_t k[2][KSTEPS]; u32x4_t v[DTILES]; };
  // Positions are clamped into [start, pos] for addresses only; a clamped position stays in its half of 16.
  auto issue = [&](int tile, Tile& tl) {
    const int base = tile * 32;
    const int page_lo = table[min(max(base, start), pos) >> block_shift];
    const int page_hi = table[min(max(base + 16, start), pos) >> block_shift];
    const bf16_t* kpage = k_cache + static_cast<size_t>(keys_in_upper_half ? page_hi : page_lo) * page_stride + head_off;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = min(max(base + krow0 + u * 4, start), pos);
      const bf16_t* kr = kpage + static_cast<size_t>(kp & in_page) * DH;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        // Every load is issued whatever the lane (a load under a lane's condition makes the count of loads
        // in flight unknown to the compiler, which then waits for all of them): a head size that is no
        // multiple of 32 reads its last step's upper pieces from the row's start and drops them.
        const int d = st * 32 + quad * 8;
        const bool inside = DH % 32 == 0 || d < DH;
        const u32x4_t piece = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kr + (inside ? d : 0)));
        tl.k[u][st] = inside ? piece : u32x4_t{0, 0, 0, 0};
      }
    }
    const int vp = min(max(base + quad * 8, start / 8 * 8), pos / 8 * 8);
    const bf16_t* vr = v_cache + static_cast<size_t>(values_in_upper_half ? page_hi : page_lo) * page_stride + head_off +
                       (vp & in_page) + dim_off;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
      tl.v[dt] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vr + static_cast<size_t>(dt) * 16 * block_size));
  };

  // Tile i of the wave lives in set i % DEPTH. The groups of DEPTH tiles in the middle issue and compute
  // without a condition, so the compiler knows how many loads are in flight and waits for the oldest tile
  // only; the first DEPTH - 1 tiles before and the last 2 DEPTH - 2 at most after them are issued under
  // conditions, where it waits for more than it must.
  Tile ring[DEPTH];
#pragma unroll
  for (int j = 0; j < DEPTH - 1; ++j)
    if (tile_begin + j < tile_end) issue(tile_begin + j, ring[j]);
  if constexpr (PREPARE) {
    // After the first tiles' loads are on their way: the group's queries, HEADS_AT_ONCE heads at a time with a
    // head's lanes together, and the newest key (lanes 0 .. LPH - 1) and value (the next LPH lanes).
    constexpr int LPH = DH / 8, HALF = DH / 2, HEADS_AT_ONCE = TIE_WAVE / LPH;
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[16 * DH];
    const float* row = src.qkv + static_cast<size_t>(t) * src.in_row;
    const float* angles = src.angles + static_cast<size_t>(t) * DH;
    const int p0 = (lane % LPH) * 4;
    // All loads first, so that they share one trip to memory: the first HEADS_AT_ONCE query heads (lanes beyond
    // the group read its last head again) and, in the wave that takes the newest token, its key (the lanes
    // of even heads-worth) or value (odd), 4 + 4 elements a lane like a query's.
    const int g_first = lane / LPH;
    const float* q_in = row + (static_cast<size_t>(kvh) * G + min(g_first, G - 1)) * DH;
    qk_f4_t qa = load4_planes(q_in + p0, src.plane_stride, src.planes);
    qk_f4_t qb = load4_planes(q_in + HALF + p0, src.plane_stride, src.planes);
    qk_f4_t na = {0.f, 0.f, 0.f, 0.f}, nb = na;
    const bool value_lane = (g_first & 1) != 0;
    if (takes_newest) {
      const float* n_in = row + static_cast<size_t>(H + kvh + (value_lane ? KVH : 0)) * DH;
      na = load4_planes(n_in + p0, src.plane_stride, src.planes);
      nb = load4_planes(n_in + HALF + p0, src.plane_stride, src.planes);
    }
    if (g_first < G) {
      if (src.q_weight != nullptr) qk_head_norm<LPH>(qa, qb, src.q_weight, src.eps, p0);
      qk_f4_t o1, o2;
      qk_rotate_by_table<LPH>(qa, qb, angles, p0, o1, o2);
      store4(q_lds + g_first * DH + p0, o1);
      store4(q_lds + g_first * DH + HALF + p0, o2);
    }
    if (takes_newest) {
      const int page = table[pos >> block_shift];
      const int off = pos & (block_size - 1);
      if (lane < LPH) {
        if (src.k_weight != nullptr) qk_head_norm<LPH>(na, nb, src.k_weight, src.eps, p0);
        qk_f4_t o1, o2;
        qk_rotate_by_table<LPH>(na, nb, angles, p0, o1, o2);
        bf16_t* dst = k_cache + static_cast<size_t>(page) * page_stride + head_off + static_cast<size_t>(off) * DH;
        store4(dst + p0, o1);
        store4(dst + HALF + p0, o2);
        store4(newest_lds + p0, o1);
        store4(newest_lds + HALF + p0, o2);
      } else if (lane < 2 * LPH) {
        // In a page the dimensions of a value lie block_size apart.
        bf16_t* dst = v_cache + static_cast<size_t>(page) * page_stride + head_off + off;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          store_from_float(dst + static_cast<size_t>(p0 + j) * block_size, na[j]);
          store_from_float(dst + static_cast<size_t>(HALF + p0 + j) * block_size, nb[j]);
        }
        store4(newest_lds + DH + p0, na);
        store4(newest_lds + DH + HALF + p0, nb);
      }
    }
    for (int g0 = HEADS_AT_ONCE; g0 < G; g0 += HEADS_AT_ONCE) {
      const int g = g0 + lane / LPH;
      if (g < G) {
        const float* in = row + (static_cast<size_t>(kvh) * G + g) * DH;
        qk_f4_t a = load4_planes(in + p0, src.plane_stride, src.planes);
        qk_f4_t b = load4_planes(in + HALF + p0, src.plane_stride, src.planes);
        if (src.q_weight != nullptr) qk_head_norm<LPH>(a, b, src.q_weight, src.eps, p0);
        qk_f4_t o1, o2;
        qk_rotate_by_table<LPH>(a, b, angles, p0, o1, o2);
        store4(q_lds + g * DH + p0, o1);
        store4(q_lds + g * DH + HALF + p0, o2);
      }
    }
    __syncthreads();   // one wave: the writes above are done before the reads below
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      const int d = st * 32 + quad * 8;
      qf[st] = (col < G && d < DH) ? *reinterpret_cast<const u32x4_t*>(q_lds + col * DH + d) : u32x4_t{0, 0, 0, 0};
    }
  }
  int tile = tile_begin;
  for (; tile + 2 * DEPTH - 2 < tile_end; tile += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      issue(tile + j + DEPTH - 1, ring[(j + DEPTH - 1) % DEPTH]);
      attend_tile(ring[j].k, ring[j].v, qf, acc, m, l, (tile + j) * 32, start, last_cached, quad, scale_log2e);
    }
  }
#pragma unroll
  for (int j = 0; j < 2 * DEPTH - 2; ++j) {
    if (tile + j < tile_end) {
      if (j < DEPTH - 1 && tile + j + DEPTH - 1 < tile_end) issue(tile + j + DEPTH - 1, ring[(j + DEPTH - 1) % DEPTH]);
      attend_tile(ring[j % DEPTH].k, ring[j % DEPTH].v, qf, acc, m, l, (tile + j) * 32, start, last_cached, quad,
                    scale_log2e);
    }
  }

  if constexpr (PREPARE) {
    if (takes_newest) {
      // The newest key by itself: its score for this lane's column from the 32 dimensions the lane holds of the
      // query, summed over the four quads; then one step of the online softmax with a single key, the
      // probability rounded to bfloat16 as the tiles' are.
      float dot = 0.f;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        const int d = st * 32 + quad * 8;
        if (DH % 32 == 0 || d < DH) {
          const u32x4_t kq = *reinterpret_cast<const u32x4_t*>(newest_lds + d);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            dot = fmaf(__uint_as_float(qf[st][e] << 16), __uint_as_float(kq[e] << 16), dot);
            dot = fmaf(__uint_as_float(qf[st][e] & 0xffff0000u), __uint_as_float(kq[e] & 0xffff0000u), dot);
          }
        }
      }
      dot += __shfl_xor(dot, 16, TIE_WAVE);
      dot += __shfl_xor(dot, 32, TIE_WAVE);
      const float m_new = fmaxf(m, dot);
      const float neg_mc = -m_new * scale_log2e;
      const float corr = __builtin_amdgcn_exp2f(fmaf(m, scale_log2e, neg_mc));   // m = -inf: 0
      const float p = __builtin_amdgcn_exp2f(fmaf(dot, scale_log2e, neg_mc));
      const float p_rounded = __uint_as_float(pack_bf16x2(p, 0.f) << 16);
      l = l * corr + (quad == 0 ? p : 0.f);
      m = m_new;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
        const u32x2_t vv = *reinterpret_cast<const u32x2_t*>(newest_lds + DH + dt * 16 + quad * 4);
        acc[dt][0] = fmaf(p_rounded, __uint_as_float(vv.x << 16), acc[dt][0] * corr);
        acc[dt][1] = fmaf(p_rounded, __uint_as_float(vv.x & 0xffff0000u), acc[dt][1] * corr);
        acc[dt][2] = fmaf(p_rounded, __uint_as_float(vv.y << 16), acc[dt][2] * corr);
        acc[dt][3] = fmaf(p_rounded, __uint_as_float(vv.y & 0xffff0000u), acc[dt][3] * corr);
      }
    }
  }
  l += __shfl_xor(l, 16, TIE_WAVE);
  l += __shfl_xor(l, 32, TIE_WAVE);
  if (col >= G) return;
  store_share(acc, m, l, out, part_o, part_ml, t, blockIdx.z, kvh * G + col, H, quad, nsplit, split, scale_log2e);
}

#include "attention_merge.h"

extern "C" int tie_attention_decode_head_dim() { return DH; }
extern "C" int tie_attention_max_splits() { return MERGE_MAX_SPLITS; }

constexpr bool PREPARE_HEAD_DIM = DH == 32 || DH == 64 || DH == 128 || DH == 256;

static int launch_decode(const bf16_t* q, const QkSource* src, bf16_t* k_cache, bf16_t* v_cache, bf16_t* out,
                         float* part_o, float* part_ml, const int* query_start, const int* context_lens,
                         const int* block_tables, const int* seq_ids, int num_seqs, int H, int KVH, int block_size,
                         int max_blocks, float scale, int window, int nsplit, const int* share_tiles, int depth,
                         hipStream_t stream) {
  if (num_seqs <= 0 || num_seqs > 65535 || H <= 0 || KVH <= 0 || KVH > 65535 || H % KVH != 0 || H / KVH > 16 ||
      block_size < 4 || (block_size & (block_size - 1)) != 0 || max_blocks <= 0 || nsplit <= 0 ||
      nsplit > MERGE_MAX_SPLITS || depth < 0 || depth > 4 || (depth > 1 && block_size < 16) ||
      !(scale > 0.f))   // the running maximum is kept on unscaled scores
    return TIE_BAD_ARGUMENT;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr)) return TIE_BAD_ARGUMENT;
  // Measured: the ring of three register sets where the keys are cut into shares, of four where a wave walks
  // a whole sequence.
  if (depth == 0) depth = block_size < 16 ? 1 : (nsplit == 1 ? 4 : 3);
  if (src != nullptr && (depth < 2 || !PREPARE_HEAD_DIM)) return TIE_BAD_ARGUMENT;
  if (share_tiles != nullptr && (depth < 2 || nsplit == 1)) return TIE_BAD_ARGUMENT;   // the ring kernel's, with a merge
  const dim3 grid(nsplit, KVH, num_seqs);
  const int block_shift = __builtin_ctz(block_size);
  const float scale_log2e = scale * 1.44269504088896340736f;
#define ARGS out, part_o, part_ml, query_start, context_lens, block_tables, seq_ids, H, KVH, block_size, block_shift, \
             max_blocks, scale_log2e, window, nsplit
#define LAUNCH_RING(DEPTH)                                                                                   \
  {                                                                                                          \
    if (src == nullptr) {                                                                                    \
      attention_decode_ring_kernel<DEPTH, false><<<grid, TIE_WAVE, 0, stream>>>(q, k_cache, v_cache, ARGS,   \
                                                                                share_tiles, QkSource{});    \
    } else if constexpr (PREPARE_HEAD_DIM) {                                                                 \
      attention_decode_ring_kernel<DEPTH, true><<<grid, TIE_WAVE, 0, stream>>>(q, k_cache, v_cache, ARGS,    \
                                                                               share_tiles, *src);           \
    }                                                                                                        \
  }
  if (depth == 4) LAUNCH_RING(4)
  else if (depth == 3) LAUNCH_RING(3)
  else if (depth == 2) LAUNCH_RING(2)
  else if (block_size % 8 == 0) attention_decode_kernel<true><<<grid, TIE_WAVE, 0, stream>>>(q, k_cache, v_cache, ARGS);
  else attention_decode_kernel<false><<<grid, TIE_WAVE, 0, stream>>>(q, k_cache, v_cache, ARGS);
#undef LAUNCH_RING
#undef ARGS
  int status = tie_launch_status();
  if (status != TIE_OK || nsplit == 1) return status;
  launch_attention_merge(part_o, part_ml, out, nullptr, query_start, seq_ids, H, nsplit, num_seqs, stream);
  return tie_launch_status();
}

// depth: 0 = by the rule, 1 = the kernel that looks its pages up per lane (any page size), 2 to 4 = the ring
// kernel with that many register sets (pages of 16 positions or more); for tests and sweeps.
// share_tiles (or null): one int on the device, the tiles of 32 keys of a share where the sequences' lengths differ
// much (the ring kernel and more than one share only; 0 there means shares by each sequence's own length).
extern "C" int tie_attention_decode_bf16_with(const void* q, const void* k_cache, const void* v_cache, void* out,
                                              float* part_o, float* part_ml, const int* query_start,
                                              const int* context_lens, const int* block_tables, const int* seq_ids,
                                              int num_seqs, int H, int KVH, int block_size, int max_blocks,
                                              float scale, int window, int nsplit, const int* share_tiles, int depth,
                                              hipStream_t stream) {
  return launch_decode(static_cast<const bf16_t*>(q), nullptr, static_cast<bf16_t*>(const_cast<void*>(k_cache)),
                       static_cast<bf16_t*>(const_cast<void*>(v_cache)), static_cast<bf16_t*>(out), part_o, part_ml,
                       query_start, context_lens, block_tables, seq_ids, num_seqs, H, KVH, block_size, max_blocks,
                       scale, window, nsplit, share_tiles, depth, stream);
}

// The same for a step of single decoded tokens whose queries, newest keys and values still lie in the QKV
// projection's output: qkv is float32 [planes][rows][in_row] (plane p at qkv + p * plane_stride; a row holds H
// query heads, KVH key heads, KVH value heads), summed over the planes by the kernel; q_weight / k_weight (or
// null) the per-head RMS norm weights with eps; angles [rows][head_dim] the step's table of cos and sin.
// write_kv = 0 where the cache is another layer's and holds the token already. Pages of 16 positions or more
// and head sizes 32, 64, 128, 256; refused otherwise (tie_attention_decode_prepares tells).
extern "C" int tie_attention_decode_prepares(int block_size) { return PREPARE_HEAD_DIM && block_size >= 16 ? 1 : 0; }

extern "C" int tie_attention_decode_prepared_bf16(const float* qkv, long plane_stride, int planes, int in_row,
                                                  const float* q_weight, const float* k_weight, float eps,
                                                  const float* angles, int write_kv, void* k_cache, void* v_cache,
                                                  void* out, float* part_o, float* part_ml, const int* query_start,
                                                  const int* context_lens, const int* block_tables,
                                                  const int* seq_ids, int num_seqs, int H, int KVH, int block_size,
                                                  int max_blocks, float scale, int window, int nsplit,
                                                  const int* share_tiles, int depth, hipStream_t stream) {
  if (qkv == nullptr || angles == nullptr || planes < 1 || planes > 8 || plane_stride < 0 || block_size < 16 ||
      depth == 1 || H <= 0 || KVH <= 0 || in_row < (H + 2 * KVH) * DH || in_row % 4 != 0 || plane_stride % 4 != 0 ||
      reinterpret_cast<uintptr_t>(qkv) % 16 != 0 || reinterpret_cast<uintptr_t>(angles) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(q_weight) % 16 != 0 || reinterpret_cast<uintptr_t>(k_weight) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(k_cache) % 16 != 0)
    return TIE_BAD_ARGUMENT;
  const QkSource src = {qkv, static_cast<size_t>(plane_stride), planes, in_row, q_weight, k_weight, eps, angles, write_kv};
  return launch_decode(nullptr, &src, static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache),
                       static_cast<bf16_t*>(out), part_o, part_ml, query_start, context_lens, block_tables, seq_ids,
                       num_seqs, H, KVH, block_size, max_blocks, scale, window, nsplit, share_tiles, depth, stream);
}

extern "C" int tie_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                         float* part_o, float* part_ml, const int* query_start,
                                         const int* context_lens, const int* block_tables, const int* seq_ids,
                                         int num_seqs, int H, int KVH, int block_size, int max_blocks, float scale,
                                         int window, int nsplit, hipStream_t stream) {
  return tie_attention_decode_bf16_with(q, k_cache, v_cache, out, part_o, part_ml, query_start, context_lens,
                                        block_tables, seq_ids, num_seqs, H, KVH, block_size, max_blocks, scale, window,
                                        nsplit, nullptr, 0, stream);
}
