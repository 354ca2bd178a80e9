// Absorbed-MLA decode attention over the paged latent KV cache, gfx950 (CDNA4).
//
//   s_i = scale * (q_lat[h] . c_i + q_rope[h] . r_i),  p = softmax_i(s),  o[h] = sum_i p_i c_i
//
// One query token per sequence, all heads share one latent KV stream (MQA), so the
// head axis is the free MFMA dimension and the latent row is read from HBM once and used
// as both K (with the 64 rope columns appended) and V.
//
// Work decomposition
//   workgroup = (kv chunk, sequence, group of 64 heads); 4 wavefronts, 16 heads each, one
//   workgroup per CU. A chunk is `chunk_tiles` tiles of 64 tokens. Two tile buffers in LDS;
//   bf16 tiles are filled by direct global->LDS loads (global_load_lds_dwordx4: no staging
//   registers, no ds_write), issued one tile ahead of the math; FP8 tiles are dequantised
//   to bf16 through registers on their way into LDS.
//
// MFMA formulation (v_mfma_f32_16x16x32_bf16; A: lane holds row l%16, k = 8*(l/16)..+7;
// B: lane holds column l%16, same k; D: lane holds rows 4*(l/16)..+3 of column l%16)
//   S^T[token][head] = K[token][:] . Q[head][:]   A = K fragment from LDS (ds_read_b128),
//                                                 B = Q fragment, resident in registers.
//   D puts four consecutive tokens of one head in a lane, which is exactly the B operand
//   of the second product once the contraction index is ordered as
//   kappa = 8g+e <-> token 32u+4g+e, kappa = 8g+4+e <-> token 32u+16+4g+e:
//   O^T[dv][head] += V^T[dv][token] . P[token][head]   A = V^T fragment, read from the
//   row-major tile with ds_read_b64_tr_b16 (a 4x16 transpose per 16 lanes), B = P.
//   So P never leaves registers and the online-softmax statistics of a head live in the
//   four lanes {h, h+16, h+32, h+48}: two wavefront shuffles per reduction.
//   Each wavefront is alone on its SIMD, so LDS latency is hidden inside the instruction
//   stream: operand fragments are fetched eight MFMAs ahead into a second register set.
//
// LDS tile: latent region 64 rows x 1024 B, then rope region 64 rows x 128 B; the 16-byte
//   chunk index inside a row is XORed with f(token & 7) = ((t & 3) << 1) | (t >> 2): eight
//   consecutive tokens hit eight distinct 16-byte bank groups for the K reads and four
//   consecutive tokens hit four distinct 32-byte groups for the transposed V reads. With
//   direct loads the swizzle is applied on the global side: lane L of a row fetches chunk L ^ f.
//
// Online softmax keeps a reference maximum per head and only moves it (rescaling O) when a
// tile's maximum exceeds it by more than 2^8, so exponentials stay below 256 and most
// tiles skip the rescale.
//
// Chunks of one sequence are merged by a second small kernel from fp32 partials
// (normalised O and log2-domain LSE) held in the caller's workspace.
#include <cstdlib>

#include "kernels.h"

namespace mlakv {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

constexpr int kThreads = 256;
constexpr int kLatRowBytes = kLatentDim * 2;                 // 1024
constexpr int kRopeRowBytes = kRopeDim * 2;                  // 128
constexpr int kLatRegion = kTileTokens * kLatRowBytes;       // 65536
constexpr int kTileBytes = kLatRegion + kTileTokens * kRopeRowBytes;  // 73728
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;        // 18
constexpr int kDvTiles = kLatentDim / 16;                    // 32
constexpr int kTableEntries = 2048;                          // block-table entries of one chunk staged in LDS
constexpr int kLdsBytes = 2 * kTileBytes + kTableEntries * 4;
constexpr float kRescaleThreshold = 8.0f;                    // log2 domain

__device__ __forceinline__ int Uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
// LDS is 64 banks x 4 B (256 B per clock): a ds_read_b128 serves 16 lanes per clock, a
// ds_read_b64_tr_b16 32 lanes. Latent rows (1024 B): the chunk index is XORed with a 4-bit
// function of the token so that 16 consecutive tokens land in 16 distinct 16-byte slots (K
// reads) and 8 consecutive tokens in 8 distinct 32-byte slots (transposed V reads). Rope rows
// (128 B, two per 256 B): 3-bit XOR by token/2.
__device__ __forceinline__ int SwizzleLat(int token) { return ((token & 7) << 1) | ((token >> 3) & 1); }
__device__ __forceinline__ int SwizzleRope(int token) { return (token >> 1) & 7; }
__device__ __forceinline__ int LatOffset(int token, int chunk) { return token * kLatRowBytes + ((chunk ^ SwizzleLat(token)) << 4); }
__device__ __forceinline__ int RopeOffset(int token, int chunk) {
  return kLatRegion + token * kRopeRowBytes + ((chunk ^ SwizzleRope(token)) << 4);
}

__device__ __forceinline__ u32x4 GlobalLoad16(const char* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void DirectLoad16(const char* global, unsigned char* lds_wave_base) {
  // Lane L's 16 bytes land at lds_wave_base + 16 * L; lds_wave_base is wave-uniform.
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// Where the rows of one tile live. Block-table entries of the chunk are staged once in LDS
// (-1 marks an entry outside the pool), so a tile's row addresses need no dependent global
// load. ALIGNED (block_size a multiple of 64): the whole tile sits in one physical block.
template <bool ALIGNED>
struct TileMap {
  const int* entries;  // LDS
  int first_block, block_size, seq_len;
  int tile_block, tile_slot0;  // ALIGNED only

  __device__ __forceinline__ void Begin(int tile) {
    if (ALIGNED) {
      const int pos0 = tile * kTileTokens;
      const int logical = pos0 / block_size;
      tile_block = entries[logical - first_block];
      tile_slot0 = pos0 - logical * block_size;
    }
  }
  // Physical block (clamped to a readable one) and slot of row `r` of tile `tile`; returns
  // whether the row is real (inside the sequence, behind a valid table entry).
  __device__ __forceinline__ bool Row(int tile, int r, int* block, int* slot) const {
    const int pos = tile * kTileTokens + r;
    if (ALIGNED) {
      *block = tile_block < 0 ? 0 : tile_block;
      *slot = pos < seq_len ? tile_slot0 + r : 0;
      return pos < seq_len && tile_block >= 0;
    }
    const int clamped = pos < seq_len ? pos : seq_len - 1;
    const int logical = clamped / block_size;
    const int entry = entries[logical - first_block];
    *block = entry < 0 ? 0 : entry;
    *slot = clamped - logical * block_size;
    return pos < seq_len && entry >= 0;
  }
};

// ---- bf16 tiles: direct global -> LDS ----------------------------------------------------

// Lane-constant byte offsets of the chunk a lane fetches for the rows its wave owns: a wave
// owns latent rows w, w+4, ... (16 of them; row & 15 takes four values) and rope row groups w, w+4.
struct IssueLane {
  int lat[4];   // latent rows with (row >> 2) & 3 == j
  int rope[2];  // rope groups w and w + 4
};

template <bool ALIGNED>
__device__ __forceinline__ void IssueTileBf16(const AttnArgs& a, TileMap<ALIGNED>& map, const IssueLane& il, int tile,
                                              unsigned char* buf, int tid) {
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  map.Begin(tile);
  const int rows = map.seq_len - tile * kTileTokens;  // real rows in this tile, >= 1
  if (ALIGNED && rows >= kTileTokens && map.tile_block >= 0) {
    // The whole tile is real and sits in one physical block: uniform base + row pitch.
    const int block = Uniform(map.tile_block), slot0 = Uniform(map.tile_slot0);
    const char* latent = a.latent.base + block * a.latent.block_stride + (slot0 + wave) * a.latent.row_stride;
    const int64_t pitch = 4 * a.latent.row_stride;
#pragma unroll
    for (int i = 0; i < 16; ++i) DirectLoad16(latent + i * pitch + il.lat[i & 3], buf + (wave + 4 * i) * kLatRowBytes);
    const char* rope = a.rope.base + block * a.rope.block_stride + (slot0 + (lane >> 3)) * a.rope.row_stride;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int group = wave + 4 * i;
      DirectLoad16(rope + group * 8 * a.rope.row_stride + il.rope[i], buf + kLatRegion + group * 8 * kRopeRowBytes);
    }
    return;
  }
  int block[16], slot[16];
  bool real[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) real[i] = map.Row(tile, wave + 4 * i, &block[i], &slot[i]);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = wave + 4 * i;  // wave-uniform
    unsigned char* dst = buf + row * kLatRowBytes;
    if (real[i]) {
      const char* src = a.latent.base + Uniform(block[i]) * a.latent.block_stride + Uniform(slot[i]) * a.latent.row_stride;
      DirectLoad16(src + il.lat[i & 3], dst);
    } else {
      *reinterpret_cast<u32x4*>(dst + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }
  // rope: one wave access covers 8 rows x 128 B
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int group = wave + 4 * i;  // wave-uniform: rows 8*group .. 8*group+7
    const int row = 8 * group + (lane >> 3);
    int rblock, rslot;
    const bool rreal = map.Row(tile, row, &rblock, &rslot);
    unsigned char* dst = buf + kLatRegion + group * 8 * kRopeRowBytes;
    if (rreal) {
      const char* src = a.rope.base + rblock * a.rope.block_stride + rslot * a.rope.row_stride;
      DirectLoad16(src + il.rope[i], dst);
    } else {
      *reinterpret_cast<u32x4*>(dst + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }
}

// ---- FP8 tiles: global -> registers -> (dequantise) -> LDS ------------------------------------

// 8 latent chunks + 1 rope chunk of 16 codes per thread, and their row scales (0 for a row
// that is not real).
struct TileRegsFp8 {
  u32x4 v[9];
  float scale[9];
};

template <bool ALIGNED>
__device__ __forceinline__ void LoadTileFp8(TileRegsFp8& r, const AttnArgs& a, TileMap<ALIGNED>& map, int tile, int tid) {
  map.Begin(tile);
  int block[9], slot[9];
  bool real[9];
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    const int token = i < 8 ? (tid + kThreads * i) >> 5 : tid >> 2;
    real[i] = map.Row(tile, token, &block[i], &slot[i]);
  }
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    const int chunk = i < 8 ? (tid + kThreads * i) & 31 : tid & 3;
    const Plane& plane = i < 8 ? a.latent : a.rope;
    r.v[i] = GlobalLoad16(plane.base + block[i] * plane.block_stride + slot[i] * plane.row_stride + chunk * 16);
    const float scale = reinterpret_cast<const float*>(a.scale.base + block[i] * a.scale.block_stride)[slot[i]];
    r.scale[i] = real[i] ? scale : 0.0f;
  }
}

__device__ __forceinline__ unsigned int PackBf16(float lo, float hi) {
  const bf16x2 packed = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(unsigned int, packed);
}

// Four E4M3 codes of one dword -> four bf16 (two dwords), scaled.
__device__ __forceinline__ void Dequant4(unsigned int codes, float scale, unsigned int* lo, unsigned int* hi) {
  const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes), false);
  const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes), true);
  *lo = PackBf16(a.x * scale, a.y * scale);
  *hi = PackBf16(b.x * scale, b.y * scale);
}

__device__ __forceinline__ void StoreTileFp8(const TileRegsFp8& r, unsigned char* buf, int tid) {
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    u32x4 first, second;
    unsigned int lo, hi;
    Dequant4(r.v[i].x, r.scale[i], &lo, &hi);
    first.x = lo;
    first.y = hi;
    Dequant4(r.v[i].y, r.scale[i], &lo, &hi);
    first.z = lo;
    first.w = hi;
    Dequant4(r.v[i].z, r.scale[i], &lo, &hi);
    second.x = lo;
    second.y = hi;
    Dequant4(r.v[i].w, r.scale[i], &lo, &hi);
    second.z = lo;
    second.w = hi;
    if (r.scale[i] == 0.0f) {  // not a real row: zeros, whatever the fetched codes were
      first = u32x4{0u, 0u, 0u, 0u};
      second = first;
    }
    if (i < 8) {
      const int idx = tid + kThreads * i;
      const int token = idx >> 5, chunk = 2 * (idx & 31);
      *reinterpret_cast<u32x4*>(buf + LatOffset(token, chunk)) = first;
      *reinterpret_cast<u32x4*>(buf + LatOffset(token, chunk + 1)) = second;
    } else {
      const int token = tid >> 2, chunk = 2 * (tid & 3);
      *reinterpret_cast<u32x4*>(buf + RopeOffset(token, chunk)) = first;
      *reinterpret_cast<u32x4*>(buf + RopeOffset(token, chunk + 1)) = second;
    }
  }
}

// ---- main kernel -------------------------------------------------------------------

template <bool FP8, bool ALIGNED>
__global__ __launch_bounds__(kThreads, 1) void MlaDecodeKernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i16 = lane & 15;
  const int chunk_index = blockIdx.x;
  const int seq = blockIdx.y;
  const int head_base = blockIdx.z * 64 + wave * 16;
  const bool active = head_base < a.heads;  // wave-uniform
  const int head = head_base + i16;

  const int seq_len = Uniform(a.seq_lens[seq]);
  const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  const int tile_begin = chunk_index * a.chunk_tiles;
  const bool direct = a.max_chunks == 1;  // single chunk: write the final output here
  if (tile_begin >= num_tiles) {
    if (direct && active) {  // empty sequence: zeros, lse = -inf
      char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
      for (int n = g; n < kLatentDim / 8; n += 4) *reinterpret_cast<u32x4*>(out + n * 16) = u32x4{0u, 0u, 0u, 0u};
      if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    }
    return;
  }
  const int tile_end = min(tile_begin + a.chunk_tiles, num_tiles);

  // Stage this chunk's block-table entries in LDS.
  int* table_lds = reinterpret_cast<int*>(lds + 2 * kTileBytes);
  TileMap<ALIGNED> map;
  map.entries = table_lds;
  map.block_size = a.block_size;
  map.seq_len = seq_len;
  {
    const int first_pos = tile_begin * kTileTokens;
    const int last_pos = min(tile_end * kTileTokens, seq_len) - 1;
    map.first_block = first_pos / a.block_size;
    const int count = last_pos / a.block_size - map.first_block + 1;  // <= kTableEntries, ensured by the plan
    const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride + map.first_block;
    for (int i = tid; i < count; i += kThreads) {
      const int entry = table_row[i];
      table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : -1;
    }
  }

  // Q fragments: lane (head i16, k-group g) holds Q[head][32*ks + 8g .. +7].
  bf16x8 q[kKSteps];
  if (active) {
    const char* q_latent = a.q_latent + seq * a.q_latent_seq_stride + head * a.q_latent_head_stride;
    const char* q_rope = a.q_rope + seq * a.q_rope_seq_stride + head * a.q_rope_head_stride;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      const int d0 = 32 * ks + 8 * g;
      const char* p = d0 < kLatentDim ? q_latent + d0 * 2 : q_rope + (d0 - kLatentDim) * 2;
      q[ks] = __builtin_bit_cast(bf16x8, GlobalLoad16(p));
    }
  }

  f32x4 o[kDvTiles];
#pragma unroll
  for (int n = 0; n < kDvTiles; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_ref = -__builtin_inff();  // reference maximum of the exponentials, log2 domain
  float l_run = 0.0f;               // this lane's share of the running denominator

  // Lane-constant LDS offsets.
  // K reads: token = 16t + i16, chunk = 4 ks + g (latent, ks < 16) or 4 (ks - 16) + g (rope).
  const int k_lat = i16 * kLatRowBytes, k_rope = kLatRegion + i16 * kRopeRowBytes;
  int k_e[4], kr_e[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) k_e[j] = ((4 * j + g) ^ SwizzleLat(i16)) << 4;
#pragma unroll
  for (int j = 0; j < 2; ++j) kr_e[j] = ((4 * j + g) ^ SwizzleRope(i16)) << 4;
  // V reads: token = 32u (+16) + 4g + i16/4, chunk = 2n + (i16 & 3) / 2, 8-byte half i16 & 1.
  const int v_row = 4 * g + (i16 >> 2);
  const int v_lane = v_row * kLatRowBytes + (i16 & 1) * 8;
  int v_e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v_e[j] = ((2 * j + ((i16 & 3) >> 1)) ^ SwizzleLat(v_row)) << 4;
  // Direct loads: lane L of a latent row fetches chunk L ^ swizzle(row); rows of this wave.
  IssueLane il;
  {
    const int w = Uniform(tid >> 6);
#pragma unroll
    for (int j = 0; j < 4; ++j) il.lat[j] = (lane ^ SwizzleLat(w + 4 * j)) << 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) il.rope[j] = ((lane & 7) ^ SwizzleRope(8 * (w + 4 * j) + (lane >> 3))) << 4;
  }

  __syncthreads();  // table entries visible
  TileRegsFp8 regs;
  if (FP8) {
    LoadTileFp8(regs, a, map, tile_begin, tid);
    StoreTileFp8(regs, lds, tid);
    if (tile_begin + 1 < tile_end) LoadTileFp8(regs, a, map, tile_begin + 1, tid);
  } else {
    IssueTileBf16(a, map, il, tile_begin, lds, tid);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    unsigned char* cur = lds + ((tile - tile_begin) & 1) * kTileBytes;
    unsigned char* nxt = lds + (((tile - tile_begin) & 1) ^ 1) * kTileBytes;

    // The other buffer was last read before the barrier that ended the previous iteration.
    if (!FP8 && tile + 1 < tile_end && !(a.debug & 8)) IssueTileBf16(a, map, il, tile + 1, nxt, tid);

    f32x4 s[4];
    if (active && !(a.debug & 1)) {
      // ---- S^T = K Q^T, K fragments fetched eight MFMAs (two k-steps) ahead ----
#pragma unroll
      for (int t = 0; t < 4; ++t) s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      bf16x8 kb[2][8];
      const auto load_k = [&](bf16x8* dst, int pair) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const int ks = 2 * pair + kk;
          const int base = ks < 16 ? k_lat + (ks >> 2) * 256 + k_e[ks & 3] : k_rope + kr_e[ks & 1];
          const int row_pitch = ks < 16 ? kLatRowBytes : kRopeRowBytes;
#pragma unroll
          for (int t = 0; t < 4; ++t) dst[kk * 4 + t] = *reinterpret_cast<const bf16x8*>(cur + base + t * 16 * row_pitch);
        }
      };
      load_k(kb[0], 0);
#pragma unroll
      for (int pair = 0; pair < kKSteps / 2; ++pair) {
        if (pair + 1 < kKSteps / 2) load_k(kb[(pair + 1) & 1], pair + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[pair & 1][kk * 4 + t], q[2 * pair + kk], s[t], 0, 0, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    if (FP8 && tile + 1 < tile_end) {
      StoreTileFp8(regs, nxt, tid);
      if (tile + 2 < tile_end) LoadTileFp8(regs, a, map, tile + 2, tid);
    }

    if (active) {
      // ---- online softmax; lane holds tokens 16t + 4g + j of head i16 ----
      const int valid = seq_len - tile * kTileTokens;  // >= 1
      float tile_max = -__builtin_inff();
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float v = s[t][j] * a.scale_log2;
          if (valid < kTileTokens && 16 * t + 4 * g + j >= valid) v = -__builtin_inff();
          s[t][j] = v;
          tile_max = fmaxf(tile_max, v);
        }
      }
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16));
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
      // Move the reference only when some head's maximum outgrew it by more than the threshold.
      if (__builtin_amdgcn_ballot_w64(tile_max > m_ref + kRescaleThreshold) != 0) {
        const float m_new = fmaxf(m_ref, tile_max);  // finite: token 0 of the tile is valid
        const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
        l_run *= alpha;
        m_ref = m_new;
#pragma unroll
        for (int n = 0; n < kDvTiles; ++n) o[n] *= alpha;
      }
      float row_sum = 0.0f;
      bf16x8 p[2];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float e = (a.debug & 2) ? 1.0f : __builtin_amdgcn_exp2f(s[t][j] - m_ref);
          row_sum += e;
          p[t >> 1][(t & 1) * 4 + j] = static_cast<__bf16>(e);
        }
      }
      l_run += row_sum;

      // ---- O^T += V^T P, V fragments fetched eight MFMAs ahead ----
      bf16x8 vb[2][8];
      const auto load_v = [&](bf16x8* dst, int group) {  // group: u = group / 4, n = 8 * (group % 4) .. +7
        const unsigned char* vbase = cur + v_lane + (group >> 2) * 32 * kLatRowBytes;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int n = 8 * (group & 3) + j;
          const unsigned char* addr = vbase + (n >> 3) * 256 + v_e[n & 7];
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4*)(addr + 16 * kLatRowBytes));
          dst[j] = __builtin_shufflevector(__builtin_bit_cast(bf16x4, lo), __builtin_bit_cast(bf16x4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
        }
      };
      if (!(a.debug & 4)) load_v(vb[0], 0);
#pragma unroll
      for (int group = 0; group < 8 && !(a.debug & 4); ++group) {
        if (group + 1 < 8) load_v(vb[(group + 1) & 1], group + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int n = 8 * (group & 3) + j;
          o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb[group & 1][j], p[group >> 2], o[n], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (!FP8) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next tile has landed in LDS
    __syncthreads();
  }

  if (!active) return;
  float l_total = l_run + __shfl_xor(l_run, 16);
  l_total += __shfl_xor(l_total, 32);
  const float inv = 1.0f / l_total;
  const float lse2 = m_ref + __builtin_amdgcn_logf(l_total);  // v_log_f32 is log2
  if (direct) {
    char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
#pragma unroll
    for (int n = 0; n < kDvTiles; ++n) {
      u32x2 packed;
      packed.x = PackBf16(o[n][0] * inv, o[n][1] * inv);
      packed.y = PackBf16(o[n][2] * inv, o[n][3] * inv);
      *reinterpret_cast<u32x2*>(out + (16 * n + 4 * g) * 2) = packed;
    }
    if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = lse2 * 0.6931471805599453f;
  } else {
    const int64_t row = (static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head;
    float* partial = a.partial_out + row * kLatentDim;
#pragma unroll
    for (int n = 0; n < kDvTiles; ++n) *reinterpret_cast<f32x4*>(partial + 16 * n + 4 * g) = o[n] * inv;
    if (g == 0) a.partial_lse[row] = lse2;
  }
}

// Merges the chunks of one (sequence, head): out = sum_c w_c O_c / sum_c w_c with
// w_c = 2^(lse2_c - max lse2). 128 threads, 4 output columns each.
__global__ __launch_bounds__(128) void MlaCombineKernel(AttnArgs a) {
  const int head = blockIdx.x, seq = blockIdx.y;
  const int tid = threadIdx.x;
  const int seq_len = a.seq_lens[seq];
  const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  const int chunks = (num_tiles + a.chunk_tiles - 1) / a.chunk_tiles;
  char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride + tid * 8;
  if (chunks == 0) {
    *reinterpret_cast<u32x2*>(out) = u32x2{0u, 0u};
    if (a.lse != nullptr && tid == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    return;
  }
  const int64_t row0 = static_cast<int64_t>(seq) * a.max_chunks * a.heads + head;
  float m = -__builtin_inff();
  for (int c = 0; c < chunks; ++c) m = fmaxf(m, a.partial_lse[row0 + static_cast<int64_t>(c) * a.heads]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float denom = 0.0f;
  for (int c = 0; c < chunks; ++c) {
    const int64_t row = row0 + static_cast<int64_t>(c) * a.heads;
    const float w = __builtin_amdgcn_exp2f(a.partial_lse[row] - m);
    const f32x4 v = *reinterpret_cast<const f32x4*>(a.partial_out + row * kLatentDim + tid * 4);
    acc += v * w;
    denom += w;
  }
  const float inv = 1.0f / denom;
  u32x2 packed;
  packed.x = PackBf16(acc[0] * inv, acc[1] * inv);
  packed.y = PackBf16(acc[2] * inv, acc[3] * inv);
  *reinterpret_cast<u32x2*>(out) = packed;
  if (a.lse != nullptr && tid == 0) a.lse[seq * a.heads + head] = (m + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f;
}

template <bool FP8, bool ALIGNED>
hipError_t Launch(const AttnArgs& args, const dim3& grid, hipStream_t stream) {
  // Dynamic LDS above 64 KB needs the attribute once per kernel and process.
  static const hipError_t prepared = hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaDecodeKernel<FP8, ALIGNED>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (prepared != hipSuccess) return prepared;
  hipLaunchKernelGGL((MlaDecodeKernel<FP8, ALIGNED>), grid, dim3(kThreads), kLdsBytes, stream, args);
  return hipGetLastError();
}

}  // namespace

hipError_t PrepareAttnKernels() { return hipSuccess; }

hipError_t LaunchAttnDecode(const AttnArgs& args_in, hipStream_t stream) {
  AttnArgs args = args_in;
  static const int debug = std::getenv("MLAKV_ATTN_DEBUG") ? std::atoi(std::getenv("MLAKV_ATTN_DEBUG")) : 0;
  args.debug = debug;
  if (args.batch <= 0) return hipSuccess;
  const dim3 grid(args.max_chunks, args.batch, (args.heads + 63) / 64);
  const bool aligned = args.block_size % kTileTokens == 0;
  hipError_t e;
  if (args.fp8) e = aligned ? Launch<true, true>(args, grid, stream) : Launch<true, false>(args, grid, stream);
  else e = aligned ? Launch<false, true>(args, grid, stream) : Launch<false, false>(args, grid, stream);
  if (e != hipSuccess) return e;
  if (args.max_chunks > 1) {
    hipLaunchKernelGGL(MlaCombineKernel, dim3(args.heads, args.batch), dim3(128), 0, stream, args);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace mlakv
