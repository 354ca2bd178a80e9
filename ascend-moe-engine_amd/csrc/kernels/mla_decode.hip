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
//   workgroup per CU. A chunk is `chunk_tiles` tiles of 32 tokens. LDS holds a ring of four
//   tile buffers: while tile i feeds the second product and tile i+1 the first, tiles i+2 and
//   i+3 are in flight from HBM. bf16 tiles are filled by direct global->LDS loads
//   (global_load_lds_dwordx4: no staging registers, no ds_write); FP8 tiles are dequantised
//   to bf16 through registers on their way into LDS.
//
// MFMA formulation (v_mfma_f32_16x16x32_bf16; A: lane holds row l%16, k = 8*(l/16)..+7;
// B: lane holds column l%16, same k; D: lane holds rows 4*(l/16)..+3 of column l%16)
//   S^T[token][head] = K[token][:] . Q[head][:]   A = K fragment from LDS (ds_read_b128),
//                                                 B = Q fragment, resident in registers.
//   D puts four consecutive tokens of one head in a lane, which is exactly the B operand
//   of the second product once the contraction index is ordered as
//   kappa = 8g+e <-> token 4g+e, kappa = 8g+4+e <-> token 16+4g+e:
//   O^T[dv][head] += V^T[dv][token] . P[token][head]   A = V^T fragment, read from the
//   row-major tile with ds_read_b64_tr_b16 (a 4x16 transpose per 16 lanes), B = P.
//   So P never leaves registers and the online-softmax statistics of a head live in the
//   four lanes {h, h+16, h+32, h+48}: two v_permlane swaps per reduction.
//
// Software pipeline: each wavefront is alone on its SIMD, so nothing hides latency but the
// instruction order. The loop body is written out step by step (one MFMA, the LDS read that
// refills its operand register several steps ahead, and a slice of the softmax of the
// previous tile) with a scheduling fence after every step: the softmax VALU work of tile i
// (exponentials, denominator, P) runs in the shadow of the S^T MFMAs of tile i+1, and the score
// scaling and maximum of tile i+1 in the shadow of the O^T MFMAs of tile i.
//
// LDS tile: latent region 32 rows x 1024 B, then rope region 32 rows x 128 B; the 16-byte
//   chunk index inside a row is XORed with a function of the token (see SwizzleLat). With
//   direct loads the swizzle is applied on the global side: lane L of a row fetches chunk L ^ f.
//
// Online softmax keeps a reference maximum per head and only moves it (rescaling O) when a
// tile's maximum exceeds it by more than 2^8, so exponentials stay below 256 and most
// tiles skip the rescale.
//
// Chunks of one sequence are merged by a second small kernel from partials (normalised O in
// bf16, log2-domain LSE in fp32) held in the caller's workspace.
#include <utility>

#include "kernels.h"

#pragma clang diagnostic ignored "-Winline-asm"

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
constexpr int kLatRegion = kTileTokens * kLatRowBytes;       // 32768
constexpr int kTileBytes = kLatRegion + kTileTokens * kRopeRowBytes;  // 36864
constexpr int kRing = 4;                                     // tile buffers in LDS
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;        // 18
constexpr int kQkSteps = 2 * kKSteps;                        // 36 MFMAs: 18 k-steps x 2 token subtiles
constexpr int kDvTiles = kLatentDim / 16;                    // 32
constexpr int kTableEntries = 2048;                          // block-table entries of one chunk staged in LDS
constexpr int kLdsBytes = kRing * kTileBytes + kTableEntries * 4;
constexpr int kLoadsPerTile = kTileTokens / 4 + 1;           // direct loads one wave issues for a full tile
constexpr int kUnknownLoads = -1;
constexpr float kRescaleThreshold = 8.0f;                    // log2 domain
constexpr int kKAhead = 8;                                   // K fragments in flight ahead of their MFMA
constexpr int kVAhead = 4;                                   // V fragments (two transposed reads each)
static_assert(kTileTokens == 32, "the fragment maps below are written for 32-token tiles");

__device__ __forceinline__ int Uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Calls f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N - 1>): the
// pipeline steps are distinct pieces of straight-line code, selected at compile time.
template <typename F, int... I>
__device__ __forceinline__ void StaticForImpl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void StaticFor(F&& f) {
  StaticForImpl(f, std::make_integer_sequence<int, N>{});
}

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

// Direct global->LDS loads: lane L's 16 bytes land at lds_wave_base + 16 * L (the LDS base
// travels in M0 and is wave-uniform). They are issued from inline assembly so that the
// compiler does not serialise every later LDS read behind them; the kernel waits for them
// itself with WaitLoads() before the workgroup barrier that publishes a tile.
__device__ __forceinline__ void DirectLoad16(const char* uniform_base, int lane_offset, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_offset), "s"(uniform_base), "s"(lds_wave_base)
               : "memory", "m0");
}
__device__ __forceinline__ void DirectLoad16PerLane(const char* lane_pointer, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(lane_pointer), "s"(lds_wave_base)
               : "memory", "m0");
}
// Waits until at most `newer` of this wave's vector-memory loads are outstanding (loads
// complete in issue order). Anything but a whole number of full tiles waits for everything.
__device__ __forceinline__ void WaitLoads(int newer) {
  if (newer == 2 * kLoadsPerTile) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerTile) : "memory");
  } else if (newer == kLoadsPerTile) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerTile) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
}

// The O accumulators must stay in accumulation registers for the whole loop (the 256
// architectural VGPRs are needed for the query, the operand fragments and the scores), so
// the second product is issued from inline assembly with the accumulator pinned to the AGPR
// class. The compiler does not see an MFMA there and inserts no wait states around it:
// FIRST adds the two the hardware wants between a v_accvgpr_write and an MFMA that reads the
// register as its addend, LAST the (at most 19) it wants before a VALU instruction may read
// an MFMA result; the MFMAs of one product retire in order, so covering the last covers all.
template <bool FIRST, bool LAST>
__device__ __forceinline__ void MfmaPinned(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  if (FIRST) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  } else if (LAST) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 3" : "+a"(acc) : "v"(a), "v"(b));
  } else {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
}

// max over the four lanes {l%16, +16, +32, +48}: v_permlane16_swap exchanges odd and even rows
// of 16 lanes between its two operands, v_permlane32_swap the two halves of the wave.
__device__ __forceinline__ float MaxAcrossRows16(float x) {
  const unsigned bits = __builtin_bit_cast(unsigned, x);
  const u32x2 swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  const unsigned a = swapped.x, b = swapped.y;
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float MaxAcrossHalves(float x) {
  const unsigned bits = __builtin_bit_cast(unsigned, x);
  const u32x2 swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  const unsigned a = swapped.x, b = swapped.y;
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float SumAcrossHeadLanes(float x) {
  unsigned bits = __builtin_bit_cast(unsigned, x);
  u32x2 swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  unsigned a = swapped.x, b = swapped.y;
  const float s = __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
  bits = __builtin_bit_cast(unsigned, s);
  swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  a = swapped.x;
  b = swapped.y;
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}

// Where the rows of one tile live. Block-table entries of the chunk are staged once in LDS
// (-1 marks an entry outside the pool), so a tile's row addresses need no dependent global
// load. ALIGNED (block_size a multiple of the tile): the whole tile sits in one physical block.
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
// owns latent rows w, w+4, ... (8 of them; row & 15 takes four values) and rope rows 8w..8w+7.
struct IssueLane {
  int lat[4];  // latent rows with (row >> 2) & 3 == j
  int rope;    // this lane's rope row and chunk, relative to rope row 8w
  int rope_chunk;
};

// Issues the loads of one tile into the buffer at LDS address `buf`; rows that are not real
// are zero-filled instead. Returns how many loads this wave issued when that is the same for
// every tile of this shape (a full tile), kUnknownLoads otherwise.
template <bool ALIGNED>
__device__ __forceinline__ int IssueTileBf16(const AttnArgs& a, TileMap<ALIGNED>& map, const IssueLane& il, int tile,
                                             unsigned buf, unsigned char* buf_ptr, int tid) {
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  map.Begin(tile);
  const int rows = map.seq_len - tile * kTileTokens;  // real rows in this tile, >= 1
  if (ALIGNED && rows >= kTileTokens && map.tile_block >= 0) {
    // The whole tile is real and sits in one physical block: uniform base + row pitch.
    const int block = Uniform(map.tile_block), slot0 = Uniform(map.tile_slot0);
    const char* latent = a.latent.base + block * a.latent.block_stride + (slot0 + wave) * a.latent.row_stride;
    const int64_t pitch = 4 * a.latent.row_stride;
#pragma unroll
    for (int i = 0; i < kTileTokens / 4; ++i) DirectLoad16(latent + i * pitch, il.lat[i & 3], buf + (wave + 4 * i) * kLatRowBytes);
    const char* rope = a.rope.base + block * a.rope.block_stride + (slot0 + 8 * wave) * a.rope.row_stride;
    DirectLoad16(rope, il.rope, buf + kLatRegion + wave * 8 * kRopeRowBytes);
    return kLoadsPerTile;
  }
  int block[kTileTokens / 4], slot[kTileTokens / 4];
  bool real[kTileTokens / 4];
  bool all_real = true;
#pragma unroll
  for (int i = 0; i < kTileTokens / 4; ++i) {
    real[i] = map.Row(tile, wave + 4 * i, &block[i], &slot[i]);
    all_real = all_real && real[i];
  }
  int rblock, rslot;
  const bool rreal = map.Row(tile, 8 * wave + (lane >> 3), &rblock, &rslot);
  all_real = all_real && (__builtin_amdgcn_ballot_w64(!rreal) == 0);
#pragma unroll
  for (int i = 0; i < kTileTokens / 4; ++i) {
    const int row = wave + 4 * i;  // wave-uniform
    if (real[i]) {
      const char* src = a.latent.base + Uniform(block[i]) * a.latent.block_stride + Uniform(slot[i]) * a.latent.row_stride;
      DirectLoad16(src, il.lat[i & 3], buf + row * kLatRowBytes);
    } else {
      *reinterpret_cast<u32x4*>(buf_ptr + row * kLatRowBytes + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }
  // rope: one wave access covers 8 rows x 128 B, each lane resolving its own row
  if (all_real) {
    DirectLoad16PerLane(a.rope.base + rblock * a.rope.block_stride + rslot * a.rope.row_stride + il.rope_chunk,
                        buf + kLatRegion + wave * 8 * kRopeRowBytes);
    return kLoadsPerTile;
  }
  if (rreal) {
    DirectLoad16PerLane(a.rope.base + rblock * a.rope.block_stride + rslot * a.rope.row_stride + il.rope_chunk,
                        buf + kLatRegion + wave * 8 * kRopeRowBytes);
  } else {
    *reinterpret_cast<u32x4*>(buf_ptr + kLatRegion + wave * 8 * kRopeRowBytes + lane * 16) = u32x4{0u, 0u, 0u, 0u};
  }
  return kUnknownLoads;
}

// ---- FP8 tiles: global -> registers -> (dequantise) -> LDS ------------------------------------

// 4 latent chunks + (first two waves) 1 rope chunk of 16 codes per thread, and their row
// scales (0 for a row that is not real).
struct TileRegsFp8 {
  u32x4 v[5];
  float scale[5];
};

template <bool ALIGNED>
__device__ __forceinline__ void LoadTileFp8(TileRegsFp8& r, const AttnArgs& a, TileMap<ALIGNED>& map, int tile, int tid) {
  map.Begin(tile);
  int block[5], slot[5];
  bool real[5];
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int token = i < 4 ? (tid + kThreads * i) >> 5 : (tid & 127) >> 2;
    real[i] = map.Row(tile, token, &block[i], &slot[i]);
  }
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    if (i == 4 && tid >= 128) break;  // wave-uniform: 32 rope rows x 4 chunks
    const int chunk = i < 4 ? (tid + kThreads * i) & 31 : tid & 3;
    const Plane& plane = i < 4 ? a.latent : a.rope;
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
  for (int i = 0; i < 5; ++i) {
    if (i == 4 && tid >= 128) break;
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
    if (i < 4) {
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

// Online-softmax state of one wave: lane (head i16, token group g).
struct Softmax {
  float m_ref;   // reference maximum of the exponentials, log2 domain
  float l_run;   // this lane's share of the running denominator
  float x[8];    // scaled scores, then exponentials, of tokens 4g+j (x[0..3]) and 16+4g+j (x[4..7])
  float tile_max;
  bf16x8 p;
};

template <bool FP8, bool ALIGNED>
__global__ __launch_bounds__(kThreads, 1) void MlaDecodeKernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, i16 = lane & 15;
  const int chunk_index = blockIdx.x;
  const int seq = blockIdx.y;
  const int head_base = blockIdx.z * 64 + wave * 16;
  const bool active = head_base < a.heads;  // wave-uniform
  const int head = head_base + i16;
  const bool direct = a.max_chunks == 1;  // single chunk: write the final output here

  // Q fragments: lane (head i16, k-group g) holds Q[head][32*ks + 8g .. +7]. Issued first so
  // that they travel while the lengths and the block table are fetched.
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

  // Stage this chunk's block-table entries in LDS. The range is bounded by the chunk and the
  // table row, not by the sequence length, so it does not wait for the length to arrive;
  // entries past the sequence are never used.
  const int tile_begin = chunk_index * a.chunk_tiles;
  int* table_lds = reinterpret_cast<int*>(lds + kRing * kTileBytes);
  TileMap<ALIGNED> map;
  map.entries = table_lds;
  map.block_size = a.block_size;
  {
    const int first_pos = tile_begin * kTileTokens;
    const int last_pos = first_pos + a.chunk_tiles * kTileTokens - 1;
    map.first_block = first_pos / a.block_size;
    int count = last_pos / a.block_size - map.first_block + 1;  // <= kTableEntries, ensured by the plan
    count = min(count, a.table_stride - map.first_block);
    const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride + map.first_block;
    for (int i = tid; i < count; i += kThreads) {
      const int entry = table_row[i];
      table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : -1;
    }
  }
  // A length beyond what the table row can address is clamped: every position below it has a
  // staged entry.
  const int seq_len = static_cast<int>(
      min(static_cast<int64_t>(Uniform(a.seq_lens[seq])), static_cast<int64_t>(a.table_stride) * a.block_size));
  map.seq_len = seq_len;
  const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  if (tile_begin >= num_tiles) {
    if (direct && active) {  // empty sequence: zeros, lse = -inf
      char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
      for (int n = g; n < kLatentDim / 8; n += 4) *reinterpret_cast<u32x4*>(out + n * 16) = u32x4{0u, 0u, 0u, 0u};
      if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    }
    return;
  }
  const int ntiles = min(a.chunk_tiles, num_tiles - tile_begin);  // tiles of this chunk, >= 1

  f32x4 o[kDvTiles];
#pragma unroll
  for (int n = 0; n < kDvTiles; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  Softmax sm;
  sm.m_ref = 0.0f;
  sm.l_run = 0.0f;

  // Lane-constant LDS offsets.
  // K reads: token = 16t + i16, chunk = 4 ks + g (latent, ks < 16) or 4 (ks - 16) + g (rope).
  const int k_lat = i16 * kLatRowBytes, k_rope = kLatRegion + i16 * kRopeRowBytes;
  int k_e[4], kr_e[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) k_e[j] = ((4 * j + g) ^ SwizzleLat(i16)) << 4;
#pragma unroll
  for (int j = 0; j < 2; ++j) kr_e[j] = ((4 * j + g) ^ SwizzleRope(i16)) << 4;
  // V reads: token = (16 +) 4g + i16/4, chunk = 2n + (i16 & 3) / 2, 8-byte half i16 & 1.
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
    il.rope_chunk = ((lane & 7) ^ SwizzleRope(8 * w + (lane >> 3))) << 4;
    il.rope = (lane >> 3) * static_cast<int>(a.rope.row_stride) + il.rope_chunk;
  }

  const auto ring = [&](int i) __attribute__((always_inline)) { return (i & (kRing - 1)) * kTileBytes; };

  // K fragment of pipeline step `step` (k-step step/2, token subtile step&1) of the tile at `buf`.
  const auto k_frag = [&](const unsigned char* buf, int step) __attribute__((always_inline)) {
    const int ks = step >> 1, t = step & 1;
    const int offset = ks < 16 ? k_lat + (ks >> 2) * 256 + k_e[ks & 3] + t * 16 * kLatRowBytes
                               : k_rope + kr_e[ks & 1] + t * 16 * kRopeRowBytes;
    return *reinterpret_cast<const bf16x8*>(buf + offset);
  };
  // V^T fragment of output tile n (dv 16n..16n+15) over the 32 tokens of the tile at `buf`.
  const auto v_frag = [&](const unsigned char* buf, int n) __attribute__((always_inline)) {
    const unsigned char* addr = buf + v_lane + (n >> 3) * 256 + v_e[n & 7];
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr + 16 * kLatRowBytes));
    return __builtin_shufflevector(__builtin_bit_cast(bf16x4, lo), __builtin_bit_cast(bf16x4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
  };

  // The softmax of a tile is cut in two halves that hide behind different MFMA phases.
  // ScoreStep (behind the second product of the previous tile): scale, mask and the tile
  // maximum of fresh scores. ExpStep (behind the first product of the next tile): exponentials
  // against the reference maximum, denominator, bf16 P operand. Between the two, outside any
  // pipelined region, the reference maximum moves if it has to (rare; rescales O).
  const auto score_step = [&](auto step_c, const f32x4* s, int tile_rel) __attribute__((always_inline)) {
    constexpr int step = decltype(step_c)::value;
    if constexpr (step == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) sm.x[j] = s[0][j] * a.scale_log2;
    } else if constexpr (step == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j) sm.x[4 + j] = s[1][j] * a.scale_log2;
    } else if constexpr (step == 3) {
      const int valid = seq_len - (tile_begin + tile_rel) * kTileTokens;  // >= 1
      if (valid < kTileTokens) {  // wave-uniform: only the last tile of a sequence
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (16 * (j >> 2) + 4 * g + (j & 3) >= valid) sm.x[j] = -__builtin_inff();
        }
      }
    } else if constexpr (step == 4) {
      sm.tile_max = fmaxf(fmaxf(fmaxf(sm.x[0], sm.x[1]), fmaxf(sm.x[2], sm.x[3])),
                          fmaxf(fmaxf(sm.x[4], sm.x[5]), fmaxf(sm.x[6], sm.x[7])));
    } else if constexpr (step == 6) {
      sm.tile_max = MaxAcrossRows16(sm.tile_max);
    } else if constexpr (step == 8) {
      sm.tile_max = MaxAcrossHalves(sm.tile_max);
    }
  };
  constexpr int kScoreSteps = 9;
  const auto exp_step = [&](auto step_c) __attribute__((always_inline)) {
    constexpr int step = decltype(step_c)::value;
    if constexpr (step <= 6 && (step & 1) == 0) {
      sm.x[step] = __builtin_amdgcn_exp2f(sm.x[step] - sm.m_ref);
      sm.x[step + 1] = __builtin_amdgcn_exp2f(sm.x[step + 1] - sm.m_ref);
    } else if constexpr (step == 8) {
      sm.l_run += ((sm.x[0] + sm.x[1]) + (sm.x[2] + sm.x[3])) + ((sm.x[4] + sm.x[5]) + (sm.x[6] + sm.x[7]));
    } else if constexpr (step == 10) {
#pragma unroll
      for (int j = 0; j < 8; ++j) sm.p[j] = static_cast<__bf16>(sm.x[j]);
    }
  };
  constexpr int kExpSteps = 11;
  // Moves the reference maximum when some head's tile maximum outgrew it by more than the
  // threshold; O and the denominator are rescaled to the new reference.
  const auto move_reference = [&]() __attribute__((always_inline)) {
    if (__builtin_amdgcn_ballot_w64(sm.tile_max > sm.m_ref + kRescaleThreshold) != 0) {
      const float m_new = fmaxf(sm.m_ref, sm.tile_max);  // finite: token 0 of the tile is valid
      const float alpha = __builtin_amdgcn_exp2f(sm.m_ref - m_new);
      sm.l_run *= alpha;
      sm.m_ref = m_new;
#pragma unroll
      for (int n = 0; n < kDvTiles; ++n) o[n] *= alpha;
    }
  };

  // S^T of the tile at `buf` into s_out. With OVERLAP the exponentials of the previous tile
  // are spread over the steps and the first V fragments of `vbuf` are fetched at the tail.
  bf16x8 vf[kVAhead];
  const auto qk = [&](const unsigned char* buf, f32x4* s_out, auto overlap_c, const unsigned char* vbuf)
                      __attribute__((always_inline)) {
    constexpr bool overlap = decltype(overlap_c)::value;
    f32x4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    bf16x8 kf[kKAhead];
#pragma unroll
    for (int d = 0; d < kKAhead; ++d) kf[d] = k_frag(buf, d);
    __builtin_amdgcn_sched_barrier(0);
    StaticFor<kQkSteps>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int step = decltype(step_c)::value;
      constexpr int slot = (step & 1) * 2 + ((step >> 1) & 1);  // two accumulators per token subtile
      acc[slot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[step % kKAhead], q[step >> 1], acc[slot], 0, 0, 0);
      if constexpr (step + kKAhead < kQkSteps) {
        kf[step % kKAhead] = k_frag(buf, step + kKAhead);
      } else if constexpr (overlap && step + kKAhead - kQkSteps < kVAhead) {
        vf[step + kKAhead - kQkSteps] = v_frag(vbuf, step + kKAhead - kQkSteps);
      }
      if constexpr (overlap && step < kExpSteps) exp_step(step_c);
      __builtin_amdgcn_sched_barrier(0);
    });
    s_out[0] = acc[0] + acc[1];
    s_out[1] = acc[2] + acc[3];
  };

  // O^T += V^T P over the tile at `buf`; the first kVAhead fragments are already in vf. With
  // OVERLAP the scores `s_new` of tile `tile_rel` are scaled, masked and reduced to their maximum.
  const auto pv = [&](const unsigned char* buf, auto overlap_c, const f32x4* s_new, int tile_rel)
                      __attribute__((always_inline)) {
    constexpr bool overlap = decltype(overlap_c)::value;
    StaticFor<kDvTiles>([&](auto n_c) __attribute__((always_inline)) {
      constexpr int n = decltype(n_c)::value;
      o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[n % kVAhead], sm.p, o[n], 0, 0, 0);
      if constexpr (n + kVAhead < kDvTiles) vf[n % kVAhead] = v_frag(buf, n + kVAhead);
      if constexpr (overlap && n < kScoreSteps) score_step(n_c, s_new, tile_rel);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // The query must have arrived before the tile loads are issued: the compiler's own wait for
  // it would otherwise also wait for every tile load issued in between.
  if (active) {
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) asm volatile("" ::"v"(q[ks]));
  }
  __syncthreads();  // table entries visible

  // Prologue: tiles 0..2 on their way, tile 0 landed, S^T of tile 0.
  TileRegsFp8 regs;
  int newest_loads = kUnknownLoads;  // loads this wave issued for the newest tile in flight
  if (FP8) {
    LoadTileFp8(regs, a, map, tile_begin, tid);
    StoreTileFp8(regs, lds + ring(0), tid);
    if (1 < ntiles) {
      LoadTileFp8(regs, a, map, tile_begin + 1, tid);
      StoreTileFp8(regs, lds + ring(1), tid);
    }
    if (2 < ntiles) LoadTileFp8(regs, a, map, tile_begin + 2, tid);
  } else {
    int in_flight = 0;  // loads of tiles 1 and 2, when known
    bool known = true;
    IssueTileBf16(a, map, il, tile_begin, lds_base + ring(0), lds + ring(0), tid);
    for (int i = 1; i < 3 && i < ntiles; ++i) {
      newest_loads = IssueTileBf16(a, map, il, tile_begin + i, lds_base + ring(i), lds + ring(i), tid);
      known = known && newest_loads == kLoadsPerTile;
      in_flight += kLoadsPerTile;
    }
    WaitLoads(known ? in_flight : 0);
  }
  __syncthreads();
  if (active) {
    // S^T of tile 0 and its maximum, which becomes the first reference (O is still zero).
    f32x4 s_first[2];
    qk(lds + ring(0), s_first, std::false_type{}, nullptr);
    StaticFor<kScoreSteps>([&](auto step_c) __attribute__((always_inline)) { score_step(step_c, s_first, 0); });
    sm.m_ref = sm.tile_max;
  }

  for (int i = 0; i < ntiles; ++i) {
    // Tile i+1 must have landed; tile i+2 may still be in flight. The barrier also retires
    // every wave's reads of tile i-1, whose buffer tile i+3 reuses.
    if (i + 1 < ntiles) {
      if (!FP8) WaitLoads(i + 2 < ntiles && newest_loads == kLoadsPerTile ? kLoadsPerTile : 0);
      __syncthreads();
    }
    if (FP8) {
      if (i + 2 < ntiles) StoreTileFp8(regs, lds + ring(i + 2), tid);
      if (i + 3 < ntiles) LoadTileFp8(regs, a, map, tile_begin + i + 3, tid);
    } else if (i + 3 < ntiles) {
      newest_loads = IssueTileBf16(a, map, il, tile_begin + i + 3, lds_base + ring(i + 3), lds + ring(i + 3), tid);
    }
    if (active) {
      const unsigned char* cur = lds + ring(i);
      f32x4 s_next[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
      if (i + 1 < ntiles) {
        qk(lds + ring(i + 1), s_next, std::true_type{}, cur);  // + exponentials of tile i
      } else {
        StaticFor<kExpSteps>([&](auto step_c) __attribute__((always_inline)) { exp_step(step_c); });
#pragma unroll
        for (int d = 0; d < kVAhead; ++d) vf[d] = v_frag(cur, d);
      }
      pv(cur, std::true_type{}, s_next, i + 1);  // + scores of tile i+1 (unused after the last tile)
      if (i + 1 < ntiles) move_reference();
    }
  }

  if (!active) return;
  const float l_total = SumAcrossHeadLanes(sm.l_run);
  const float inv = 1.0f / l_total;
  const float lse2 = sm.m_ref + __builtin_amdgcn_logf(l_total);  // v_log_f32 is log2
  char* out_row;
  if (direct) {
    out_row = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
    if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = lse2 * 0.6931471805599453f;
  } else {
    const int64_t row = (static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head;
    out_row = a.partial_out + row * (kLatentDim * 2);
    if (g == 0) a.partial_lse[row] = lse2;
  }
#pragma unroll
  for (int n = 0; n < kDvTiles; ++n) {
    u32x2 packed;
    packed.x = PackBf16(o[n][0] * inv, o[n][1] * inv);
    packed.y = PackBf16(o[n][2] * inv, o[n][3] * inv);
    *reinterpret_cast<u32x2*>(out_row + (16 * n + 4 * g) * 2) = packed;
  }
}

// Merges the chunks of one (sequence, head): out = sum_c w_c O_c / sum_c w_c with
// w_c = 2^(lse2_c - max lse2). 256 threads = 4 heads x 64 lanes, 8 output columns per lane;
// the loads of up to eight chunks are issued before the first is used.
constexpr int kCombineHeads = 4;
__global__ __launch_bounds__(256) void MlaCombineKernel(AttnArgs a) {
  const int head = blockIdx.x * kCombineHeads + (threadIdx.x >> 6), seq = blockIdx.y;
  const int lane = threadIdx.x & 63;
  if (head >= a.heads) return;
  const int seq_len = static_cast<int>(
      min(static_cast<int64_t>(a.seq_lens[seq]), static_cast<int64_t>(a.table_stride) * a.block_size));  // as in the main kernel
  const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  const int chunks = min((num_tiles + a.chunk_tiles - 1) / a.chunk_tiles, a.max_chunks);
  char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride + lane * 16;
  if (chunks == 0) {
    *reinterpret_cast<u32x4*>(out) = u32x4{0u, 0u, 0u, 0u};
    if (a.lse != nullptr && lane == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    return;
  }
  const int64_t row0 = static_cast<int64_t>(seq) * a.max_chunks * a.heads + head;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
  float m = -__builtin_inff(), denom = 0.0f;
  for (int c0 = 0; c0 < chunks; c0 += 8) {
    u32x4 v[8];
    float l[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = min(c0 + u, chunks - 1);
      const int64_t row = row0 + static_cast<int64_t>(c) * a.heads;
      l[u] = c0 + u < chunks ? a.partial_lse[row] : -__builtin_inff();
      v[u] = GlobalLoad16(a.partial_out + row * (kLatentDim * 2) + lane * 16);
    }
    float group_max = m;
#pragma unroll
    for (int u = 0; u < 8; ++u) group_max = fmaxf(group_max, l[u]);
    const float rescale = __builtin_amdgcn_exp2f(m - group_max);  // 0 on the first group
    m = group_max;
    denom *= rescale;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= rescale;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float w = __builtin_amdgcn_exp2f(l[u] - m);  // 0 for the padding slots
      denom += w;
      const unsigned words[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] += w * __builtin_bit_cast(float, words[j] << 16);
        acc[2 * j + 1] += w * __builtin_bit_cast(float, words[j] & 0xffff0000u);
      }
    }
  }
  const float inv = 1.0f / denom;
  u32x4 packed;
  packed.x = PackBf16(acc[0] * inv, acc[1] * inv);
  packed.y = PackBf16(acc[2] * inv, acc[3] * inv);
  packed.z = PackBf16(acc[4] * inv, acc[5] * inv);
  packed.w = PackBf16(acc[6] * inv, acc[7] * inv);
  *reinterpret_cast<u32x4*>(out) = packed;
  if (a.lse != nullptr && lane == 0) a.lse[seq * a.heads + head] = (m + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f;
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

hipError_t LaunchAttnDecode(const AttnArgs& args, hipStream_t stream) {
  if (args.batch <= 0) return hipSuccess;
  const dim3 grid(args.max_chunks, args.batch, (args.heads + 63) / 64);
  const bool aligned = args.block_size % kTileTokens == 0;
  hipError_t e;
  if (args.fp8) e = aligned ? Launch<true, true>(args, grid, stream) : Launch<true, false>(args, grid, stream);
  else e = aligned ? Launch<false, true>(args, grid, stream) : Launch<false, false>(args, grid, stream);
  if (e != hipSuccess) return e;
  if (args.max_chunks > 1) {
    hipLaunchKernelGGL(MlaCombineKernel, dim3((args.heads + kCombineHeads - 1) / kCombineHeads, args.batch), dim3(256), 0,
                       stream, args);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace mlakv
