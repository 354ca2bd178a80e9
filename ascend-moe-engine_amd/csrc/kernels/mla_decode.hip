// Absorbed-MLA decode attention over the paged latent KV cache, gfx950 (CDNA4).
//
//   s_i = scale * (q_lat[h] . c_i + q_rope[h] . r_i),  p = softmax_i(s),  o[h] = sum_i p_i c_i
//
// One query token per sequence, all heads share one latent KV stream (MQA), so the
// head axis is the free MFMA dimension and the latent row is read from HBM once and used
// as both K (with the 64 rope columns appended) and V.
//
// Work decomposition
//   workgroup = (kv chunk, sequence, group of 64 heads), one workgroup per CU, 8 wavefronts in
//   two roles, one of each role per SIMD:
//     score waves 0..3 (16 heads each) hold the query in registers, compute S^T = K Q^T for a
//       tile, run the online softmax and publish P (bf16, already in MFMA operand layout)
//       through LDS, one tile ahead of
//     output waves 4..7, which hold the O accumulators and compute O^T += V^T P.
//   A single wave per SIMD is bound by instruction issue (one instruction per four cycles,
//   every stall exposed); with the two roles the softmax VALU work, the LDS traffic and the
//   MFMAs of neighbouring tiles overlap in hardware, and neither role has to hold both the
//   query (72 registers) and O (128 registers).
//   A chunk is `chunk_tiles` tiles of 32 tokens. LDS holds a ring of four tile buffers: while
//   tile i feeds the second product and tile i+1 the first, tiles i+2 and i+3 are in flight
//   from HBM. bf16 tiles are filled by direct global->LDS loads (global_load_lds_dwordx4: no
//   staging registers, no ds_write) issued by all eight waves; FP8 tiles are dequantised to
//   bf16 through registers on their way into LDS. One workgroup barrier per tile publishes
//   tile i+1 and P(i) and retires tile i-1.
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
//   So a score lane writes its eight P values as one 16-byte LDS store and the output lane
//   with the same lane id reads them back as its B operand; the online-softmax statistics of
//   a head live in the four lanes {h, h+16, h+32, h+48}: two v_permlane swaps per reduction.
//   Operand fragments are fetched several MFMAs ahead, with a scheduling fence per step.
//
// LDS tile: latent region 32 rows x 1024 B, then rope region 32 rows x 128 B; the 16-byte
//   chunk index inside a row is XORed with a function of the token (see SwizzleLat). With
//   direct loads the swizzle is applied on the global side: lane L of a row fetches chunk L ^ f.
//
// Online softmax keeps a reference maximum per head and only moves it when a tile's maximum
// exceeds it by more than 2^8, so exponentials stay below 256; when it moves, the score wave
// hands the factor to its output wave, which rescales O before adding the tile.
//
// Chunks of one sequence are merged by a second small kernel from partials (normalised O in
// bf16, log2-domain LSE in fp32) held in the caller's workspace.
#include <utility>

#include "kernels.h"

#pragma clang diagnostic ignored "-Winline-asm"

// Development timeline (built only with -DMLAKV_ATTN_TRACE): lane 0 of waves 0 and 4 of every
// workgroup stamps the 100 MHz wall clock into a caller-provided buffer.
#ifdef MLAKV_ATTN_TRACE
#include <cstdlib>
#define MLAKV_STAMP(slot)                                                                              \
  do {                                                                                                 \
    if (a.trace != nullptr && lane == 0 && (wave == 0 || wave == 4) && (slot) >= 0 && (slot) < 32) {                     \
      a.trace[((blockIdx.y * gridDim.x + blockIdx.x) * 2 + (wave >> 2)) * 32 + (slot)] = __builtin_amdgcn_s_memrealtime(); \
    }                                                                                                  \
  } while (0)
#else
#define MLAKV_STAMP(slot) \
  do {                    \
  } while (0)
#endif

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

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kScoreWaves = 4;
constexpr int kLatRowBytes = kLatentDim * 2;                 // 1024
constexpr int kRopeRowBytes = kRopeDim * 2;                  // 128
constexpr int kLatRegion = kTileTokens * kLatRowBytes;       // 32768
constexpr int kTileBytes = kLatRegion + kTileTokens * kRopeRowBytes;  // 36864
constexpr int kRing = 4;                                     // tile buffers in LDS
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;        // 18
constexpr int kQkSteps = 2 * kKSteps;                        // 36 MFMAs: 18 k-steps x 2 token subtiles
constexpr int kDvTiles = kLatentDim / 16;                    // 32
constexpr int kTableEntries = 1024;                          // block-table entries of one chunk staged in LDS
// LDS map after the ring.
constexpr int kTableOff = kRing * kTileBytes;                // int[kTableEntries]
constexpr int kPOff = kTableOff + kTableEntries * 4;         // P[2][4 waves][64 lanes] x 16 B
constexpr int kAlphaOff = kPOff + 2 * kScoreWaves * 64 * 16; // alpha[2][4][64] fp32
constexpr int kInvOff = kAlphaOff + 2 * kScoreWaves * 64 * 4;  // 1/denominator[4][64] fp32
constexpr int kFlagOff = kInvOff + kScoreWaves * 64 * 4;     // rescale flag[2][4] int
constexpr int kLdsBytes = kFlagOff + 64;
static_assert(kLdsBytes <= 160 * 1024, "one workgroup owns the LDS of a CU");
constexpr int kRowsPerWave = kTileTokens / kWaves;           // latent rows one wave fetches per tile
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
// ds_read_b64_tr_b16 32 lanes. Latent rows (1024 B): the 16-byte chunk index is XORed with a
// 4-bit function of the token, (g32 << 1) | (token >> 3 & 1). g32 picks the 32-byte slot inside
// a 256-byte window and is distinct over each of the token sets {0..7}, {8..15}, {0..3, 8..11}
// and {4..7, 12..15}: the transposed V reads of 32 lanes touch eight rows, and the measured
// conflict count says the hardware pairs lanes 0-15 with 32-47, not with 16-31. The low bit
// separates the two tokens that share a g32, so the 16 tokens of a K read land in 16 distinct
// 16-byte slots. Rope rows (128 B, two per 256 B): 3-bit XOR by token/2.
__device__ __forceinline__ int SwizzleLat(int token) {
  const int g32 = (token & 3) | ((((token >> 2) ^ (token >> 3)) & 1) << 2);
  return (g32 << 1) | ((token >> 3) & 1);
}
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
  // The base and the LDS address must sit in scalar registers whatever the compiler concluded
  // about their uniformity.
  const unsigned long long bits = reinterpret_cast<unsigned long long>(uniform_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits >> 32));
  const unsigned long long base = (static_cast<unsigned long long>(hi) << 32) | lo;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_offset), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
               : "memory", "m0");
}
__device__ __forceinline__ void DirectLoad16PerLane(const char* lane_pointer, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(lane_pointer), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
               : "memory", "m0");
}
// Waits until at most `tiles` later tiles' worth of this wave's loads are outstanding (loads
// complete in issue order); `per_tile` is 4 or 5 (waves that also fetch rope rows).
__device__ __forceinline__ void WaitLoads(int tiles, int per_tile) {
  if (tiles == 2 && per_tile == 4) {
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  } else if (tiles == 2 && per_tile == 5) {
    asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
  } else if (tiles == 1 && per_tile == 4) {
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  } else if (tiles == 1 && per_tile == 5) {
    asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
  int tile_block, tile_slot0;  // ALIGNED only: where the tile of the last Begin() sits
  int next_entry, next_slot0;  // ALIGNED only: cursor of the next tile (tiles are begun in order)

  // Tiles are begun in increasing order starting with the first tile of the chunk, so the
  // ALIGNED case walks a cursor instead of dividing.
  __device__ __forceinline__ void Begin(int tile) {
    if (ALIGNED) {
      tile_block = entries[next_entry];
      tile_slot0 = next_slot0;
      next_slot0 += kTileTokens;
      if (next_slot0 >= block_size) {
        next_slot0 = 0;
        ++next_entry;
      }
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

// Lane-constant byte offsets of the chunk a lane fetches for the rows its wave owns: wave w
// of 8 owns latent rows w, w+8, w+16, w+24 (row & 15 takes two values); waves 4..7 also own
// the rope rows 8(w-4) .. 8(w-4)+7.
struct IssueLane {
  int lat[2];      // latent rows w + 8i with i & 1 == j
  int rope;        // this lane's rope row and chunk, relative to the first rope row of the wave
  int rope_chunk;
};

__device__ __forceinline__ int LoadsPerTile(int wave) { return kRowsPerWave + (wave >= kScoreWaves ? 1 : 0); }

// Issues this wave's loads of one tile into the buffer at LDS address `buf`; rows that are not
// real are zero-filled instead. Returns true when the wave issues exactly LoadsPerTile(wave)
// loads (a full tile), false when the number is not known.
template <bool ALIGNED>
__device__ __forceinline__ bool IssueTileBf16(const AttnArgs& a, TileMap<ALIGNED>& map, const IssueLane& il, int tile,
                                              unsigned buf, unsigned char* buf_ptr, int tid) {
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  const bool rope_wave = wave >= kScoreWaves;
  const int rope_group = wave - kScoreWaves;
  map.Begin(tile);
  const int rows = map.seq_len - tile * kTileTokens;  // real rows in this tile, >= 1
  if (ALIGNED && rows >= kTileTokens && map.tile_block >= 0) {
    // The whole tile is real and sits in one physical block: uniform base + row pitch.
    const int block = Uniform(map.tile_block), slot0 = Uniform(map.tile_slot0);
    const char* latent = a.latent.base + block * a.latent.block_stride + (slot0 + wave) * a.latent.row_stride;
    const int64_t pitch = kWaves * a.latent.row_stride;
    const char* rope = a.rope.base + block * a.rope.block_stride + (slot0 + 8 * rope_group) * a.rope.row_stride;
#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) DirectLoad16(latent + i * pitch, il.lat[i & 1], buf + (wave + kWaves * i) * kLatRowBytes);
    if (rope_wave) DirectLoad16(rope, il.rope, buf + kLatRegion + rope_group * 8 * kRopeRowBytes);
    return true;
  }
  // Rare path (last tile of a sequence, unaligned block sizes, bad table entries): one row at a
  // time, kept as a loop so that it costs little code.
  bool all_real = true;
#pragma nounroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int row = wave + kWaves * i;  // wave-uniform
    int block, slot;
    const bool real = map.Row(tile, row, &block, &slot);
    all_real = all_real && real;
    if (real) {
      const char* src = a.latent.base + Uniform(block) * a.latent.block_stride + Uniform(slot) * a.latent.row_stride;
      DirectLoad16(src, (lane ^ SwizzleLat(row)) << 4, buf + row * kLatRowBytes);
    } else {
      *reinterpret_cast<u32x4*>(buf_ptr + row * kLatRowBytes + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }
  if (!rope_wave) return all_real;
  // rope: one wave access covers 8 rows x 128 B, each lane resolving its own row
  int rblock, rslot;
  const bool rreal = map.Row(tile, 8 * rope_group + (lane >> 3), &rblock, &rslot);
  const char* rsrc = a.rope.base + rblock * a.rope.block_stride + rslot * a.rope.row_stride + il.rope_chunk;
  const unsigned rdst = buf + kLatRegion + rope_group * 8 * kRopeRowBytes;
  if (__builtin_amdgcn_ballot_w64(!rreal) == 0) {
    DirectLoad16PerLane(rsrc, rdst);
    return all_real;
  }
  if (rreal) {
    DirectLoad16PerLane(rsrc, rdst);
  } else {
    *reinterpret_cast<u32x4*>(buf_ptr + kLatRegion + rope_group * 8 * kRopeRowBytes + lane * 16) = u32x4{0u, 0u, 0u, 0u};
  }
  return false;
}

// ---- FP8 tiles: global -> registers -> (dequantise) -> LDS ------------------------------------

// 2 latent chunks + (first two waves) 1 rope chunk of 16 codes per thread, and their row
// scales (0 for a row that is not real).
struct TileRegsFp8 {
  u32x4 v[3];
  float scale[3];
};

template <bool ALIGNED>
__device__ __forceinline__ void LoadTileFp8(TileRegsFp8& r, const AttnArgs& a, TileMap<ALIGNED>& map, int tile, int tid) {
  map.Begin(tile);
  int block[3], slot[3];
  bool real[3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int token = i < 2 ? (tid + kThreads * i) >> 5 : (tid & 127) >> 2;
    real[i] = map.Row(tile, token, &block[i], &slot[i]);
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    if (i == 2 && tid >= 128) break;  // wave-uniform: 32 rope rows x 4 chunks
    const int chunk = i < 2 ? (tid + kThreads * i) & 31 : tid & 3;
    const Plane& plane = i < 2 ? a.latent : a.rope;
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
  for (int i = 0; i < 3; ++i) {
    if (i == 2 && tid >= 128) break;
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
    if (i < 2) {
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
__global__ __launch_bounds__(kThreads) void MlaDecodeKernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  const bool score_wave = wave < kScoreWaves;   // wave-uniform role
  const int hw = wave & (kScoreWaves - 1);      // which 16 heads of the 64
  const int g = lane >> 4, i16 = lane & 15;
  const int chunk_index = blockIdx.x;
  const int seq = blockIdx.y;
  const int head_base = blockIdx.z * 64 + hw * 16;
  const bool active = head_base < a.heads;  // wave-uniform
  const int head = head_base + i16;
  const bool direct = a.max_chunks == 1;  // single chunk: write the final output here
  const int per_tile = LoadsPerTile(wave);
  MLAKV_STAMP(0);

  // Q fragments (score waves): lane (head i16, k-group g) holds Q[head][32*ks + 8g .. +7].
  // Issued first so that they travel while the lengths and the block table are fetched.
  bf16x8 q[kKSteps];
  if (score_wave && active) {
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
  int* table_lds = reinterpret_cast<int*>(lds + kTableOff);
  TileMap<ALIGNED> map;
  map.entries = table_lds;
  map.block_size = a.block_size;
  {
    const int first_pos = tile_begin * kTileTokens;
    const int last_pos = first_pos + a.chunk_tiles * kTileTokens - 1;
    map.first_block = first_pos / a.block_size;
    map.next_entry = 0;
    map.next_slot0 = first_pos - map.first_block * a.block_size;
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
    if (active && direct) {  // empty sequence: zeros, lse = -inf
      if (score_wave) {
        if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
      } else {
        char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
        for (int n = g; n < kLatentDim / 8; n += 4) *reinterpret_cast<u32x4*>(out + n * 16) = u32x4{0u, 0u, 0u, 0u};
      }
    } else if (active && score_wave && g == 0) {  // empty chunk: the merge reads every chunk's LSE
      a.partial_lse[(static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head] = -__builtin_inff();
    }
    return;
  }
  const int ntiles = min(a.chunk_tiles, num_tiles - tile_begin);  // tiles of this chunk, >= 1

  // Direct loads: lane L of a latent row fetches chunk L ^ swizzle(row); rows of this wave.
  IssueLane il;
#pragma unroll
  for (int j = 0; j < 2; ++j) il.lat[j] = (lane ^ SwizzleLat(wave + kWaves * j)) << 4;
  il.rope_chunk = ((lane & 7) ^ SwizzleRope(8 * (wave - kScoreWaves) + (lane >> 3))) << 4;
  il.rope = (lane >> 3) * static_cast<int>(a.rope.row_stride) + il.rope_chunk;

  const auto ring = [&](int i) __attribute__((always_inline)) { return (i & (kRing - 1)) * kTileBytes; };

  // The query must have arrived before the tile loads are issued: the compiler's own wait for
  // it would otherwise also wait for every tile load issued in between.
  if (score_wave && active) {
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) asm volatile("" ::"v"(q[ks]));
  }
  MLAKV_STAMP(1);
  __syncthreads();  // table entries visible

  // Prologue: tiles 0..2 on their way, tile 0 landed and published.
  TileRegsFp8 regs;
  bool newest_known = false;  // the newest tile in flight took exactly per_tile loads of this wave
  if (FP8) {
    LoadTileFp8(regs, a, map, tile_begin, tid);
    StoreTileFp8(regs, lds + ring(0), tid);
    if (1 < ntiles) {
      LoadTileFp8(regs, a, map, tile_begin + 1, tid);
      StoreTileFp8(regs, lds + ring(1), tid);
    }
    if (2 < ntiles) LoadTileFp8(regs, a, map, tile_begin + 2, tid);
  } else {
    int in_flight = 0;  // tiles 1 and 2
    bool known = true;
    IssueTileBf16(a, map, il, tile_begin, lds_base + ring(0), lds + ring(0), tid);
    for (int i = 1; i < 3 && i < ntiles; ++i) {
      newest_known = IssueTileBf16(a, map, il, tile_begin + i, lds_base + ring(i), lds + ring(i), tid);
      known = known && newest_known;
      ++in_flight;
    }
    MLAKV_STAMP(2);
    WaitLoads(known ? in_flight : 0, per_tile);
  }
  __syncthreads();
  MLAKV_STAMP(3);

  // Top of iteration i, both roles: tile i+1 must have landed (tile i+2 may still be in
  // flight); the barrier publishes it together with P(i) and retires every wave's reads of
  // tile i-1, whose ring slot tile i+3 then reuses.
  const auto advance = [&](int i) __attribute__((always_inline)) {
    MLAKV_STAMP(4 + 6 * i);
    if (!FP8 && i + 1 < ntiles) WaitLoads(i + 2 < ntiles && newest_known ? 1 : 0, per_tile);
    __syncthreads();
    MLAKV_STAMP(5 + 6 * i);
    if (FP8) {
      if (i + 2 < ntiles) StoreTileFp8(regs, lds + ring(i + 2), tid);
      if (i + 3 < ntiles) LoadTileFp8(regs, a, map, tile_begin + i + 3, tid);
    } else if (i + 3 < ntiles) {
      newest_known = IssueTileBf16(a, map, il, tile_begin + i + 3, lds_base + ring(i + 3), lds + ring(i + 3), tid);
    }
    MLAKV_STAMP(6 + 6 * i);
  };

  unsigned char* p_lds = lds + kPOff + (hw * 64 + lane) * 16;           // + parity * kScoreWaves * 64 * 16
  float* alpha_lds = reinterpret_cast<float*>(lds + kAlphaOff) + hw * 64 + lane;  // + parity * kScoreWaves * 64
  float* inv_lds = reinterpret_cast<float*>(lds + kInvOff) + hw * 64 + lane;
  int* flag_lds = reinterpret_cast<int*>(lds + kFlagOff) + hw;          // + parity * kScoreWaves

  if (score_wave) {
    // ---------------------------------------------------------------- score waves
    // K reads: token = 16t + i16, chunk = 4 ks + g (latent, ks < 16) or 4 (ks - 16) + g (rope).
    const int k_lat = i16 * kLatRowBytes, k_rope = kLatRegion + i16 * kRopeRowBytes;
    int k_e[4], kr_e[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) k_e[j] = ((4 * j + g) ^ SwizzleLat(i16)) << 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) kr_e[j] = ((4 * j + g) ^ SwizzleRope(i16)) << 4;
    // K fragment of pipeline step `step` (k-step step/2, token subtile step&1) of the tile at `buf`.
    const auto k_frag = [&](const unsigned char* buf, int step) __attribute__((always_inline)) {
      const int ks = step >> 1, t = step & 1;
      const int offset = ks < 16 ? k_lat + (ks >> 2) * 256 + k_e[ks & 3] + t * 16 * kLatRowBytes
                                 : k_rope + kr_e[ks & 1] + t * 16 * kRopeRowBytes;
      return *reinterpret_cast<const bf16x8*>(buf + offset);
    };

    float m_ref = -__builtin_inff();  // reference maximum of the exponentials, log2 domain
    float l_run = 0.0f;               // this lane's share of the running denominator

    // S^T of tile `tile_rel`, its softmax against the running reference, P and the rescale
    // request into the LDS slots of the tile's parity.
    const auto score_tile = [&](int tile_rel) __attribute__((always_inline)) {
      const unsigned char* buf = lds + ring(tile_rel);
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
        if constexpr (step + kKAhead < kQkSteps) kf[step % kKAhead] = k_frag(buf, step + kKAhead);
        __builtin_amdgcn_sched_barrier(0);
      });
      MLAKV_STAMP(7 + 6 * (tile_rel - 1));
      // lane holds tokens 4g+j (x[0..3]) and 16+4g+j (x[4..7]) of head i16
      float x[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = (acc[0][j] + acc[1][j]) * a.scale_log2;
        x[4 + j] = (acc[2][j] + acc[3][j]) * a.scale_log2;
      }
      const int valid = seq_len - (tile_begin + tile_rel) * kTileTokens;  // >= 1
      if (valid < kTileTokens) {  // wave-uniform: only the last tile of a sequence
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (16 * (j >> 2) + 4 * g + (j & 3) >= valid) x[j] = -__builtin_inff();
        }
      }
      float tile_max = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
      tile_max = MaxAcrossHalves(MaxAcrossRows16(tile_max));
      const int parity = tile_rel & 1;
      // Move the reference only when some head's maximum outgrew it by more than the threshold.
      const bool moved = __builtin_amdgcn_ballot_w64(tile_max > m_ref + kRescaleThreshold) != 0;
      if (moved) {
        const float m_new = fmaxf(m_ref, tile_max);  // finite: token 0 of the tile is valid
        const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
        l_run *= alpha;
        m_ref = m_new;
        alpha_lds[parity * kScoreWaves * 64] = alpha;
      }
      if (lane == 0) flag_lds[parity * kScoreWaves] = moved && tile_rel != 0 ? 1 : 0;  // O is still zero on the first tile
      bf16x8 p;
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = __builtin_amdgcn_exp2f(x[j] - m_ref);
        sum += e;
        p[j] = static_cast<__bf16>(e);
      }
      l_run += sum;
      *reinterpret_cast<bf16x8*>(p_lds + parity * kScoreWaves * 64 * 16) = p;
      MLAKV_STAMP(8 + 6 * (tile_rel - 1));
    };

    if (active) score_tile(0);
    for (int i = 0; i < ntiles; ++i) {
      advance(i);
      if (active && i + 1 < ntiles) score_tile(i + 1);
    }
    if (active) {
      const float l_total = SumAcrossHeadLanes(l_run);
      *inv_lds = 1.0f / l_total;
      const float lse2 = m_ref + __builtin_amdgcn_logf(l_total);  // v_log_f32 is log2
      if (g == 0) {
        if (direct) {
          if (a.lse != nullptr) a.lse[seq * a.heads + head] = lse2 * 0.6931471805599453f;
        } else {
          a.partial_lse[(static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head] = lse2;
        }
      }
    }
    MLAKV_STAMP(29);
    __syncthreads();  // 1/denominator visible to the output waves
    MLAKV_STAMP(30);
  } else {
    // ---------------------------------------------------------------- output waves
    // V reads: token = (16 +) 4g + i16/4, chunk = 2n + (i16 & 3) / 2, 8-byte half i16 & 1.
    const int v_row = 4 * g + (i16 >> 2);
    const int v_lane = v_row * kLatRowBytes + (i16 & 1) * 8;
    int v_e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v_e[j] = ((2 * j + ((i16 & 3) >> 1)) ^ SwizzleLat(v_row)) << 4;
    // V^T fragment of output tile n (dv 16n..16n+15) over the 32 tokens of the tile at `buf`.
    const auto v_frag = [&](const unsigned char* buf, int n) __attribute__((always_inline)) {
      const unsigned char* addr = buf + v_lane + (n >> 3) * 256 + v_e[n & 7];
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr + 16 * kLatRowBytes));
      return __builtin_shufflevector(__builtin_bit_cast(bf16x4, lo), __builtin_bit_cast(bf16x4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
    };

    f32x4 o[kDvTiles];
#pragma unroll
    for (int n = 0; n < kDvTiles; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int i = 0; i < ntiles; ++i) {
      advance(i);
      if (active) {
        const unsigned char* buf = lds + ring(i);
        const int parity = i & 1;
        bf16x8 vf[kVAhead];
#pragma unroll
        for (int d = 0; d < kVAhead; ++d) vf[d] = v_frag(buf, d);
        const bf16x8 p = *reinterpret_cast<const bf16x8*>(p_lds + parity * kScoreWaves * 64 * 16);
        if (Uniform(flag_lds[parity * kScoreWaves]) != 0) {  // the reference maximum moved: rescale O first
          const float alpha = alpha_lds[parity * kScoreWaves * 64];
#pragma unroll
          for (int n = 0; n < kDvTiles; ++n) o[n] *= alpha;
        }
        __builtin_amdgcn_sched_barrier(0);
        StaticFor<kDvTiles>([&](auto n_c) __attribute__((always_inline)) {
          constexpr int n = decltype(n_c)::value;
          o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[n % kVAhead], p, o[n], 0, 0, 0);
          if constexpr (n + kVAhead < kDvTiles) vf[n % kVAhead] = v_frag(buf, n + kVAhead);
          __builtin_amdgcn_sched_barrier(0);
        });
        MLAKV_STAMP(7 + 6 * i);
      }
    }
    MLAKV_STAMP(29);
    __syncthreads();  // 1/denominator from the score waves
    MLAKV_STAMP(30);
    if (active) {
      const float inv = *inv_lds;
      char* out_row;
      if (direct) {
        out_row = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
      } else {
        const int64_t row = (static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head;
        out_row = a.partial_out + row * (kLatentDim * 2);
      }
#pragma unroll
      for (int n = 0; n < kDvTiles; ++n) {
        u32x2 packed;
        packed.x = PackBf16(o[n][0] * inv, o[n][1] * inv);
        packed.y = PackBf16(o[n][2] * inv, o[n][3] * inv);
        __builtin_nontemporal_store(packed, reinterpret_cast<u32x2*>(out_row + (16 * n + 4 * g) * 2));
      }
    }
    MLAKV_STAMP(31);
  }
}

// Merges the chunks of one (sequence, head): out = sum_c w_c O_c / sum_c w_c with
// w_c = 2^(lse2_c - max lse2). 256 threads = 4 heads x 64 lanes, 8 output columns per lane.
// Every chunk slot carries an LSE (-inf for a chunk past the end of its sequence, whose O slot
// was never written), so all loads of a group of eight chunks are issued at once, with no
// dependence on the sequence length.
constexpr int kCombineHeads = 4;
__global__ __launch_bounds__(256) void MlaCombineKernel(AttnArgs a) {
  const int head = blockIdx.x * kCombineHeads + (threadIdx.x >> 6), seq = blockIdx.y;
  const int lane = threadIdx.x & 63;
  if (head >= a.heads) return;
  const int chunks = a.max_chunks;
  const int64_t row0 = static_cast<int64_t>(seq) * chunks * a.heads + head;
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
      v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.partial_out + row * (kLatentDim * 2) + lane * 16));
    }
    float group_max = m;
#pragma unroll
    for (int u = 0; u < 8; ++u) group_max = fmaxf(group_max, l[u]);
    if (group_max == -__builtin_inff()) continue;  // nothing but empty chunks so far
    const float rescale = __builtin_amdgcn_exp2f(m - group_max);  // 0 on the first group
    m = group_max;
    denom *= rescale;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= rescale;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (l[u] == -__builtin_inff()) continue;  // empty or padding slot: its O bytes are not data
      const float w = __builtin_amdgcn_exp2f(l[u] - m);
      denom += w;
      const unsigned words[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] += w * __builtin_bit_cast(float, words[j] << 16);
        acc[2 * j + 1] += w * __builtin_bit_cast(float, words[j] & 0xffff0000u);
      }
    }
  }
  char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride + lane * 16;
  if (denom == 0.0f) {  // empty sequence
    *reinterpret_cast<u32x4*>(out) = u32x4{0u, 0u, 0u, 0u};
    if (a.lse != nullptr && lane == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    return;
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

hipError_t LaunchAttnDecode(const AttnArgs& args_in, hipStream_t stream) {
  AttnArgs args = args_in;
#ifdef MLAKV_ATTN_TRACE
  args.trace = std::getenv("MLAKV_ATTN_TRACE_PTR") ? reinterpret_cast<unsigned long long*>(std::strtoull(std::getenv("MLAKV_ATTN_TRACE_PTR"), nullptr, 0)) : nullptr;
#endif
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
