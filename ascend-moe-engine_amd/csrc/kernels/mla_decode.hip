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
#include <mutex>
#include <utility>

#include "kernels.h"
#include "mx_quant_device.h"

#pragma clang diagnostic ignored "-Winline-asm"

// Development timeline (built only with -DMLAKV_ATTN_TRACE): lane 0 of every wave of every
// workgroup stamps the 100 MHz wall clock into a caller-provided buffer.
#ifdef MLAKV_ATTN_TRACE
#include <cstdlib>
#define MLAKV_STAMP(slot)                                                                              \
  do {                                                                                                 \
    if (a.trace != nullptr && lane == 0 && (slot) >= 0 && (slot) < 40) {                                                 \
      a.trace[((blockIdx.y * gridDim.x + blockIdx.x) * 8 + wave) * 40 + (slot)] = __builtin_amdgcn_s_memrealtime();       \
    }                                                                                                  \
  } while (0)
#else
#define MLAKV_STAMP(slot) \
  do {                    \
  } while (0)
#endif

namespace mlakv {
namespace {

constexpr int kXcds = 8;
constexpr bool kLateIssue = true;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kScoreWaves = 4;
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;        // 18
constexpr int kQkSteps = 2 * kKSteps;                        // 36 MFMAs: 18 k-steps x 2 token subtiles
constexpr int kDvTiles = kLatentDim / 16;                    // 32
constexpr int kTableEntries = 1024;                          // block-table entries of one chunk staged in LDS
static_assert(kTileTokens == 32, "the fragment maps below are written for 32-token tiles");

// LDS geometry. A bf16 tile is 32 latent rows of 1024 B followed by 32 rope rows of 128 B. An
// FP8 tile keeps the E4M3 codes as they are in the cache (32 x 512 B, 32 x 64 B) followed by the
// 32 fp32 row scales, padded to a multiple of 512 B so that the XOR-swizzled part of an address
// can be formed before the tile base is added. The bf16 ring is as deep as the 160 KB allow; the
// FP8 ring could hold seven tiles and measured fastest with five.
template <bool FP8>
struct Geom {
  static constexpr int kLatRow = FP8 ? kLatentDim : kLatentDim * 2;
  static constexpr int kRopeRow = FP8 ? kRopeDim : kRopeDim * 2;
  static constexpr int kLatRegion = kTileTokens * kLatRow;
  static constexpr int kScaleOff = kLatRegion + kTileTokens * kRopeRow;  // FP8 only
  static constexpr int kTileBytes = FP8 ? ((kScaleOff + kTileTokens * 4 + 511) / 512) * 512 : kScaleOff;
  static constexpr int kRing = FP8 ? 5 : 4;
  static constexpr int kTableOff = kRing * kTileBytes;                 // int[kTableEntries]
  static constexpr int kPOff = kTableOff + kTableEntries * 4;          // P[2][4 waves][64 lanes] x 16 B
  static constexpr int kAlphaOff = kPOff + 2 * kScoreWaves * 64 * 16;  // alpha[2][4][64] fp32
  static constexpr int kInvOff = kAlphaOff + 2 * kScoreWaves * 64 * 4; // 1/denominator[4][64] fp32
  static constexpr int kFlagOff = kInvOff + kScoreWaves * 64 * 4;      // rescale flag[2][4] int
  static constexpr int kLdsBytes = kFlagOff + 64;
  static_assert(kLdsBytes <= 160 * 1024, "one workgroup owns the LDS of a CU");
  __device__ static __forceinline__ int Slot(int i) { return (kRing == 4 ? (i & 3) : (i % kRing)) * kTileBytes; }
};
constexpr int kRowsPerWave = kTileTokens / kWaves;           // bf16: latent rows one wave fetches per tile
constexpr float kRescaleThreshold = 8.0f;                    // log2 domain
constexpr int kKAhead = 8;                                   // bf16 K fragments in flight ahead of their MFMA
constexpr int kKAhead8 = 4;                                  // FP8 K reads (two fragments each) in flight
constexpr int kVAhead = 3;                                   // V fragments in flight (of the eight an output wave fetches per tile)

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
// FP8 rows (512 B of codes): 4-bit XOR that is distinct over 16 consecutive tokens (K reads) and
// over the token sets {0..3, 8..11, 16..19, 24..27} and {4..7, 12..15, 20..23, 28..31} (the rows
// 32 lanes of a transposed 8-bit V read touch). Rope rows (64 B, four per 256 B): XOR by token/4.
__device__ __forceinline__ int SwizzleLat8(int token) { return (token & 15) ^ ((token >> 4) << 2); }
__device__ __forceinline__ int SwizzleRope8(int token) { return (token >> 2) & 3; }

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
// Waits until at most `newer` of this wave's vector-memory loads are outstanding (loads complete
// in issue order; the count is an immediate of s_waitcnt, hence the switch).
__device__ __forceinline__ void WaitLoads(int newer) {
  switch (newer) {
#define MLAKV_WAIT_CASE(n) \
  case n:                  \
    asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory"); \
    break;
    MLAKV_WAIT_CASE(1) MLAKV_WAIT_CASE(2) MLAKV_WAIT_CASE(3) MLAKV_WAIT_CASE(4) MLAKV_WAIT_CASE(5) MLAKV_WAIT_CASE(6)
    MLAKV_WAIT_CASE(7) MLAKV_WAIT_CASE(8) MLAKV_WAIT_CASE(9) MLAKV_WAIT_CASE(10) MLAKV_WAIT_CASE(11) MLAKV_WAIT_CASE(12)
    MLAKV_WAIT_CASE(13) MLAKV_WAIT_CASE(14) MLAKV_WAIT_CASE(15) MLAKV_WAIT_CASE(16) MLAKV_WAIT_CASE(17) MLAKV_WAIT_CASE(18)
    MLAKV_WAIT_CASE(19) MLAKV_WAIT_CASE(20) MLAKV_WAIT_CASE(21) MLAKV_WAIT_CASE(22) MLAKV_WAIT_CASE(23) MLAKV_WAIT_CASE(24)
#undef MLAKV_WAIT_CASE
    default:
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
__device__ __forceinline__ unsigned UMaxAcrossHeadLanes(unsigned bits) {
  u32x2 swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  unsigned a = swapped.x, b = swapped.y;
  bits = max(a, b);
  swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  a = swapped.x;
  b = swapped.y;
  return max(a, b);
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
  // Selected-token mode (never ALIGNED): `entries` holds, for each of the chunk's selected tokens
  // from position `first_pos` of the selection on, the linear pool slot of that token (-1: behind
  // a bad table entry), and `seq_len` is the number of selected tokens.
  bool sparse;
  int first_pos;
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
    if (sparse) {
      const int linear = pos < seq_len ? entries[pos - first_pos] : -1;
      const int usable = linear < 0 ? 0 : linear;
      *block = usable / block_size;
      *slot = usable - *block * block_size;
      return linear >= 0;
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
  int partner_lat[2];  // the same for the rows of wave w - 4 (output waves only)
  int rope;        // this lane's rope row and chunk, relative to the first rope row of the wave
  int rope_chunk;
};

__device__ __forceinline__ int LoadsPerTile(int wave) { return kRowsPerWave + (wave >= kScoreWaves ? 1 : 0); }

// Issues this wave's loads of one tile into the buffer at LDS address `buf`; rows that are not
// real are zero-filled instead. Returns true when the wave issues exactly LoadsPerTile(wave)
// loads (a full tile), false when the number is not known.
// WITH_PARTNER: an output wave also fetches the latent rows of the score wave it is paired with
// (wave - kScoreWaves), for the tiles that the output waves issue alone.
template <bool ALIGNED, bool WITH_PARTNER = false>
__device__ __forceinline__ bool IssueTileBf16(const AttnArgs& a, TileMap<ALIGNED>& map, const IssueLane& il, int tile,
                                              unsigned buf, unsigned char* buf_ptr, int tid) {
  using G = Geom<false>;
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
    for (int i = 0; i < kRowsPerWave; ++i) DirectLoad16(latent + i * pitch, il.lat[i & 1], buf + (wave + kWaves * i) * G::kLatRow);
    if (WITH_PARTNER) {
      const char* partner = latent - kScoreWaves * a.latent.row_stride;
#pragma unroll
      for (int i = 0; i < kRowsPerWave; ++i) {
        DirectLoad16(partner + i * pitch, il.partner_lat[i & 1], buf + (wave - kScoreWaves + kWaves * i) * G::kLatRow);
      }
    }
    if (rope_wave) DirectLoad16(rope, il.rope, buf + G::kLatRegion + rope_group * 8 * G::kRopeRow);
    return true;
  }
  // Rare path (last tile of a sequence, unaligned block sizes, bad table entries): one row at a
  // time, kept as a loop so that it costs little code.
  bool all_real = true;
#pragma nounroll
  for (int i = 0; i < (WITH_PARTNER ? 2 : 1) * kRowsPerWave; ++i) {
    // wave-uniform; with a partner the wave walks rows (wave - 4) + 4 i, its partner's and its own in turn
    const int row = WITH_PARTNER ? wave - kScoreWaves + kScoreWaves * i : wave + kWaves * i;
    int block, slot;
    const bool real = map.Row(tile, row, &block, &slot);
    all_real = all_real && real;
    if (real) {
      const char* src = a.latent.base + Uniform(block) * a.latent.block_stride + Uniform(slot) * a.latent.row_stride;
      DirectLoad16(src, (lane ^ SwizzleLat(row)) << 4, buf + row * G::kLatRow);
    } else {
      *reinterpret_cast<u32x4*>(buf_ptr + row * G::kLatRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }
  if (!rope_wave) return all_real;
  // rope: one wave access covers 8 rows x 128 B, each lane resolving its own row
  int rblock, rslot;
  const bool rreal = map.Row(tile, 8 * rope_group + (lane >> 3), &rblock, &rslot);
  const char* rsrc = a.rope.base + rblock * a.rope.block_stride + rslot * a.rope.row_stride + il.rope_chunk;
  const unsigned rdst = buf + G::kLatRegion + rope_group * 8 * G::kRopeRow;
  if (__builtin_amdgcn_ballot_w64(!rreal) == 0) {
    DirectLoad16PerLane(rsrc, rdst);
    return all_real;
  }
  if (rreal) {
    DirectLoad16PerLane(rsrc, rdst);
  } else {
    *reinterpret_cast<u32x4*>(buf_ptr + G::kLatRegion + rope_group * 8 * G::kRopeRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
  }
  return false;
}

// ---- FP8 tiles: direct global -> LDS, codes and row scales as they are in the cache -------------

// Wave w of 8 owns the latent row pairs {2w, 2w+1} and {16+2w, 17+2w} (a 512-byte row is half a
// wave access); waves 4 and 5 also own the rope rows 16(w-4) .. +15 (64 B each), wave 6 the 32
// row scales (128 B, eight lanes).
struct IssueLane8 {
  int lat[2];  // byte offset of this lane's chunk from the first row of pair i
  int rope;
};

__device__ __forceinline__ int LoadsPerTile8(int wave) { return 2 + (wave >= 4 && wave <= 6 ? 1 : 0); }

// FP8 counterpart of IssueTileBf16. The rare path stages through registers; rows that are not
// real get zero codes and a zero scale.
template <bool ALIGNED>
__device__ __forceinline__ bool IssueTileFp8(const AttnArgs& a, TileMap<ALIGNED>& map, const IssueLane8& il, int tile,
                                             unsigned buf, unsigned char* buf_ptr, int tid) {
  using G = Geom<true>;
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  map.Begin(tile);
  const int rows = map.seq_len - tile * kTileTokens;  // real rows in this tile, >= 1
  if (ALIGNED && rows >= kTileTokens && map.tile_block >= 0) {
    const int block = Uniform(map.tile_block), slot0 = Uniform(map.tile_slot0);
    const char* latent = a.latent.base + block * a.latent.block_stride + (slot0 + 2 * wave) * a.latent.row_stride;
    const int64_t pitch = 16 * a.latent.row_stride;
#pragma unroll
    for (int i = 0; i < 2; ++i) DirectLoad16(latent + i * pitch, il.lat[i], buf + (2 * wave + 16 * i) * G::kLatRow);
    if (wave == 4 || wave == 5) {
      const int h = wave - 4;
      const char* rope = a.rope.base + block * a.rope.block_stride + (slot0 + 16 * h) * a.rope.row_stride;
      DirectLoad16(rope, il.rope, buf + G::kLatRegion + 16 * h * G::kRopeRow);
    } else if (wave == 6) {
      const char* scale = a.scale.base + block * a.scale.block_stride + slot0 * 4;
      if (lane < kTileTokens * 4 / 16) DirectLoad16(scale, lane * 16, buf + G::kScaleOff);
    }
    return true;
  }
#pragma nounroll
  for (int i = 0; i < 2; ++i) {
    const int row = 2 * wave + 16 * i + (lane >> 5);
    int block, slot;
    const bool real = map.Row(tile, row, &block, &slot);
    u32x4 codes = GlobalLoad16(a.latent.base + block * a.latent.block_stride + slot * a.latent.row_stride + (lane & 31) * 16);
    if (!real) codes = u32x4{0u, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(buf_ptr + row * G::kLatRow + (((lane & 31) ^ SwizzleLat8(row)) << 4)) = codes;
  }
  if (wave == 4 || wave == 5) {
    const int row = 16 * (wave - 4) + (lane >> 2);
    int block, slot;
    const bool real = map.Row(tile, row, &block, &slot);
    u32x4 codes = GlobalLoad16(a.rope.base + block * a.rope.block_stride + slot * a.rope.row_stride + (lane & 3) * 16);
    if (!real) codes = u32x4{0u, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(buf_ptr + G::kLatRegion + row * G::kRopeRow + (((lane & 3) ^ SwizzleRope8(row)) << 4)) = codes;
  } else if (wave == 6 && lane < kTileTokens) {
    int block, slot;
    const bool real = map.Row(tile, lane, &block, &slot);
    const float scale = reinterpret_cast<const float*>(a.scale.base + block * a.scale.block_stride)[slot];
    reinterpret_cast<float*>(buf_ptr + G::kScaleOff)[lane] = real ? scale : 0.0f;
  }
  return false;
}

__device__ __forceinline__ unsigned int PackBf16(float lo, float hi) {
  const bf16x2 packed = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(unsigned int, packed);
}

// Eight E4M3 codes (two dwords) -> eight bf16, exactly (unit scale; the row scale is applied to
// the scores and to P instead, in fp32).
__device__ __forceinline__ bf16x8 CodesToBf16(unsigned lo, unsigned hi) {
  const bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
  const bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
  const bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
  const bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
  return bf16x8{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
}

// ---- main kernel -------------------------------------------------------------------

// MXQ: the single-chunk launch also quantises its output (and its bf16 output is optional). Kept
// out of the common instantiation, whose register allocation has no room to spare.
// SPARSE: the sequence attends to the tokens listed in a.sparse_indices instead of to its whole
// context (never ALIGNED: every row is located on its own).
template <bool FP8, bool ALIGNED, bool MXQ, bool SPARSE>
__global__ __launch_bounds__(kThreads) void MlaDecodeKernel(AttnArgs a) {
  static_assert(!(SPARSE && (ALIGNED || MXQ)), "selected-token attention uses the row-at-a-time path");
  // bf16 tiles: the output waves, which have no query to wait for, issue the first tiles of the
  // ring alone (their own rows and those of their partner score waves) as soon as they know the
  // block-table entries; the score waves join from the first loop iteration on.
  constexpr bool kSoloPrologue = !FP8 && !SPARSE;
  using G = Geom<FP8>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  const bool score_wave = wave < kScoreWaves;   // wave-uniform role
  const int hw = wave & (kScoreWaves - 1);      // which 16 heads of the 64
  const int g = lane >> 4, i16 = lane & 15;
  // Workgroups are handed to the eight XCDs round-robin by linear id, and each XCD has its own
  // L2. The chunks of one sequence all read the same 72 KB of Q, so they are placed on one XCD:
  // XCD x takes the contiguous range of (sequence, chunk) pairs [x, x+1) * pairs / 8.
  int chunk_index = blockIdx.x;
  int seq = blockIdx.y;
  {
    const int pairs = gridDim.x * gridDim.y;
    if ((pairs & (kXcds - 1)) == 0) {
      const int linear = blockIdx.y * gridDim.x + blockIdx.x;
      const int pair = (linear & (kXcds - 1)) * (pairs / kXcds) + linear / kXcds;
      seq = pair / static_cast<int>(gridDim.x);
      chunk_index = pair - seq * static_cast<int>(gridDim.x);
    }
  }
  const int head_base = blockIdx.z * 64 + hw * 16;
  const bool active = head_base < a.heads;  // wave-uniform
  const int head = head_base + i16;
  const bool direct = a.max_chunks == 1;  // single chunk: write the final output here
  const int per_tile = FP8 ? LoadsPerTile8(wave) : LoadsPerTile(wave);
  MLAKV_STAMP(0);

  // Q fragments (score waves): lane (head i16, k-group g) holds, for k-step ks, the eight query
  // elements that meet the lane's K fragment of that step: Q[head][32 ks + 8g .. +7] for bf16
  // tiles; for FP8 tiles one 16-byte K read feeds two k-steps, so the order inside each 64-wide
  // window is Q[head][64 (ks/2) + 16g + 8 (ks&1) .. +7]. (Loaded further down, once the
  // lengths and table entries have been asked for.)
  bf16x8 q[kKSteps];
  const auto load_q = [&]() __attribute__((always_inline)) {
    const char* q_latent = a.q_latent + seq * a.q_latent_seq_stride + head * a.q_latent_head_stride;
    const char* q_rope = a.q_rope + seq * a.q_rope_seq_stride + head * a.q_rope_head_stride;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      const int d0 = FP8 ? 64 * (ks >> 1) + 16 * g + 8 * (ks & 1) : 32 * ks + 8 * g;
      const char* p = d0 < kLatentDim ? q_latent + d0 * 2 : q_rope + (d0 - kLatentDim) * 2;
      q[ks] = __builtin_bit_cast(bf16x8, GlobalLoad16(p));
    }
  };

  // Stage this chunk's block-table entries in LDS. The range is bounded by the chunk and the
  // table row, not by the sequence length, so it does not wait for the length to arrive;
  // entries past the sequence are never used.
  const int tile_begin = chunk_index * a.chunk_tiles;
  int* table_lds = reinterpret_cast<int*>(lds + G::kTableOff);
  TileMap<ALIGNED> map;
  map.entries = table_lds;
  map.block_size = a.block_size;
  map.sparse = SPARSE;
  map.first_pos = tile_begin * kTileTokens;
  if constexpr (!SPARSE) {
    const int first_pos = tile_begin * kTileTokens;
    const int last_pos = first_pos + a.chunk_tiles * kTileTokens - 1;
    map.first_block = first_pos / a.block_size;
    map.next_entry = 0;
    map.next_slot0 = first_pos - map.first_block * a.block_size;
    int count = last_pos / a.block_size - map.first_block + 1;  // <= kTableEntries, ensured by the plan
    count = min(count, a.table_stride - map.first_block);
    const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride + map.first_block;
    // kSoloPrologue: every wave stages all entries itself (the same values to the same
    // addresses), so that it can read them back without waiting for the other waves.
    for (int i = kSoloPrologue ? lane : tid; i < count; i += kSoloPrologue ? 64 : kThreads) {
      const int entry = table_row[i];
      table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : -1;
    }
  }
  MLAKV_STAMP(34);
  // A length beyond what the table row can address is clamped: every position below it has a
  // staged entry.
  int seq_len = static_cast<int>(
      min(static_cast<int64_t>(Uniform(a.seq_lens[seq])), static_cast<int64_t>(a.table_stride) * a.block_size));
  if constexpr (SPARSE) {
    // The selection ends at its first entry that is negative or not inside the context. Then
    // this chunk's part of it is resolved to pool slots through the block table.
    const int context = seq_len;
    const int32_t* selection = a.sparse_indices + static_cast<int64_t>(seq) * a.sparse_seq_stride;
    int* count_lds = reinterpret_cast<int*>(lds + G::kFlagOff) + 2 * kScoreWaves;
    if (tid == 0) *count_lds = a.sparse_count;
    __syncthreads();
    for (int i = tid; i < a.sparse_count; i += kThreads) {
      const int index = selection[i];
      if (index < 0 || index >= context) atomicMin(count_lds, i);
    }
    __syncthreads();
    seq_len = Uniform(*count_lds);
    const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;
    const int chunk_tokens = min(a.chunk_tiles * kTileTokens, seq_len - map.first_pos);  // <= kTableEntries, ensured by the plan
    for (int i = tid; i < chunk_tokens; i += kThreads) {
      const int index = selection[map.first_pos + i];  // inside [0, context): before the end of the selection
      const int logical = index / a.block_size;
      const int entry = table_row[logical];
      table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks)
                         ? entry * a.block_size + (index - logical * a.block_size)
                         : -1;
    }
  }
  map.seq_len = seq_len;
  MLAKV_STAMP(33);
  // Vector memory requests of a CU are served in order: the query (72 KB per workgroup) is asked
  // for only now, behind the few bytes of lengths and table entries that the first tile
  // addresses depend on.
  if (score_wave && active) load_q();
  MLAKV_STAMP(32);
  const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  if (tile_begin >= num_tiles) {
    if (active && direct) {  // empty sequence: zeros, lse = -inf
      if (score_wave) {
        if (a.lse != nullptr && g == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
      } else {
        if (!MXQ || a.out != nullptr) {
          char* out = a.out + seq * a.out_seq_stride + head * a.out_head_stride;
          for (int n = g; n < kLatentDim / 8; n += 4) *reinterpret_cast<u32x4*>(out + n * 16) = u32x4{0u, 0u, 0u, 0u};
        }
        if constexpr (MXQ) {  // zeros quantise to zero codes under the smallest scale
          char* codes = a.out_codes + seq * a.out_codes_seq_stride + head * a.out_codes_head_stride;
          for (int n = g; n < kLatentDim / 16; n += 4) *reinterpret_cast<u32x4*>(codes + n * 16) = u32x4{0u, 0u, 0u, 0u};
          if (g == 0) *reinterpret_cast<u32x4*>(a.out_scales + seq * a.out_scales_seq_stride + head * a.out_scales_head_stride) = u32x4{0u, 0u, 0u, 0u};
        }
      }
    } else if (active && score_wave && g == 0) {  // empty chunk: the merge reads every chunk's LSE
      a.partial_lse[(static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + head] = -__builtin_inff();
    }
    return;
  }
  const int ntiles = min(a.chunk_tiles, num_tiles - tile_begin);  // tiles of this chunk, >= 1

  // Direct loads: lane L of a latent row fetches chunk L ^ swizzle(row); rows of this wave.
  IssueLane il;
  IssueLane8 il8;
  if (FP8) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = 2 * wave + 16 * j + (lane >> 5);
      il8.lat[j] = (lane >> 5) * static_cast<int>(a.latent.row_stride) + (((lane & 31) ^ SwizzleLat8(row)) << 4);
    }
    const int rope_row = 16 * (wave & 1) + (lane >> 2);
    il8.rope = (lane >> 2) * static_cast<int>(a.rope.row_stride) + (((lane & 3) ^ SwizzleRope8(rope_row)) << 4);
  } else {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      il.lat[j] = (lane ^ SwizzleLat(wave + kWaves * j)) << 4;
      il.partner_lat[j] = (lane ^ SwizzleLat((wave & (kScoreWaves - 1)) + kWaves * j)) << 4;
    }
    il.rope_chunk = ((lane & 7) ^ SwizzleRope(8 * (wave - kScoreWaves) + (lane >> 3))) << 4;
    il.rope = (lane >> 3) * static_cast<int>(a.rope.row_stride) + il.rope_chunk;
  }

  const auto ring = [&](int i) __attribute__((always_inline)) { return G::Slot(i); };
  // Issues this wave's loads of chunk-relative tile t; returns whether their number is known.
  const auto issue = [&](int t) __attribute__((always_inline)) {
    if constexpr (FP8) {
      return IssueTileFp8(a, map, il8, tile_begin + t, lds_base + ring(t), lds + ring(t), tid);
    } else {
      return IssueTileBf16(a, map, il, tile_begin + t, lds_base + ring(t), lds + ring(t), tid);
    }
  };

  // The query must have arrived before this wave issues tile loads: the compiler's own wait for
  // it would otherwise also wait for every tile load issued in between.
  MLAKV_STAMP(35);
  // Every wave passes through it, whether it asked for the query or not: were it skipped on
  // some path, the compiler would have to assume the query still in flight wherever the paths
  // meet again, and would wait for it -- with counts that know nothing of the tile loads, so in
  // effect for every tile in flight -- inside the score loop, at every use.
#pragma unroll
  for (int ks = 0; ks < kKSteps; ++ks) asm volatile("" ::"v"(q[ks]));
  MLAKV_STAMP(1);
  if constexpr (!kSoloPrologue) __syncthreads();  // table entries visible

  // Prologue: tiles 0 .. kRing-2 on their way, tile 0 landed and published. A tile whose load
  // count is not known (rare path) makes every wait up to and including its own a full one.
  int last_unknown = -1;  // newest tile issued with an unknown number of loads
  int issued = 0;         // tiles issued so far
  for (; issued < G::kRing - 1 && issued < ntiles; ++issued) {
    if constexpr (kSoloPrologue) {
      if (score_wave) {
        map.Begin(issued);  // keeps the cursor in step with the tiles this wave does not issue
      } else if (!IssueTileBf16<ALIGNED, true>(a, map, il, tile_begin + issued, lds_base + ring(issued), lds + ring(issued), tid)) {
        last_unknown = issued;
      }
    } else {
      if (!issue(issued)) last_unknown = issued;
    }
  }
  // Loads this wave has in flight that are newer than those of tile t: the first `solo_tiles`
  // tiles carry `solo_loads` each, the later ones `per_tile`.
  const int solo_tiles = kSoloPrologue ? issued : 0;
  const int solo_loads = score_wave ? 0 : per_tile + kRowsPerWave;
  const auto newer_than = [&](int t) __attribute__((always_inline)) {
    const int solo = max(0, min(issued, solo_tiles) - (t + 1));
    const int shared = max(0, issued - max(t + 1, solo_tiles));
    return solo * solo_loads + shared * per_tile;
  };
  MLAKV_STAMP(2);
  WaitLoads(last_unknown >= 0 ? 0 : newer_than(0));
  __syncthreads();
  MLAKV_STAMP(3);

  // Top of iteration i, both roles: tile i+1 must have landed (later tiles may still be in
  // flight); the barrier publishes it together with P(i) and retires every wave's reads of
  // tile i-1, whose ring slot the next tile to be issued reuses.
  const auto publish = [&](int i) __attribute__((always_inline)) {
    MLAKV_STAMP((i) < 4 ? 4 + 6 * (i) : -1);
    if (i + 1 < ntiles) WaitLoads(last_unknown >= i + 1 ? 0 : newer_than(i + 1));
    __syncthreads();
    MLAKV_STAMP((i) < 4 ? 5 + 6 * (i) : -1);
  };
  // Issues the next tile of the ring (tile i + kRing - 1 during iteration i), right after
  // publish(i): the memory-bound shapes want every load in flight as early as possible (issuing
  // after the score waves' MFMA phase, to skew the two MFMA phases of a SIMD, gained 6 % where
  // the kernel is compute-bound and lost 4 % where it is not).
  const auto issue_next = [&](int i) __attribute__((always_inline)) {
    if (issued < ntiles) {
      if (!issue(issued)) last_unknown = issued;
      ++issued;
    }
    MLAKV_STAMP((i) < 4 ? 6 + 6 * (i) : -1);
  };

  unsigned char* p_lds = lds + G::kPOff + (hw * 64 + lane) * 16;           // + parity * kScoreWaves * 64 * 16
  float* alpha_lds = reinterpret_cast<float*>(lds + G::kAlphaOff) + hw * 64 + lane;  // + parity * kScoreWaves * 64
  float* inv_lds = reinterpret_cast<float*>(lds + G::kInvOff) + hw * 64 + lane;
  int* flag_lds = reinterpret_cast<int*>(lds + G::kFlagOff) + hw;          // + parity * kScoreWaves

  if (score_wave) {
    // ---------------------------------------------------------------- score waves
    // bf16 K reads: token = 16t + i16, chunk = 4 ks + g (latent, ks < 16) or 4 (ks - 16) + g (rope).
    const int k_lat = i16 * Geom<false>::kLatRow, k_rope = Geom<false>::kLatRegion + i16 * Geom<false>::kRopeRow;
    int k_e[4], kr_e[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) k_e[j] = ((4 * j + g) ^ SwizzleLat(i16)) << 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) kr_e[j] = ((4 * j + g) ^ SwizzleRope(i16)) << 4;
    // K fragment of pipeline step `step` (k-step step/2, token subtile step&1) of the tile at `buf`.
    const auto k_frag = [&](const unsigned char* buf, int step) __attribute__((always_inline)) {
      const int ks = step >> 1, t = step & 1;
      const int offset = ks < 16 ? k_lat + (ks >> 2) * 256 + k_e[ks & 3] + t * 16 * Geom<false>::kLatRow
                                 : k_rope + kr_e[ks & 1] + t * 16 * Geom<false>::kRopeRow;
      return *reinterpret_cast<const bf16x8*>(buf + offset);
    };
    // FP8 K reads: read u = 2 kp + t fetches the 16 codes k = 64 kp + 16 g .. +15 of token 16t + i16
    // (k-steps 2kp and 2kp+1): chunk (4 kp + g) ^ swizzle(token) of the 512-byte row; kp = 8 is the
    // rope row (chunk g ^ swizzle). The tile base is a multiple of 512, so the XOR with kp << 6 is
    // applied to the lane-constant part.
    int k8_lat[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) k8_lat[t] = (16 * t + i16) * Geom<true>::kLatRow + ((g ^ SwizzleLat8(16 * t + i16)) << 4);
    const int k8_rope = Geom<true>::kLatRegion + i16 * Geom<true>::kRopeRow + ((g ^ SwizzleRope8(i16)) << 4);
    const auto k8_read = [&](const unsigned char* buf, int u) __attribute__((always_inline)) {
      const int kp = u >> 1, t = u & 1;
      const int offset = kp < 8 ? (k8_lat[t] ^ (kp << 6)) : k8_rope + t * 16 * Geom<true>::kRopeRow;
      return *reinterpret_cast<const u32x4*>(buf + offset);
    };

    float m_ref = -__builtin_inff();  // reference maximum of the exponentials, log2 domain
    float l_run = 0.0f;               // this lane's share of the running denominator

    // S^T of tile `tile_rel`, its softmax against the running reference, P and the rescale
    // request into the LDS slots of the tile's parity.
    const auto score_tile = [&](int tile_rel, int issue_iteration) __attribute__((always_inline)) {
      const unsigned char* buf = lds + ring(tile_rel);
      f32x4 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      f32x4 row_scale[2];  // FP8: scales of tokens 4g+j and 16+4g+j
      if constexpr (FP8) {
        const float* scales = reinterpret_cast<const float*>(buf + G::kScaleOff);
        row_scale[0] = *reinterpret_cast<const f32x4*>(scales + 4 * g);
        row_scale[1] = *reinterpret_cast<const f32x4*>(scales + 16 + 4 * g);
        u32x4 kr[kKAhead8];
#pragma unroll
        for (int d = 0; d < kKAhead8; ++d) kr[d] = k8_read(buf, d);
        __builtin_amdgcn_sched_barrier(0);
        StaticFor<kKSteps>([&](auto u_c) __attribute__((always_inline)) {
          constexpr int u = decltype(u_c)::value;  // kp = u / 2, token subtile t = u & 1
          const u32x4 codes = kr[u % kKAhead8];
          if constexpr (u + kKAhead8 < kKSteps) kr[u % kKAhead8] = k8_read(buf, u + kKAhead8);
          constexpr int t = u & 1, kp = u >> 1;
          acc[2 * t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(CodesToBf16(codes.x, codes.y), q[2 * kp], acc[2 * t], 0, 0, 0);
          acc[2 * t + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(CodesToBf16(codes.z, codes.w), q[2 * kp + 1], acc[2 * t + 1], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
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
      }
      MLAKV_STAMP(tile_rel >= 1 && tile_rel <= 4 ? 7 + 6 * (tile_rel - 1) : -1);
      if (kLateIssue && issue_iteration >= 0) issue_next(issue_iteration);
      // lane holds tokens 4g+j (x[0..3]) and 16+4g+j (x[4..7]) of head i16
      float x[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = (acc[0][j] + acc[1][j]) * a.scale_log2;
        x[4 + j] = (acc[2][j] + acc[3][j]) * a.scale_log2;
        if constexpr (FP8) {  // the codes were multiplied unscaled
          x[j] *= row_scale[0][j];
          x[4 + j] *= row_scale[1][j];
        }
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
        p[j] = static_cast<__bf16>(FP8 ? e * row_scale[j >> 2][j & 3] : e);  // FP8: V is multiplied unscaled as well
      }
      l_run += sum;
      *reinterpret_cast<bf16x8*>(p_lds + parity * kScoreWaves * 64 * 16) = p;
      MLAKV_STAMP(tile_rel >= 1 && tile_rel <= 4 ? 8 + 6 * (tile_rel - 1) : -1);
    };

    if (active) score_tile(0, -1);
    for (int i = 0; i < ntiles; ++i) {
      publish(i);
      const bool scores = active && i + 1 < ntiles;
      if (!kLateIssue || !scores) issue_next(i);
      if (scores) score_tile(i + 1, i);
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
    // bf16 V reads: token = (16 +) 4g + i16/4, chunk = 2n + (i16 & 3) / 2, 8-byte half i16 & 1.
    const int v_row = 4 * g + (i16 >> 2);
    const int v_lane = v_row * Geom<false>::kLatRow + (i16 & 1) * 8;
    int v_e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v_e[j] = ((2 * j + ((i16 & 3) >> 1)) ^ SwizzleLat(v_row)) << 4;
    // FP8 V reads (ds_read_b64_tr_b8: output lane i of a 16-lane group, element e <- byte i & 7 of
    // the 8 bytes addressed by lane 2e + (i >> 3)): as a source, lane j addresses bytes
    // 16n + 8 (j & 1) .. +7 of the row of token kappa = j >> 1 (tokens 4g + kappa, 16 + 4g + kappa - 4).
    const int v8_token = 4 * g + ((i16 >> 1) & 3) + 16 * (i16 >> 3);
    const int v8_base = v8_token * Geom<true>::kLatRow + (SwizzleLat8(v8_token) << 4) + 8 * (i16 & 1);
    // Raw V^T fragment of output tile n (dv 16n..16n+15) over the 32 tokens of the tile at `buf`:
    // eight bf16 for bf16 tiles, eight codes in the low two dwords for FP8 tiles.
    const auto v_fetch = [&](const unsigned char* buf, int n) __attribute__((always_inline)) {
      if constexpr (FP8) {
        const i32x2 codes = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(buf + (v8_base ^ (n << 4))));
        return u32x4{static_cast<unsigned>(codes.x), static_cast<unsigned>(codes.y), 0u, 0u};
      } else {
        const unsigned char* addr = buf + v_lane + (n >> 3) * 256 + v_e[n & 7];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr + 16 * Geom<false>::kLatRow));
        return __builtin_bit_cast(u32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    const auto v_operand = [&](const u32x4& raw) __attribute__((always_inline)) {
      if constexpr (FP8) {
        return CodesToBf16(raw.x, raw.y);
      } else {
        return __builtin_bit_cast(bf16x8, raw);
      }
    };

    // Output wave w owns the 128 output columns [128 w, 128 w + 128) of all 64 heads of the group:
    // every V^T fragment is then fetched (and, for FP8, converted) by one wave only, and meets the
    // P fragments of the four score waves. (With one head block per output wave, each of the four
    // read and converted all of V.) Head blocks past the group's heads are computed on whatever
    // their LDS slots hold and never written.
    constexpr int kDvPerWave = kDvTiles / (kWaves - kScoreWaves);
    const int hba = min(kScoreWaves, (a.heads - static_cast<int>(blockIdx.z) * 64 + 15) >> 4);  // head blocks in use
    const unsigned char* p_all = lds + G::kPOff + lane * 16;                                   // + (parity * 4 + hb) * 64 * 16
    const float* alpha_all = reinterpret_cast<const float*>(lds + G::kAlphaOff) + lane;      // + (parity * 4 + hb) * 64
    const float* inv_all = reinterpret_cast<const float*>(lds + G::kInvOff) + lane;          // + hb * 64
    const int* flag_all = reinterpret_cast<const int*>(lds + G::kFlagOff);                   // [parity * 4 + hb]
    f32x4 o[kScoreWaves][kDvPerWave];
#pragma unroll
    for (int hb = 0; hb < kScoreWaves; ++hb) {
#pragma unroll
      for (int n = 0; n < kDvPerWave; ++n) o[hb][n] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    for (int i = 0; i < ntiles; ++i) {
      publish(i);
      issue_next(i);
      {
        const unsigned char* buf = lds + ring(i);
        const int parity = i & 1;
        // the four rescale flags of the tile in one read; a moved reference maximum is the exception
        const i32x4 flags = *reinterpret_cast<const i32x4*>(flag_all + parity * kScoreWaves);
        if (Uniform(flags.x | flags.y | flags.z | flags.w) != 0) {
          const int moved[kScoreWaves] = {flags.x, flags.y, flags.z, flags.w};
#pragma unroll
          for (int hb = 0; hb < kScoreWaves; ++hb) {
            if (Uniform(moved[hb]) != 0) {  // that block's reference maximum moved: rescale its O first
              const float alpha = alpha_all[(parity * kScoreWaves + hb) * 64];
#pragma unroll
              for (int n = 0; n < kDvPerWave; ++n) o[hb][n] *= alpha;
            }
          }
        }
        u32x4 vf[kVAhead];
#pragma unroll
        for (int d = 0; d < kVAhead; ++d) vf[d] = v_fetch(buf, kDvPerWave * hw + d);
        bf16x8 p[kScoreWaves];
#pragma unroll
        for (int hb = 0; hb < kScoreWaves; ++hb) p[hb] = *reinterpret_cast<const bf16x8*>(p_all + (parity * kScoreWaves + hb) * 64 * 16);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (FP8) {
          // the next fragment is converted while this one's four MFMAs run
          bf16x8 v = v_operand(vf[0]);
          if constexpr (kVAhead < kDvPerWave) vf[0] = v_fetch(buf, kDvPerWave * hw + kVAhead);
          StaticFor<kDvPerWave>([&](auto n_c) __attribute__((always_inline)) {
            constexpr int n = decltype(n_c)::value;
            bf16x8 v_next = v;
            if constexpr (n + 1 < kDvPerWave) v_next = v_operand(vf[(n + 1) % kVAhead]);
#pragma unroll
            for (int hb = 0; hb < kScoreWaves; ++hb) o[hb][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, p[hb], o[hb][n], 0, 0, 0);
            if constexpr (n + 1 + kVAhead < kDvPerWave) vf[(n + 1) % kVAhead] = v_fetch(buf, kDvPerWave * hw + n + 1 + kVAhead);
            v = v_next;
            __builtin_amdgcn_sched_barrier(0);
          });
        } else {
          StaticFor<kDvPerWave>([&](auto n_c) __attribute__((always_inline)) {
            constexpr int n = decltype(n_c)::value;
            const bf16x8 v = v_operand(vf[n % kVAhead]);
#pragma unroll
            for (int hb = 0; hb < kScoreWaves; ++hb) o[hb][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, p[hb], o[hb][n], 0, 0, 0);
            if constexpr (n + kVAhead < kDvPerWave) vf[n % kVAhead] = v_fetch(buf, kDvPerWave * hw + n + kVAhead);
            __builtin_amdgcn_sched_barrier(0);
          });
        }
        MLAKV_STAMP((i) < 4 ? 7 + 6 * (i) : -1);
      }
    }
    MLAKV_STAMP(29);
    __syncthreads();  // 1/denominator from the score waves
    MLAKV_STAMP(30);
    const int group_head0 = static_cast<int>(blockIdx.z) * 64;
    // Row (bf16 [512]) of head `h` of this group in the launch's output: the final output when
    // there is one chunk, this chunk's partial otherwise.
    const auto row_of = [&](int h) __attribute__((always_inline)) -> char* {
      if (direct) return a.out + seq * a.out_seq_stride + (group_head0 + h) * a.out_head_stride;
      const int64_t row = (static_cast<int64_t>(seq) * a.max_chunks + chunk_index) * a.heads + group_head0 + h;
      return a.partial_out + row * (kLatentDim * 2);
    };
    if (MXQ && direct) {
      // Quantising epilogue of the single-chunk case: a block of 32 columns is a pair of this
      // wave's column tiles over the four lanes that share a head; the wave covers blocks
      // 4 w .. 4 w + 3 of every head.
#pragma unroll
      for (int hb = 0; hb < kScoreWaves; ++hb) {
        if (hb >= hba) continue;
        const int h = 16 * hb + i16;
        const float inv = inv_all[hb * 64];
        char* codes_row = a.out_codes + seq * a.out_codes_seq_stride + (group_head0 + h) * a.out_codes_head_stride;
        char* out_row = a.out == nullptr ? nullptr : row_of(h);
        unsigned scale_codes = 0u;
#pragma unroll
        for (int k = 0; k < kDvPerWave / 2; ++k) {
          u32x2 packed[2];
          unsigned magnitude = 0u;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int n = 2 * k + half;
            packed[half].x = PackBf16(o[hb][n][0] * inv, o[hb][n][1] * inv);
            packed[half].y = PackBf16(o[hb][n][2] * inv, o[hb][n][3] * inv);
            magnitude = MxMagnitudeMax(packed[half].y, MxMagnitudeMax(packed[half].x, magnitude));
            if (out_row != nullptr) {
              __builtin_nontemporal_store(packed[half], reinterpret_cast<u32x2*>(out_row + (16 * (kDvPerWave * hw + n) + 4 * g) * 2));
            }
          }
          magnitude = UMaxAcrossHeadLanes(magnitude);
          const MxScale s = MxScaleFromMaxBits(magnitude);
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const unsigned four = MxEncodeWord(packed[half].x, s) | (MxEncodeWord(packed[half].y, s) << 16);
            __builtin_nontemporal_store(four, reinterpret_cast<unsigned*>(codes_row + 16 * (kDvPerWave * hw + 2 * k + half) + 4 * g));
          }
          scale_codes |= s.code << (8 * k);
        }
        if (g == 0) {
          *reinterpret_cast<unsigned*>(a.out_scales + seq * a.out_scales_seq_stride + (group_head0 + h) * a.out_scales_head_stride +
                                       (kDvPerWave / 2) * hw) = scale_codes;
        }
      }
    } else {
      // The accumulators hold O^T (lane = head i16 of a block, four columns per 16-column tile),
      // which stored as it is would write 8-byte pieces of sixteen different rows per
      // instruction. The tile ring is dead after the last barrier: each output wave transposes
      // its 256-byte slices of the 64 rows through its own part of it and writes them 16 bytes per
      // lane, four whole slices per instruction. A row stride of 272 bytes (= 4 banks mod 64)
      // spreads the 8-byte writes of a half-wave over all banks.
      constexpr int kSliceBytes = kDvPerWave * 16 * 2;  // 256
      constexpr int kStageRow = kSliceBytes + 16;
      static_assert((kWaves - kScoreWaves) * 64 * kStageRow <= G::kRing * G::kTileBytes, "the staging rows fit in the ring");
      unsigned char* stage = lds + G::Slot(0) + hw * (64 * kStageRow);
#pragma unroll
      for (int hb = 0; hb < kScoreWaves; ++hb) {
        const float inv = inv_all[hb * 64];
#pragma unroll
        for (int n = 0; n < kDvPerWave; ++n) {
          u32x2 packed;
          packed.x = PackBf16(o[hb][n][0] * inv, o[hb][n][1] * inv);
          packed.y = PackBf16(o[hb][n][2] * inv, o[hb][n][3] * inv);
          *reinterpret_cast<u32x2*>(stage + (16 * hb + i16) * kStageRow + (16 * n + 4 * g) * 2) = packed;
        }
      }
      // Same wave wrote and reads: the LDS queue is in order, no barrier needed.
      const int piece = lane & 15, sub = lane >> 4;
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        const int h = 4 * it + sub;
        if (h < 16 * hba) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(stage + h * kStageRow + piece * 16);
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(row_of(h) + kSliceBytes * hw + piece * 16));
        }
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
__global__ __launch_bounds__(kCombineHeads * 64) void MlaCombineKernel(AttnArgs a) {
  // Workgroups go to the XCDs round-robin by linear id; the main kernel put all chunks of a
  // sequence on XCD seq / (batch / 8), and the partials are most likely still in that L2.
  int group = blockIdx.x, seq = blockIdx.y;
  if ((gridDim.y & (kXcds - 1)) == 0) {
    const int linear = blockIdx.y * gridDim.x + blockIdx.x;
    const int within = linear / kXcds;
    seq = (linear & (kXcds - 1)) * (gridDim.y / kXcds) + within / static_cast<int>(gridDim.x);
    group = within % static_cast<int>(gridDim.x);
  }
  const int head = group * kCombineHeads + (threadIdx.x >> 6);
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
  // An empty sequence (no live chunk) yields zeros and lse = -inf.
  const float inv = denom == 0.0f ? 0.0f : 1.0f / denom;
  u32x4 packed;
  packed.x = PackBf16(acc[0] * inv, acc[1] * inv);
  packed.y = PackBf16(acc[2] * inv, acc[3] * inv);
  packed.z = PackBf16(acc[4] * inv, acc[5] * inv);
  packed.w = PackBf16(acc[6] * inv, acc[7] * inv);
  if (a.out != nullptr) *reinterpret_cast<u32x4*>(a.out + seq * a.out_seq_stride + head * a.out_head_stride + lane * 16) = packed;
  if (a.out_codes != nullptr) {
    // Quantising epilogue (the reference's stage behind the attention): the four lanes of a
    // block of 32 columns are neighbours; the codes come from the bf16-rounded values, as they
    // would from the bf16 tensor.
    unsigned magnitude = 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) magnitude = MxMagnitudeMax(packed[i], magnitude);
    magnitude = max(magnitude, static_cast<unsigned>(__shfl_xor(static_cast<int>(magnitude), 1)));
    magnitude = max(magnitude, static_cast<unsigned>(__shfl_xor(static_cast<int>(magnitude), 2)));
    const MxScale s = MxScaleFromMaxBits(magnitude);
    u32x2 codes;
    codes.x = MxEncodeWord(packed.x, s) | (MxEncodeWord(packed.y, s) << 16);
    codes.y = MxEncodeWord(packed.z, s) | (MxEncodeWord(packed.w, s) << 16);
    *reinterpret_cast<u32x2*>(a.out_codes + seq * a.out_codes_seq_stride + head * a.out_codes_head_stride + lane * 8) = codes;
    if ((lane & 3) == 0) {
      reinterpret_cast<unsigned char*>(a.out_scales + seq * a.out_scales_seq_stride + head * a.out_scales_head_stride)[lane >> 2] =
          static_cast<unsigned char>(s.code);
    }
  }
  if (a.lse != nullptr && lane == 0) {
    a.lse[seq * a.heads + head] = denom == 0.0f ? -__builtin_inff() : (m + __builtin_amdgcn_logf(denom)) * 0.6931471805599453f;
  }
}

template <bool FP8, bool ALIGNED, bool MXQ, bool SPARSE>
hipError_t Launch(const AttnArgs& args, const dim3& grid, hipStream_t stream) {
  // Dynamic LDS above 64 KB needs the attribute once per kernel and process.
  static const hipError_t prepared = hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaDecodeKernel<FP8, ALIGNED, MXQ, SPARSE>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, Geom<FP8>::kLdsBytes);
  if (prepared != hipSuccess) return prepared;
  hipLaunchKernelGGL((MlaDecodeKernel<FP8, ALIGNED, MXQ, SPARSE>), grid, dim3(kThreads), Geom<FP8>::kLdsBytes, stream, args);
  return hipGetLastError();
}

template <bool MXQ>
hipError_t LaunchByCache(const AttnArgs& args, const dim3& grid, hipStream_t stream) {
  const bool aligned = args.block_size % kTileTokens == 0;
  if (args.fp8) return aligned ? Launch<true, true, MXQ, false>(args, grid, stream) : Launch<true, false, MXQ, false>(args, grid, stream);
  return aligned ? Launch<false, true, MXQ, false>(args, grid, stream) : Launch<false, false, MXQ, false>(args, grid, stream);
}

}  // namespace

hipError_t PrepareAttnKernels() { return hipSuccess; }

// Split-KV partials for callers that cannot allocate: one array per GPU, held from module load to
// process exit. In host code the array's name only stands for the symbol; its address on the
// current device comes from hipGetSymbolAddress, once per device, and everything (kernel
// arguments included) uses that address.
static __device__ __align__(256) unsigned char scratch[kAttnStaticScratchBytes];

hipError_t AttnStaticScratch(char** address) {
  constexpr int kMaxDevices = 64;
  static std::mutex guard;
  static char* per_device[kMaxDevices] = {};
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(guard);
  if (per_device[device] == nullptr) {
    void* resolved = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&resolved, HIP_SYMBOL(scratch)); e != hipSuccess) return e;
    if (resolved == nullptr) return hipErrorInvalidSymbol;
    per_device[device] = static_cast<char*>(resolved);
  }
  *address = per_device[device];
  return hipSuccess;
}

hipError_t LaunchAttnDecode(const AttnArgs& args_in, hipStream_t stream) {
  AttnArgs args = args_in;
#ifdef MLAKV_ATTN_TRACE
  args.trace = std::getenv("MLAKV_ATTN_TRACE_PTR") ? reinterpret_cast<unsigned long long*>(std::strtoull(std::getenv("MLAKV_ATTN_TRACE_PTR"), nullptr, 0)) : nullptr;
#endif
  if (args.batch <= 0) return hipSuccess;
  const dim3 grid(args.max_chunks, args.batch, (args.heads + 63) / 64);
  // With several chunks the merge kernel owns the final output and the optional quantisation.
  const bool quantise_here = args.max_chunks == 1 && args.out_codes != nullptr;
  hipError_t e;
  if (args.sparse_indices != nullptr) {
    e = args.fp8 ? Launch<true, false, false, true>(args, grid, stream) : Launch<false, false, false, true>(args, grid, stream);
  } else {
    e = quantise_here ? LaunchByCache<true>(args, grid, stream) : LaunchByCache<false>(args, grid, stream);
  }
  if (e != hipSuccess) return e;
  if (args.max_chunks > 1) {
    hipLaunchKernelGGL(MlaCombineKernel, dim3((args.heads + kCombineHeads - 1) / kCombineHeads, args.batch), dim3(kCombineHeads * 64), 0,
                       stream, args);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace mlakv
