// Absorbed-MLA decode attention over the paged latent KV cache, gfx950 (CDNA4).
//
//   s_i = scale * (q_lat[h] . c_i + q_rope[h] . r_i),  p = softmax_i(s),  o[h] = sum_i p_i c_i
//
// One query token per sequence, all heads share one latent KV stream (MQA), so the
// head axis is the free MFMA dimension and the latent row is read from HBM once and used
// as both K (with the 64 rope columns appended) and V.
//
// Work decomposition
//   The contexts of the batch, in 32-token tiles, laid end to end, are cut into as many equal
//   work units as there are CUs; a workgroup (one per CU, all 64 heads of a group) walks the
//   segments of its unit, each a tile range of one sequence (see "work decomposition" below).
//   8 wavefronts in two roles, one of each role per SIMD:
//     score waves 0..3 (16 heads each) hold the query in registers, compute S^T = K Q^T for a
//       tile, run the online softmax and publish P (bf16, already in MFMA operand layout)
//       through LDS, one tile ahead of
//     output waves 4..7, which hold the O accumulators and compute O^T += V^T P.
//   A single wave per SIMD is bound by instruction issue (one instruction per four cycles,
//   every stall exposed); with the two roles the softmax VALU work, the LDS traffic and the
//   MFMAs of neighbouring tiles overlap in hardware, and neither role has to hold both the
//   query (72 registers) and O (128 registers).
//   LDS holds a ring of four tile buffers: while
//   tile i feeds the second product and tile i+1 the first, tiles i+2 and i+3 are in flight
//   from HBM. bf16 tiles are filled by direct global->LDS loads (global_load_lds_dwordx4: no
//   staging registers, no ds_write) issued by all eight waves; FP8 tiles arrive the same way as
//   codes and are converted at the MFMA operand. One workgroup barrier per tile publishes
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
// Segments that do not hold a whole sequence leave partials (normalised O in bf16, log2-domain
// LSE in fp32) in the caller's workspace; they are merged inside the same launch, or by a second
// small kernel when the launch has no counters to meet on.
#include <algorithm>
#include <mutex>
#include <utility>

#include "kernels.h"

#include <cstddef>
#include "mx_quant_device.h"

#pragma clang diagnostic ignored "-Winline-asm"

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
typedef unsigned long long u64;

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kScoreWaves = 4;
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;        // 18
constexpr int kQkSteps = 2 * kKSteps;                        // 36 MFMAs: 18 k-steps x 2 token subtiles
constexpr int kDvTiles = kLatentDim / 16;                    // 32
constexpr int kTableEntries = kAttnTableEntries;             // block-table entries of one segment staged in LDS
constexpr int kMaxDuties = 64;                               // merges a workgroup has promised and not yet carried out
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
  static constexpr int kDutyOff = kFlagOff + 64;                       // i32x4[kMaxDuties]
  static constexpr int kFoundOff = kDutyOff + kMaxDuties * 16;         // unsigned[kMaxDuties]
  static constexpr int kLdsBytes = kFoundOff + kMaxDuties * 4;
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
// (four bytes per lane: lane L's dword lands at lds_wave_base + 4 * L)
__device__ __forceinline__ void DirectLoad4PerLane(const char* lane_pointer, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
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
  // from position `first_pos` of the selection on, the physical block and the slot inside it as
  // (block << slot_bits) | slot (-1: behind a bad table entry), so that a row is located without a
  // division; `seq_len` is the number of selected tokens.
  bool sparse;
  int first_pos;
  int slot_bits;  // ceil(log2(block_size))
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
      const int packed = pos < seq_len ? entries[pos - first_pos] : -1;
      const int usable = packed < 0 ? 0 : packed;
      *block = usable >> slot_bits;
      *slot = usable & ((1 << slot_bits) - 1);
      return packed >= 0;
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
  if constexpr (!ALIGNED && !WITH_PARTNER) {
    // Every row is located first (the LDS reads of the staged entries go out together; the loads
    // below are opaque to the compiler and would otherwise keep each read behind the load before it).
    int blocks[kRowsPerWave], slots[kRowsPerWave];
    bool reals[kRowsPerWave];
#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) reals[i] = map.Row(tile, wave + kWaves * i, &blocks[i], &slots[i]);
#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) {
      const int row = wave + kWaves * i;  // wave-uniform
      all_real = all_real && reals[i];
      if (reals[i]) {
        const char* src = a.latent.base + Uniform(blocks[i]) * a.latent.block_stride + Uniform(slots[i]) * a.latent.row_stride;
        DirectLoad16(src, (lane ^ SwizzleLat(row)) << 4, buf + row * G::kLatRow);
      } else {
        *reinterpret_cast<u32x4*>(buf_ptr + row * G::kLatRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
      }
    }
  } else {
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

// Whether a row's start inside its plane can be formed in 16-byte units with 24-bit multiplies
// and held in 32 bits (what the whole-selection units of 16 heads stage per selected token).
__host__ __device__ __forceinline__ bool PlainRowsAddressable(const AttnArgs& a) {
  const int64_t limit = int64_t{1} << 28;  // strides in 16-byte units below 2^24
  return a.latent.block_stride < limit && a.rope.block_stride < limit && a.latent.row_stride < limit && a.rope.row_stride < limit &&
         a.num_blocks <= (1 << 24) && a.num_blocks * a.latent.block_stride < (int64_t{1} << 36) &&
         a.num_blocks * a.rope.block_stride < (int64_t{1} << 36) &&
         // (FP8: a row's scale, in 4-byte units from its plane's base)
         (!a.fp8 || a.num_blocks * a.scale.block_stride < (int64_t{1} << 34));
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

// ---- work decomposition --------------------------------------------------------------------
//
// The sequences' contexts, counted in 32-token tiles, are laid end to end on one flat tile axis,
// and that axis is cut into work units of `tiles_per_unit` tiles: as many units as the launch
// has workgroups (per group of 64 heads) when the batch is large enough, so that every CU streams
// the same number of tiles whatever the individual lengths are. Every workgroup derives the cut
// from the live lengths itself (one prefix sum over the batch); nothing depends on the host
// knowing them. A unit is a run of segments, each a tile range of one sequence:
//   * a segment that holds a whole sequence writes the final output;
//   * any other segment writes a partial (normalised O in bf16, log2-domain LSE in fp32) to the
//     caller's workspace: slot `max_units + seq` for the segment with the sequence's first tile,
//     slot `unit` for a later one (a unit starts inside at most one sequence).
// The partials of a sequence are merged inside the same launch: every contributor announces its
// partial on a per-sequence counter and then merges its share of the heads once the counter is
// full. Waiting is bounded, and a share whose owner gave up (or has not claimed it by then) is
// taken by the contributor that arrived last, so the launch finishes whatever the order in which
// workgroups get to run.

constexpr int kMergeHeads = 8;   // heads of one merge step: one per wave

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves: four shifted adds
// inside each row of 16 lanes, then lane 15 of rows 0 and 2 onto rows 1 and 3, then lane 31 onto
// the upper half. Lanes a move does not reach add zero.
__device__ __forceinline__ int WaveInclusiveScan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// 64 consecutive sequences, one per lane: tokens that count, tiles, and the running totals of
// tiles and of sequences that have tiles, up to and including the lane's sequence. Windows are
// visited in increasing order.
// The live length of a sequence: from the argument block when the caller knew it on the host.
// One load either way: the source is chosen as an address (AttnArgs is the kernels' only explicit
// argument, so it starts the kernel-argument segment); a select between two loaded values cost the
// launch pair 1 to 3 us.
__device__ __forceinline__ int LiveLength(const AttnArgs& a, int seq) {
  const int32_t* lengths = a.seq_lens;
  if (a.inline_count > 0) {
    const char* segment = (const char*)__builtin_amdgcn_kernarg_segment_ptr();  // (constant -> generic address space)
    lengths = reinterpret_cast<const int32_t*>(segment + offsetof(AttnArgs, inline_lens));
  }
  return lengths[seq];
}

template <bool SPARSE>
struct SeqWindow {
  int base;   // first sequence of the window; uniform
  int tok, tiles, incl_tiles, incl_live;

  __device__ __forceinline__ void Load(const AttnArgs& a, int lane, int new_base, int carry_tiles, int carry_live) {
    base = new_base;
    const int seq = base + lane;
    int n = 0;
    if (seq < a.batch) {
      if (SPARSE) {
        n = a.sparse_count;
      } else {
        n = min(max(LiveLength(a, seq), 0), a.max_tokens);
      }
    }
    tok = n;
    tiles = (n + kTileTokens - 1) / kTileTokens;
    incl_tiles = carry_tiles + WaveInclusiveScan(tiles);
    incl_live = carry_live + WaveInclusiveScan(tiles != 0 ? 1 : 0);
  }
  __device__ __forceinline__ void Next(const AttnArgs& a, int lane) { Load(a, lane, base + 64, EndTiles(), EndLive()); }
  __device__ __forceinline__ int EndTiles() const { return __builtin_amdgcn_readlane(incl_tiles, 63); }
  __device__ __forceinline__ int EndLive() const { return __builtin_amdgcn_readlane(incl_live, 63); }
  __device__ __forceinline__ int Tok(int seq) const { return __builtin_amdgcn_readlane(tok, seq - base); }
  __device__ __forceinline__ int Tiles(int seq) const { return __builtin_amdgcn_readlane(tiles, seq - base); }
  // End of sequence `seq` on the flat axis on which every sequence with tiles is preceded by `pad` idle positions.
  __device__ __forceinline__ int End(int seq, int pad) const {
    return __builtin_amdgcn_readlane(incl_tiles, seq - base) + pad * __builtin_amdgcn_readlane(incl_live, seq - base);
  }
  __device__ __forceinline__ int EndOfLane(int pad) const { return incl_tiles + pad * incl_live; }
  // The tile count shared by every sequence of the window that has tiles (0: none has, -1: they differ).
  __device__ __forceinline__ int CommonTiles() const {
    const u64 live = __builtin_amdgcn_ballot_w64(tiles != 0);
    if (live == 0) return 0;
    const int first = __builtin_amdgcn_readlane(tiles, __builtin_ctzll(live));
    return __builtin_amdgcn_ballot_w64(tiles != 0 && tiles != first) == 0 ? first : -1;
  }
};

// Tiles per work unit for a launch whose sequences add up to `total_tiles`: an equal share per
// workgroup, not below what amortises a query load and not above what a segment's staged
// block-table entries can address (or the plan's fixed value).
__host__ __device__ __forceinline__ int TilesPerUnit(const AttnArgs& a, int total_tiles, int work_groups) {
  int share;
  if (a.forced_unit_tiles > 0) {
    share = a.forced_unit_tiles;
  } else if ((work_groups & (work_groups - 1)) == 0) {  // the usual case, without a division
    share = (total_tiles + work_groups - 1) >> __builtin_ctz(work_groups);
  } else {
    share = (total_tiles + work_groups - 1) / work_groups;
  }
  const int least = a.forced_unit_tiles > 0 ? 1 : a.min_unit_tiles;
  const int raised = share > least ? share : least;
  return raised < a.cap_unit_tiles ? raised : a.cap_unit_tiles;
}

// How a launch cuts its work. Entering a sequence in the middle of a unit costs a workgroup about
// as much as kBoundaryTiles tiles (the query, the table entries and the first tiles of the new
// sequence arrive while nothing is computed), and the launch lasts as long as its slowest
// workgroup. So the flat axis gives every sequence with tiles kBoundaryTiles idle positions in
// front of its tiles: units are equal on that axis, and one that enters sequences on its way
// gets that many fewer tiles. When every sequence has the same number of tiles and units divide
// it, unit and sequence boundaries coincide anyway and the axis stays unpadded.
constexpr int kBoundaryTiles = kAttnBoundaryTiles;
struct Cut {
  int pad;             // idle positions in front of every sequence that has tiles
  int total;           // length of the flat axis
  int tiles_per_unit;  // positions per unit
};
__host__ __device__ __forceinline__ Cut MakeCut(const AttnArgs& a, int total_tiles, int live_sequences, int common_tiles, int work_groups) {
  Cut cut;
  cut.pad = 0;
  cut.total = total_tiles;
  cut.tiles_per_unit = TilesPerUnit(a, total_tiles, work_groups);
  const bool coincide = live_sequences <= 1 || (common_tiles > 0 && common_tiles % cut.tiles_per_unit == 0);
  if (!coincide) {
    cut.pad = kBoundaryTiles;
    cut.total = total_tiles + kBoundaryTiles * live_sequences;
    cut.tiles_per_unit = TilesPerUnit(a, cut.total, work_groups);
  }
  return cut;
}

// Stores and loads that other CUs' accesses of the same kind see without a cache write-back or
// invalidate in between (agent scope: the sc1 bit): the partials and the counters travel through
// these. The 16-byte forms have no builtin; a load's result is ready after WaitAgentLoads on it.
// (The compiler does not know that the statement reads `v` for a few cycles after issue, as a
// store of more than 8 bytes does: the s_nop keeps a following write of those registers away.)
__device__ __forceinline__ void StoreAgent16(char* p, const u32x4& v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ u32x4 LoadAgent16(const char* p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
// Waits for every outstanding vector-memory operation of the wave; the loaded registers pass
// through the statement so that no use of them can be scheduled ahead of it.
__device__ __forceinline__ void WaitAgentLoads(u32x4 (&v)[8]) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
               :
               : "memory");
}
__device__ __forceinline__ void StoreAgentF32(float* p, float v) {
  __hip_atomic_store(reinterpret_cast<unsigned*>(p), __builtin_bit_cast(unsigned, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float LoadAgentF32(const float* p) {
  return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<unsigned*>(const_cast<float*>(p)), __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT));
}

// Row index of (head group z, partial slot, head of the group) in the partial arrays.
__device__ __forceinline__ int64_t PartialRow(const AttnArgs& a, int z, int slot, int head_in_group) {
  return (static_cast<int64_t>(z) * (a.max_units + a.batch) + slot) * 64 + head_in_group;
}

// Final output rows of an empty sequence (zeros, lse = -inf): wave w takes heads w, w + 8, ... of the group.
template <bool MXQ>
__device__ __forceinline__ void ZeroFill(const AttnArgs& a, int z, int seq, int wave, int lane) {
  const int heads_here = min(64, a.heads - 64 * z);
  for (int h = wave; h < heads_here; h += kWaves) {
    const int head = 64 * z + h;
    if (a.out != nullptr) *reinterpret_cast<u32x4*>(a.out + seq * a.out_seq_stride + head * a.out_head_stride + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    if (a.lse != nullptr && lane == 0) a.lse[seq * a.heads + head] = -__builtin_inff();
    if constexpr (MXQ) {  // zeros quantise to zero codes under the smallest scale
      if (lane < kLatentDim / 16) *reinterpret_cast<u32x4*>(a.out_codes + seq * a.out_codes_seq_stride + head * a.out_codes_head_stride + lane * 16) = u32x4{0u, 0u, 0u, 0u};
      if (lane == 0) *reinterpret_cast<u32x4*>(a.out_scales + seq * a.out_scales_seq_stride + head * a.out_scales_head_stride) = u32x4{0u, 0u, 0u, 0u};
    }
  }
}

// Merges the `n` partials of (sequence, head): out = sum_c w_c O_c / sum_c w_c with
// w_c = 2^(lse2_c - max lse2), in the order of the sequence's tiles. One wave, 8 output columns
// per lane. Partial 0 sits in slot `first_slot`, partial i > 0 in slot `u0 + i`. Every partial
// carries an LSE (-inf for an empty one, whose O row is not data), so the loads of a group of
// eight partials are issued together.
// AGENT: the partials were written by other CUs of this launch (agent-scope loads); otherwise by
// an earlier launch (plain streaming loads).
template <bool MXQ, bool AGENT>
__device__ __forceinline__ void MergeHead(const AttnArgs& a, int z, int seq, int head_in_group, int first_slot, int u0, int n, int lane) {
  const int head = 64 * z + head_in_group;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
  float m = -__builtin_inff(), denom = 0.0f;
  for (int c0 = 0; c0 < n; c0 += 8) {
    u32x4 v[8];
    float l[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = min(c0 + u, n - 1);
      const int64_t row = PartialRow(a, z, c == 0 ? first_slot : u0 + c, head_in_group);
      if constexpr (AGENT) {
        l[u] = c0 + u < n ? LoadAgentF32(a.partial_lse + row) : -__builtin_inff();
        v[u] = LoadAgent16(a.partial_out + row * (kLatentDim * 2) + lane * 16);
      } else {
        l[u] = c0 + u < n ? a.partial_lse[row] : -__builtin_inff();
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.partial_out + row * (kLatentDim * 2) + lane * 16));
      }
    }
    if constexpr (AGENT) WaitAgentLoads(v);
    float group_max = m;
#pragma unroll
    for (int u = 0; u < 8; ++u) group_max = fmaxf(group_max, l[u]);
    if (group_max == -__builtin_inff()) continue;  // nothing but empty partials so far
    const float rescale = __builtin_amdgcn_exp2f(m - group_max);  // 0 on the first group
    m = group_max;
    denom *= rescale;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= rescale;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (l[u] == -__builtin_inff()) continue;  // empty or padding slot
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
  // Nothing but empty partials yields zeros and lse = -inf.
  const float inv = denom == 0.0f ? 0.0f : 1.0f / denom;
  u32x4 packed;
  packed.x = PackBf16(acc[0] * inv, acc[1] * inv);
  packed.y = PackBf16(acc[2] * inv, acc[3] * inv);
  packed.z = PackBf16(acc[4] * inv, acc[5] * inv);
  packed.w = PackBf16(acc[6] * inv, acc[7] * inv);
  if (a.out != nullptr) *reinterpret_cast<u32x4*>(a.out + seq * a.out_seq_stride + head * a.out_head_stride + lane * 16) = packed;
  if constexpr (MXQ) {
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

// ---- main kernel -------------------------------------------------------------------

// MXQ: the launch also quantises its output (and its bf16 output is optional). Kept out of the
// common instantiation, whose register allocation has no room to spare.
// SPARSE: every sequence attends to the tokens listed in a.sparse_indices instead of to its whole
// context (never ALIGNED: every row is located on its own); on the flat tile axis every sequence
// counts with the full length of the list.
template <bool FP8, bool ALIGNED, bool MXQ, bool SPARSE>
__global__ __launch_bounds__(kThreads) void MlaDecodeKernel(AttnArgs a) {
  static_assert(!(SPARSE && ALIGNED), "selected-token attention uses the row-at-a-time path");
  // bf16 tiles: the output waves, which have no query to wait for, issue the first tiles of the
  // ring alone (their own rows and those of their partner score waves) as soon as they know the
  // block-table entries; the score waves join from the first loop iteration on.
  constexpr bool kSoloPrologue = !FP8 && !SPARSE;
  using G = Geom<FP8>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
  const int tid0 = threadIdx.x;
  const int lane0 = tid0 & 63, wave0 = Uniform(tid0 >> 6);
  // Workgroups are handed to the eight XCDs round-robin by linear id, and each XCD has its own
  // L2. Neighbouring units mostly belong to one sequence and read the same 72 KB of Q, so XCD x
  // takes the contiguous range of units [x, x+1) * W / 8.
  const int work_groups = gridDim.x;
  int wg = blockIdx.x;
  if ((work_groups & (kXcds - 1)) == 0) wg = (wg & (kXcds - 1)) * (work_groups / kXcds) + wg / kXcds;
  const int z = blockIdx.y;  // group of 64 heads

  // Every wave walks the batch itself: the total number of tiles fixes the cut of the flat axis.
  // On the way the empty sequences (no tile, so no unit) get their zeros, spread over the workgroups.
  SeqWindow<SPARSE> win;
  win.Load(a, lane0, 0, 0, 0);
  int common_tiles = 0;  // the tile count all sequences with tiles share; -1 when they differ
  for (;;) {
    if constexpr (!SPARSE) {
      u64 empties = __builtin_amdgcn_ballot_w64(win.base + lane0 < a.batch && win.tiles == 0);
      while (empties != 0) {
        const int s = win.base + __builtin_ctzll(empties);
        if (s % work_groups == wg) ZeroFill<MXQ>(a, z, s, wave0, lane0);
        empties &= empties - 1;
      }
    }
    const int here = win.CommonTiles();
    if (here != 0) common_tiles = common_tiles == 0 || common_tiles == here ? here : -1;
    if (win.base + 64 >= a.batch) break;
    win.Next(a, lane0);
  }
  const Cut cut = MakeCut(a, win.EndTiles(), win.EndLive(), common_tiles, work_groups);
  const int tiles_per_unit = cut.tiles_per_unit, total_tiles = cut.total, pad = cut.pad;
  // unit u covers positions [u, u + 1) * tiles_per_unit of the flat axis; there are
  // ceil(total / tiles_per_unit) units, at most a.max_units (ensured by the plan)
  if (static_cast<int64_t>(wg) * tiles_per_unit >= total_tiles) return;
  if (win.base != 0) win.Load(a, lane0, 0, 0, 0);

  // Q fragments (score waves): lane (head i16, k-group g) holds, for k-step ks, the eight query
  // elements that meet the lane's K fragment of that step: Q[head][32 ks + 8g .. +7] for bf16
  // tiles; for FP8 tiles one 16-byte K read feeds two k-steps, so the order inside each 64-wide
  // window is Q[head][64 (ks/2) + 16g + 8 (ks&1) .. +7]. (Loaded per segment, once the table
  // entries have been asked for.)

  const auto ring = [&](int i) __attribute__((always_inline)) { return G::Slot(i); };
  int* table_lds = reinterpret_cast<int*>(lds + G::kTableOff);
  int* scalar_lds = reinterpret_cast<int*>(lds + G::kFlagOff) + 2 * kScoreWaves;  // a few words for workgroup-wide values
  i32x4* duty_lds = reinterpret_cast<i32x4*>(lds + G::kDutyOff);
  int duties = 0;  // uniform over the workgroup
  const int group_head0 = z * 64;
  const int heads_here = min(64, a.heads - group_head0);
  const int hba = (heads_here + 15) >> 4;  // head blocks in use
  unsigned* const sync_group = a.sync == nullptr ? nullptr : a.sync + static_cast<int64_t>(z) * a.batch * 2;

  // Carries out the merges promised so far; entry: (sequence, first unit, partials, rank). Two
  // words per (head group, sequence), zero between launches:
  //   word 0: partials announced (low 16 bits) | contributors that gave up waiting (high 16 bits)
  //   word 1: contributors that are through with word 0; the last of them clears both.
  // A contributor announces its partial, waits (bounded) until all are announced and merges its
  // share of the heads, rank, rank + n, ... in steps of eight heads. One that gives up before the
  // count is full says so in the same word and leaves; the contributor whose announcement fills
  // the count sees that somebody gave up (not who) and merges every share. A share may then be
  // merged twice, by its owner as well: both write the same bytes.
  const auto flush_duties = [&]() __attribute__((always_inline)) {
    const int merge_units = (heads_here + kMergeHeads - 1) / kMergeHeads;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's partial stores are complete
    __syncthreads();                                  // every wave's are, and the entries are visible
    // All announcements first (a workgroup with several units may hold several partials of one
    // sequence); thread 0 keeps what each found.
    unsigned* found_lds = reinterpret_cast<unsigned*>(lds + G::kFoundOff);
    if (tid0 == 0) {
      for (int d = 0; d < duties; ++d) {
        found_lds[d] = __hip_atomic_fetch_add(sync_group + duty_lds[d].x * 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    for (int d = 0; d < duties; ++d) {
      const i32x4 duty = duty_lds[d];
      const int seq = Uniform(duty.x), u0 = Uniform(duty.y), n = Uniform(duty.z), rank = Uniform(duty.w);
      unsigned* words = sync_group + seq * 2;
      unsigned through = 0u;
      if (tid0 == 0) {
        const unsigned before = found_lds[d];
        int share = 1;  // 0: leave it to the last contributor, 1: own share, 2: every share
        if ((before & 0xffffu) == static_cast<unsigned>(n - 1)) {
          share = (before >> 16) != 0u ? 2 : 1;
        } else {
          const u64 t0 = __builtin_amdgcn_s_memrealtime();
          for (;;) {
            if ((__hip_atomic_load(words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffffu) == static_cast<unsigned>(n)) break;
            if (__builtin_amdgcn_s_memrealtime() - t0 >= static_cast<u64>(a.spin_ticks)) {
              // giving up: unless the count filled in the meantime, the last contributor will know
              const unsigned found = __hip_atomic_fetch_add(words, 0x10000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              if ((found & 0xffffu) != static_cast<unsigned>(n)) share = 0;
              break;
            }
            __builtin_amdgcn_s_sleep(2);
          }
        }
        // through with word 0; the answer is looked at after the merge
        through = __hip_atomic_fetch_add(words + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        scalar_lds[1] = share;
      }
      __syncthreads();
      const int share = Uniform(scalar_lds[1]);
      if (share != 0) {
        for (int u = share == 2 ? 0 : rank; u < merge_units; u += share == 2 ? 1 : n) {
          const int h = u * kMergeHeads + wave0;
          if (h < heads_here) MergeHead<MXQ, true>(a, z, seq, h, a.max_units + seq, u0, n, lane0);
        }
      }
      __syncthreads();  // scalar_lds[1] is free again
      if (tid0 == 0 && through == static_cast<unsigned>(n - 1)) {
        __hip_atomic_store(words, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(words + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    duties = 0;
  };

  bool first_segment = true;
  for (int unit = wg; static_cast<int64_t>(unit) * tiles_per_unit < total_tiles; unit += work_groups) {
    const int flat_end = min(total_tiles, (unit + 1) * tiles_per_unit);
    int flat = unit * tiles_per_unit;
    while (win.End(win.base + 63, pad) <= flat) win.Next(a, lane0);
    int seq = win.base + __builtin_ctzll(__builtin_amdgcn_ballot_w64(win.EndOfLane(pad) > flat));
    while (flat < flat_end) {
      // Sequence `seq` holds positions [seq_begin - pad, seq_end) of the flat axis, its tiles the
      // last Tiles(seq) of them; the unit's part of those tiles is the segment.
      const int seq_end = win.End(seq, pad), seq_begin = seq_end - win.Tiles(seq);
      const int segment_begin = max(flat, seq_begin), segment_end = min(flat_end, seq_end);
      flat = segment_end;
      if (segment_begin >= segment_end) {
        flat = min(flat_end, seq_end);  // only idle positions of this sequence fall into the unit
      } else {
        const int tile_begin = segment_begin - seq_begin;          // first tile of the segment inside its sequence
        const int segment_tiles = segment_end - segment_begin;     // >= 1
        const bool holds_first = tile_begin == 0, holds_last = segment_end == seq_end;
        const bool direct = holds_first && holds_last;    // the whole sequence: write the final output here
        const int slot = holds_first ? a.max_units + seq : unit;
        int seq_len = win.Tok(seq);

        if (!first_segment) __syncthreads();  // the previous segment's staging rows, table entries and P slots are free
        first_segment = false;

        // Everything that depends on the thread id alone is formed here, per segment, from a copy
        // of the id that the compiler cannot see through: hoisted out of the segment loop, these
        // values would stay live through both roles' tile loops, where no register is to spare.
        int tid = tid0;
        asm volatile("" : "+v"(tid));
        const int lane = tid & 63, wave = Uniform(tid >> 6);
        const bool score_wave = wave < kScoreWaves;   // wave-uniform role
        const int hw = wave & (kScoreWaves - 1);      // which 16 heads of the 64
        const int g = lane >> 4, i16 = lane & 15;
        const int head_base = z * 64 + hw * 16;
        const bool active = head_base < a.heads;  // wave-uniform
        const int head = head_base + i16;
        const int per_tile = FP8 ? LoadsPerTile8(wave) : LoadsPerTile(wave);
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

        unsigned char* p_lds = lds + G::kPOff + (hw * 64 + lane) * 16;           // + parity * kScoreWaves * 64 * 16
        float* alpha_lds = reinterpret_cast<float*>(lds + G::kAlphaOff) + hw * 64 + lane;  // + parity * kScoreWaves * 64
        float* inv_lds = reinterpret_cast<float*>(lds + G::kInvOff) + hw * 64 + lane;
        int* flag_lds = reinterpret_cast<int*>(lds + G::kFlagOff) + hw;          // + parity * kScoreWaves

        // Stage this segment's block-table entries in LDS.
        TileMap<ALIGNED> map;
        map.entries = table_lds;
        map.block_size = a.block_size;
        map.sparse = SPARSE;
        map.first_pos = tile_begin * kTileTokens;
        map.slot_bits = a.block_size > 1 ? 32 - __builtin_clz(static_cast<unsigned>(a.block_size - 1)) : 0;
        map.first_block = 0;
        map.next_entry = 0;
        map.next_slot0 = 0;
        map.tile_block = 0;
        map.tile_slot0 = 0;
        int staged[kTableEntries / 64];  // kSoloPrologue: this lane's table entries on their way to LDS
        int staged_count = 0;
        const auto write_table = [&]() __attribute__((always_inline)) {
          if constexpr (kSoloPrologue) {
  #pragma unroll
            for (int j = 0; j < kTableEntries / 64; ++j) {
              const int i = lane + 64 * j;
              if (i < staged_count) table_lds[i] = static_cast<unsigned>(staged[j]) < static_cast<unsigned>(a.num_blocks) ? staged[j] : -1;
            }
          }
        };
        if constexpr (!SPARSE) {
          const int first_pos = tile_begin * kTileTokens;
          const int last_pos = first_pos + segment_tiles * kTileTokens - 1;
          map.first_block = first_pos / a.block_size;
          map.next_slot0 = first_pos - map.first_block * a.block_size;
          int count = last_pos / a.block_size - map.first_block + 1;  // <= kTableEntries, ensured by the plan's cap
          count = min(count, a.table_stride - map.first_block);
          const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride + map.first_block;
          if constexpr (kSoloPrologue) {
            // Every wave stages all entries itself (the same values to the same addresses), so that it
            // can read them back without waiting for the other waves. Here they are only asked for;
            // each role writes them to LDS where it first needs them (write_table below).
            staged_count = count;
  #pragma unroll
            for (int j = 0; j < kTableEntries / 64; ++j) {
              const int i = lane + 64 * j;
              staged[j] = i < count ? table_row[i] : -1;
            }
          } else {
            for (int i = tid; i < count; i += kThreads) {
              const int entry = table_row[i];
              table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : -1;
            }
          }
        } else {
          // The selection ends at its first entry that is negative or not inside the context. Then
          // this segment's part of it is resolved to pool slots through the block table.
          const int context = static_cast<int>(
              min(static_cast<int64_t>(max(Uniform(LiveLength(a, seq)), 0)), static_cast<int64_t>(a.table_stride) * a.block_size));
          const int32_t* selection = a.sparse_indices + static_cast<int64_t>(seq) * a.sparse_seq_stride;
          if (tid == 0) scalar_lds[0] = a.sparse_count;
          __syncthreads();
          for (int i = tid; i < a.sparse_count; i += kThreads) {
            const int index = selection[i];
            if (index < 0 || index >= context) atomicMin(scalar_lds, i);
          }
          __syncthreads();
          seq_len = Uniform(scalar_lds[0]);
          const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;
          const int segment_tokens = min(segment_tiles * kTileTokens, seq_len - map.first_pos);  // <= kTableEntries, ensured by the plan's cap
          for (int i = tid; i < segment_tokens; i += kThreads) {
            const int index = selection[map.first_pos + i];  // inside [0, context): before the end of the selection
            const int logical = index / a.block_size;
            const int entry = table_row[logical];
            table_lds[i] = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks)
                               ? (entry << map.slot_bits) | (index - logical * a.block_size)
                               : -1;
          }
        }
        map.seq_len = seq_len;
        const int num_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
        // tiles of this segment that exist (a selection may end before the list does)
        const int ntiles = min(segment_tiles, num_tiles - tile_begin);
        if (SPARSE && ntiles <= 0) {
          if (direct) {
            ZeroFill<MXQ>(a, z, seq, wave, lane);
          } else if (active && score_wave && g == 0) {  // empty partial: the merge reads every partial's LSE
            StoreAgentF32(a.partial_lse + PartialRow(a, z, slot, hw * 16 + i16), -__builtin_inff());
          }
        } else {
          const auto issue = [&](int t) __attribute__((always_inline)) {
            if constexpr (FP8) {
              return IssueTileFp8(a, map, il8, tile_begin + t, lds_base + ring(t), lds + ring(t), tid);
            } else {
              return IssueTileBf16(a, map, il, tile_begin + t, lds_base + ring(t), lds + ring(t), tid);
            }
          };
          // Prologue (each role runs its own copy, below): tiles 0 .. kRing-2 on their way, tile 0
          // landed and published. A tile whose load count is not known (rare path) makes every wait
          // up to and including its own a full one.
          int last_unknown = -1;  // newest tile issued with an unknown number of loads
          int issued = 0;         // tiles issued so far
          // Loads this wave has in flight that are newer than those of tile t: the first `solo_tiles`
          // tiles carry `solo_loads` each, the later ones `per_tile`.
          const int solo_tiles = kSoloPrologue ? min(G::kRing - 1, ntiles) : 0;
          const int solo_loads = score_wave ? 0 : per_tile + kRowsPerWave;
          const auto newer_than = [&](int t) __attribute__((always_inline)) {
            const int solo = max(0, min(issued, solo_tiles) - (t + 1));
            const int shared = max(0, issued - max(t + 1, solo_tiles));
            return solo * solo_loads + shared * per_tile;
          };
          // Top of iteration i, both roles: tile i+1 must have landed (later tiles may still be in
          // flight); the barrier publishes it together with P(i) and retires every wave's reads of
          // tile i-1, whose ring slot the next tile to be issued reuses.
          const auto publish = [&](int i) __attribute__((always_inline)) {
            if (i + 1 < ntiles) WaitLoads(last_unknown >= i + 1 ? 0 : newer_than(i + 1));
            __syncthreads();
          };
          // Issues the next tile of the ring (tile i + kRing - 1 during iteration i).
          const auto issue_next = [&](int i) __attribute__((always_inline)) {
            if (issued < ntiles) {
              if (!issue(issued)) last_unknown = issued;
              ++issued;
            }
          };

          if (score_wave) {
            // ---------------------------------------------------------------- score waves
            // Vector memory requests of a CU are served in order: the query (72 KB per workgroup) is
            // asked for behind the few bytes of table entries that the first tile addresses depend on.
            // It lives in this role's branch only; the output waves' prologue has no room for it.
            bf16x8 q[kKSteps];
            if (active) {
              const char* q_latent = a.q_latent + seq * a.q_latent_seq_stride + head * a.q_latent_head_stride;
              const char* q_rope = a.q_rope + seq * a.q_rope_seq_stride + head * a.q_rope_head_stride;
  #pragma unroll
              for (int ks = 0; ks < kKSteps; ++ks) {
                const int d0 = FP8 ? 64 * (ks >> 1) + 16 * g + 8 * (ks & 1) : 32 * ks + 8 * g;
                const char* p = d0 < kLatentDim ? q_latent + d0 * 2 : q_rope + (d0 - kLatentDim) * 2;
                q[ks] = __builtin_bit_cast(bf16x8, GlobalLoad16(p));
              }
            } else {
  #pragma unroll
              for (int ks = 0; ks < kKSteps; ++ks) q[ks] = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
            }
            write_table();  // asked for before the query, so it is here first
            // Shared prologue: the table entries become visible here, before this wave waits for its
            // query, so that the output waves start their tile loads a query latency earlier.
            if constexpr (!kSoloPrologue) __syncthreads();
            // The query must have arrived before this wave issues tile loads: the compiler's own wait
            // for it would otherwise also wait for every tile load issued in between. Both paths above
            // pass through the statement: were it skipped on one, the compiler would have to assume the
            // query still in flight where they meet again, and would wait for it -- with counts that
            // know nothing of the tile loads, so in effect for every tile in flight -- inside the
            // score loop, at every use.
  #pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks) asm volatile("" ::"v"(q[ks]));
            for (; issued < G::kRing - 1 && issued < ntiles; ++issued) {
              if constexpr (kSoloPrologue) {
                map.Begin(issued);  // keeps the cursor in step with the tiles this wave does not issue
              } else {
                if (!issue(issued)) last_unknown = issued;
              }
            }
            WaitLoads(last_unknown >= 0 ? 0 : newer_than(0));
            __syncthreads();

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
                  constexpr int slot_acc = (step & 1) * 2 + ((step >> 1) & 1);  // two accumulators per token subtile
                  acc[slot_acc] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[step % kKAhead], q[step >> 1], acc[slot_acc], 0, 0, 0);
                  if constexpr (step + kKAhead < kQkSteps) kf[step % kKAhead] = k_frag(buf, step + kKAhead);
                  __builtin_amdgcn_sched_barrier(0);
                });
              }
              // the score waves ask for their rows of the next ring tile behind the QK phase
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
                  StoreAgentF32(a.partial_lse + PartialRow(a, z, slot, hw * 16 + i16), lse2);
                }
              }
            }
            __syncthreads();  // 1/denominator visible to the output waves
          } else {
            // ---------------------------------------------------------------- output waves
            write_table();
            if constexpr (!kSoloPrologue) __syncthreads();  // table entries visible
            for (; issued < G::kRing - 1 && issued < ntiles; ++issued) {
              if constexpr (kSoloPrologue) {
                // bf16 tiles: these waves have no query to wait for and issue the first tiles of the ring
                // alone, their own rows and those of their partner score waves
                if (!IssueTileBf16<ALIGNED, true>(a, map, il, tile_begin + issued, lds_base + ring(issued), lds + ring(issued), tid)) {
                  last_unknown = issued;
                }
              } else {
                if (!issue(issued)) last_unknown = issued;
              }
            }
            WaitLoads(last_unknown >= 0 ? 0 : newer_than(0));
            __syncthreads();

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
            // P fragments of the four score waves. Head blocks past the group's heads are computed on
            // whatever their LDS slots hold and never written.
            constexpr int kDvPerWave = kDvTiles / (kWaves - kScoreWaves);
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
              }
            }
            __syncthreads();  // 1/denominator from the score waves
            if (MXQ && direct) {
              // Quantising epilogue of a whole sequence: a block of 32 columns is a pair of this
              // wave's column tiles over the four lanes that share a head; the wave covers blocks
              // 4 w .. 4 w + 3 of every head.
  #pragma unroll
              for (int hb = 0; hb < kScoreWaves; ++hb) {
                if (hb >= hba) continue;
                const int h = 16 * hb + i16;
                const float inv = inv_all[hb * 64];
                char* codes_row = a.out_codes + seq * a.out_codes_seq_stride + (group_head0 + h) * a.out_codes_head_stride;
                char* out_row = a.out == nullptr ? nullptr : a.out + seq * a.out_seq_stride + (group_head0 + h) * a.out_head_stride;
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
              if (direct) {
                char* out0 = a.out + seq * a.out_seq_stride + group_head0 * a.out_head_stride + kSliceBytes * hw + piece * 16;
  #pragma unroll
                for (int it = 0; it < 16; ++it) {
                  const int h = 4 * it + sub;
                  if (h < 16 * hba) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + h * kStageRow + piece * 16);
                    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out0 + h * a.out_head_stride));
                  }
                }
              } else {
                char* out0 = a.partial_out + PartialRow(a, z, slot, 0) * (kLatentDim * 2) + kSliceBytes * hw + piece * 16;
  #pragma unroll
                for (int it = 0; it < 16; ++it) {
                  const int h = 4 * it + sub;
                  if (h < 16 * hba) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + h * kStageRow + piece * 16);
                    if (sync_group != nullptr) {
                      StoreAgent16(out0 + h * (kLatentDim * 2), v);
                    } else {
                      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out0 + h * (kLatentDim * 2)));
                    }
                  }
                }
              }
            }
          }
        }

        if (!direct && sync_group != nullptr) {
          // A merge to take part in once this workgroup's units are done (all its partials are
          // announced together then: nothing waits in between).
          if (tid == 0) {
            const int first_unit = seq_begin / tiles_per_unit;
            const int partials = (seq_end - 1) / tiles_per_unit - first_unit + 1;
            duty_lds[duties] = i32x4{seq, first_unit, partials, unit - first_unit};
          }
          ++duties;
          if (duties == kMaxDuties) flush_duties();
        }

      }
      if (flat < flat_end) {  // the next sequence that has tiles
        do {
          ++seq;
          if (seq >= win.base + 64) win.Next(a, lane0);
        } while (win.Tiles(seq) == 0);
      }
    }
  }
  if (duties != 0) flush_duties();
}

// The merge as a launch of its own, for launches that have no counters to meet on: block =
// (eight heads, sequence, head group); every wave repeats the cut of the flat tile axis and merges
// one head.
template <bool MXQ, bool SPARSE>
__global__ __launch_bounds__(kMergeHeads * 64) void MlaMergeKernel(AttnArgs a) {
  const int lane = threadIdx.x & 63, wave = Uniform(threadIdx.x >> 6);
  // Workgroups go to the XCDs round-robin by linear id. The main launch put the units of XCD x's
  // share of the flat tile axis on XCD x; with equal lengths that is the x-th eighth of the
  // sequences, whose partials are most likely still in that L2.
  int seq = blockIdx.y, group = blockIdx.x;
  const int z = blockIdx.z;
  if ((gridDim.y & (kXcds - 1)) == 0) {
    const int linear = blockIdx.y * gridDim.x + blockIdx.x;
    const int within = linear / kXcds;
    seq = (linear & (kXcds - 1)) * (gridDim.y / kXcds) + within / static_cast<int>(gridDim.x);
    group = within % static_cast<int>(gridDim.x);
  }
  const int h = group * kMergeHeads + wave;
  if (h >= min(64, a.heads - 64 * z)) return;
  SeqWindow<SPARSE> win;
  win.Load(a, lane, 0, 0, 0);
  int end_tiles = 0, end_live = 0, seq_tiles = 0, common_tiles = 0;
  for (;;) {
    if (seq >= win.base && seq < win.base + 64) {
      end_tiles = win.End(seq, 0);
      end_live = win.End(seq, 1) - end_tiles;
      seq_tiles = win.Tiles(seq);
    }
    const int here = win.CommonTiles();
    if (here != 0) common_tiles = common_tiles == 0 || common_tiles == here ? here : -1;
    if (win.base + 64 >= a.batch) break;
    win.Next(a, lane);
  }
  if (seq_tiles == 0) return;
  const Cut cut = MakeCut(a, win.EndTiles(), win.EndLive(), common_tiles, a.work_groups);
  const int seq_end = end_tiles + cut.pad * end_live;
  const int first_unit = (seq_end - seq_tiles) / cut.tiles_per_unit;
  const int partials = (seq_end - 1) / cut.tiles_per_unit - first_unit + 1;
  if (partials == 1) return;  // written by the workgroup that held the whole sequence
  MergeHead<MXQ, false>(a, z, seq, h, a.max_units + seq, first_unit, partials, lane);
}

// ---- selected-token attention in whole-sequence units of 16 heads ----------------------------
//
// A selection of a few hundred tokens is a dozen tiles. Cut into one unit per CU it is all fixed
// cost: every workgroup fetches the 72-KB query of 64 heads for its two or three tiles and leaves
// 64 KB of partials that a second launch reads back. Here a workgroup takes the whole selection
// of one sequence for one block of 16 heads: an 18-KB query, no partials, no merge, the output
// written once. The head blocks of a sequence run on one XCD at the same time, so the rows they
// all read come from HBM once and from that L2 afterwards. Eight waves in two roles:
//   score waves 0..3 fetch the tiles (the output waves' work per tile is the longer chain, so they
//     issue no loads); wave (t, kh) multiplies token subtile t of the tile (16 tokens) with one
//     half of the 18 k-steps for the 16 heads and leaves its 16 x 16 partial of S^T in LDS, one
//     tile ahead of
//   output waves 4..7, each of which adds the partials, runs the online softmax of all 16 heads
//     itself (every output wave the same arithmetic on the same numbers, so the four agree on the
//     reference maximum without exchanging it), forms P in registers as its MFMA operand and
//     multiplies it with its 128 columns of V.
// The tile ring, the operand layouts and the barrier per tile are those of the kernel above.
//
// HALVES: two workgroups per (sequence, 16 heads), neighbours on one XCD, each with one half of the
// selection's tiles, so that twice as many CUs (and twice as many rows in flight) work on a launch
// that has fewer units than the chip has CUs. The exchange is a matter between the two output waves
// that hold the same 128 columns, one in each workgroup: each leaves its normalised slice (bf16
// rows and a log2-domain LSE per head, agent-scope stores) in the workspace and counts itself on
// the word of (pair, slice); the one that finds the other's count there reads that slice back,
// combines the two and writes the output. Nobody waits, no barrier is involved: the first to
// arrive leaves. The words are zero between launches (the second to arrive clears its word). A
// selection of a single tile is taken by the first workgroup alone.
constexpr int kHbWaves = kWaves, kHbThreads = kHbWaves * 64;
constexpr int kHbLoaders = kScoreWaves;  // the waves that fetch the tiles when every row is a plain row
template <bool FP8>
struct GeomHeadBlock {
  using T = Geom<FP8>;
  static constexpr int kRing = FP8 ? 7 : 4;    // an FP8 tile is half the bytes: seven of them, five on their way
  static constexpr int kTables = FP8 ? 3 : 2;  // FP8: the row's scale as well, in 4-byte units
  static constexpr int kTableOff = kRing * T::kTileBytes;                          // unsigned[kTables][kAttnHeadBlockTokens]: where a selected token's latent and rope rows start, in 16-byte units from the plane's base
  static constexpr int kSOff = kTableOff + kTables * kAttnHeadBlockTokens * 4;     // S^T partials [2][4 waves][64 lanes] x 16 B
  static constexpr int kEndOff = kSOff;  // int[2][kHbWaves], before the first S is written: where each wave saw the selection end, and whether it saw a bad table entry
  static constexpr int kLdsBytes = kSOff + 2 * kScoreWaves * 64 * 16;
  static_assert(kLdsBytes <= 160 * 1024, "one workgroup owns the LDS of a CU");
  __device__ static __forceinline__ int Slot(int i) { return (kRing == 4 ? (i & 3) : (i % kRing)) * T::kTileBytes; }
};
// k-steps of one score wave: half of the 18 for bf16 tiles; FP8 codes are read 16 at a time (two
// k-steps), so the nine reads of a token are split five and four.
template <bool FP8>
constexpr int kHeadBlockKSteps = FP8 ? 10 : kKSteps / 2;

template <bool HALVES, bool FP8>
__global__ __launch_bounds__(kHbThreads) void MlaSelectedHeadBlockKernel(AttnArgs a) {
  using G = GeomHeadBlock<FP8>;
  using T = Geom<FP8>;
  constexpr int kQSteps = kHeadBlockKSteps<FP8>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = Uniform(static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds)));
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = Uniform(tid >> 6);
  // Workgroups go to the XCDs round-robin by linear id: ids x, x + 8, x + 16, ... share XCD x, and
  // the head blocks of a sequence are neighbours among them.
  const int head_blocks = a.heads >> 4;  // heads is a multiple of 16
  const int rest = blockIdx.x >> 3;
  const int half = HALVES ? rest & 1 : 0;
  const int unit = HALVES ? rest >> 1 : rest;
  const int hb = unit % head_blocks;
  const int seq = (unit / head_blocks) * kXcds + (blockIdx.x & (kXcds - 1));
  if (seq >= a.batch) return;
  const bool score_wave = wave < kScoreWaves;
  const int hw = wave & (kScoreWaves - 1);
  const int g = lane >> 4, i16 = lane & 15;
  const int head = 16 * hb + i16;

  // The selection ends at its first entry that is negative or not inside the context. Every
  // thread resolves one or two entries to pool slots through the block table; the loads that the
  // first tile's addresses depend on go out first, the query behind them.
  unsigned* latent_rows = reinterpret_cast<unsigned*>(lds + G::kTableOff);
  unsigned* rope_rows = latent_rows + kAttnHeadBlockTokens;
  unsigned* scale_rows = rope_rows + kAttnHeadBlockTokens;  // FP8 only
  constexpr unsigned kNoRow = 0xffffffffu;  // a selected token behind a block-table entry that is not a block of the pool
  int* end_lds = reinterpret_cast<int*>(lds + G::kEndOff);
  const int context = static_cast<int>(
      min(static_cast<int64_t>(max(Uniform(LiveLength(a, seq)), 0)), static_cast<int64_t>(a.table_stride) * a.block_size));
  const int32_t* selection = a.sparse_indices + static_cast<int64_t>(seq) * a.sparse_seq_stride;
  const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;
  const int slot_bits = a.block_size > 1 ? 32 - __builtin_clz(static_cast<unsigned>(a.block_size - 1)) : 0;
  constexpr int kPerThread = (kAttnHeadBlockTokens + kHbThreads - 1) / kHbThreads;
  int index[kPerThread];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int i = tid + kHbThreads * j;
    // (no selection: the sequence's own positions 0 .. context - 1, a whole context of up to sparse_count tokens)
    index[j] = i < a.sparse_count ? (a.sparse_indices != nullptr ? selection[i] : i) : -1;
  }
  // Q fragments of a score wave: lane (head i16, k-group g) holds Q[head][32 ks + 8 g .. +7] for the
  // nine k-steps ks of its half. FP8: the code reads cover k = 64 kp + 16 g .. + 15 (two k-steps),
  // the first half of the waves takes reads kp = 0 .. 4, the second kp = 5 .. 8 (8 is the rope row).
  bf16x8 q[kQSteps];
  if (score_wave) {
    const int kh = hw >> 1;
    const char* q_latent = a.q_latent + seq * a.q_latent_seq_stride + head * a.q_latent_head_stride;
    const char* q_rope = a.q_rope + seq * a.q_rope_seq_stride + head * a.q_rope_head_stride;
#pragma unroll
    for (int c = 0; c < kQSteps; ++c) {
      const int d0 = FP8 ? 64 * (5 * kh + (c >> 1)) + 16 * g + 8 * (c & 1) : 32 * (kQSteps * kh + c) + 8 * g;
      const char* p = d0 < kLatentDim ? q_latent + d0 * 2 : q_rope + (d0 - kLatentDim) * 2;
      if (d0 < kLatentDim + kRopeDim) {  // (the second half of the FP8 reads has four of them)
        q[c] = __builtin_bit_cast(bf16x8, GlobalLoad16(p));
      } else {
        q[c] = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
      }
    }
  } else {
#pragma unroll
    for (int c = 0; c < kQSteps; ++c) q[c] = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
  }
  int wave_end = a.sparse_count;
  bool any_outside = false;
  const bool shift = (a.block_size & (a.block_size - 1)) == 0;
  // Row starts in 16-byte units, by 24-bit multiplies (the launcher sends pools that these do not
  // cover to the split units: PlainRowsAddressable).
  const unsigned lat_block16 = static_cast<unsigned>(a.latent.block_stride >> 4), lat_row16 = static_cast<unsigned>(a.latent.row_stride >> 4);
  const unsigned rope_block16 = static_cast<unsigned>(a.rope.block_stride >> 4), rope_row16 = static_cast<unsigned>(a.rope.row_stride >> 4);
  const unsigned scale_block4 = FP8 ? static_cast<unsigned>(a.scale.block_stride >> 2) : 0u;
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int i = tid + kHbThreads * j;
    const bool good = index[j] >= 0 && index[j] < context;  // false behind the list's end as well
    const u64 bad = __builtin_amdgcn_ballot_w64(!good);
    if (bad != 0) wave_end = min(wave_end, kHbThreads * j + 64 * wave + static_cast<int>(__builtin_ctzll(bad)));
    if (good && i < kAttnHeadBlockTokens) {
      const int logical = shift ? index[j] >> slot_bits : index[j] / a.block_size;
      const int entry = table_row[logical];
      const bool inside = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks);
      const unsigned block = static_cast<unsigned>(entry), in_block = static_cast<unsigned>(index[j] - logical * a.block_size);
      latent_rows[i] = inside ? __umul24(block, lat_block16) + __umul24(in_block, lat_row16) : kNoRow;
      rope_rows[i] = inside ? __umul24(block, rope_block16) + __umul24(in_block, rope_row16) : kNoRow;
      if constexpr (FP8) scale_rows[i] = inside ? block * scale_block4 + in_block : kNoRow;
      if (!inside) any_outside = true;
    }
  }
  if (lane == 0) {
    end_lds[wave] = wave_end;
    end_lds[kHbWaves + wave] = __builtin_amdgcn_ballot_w64(any_outside) != 0 ? 1 : 0;
  }
  // Every role passes this statement with the query in hand: a wait of the compiler's for it further
  // down would not know of the tile loads issued from inline assembly, and would wait for them all.
#pragma unroll
  for (int c = 0; c < kQSteps; ++c) asm volatile("" ::"v"(q[c]));
  __syncthreads();
  int seq_len = a.sparse_count, outside = 0;
#pragma unroll
  for (int w = 0; w < kHbWaves; ++w) {
    seq_len = min(seq_len, end_lds[w]);
    outside |= end_lds[kHbWaves + w];
  }
  seq_len = Uniform(seq_len);
  // Every row a real row of the pool (the usual case): the tile loads need no case distinction.
  const bool plain_rows = Uniform(outside) == 0;
  const int all_tiles = (seq_len + kTileTokens - 1) / kTileTokens;
  // two workgroups share a selection of at least two tiles: the first ceil(all / 2), then the rest
  const bool shared = HALVES && all_tiles >= 2;
  if (HALVES && !shared && half != 0) return;
  const int first_tile = shared && half != 0 ? (all_tiles + 1) >> 1 : 0;
  const int ntiles = shared ? (half != 0 ? all_tiles >> 1 : (all_tiles + 1) >> 1) : all_tiles;
  if (ntiles == 0) {  // nothing selected: zeros, lse = -inf
    for (int h = wave; h < 16; h += kHbWaves) {
      *reinterpret_cast<u32x4*>(a.out + seq * a.out_seq_stride + (16 * hb + h) * a.out_head_stride + lane * 16) = u32x4{0u, 0u, 0u, 0u};
      if (a.lse != nullptr && lane == 0) a.lse[seq * a.heads + 16 * hb + h] = -__builtin_inff();
    }
    return;
  }

  // The head blocks of a sequence walk its tiles from different starting points (the order of the
  // tiles only changes the rounding): at any time they ask for different rows, and what one has
  // fetched the others find in the L2.
  const int rotate = hb * ntiles / head_blocks;
  const auto tile_of = [&](int i) __attribute__((always_inline)) {
    return first_tile + (i + rotate < ntiles ? i + rotate : i + rotate - ntiles);
  };
  // The score waves fetch the tiles: wave w the latent rows w, w + 4, ... (one row per load: lane L
  // asks for the 16 bytes that belong at 16 L of the swizzled LDS row) and the rope rows 8 w .. 8 w + 7
  // (one load, a row per eight lanes). A lane's address is the plane's base, its own chunk and the
  // row's staged start; positions behind the selection's end repeat its last row (finite values
  // that the softmax masks). A row that is not a row of the pool becomes zeros.
  // FP8 tiles: a load covers two latent rows of 512 bytes (wave w the row pairs w, w + 4, w + 8,
  // w + 12), waves 0 and 1 add sixteen 64-byte rope rows each, waves 2 and 3 the 32 row scales (a
  // dword per lane; both waves, the same bytes, so that every wave has the same count of loads).
  constexpr int kRowsPerLoader = FP8 ? 4 : kTileTokens / kHbLoaders, kPlainLoads = kRowsPerLoader + 1;
  int lat_row[4];  // FP8: the tile row behind each of this lane's latent loads
  const char* lat_lane[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if constexpr (FP8) {
      lat_row[j] = 2 * (wave + kHbLoaders * j) + (lane >> 5);
      lat_lane[j] = a.latent.base + (((lane & 31) ^ SwizzleLat8(lat_row[j])) << 4);
    } else {
      lat_row[j] = 0;
      lat_lane[j] = a.latent.base + ((lane ^ SwizzleLat(wave + kHbLoaders * j)) << 4);
    }
  }
  // the lane's row of the fifth load: a rope row (waves 0, 1 for FP8), or the token whose scale it fetches
  const int extra_row = FP8 ? (wave < 2 ? 16 * wave + (lane >> 2) : (lane & 31)) : 8 * wave + (lane >> 3);
  const char* rope_lane = FP8 ? a.rope.base + (((lane & 3) ^ SwizzleRope8(extra_row)) << 4)
                              : a.rope.base + (((lane & 7) ^ SwizzleRope(extra_row)) << 4);
  const int per_tile = wave < kHbLoaders ? kPlainLoads : 0;
  int last_unknown = -1;  // newest tile issued with an unknown number of loads (a row that is not real)
  int issued = 0;
  const auto issue_next = [&]() __attribute__((always_inline)) {
    if (issued < ntiles) {
      if (wave < kHbLoaders) {
        const int first = tile_of(issued) * kTileTokens, last = seq_len - 1;
        const unsigned buf = lds_base + G::Slot(issued);
        unsigned char* tile = lds + G::Slot(issued);
        if constexpr (FP8) {
          unsigned starts[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) starts[r] = latent_rows[min(first + lat_row[r], last)];
          const bool scale_wave = wave >= 2;
          const unsigned extra_start = (scale_wave ? scale_rows : rope_rows)[min(first + extra_row, last)];
          const unsigned extra_dst = scale_wave ? buf + T::kScaleOff : buf + T::kLatRegion + wave * 16 * T::kRopeRow;
          const char* extra_src = scale_wave ? a.scale.base + (static_cast<u64>(extra_start) << 2) : rope_lane + (static_cast<u64>(extra_start) << 4);
          if (plain_rows) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              DirectLoad16PerLane(lat_lane[r] + (static_cast<u64>(starts[r]) << 4), buf + 2 * (wave + kHbLoaders * r) * T::kLatRow);
            }
            if (scale_wave) {
              DirectLoad4PerLane(extra_src, extra_dst);
            } else {
              DirectLoad16PerLane(extra_src, extra_dst);
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (starts[r] != kNoRow) {
                DirectLoad16PerLane(lat_lane[r] + (static_cast<u64>(starts[r]) << 4), buf + 2 * (wave + kHbLoaders * r) * T::kLatRow);
              } else {
                *reinterpret_cast<u32x4*>(tile + 2 * (wave + kHbLoaders * r) * T::kLatRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
              }
            }
            if (scale_wave) {
              if (extra_start != kNoRow) {
                DirectLoad4PerLane(extra_src, extra_dst);
              } else {
                reinterpret_cast<float*>(tile + T::kScaleOff)[lane] = 0.0f;
              }
            } else if (extra_start != kNoRow) {
              DirectLoad16PerLane(extra_src, extra_dst);
            } else {
              *reinterpret_cast<u32x4*>(tile + T::kLatRegion + wave * 16 * T::kRopeRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
            }
            last_unknown = issued;
          }
        } else {
          unsigned starts[kRowsPerLoader];
#pragma unroll
          for (int r = 0; r < kRowsPerLoader; ++r) starts[r] = latent_rows[min(first + wave + kHbLoaders * r, last)];
          const unsigned rope_start = rope_rows[min(first + extra_row, last)];
          if (plain_rows) {
#pragma unroll
            for (int r = 0; r < kRowsPerLoader; ++r) {
              DirectLoad16PerLane(lat_lane[r & 3] + (static_cast<u64>(starts[r]) << 4), buf + (wave + kHbLoaders * r) * T::kLatRow);
            }
            DirectLoad16PerLane(rope_lane + (static_cast<u64>(rope_start) << 4), buf + T::kLatRegion + wave * 8 * T::kRopeRow);
          } else {
#pragma unroll
            for (int r = 0; r < kRowsPerLoader; ++r) {
              const int row = wave + kHbLoaders * r;
              if (Uniform(starts[r]) != kNoRow) {
                DirectLoad16PerLane(lat_lane[r & 3] + (static_cast<u64>(starts[r]) << 4), buf + row * T::kLatRow);
              } else {
                *reinterpret_cast<u32x4*>(tile + row * T::kLatRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
              }
            }
            if (rope_start != kNoRow) {
              DirectLoad16PerLane(rope_lane + (static_cast<u64>(rope_start) << 4), buf + T::kLatRegion + wave * 8 * T::kRopeRow);
            } else {
              *reinterpret_cast<u32x4*>(tile + T::kLatRegion + wave * 8 * T::kRopeRow + lane * 16) = u32x4{0u, 0u, 0u, 0u};
            }
            last_unknown = issued;
          }
        }
      }
      ++issued;
    }
  };
  // Waits until tile t has landed: this wave's loads of the tiles issued after it may stay in flight
  // (the ring holds the tile in use, the next one and the rest on their way: up to kRing - 2 newer
  // tiles in the prologue, one fewer in the loop, none at the end).
  const auto wait_tile = [&](int t) __attribute__((always_inline)) {
    if (per_tile == 0) return;
    const int newer_tiles = last_unknown >= t ? 0 : issued - (t + 1);
    if (newer_tiles <= 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if (newer_tiles == 1) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kPlainLoads) : "memory");
    } else if (newer_tiles == 2 || G::kRing == 4) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kPlainLoads) : "memory");
    } else if (newer_tiles == 3) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * kPlainLoads) : "memory");
    } else if (newer_tiles == 4) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * kPlainLoads) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(5 * kPlainLoads) : "memory");
    }
  };
  // Top of iteration i, both roles: tile i + 1 has landed; the barrier publishes it together with
  // S(i) and retires every wave's reads of tile i - 1, whose ring slot the next tile reuses.
  const auto publish = [&](int i) __attribute__((always_inline)) {
    if (i + 1 < ntiles) wait_tile(i + 1);
    __syncthreads();
  };
  for (int t = 0; t < G::kRing - 1; ++t) issue_next();
  wait_tile(0);
  __syncthreads();

  f32x4* s_lds = reinterpret_cast<f32x4*>(lds + G::kSOff) + lane;  // + (parity * kScoreWaves + score wave) * 64
  if (score_wave) {
    // ------------------------------------------------------------------ score waves
    const int t = hw & 1;
    const int k_lat = (16 * t + i16) * T::kLatRow, k_rope = T::kLatRegion + (16 * t + i16) * T::kRopeRow;
    int k_e[4], kr_e[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) k_e[j] = ((4 * j + g) ^ SwizzleLat(i16)) << 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) kr_e[j] = ((4 * j + g) ^ SwizzleRope(i16)) << 4;
    // FP8: read kp fetches the 16 codes k = 64 kp + 16 g .. + 15 of token 16 t + i16 (two k-steps):
    // chunk (4 kp + g) ^ swizzle(token) of the 512-byte row; kp = 8 is the rope row. The products
    // are of the codes as they are: the row's scale meets the sums in the output waves.
    const int k8_lat = (16 * t + i16) * T::kLatRow + ((g ^ SwizzleLat8(16 * t + i16)) << 4);
    const int k8_rope = T::kLatRegion + (16 * t + i16) * T::kRopeRow + ((g ^ SwizzleRope8(16 * t + i16)) << 4);
    const auto score_tile = [&](int tile, auto kh_c) __attribute__((always_inline)) {
      constexpr int kh = decltype(kh_c)::value;
      const unsigned char* buf = lds + G::Slot(tile);
      f32x4 acc[3];
#pragma unroll
      for (int j = 0; j < 3; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (FP8) {
        constexpr int kReads = kh == 0 ? 5 : 4;
        u32x4 codes[kReads];
        StaticFor<kReads>([&](auto c_c) __attribute__((always_inline)) {
          constexpr int c = decltype(c_c)::value, kp = 5 * kh + c;
          codes[c] = *reinterpret_cast<const u32x4*>(buf + (kp < 8 ? (k8_lat ^ (kp << 6)) : k8_rope));
        });
        StaticFor<kReads>([&](auto c_c) __attribute__((always_inline)) {
          constexpr int c = decltype(c_c)::value;
          acc[(2 * c) % 3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(CodesToBf16(codes[c].x, codes[c].y), q[2 * c], acc[(2 * c) % 3], 0, 0, 0);
          acc[(2 * c + 1) % 3] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(CodesToBf16(codes[c].z, codes[c].w), q[2 * c + 1], acc[(2 * c + 1) % 3], 0, 0, 0);
        });
      } else {
        bf16x8 kf[kQSteps];
        StaticFor<kQSteps>([&](auto c_c) __attribute__((always_inline)) {
          constexpr int c = decltype(c_c)::value, ks = kQSteps * kh + c;
          const int offset = ks < 16 ? k_lat + (ks >> 2) * 256 + k_e[ks & 3] : k_rope + kr_e[ks & 1];
          kf[c] = *reinterpret_cast<const bf16x8*>(buf + offset);
        });
        StaticFor<kQSteps>([&](auto c_c) __attribute__((always_inline)) {
          constexpr int c = decltype(c_c)::value;
          acc[c % 3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[c], q[c], acc[c % 3], 0, 0, 0);
        });
      }
      s_lds[((tile & 1) * kScoreWaves + hw) * 64] = acc[0] + acc[1] + acc[2];
    };
    const bool upper = (hw >> 1) != 0;  // wave-uniform: which half of the k-steps
    const auto score = [&](int tile) __attribute__((always_inline)) {
      if (upper) {
        score_tile(tile, std::integral_constant<int, 1>{});
      } else {
        score_tile(tile, std::integral_constant<int, 0>{});
      }
    };
    score(0);
    for (int i = 0; i < ntiles; ++i) {
      publish(i);
      issue_next();
      if (i + 1 < ntiles) score(i + 1);
    }
    __syncthreads();  // every output wave is through with the last tile (the ring becomes their staging space)
  } else {
    // ------------------------------------------------------------------ output waves
    // bf16 V reads as in the kernel above: token = (16 +) 4g + i16/4, chunk = 2n + (i16 & 3) / 2, 8-byte half i16 & 1.
    const int v_row = 4 * g + (i16 >> 2);
    const int v_lane = v_row * T::kLatRow + (i16 & 1) * 8;
    int v_e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v_e[j] = ((2 * j + ((i16 & 3) >> 1)) ^ SwizzleLat(v_row)) << 4;
    // FP8 V reads as in the kernel above (ds_read_b64_tr_b8): as a source, lane j of a 16-lane group
    // addresses bytes 16 n + 8 (j & 1) .. + 7 of the row of token 4 g + (j >> 1 & 3) + 16 (j >> 3).
    const int v8_token = 4 * g + ((i16 >> 1) & 3) + 16 * (i16 >> 3);
    const int v8_base = v8_token * Geom<true>::kLatRow + (SwizzleLat8(v8_token) << 4) + 8 * (i16 & 1);
    const auto v_fetch = [&](const unsigned char* buf, int n) __attribute__((always_inline)) {
      if constexpr (FP8) {
        const i32x2 codes = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(buf + (v8_base ^ (n << 4))));
        return CodesToBf16(static_cast<unsigned>(codes.x), static_cast<unsigned>(codes.y));
      } else {
        const unsigned char* addr = buf + v_lane + (n >> 3) * 256 + v_e[n & 7];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr + 16 * T::kLatRow));
        return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    constexpr int kDvPerWave = kDvTiles / (kWaves - kScoreWaves);  // 8 column tiles: columns [128 hw, 128 hw + 128)
    f32x4 o[kDvPerWave];
#pragma unroll
    for (int n = 0; n < kDvPerWave; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = -__builtin_inff();  // reference maximum of the exponentials, log2 domain
    float l_run = 0.0f;               // this lane's share of the running denominator

    for (int i = 0; i < ntiles; ++i) {
      publish(i);
      issue_next();
      const unsigned char* buf = lds + G::Slot(i);
      const f32x4* s = s_lds + (i & 1) * kScoreWaves * 64;
      const f32x4 s0 = s[0], s1 = s[64], s2 = s[128], s3 = s[192];
      bf16x8 vf[kDvPerWave];
      StaticFor<kDvPerWave>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int n = decltype(n_c)::value;
        vf[n] = v_fetch(buf, kDvPerWave * hw + n);
      });
      // lane holds tokens 4g+j (x[0..3]) and 16+4g+j (x[4..7]) of head i16
      float x[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = (s0[j] + s2[j]) * a.scale_log2;
        x[4 + j] = (s1[j] + s3[j]) * a.scale_log2;
      }
      f32x4 row_scale[2] = {f32x4{1.f, 1.f, 1.f, 1.f}, f32x4{1.f, 1.f, 1.f, 1.f}};  // FP8: of tokens 4g+j and 16+4g+j
      if constexpr (FP8) {  // the codes were multiplied unscaled
        const float* scales = reinterpret_cast<const float*>(buf + T::kScaleOff);
        row_scale[0] = *reinterpret_cast<const f32x4*>(scales + 4 * g);
        row_scale[1] = *reinterpret_cast<const f32x4*>(scales + 16 + 4 * g);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[j] *= row_scale[0][j];
          x[4 + j] *= row_scale[1][j];
        }
      }
      const int valid = seq_len - tile_of(i) * kTileTokens;  // >= 1
      if (valid < kTileTokens) {                             // only the last tile of the selection
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (16 * (j >> 2) + 4 * g + (j & 3) >= valid) x[j] = -__builtin_inff();
        }
      }
      float tile_max = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
      tile_max = MaxAcrossHalves(MaxAcrossRows16(tile_max));
      // Move the reference only when some head's maximum outgrew it by more than the threshold.
      if (__builtin_amdgcn_ballot_w64(tile_max > m_ref + kRescaleThreshold) != 0) {
        const float m_new = fmaxf(m_ref, tile_max);  // finite: token 0 of the tile is valid
        const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
        l_run *= alpha;
        m_ref = m_new;
        if (i != 0) {  // O is still zero on the first tile (and alpha is exp2(-inf - m) there)
#pragma unroll
          for (int n = 0; n < kDvPerWave; ++n) o[n] *= alpha;
        }
      }
      bf16x8 p;
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = __builtin_amdgcn_exp2f(x[j] - m_ref);
        sum += e;
        p[j] = static_cast<__bf16>(FP8 ? e * row_scale[j >> 2][j & 3] : e);  // V = codes x the row's scale
      }
      l_run += sum;
      StaticFor<kDvPerWave>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int n = decltype(n_c)::value;
        o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[n], p, o[n], 0, 0, 0);
      });
    }
    __syncthreads();  // every output wave is through with the last tile
    const float l_total = SumAcrossHeadLanes(l_run);
    const float inv = 1.0f / l_total;
    float lse2 = m_ref + __builtin_amdgcn_logf(l_total);  // v_log_f32 is log2
#pragma unroll
    for (int n = 0; n < kDvPerWave; ++n) o[n] *= inv;
    // The accumulators hold O^T (lane = head i16, four columns per 16-column tile); each wave turns
    // its 256-byte slices of the 16 rows through its own part of the dead ring (row stride 272 B)
    // and writes them 16 bytes per lane, four whole slices per instruction.
    constexpr int kSliceBytes = kDvPerWave * 16 * 2;  // 256
    constexpr int kStageRow = kSliceBytes + 16;
    unsigned char* stage = lds + G::Slot(0) + hw * (16 * kStageRow);
    const int piece = lane & 15, sub = lane >> 4;
    // (same wave writes and reads the staging rows: the LDS queue is in order, no barrier needed)
    const auto rows_of_o = [&](u32x4 (&v)[4]) __attribute__((always_inline)) {
#pragma unroll
      for (int n = 0; n < kDvPerWave; ++n) {
        u32x2 packed;
        packed.x = PackBf16(o[n][0], o[n][1]);
        packed.y = PackBf16(o[n][2], o[n][3]);
        *reinterpret_cast<u32x2*>(stage + i16 * kStageRow + (16 * n + 4 * g) * 2) = packed;
      }
#pragma unroll
      for (int it = 0; it < 4; ++it) v[it] = *reinterpret_cast<const u32x4*>(stage + (4 * it + sub) * kStageRow + piece * 16);
    };
    u32x4 v[4];
    if (shared) {
      // This half's partial at (pair, half) of the workspace: 16 rows of 1 KB, and behind the rows
      // of all pairs the 16 LSEs once per slice, so that each wave's count covers what its partner reads.
      const int pair = seq * head_blocks + hb;
      const int64_t row0 = static_cast<int64_t>(2 * pair + half) * 16, other0 = static_cast<int64_t>(2 * pair + (half ^ 1)) * 16;
      float* lses = reinterpret_cast<float*>(a.partial_out + static_cast<int64_t>(a.batch) * head_blocks * 32 * (kLatentDim * 2));
      rows_of_o(v);
      char* mine = a.partial_out + row0 * (kLatentDim * 2) + kSliceBytes * hw + piece * 16;
#pragma unroll
      for (int it = 0; it < 4; ++it) StoreAgent16(mine + (4 * it + sub) * (kLatentDim * 2), v[it]);
      if (g == 0) StoreAgentF32(lses + (row0 * 4 + 16 * hw) + i16, lse2);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's partial stores are complete
      unsigned* word = a.sync + 4 * pair + hw;
      unsigned arrived = 0u;
      if (lane == 0) arrived = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (Uniform(arrived) == 0u) return;  // the other half's wave will find this slice
      if (lane == 0) __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const float lse2_other = LoadAgentF32(lses + (other0 * 4 + 16 * hw) + i16);
      const char* theirs = a.partial_out + other0 * (kLatentDim * 2) + kSliceBytes * hw + piece * 16;
#pragma unroll
      for (int it = 0; it < 4; ++it) v[it] = LoadAgent16(theirs + (4 * it + sub) * (kLatentDim * 2));
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
#pragma unroll
      for (int it = 0; it < 4; ++it) *reinterpret_cast<u32x4*>(stage + (4 * it + sub) * kStageRow + piece * 16) = v[it];
      // Whichever half arrives second, the result is the same: both partials enter as the bf16
      // rows that were stored, the first half's term first.
      const float top = fmaxf(lse2, lse2_other);
      const float w_mine = __builtin_amdgcn_exp2f(lse2 - top), w_theirs = __builtin_amdgcn_exp2f(lse2_other - top);
      const float inv_w = 1.0f / (w_mine + w_theirs);
      const bool second_half = half != 0;
      const float c_first = (second_half ? w_theirs : w_mine) * inv_w, c_second = (second_half ? w_mine : w_theirs) * inv_w;
#pragma unroll
      for (int n = 0; n < kDvPerWave; ++n) {
        const u32x2 packed = *reinterpret_cast<const u32x2*>(stage + i16 * kStageRow + (16 * n + 4 * g) * 2);
        const float theirs[4] = {__builtin_bit_cast(float, packed.x << 16), __builtin_bit_cast(float, packed.x & 0xffff0000u),
                                 __builtin_bit_cast(float, packed.y << 16), __builtin_bit_cast(float, packed.y & 0xffff0000u)};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float mine = static_cast<float>(static_cast<__bf16>(o[n][j]));
          o[n][j] = (second_half ? theirs[j] : mine) * c_first + (second_half ? mine : theirs[j]) * c_second;
        }
      }
      lse2 = top + __builtin_amdgcn_logf(w_mine + w_theirs);
    }
    if (hw == 0 && g == 0 && a.lse != nullptr) a.lse[seq * a.heads + head] = lse2 * 0.6931471805599453f;
    rows_of_o(v);
    char* out0 = a.out + seq * a.out_seq_stride + (16 * hb) * a.out_head_stride + kSliceBytes * hw + piece * 16;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      __builtin_nontemporal_store(v[it], reinterpret_cast<u32x4*>(out0 + (4 * it + sub) * a.out_head_stride));
    }
  }
}

// Dynamic LDS above 64 KB needs the attribute per kernel and device (PrepareAttnKernels).
template <bool FP8, bool ALIGNED, bool MXQ, bool SPARSE>
hipError_t PrepareDecode() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaDecodeKernel<FP8, ALIGNED, MXQ, SPARSE>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, Geom<FP8>::kLdsBytes);
}
template <bool HALVES, bool FP8>
hipError_t PrepareHeadBlock() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaSelectedHeadBlockKernel<HALVES, FP8>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, GeomHeadBlock<FP8>::kLdsBytes);
}
template <bool HALVES, bool FP8>
hipError_t LaunchHeadBlock(const AttnArgs& args, const dim3& units, hipStream_t stream) {
  hipLaunchKernelGGL((MlaSelectedHeadBlockKernel<HALVES, FP8>), units, dim3(kHbThreads), GeomHeadBlock<FP8>::kLdsBytes, stream, args);
  return hipGetLastError();
}
template <bool MXQ, bool SPARSE>
hipError_t PrepareMerge() {
  hipFuncAttributes attributes;
  return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&MlaMergeKernel<MXQ, SPARSE>));
}

template <bool FP8, bool ALIGNED, bool MXQ, bool SPARSE>
hipError_t Launch(const AttnArgs& args, const dim3& grid, hipStream_t stream) {
  hipLaunchKernelGGL((MlaDecodeKernel<FP8, ALIGNED, MXQ, SPARSE>), grid, dim3(kThreads), Geom<FP8>::kLdsBytes, stream, args);
  return hipGetLastError();
}

template <bool MXQ>
hipError_t LaunchByCache(const AttnArgs& args, const dim3& grid, hipStream_t stream) {
  const bool aligned = args.block_size % kTileTokens == 0;
  if (args.fp8) return aligned ? Launch<true, true, MXQ, false>(args, grid, stream) : Launch<true, false, MXQ, false>(args, grid, stream);
  return aligned ? Launch<false, true, MXQ, false>(args, grid, stream) : Launch<false, false, MXQ, false>(args, grid, stream);
}

// Meeting points of the in-launch merge: two words per (head group, sequence), all zero between
// launches (the last contributor to leave a sequence clears its words). A launch takes the next of kSyncRegions
// regions, so that launches running side by side on different streams do not share counters.
constexpr int kSyncRegions = 16;
static __device__ __align__(256) unsigned int sync_words[kSyncRegions][kAttnSyncSequences * 2];

hipError_t SyncRegion(unsigned** region) {
  constexpr int kMaxDevices = 64;
  static std::mutex guard;
  static unsigned* per_device[kMaxDevices] = {};
  static unsigned next[kMaxDevices] = {};
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(guard);
  if (per_device[device] == nullptr) {
    void* resolved = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&resolved, HIP_SYMBOL(sync_words)); e != hipSuccess) return e;
    if (resolved == nullptr) return hipErrorInvalidSymbol;
    per_device[device] = static_cast<unsigned*>(resolved);
  }
  *region = per_device[device] + static_cast<size_t>(next[device]++ % kSyncRegions) * (kAttnSyncSequences * 2);
  return hipSuccess;
}

}  // namespace

hipError_t PrepareAttnKernels() {
  static std::mutex guard;
  static PerDeviceOnce once;
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 0 || device >= PerDeviceOnce::kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(guard);
  if (once.state[device] == 1) return hipSuccess;
  const hipError_t results[] = {
      PrepareDecode<false, true, false, false>(), PrepareDecode<false, false, false, false>(),
      PrepareDecode<true, true, false, false>(),  PrepareDecode<true, false, false, false>(),
      PrepareDecode<false, true, true, false>(),  PrepareDecode<false, false, true, false>(),
      PrepareDecode<true, true, true, false>(),   PrepareDecode<true, false, true, false>(),
      PrepareDecode<false, false, false, true>(), PrepareDecode<true, false, false, true>(),
      PrepareMerge<false, false>(), PrepareMerge<true, false>(), PrepareMerge<false, true>(),
      PrepareHeadBlock<false, false>(), PrepareHeadBlock<true, false>(), PrepareHeadBlock<false, true>(), PrepareHeadBlock<true, true>()};
  for (const hipError_t e : results) {
    if (e != hipSuccess) return e;
  }
  once.state[device] = 1;
  return hipSuccess;
}

// Whether any sequence of the launch is cut into several work units, i.e. whether partials will be
// written that the merge has to put together. The host can tell when it knows the token counts:
// a selection has the same count for every sequence, and lengths that ride in the argument block
// are here; it then makes the cut the kernels make (same functions). Lengths in device memory: yes.
bool AnySequenceSplit(const AttnArgs& a) {
  const bool sparse = a.sparse_indices != nullptr;
  if (!sparse && a.inline_count <= 0) return true;
  const auto tiles_of = [&](int seq) {
    const int tokens = sparse ? a.sparse_count : std::min(std::max(a.inline_lens[seq], 0), a.max_tokens);
    return (tokens + kTileTokens - 1) / kTileTokens;
  };
  int total = 0, live = 0, common = 0;  // as SeqWindow accumulates them
  for (int seq = 0; seq < a.batch; ++seq) {
    const int tiles = tiles_of(seq);
    if (tiles == 0) continue;
    total += tiles;
    ++live;
    common = common == 0 || common == tiles ? tiles : -1;
  }
  if (live == 0) return false;
  const Cut cut = MakeCut(a, total, live, common, a.work_groups);
  int end_tiles = 0, end_live = 0;
  for (int seq = 0; seq < a.batch; ++seq) {
    const int tiles = tiles_of(seq);
    if (tiles == 0) continue;
    end_tiles += tiles;
    ++end_live;
    const int seq_end = end_tiles + cut.pad * end_live;
    if ((seq_end - 1) / cut.tiles_per_unit != (seq_end - tiles) / cut.tiles_per_unit) return true;
  }
  return false;
}

// Whole-selection units of 16 heads, one workgroup per unit or two (head_block_units 1 / 2).
static hipError_t LaunchHeadBlockUnits(AttnArgs& args, hipStream_t stream) {
  const int sequences_per_xcd = (args.batch + kXcds - 1) / kXcds;
  const int64_t pairs = static_cast<int64_t>(args.batch) * (args.heads / 16);
  // Two workgroups per unit meet on four words each of this launch's counters and leave their
  // partials in the first 2 x 16 x pairs rows of the workspace, the LSEs behind them (the plan
  // sizes the workspace for that).
  const bool halves = args.head_block_units == 2 && pairs * 4 <= kAttnSyncSequences * 2 && args.partial_out != nullptr;
  if (halves) {
    if (hipError_t sync_error = SyncRegion(&args.sync); sync_error != hipSuccess) return sync_error;
    const dim3 units(kXcds * (args.heads / 16) * 2 * sequences_per_xcd);
    return args.fp8 ? LaunchHeadBlock<true, true>(args, units, stream) : LaunchHeadBlock<true, false>(args, units, stream);
  }
  const dim3 units(kXcds * (args.heads / 16) * sequences_per_xcd);
  return args.fp8 ? LaunchHeadBlock<false, true>(args, units, stream) : LaunchHeadBlock<false, false>(args, units, stream);
}

hipError_t LaunchAttnDecode(const AttnArgs& args_in, hipStream_t stream) {
  AttnArgs args = args_in;
  if (args.batch <= 0) return hipSuccess;
  if (hipError_t e = PrepareAttnKernels(); e != hipSuccess) return e;
  const int head_groups = (args.heads + 63) / 64;
  const bool merge_in_launch = args.merge_in_launch && static_cast<int64_t>(args.batch) * head_groups <= kAttnSyncSequences;
  args.sync = nullptr;
  if (merge_in_launch) {
    if (hipError_t e = SyncRegion(&args.sync); e != hipSuccess) return e;
  }
  const dim3 grid(args.work_groups, head_groups);
  const bool quantise = args.out_codes != nullptr;
  const bool sparse = args.sparse_indices != nullptr;
  hipError_t e;
  if (sparse) {
    if (quantise) return hipErrorInvalidValue;
    // a selected token is staged as (block << ceil(log2(block_size))) | slot in 31 bits
    int slot_bits = 0;
    while ((int64_t{1} << slot_bits) < args.block_size) ++slot_bits;
    if ((static_cast<int64_t>(args.num_blocks) << slot_bits) > (int64_t{1} << 31)) return hipErrorInvalidValue;
    // (a pool whose rows the 32-bit starts of the whole-selection units cannot address goes to the split units)
    if (args.head_block_units != 0 && PlainRowsAddressable(args)) {
      if (args.sparse_count > kAttnHeadBlockTokens || args.heads % 16 != 0 || args.out == nullptr) return hipErrorInvalidValue;
      return LaunchHeadBlockUnits(args, stream);
    }
    e = args.fp8 ? Launch<true, false, false, true>(args, grid, stream) : Launch<false, false, false, true>(args, grid, stream);
  } else if (args.head_block_units != 0 && !quantise && args.out != nullptr && args.heads % 16 == 0 && args.sparse_count > 0 &&
             args.sparse_count <= kAttnHeadBlockTokens && PlainRowsAddressable(args)) {
    // a whole context of up to sparse_count tokens in the units of the selected-token attention: no
    // selection, a sequence attends to its own positions
    return LaunchHeadBlockUnits(args, stream);
  } else {
    e = quantise ? LaunchByCache<true>(args, grid, stream) : LaunchByCache<false>(args, grid, stream);
  }
  if (e != hipSuccess || merge_in_launch) return e;
  if (!AnySequenceSplit(args)) return hipSuccess;  // every sequence is written by the one unit that holds it
  const dim3 merge_grid((std::min(64, args.heads) + kMergeHeads - 1) / kMergeHeads, args.batch, head_groups);
  if (sparse) {
    hipLaunchKernelGGL((MlaMergeKernel<false, true>), merge_grid, dim3(kMergeHeads * 64), 0, stream, args);
  } else if (quantise) {
    hipLaunchKernelGGL((MlaMergeKernel<true, false>), merge_grid, dim3(kMergeHeads * 64), 0, stream, args);
  } else {
    hipLaunchKernelGGL((MlaMergeKernel<false, false>), merge_grid, dim3(kMergeHeads * 64), 0, stream, args);
  }
  return hipGetLastError();
}

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

}  // namespace mlakv
