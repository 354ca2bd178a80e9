// Paged KV data movement for gfx950: append (scatter of token rows into physical blocks),
// block-table gather, compaction block copy; bf16 byte copies and the FP8-E4M3 row-scaled
// variants (quantize on append, dequantize on gather).
//
// All three are HBM-bound. One wavefront owns one work item (a token row for append, a
// run of rows of one physical block for gather/compaction); every lane moves 16 bytes per
// access (global_load/store_dwordx4), so a 1024-byte latent row is exactly one wave access
// and eight 128-byte rope rows are another. The block-table entry and all row bases are
// wave-uniform, so the address arithmetic stays in scalar registers.
#include <mutex>

#include "kernels.h"

#include <hip/hip_ext.h>

#include <type_traits>

namespace mlakv {
namespace {

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int kWave = 64;
constexpr int kWavesPerGroup = 4;
constexpr int kThreads = kWave * kWavesPerGroup;

// Every byte is touched once: non-temporal on both sides measured 3-8% faster than cached
// accesses for the gather.
__device__ __forceinline__ u32x4 Load16(const char* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void Store16(char* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x2 Load8(const char* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
}
__device__ __forceinline__ void Store8(char* p, u32x2 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
}
__device__ __forceinline__ int Uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Copies `nrows` rows of CH 16-byte chunks with one wavefront; U accesses in flight.
template <int CH>
__device__ __forceinline__ void CopyRows(const char* src, int64_t src_row_stride, char* dst, int64_t dst_row_stride,
                                         int nrows, int lane) {
  static_assert(CH <= kWave && (kWave % CH) == 0, "a row is at most one wave access");
  constexpr int kRowsPerAccess = kWave / CH;
  constexpr int U = 8;
  const int sub = lane / CH;
  const int chunk = lane % CH;
  const char* s = src + sub * src_row_stride + chunk * 16;
  char* d = dst + sub * dst_row_stride + chunk * 16;
  int r = 0;
  for (; r + kRowsPerAccess * U <= nrows; r += kRowsPerAccess * U) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = Load16(s + static_cast<int64_t>(r + u * kRowsPerAccess) * src_row_stride);
#pragma unroll
    for (int u = 0; u < U; ++u) Store16(d + static_cast<int64_t>(r + u * kRowsPerAccess) * dst_row_stride, v[u]);
  }
  if (r < nrows) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = r + u * kRowsPerAccess;
      if (row + sub < nrows) v[u] = Load16(s + static_cast<int64_t>(row) * src_row_stride);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = r + u * kRowsPerAccess;
      if (row + sub < nrows) Store16(d + static_cast<int64_t>(row) * dst_row_stride, v[u]);
    }
  }
}

// ---- number formats ---------------------------------------------------------

__device__ __forceinline__ float Bf16ToF32(unsigned int bits16) { return __builtin_bit_cast(float, bits16 << 16); }

// Round to nearest even; inputs here are finite.
__device__ __forceinline__ unsigned int F32ToBf16(float v) {
  unsigned int bits = __builtin_bit_cast(unsigned int, v);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return bits >> 16;
}

// Two floats -> two bf16 in one dword, rounded to nearest even by the conversion instruction
// (v_cvt_pk_bf16_f32; a NaN stays a quiet NaN of its sign).
__device__ __forceinline__ unsigned int PackBf16Pair(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const bf16x2_t packed = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(unsigned int, packed);
}

// Eight E4M3 codes -> eight bf16, each decoded value times `scale`, rounded to nearest even.
__device__ __forceinline__ u32x4 Dequant8(u32x2 codes, float scale) {
  const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes.x), false);
  const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes.x), true);
  const f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes.y), false);
  const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(codes.y), true);
  u32x4 out;
  out.x = PackBf16Pair(a.x * scale, a.y * scale);
  out.y = PackBf16Pair(b.x * scale, b.y * scale);
  out.z = PackBf16Pair(c.x * scale, c.y * scale);
  out.w = PackBf16Pair(d.x * scale, d.y * scale);
  return out;
}

// ---- append -----------------------------------------------------------------

// One wavefront per (run of consecutive tokens, layer). bf16: 64 lanes move a latent row, 8 lanes
// a rope row. The source rows do not depend on the slots, so all of a wavefront's loads (slots
// and rows) are issued together: with the row fetched only after its slot had arrived, a
// prefill-sized append was bound by two memory latencies per row. The quantising kernel, which has
// a shuffle reduction and a division per row to hide, takes four rows per wavefront.
struct StoreWordsArgs {
  int32_t words[kMaxStoreWords];
};
// The step's metadata riding in the argument block of an append launch: `count` words for `dst`
// (the slot mapping comes first in them), then `pairs` (index, value) couples for `scatter_dst`.
struct StepWords {
  StoreWordsArgs args;
  int32_t count, pairs;
  int32_t* dst;
  int32_t* scatter_dst;
};
struct NoStepWords {};

// Slot of `token`: from the argument block when the launch carries the step's words (the copy in
// memory is being written by the first workgroup of this very launch), else from memory.
template <typename WORDS>
__device__ __forceinline__ int SlotOf(const AppendArgs& a, const WORDS& w, int token) {
  if constexpr (std::is_same<WORDS, StepWords>::value) {
    return w.args.words[token];
  } else {
    return a.slots[token];
  }
}
template <typename WORDS>
__device__ __forceinline__ void StoreStepWords(const WORDS& w) {
  if constexpr (std::is_same<WORDS, StepWords>::value) {
    if (blockIdx.x == 0 && blockIdx.y == 0) {
      for (int i = threadIdx.x; i < w.count; i += kThreads) w.dst[i] = w.args.words[i];
      for (int i = threadIdx.x; i < w.pairs; i += kThreads) w.scatter_dst[w.args.words[w.count + 2 * i]] = w.args.words[w.count + 2 * i + 1];
    }
  }
}

constexpr int kAppendRows = 4;      // FP8: rows per wavefront
constexpr int kAppendRowsBf16 = 1;  // bf16: a pure copy ran fastest with one row per wavefront (8 layers x 311k rows: 984 us, 1081 with two, 1106 with four)

template <typename WORDS>
__global__ __launch_bounds__(kThreads) void AppendBf16Kernel(AppendArgs a, WORDS w) {
  StoreStepWords(w);
  const int lane = threadIdx.x & (kWave - 1);
  const int token0 = Uniform((blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6)) * kAppendRowsBf16);
  const int layer = blockIdx.y;
  if (token0 >= a.num_tokens) return;
  int my_slot = -1;
  if (lane < kAppendRowsBf16 && token0 + lane < a.num_tokens) my_slot = SlotOf(a, w, token0 + lane);
  static_assert(kLatentDim * 2 / 16 == kWave, "one latent row is one wave access");
  const bool rope_lane = lane < kRopeDim * 2 / 16;
  const char* latent_src = a.latent_src.base + layer * a.latent_src.layer_stride;
  const char* rope_src = a.rope_src.base + layer * a.rope_src.layer_stride;
  u32x4 v[kAppendRowsBf16], r[kAppendRowsBf16];
  // a row past the end repeats the last one: loaded, never stored (its slot lane holds -1)
#pragma unroll
  for (int i = 0; i < kAppendRowsBf16; ++i) v[i] = Load16(latent_src + min(token0 + i, a.num_tokens - 1) * a.latent_src.row_stride + lane * 16);
  if (rope_lane) {  // one branch around all rope loads: a branch per row made the compiler wait between the rows
#pragma unroll
    for (int i = 0; i < kAppendRowsBf16; ++i) r[i] = Load16(rope_src + min(token0 + i, a.num_tokens - 1) * a.rope_src.row_stride + lane * 16);
  }
  char* latent_dst[kAppendRowsBf16];
  char* rope_dst[kAppendRowsBf16];
  bool live[kAppendRowsBf16];
#pragma unroll
  for (int i = 0; i < kAppendRowsBf16; ++i) {
    const int slot = __builtin_amdgcn_readlane(my_slot, i);
    const int block = slot < 0 ? 0 : slot / a.block_size;
    const int in_block = slot < 0 ? 0 : slot - block * a.block_size;
    live[i] = slot >= 0 && block < a.num_blocks;
    latent_dst[i] = a.latent.base + layer * a.latent.layer_stride + block * a.latent.block_stride + in_block * a.latent.row_stride;
    rope_dst[i] = a.rope.base + layer * a.rope.layer_stride + block * a.rope.block_stride + in_block * a.rope.row_stride;
  }
#pragma unroll
  for (int i = 0; i < kAppendRowsBf16; ++i) {
    if (live[i]) Store16(latent_dst[i] + lane * 16, v[i]);
  }
  if (rope_lane) {
#pragma unroll
    for (int i = 0; i < kAppendRowsBf16; ++i) {
      if (live[i]) Store16(rope_dst[i] + lane * 16, r[i]);
    }
  }
}

// Two quotients -> two E4M3 codes in the low half of a dword. v_cvt_pk_fp8_f32 rounds to nearest
// even onto the OCP E4M3FN grid (subnormal grid 2^-9 below 2^-6 included): checked against a
// software encoder over every float bit pattern below 464; beyond that it returns NaN, so the
// clamp to +-448 provides the saturation for every other number. A NaN keeps its sign and becomes
// the format's NaN (a clamp made of minima and maxima would turn it into -448).
__device__ __forceinline__ unsigned int E4m3EncodePair(float a, float b) {
  const unsigned nan_a = ((__builtin_bit_cast(unsigned, a) >> 24) & 0x80u) | 0x7fu, nan_b = ((__builtin_bit_cast(unsigned, b) >> 24) & 0x80u) | 0x7fu;
  const bool a_is_nan = a != a, b_is_nan = b != b;
  a = fminf(fmaxf(a, -448.0f), 448.0f);
  b = fminf(fmaxf(b, -448.0f), 448.0f);
  const unsigned codes = static_cast<unsigned int>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xffffu;
  return (a_is_nan ? nan_a : codes & 0xffu) | ((b_is_nan ? nan_b : codes >> 8) << 8);
}

// Maximum over the 64 lanes, in every lane, of values that are neither negative nor NaN, without
// the LDS crossbar: their bit patterns order like the values, so the steps are integer maxima, four
// with data-parallel-primitive operands inside each row of 16 lanes (neighbour, other pair, mirrored
// half, mirrored row), then v_permlane16_swap (odd and even rows) and v_permlane32_swap (the two
// halves). A shuffle per step (ds_bpermute and a wait for it, six times in a row) and float maxima
// that re-quiet their operands made the FP8 append arithmetic-bound.
template <int CONTROL>
__device__ __forceinline__ unsigned DppMaxU32(unsigned x) {
  const int bits = static_cast<int>(x);
  return max(x, static_cast<unsigned>(__builtin_amdgcn_update_dpp(bits, bits, CONTROL, 0xf, 0xf, true)));
}
__device__ __forceinline__ float WaveMaxNonNegative(float value) {
  typedef __attribute__((ext_vector_type(2))) unsigned int u32x2_t;
  unsigned x = __builtin_bit_cast(unsigned, value);
  x = DppMaxU32<0xB1>(x);   // quad_perm [1,0,3,2]
  x = DppMaxU32<0x4E>(x);   // quad_perm [2,3,0,1]
  x = DppMaxU32<0x141>(x);  // row_half_mirror
  x = DppMaxU32<0x140>(x);  // row_mirror
  u32x2_t swapped = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  x = max(static_cast<unsigned>(swapped.x), static_cast<unsigned>(swapped.y));
  swapped = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  return __builtin_bit_cast(float, max(static_cast<unsigned>(swapped.x), static_cast<unsigned>(swapped.y)));
}

// Quantises one row held by a wave (lane: 8 latent values, 1 rope value) and stores codes and
// scale: per-row absmax by wave shuffles, scale = absmax/448, code = e4m3(x / scale) with the
// correctly rounded quotient.
__device__ __forceinline__ void QuantizeRowAndStore(const AppendArgs& a, int layer, int block, int in_block, int lane,
                                                    const float (&x)[8], float y) {
  float absmax = fmaxf(0.0f, fabsf(y));  // a NaN never becomes the maximum (a row of nothing but NaNs has absmax 0)
#pragma unroll
  for (int i = 0; i < 8; ++i) absmax = fmaxf(absmax, fabsf(x[i]));
  absmax = WaveMaxNonNegative(absmax);
  // The usual row: a maximum in [2^-100, the largest finite float] (as bit patterns, on the scalar
  // unit: the value is the same in every lane).
  const unsigned absmax_bits = __builtin_amdgcn_readfirstlane(__builtin_bit_cast(unsigned, absmax));
  const bool usual = absmax_bits - 0x0d800000u <= 0x7f7fffffu - 0x0d800000u;
  // scale = absmax / 448, correctly rounded. In the usual range three operations do it: with
  // y = RN(1/448), q = absmax * y, then q + (absmax - 448 q) * y in one fused step each. absmax is a
  // bf16 value; that the result equals the rounded quotient was checked for every one of the
  // 29,184 bf16 values of that range in exact arithmetic (tests/test_oracle_formats.py).
  float scale;
  if (usual) {
    const float y448 = __builtin_bit_cast(float, 0x3b124925u);
    const float q0 = absmax * y448;
    scale = __builtin_fmaf(__builtin_fmaf(-448.0f, q0, absmax), y448, q0);
  } else {
    scale = absmax == 0.0f ? 1.0f : absmax / 448.0f;
  }
  // code = e4m3(x / scale) with the correctly rounded fp32 quotient. Nine divisions per lane made
  // this kernel compute-bound, so the quotient is first taken as x * r with r the hardware's
  // reciprocal of the scale (within one unit in the last place): the product is within 2^-22
  // relative of the rounded quotient (2^-23 from r, 2^-24 from each of the two roundings); the
  // encoding is monotone, so if the two ends of that interval (widened to 2^-21) encode alike, so
  // does the exact quotient. Only a lane that holds a value this close to a rounding boundary of
  // the E4M3 grid (about one in 10^5 values) divides. A scale so small that its reciprocal leaves the
  // normal range (the instruction reads a subnormal as zero) sends the whole row to the divisions,
  // and so does an infinite one (quotients 0 and NaN). A usual row needs no clamp: its quotients
  // stay below 448 (1 + 2^-21), which the conversion rounds to 448, and a NaN stays one.
  const float inverse = __builtin_amdgcn_rcpf(scale);
  float q[9];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = x[i] * inverse;
  q[8] = y * inverse;
  constexpr float kWiden = 4.76837158203125e-07f;  // 2^-21
  // four codes per dword: the conversion writes one half of its destination and keeps the other
  const auto four_codes = [&](float widen, int i) __attribute__((always_inline)) {
    const int low = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_fmaf(q[i], widen, q[i]), __builtin_fmaf(q[i + 1], widen, q[i + 1]), 0, false);
    return static_cast<unsigned>(
        __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_fmaf(q[i + 2], widen, q[i + 2]), __builtin_fmaf(q[i + 3], widen, q[i + 3]), low, true));
  };
  const unsigned below_lo = four_codes(-kWiden, 0), below_hi = four_codes(-kWiden, 4);
  const unsigned above_lo = four_codes(kWiden, 0), above_hi = four_codes(kWiden, 4);
  const unsigned below_rope = static_cast<unsigned>(__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_fmaf(q[8], -kWiden, q[8]), 0.0f, 0, false));
  const unsigned above_rope = static_cast<unsigned>(__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_fmaf(q[8], kWiden, q[8]), 0.0f, 0, false));
  const bool settled = usual && below_lo == above_lo && below_hi == above_hi && ((below_rope ^ above_rope) & 0xffu) == 0u;
  u32x2 lq;
  unsigned int rq;
  if (settled) {
    lq.x = below_lo;
    lq.y = below_hi;
    rq = below_rope & 0xffu;
  } else {
    lq.x = E4m3EncodePair(x[0] / scale, x[1] / scale) | (E4m3EncodePair(x[2] / scale, x[3] / scale) << 16);
    lq.y = E4m3EncodePair(x[4] / scale, x[5] / scale) | (E4m3EncodePair(x[6] / scale, x[7] / scale) << 16);
    rq = E4m3EncodePair(y / scale, 0.0f) & 0xffu;
  }
  char* latent_dst = a.latent.base + layer * a.latent.layer_stride + block * a.latent.block_stride +
                     in_block * a.latent.row_stride;
  char* rope_dst = a.rope.base + layer * a.rope.layer_stride + block * a.rope.block_stride + in_block * a.rope.row_stride;
  Store8(latent_dst + lane * 8, lq);
  reinterpret_cast<unsigned char*>(rope_dst)[lane] = static_cast<unsigned char>(rq);
  if (lane == 0) {
    float* scale_dst = reinterpret_cast<float*>(a.scale.base + layer * a.scale.layer_stride + block * a.scale.block_stride) + in_block;
    *scale_dst = scale;
  }
}

// Quantize-on-append: per-row absmax over latent+rope by wave shuffles, scale = absmax/448,
// code = e4m3(x / scale) with the correctly rounded quotient. Each lane quantizes the 8 latent
// values it loaded (8-byte store) and one of the 64 rope values (1-byte store).
template <typename WORDS>
__global__ __launch_bounds__(kThreads) void AppendFp8Kernel(AppendArgs a, WORDS w) {
  static_assert(kRopeDim == kWave, "one rope element per lane");
  StoreStepWords(w);
  const int lane = threadIdx.x & (kWave - 1);
  const int token0 = Uniform((blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6)) * kAppendRows);
  const int layer = blockIdx.y;
  if (token0 >= a.num_tokens) return;
  int my_slot = -1;
  if (lane < kAppendRows && token0 + lane < a.num_tokens) my_slot = SlotOf(a, w, token0 + lane);
  // the usual block sizes are powers of two: a shift then, not a division per row
  const int block_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(static_cast<unsigned>(a.block_size)) : -1;
  u32x4 lv[kAppendRows];
  unsigned short rv[kAppendRows];
#pragma unroll
  for (int i = 0; i < kAppendRows; ++i) {
    const int token = min(token0 + i, a.num_tokens - 1);  // a repeated row is loaded and never stored
    lv[i] = Load16(a.latent_src.base + layer * a.latent_src.layer_stride + token * a.latent_src.row_stride + lane * 16);
    rv[i] = *reinterpret_cast<const unsigned short*>(a.rope_src.base + layer * a.rope_src.layer_stride + token * a.rope_src.row_stride + lane * 2);
  }
#pragma unroll
  for (int i = 0; i < kAppendRows; ++i) {
    const int slot = __builtin_amdgcn_readlane(my_slot, i);
    if (slot < 0) continue;
    const int block = block_shift >= 0 ? slot >> block_shift : slot / a.block_size;
    const int in_block = slot - block * a.block_size;
    if (block >= a.num_blocks) continue;
    float x[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x[2 * j] = Bf16ToF32(lv[i][j] & 0xffffu);
      x[2 * j + 1] = Bf16ToF32(lv[i][j] >> 16);
    }
    QuantizeRowAndStore(a, layer, block, in_block, lane, x, Bf16ToF32(rv[i]));
  }
}

// ---- latent RMSNorm + key RoPE + append ---------------------------------------------------

// One wavefront per token of one layer: lane l holds latent elements 8l..8l+7 and rope element l.
//   y = x * gamma / sqrt(mean(x^2) + eps)   (fp32; sum of squares by wave shuffles)
//   r'[i] = r[i] cos[i] - r[i+32] sin[i],  r'[i+32] = r[i+32] cos[i+32] + r[i] sin[i+32]  ("half" rotation)
// both rounded to bf16 (nearest even) and written to the cache row of slot[t] (quantised first for
// an FP8 cache, from the bf16 values, as the unfused stages would) and to the optional outputs.
// Query rope slices, rotated in place: a wavefront takes eight heads of one token, eight lanes per
// head, 16 bytes (8 values) per lane. The partner half of a head sits four lanes away.
constexpr int kQueryHeadsPerItem = 8;

__device__ __forceinline__ void RotateQueryHeads(const NormRopeAppendArgs& n, int token, int head0, int lane) {
  static_assert(kRopeDim == 64, "eight lanes of eight values cover a head's rope slice");
  const int head = head0 + (lane >> 3);
  const int part = lane & 7;
  if (head >= n.num_heads) return;
  const int position = Uniform(n.positions[token]);
  char* q = n.q_rope + token * n.q_rope_token_stride + head * n.q_rope_head_stride + part * 16;
  const u32x4 qv = Load16(q);
  const u32x4 cv = *reinterpret_cast<const u32x4*>(n.rope_cos + position * n.rope_table_row_stride + part * 16);
  const u32x4 sv = *reinterpret_cast<const u32x4*>(n.rope_sin + position * n.rope_table_row_stride + part * 16);
  u32x4 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned pv = __shfl_xor(qv[i], 4);
    unsigned packed = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float x = Bf16ToF32((qv[i] >> (16 * h)) & 0xffffu), partner = Bf16ToF32((pv >> (16 * h)) & 0xffffu);
      const float c = Bf16ToF32((cv[i] >> (16 * h)) & 0xffffu), s = Bf16ToF32((sv[i] >> (16 * h)) & 0xffffu);
      packed |= F32ToBf16(part < 4 ? x * c - partner * s : x * c + partner * s) << (16 * h);
    }
    out[i] = packed;
  }
  Store16(q, out);
}

// R rows per wavefront when no query heads ride along: a row's table loads wait for its position,
// so a wavefront spends two memory latencies on a row, and two rows share them.
template <bool FP8, int R>
__global__ __launch_bounds__(kThreads) void NormRopeAppendKernel(NormRopeAppendArgs n) {
  static_assert(kRopeDim == kWave && kLatentDim == 8 * kWave, "lane = 8 latent + 1 rope element");
  const AppendArgs& a = n.append;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave_item = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  const int item_token = wave_item / n.items_per_token;  // items_per_token == 1 whenever R > 1
  const int sub_item = wave_item - item_token * n.items_per_token;
  const int token0 = Uniform(item_token * R);
  if (token0 >= a.num_tokens) return;
  if (sub_item > 0) {
    RotateQueryHeads(n, token0, (sub_item - 1) * kQueryHeadsPerItem, lane);
    return;
  }
  const u32x4 gv = *reinterpret_cast<const u32x4*>(n.gamma + lane * 16);
  u32x4 lv[R];
  unsigned short rv[R], cv[R], sv[R];
  int slot[R];
  bool live[R];
#pragma unroll
  for (int k = 0; k < R; ++k) {
    live[k] = token0 + k < a.num_tokens;  // wave-uniform
    const int token = live[k] ? token0 + k : token0;
    const char* row = n.kv_a + token * n.kv_a_row_stride;
    lv[k] = Load16(row + lane * 16);
    rv[k] = *reinterpret_cast<const unsigned short*>(row + kLatentDim * 2 + lane * 2);
    const int position = Uniform(n.positions[token]);
    cv[k] = *reinterpret_cast<const unsigned short*>(n.rope_cos + position * n.rope_table_row_stride + lane * 2);
    sv[k] = *reinterpret_cast<const unsigned short*>(n.rope_sin + position * n.rope_table_row_stride + lane * 2);
    slot[k] = Uniform(a.slots[token]);
  }
  float g[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    g[2 * i] = Bf16ToF32(gv[i] & 0xffffu);
    g[2 * i + 1] = Bf16ToF32(gv[i] >> 16);
  }
#pragma unroll
  for (int k = 0; k < R; ++k) {
    if (!live[k]) continue;
    const int token = token0 + k;
    const float r = Bf16ToF32(rv[k]), c = Bf16ToF32(cv[k]), s = Bf16ToF32(sv[k]);
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = Bf16ToF32(lv[k][i] & 0xffffu);
      x[2 * i + 1] = Bf16ToF32(lv[k][i] >> 16);
    }
    float sum_squares = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum_squares += x[i] * x[i];
#pragma unroll
    for (int offset = 32; offset >= 1; offset >>= 1) sum_squares += __shfl_xor(sum_squares, offset);
    const float rstd = 1.0f / __builtin_sqrtf(sum_squares * (1.0f / kLatentDim) + n.epsilon);
    u32x4 yv;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned lo = F32ToBf16(x[2 * i] * rstd * g[2 * i]), hi = F32ToBf16(x[2 * i + 1] * rstd * g[2 * i + 1]);
      yv[i] = lo | (hi << 16);
      x[2 * i] = Bf16ToF32(lo);
      x[2 * i + 1] = Bf16ToF32(hi);
    }
    const float partner = __shfl_xor(r, 32);
    const unsigned rotated = F32ToBf16(lane < 32 ? r * c - partner * s : r * c + partner * s);
    if (n.latent_out != nullptr) Store16(n.latent_out + token * n.latent_out_row_stride + lane * 16, yv);
    if (n.rope_out != nullptr) *reinterpret_cast<unsigned short*>(n.rope_out + token * n.rope_out_row_stride + lane * 2) = static_cast<unsigned short>(rotated);
    if (slot[k] < 0) continue;
    const int block = slot[k] / a.block_size;
    const int in_block = slot[k] - block * a.block_size;
    if (block >= a.num_blocks) continue;
    if (FP8) {
      QuantizeRowAndStore(a, 0, block, in_block, lane, x, Bf16ToF32(rotated));
    } else {
      char* latent_dst = a.latent.base + block * a.latent.block_stride + in_block * a.latent.row_stride;
      char* rope_dst = a.rope.base + block * a.rope.block_stride + in_block * a.rope.row_stride;
      Store16(latent_dst + lane * 16, yv);
      *reinterpret_cast<unsigned short*>(rope_dst + lane * 2) = static_cast<unsigned short>(rotated);
    }
  }
}

// ---- gather -----------------------------------------------------------------

// Work item (one wavefront) = `rows_per_item` consecutive token slots of one logical block of
// one sequence in one layer. grid = (items / 4, batch, layers).
struct GatherItem {
  int seq, layer, physical_block, row0, nrows;
  int64_t out_row0;
  bool valid;
};

__device__ __forceinline__ GatherItem ResolveGatherItem(const GatherArgs& g, int rows_per_item) {
  GatherItem item;
  item.valid = false;
  const int wave_item = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  item.seq = blockIdx.y;
  item.layer = blockIdx.z;
  const int seq_len = Uniform(g.seq_lens[item.seq]);
  const int items_per_block = g.block_size / rows_per_item;
  const int logical_block = wave_item / items_per_block;
  item.row0 = (wave_item - logical_block * items_per_block) * rows_per_item;
  const int position0 = logical_block * g.block_size + item.row0;
  if (position0 >= seq_len) return item;
  item.nrows = min(rows_per_item, seq_len - position0);
  item.physical_block = Uniform(g.block_table[static_cast<int64_t>(item.seq) * g.table_stride + logical_block]);
  if (static_cast<unsigned>(item.physical_block) >= static_cast<unsigned>(g.num_blocks)) return item;
  item.out_row0 = static_cast<int64_t>(Uniform(g.cu_seq_lens[item.seq])) + position0;
  item.valid = true;
  return item;
}

__global__ __launch_bounds__(kThreads) void GatherBf16Kernel(GatherArgs g, int rows_per_item) {
  const GatherItem item = ResolveGatherItem(g, rows_per_item);
  if (!item.valid) return;
  const int lane = threadIdx.x & (kWave - 1);
  const char* latent_src = g.latent.base + item.layer * g.latent.layer_stride +
                           item.physical_block * g.latent.block_stride + item.row0 * g.latent.row_stride;
  char* latent_dst = g.latent_dst.base + item.layer * g.latent_dst.layer_stride + item.out_row0 * g.latent_dst.row_stride;
  CopyRows<kLatentDim * 2 / 16>(latent_src, g.latent.row_stride, latent_dst, g.latent_dst.row_stride, item.nrows, lane);
  const char* rope_src = g.rope.base + item.layer * g.rope.layer_stride + item.physical_block * g.rope.block_stride +
                         item.row0 * g.rope.row_stride;
  char* rope_dst = g.rope_dst.base + item.layer * g.rope_dst.layer_stride + item.out_row0 * g.rope_dst.row_stride;
  CopyRows<kRopeDim * 2 / 16>(rope_src, g.rope.row_stride, rope_dst, g.rope_dst.row_stride, item.nrows, lane);
}

// Fast path for block sizes that are a multiple of WG_ROWS: one workgroup owns WG_ROWS
// consecutive rows of one physical block. Each wave moves WG_ROWS/4 latent rows (one
// 1024-byte row per access) and the first WG_ROWS/8 waves move eight 128-byte rope rows
// each, so full items run without any per-lane predicate. The three table reads are
// independent and issued together.
// Measured on MI355X (batch 32, contexts 128..2048, 43 layers): 8 rows per workgroup beats 16
// and 32 (5.77 vs 5.54 vs 5.43 TB/s), and holding residency to five workgroups per CU with
// an unused LDS reservation adds another 1.5%: fewer concurrent streams keep DRAM pages open.
constexpr int kGatherTileRows = 8;
constexpr int kGatherLdsReserve = 32000;

template <int WG_ROWS>
__global__ __launch_bounds__(kThreads) void GatherBf16TileKernel(GatherArgs g, int items_per_block) {
  static_assert(WG_ROWS % 8 == 0 && WG_ROWS <= 32, "rope rows go eight per wave access");
  constexpr int kLatentRowsPerWave = WG_ROWS / kWavesPerGroup;
  constexpr int kRopeWaves = WG_ROWS / 8;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = Uniform(threadIdx.x >> 6);
  const int seq = blockIdx.y;
  const int layer = blockIdx.z;
  const int logical_block = blockIdx.x / items_per_block;
  const int row0 = (blockIdx.x - logical_block * items_per_block) * WG_ROWS;
  const int seq_len = Uniform(g.seq_lens[seq]);
  const int64_t out_base = Uniform(g.cu_seq_lens[seq]);
  const int physical_block = Uniform(g.block_table[static_cast<int64_t>(seq) * g.table_stride + logical_block]);
  const int position0 = logical_block * g.block_size + row0;
  if (position0 >= seq_len) return;
  if (static_cast<unsigned>(physical_block) >= static_cast<unsigned>(g.num_blocks)) return;
  const int nrows = min(WG_ROWS, seq_len - position0);
  const int64_t out_row0 = out_base + position0;
  const char* latent_src = g.latent.base + layer * g.latent.layer_stride + physical_block * g.latent.block_stride +
                           (row0 + wave * kLatentRowsPerWave) * g.latent.row_stride + lane * 16;
  char* latent_dst = g.latent_dst.base + layer * g.latent_dst.layer_stride +
                     (out_row0 + wave * kLatentRowsPerWave) * g.latent_dst.row_stride + lane * 16;
  const int sub = lane >> 3, chunk = lane & 7;
  const char* rope_src = g.rope.base + layer * g.rope.layer_stride + physical_block * g.rope.block_stride +
                         (row0 + wave * 8 + sub) * g.rope.row_stride + chunk * 16;
  char* rope_dst = g.rope_dst.base + layer * g.rope_dst.layer_stride + (out_row0 + wave * 8 + sub) * g.rope_dst.row_stride +
                   chunk * 16;
  if (nrows == WG_ROWS) {
    u32x4 v[kLatentRowsPerWave];
    u32x4 r;
#pragma unroll
    for (int u = 0; u < kLatentRowsPerWave; ++u) v[u] = Load16(latent_src + u * g.latent.row_stride);
    if (wave < kRopeWaves) r = Load16(rope_src);
#pragma unroll
    for (int u = 0; u < kLatentRowsPerWave; ++u) Store16(latent_dst + u * g.latent_dst.row_stride, v[u]);
    if (wave < kRopeWaves) Store16(rope_dst, r);
  } else {
#pragma unroll
    for (int u = 0; u < kLatentRowsPerWave; ++u) {
      if (wave * kLatentRowsPerWave + u < nrows) {
        Store16(latent_dst + u * g.latent_dst.row_stride, Load16(latent_src + u * g.latent.row_stride));
      }
    }
    if (wave * 8 + sub < nrows) Store16(rope_dst, Load16(rope_src));
  }
}

// FP8 rows: each lane decodes 8 codes (8-byte load) to 8 bf16 (16-byte store).
__global__ __launch_bounds__(kThreads) void GatherFp8Kernel(GatherArgs g, int rows_per_item) {
  const GatherItem item = ResolveGatherItem(g, rows_per_item);
  if (!item.valid) return;
  const int lane = threadIdx.x & (kWave - 1);
  const char* latent_src = g.latent.base + item.layer * g.latent.layer_stride +
                           item.physical_block * g.latent.block_stride + item.row0 * g.latent.row_stride;
  const char* rope_src = g.rope.base + item.layer * g.rope.layer_stride + item.physical_block * g.rope.block_stride +
                         item.row0 * g.rope.row_stride;
  const float* scales = reinterpret_cast<const float*>(g.scale.base + item.layer * g.scale.layer_stride +
                                                       item.physical_block * g.scale.block_stride) + item.row0;
  char* latent_dst = g.latent_dst.base + item.layer * g.latent_dst.layer_stride + item.out_row0 * g.latent_dst.row_stride;
  char* rope_dst = g.rope_dst.base + item.layer * g.rope_dst.layer_stride + item.out_row0 * g.rope_dst.row_stride;
  constexpr int U = 4;
  // latent: one row (512 codes) per wave access
  for (int r = 0; r < item.nrows; r += U) {
    u32x2 codes[U];
    float scale[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (r + u < item.nrows) {
        codes[u] = Load8(latent_src + static_cast<int64_t>(r + u) * g.latent.row_stride + lane * 8);
        scale[u] = scales[r + u];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (r + u < item.nrows) Store16(latent_dst + static_cast<int64_t>(r + u) * g.latent_dst.row_stride + lane * 16, Dequant8(codes[u], scale[u]));
    }
  }
  // rope: eight rows (64 codes each) per wave access
  const int sub = lane >> 3, chunk = lane & 7;
  for (int r = 0; r < item.nrows; r += 8) {
    const int row = r + sub;
    if (row < item.nrows) {
      const u32x2 codes = Load8(rope_src + static_cast<int64_t>(row) * g.rope.row_stride + chunk * 8);
      Store16(rope_dst + static_cast<int64_t>(row) * g.rope_dst.row_stride + chunk * 16, Dequant8(codes, scales[row]));
    }
  }
}

// ---- compaction copy ----------------------------------------------------------

// Work item = `rows_per_item` slots of one (src, dst) block pair in one layer.
template <int LATENT_CH, int ROPE_CH>
__global__ __launch_bounds__(kThreads) void CopyBlocksKernel(CopyBlocksArgs c, int rows_per_item) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave_item = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  const int layer = blockIdx.y;
  const int items_per_block = c.block_size / rows_per_item;
  const int move = wave_item / items_per_block;
  if (move >= c.num_moves) return;
  const int row0 = (wave_item - move * items_per_block) * rows_per_item;
  const int src = Uniform(c.moves[2 * move]);
  const int dst = Uniform(c.moves[2 * move + 1]);
  if (static_cast<unsigned>(src) >= static_cast<unsigned>(c.num_blocks) ||
      static_cast<unsigned>(dst) >= static_cast<unsigned>(c.num_blocks)) return;
  char* latent = c.latent.base + layer * c.latent.layer_stride + row0 * c.latent.row_stride;
  CopyRows<LATENT_CH>(latent + src * c.latent.block_stride, c.latent.row_stride, latent + dst * c.latent.block_stride,
                      c.latent.row_stride, rows_per_item, lane);
  char* rope = c.rope.base + layer * c.rope.layer_stride + row0 * c.rope.row_stride;
  CopyRows<ROPE_CH>(rope + src * c.rope.block_stride, c.rope.row_stride, rope + dst * c.rope.block_stride,
                    c.rope.row_stride, rows_per_item, lane);
  if (c.has_scale) {
    char* scale = c.scale.base + layer * c.scale.layer_stride + row0 * 4;
    for (int r = lane; r < rows_per_item; r += kWave) {
      reinterpret_cast<float*>(scale + dst * c.scale.block_stride)[r] =
          reinterpret_cast<const float*>(scale + src * c.scale.block_stride)[r];
    }
  }
}

// Largest divisor of block_size that is at most `want` (work-item granularity).
int RowsPerItem(int block_size, int want) {
  int rows = block_size < want ? block_size : want;
  while (block_size % rows != 0) --rows;
  return rows;
}

int DivUp(int a, int b) { return (a + b - 1) / b; }

// ---- per-step metadata ---------------------------------------------------------

__global__ __launch_bounds__(kThreads) void StoreWordsKernel(StoreWordsArgs args, int count, int32_t* dst, int pairs,
                                                             int32_t* scatter_dst) {
  for (int i = threadIdx.x; i < count; i += kThreads) dst[i] = args.words[i];
  for (int i = threadIdx.x; i < pairs; i += kThreads) scatter_dst[args.words[count + 2 * i]] = args.words[count + 2 * i + 1];
}

}  // namespace

hipError_t LaunchAppend(const AppendArgs& args, hipStream_t stream) {
  if (args.num_tokens <= 0 || args.num_layers <= 0) return hipSuccess;
  if (args.fp8) {
    const dim3 grid(DivUp(args.num_tokens, kWavesPerGroup * kAppendRows), args.num_layers);
    hipLaunchKernelGGL(AppendFp8Kernel<NoStepWords>, grid, dim3(kThreads), 0, stream, args, NoStepWords{});
  } else {
    const dim3 grid(DivUp(args.num_tokens, kWavesPerGroup * kAppendRowsBf16), args.num_layers);
    hipLaunchKernelGGL(AppendBf16Kernel<NoStepWords>, grid, dim3(kThreads), 0, stream, args, NoStepWords{});
  }
  return hipGetLastError();
}

hipError_t LaunchAppendWithWords(const AppendArgs& args, const int32_t* host_words, int count, int32_t* dst, const int32_t* host_pairs,
                                 int pairs, int32_t* scatter_dst, hipStream_t stream) {
  if (args.num_tokens <= 0 || args.num_layers <= 0 || count < args.num_tokens || pairs < 0 || count + 2 * pairs > kMaxStoreWords ||
      host_words == nullptr || dst == nullptr || (pairs > 0 && (host_pairs == nullptr || scatter_dst == nullptr))) {
    return hipErrorInvalidValue;
  }
  StepWords words;
  for (int i = 0; i < count; ++i) words.args.words[i] = host_words[i];
  for (int i = 0; i < 2 * pairs; ++i) words.args.words[count + i] = host_pairs[i];
  words.count = count;
  words.pairs = pairs;
  words.dst = dst;
  words.scatter_dst = scatter_dst;
  if (args.fp8) {
    const dim3 grid(DivUp(args.num_tokens, kWavesPerGroup * kAppendRows), args.num_layers);
    hipLaunchKernelGGL(AppendFp8Kernel<StepWords>, grid, dim3(kThreads), 0, stream, args, words);
  } else {
    const dim3 grid(DivUp(args.num_tokens, kWavesPerGroup * kAppendRowsBf16), args.num_layers);
    hipLaunchKernelGGL(AppendBf16Kernel<StepWords>, grid, dim3(kThreads), 0, stream, args, words);
  }
  return hipGetLastError();
}

hipError_t LaunchNormRopeAppend(const NormRopeAppendArgs& args, hipStream_t stream) {
  if (args.append.num_tokens <= 0) return hipSuccess;
  NormRopeAppendArgs launch = args;
  launch.items_per_token = 1 + (args.q_rope != nullptr ? DivUp(args.num_heads, kQueryHeadsPerItem) : 0);
  constexpr int kRowsAlone = 2;  // rows per wavefront when there are no query heads
  const int rows = launch.items_per_token == 1 ? kRowsAlone : 1;
  const int64_t items = static_cast<int64_t>(DivUp(args.append.num_tokens, rows)) * launch.items_per_token;
  if (items > 0x7fffffff - kWavesPerGroup) return hipErrorInvalidValue;  // the kernel indexes work items in 32 bits
  const dim3 grid(DivUp(static_cast<int>(items), kWavesPerGroup));
  if (args.append.fp8) {
    if (rows == 1) hipLaunchKernelGGL((NormRopeAppendKernel<true, 1>), grid, dim3(kThreads), 0, stream, launch);
    else hipLaunchKernelGGL((NormRopeAppendKernel<true, kRowsAlone>), grid, dim3(kThreads), 0, stream, launch);
  } else {
    if (rows == 1) hipLaunchKernelGGL((NormRopeAppendKernel<false, 1>), grid, dim3(kThreads), 0, stream, launch);
    else hipLaunchKernelGGL((NormRopeAppendKernel<false, kRowsAlone>), grid, dim3(kThreads), 0, stream, launch);
  }
  return hipGetLastError();
}

namespace {
// The plain launch, or the one that stamps the dispatch's own start and end into two events.
template <typename Kernel, typename... Args>
void LaunchMaybeTimed(Kernel kernel, const dim3& grid, const dim3& block, unsigned lds_bytes, hipStream_t stream, hipEvent_t start,
                      hipEvent_t stop, Args... args) {
  if (start != nullptr && stop != nullptr) {
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, start, stop, 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args...);
  }
}
}  // namespace

hipError_t LaunchGather(const GatherArgs& args, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
  if (args.batch <= 0 || args.num_layers <= 0 || args.max_seq_len <= 0) return hipSuccess;
  const int blocks = DivUp(args.max_seq_len, args.block_size);
  if (!args.fp8 && args.block_size % kGatherTileRows == 0) {
    const int per_block = args.block_size / kGatherTileRows;
    const dim3 tile_grid(blocks * per_block, args.batch, args.num_layers);
    LaunchMaybeTimed(GatherBf16TileKernel<kGatherTileRows>, tile_grid, dim3(kThreads), kGatherLdsReserve, stream, start, stop, args,
                     per_block);
    return hipGetLastError();
  }
  // Two-row items measured fastest for the generic kernels as well (more, shorter waves).
  const int rows_per_item = RowsPerItem(args.block_size, args.fp8 ? 4 : 2);
  const int items_per_block = args.block_size / rows_per_item;
  const dim3 grid(DivUp(blocks * items_per_block, kWavesPerGroup), args.batch, args.num_layers);
  if (args.fp8) {
    LaunchMaybeTimed(GatherFp8Kernel, grid, dim3(kThreads), 0, stream, start, stop, args, rows_per_item);
  } else {
    LaunchMaybeTimed(GatherBf16Kernel, grid, dim3(kThreads), 0, stream, start, stop, args, rows_per_item);
  }
  return hipGetLastError();
}

hipError_t LaunchStoreWords(const int32_t* host_words, int count, int32_t* dst, hipStream_t stream) {
  return LaunchStoreWords(host_words, count, dst, nullptr, 0, nullptr, stream);
}

hipError_t LaunchStoreWords(const int32_t* host_words, int count, int32_t* dst, const int32_t* host_pairs, int pairs,
                            int32_t* scatter_dst, hipStream_t stream) {
  if (count <= 0 && pairs <= 0) return hipSuccess;
  if (count < 0 || pairs < 0 || count + 2 * pairs > kMaxStoreWords) return hipErrorInvalidValue;
  if ((count > 0 && (host_words == nullptr || dst == nullptr)) || (pairs > 0 && (host_pairs == nullptr || scatter_dst == nullptr))) {
    return hipErrorInvalidValue;
  }
  StoreWordsArgs args;
  for (int i = 0; i < count; ++i) args.words[i] = host_words[i];
  for (int i = 0; i < 2 * pairs; ++i) args.words[count + i] = host_pairs[i];
  hipLaunchKernelGGL(StoreWordsKernel, dim3(1), dim3(kThreads), 0, stream, args, count, dst, pairs, scatter_dst);
  return hipGetLastError();
}

hipError_t LaunchCopyBlocks(const CopyBlocksArgs& args, hipStream_t stream) {
  if (args.num_moves <= 0 || args.num_layers <= 0) return hipSuccess;
  // Two-row items: measured 6.0 TB/s against 5.4 TB/s with 16-row items (1196 blocks x 8 layers).
  const int rows_per_item = RowsPerItem(args.block_size, 2);
  const int items_per_block = args.block_size / rows_per_item;
  const dim3 grid(DivUp(args.num_moves * items_per_block, kWavesPerGroup), args.num_layers);
  if (args.latent_row_bytes == kLatentDim * 2 && args.rope_row_bytes == kRopeDim * 2) {
    hipLaunchKernelGGL((CopyBlocksKernel<64, 8>), grid, dim3(kThreads), 0, stream, args, rows_per_item);
  } else if (args.latent_row_bytes == kLatentDim && args.rope_row_bytes == kRopeDim) {
    hipLaunchKernelGGL((CopyBlocksKernel<32, 4>), grid, dim3(kThreads), 0, stream, args, rows_per_item);
  } else {
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t PreparePagedCopyKernels() {
  static std::mutex guard;
  static PerDeviceOnce once;
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 0 || device >= PerDeviceOnce::kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(guard);
  if (once.state[device] == 1) return hipSuccess;
  const void* kernels[] = {
      reinterpret_cast<const void*>(&AppendBf16Kernel<NoStepWords>), reinterpret_cast<const void*>(&AppendBf16Kernel<StepWords>),
      reinterpret_cast<const void*>(&AppendFp8Kernel<NoStepWords>),  reinterpret_cast<const void*>(&AppendFp8Kernel<StepWords>),
      reinterpret_cast<const void*>(&GatherBf16TileKernel<kGatherTileRows>), reinterpret_cast<const void*>(&GatherBf16Kernel),
      reinterpret_cast<const void*>(&GatherFp8Kernel), reinterpret_cast<const void*>(&CopyBlocksKernel<64, 8>),
      reinterpret_cast<const void*>(&CopyBlocksKernel<32, 4>), reinterpret_cast<const void*>(&StoreWordsKernel)};
  for (const void* kernel : kernels) {
    hipFuncAttributes attributes;
    if (hipError_t e = hipFuncGetAttributes(&attributes, kernel); e != hipSuccess) return e;
  }
  once.state[device] = 1;
  return hipSuccess;
}

}  // namespace mlakv
