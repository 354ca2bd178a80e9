// Lightning Indexer for one decode token per sequence: scores of every cached token from FP8
// index keys in a paged pool, then the top-k token positions (the operator behind
// aclnnQuantLightningIndexer, reference include/moe/core/op_table.hpp:964-1006; arithmetic order of
// the vendored kernel, third_party/ops_transformer/attention/quant_lightning_indexer/op_kernel/
// arch35/vf/quant_lightning_indexer_vector1.h:288-330, selection rule of arch35/
// quant_lightning_indexer_service_vector.h:446-541).
//
//   score[t] = key_scale[t] * sum_h (W[h] * query_scale[h]) * ReLU(q_h . k_t)      -> bf16, ties away
//   out      = positions of the sparse_count largest scores (ties: lower position first)
//
// Two kernels: the scores as order-preserving 16-bit keys into a workspace (HBM-bound: 132 bytes
// read per cached token), then one workgroup per sequence selects by two 8-bit histograms and an
// ordered compaction. The 64 x 128 x tokens products run on the bf16 MFMA after an exact
// E4M3 -> bf16 conversion: the FP8 MFMA of this part does not keep full fp32 precision while it
// accumulates (scores came out about 1e-4 off, enough to move 3 % of the bf16 keys by one step),
// and both forms take 16 cycles for 32 elements.
#include <mutex>

#include "kernels.h"

// (the direct global -> LDS loads name M0, which they set themselves, in their clobber lists)
#pragma clang diagnostic ignored "-Winline-asm"

namespace mlakv {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int kIndexDim = 128;
static_assert(kIndexDim == 4 * 32, "four lane groups of 32 elements cover an index key");
constexpr int kScoreThreads = 512;
constexpr int kTokensPerWave = 64;
constexpr int kTokensPerGroup = (kScoreThreads / 64) * kTokensPerWave;

__device__ __forceinline__ float Bf16BitsToF32(unsigned bits) { return __builtin_bit_cast(float, bits << 16); }

// Eight E4M3 codes (two dwords) -> eight bf16, exactly (every E4M3 value is a bf16 value).
__device__ __forceinline__ bf16x8 CodesToBf16(unsigned lo, unsigned hi) {
  const bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
  const bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
  const bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
  const bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
  return bf16x8{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
}

// fp32 -> bf16 with ties away from zero, then the order-preserving key: NaN lowest, negative values
// inverted, the others with the sign bit set.
__device__ __forceinline__ unsigned ScoreKey(float score) {
  const unsigned bits = __builtin_bit_cast(unsigned, score);
  unsigned b = (bits & 0x7fffffffu) > 0x7f800000u ? 0x7fc0u : ((bits + 0x8000u) >> 16);
  if (b == 0x7fc0u) return 0u;
  return (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
}

// Address pieces of cached token `token` of a sequence, clamped to the last position `limit - 1`
// that the table row can address. The limit does not depend on the sequence length, so the
// lookup need not wait for it; a token past the end of its sequence resolves to some readable
// row whose score is never written.
__device__ __forceinline__ void LocateToken(const IndexerArgs& a, const int32_t* table_row, int token, int limit, int* block,
                                            int* slot) {
  const int clamped = token < limit ? token : limit - 1;
  const int logical = clamped / a.block_size;
  const int entry = table_row[logical];
  *block = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : 0;
  *slot = clamped - logical * a.block_size;
}

// Sum over the four lanes {r, r + 16, r + 32, r + 48}, left in all of them.
__device__ __forceinline__ float SumAcrossGroups(float x) {
  unsigned bits = __builtin_bit_cast(unsigned, x);
  u32x2 swapped = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  const float s = __builtin_bit_cast(float, static_cast<unsigned>(swapped.x)) + __builtin_bit_cast(float, static_cast<unsigned>(swapped.y));
  bits = __builtin_bit_cast(unsigned, s);
  swapped = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  return __builtin_bit_cast(float, static_cast<unsigned>(swapped.x)) + __builtin_bit_cast(float, static_cast<unsigned>(swapped.y));
}

// Direct global->LDS load: lane L's 16 bytes land at lds_wave_base + 16 * L (the LDS base travels
// in M0 and is wave-uniform). Issued from inline assembly, so the kernel waits for it itself.
__device__ __forceinline__ void DirectLoad16PerLane(const char* lane_pointer, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(lane_pointer), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
               : "memory", "m0");
}

// Rows of 128 bytes (an index key, or the 128 query codes of a head) sit in LDS as eight 16-byte
// pieces, piece c of row t at position c ^ Swizzle(t): the sixteen rows that the lanes of an MFMA
// operand read together then fall into sixteen different bank groups.
__device__ __forceinline__ int Swizzle(int row) { return (row >> 1) & 7; }

// One wavefront scores 64 consecutive tokens in four groups of 16: A = query (16 heads x 32
// elements per MFMA), B = keys (32 elements x 16 tokens), both converted to bf16 exactly; four
// k-steps and HB head blocks. Lane (r = lane % 16, g = lane / 16) holds elements [32g, 32g + 32)
// of head r (A) and of token r (B); a k-step takes eight of them from both, so the element order
// inside the dot product is the same on both sides. The product leaves heads 4g .. 4g + 3 of
// token r in lane (r, g): the weighted sum over the heads is a few additions inside the lane and
// two lane exchanges, and lane (r, g) ends up writing the key of token 16g + r: one 128-byte
// store per wavefront.
// A lane that fetched its operand rows itself would touch sixteen different 128-byte lines per
// quarter-wave (measured: 4.9 M cache accesses for 35 MB, the L1's lookup rate was the bound),
// so keys and query come in through LDS instead: every load instruction moves eight whole rows
// (1 KB, consecutive lanes fetch consecutive pieces), and the operand reads are LDS reads. A
// wavefront reads only the keys it fetched itself; the query is shared by the workgroup.
template <int HB>
__global__ __launch_bounds__(kScoreThreads) void IndexerScoreKernel(IndexerArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
  constexpr int kQueryBytes = HB * 16 * kIndexDim * 2;  // the query as bf16: converted once per workgroup, not once per wavefront
  const int seq = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int group0 = blockIdx.x * kTokensPerGroup;
  const int token0 = group0 + wave * kTokensPerWave;
  if (group0 >= a.max_seq_len) return;
  const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;
  // Rounds of loads, each behind the one it depends on and nothing else: the sequence length, the
  // table entries, the query and the weights together; then the keys; the scores leave last.
  const int raw_len = a.seq_lens[seq];
  const int limit = a.max_seq_len;  // the caller's table rows address at least this many positions (checked on the host)

  // Query codes: HB * 16 rows of 128, eight rows per wavefront (16 codes per lane) for the first
  // 2 HB wavefronts; they go to LDS as bf16 further down, with the rest of this round of loads.
  static_assert(2 * HB <= kScoreThreads / 64, "one load of query codes per wavefront at most");
  const bool converts_query = wave < 2 * HB;
  const int query_head = 8 * wave + (lane >> 3);
  u32x4 query_codes = {0u, 0u, 0u, 0u};
  if (converts_query) {
    query_codes = *reinterpret_cast<const u32x4*>(a.query + seq * a.query_seq_stride + query_head * a.query_head_stride + (lane & 7) * 16);
  }
  // wave-uniform: whether the weight and scale rows of every sequence start on 8 and 16 bytes
  const bool rows_aligned = ((reinterpret_cast<uintptr_t>(a.weights) | static_cast<uintptr_t>(a.weights_seq_stride)) & 7) == 0 &&
                            ((reinterpret_cast<uintptr_t>(a.query_scale) | static_cast<uintptr_t>(a.query_scale_seq_stride) * 4) & 15) == 0;
  // Head weights and query scales of heads 16 hb + 4 g + j, the rows this lane holds of every
  // product: four consecutive heads are 8 bytes of weights and 16 bytes of scales. All of them are
  // asked for here, with the query and the table entries, and turned into w[][] only below, once
  // everything of this round has been asked for: used one block at a time they cost a memory
  // latency per block of heads before the first key was asked for.
  float w[HB][4];
  u32x2 weight_pairs[HB];
  f32x4 scale_fours[HB];
  if (rows_aligned) {
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      weight_pairs[hb] = *reinterpret_cast<const u32x2*>(a.weights + seq * a.weights_seq_stride + (16 * hb + 4 * g) * 2);
      scale_fours[hb] = *reinterpret_cast<const f32x4*>(a.query_scale + seq * a.query_scale_seq_stride + 16 * hb + 4 * g);
    }
  } else {
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      const unsigned short* weights = reinterpret_cast<const unsigned short*>(a.weights + seq * a.weights_seq_stride + (16 * hb + 4 * g) * 2);
      const float* scales = a.query_scale + seq * a.query_scale_seq_stride + 16 * hb + 4 * g;
      weight_pairs[hb] = u32x2{static_cast<unsigned>(weights[0]) | (static_cast<unsigned>(weights[1]) << 16),
                               static_cast<unsigned>(weights[2]) | (static_cast<unsigned>(weights[3]) << 16)};
      scale_fours[hb] = f32x4{scales[0], scales[1], scales[2], scales[3]};
    }
  }

  // Where this wave's tokens live: lane L needs token L / 8 + 8 i for load i and token L for its
  // scale. With blocks of at least 64 tokens the 64 tokens span at most two table entries.
  const bool wave_in_range = token0 < limit;
  const bool two_entries = a.block_size >= kTokensPerWave && token0 + kTokensPerWave <= limit;
  int logical0 = 0, slot0 = 0, entry0 = 0, entry1 = 0;
  if (two_entries) {
    logical0 = token0 / a.block_size;
    slot0 = token0 - logical0 * a.block_size;
    entry0 = table_row[logical0];
    entry1 = table_row[min(logical0 + 1, a.table_stride - 1)];
    entry0 = static_cast<unsigned>(entry0) < static_cast<unsigned>(a.num_blocks) ? entry0 : 0;
    entry1 = static_cast<unsigned>(entry1) < static_cast<unsigned>(a.num_blocks) ? entry1 : 0;
  }
  const auto locate = [&](int offset, int* block, int* slot) __attribute__((always_inline)) {
    if (two_entries) {
      const int at = slot0 + offset;
      const bool next = at >= a.block_size;
      *block = next ? entry1 : entry0;
      *slot = next ? at - a.block_size : at;
    } else {
      LocateToken(a, table_row, token0 + offset, limit, block, slot);
    }
  };

#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    w[hb][0] = Bf16BitsToF32(weight_pairs[hb].x & 0xffffu) * scale_fours[hb][0];
    w[hb][1] = Bf16BitsToF32(weight_pairs[hb].x >> 16) * scale_fours[hb][1];
    w[hb][2] = Bf16BitsToF32(weight_pairs[hb].y & 0xffffu) * scale_fours[hb][2];
    w[hb][3] = Bf16BitsToF32(weight_pairs[hb].y >> 16) * scale_fours[hb][3];
  }
  // The query as bf16, 256 bytes per head, 16-byte piece p of head h at position p ^ (h % 16): the
  // sixteen heads that the lanes of an MFMA operand read together fall into sixteen bank groups.
  if (converts_query) {
    unsigned char* row = lds + query_head * (kIndexDim * 2);
    const int piece = 2 * (lane & 7), turn = query_head & 15;
    *reinterpret_cast<bf16x8*>(row + ((piece ^ turn) << 4)) = CodesToBf16(query_codes.x, query_codes.y);
    *reinterpret_cast<bf16x8*>(row + (((piece + 1) ^ turn) << 4)) = CodesToBf16(query_codes.z, query_codes.w);
  }
  const int seq_len = min(raw_len, a.max_seq_len);
  if (seq_len <= a.sparse_count || group0 >= seq_len) {  // the whole workgroup; short sequences select everything without scores
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS that is no longer this workgroup's
    return;
  }

  const unsigned key_lds = lds_base + kQueryBytes + wave * (kTokensPerWave * kIndexDim);
  float my_scale = 0.0f;  // of token token0 + lane
  if (wave_in_range && token0 < seq_len) {
    if (two_entries && slot0 + kTokensPerWave <= a.block_size) {
      // the usual case, all 64 tokens in one block: one address, a constant step between the loads
      const char* src = a.key_base + entry0 * a.key_block_stride + (slot0 + (lane >> 3)) * a.key_row_stride;
      const int64_t step = 8 * a.key_row_stride;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        DirectLoad16PerLane(src + i * step + (((lane & 7) ^ Swizzle(8 * i + (lane >> 3))) << 4), key_lds + i * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int t = 8 * i + (lane >> 3);
        int block, slot;
        locate(t, &block, &slot);
        const char* src = a.key_base + block * a.key_block_stride + slot * a.key_row_stride + (((lane & 7) ^ Swizzle(t)) << 4);
        DirectLoad16PerLane(src, key_lds + i * 1024);
      }
    }
    int block, slot;
    locate(lane, &block, &slot);
    my_scale = a.key_scale_base[block * a.key_scale_block_stride + slot];
  }
  // Loads return in issue order: keys (two loads per group of 16 tokens), then the scale. A group
  // is scored while the later ones are still on their way. A wave past the end of its sequence
  // asked for no keys.
  __syncthreads();  // the query rows the other waves converted
  if (token0 >= seq_len) return;

  const unsigned char* q_lds = lds;
  const unsigned char* k_lds = lds + kQueryBytes + wave * (kTokensPerWave * kIndexDim);
  bf16x8 q[HB][4];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      q[hb][s] = *reinterpret_cast<const bf16x8*>(q_lds + (16 * hb + r) * (kIndexDim * 2) + (((4 * g + s) ^ r) << 4));
    }
  }
  float mine = 0.0f;  // score of token 16 g + r before its key scale
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
    if (rg == 0) asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
    if (rg == 1) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
    if (rg == 2) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    if (rg == 3) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    const int t = 16 * rg + r;
    const u32x4 lo = *reinterpret_cast<const u32x4*>(k_lds + t * kIndexDim + (((2 * g) ^ Swizzle(t)) << 4));
    const u32x4 hi = *reinterpret_cast<const u32x4*>(k_lds + t * kIndexDim + (((2 * g + 1) ^ Swizzle(t)) << 4));
    const bf16x8 k[4] = {CodesToBf16(lo.x, lo.y), CodesToBf16(lo.z, lo.w), CodesToBf16(hi.x, hi.y), CodesToBf16(hi.z, hi.w)};
    float sum[2] = {0.0f, 0.0f};  // heads 4g + {0, 2} and 4g + {1, 3} of every block, token 16 rg + r
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(q[hb][s], k[s], acc, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; ++j) sum[j & 1] = __builtin_fmaf(fmaxf(acc[j], 0.0f), w[hb][j], sum[j & 1]);
    }
    const float total = SumAcrossGroups(sum[0] + sum[1]);  // every lane (r, *) has token 16 rg + r
    if (rg == g) mine = total;
  }
  const int token = token0 + lane;  // = token0 + 16 g + r
  if (token < seq_len) a.keys[seq * a.keys_stride + token] = static_cast<unsigned short>(ScoreKey(mine * my_scale));
}

constexpr int kSelectThreads = 1024;
constexpr int kSelectWaves = kSelectThreads / 64;
constexpr int kKeysPerThread = 8;                              // one 16-byte load
constexpr int kKeysPerPass = kSelectThreads * kKeysPerThread;  // 8192

// kKeysPerThread consecutive keys of a sequence starting at `first` (a multiple of 8; rows are
// 256-byte aligned); keys past the end read as -1, below every real key.
__device__ __forceinline__ void LoadKeys(const unsigned short* keys, int first, int n, int (&out)[kKeysPerThread]) {
#pragma unroll
  for (int part = 0; part < kKeysPerThread / 8; ++part) {
    const int at = first + 8 * part;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (at < n) v = *reinterpret_cast<const u32x4*>(keys + at);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[8 * part + 2 * i] = at + 2 * i < n ? static_cast<int>(v[i] & 0xffffu) : -1;
      out[8 * part + 2 * i + 1] = at + 2 * i + 1 < n ? static_cast<int>(v[i] >> 16) : -1;
    }
  }
}

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS crossbar, no
// wait per step): four shifted adds inside each row of 16 lanes, then lane 15 of rows 0 and 2 onto
// rows 1 and 3, then lane 31 onto the upper half. Lanes a move does not reach add zero.
__device__ __forceinline__ int WaveInclusiveScan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// The byte value that holds the `wanted`-th largest entry of a 256-bin histogram, and the number
// of entries above that bin, found by the first wavefront (four bins per lane, a suffix sum over
// the lanes) and handed to everyone through `result`.
__device__ __forceinline__ void FindBin(const int* histogram, int wanted, int* result, int tid) {
  if (tid < 64) {
    int bins[4], mine = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bins[i] = histogram[4 * tid + i];
      mine += bins[i];
    }
    // the sum over the lanes above this one: everything minus this lane's inclusive prefix
    const int inclusive = WaveInclusiveScan(mine);
    int above = __builtin_amdgcn_readlane(inclusive, 63) - inclusive;
#pragma unroll
    for (int i = 3; i >= 0; --i) {
      if (above < wanted && wanted <= above + bins[i]) {
        result[0] = 4 * tid + i;
        result[1] = above;
      }
      above += bins[i];
    }
  }
}

// One workgroup per sequence. The k-th largest key is found by its high and then its low byte (two
// 256-bin histograms); then an ordered compaction writes the positions above it and the first ones
// equal to it. Thread t holds keys 8t .. 8t+7 of each pass of 8192, so thread order is position
// order. (Measured at 8192 keys: this 7.1 us; 256 threads of 32 keys 10.0 us; sixteen one-bit
// counting rounds 14 us; one atomic per key with a serial bin search 31.6 us.)
__global__ __launch_bounds__(kSelectThreads) void IndexerSelectKernel(IndexerArgs a) {
  __shared__ int histograms[2][256];  // of the high bytes, then of the low bytes among the keys with the high byte found
  __shared__ int founds[2][2];
  __shared__ int wave_counts[kSelectWaves];
  const int seq = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = max(min(a.seq_lens[seq], a.max_seq_len), 0);
  const int k = a.sparse_count;
  int32_t* out = a.indices_out + seq * a.indices_seq_stride;
  if (n <= k) {
    for (int i = tid; i < k; i += kSelectThreads) out[i] = i < n ? i : -1;
    return;
  }
  const unsigned short* keys = a.keys + seq * a.keys_stride;
  const int passes = (n + kKeysPerPass - 1) / kKeysPerPass;
  int first[kKeysPerThread];  // the keys of pass 0 stay in registers; later passes are read again from L2
  LoadKeys(keys, tid * kKeysPerThread, n, first);

  int prefix = 0, wanted = k;  // the bytes of the k-th largest key decided so far; how many of the candidates are wanted
  // both histograms are cleared here and each round has its own result words, so a round is two
  // barriers: the counts complete, the bin found
  if (tid < 512) histograms[tid >> 8][tid & 255] = 0;
  __syncthreads();
#pragma unroll
  for (int shift = 8; shift >= 0; shift -= 8) {
    int* histogram = histograms[shift == 8 ? 0 : 1];
    int* found = founds[shift == 8 ? 0 : 1];
    for (int pass = 0; pass < passes; ++pass) {
      int more[kKeysPerThread];
      if (pass > 0) LoadKeys(keys, pass * kKeysPerPass + tid * kKeysPerThread, n, more);
      const int (&mine)[kKeysPerThread] = pass == 0 ? first : more;
      // Candidates: real keys (shift 8) or keys whose high byte is the one found (shift 0).
      // Scores crowd into a few exponents, so the candidates that share the byte of the thread's
      // first key go in as one addition instead of one each to the same counter.
      const int lead = (mine[0] >> shift) & 255;
      int same = 0;
#pragma unroll
      for (int i = 0; i < kKeysPerThread; ++i) {
        const int key = mine[i];
        const bool candidate = shift == 8 ? key >= 0 : (key >> 8) == prefix;
        const int byte = (key >> shift) & 255;
        if (candidate && byte == lead) {
          ++same;
        } else if (candidate) {
          atomicAdd(&histogram[byte], 1);
        }
      }
      if (same > 0) atomicAdd(&histogram[lead], same);
    }
    __syncthreads();
    FindBin(histogram, wanted, found, tid);
    __syncthreads();
    prefix = shift == 8 ? found[0] : (prefix << 8) | found[0];
    wanted -= found[1];
  }
  const int threshold = prefix, equal_wanted = wanted, greater_total = k - wanted;

  int greater_done = 0, equal_done = 0;
  for (int pass = 0; pass < passes; ++pass) {
    int mine[kKeysPerThread];
    if (pass == 0) {
#pragma unroll
      for (int i = 0; i < kKeysPerThread; ++i) mine[i] = first[i];
    } else {
      LoadKeys(keys, pass * kKeysPerPass + tid * kKeysPerThread, n, mine);
    }
    int greater = 0, equal = 0;
#pragma unroll
    for (int i = 0; i < kKeysPerThread; ++i) {
      greater += mine[i] > threshold ? 1 : 0;
      equal += mine[i] == threshold ? 1 : 0;
    }
    // exclusive prefix over the threads of both counts at once (each below 2^16 per pass)
    const int packed = greater | (equal << 16);
    const int inclusive = WaveInclusiveScan(packed);
    __syncthreads();  // wave_counts of the previous pass have been read
    if (lane == 63) wave_counts[wave] = inclusive;
    __syncthreads();
    int before = inclusive - packed, all = 0;
#pragma unroll
    for (int v = 0; v < kSelectWaves; ++v) {
      const int c = wave_counts[v];
      if (v < wave) before += c;
      all += c;
    }
    int greater_at = greater_done + (before & 0xffff), equal_at = equal_done + (before >> 16);
    const int base = pass * kKeysPerPass + tid * kKeysPerThread;
#pragma unroll
    for (int i = 0; i < kKeysPerThread; ++i) {
      if (mine[i] > threshold) {
        out[greater_at++] = base + i;
      } else if (mine[i] == threshold) {
        if (equal_at < equal_wanted) out[greater_total + equal_at] = base + i;
        ++equal_at;
      }
    }
    greater_done += all & 0xffff;
    equal_done += all >> 16;
  }
}

// Index-key append: sixteen lanes per token (eight bf16 values each), four tokens per wavefront.
// The row's absmax by four lane exchanges, scale = absmax / 448, codes from the correctly rounded
// quotient (the E4M3 conversion saturates behind a clamp to +-448).
__global__ __launch_bounds__(256) void IndexKeyAppendKernel(IndexKeyAppendArgs a) {
  const int lane = threadIdx.x & 63;
  const int token = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);
  const int piece = lane & 15;
  const bool real = token < a.num_tokens;
  const int row = real ? token : a.num_tokens - 1;  // a repeated row is loaded and never stored
  const u32x4 words = *reinterpret_cast<const u32x4*>(a.src + row * a.src_row_stride + piece * 16);
  const int slot = a.slots[row];
  float x[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = Bf16BitsToF32(words[i] & 0xffffu);
    x[2 * i + 1] = Bf16BitsToF32(words[i] >> 16);
  }
  float absmax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) absmax = fmaxf(absmax, fabsf(x[i]));
#pragma unroll
  for (int offset = 1; offset < 16; offset <<= 1) absmax = fmaxf(absmax, __shfl_xor(absmax, offset));
  const float scale = absmax == 0.0f ? 1.0f : absmax / 448.0f;
  u32x2 codes;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = fminf(fmaxf(x[4 * half + i] / scale, -448.0f), 448.0f);
    int word = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
    word = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], word, true);
    codes[half] = static_cast<unsigned>(word);
  }
  if (!real || slot < 0) return;
  const int block = slot / a.block_size;
  if (block >= a.num_blocks) return;
  const int in_block = slot - block * a.block_size;
  *reinterpret_cast<u32x2*>(a.key_base + block * a.key_block_stride + in_block * a.key_row_stride + piece * 8) = codes;
  if (piece == 0) a.key_scale_base[block * a.key_scale_block_stride + in_block] = scale;
}

// Dynamic LDS above 64 KB needs the attribute per kernel and device (PrepareIndexerKernels).
template <int HB>
hipError_t PrepareScore() {
  constexpr int kLdsBytes = HB * 16 * kIndexDim * 2 + kTokensPerGroup * kIndexDim;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&IndexerScoreKernel<HB>), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
}

template <int HB>
hipError_t LaunchScore(const IndexerArgs& args, const dim3& grid, hipStream_t stream) {
  constexpr int kLdsBytes = HB * 16 * kIndexDim * 2 + kTokensPerGroup * kIndexDim;  // the query as bf16 + the key codes of eight waves
  hipLaunchKernelGGL(IndexerScoreKernel<HB>, grid, dim3(kScoreThreads), kLdsBytes, stream, args);
  return hipGetLastError();
}

}  // namespace

hipError_t PrepareIndexerKernels() {
  static std::mutex guard;
  static PerDeviceOnce once;
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 0 || device >= PerDeviceOnce::kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(guard);
  if (once.state[device] == 1) return hipSuccess;
  const hipError_t results[] = {PrepareScore<1>(), PrepareScore<2>(), PrepareScore<3>(), PrepareScore<4>()};
  for (const hipError_t e : results) {
    if (e != hipSuccess) return e;
  }
  for (const void* kernel : {reinterpret_cast<const void*>(&IndexerSelectKernel), reinterpret_cast<const void*>(&IndexKeyAppendKernel)}) {
    hipFuncAttributes attributes;
    if (hipError_t e = hipFuncGetAttributes(&attributes, kernel); e != hipSuccess) return e;
  }
  once.state[device] = 1;
  return hipSuccess;
}

hipError_t LaunchIndexKeyAppend(const IndexKeyAppendArgs& args, hipStream_t stream) {
  if (args.num_tokens <= 0) return hipSuccess;
  hipLaunchKernelGGL(IndexKeyAppendKernel, dim3((args.num_tokens + 15) / 16), dim3(256), 0, stream, args);
  return hipGetLastError();
}

hipError_t LaunchIndexer(const IndexerArgs& args, hipStream_t stream) {
  if (args.batch <= 0) return hipSuccess;
  if (hipError_t e = PrepareIndexerKernels(); e != hipSuccess) return e;
  const int groups = (args.max_seq_len + kTokensPerGroup - 1) / kTokensPerGroup;
  if (args.max_seq_len > args.sparse_count) {
    const dim3 grid(groups, args.batch);
    hipError_t e;
    switch (args.heads / 16) {
      case 1: e = LaunchScore<1>(args, grid, stream); break;
      case 2: e = LaunchScore<2>(args, grid, stream); break;
      case 3: e = LaunchScore<3>(args, grid, stream); break;
      case 4: e = LaunchScore<4>(args, grid, stream); break;
      default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(IndexerSelectKernel, dim3(args.batch), dim3(kSelectThreads), 0, stream, args);
  return hipGetLastError();
}

}  // namespace mlakv
