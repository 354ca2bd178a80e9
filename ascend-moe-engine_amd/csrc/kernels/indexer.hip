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
#include "kernels.h"

namespace mlakv {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kIndexDim = 128;
static_assert(kIndexDim == 4 * 32, "four lane groups of 32 elements cover an index key");
constexpr int kScoreThreads = 256;
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

// Address pieces of cached token `token` of sequence `seq` (clamped into the sequence).
__device__ __forceinline__ void LocateToken(const IndexerArgs& a, const int32_t* table_row, int token, int seq_len, int* block,
                                            int* slot) {
  const int clamped = token < seq_len ? token : seq_len - 1;
  const int logical = clamped / a.block_size;
  const int entry = table_row[logical];
  *block = static_cast<unsigned>(entry) < static_cast<unsigned>(a.num_blocks) ? entry : 0;
  *slot = clamped - logical * a.block_size;
}

// One wavefront scores 64 consecutive tokens in four groups of 16: A = keys (16 tokens x 32
// elements per MFMA, converted to bf16), B = query (32 elements x 16 heads), four k-steps and HB head blocks. Lane
// (r = lane % 16, g = lane / 16) holds elements [32g, 32g + 32) of token r (A) and of head r (B); a
// k-step takes eight of them from both, so the element order inside the dot product is the same
// on both sides.
template <int HB>
__global__ __launch_bounds__(kScoreThreads) void IndexerScoreKernel(IndexerArgs a) {
  const int seq = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int seq_len = min(a.seq_lens[seq], a.max_seq_len);
  const int token0 = blockIdx.x * kTokensPerGroup + wave * kTokensPerWave;
  if (seq_len <= a.sparse_count || token0 >= seq_len) return;  // short sequences select everything without scores
  const int32_t* table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;

  bf16x8 q[HB][4];
  float w[HB];
#pragma unroll
  for (int hb = 0; hb < HB; ++hb) {
    const int head = 16 * hb + r;
    const char* src = a.query + seq * a.query_seq_stride + head * a.query_head_stride + 32 * g;
    const u32x4 lo = *reinterpret_cast<const u32x4*>(src), hi = *reinterpret_cast<const u32x4*>(src + 16);
    q[hb][0] = CodesToBf16(lo.x, lo.y);
    q[hb][1] = CodesToBf16(lo.z, lo.w);
    q[hb][2] = CodesToBf16(hi.x, hi.y);
    q[hb][3] = CodesToBf16(hi.z, hi.w);
    const unsigned short weight = *reinterpret_cast<const unsigned short*>(a.weights + seq * a.weights_seq_stride + head * 2);
    w[hb] = Bf16BitsToF32(weight) * a.query_scale[seq * a.query_scale_seq_stride + head];
  }

  u32x4 k_lo[4], k_hi[4];
  float k_scale[4];  // of token 16 rg + r, fetched with its key so that no load depends on the MFMA results
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
    int block, slot;
    LocateToken(a, table_row, token0 + 16 * rg + r, seq_len, &block, &slot);
    const char* src = a.key_base + block * a.key_block_stride + slot * a.key_row_stride + 32 * g;
    k_lo[rg] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
    k_hi[rg] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + 16));
    k_scale[rg] = a.key_scale_base[block * a.key_scale_block_stride + slot];
  }
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
    const bf16x8 k[4] = {CodesToBf16(k_lo[rg].x, k_lo[rg].y), CodesToBf16(k_lo[rg].z, k_lo[rg].w),
                         CodesToBf16(k_hi[rg].x, k_hi[rg].y), CodesToBf16(k_hi[rg].z, k_hi[rg].w)};
    // lane (r, g) ends up with sum over its head column of w * relu(q . k) for tokens 4g + j
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k[s], q[hb][s], acc, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; ++j) sum[j] = __builtin_fmaf(fmaxf(acc[j], 0.0f), w[hb], sum[j]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int offset = 1; offset < 16; offset <<= 1) sum[j] += __shfl_xor(sum[j], offset);
    }
    // lanes r < 4 of each group finish token 4g + r, whose scale lane 4g + r holds
    const int token = token0 + 16 * rg + 4 * g + r;
    const float scale = __shfl(k_scale[rg], (4 * g + r) & 15);
    if (r < 4 && token < seq_len) {
      const float mine = r == 0 ? sum[0] : r == 1 ? sum[1] : r == 2 ? sum[2] : sum[3];
      a.keys[seq * a.keys_stride + token] = static_cast<unsigned short>(ScoreKey(mine * scale));
    }
  }
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
    int suffix = mine;  // inclusive sum over this lane and the lanes above it
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const int higher = __shfl_down(suffix, offset);
      if (tid + offset < 64) suffix += higher;
    }
    int above = suffix - mine;
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
  __shared__ int histogram[256];
  __shared__ int found[2];
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
#pragma unroll
  for (int shift = 8; shift >= 0; shift -= 8) {
    for (int i = tid; i < 256; i += kSelectThreads) histogram[i] = 0;
    __syncthreads();
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
    __syncthreads();
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
    int inclusive = packed;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const int below = __shfl_up(inclusive, offset);
      if (lane >= offset) inclusive += below;
    }
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

}  // namespace

hipError_t LaunchIndexer(const IndexerArgs& args, hipStream_t stream) {
  if (args.batch <= 0) return hipSuccess;
  const int groups = (args.max_seq_len + kTokensPerGroup - 1) / kTokensPerGroup;
  if (args.max_seq_len > args.sparse_count) {
    const dim3 grid(groups, args.batch);
    switch (args.heads / 16) {
      case 1: hipLaunchKernelGGL(IndexerScoreKernel<1>, grid, dim3(kScoreThreads), 0, stream, args); break;
      case 2: hipLaunchKernelGGL(IndexerScoreKernel<2>, grid, dim3(kScoreThreads), 0, stream, args); break;
      case 3: hipLaunchKernelGGL(IndexerScoreKernel<3>, grid, dim3(kScoreThreads), 0, stream, args); break;
      case 4: hipLaunchKernelGGL(IndexerScoreKernel<4>, grid, dim3(kScoreThreads), 0, stream, args); break;
      default: return hipErrorInvalidValue;
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(IndexerSelectKernel, dim3(args.batch), dim3(kSelectThreads), 0, stream, args);
  return hipGetLastError();
}

}  // namespace mlakv
