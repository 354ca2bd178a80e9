// Absorbed-MLA decode attention over the paged latent KV cache, gfx950 (CDNA4).
//
//   s_i = scale * (q_lat[h] . c_i + q_rope[h] . r_i),  p = softmax_i(s),  o[h] = sum_i p_i c_i
//
// One query token per sequence, all heads share one latent KV stream (MQA), so the
// head axis is the free MFMA dimension and the latent row is read from HBM once and used
// as both K (with the 64 rope columns appended) and V.
//
// Work decomposition
//   workgroup = (kv chunk, sequence, group of 64 heads); 4 wavefronts, 16 heads each.
//   A chunk is `chunk_tiles` tiles of 64 tokens. Tiles are staged in LDS (two buffers of
//   64 x 1152 B) through registers, one tile ahead of the math.
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
//
// LDS layout: row pitch 1152 B (72 chunks of 16 B), chunk index XORed with
//   f(token & 7) = ((t & 3) << 1) | (t >> 2): eight consecutive tokens hit eight distinct
//   16-byte bank groups for the K reads and four consecutive tokens hit four distinct
//   32-byte groups for the transposed V reads.
//
// Chunks of one sequence are merged by a second small kernel from fp32 partials
// (normalised O and log2-domain LSE) held in the caller's workspace.
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
constexpr int kRowBytes = (kLatentDim + kRopeDim) * 2;  // 1152
constexpr int kTileBytes = kTileTokens * kRowBytes;     // 73728
constexpr int kKSteps = (kLatentDim + kRopeDim) / 32;   // 18
constexpr int kDvTiles = kLatentDim / 16;               // 32
constexpr int kLdsBytes = 2 * kTileBytes;

__device__ __forceinline__ int Uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int Swizzle(int token) {
  const int t = token & 7;
  return ((t & 3) << 1) | (t >> 2);
}
__device__ __forceinline__ int LdsOffset(int token, int chunk) { return token * kRowBytes + ((chunk ^ Swizzle(token)) << 4); }

__device__ __forceinline__ u32x4 GlobalLoad16(const char* p) { return *reinterpret_cast<const u32x4*>(p); }

struct Locator {
  const int32_t* table_row;
  int block_size;
  int block_shift;  // log2(block_size) or -1
  int num_blocks;
  // Physical block and in-block slot of token position `pos`; false when the table entry is
  // outside the pool (such a row is read as zeros rather than faulting).
  __device__ __forceinline__ bool operator()(int pos, int* block, int* slot) const {
    int logical;
    if (block_shift >= 0) {
      logical = pos >> block_shift;
      *slot = pos & (block_size - 1);
    } else {
      logical = pos / block_size;
      *slot = pos - logical * block_size;
    }
    *block = table_row[logical];
    return static_cast<unsigned>(*block) < static_cast<unsigned>(num_blocks);
  }
};

// ---- tile staging: global -> registers -> LDS -------------------------------------

// bf16 rows: 16 latent chunks + 2 rope chunks of 16 B per thread.
struct TileRegsBf16 {
  u32x4 v[18];
};

__device__ __forceinline__ void LoadTile(TileRegsBf16& r, const AttnArgs& a, const Locator& locate, int tile, int seq_len,
                                         int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  const int pos0 = tile * kTileTokens;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int token = wave + 4 * i;  // wave-uniform
    const int pos = pos0 + token;
    u32x4 v = {0u, 0u, 0u, 0u};
    int block, slot;
    if (pos < seq_len && locate(pos, &block, &slot)) {
      block = Uniform(block);
      v = GlobalLoad16(a.latent.base + block * a.latent.block_stride + slot * a.latent.row_stride + lane * 16);
    }
    r.v[i] = v;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + kThreads * i;
    const int token = idx >> 3, chunk = idx & 7;
    const int pos = pos0 + token;
    u32x4 v = {0u, 0u, 0u, 0u};
    int block, slot;
    if (pos < seq_len && locate(pos, &block, &slot)) {
      v = GlobalLoad16(a.rope.base + block * a.rope.block_stride + slot * a.rope.row_stride + chunk * 16);
    }
    r.v[16 + i] = v;
  }
}

__device__ __forceinline__ void StoreTile(const TileRegsBf16& r, unsigned char* buf, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int token = wave + 4 * i;
    *reinterpret_cast<u32x4*>(buf + LdsOffset(token, lane)) = r.v[i];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + kThreads * i;
    const int token = idx >> 3, chunk = 64 + (idx & 7);
    *reinterpret_cast<u32x4*>(buf + LdsOffset(token, chunk)) = r.v[16 + i];
  }
}

// FP8 rows: 8 latent chunks + 1 rope chunk of 16 codes per thread, and their row scales.
struct TileRegsFp8 {
  u32x4 v[9];
  float scale[9];
};

__device__ __forceinline__ void LoadTile(TileRegsFp8& r, const AttnArgs& a, const Locator& locate, int tile, int seq_len,
                                         int tid) {
  const int pos0 = tile * kTileTokens;
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    int token, chunk;
    const char* base;
    int64_t block_stride, row_stride;
    if (i < 8) {
      const int idx = tid + kThreads * i;
      token = idx >> 5;
      chunk = idx & 31;
      base = a.latent.base;
      block_stride = a.latent.block_stride;
      row_stride = a.latent.row_stride;
    } else {
      token = tid >> 2;
      chunk = tid & 3;
      base = a.rope.base;
      block_stride = a.rope.block_stride;
      row_stride = a.rope.row_stride;
    }
    const int pos = pos0 + token;
    u32x4 v = {0u, 0u, 0u, 0u};
    float scale = 0.0f;
    int block, slot;
    if (pos < seq_len && locate(pos, &block, &slot)) {
      v = GlobalLoad16(base + block * block_stride + slot * row_stride + chunk * 16);
      scale = reinterpret_cast<const float*>(a.scale.base + block * a.scale.block_stride)[slot];
    }
    r.v[i] = v;
    r.scale[i] = scale;
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

__device__ __forceinline__ void StoreTile(const TileRegsFp8& r, unsigned char* buf, int tid) {
#pragma unroll
  for (int i = 0; i < 9; ++i) {
    int token, chunk;  // chunk: index of the first of two 16-byte bf16 chunks
    if (i < 8) {
      const int idx = tid + kThreads * i;
      token = idx >> 5;
      chunk = 2 * (idx & 31);
    } else {
      token = tid >> 2;
      chunk = 64 + 2 * (tid & 3);
    }
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
    *reinterpret_cast<u32x4*>(buf + LdsOffset(token, chunk)) = first;
    *reinterpret_cast<u32x4*>(buf + LdsOffset(token, chunk + 1)) = second;
  }
}

template <bool FP8>
struct TileRegsFor {
  using type = TileRegsBf16;
};
template <>
struct TileRegsFor<true> {
  using type = TileRegsFp8;
};

// ---- main kernel -------------------------------------------------------------------

template <bool FP8>
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

  Locator locate;
  locate.table_row = a.block_table + static_cast<int64_t>(seq) * a.table_stride;
  locate.block_size = a.block_size;
  locate.block_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
  locate.num_blocks = a.num_blocks;

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
  float m_run = -__builtin_inff();  // running max, log2 domain (scores * scale * log2 e)
  float l_run = 0.0f;               // this lane's share of the running denominator

  // Lane-constant LDS offsets.
  const int swk = Swizzle(i16);                  // K reads: token = 16t + i16
  const int k_lane = i16 * kRowBytes;
  const int k_e0 = ((g ^ swk) << 4), k_e1 = (((4 + g) ^ swk) << 4);
  const int v_row = 4 * g + (i16 >> 2);          // V reads: token = 32u + (16) + 4g + i16/4
  const int swv = Swizzle(v_row);
  const int v_c1 = (i16 & 3) >> 1;
  const int v_lane = v_row * kRowBytes + (i16 & 1) * 8;
  int v_e[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v_e[j] = (((2 * j + v_c1) ^ swv) << 4);

  typename TileRegsFor<FP8>::type regs;
  LoadTile(regs, a, locate, tile_begin, seq_len, tid);
  StoreTile(regs, lds, tid);
  if (tile_begin + 1 < tile_end) LoadTile(regs, a, locate, tile_begin + 1, seq_len, tid);
  __syncthreads();

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    unsigned char* cur = lds + ((tile - tile_begin) & 1) * kTileBytes;
    unsigned char* nxt = lds + (((tile - tile_begin) & 1) ^ 1) * kTileBytes;

    f32x4 s[4];
    if (active) {
#pragma unroll
      for (int t = 0; t < 4; ++t) s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        const int e = (ks & 1) ? k_e1 : k_e0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(cur + k_lane + t * 16 * kRowBytes + (ks >> 1) * 128 + e);
          s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, q[ks], s[t], 0, 0, 0);
        }
      }
    }

    // Stage the next tile while the scores are reduced. Its buffer was last read before the
    // barrier that ended the previous iteration.
    if (tile + 1 < tile_end) {
      StoreTile(regs, nxt, tid);
      if (tile + 2 < tile_end) LoadTile(regs, a, locate, tile + 2, seq_len, tid);
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
      const float m_new = fmaxf(m_run, tile_max);  // finite: token 0 of the tile is valid
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float row_sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p = __builtin_amdgcn_exp2f(s[t][j] - m_new);
          s[t][j] = p;
          row_sum += p;
        }
      }
      l_run = l_run * alpha + row_sum;
      m_run = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int n = 0; n < kDvTiles; ++n) o[n] *= alpha;
      }

      // ---- O^T += V^T P ----
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        bf16x8 p;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          p[j] = static_cast<__bf16>(s[2 * u][j]);
          p[4 + j] = static_cast<__bf16>(s[2 * u + 1][j]);
        }
        const unsigned char* vbase = cur + v_lane + u * 32 * kRowBytes;
#pragma unroll
        for (int n = 0; n < kDvTiles; ++n) {
          const unsigned char* addr = vbase + (n >> 2) * 128 + v_e[n & 3];
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4*)(addr));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4*)(addr + 16 * kRowBytes));
          const bf16x4 lo_b = __builtin_bit_cast(bf16x4, lo);
          const bf16x4 hi_b = __builtin_bit_cast(bf16x4, hi);
          const bf16x8 vf = __builtin_shufflevector(lo_b, hi_b, 0, 1, 2, 3, 4, 5, 6, 7);
          o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p, o[n], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  if (!active) return;
  float l_total = l_run + __shfl_xor(l_run, 16);
  l_total += __shfl_xor(l_total, 32);
  const float inv = 1.0f / l_total;
  const float lse2 = m_run + __builtin_amdgcn_logf(l_total);  // v_log_f32 is log2
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

}  // namespace

hipError_t PrepareAttnKernels() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaDecodeKernel<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&MlaDecodeKernel<true>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
}

hipError_t LaunchAttnDecode(const AttnArgs& args, hipStream_t stream) {
  if (args.batch <= 0) return hipSuccess;
  const dim3 grid(args.max_chunks, args.batch, (args.heads + 63) / 64);
  if (args.fp8) {
    hipLaunchKernelGGL(MlaDecodeKernel<true>, grid, dim3(kThreads), kLdsBytes, stream, args);
  } else {
    hipLaunchKernelGGL(MlaDecodeKernel<false>, grid, dim3(kThreads), kLdsBytes, stream, args);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (args.max_chunks > 1) {
    hipLaunchKernelGGL(MlaCombineKernel, dim3(args.heads, args.batch), dim3(128), 0, stream, args);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace mlakv
