// Internal launch interface between the C ABI and the gfx950 kernels. Host code fills
// these parameter blocks after validating shapes; the launchers only enqueue.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mlakv {

// Address of row (layer, block, slot) = base + layer*layer_stride + block*block_stride + slot*row_stride.
struct Plane {
  char* base;
  int64_t layer_stride;
  int64_t block_stride;
  int64_t row_stride;
};

// Token rows outside the cache: address = base + layer*layer_stride + row*row_stride.
struct Rows {
  char* base;
  int64_t layer_stride;
  int64_t row_stride;
};

struct AppendArgs {
  Plane latent, rope, scale;  // cache planes, already offset to the first layer of the launch
  Rows latent_src, rope_src;  // bf16 sources
  const int32_t* slots;
  int32_t num_tokens;
  int32_t num_layers;
  int32_t num_blocks;
  int32_t block_size;
  bool fp8;
};

// Fused latent RMSNorm + key RoPE + append of one layer: `append` carries the cache planes
// (already offset to the layer) and the slot mapping; its source fields are unused.
struct NormRopeAppendArgs {
  AppendArgs append;
  const char* kv_a;          // bf16 rows [latent 512 | rope 64]
  int64_t kv_a_row_stride;   // bytes
  const char* gamma;         // bf16 [512]
  float epsilon;
  const char* rope_cos;      // bf16 [positions][64]
  const char* rope_sin;
  int64_t rope_table_row_stride;  // bytes
  const int32_t* positions;
  char* latent_out;          // optional bf16 [tokens][512]
  int64_t latent_out_row_stride;
  char* rope_out;            // optional bf16 [tokens][64]
  int64_t rope_out_row_stride;
  char* q_rope;              // optional bf16 [tokens][heads][64], rotated in place
  int64_t q_rope_token_stride;
  int64_t q_rope_head_stride;
  int num_heads;
  int items_per_token;       // set by the launcher: 1 + groups of eight query heads
};

struct GatherArgs {
  Plane latent, rope, scale;
  Rows latent_dst, rope_dst;  // bf16 destinations
  const int32_t* block_table;
  int32_t table_stride;  // int32 elements per sequence
  const int32_t* seq_lens;
  const int32_t* cu_seq_lens;
  int32_t batch;
  int32_t max_seq_len;
  int32_t num_layers;
  int32_t num_blocks;
  int32_t block_size;
  bool fp8;
};

struct CopyBlocksArgs {
  Plane latent, rope, scale;
  const int32_t* moves;  // (src, dst) pairs
  int32_t num_moves;
  int32_t num_layers;
  int32_t num_blocks;
  int32_t block_size;
  int32_t latent_row_bytes;
  int32_t rope_row_bytes;
  bool has_scale;
};

constexpr int kAttnInlineLens = 64;

struct AttnArgs {
  Plane latent, rope, scale;  // offset to the layer of the launch; layer_stride unused
  const char* q_latent;
  int64_t q_latent_seq_stride, q_latent_head_stride;
  const char* q_rope;
  int64_t q_rope_seq_stride, q_rope_head_stride;
  const int32_t* block_table;
  int32_t table_stride;
  const int32_t* seq_lens;   // device array, unless the lengths ride in the argument block (below)
  char* out;
  int64_t out_seq_stride, out_head_stride;
  float* lse;            // optional
  // Optional block-32 MX quantisation of the output (E4M3 codes [batch][heads][512], E8M0 scales
  // [batch][heads][16]); `out` may then be null.
  char* out_codes;
  int64_t out_codes_seq_stride, out_codes_head_stride;
  char* out_scales;
  int64_t out_scales_seq_stride, out_scales_head_stride;
  // Optional selection: int32 [batch][sparse_count] token positions, valid entries first, -1
  // after them; when set the sequence attends to those tokens only.
  const int32_t* sparse_indices;
  int64_t sparse_seq_stride;  // elements
  int32_t sparse_count;
  // Workspace: partials of the segments that do not hold a whole sequence, per group of 64 heads
  // [max_units + batch][64][512] bf16 and the same rows of fp32 log2-domain LSE.
  char* partial_out;
  float* partial_lse;
  float scale_log2;      // softmax scale * log2(e)
  int32_t batch;
  int32_t heads;
  int32_t num_blocks;
  int32_t block_size;
  int32_t max_tokens;         // lengths are clamped to min(plan's max_seq_len, table_stride * block_size)
  int32_t work_groups;        // workgroups per group of 64 heads
  int32_t max_units;          // bound on the work units of a launch (per head group)
  int32_t forced_unit_tiles;  // tiles per work unit; 0: from the live lengths
  int32_t min_unit_tiles;     // the smallest unit worth a query load
  int32_t cap_unit_tiles;     // what a segment's staged block-table entries can address
  int32_t spin_ticks;         // bound of the in-launch merge's wait, in 10 ns ticks
  bool merge_in_launch;       // false: the merge is a second launch
  bool fp8;
  // Selected-token attention only: a workgroup takes the whole selection of one sequence for one
  // block of 16 heads (1: no partials, no merge), or two workgroups take half of it each and the
  // second to finish combines the two (2); sparse_count <= kAttnHeadBlockTokens. 0: the split units.
  int32_t head_block_units;
  unsigned* sync;             // set by the launcher: this launch's counters, null for a second-launch merge
  // Host-known lengths of a small batch travel here instead of through device memory: no upload,
  // no launch for it, and the kernels' first dependent load is gone. inline_count = 0: unused.
  int32_t inline_count;
  int32_t inline_lens[kAttnInlineLens];
};

struct MxQuantArgs {
  const char* x;   // bf16 [rows][cols], cols a multiple of 32, rows 16-byte aligned
  int64_t x_row_stride;
  char* codes;     // E4M3 [rows][cols], rows 8-byte aligned
  int64_t codes_row_stride;
  char* scales;    // E8M0 [rows][cols / 32]
  int64_t scales_row_stride;
  int64_t rows;
  int32_t cols;
};

struct IndexerArgs {
  const char* query;        // E4M3 [batch][heads][128]
  int64_t query_seq_stride, query_head_stride;  // bytes
  const char* weights;      // bf16 [batch][heads]
  int64_t weights_seq_stride;                   // bytes
  const float* query_scale; // fp32 [batch][heads]
  int64_t query_scale_seq_stride;               // elements
  const char* key_base;     // E4M3 [block][slot][128]
  int64_t key_block_stride, key_row_stride;     // bytes
  const float* key_scale_base;                  // fp32 [block][slot]
  int64_t key_scale_block_stride;               // elements
  const int32_t* block_table;
  int32_t table_stride;
  const int32_t* seq_lens;
  unsigned short* keys;     // workspace [batch][keys_stride]
  int64_t keys_stride;
  int32_t* indices_out;     // int32 [batch][sparse_count]
  int64_t indices_seq_stride;                   // elements
  int32_t batch, heads, num_blocks, block_size, max_seq_len, sparse_count;
};

// MLA geometry the kernels are specialised for (include/moe/core/config.hpp:78-109 defaults).
constexpr int kLatentDim = 512;
constexpr int kRopeDim = 64;
constexpr int kTileTokens = 32;
constexpr int kAttnTableEntries = 512;     // block-table entries (or selected tokens) of one segment staged in LDS
constexpr int kAttnBoundaryTiles = 4;      // what entering a sequence inside a work unit costs, in tiles (see MakeCut)
constexpr int kAttnSyncSequences = 4096;   // (head group, sequence) pairs a launch can merge in place
constexpr int kAttnHeadBlockTokens = 1024; // selected tokens a whole-sequence unit of 16 heads stages in LDS

hipError_t LaunchAppend(const AppendArgs& args, hipStream_t stream);
hipError_t LaunchNormRopeAppend(const NormRopeAppendArgs& args, hipStream_t stream);
// With both events the launch records its own start and end in them (the dispatch's timestamps:
// no marker packets of their own in the queue, unlike hipEventRecord around the launch).
hipError_t LaunchGather(const GatherArgs& args, hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);
hipError_t LaunchCopyBlocks(const CopyBlocksArgs& args, hipStream_t stream);
// Writes `count` (<= kMaxStoreWords) 32-bit words to device memory at `dst`. The words travel in
// the kernel's argument block, which the runtime copies when the launch is queued: the caller's
// buffer is free again on return, with no staging buffer, copy engine or event involved.
constexpr int kMaxStoreWords = 960;
hipError_t LaunchStoreWords(const int32_t* host_words, int count, int32_t* dst, hipStream_t stream);
// The same with `pairs` scattered words behind them: host_pairs holds (index, value) couples and
// the kernel also writes scatter_dst[index] = value; count + 2 * pairs <= kMaxStoreWords.
hipError_t LaunchStoreWords(const int32_t* host_words, int count, int32_t* dst, const int32_t* host_pairs, int pairs,
                            int32_t* scatter_dst, hipStream_t stream);
// One launch for a step's metadata and its append: the words of LaunchStoreWords travel in the
// append kernel's argument block, its first workgroup stores them, and every workgroup takes its
// slots from the block (host_words[0 .. num_tokens) is the slot mapping) instead of from memory.
hipError_t LaunchAppendWithWords(const AppendArgs& args, const int32_t* host_words, int count, int32_t* dst, const int32_t* host_pairs,
                                 int pairs, int32_t* scatter_dst, hipStream_t stream);
hipError_t LaunchAttnDecode(const AttnArgs& args, hipStream_t stream);
hipError_t LaunchMxQuant(const MxQuantArgs& args, hipStream_t stream);
hipError_t LaunchIndexer(const IndexerArgs& args, hipStream_t stream);

struct IndexKeyAppendArgs {
  char* key_base;
  int64_t key_block_stride, key_row_stride;  // bytes
  float* key_scale_base;
  int64_t key_scale_block_stride;            // elements
  int32_t num_blocks, block_size;
  const char* src;                           // bf16 [num_tokens][128]
  int64_t src_row_stride;                    // bytes
  const int32_t* slots;
  int32_t num_tokens;
};
hipError_t LaunchIndexKeyAppend(const IndexKeyAppendArgs& args, hipStream_t stream);
// Per device, once: loads this file's kernels onto the current device and sets the attributes they
// need (dynamic LDS above 64 KB), so that no first launch pays for it. Idempotent and cheap after
// the first call on a device; the attention launcher calls its own, the others are for a caller's
// warm-up (mlakvPrepare).
hipError_t PrepareAttnKernels();
hipError_t PreparePagedCopyKernels();
hipError_t PrepareIndexerKernels();
hipError_t PrepareMxQuantKernels();
// Shared by the four: runs `prepare` once per device (the current one), remembering its result.
struct PerDeviceOnce {
  static constexpr int kMaxDevices = 64;
  int state[kMaxDevices] = {};  // 0: not yet, 1: done; guarded by the caller's mutex
};
// Device memory owned by the library for the split-KV partials of attention launches whose
// caller brings no workspace: kAttnStaticScratchBytes per GPU, resolved on first use on the
// current device. Launches that use it on one GPU share it.
constexpr uint64_t kAttnStaticScratchBytes = uint64_t{24} << 20;
hipError_t AttnStaticScratch(char** address);

}  // namespace mlakv
