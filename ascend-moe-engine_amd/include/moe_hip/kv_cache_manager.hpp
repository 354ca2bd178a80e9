// Paged MLA KV cache: reservations, physical block pool, block tables and the per-step
// metadata the kernels consume.
//
// The KV part of the reference's StaticArenaManager and pipeline, generalised from one
// sequence with identity paging to a batch sharing one pool:
//   num_blocks = ceil(max_context / block_size)     src/memory/static_arena_manager.cpp:192-201
//   kv.block_table, kv.slot_mapping reservations    :298-300
//   kv.latent_cache, kv.rope_cache reservations     :315-318  ([layer][block][slot][dim] bf16)
//   per-layer slice = base + layer * layer_stride   src/pipeline/pipeline.cpp:390-395
//   slot of the step's token                         src/pipeline/pipeline.cpp:515-519 (slot = position)
//   diagnostics                                      src/pipeline/pipeline.cpp:134-136, :532-534
// What the reference does not have and this class defines: a FIFO free list over physical
// blocks (optionally Fisher-Yates shuffled by SplitMix64), block recycling when a sequence
// finishes, compaction of live blocks to the front of the pool, FP8-E4M3 rows with one
// fp32 scale per slot, and an optional fused 576-element row layout.
#pragma once

#include <memory>
#include <utility>
#include <vector>

#include "moe_hip/static_arena.hpp"

namespace moe_hip {

enum class KvDtype : int32_t { kBf16 = 0, kFp8E4m3 = 1 };

struct KvCacheConfig {
  int64_t num_layers = kNumLayers;
  int64_t block_size = 128;          // RuntimeConfig default, include/moe/core/config.hpp:271-308
  int64_t max_context_len = 8192;
  int64_t max_batch = 1;             // kTokensPerStep in the reference
  int64_t pool_blocks = 0;           // 0: max_batch * num_blocks
  MlaGeometry mla;
  KvDtype dtype = KvDtype::kBf16;
  bool fused_rows = false;
  uint64_t seed = 0;
  bool shuffle = false;
};

// Plane addressing handed to the kernels; all strides in bytes.
struct KvPlane {
  void* base = nullptr;
  int64_t layer_stride = 0, block_stride = 0, row_stride = 0;
};

struct KvCacheView {
  KvPlane latent, rope, scale;
  int32_t num_layers = 0, num_blocks = 0, block_size = 0, latent_dim = 0, rope_dim = 0;
  KvDtype dtype = KvDtype::kBf16;
};

struct PagedAttentionStats {  // include/moe/diagnostics/inference_stats.hpp:21-28
  uint64_t total_blocks_allocated = 0;
  uint64_t active_context_tokens = 0;
  uint64_t block_size = 128;
  double kv_cache_utilization = 0.0;
};

uint64_t SplitMix64(uint64_t* state);

// Host bookkeeping of the physical block pool. The table rows live in caller-provided
// storage so the cache manager can keep them in its upload mirror.
class BlockPool {
 public:
  BlockPool(int64_t num_blocks, int64_t block_size, int64_t max_seqs, int64_t max_blocks_per_seq, uint64_t seed,
            bool shuffle, int32_t* table_storage);

  void AddSequence(int64_t seq, int64_t context_len);
  int32_t AppendToken(int64_t seq);  // returns the slot of the new token
  void FreeSequence(int64_t seq);
  // Moves every live block with id >= live_blocks() into the holes below it (highest live id
  // to lowest hole); rewrites the tables; the free list becomes live..P-1 ascending.
  std::vector<std::pair<int32_t, int32_t>> Compact();

  int64_t seq_len(int64_t seq) const { return seq_len_[static_cast<size_t>(seq)]; }  // -1: unused
  int64_t seq_blocks(int64_t seq) const { return seq_blocks_[static_cast<size_t>(seq)]; }
  int64_t free_blocks() const { return count_; }
  int64_t live_blocks() const { return num_blocks_ - count_; }
  int64_t num_blocks() const { return num_blocks_; }
  int64_t max_seqs() const { return max_seqs_; }
  int64_t max_blocks_per_seq() const { return max_blocks_per_seq_; }
  const int32_t* table() const { return table_; }
  std::vector<int32_t> FreeList() const;  // head first

 private:
  int32_t Pop();
  void Push(int32_t id);
  void RequireLive(int64_t seq, const char* what) const;

  int64_t num_blocks_, block_size_, max_seqs_, max_blocks_per_seq_;
  std::vector<int32_t> ring_;
  int64_t head_ = 0, count_ = 0;
  int32_t* table_;
  std::vector<int64_t> seq_len_, seq_blocks_;
};

class KvCacheManager {
 public:
  // RESERVE phase: records the KV reservations in `arena`.
  KvCacheManager(StaticMemoryArena& arena, const KvCacheConfig& config);
  ~KvCacheManager();
  KvCacheManager(const KvCacheManager&) = delete;
  KvCacheManager& operator=(const KvCacheManager&) = delete;

  // BUILD phase, after arena.Commit(): resolves addresses, allocates the pinned staging.
  void Bind();
  bool bound() const { return bound_; }

  const KvCacheConfig& config() const { return config_; }
  int64_t num_blocks() const { return num_blocks_; }      // per sequence
  int64_t pool_blocks() const { return pool_blocks_; }
  const KvCacheView& view() const { return view_; }
  // Layer strides of the two planes (src/pipeline/pipeline.cpp:391-392).
  size_t latent_layer_stride() const { return latent_layer_stride_; }
  size_t rope_layer_stride() const { return rope_layer_stride_; }

  void AddSequence(int64_t seq, int64_t context_len);
  // Bookkeeping of one token of one sequence; returns its slot. The slot mapping that UploadStep
  // sends holds one entry per sequence, the slot of its latest token: a caller that appends
  // several tokens of a sequence between uploads (a prefill) keeps the returned slots itself.
  int32_t AppendToken(int64_t seq);
  // The same for every live sequence in one call; slots (optional, max_batch entries) receives
  // each sequence's slot, -1 for an unused entry. Returns the number of tokens appended.
  int64_t AppendTokenAll(int32_t* slots);
  void FreeSequence(int64_t seq);
  // Plans and (on a kernel-capable backend) enqueues the defragmentation copy.
  std::vector<std::pair<int32_t, int32_t>> Compact(void* stream);
  // Enqueues the H2D copies of this step's metadata; afterwards the host slot mapping is
  // reset to -1 for the next step.
  void UploadStep(void* stream);
  // UploadStep followed by the append of one row per sequence (the rows of sequence s of layer l
  // at latent_src + l * layer stride + s * row stride, bf16; sequences without a token this step
  // are skipped) into layers [layer_begin, layer_begin + layer_count). When the step's metadata
  // fits one argument block both happen in a single launch: the append kernel carries the words,
  // its first workgroup stores them, and the rows take their slots from the block. Kernel-capable
  // backends only.
  void UploadStepAndAppend(const void* latent_src, int64_t latent_layer_stride, int64_t latent_row_stride, const void* rope_src,
                           int64_t rope_layer_stride, int64_t rope_row_stride, int32_t layer_begin, int32_t layer_count, void* stream);

  PagedAttentionStats stats() const;
  const BlockPool& pool() const { return *pool_; }

  const int32_t* host_block_table() const { return host_table_.data(); }
  const int32_t* host_slot_mapping() const { return host_small_.data(); }
  const int32_t* host_seq_lens() const { return host_small_.data() + small_seq_lens_; }
  const int32_t* host_cu_seq_lens() const { return host_small_.data() + small_cu_; }
  int32_t* device_block_table() const { return d_table_; }
  int32_t* device_slot_mapping() const { return d_small_; }
  int32_t* device_seq_lens() const { return d_small_ ? d_small_ + small_seq_lens_ : nullptr; }
  int32_t* device_cu_seq_lens() const { return d_small_ ? d_small_ + small_cu_ : nullptr; }
  int32_t* device_moves() const { return d_moves_; }

  ArenaHandle block_table_handle() const { return h_table_; }
  ArenaHandle slot_mapping_handle() const { return h_slot_; }
  ArenaHandle latent_cache_handle() const { return h_latent_; }
  ArenaHandle rope_cache_handle() const { return h_rope_; }

 private:
  void RefreshSeqLens();
  bool StepFitsOneLaunch() const;
  void FinishStep();

  StaticMemoryArena& arena_;
  KvCacheConfig config_;
  int64_t num_blocks_ = 0, pool_blocks_ = 0;
  size_t latent_layer_stride_ = 0, rope_layer_stride_ = 0, scale_layer_stride_ = 0;
  ArenaHandle h_table_ = kInvalidArenaHandle, h_slot_ = kInvalidArenaHandle, h_seq_lens_ = kInvalidArenaHandle,
              h_cu_ = kInvalidArenaHandle, h_moves_ = kInvalidArenaHandle, h_latent_ = kInvalidArenaHandle,
              h_rope_ = kInvalidArenaHandle, h_scale_ = kInvalidArenaHandle;
  // Host mirrors. host_small_ replicates the device span [kv.slot_mapping .. kv.cu_seq_lens]
  // (each reservation padded to the arena alignment) so one copy uploads all three.
  std::vector<int32_t> host_table_;
  std::vector<int32_t> host_small_;
  size_t small_seq_lens_ = 0, small_cu_ = 0;  // int32 offsets inside host_small_
  bool table_dirty_ = true;
  std::vector<int32_t> pending_entries_;  // table entries (flat indices) opened by AppendToken since the last upload
  std::vector<int32_t> entry_words_;      // their (index, value) pairs, rebuilt per upload
  std::unique_ptr<BlockPool> pool_;
  // Device addresses and pinned staging (two slots, reused only after their copy drained).
  int32_t* d_table_ = nullptr;
  int32_t* d_small_ = nullptr;
  int32_t* d_moves_ = nullptr;
  void* staging_[2] = {nullptr, nullptr};
  size_t staging_bytes_ = 0;
  int staging_next_ = 0;
  void* staging_event_[2] = {nullptr, nullptr};
  bool staging_busy_[2] = {false, false};
  void* moves_staging_ = nullptr;
  std::vector<int32_t> move_words_;  // the pairs of the last compaction, as they were sent
  void* moves_event_ = nullptr;
  bool moves_busy_ = false;
  KvCacheView view_;
  bool bound_ = false;
};

// Pure arithmetic of the reference, callable without any allocation.
int64_t NumBlocksFor(int64_t max_context_len, int64_t block_size);  // throws like the reference constructor
uint64_t BackboneDeviceBytes(const MlaGeometry& mla, int64_t block_size, int64_t max_context_len);

}  // namespace moe_hip
