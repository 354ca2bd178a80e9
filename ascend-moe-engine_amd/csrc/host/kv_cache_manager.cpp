// KvCacheManager / BlockPool: KV reservations in the static arena, the physical block pool
// and the per-step metadata upload.
#include "moe_hip/kv_cache_manager.hpp"

#include <cstring>

#include "../kernels/kernels.h"

namespace moe_hip {

// ---- arithmetic mirrors ---------------------------------------------------------

int64_t NumBlocksFor(int64_t max_context_len, int64_t block_size) {
  // src/memory/static_arena_manager.cpp:192-201
  MOE_HIP_REQUIRE(block_size > 0, "paged block size must be positive");
  MOE_HIP_REQUIRE(max_context_len >= block_size,
                  "max context " << max_context_len << " is below one block of " << block_size);
  return DivideUp(max_context_len, block_size);
}

uint64_t BackboneDeviceBytes(const MlaGeometry& mla, int64_t block_size, int64_t max_context_len) {
  // src/memory/static_arena_manager.cpp:205-241. Every weight term depends only on the
  // compiled topology; only the rope tables and the paged cache depend on the arguments.
  constexpr int64_t kHidden = 4096, kQLora = 1024, kInter = 2048, kExperts = 256, kVocab = 129280, kScaleBlock = 128;
  const auto scale_cols = [](int64_t k) { return DivideUp(k, kScaleBlock); };
  const int64_t kv_row = mla.kv_row_elements();
  const int64_t q_b = kNumAttentionHeads * kv_row;
  const int64_t o_in = kNumAttentionHeads * mla.kv_lora_rank;
  uint64_t layer = 0;
  layer += 2 * kHidden;                                   // input norm (bf16)
  layer += kQLora * kHidden + kQLora * scale_cols(kHidden);  // q_a + scale (fp8)
  layer += 2 * kQLora;                                    // q_a norm
  layer += q_b * kQLora + q_b * scale_cols(kQLora);       // q_b (folded) + scale
  layer += kv_row * kHidden + kv_row * scale_cols(kHidden);  // kv_a + scale
  layer += 2 * mla.kv_lora_rank;                          // kv_a norm
  layer += kHidden * o_in + kHidden * scale_cols(o_in);   // o (folded) + scale
  layer += 2 * kHidden;                                   // post norm
  layer += 2 * kExperts * kHidden;                        // router (bf16)
  layer += 4 * kExperts;                                  // router bias (fp32)
  layer += 2 * kInter * kHidden + 2 * kInter * scale_cols(kHidden);  // shared gate/up + scale
  layer += kHidden * kInter + kHidden * scale_cols(kInter);          // shared down + scale
  const int64_t blocks = DivideUp(max_context_len, block_size);
  uint64_t total = layer * static_cast<uint64_t>(kNumLayers);
  total += 2ull * 2 * kVocab * kHidden;                   // embed_tokens + lm_head
  total += 2 * kHidden;                                   // final norm
  total += 2ull * 2 * max_context_len * mla.qk_rope_head_dim;  // cos / sin tables
  total += 2ull * blocks * block_size * mla.kv_lora_rank * kNumLayers;
  total += 2ull * blocks * block_size * mla.qk_rope_head_dim * kNumLayers;
  return total;
}

uint64_t SplitMix64(uint64_t* state) {
  uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// ---- block pool -------------------------------------------------------------------

BlockPool::BlockPool(int64_t num_blocks, int64_t block_size, int64_t max_seqs, int64_t max_blocks_per_seq,
                     uint64_t seed, bool shuffle, int32_t* table_storage)
    : num_blocks_(num_blocks),
      block_size_(block_size),
      max_seqs_(max_seqs),
      max_blocks_per_seq_(max_blocks_per_seq),
      ring_(static_cast<size_t>(num_blocks)),
      table_(table_storage),
      seq_len_(static_cast<size_t>(max_seqs), -1),
      seq_blocks_(static_cast<size_t>(max_seqs), 0) {
  MOE_HIP_REQUIRE(num_blocks > 0 && block_size > 0 && max_seqs > 0 && max_blocks_per_seq > 0, "empty block pool");
  MOE_HIP_REQUIRE(num_blocks <= INT32_MAX / block_size, "slot indices of " << num_blocks << " blocks overflow int32");
  for (int64_t id = 0; id < num_blocks; ++id) ring_[static_cast<size_t>(id)] = static_cast<int32_t>(id);
  if (shuffle) {
    uint64_t state = seed;
    for (int64_t i = num_blocks - 1; i >= 1; --i) {
      const int64_t j = static_cast<int64_t>(SplitMix64(&state) % static_cast<uint64_t>(i + 1));
      std::swap(ring_[static_cast<size_t>(i)], ring_[static_cast<size_t>(j)]);
    }
  }
  count_ = num_blocks;
  std::memset(table_, 0, static_cast<size_t>(max_seqs * max_blocks_per_seq) * sizeof(int32_t));
}

int32_t BlockPool::Pop() {
  const int32_t id = ring_[static_cast<size_t>(head_)];
  head_ = (head_ + 1) % num_blocks_;
  --count_;
  return id;
}

void BlockPool::Push(int32_t id) {
  ring_[static_cast<size_t>((head_ + count_) % num_blocks_)] = id;
  ++count_;
}

void BlockPool::RequireLive(int64_t seq, const char* what) const {
  MOE_HIP_REQUIRE(seq >= 0 && seq < max_seqs_, what << ": sequence slot " << seq << " outside [0, " << max_seqs_ << ")");
  MOE_HIP_REQUIRE(seq_len_[static_cast<size_t>(seq)] >= 0, what << ": sequence slot " << seq << " is not in use");
}

void BlockPool::AddSequence(int64_t seq, int64_t context_len) {
  MOE_HIP_REQUIRE(seq >= 0 && seq < max_seqs_, "AddSequence: sequence slot " << seq << " outside [0, " << max_seqs_ << ")");
  MOE_HIP_REQUIRE(seq_len_[static_cast<size_t>(seq)] < 0, "AddSequence: sequence slot " << seq << " is already in use");
  MOE_HIP_REQUIRE(context_len >= 0, "AddSequence: negative context length");
  const int64_t need = DivideUp(context_len, block_size_);
  MOE_HIP_REQUIRE(need <= max_blocks_per_seq_, "AddSequence: " << context_len << " tokens exceed the reserved context of "
                                                               << max_blocks_per_seq_ * block_size_);
  MOE_HIP_REQUIRE(need <= count_, "AddSequence: " << need << " blocks wanted, " << count_ << " free in the pool");
  int32_t* row = table_ + seq * max_blocks_per_seq_;
  for (int64_t i = 0; i < need; ++i) row[i] = Pop();
  seq_len_[static_cast<size_t>(seq)] = context_len;
  seq_blocks_[static_cast<size_t>(seq)] = need;
}

int32_t BlockPool::AppendToken(int64_t seq) {
  RequireLive(seq, "AppendToken");
  const int64_t position = seq_len_[static_cast<size_t>(seq)];
  int32_t* row = table_ + seq * max_blocks_per_seq_;
  int64_t& blocks = seq_blocks_[static_cast<size_t>(seq)];
  if (position % block_size_ == 0) {
    MOE_HIP_REQUIRE(blocks < max_blocks_per_seq_, "AppendToken: position " << position << " outside the reserved context of "
                                                                           << max_blocks_per_seq_ * block_size_);
    MOE_HIP_REQUIRE(count_ > 0, "AppendToken: the block pool is exhausted");
    row[blocks++] = Pop();
  }
  seq_len_[static_cast<size_t>(seq)] = position + 1;
  return static_cast<int32_t>(static_cast<int64_t>(row[position / block_size_]) * block_size_ + position % block_size_);
}

void BlockPool::FreeSequence(int64_t seq) {
  RequireLive(seq, "FreeSequence");
  int32_t* row = table_ + seq * max_blocks_per_seq_;
  for (int64_t i = 0; i < seq_blocks_[static_cast<size_t>(seq)]; ++i) {
    Push(row[i]);
    row[i] = 0;
  }
  seq_len_[static_cast<size_t>(seq)] = -1;
  seq_blocks_[static_cast<size_t>(seq)] = 0;
}

std::vector<std::pair<int32_t, int32_t>> BlockPool::Compact() {
  const int64_t live = live_blocks();
  // Which table entry owns each physical block (-1: free).
  std::vector<int64_t> owner(static_cast<size_t>(num_blocks_), -1);
  for (int64_t seq = 0; seq < max_seqs_; ++seq) {
    for (int64_t i = 0; i < seq_blocks_[static_cast<size_t>(seq)]; ++i) {
      owner[static_cast<size_t>(table_[seq * max_blocks_per_seq_ + i])] = seq * max_blocks_per_seq_ + i;
    }
  }
  std::vector<std::pair<int32_t, int32_t>> moves;
  int64_t hole = 0;
  for (int64_t source = num_blocks_ - 1; source >= live; --source) {
    const int64_t entry = owner[static_cast<size_t>(source)];
    if (entry < 0) continue;
    while (owner[static_cast<size_t>(hole)] >= 0) ++hole;
    moves.emplace_back(static_cast<int32_t>(source), static_cast<int32_t>(hole));
    table_[entry] = static_cast<int32_t>(hole);
    owner[static_cast<size_t>(hole)] = entry;
    owner[static_cast<size_t>(source)] = -1;
  }
  head_ = 0;
  count_ = num_blocks_ - live;
  for (int64_t i = 0; i < count_; ++i) ring_[static_cast<size_t>(i)] = static_cast<int32_t>(live + i);
  return moves;
}

std::vector<int32_t> BlockPool::FreeList() const {
  std::vector<int32_t> out(static_cast<size_t>(count_));
  for (int64_t i = 0; i < count_; ++i) out[static_cast<size_t>(i)] = ring_[static_cast<size_t>((head_ + i) % num_blocks_)];
  return out;
}

// ---- cache manager -------------------------------------------------------------------

namespace {
size_t ElementBytes(KvDtype dtype) { return dtype == KvDtype::kBf16 ? 2 : 1; }
}  // namespace

KvCacheManager::KvCacheManager(StaticMemoryArena& arena, const KvCacheConfig& config) : arena_(arena), config_(config) {
  MOE_HIP_REQUIRE(config_.num_layers > 0, "a KV cache needs at least one layer");
  MOE_HIP_REQUIRE(config_.max_batch > 0, "a KV cache needs at least one sequence slot");
  MOE_HIP_REQUIRE(config_.mla.kv_lora_rank > 0 && config_.mla.qk_rope_head_dim > 0, "empty MLA geometry");
  num_blocks_ = NumBlocksFor(config_.max_context_len, config_.block_size);
  pool_blocks_ = config_.pool_blocks > 0 ? config_.pool_blocks : config_.max_batch * num_blocks_;
  MOE_HIP_REQUIRE(pool_blocks_ <= INT32_MAX / config_.block_size, "the pool's slot indices overflow int32");

  const size_t element = ElementBytes(config_.dtype);
  const size_t batch = static_cast<size_t>(config_.max_batch);
  const size_t slots_per_layer = static_cast<size_t>(pool_blocks_ * config_.block_size);
  const size_t layers = static_cast<size_t>(config_.num_layers);

  // Same names and, for one sequence in bf16, the same sizes as the reference's four KV
  // reservations; the metadata trio after kv.slot_mapping is reserved back to back so one
  // copy uploads it.
  h_table_ = arena_.Reserve("kv.block_table", sizeof(int32_t) * batch * static_cast<size_t>(num_blocks_));
  h_slot_ = arena_.Reserve("kv.slot_mapping", sizeof(int32_t) * batch);
  h_seq_lens_ = arena_.Reserve("kv.seq_lens", sizeof(int32_t) * batch);
  h_cu_ = arena_.Reserve("kv.cu_seq_lens", sizeof(int32_t) * (batch + 1));
  h_moves_ = arena_.Reserve("kv.compaction_moves", 2 * sizeof(int32_t) * static_cast<size_t>(pool_blocks_));
  if (config_.fused_rows) {
    h_latent_ = arena_.Reserve("kv.latent_cache",
                               element * layers * slots_per_layer * static_cast<size_t>(config_.mla.kv_row_elements()));
    latent_layer_stride_ = element * slots_per_layer * static_cast<size_t>(config_.mla.kv_row_elements());
    rope_layer_stride_ = latent_layer_stride_;
  } else {
    h_latent_ = arena_.Reserve("kv.latent_cache",
                               element * layers * slots_per_layer * static_cast<size_t>(config_.mla.kv_lora_rank));
    h_rope_ = arena_.Reserve("kv.rope_cache",
                             element * layers * slots_per_layer * static_cast<size_t>(config_.mla.qk_rope_head_dim));
    latent_layer_stride_ = element * slots_per_layer * static_cast<size_t>(config_.mla.kv_lora_rank);
    rope_layer_stride_ = element * slots_per_layer * static_cast<size_t>(config_.mla.qk_rope_head_dim);
  }
  if (config_.dtype == KvDtype::kFp8E4m3) {
    h_scale_ = arena_.Reserve("kv.scale_cache", sizeof(float) * layers * slots_per_layer);
    scale_layer_stride_ = sizeof(float) * slots_per_layer;
  }

  host_table_.assign(batch * static_cast<size_t>(num_blocks_), 0);
  const size_t small_begin = arena_.Offset(h_slot_);
  const size_t small_end = arena_.Offset(h_cu_) + arena_.Bytes(h_cu_);
  small_seq_lens_ = (arena_.Offset(h_seq_lens_) - small_begin) / sizeof(int32_t);
  small_cu_ = (arena_.Offset(h_cu_) - small_begin) / sizeof(int32_t);
  host_small_.assign((small_end - small_begin) / sizeof(int32_t), 0);
  for (size_t s = 0; s < batch; ++s) host_small_[s] = -1;
  pool_ = std::make_unique<BlockPool>(pool_blocks_, config_.block_size, config_.max_batch, num_blocks_, config_.seed,
                                      config_.shuffle, host_table_.data());
}

KvCacheManager::~KvCacheManager() {
  IDeviceBackend& backend = arena_.backend();
  // A destructor reports nothing: after a device error the waits below may fail, and the
  // staging memory is then released without them.
  const auto quietly = [](auto&& body) {
    try {
      body();
    } catch (...) {
    }
  };
  for (int k = 0; k < 2; ++k) {
    if (staging_busy_[k]) quietly([&] { backend.SynchronizeEvent(staging_event_[k]); });
    quietly([&] { backend.DestroyEvent(staging_event_[k]); });
    quietly([&] { backend.HostPinnedFree(staging_[k]); });
  }
  if (moves_busy_) quietly([&] { backend.SynchronizeEvent(moves_event_); });
  quietly([&] { backend.DestroyEvent(moves_event_); });
  quietly([&] { backend.HostPinnedFree(moves_staging_); });
}

void KvCacheManager::Bind() {
  MOE_HIP_REQUIRE(!bound_, "the KV cache is already bound");
  MOE_HIP_REQUIRE(arena_.committed(), "Bind needs the arena to be committed first");
  IDeviceBackend& backend = arena_.backend();
  d_table_ = arena_.AddressAs<int32_t>(h_table_);
  d_small_ = arena_.AddressAs<int32_t>(h_slot_);
  d_moves_ = arena_.AddressAs<int32_t>(h_moves_);

  const size_t element = ElementBytes(config_.dtype);
  const int64_t latent_row = static_cast<int64_t>(element) * config_.mla.kv_lora_rank;
  const int64_t rope_row = static_cast<int64_t>(element) * config_.mla.qk_rope_head_dim;
  view_.latent.base = arena_.Address(h_latent_);
  view_.latent.row_stride = config_.fused_rows ? latent_row + rope_row : latent_row;
  view_.latent.block_stride = view_.latent.row_stride * config_.block_size;
  view_.latent.layer_stride = static_cast<int64_t>(latent_layer_stride_);
  if (config_.fused_rows) {
    view_.rope = view_.latent;
    view_.rope.base = static_cast<uint8_t*>(view_.latent.base) + latent_row;
  } else {
    view_.rope.base = arena_.Address(h_rope_);
    view_.rope.row_stride = rope_row;
    view_.rope.block_stride = rope_row * config_.block_size;
    view_.rope.layer_stride = static_cast<int64_t>(rope_layer_stride_);
  }
  if (config_.dtype == KvDtype::kFp8E4m3) {
    view_.scale.base = arena_.Address(h_scale_);
    view_.scale.row_stride = sizeof(float);
    view_.scale.block_stride = static_cast<int64_t>(sizeof(float)) * config_.block_size;
    view_.scale.layer_stride = static_cast<int64_t>(scale_layer_stride_);
  }
  view_.num_layers = static_cast<int32_t>(config_.num_layers);
  view_.num_blocks = static_cast<int32_t>(pool_blocks_);
  view_.block_size = static_cast<int32_t>(config_.block_size);
  view_.latent_dim = static_cast<int32_t>(config_.mla.kv_lora_rank);
  view_.rope_dim = static_cast<int32_t>(config_.mla.qk_rope_head_dim);
  view_.dtype = config_.dtype;

  staging_bytes_ = host_table_.size() * sizeof(int32_t) + host_small_.size() * sizeof(int32_t);
  for (int k = 0; k < 2; ++k) {
    staging_[k] = backend.HostPinnedMalloc(staging_bytes_);
    staging_event_[k] = backend.CreateEvent();
  }
  moves_staging_ = backend.HostPinnedMalloc(arena_.Bytes(h_moves_));
  moves_event_ = backend.CreateEvent();
  bound_ = true;
}

void KvCacheManager::AddSequence(int64_t seq, int64_t context_len) {
  pool_->AddSequence(seq, context_len);
  table_dirty_ = true;
}

int32_t KvCacheManager::AppendToken(int64_t seq) {
  const int64_t blocks_before = seq >= 0 && seq < config_.max_batch ? pool_->seq_blocks(seq) : 0;
  const int32_t slot = pool_->AppendToken(seq);
  // A token that opened a block changed one table entry: it is remembered and sent with the
  // step's small arrays instead of marking the whole table for a copy.
  if (pool_->seq_blocks(seq) != blocks_before) pending_entries_.push_back(static_cast<int32_t>(seq * num_blocks_ + blocks_before));
  host_small_[static_cast<size_t>(seq)] = slot;
  return slot;
}

int64_t KvCacheManager::AppendTokenAll(int32_t* slots) {
  int64_t appended = 0;
  for (int64_t seq = 0; seq < config_.max_batch; ++seq) {
    if (pool_->seq_len(seq) < 0) {
      if (slots != nullptr) slots[seq] = -1;
      continue;
    }
    const int32_t slot = AppendToken(seq);
    if (slots != nullptr) slots[seq] = slot;
    ++appended;
  }
  return appended;
}

void KvCacheManager::FreeSequence(int64_t seq) {
  pool_->FreeSequence(seq);
  host_small_[static_cast<size_t>(seq)] = -1;
  table_dirty_ = true;
}

void KvCacheManager::RefreshSeqLens() {
  int32_t* seq_lens = host_small_.data() + small_seq_lens_;
  int32_t* cu = host_small_.data() + small_cu_;
  int64_t running = 0;
  for (int64_t s = 0; s < config_.max_batch; ++s) {
    const int64_t len = pool_->seq_len(s) < 0 ? 0 : pool_->seq_len(s);
    seq_lens[s] = static_cast<int32_t>(len);
    cu[s] = static_cast<int32_t>(running);
    running += len;
  }
  MOE_HIP_REQUIRE(running <= INT32_MAX, "the batch holds more than 2^31 tokens");
  cu[config_.max_batch] = static_cast<int32_t>(running);
}

void KvCacheManager::UploadStep(void* stream) {
  MOE_HIP_REQUIRE(bound_, "UploadStep before Bind");
  RefreshSeqLens();
  IDeviceBackend& backend = arena_.backend();
  const size_t table_bytes = host_table_.size() * sizeof(int32_t);
  const size_t small_bytes = host_small_.size() * sizeof(int32_t);
  // The usual step changes only the small arrays (slot mapping, lengths, their prefix sums). On
  // a device that runs kernels they ride in the argument block of a one-workgroup kernel: no
  // pinned staging, no copy engine and no event per step, which together cost more stream time
  // than the append itself.
  const bool by_kernel = StepFitsOneLaunch();
  if (by_kernel) {
    entry_words_.clear();
    for (const int32_t index : pending_entries_) {
      entry_words_.push_back(index);
      entry_words_.push_back(host_table_[static_cast<size_t>(index)]);
    }
    const hipError_t e = mlakv::LaunchStoreWords(host_small_.data(), static_cast<int>(host_small_.size()),
                                                 static_cast<int32_t*>(d_small_), entry_words_.data(),
                                                 static_cast<int>(pending_entries_.size()), d_table_,
                                                 static_cast<hipStream_t>(stream));
    MOE_HIP_REQUIRE(e == hipSuccess, "UploadStep: metadata kernel launch failed");
  } else {
    if (!pending_entries_.empty()) table_dirty_ = true;  // too many for one argument block
    const int k = staging_next_;
    staging_next_ ^= 1;
    if (staging_busy_[k]) backend.SynchronizeEvent(staging_event_[k]);  // copy from two steps ago
    uint8_t* staging = static_cast<uint8_t*>(staging_[k]);
    if (table_dirty_) {
      std::memcpy(staging, host_table_.data(), table_bytes);
      backend.MemcpyAsync(d_table_, arena_.Bytes(h_table_), staging, table_bytes, CopyKind::kHostToDevice, stream);
      table_dirty_ = false;
    }
    std::memcpy(staging + table_bytes, host_small_.data(), small_bytes);
    backend.MemcpyAsync(d_small_, small_bytes, staging + table_bytes, small_bytes, CopyKind::kHostToDevice, stream);
    backend.RecordEvent(staging_event_[k], stream);
    staging_busy_[k] = true;
  }
  FinishStep();
}

// Whether the step's small arrays and the table entries opened since the last upload ((index,
// value) pairs) fit the argument block of one kernel.
bool KvCacheManager::StepFitsOneLaunch() const {
  return arena_.backend().runs_kernels() && !table_dirty_ &&
         host_small_.size() + 2 * pending_entries_.size() <= static_cast<size_t>(mlakv::kMaxStoreWords);
}

void KvCacheManager::FinishStep() {
  pending_entries_.clear();
  for (int64_t s = 0; s < config_.max_batch; ++s) host_small_[static_cast<size_t>(s)] = -1;
}

void KvCacheManager::UploadStepAndAppend(const void* latent_src, int64_t latent_layer_stride, int64_t latent_row_stride,
                                         const void* rope_src, int64_t rope_layer_stride, int64_t rope_row_stride,
                                         int32_t layer_begin, int32_t layer_count, void* stream) {
  MOE_HIP_REQUIRE(bound_, "UploadStepAndAppend before Bind");
  MOE_HIP_REQUIRE(arena_.backend().runs_kernels(), "UploadStepAndAppend needs a backend that runs kernels");
  MOE_HIP_REQUIRE(latent_src != nullptr && rope_src != nullptr, "UploadStepAndAppend: source rows are required");
  MOE_HIP_REQUIRE(layer_begin >= 0 && layer_count >= 0 && layer_begin + layer_count <= view_.num_layers,
                  "UploadStepAndAppend: layers [" << layer_begin << ", " << layer_begin + layer_count << ") outside the cache");
  mlakv::AppendArgs args{};
  const auto plane = [&](const KvPlane& p) {
    char* base = static_cast<char*>(p.base);
    return mlakv::Plane{base == nullptr ? nullptr : base + layer_begin * p.layer_stride, p.layer_stride, p.block_stride, p.row_stride};
  };
  args.latent = plane(view_.latent);
  args.rope = plane(view_.rope);
  args.scale = plane(view_.scale);
  args.latent_src = {const_cast<char*>(static_cast<const char*>(latent_src)), latent_layer_stride, latent_row_stride};
  args.rope_src = {const_cast<char*>(static_cast<const char*>(rope_src)), rope_layer_stride, rope_row_stride};
  args.slots = d_small_;
  args.num_tokens = static_cast<int32_t>(config_.max_batch);
  args.num_layers = layer_count;
  args.num_blocks = view_.num_blocks;
  args.block_size = view_.block_size;
  args.fp8 = config_.dtype == KvDtype::kFp8E4m3;
  if (layer_count == 0 || !StepFitsOneLaunch()) {
    UploadStep(stream);
    const hipError_t e = mlakv::LaunchAppend(args, static_cast<hipStream_t>(stream));
    MOE_HIP_REQUIRE(e == hipSuccess, "UploadStepAndAppend: append launch failed: " << hipGetErrorString(e));
    return;
  }
  RefreshSeqLens();
  entry_words_.clear();
  for (const int32_t index : pending_entries_) {
    entry_words_.push_back(index);
    entry_words_.push_back(host_table_[static_cast<size_t>(index)]);
  }
  const hipError_t e = mlakv::LaunchAppendWithWords(args, host_small_.data(), static_cast<int>(host_small_.size()), d_small_,
                                                    entry_words_.data(), static_cast<int>(pending_entries_.size()), d_table_,
                                                    static_cast<hipStream_t>(stream));
  MOE_HIP_REQUIRE(e == hipSuccess, "UploadStepAndAppend: launch failed: " << hipGetErrorString(e));
  FinishStep();
}

std::vector<std::pair<int32_t, int32_t>> KvCacheManager::Compact(void* stream) {
  std::vector<std::pair<int32_t, int32_t>> moves = pool_->Compact();
  table_dirty_ = true;
  // Tokens appended since the last UploadStep have their slots waiting in the mirror: a slot
  // inside a block that moves follows the block (the append kernel, which runs after the copy
  // in stream order, then writes the row where attention will look for it).
  if (!moves.empty()) {
    const int32_t bs = static_cast<int32_t>(config_.block_size);
    for (int64_t seq = 0; seq < config_.max_batch; ++seq) {
      int32_t& slot = host_small_[static_cast<size_t>(seq)];
      if (slot < 0) continue;
      const int32_t block = slot / bs;
      for (const auto& move : moves) {
        if (move.first == block) {
          slot = move.second * bs + slot % bs;
          break;
        }
      }
    }
  }
  if (moves.empty() || !bound_) return moves;
  IDeviceBackend& backend = arena_.backend();
  if (backend.runs_kernels()) {
    // The (source, destination) pairs travel in the argument blocks of small launches, 480 pairs
    // each: the runtime copies an argument block when the launch is queued, so there is no staging
    // buffer to keep alive until an event fires and no copy engine between two kernels of the stream.
    move_words_.resize(moves.size() * 2);
    for (size_t i = 0; i < moves.size(); ++i) {
      move_words_[2 * i] = moves[i].first;
      move_words_[2 * i + 1] = moves[i].second;
    }
    for (size_t done = 0; done < move_words_.size(); done += mlakv::kMaxStoreWords) {
      const size_t count = std::min(move_words_.size() - done, static_cast<size_t>(mlakv::kMaxStoreWords));
      const hipError_t e = mlakv::LaunchStoreWords(move_words_.data() + done, static_cast<int>(count), d_moves_ + done,
                                                   static_cast<hipStream_t>(stream));
      MOE_HIP_REQUIRE(e == hipSuccess, "compaction move upload failed: " << hipGetErrorString(e));
    }
  } else {
    if (moves_busy_) backend.SynchronizeEvent(moves_event_);
    int32_t* staging = static_cast<int32_t*>(moves_staging_);
    for (size_t i = 0; i < moves.size(); ++i) {
      staging[2 * i] = moves[i].first;
      staging[2 * i + 1] = moves[i].second;
    }
    const size_t bytes = moves.size() * 2 * sizeof(int32_t);
    backend.MemcpyAsync(d_moves_, arena_.Bytes(h_moves_), staging, bytes, CopyKind::kHostToDevice, stream);
    backend.RecordEvent(moves_event_, stream);
    moves_busy_ = true;
  }
  if (backend.runs_kernels()) {
    mlakv::CopyBlocksArgs args{};
    const auto plane = [](const KvPlane& p) {
      return mlakv::Plane{static_cast<char*>(p.base), p.layer_stride, p.block_stride, p.row_stride};
    };
    args.latent = plane(view_.latent);
    args.rope = plane(view_.rope);
    args.scale = plane(view_.scale);
    args.moves = d_moves_;
    args.num_moves = static_cast<int32_t>(moves.size());
    args.num_layers = view_.num_layers;
    args.num_blocks = view_.num_blocks;
    args.block_size = view_.block_size;
    const int32_t element = static_cast<int32_t>(ElementBytes(config_.dtype));
    args.latent_row_bytes = element * view_.latent_dim;
    args.rope_row_bytes = element * view_.rope_dim;
    args.has_scale = config_.dtype == KvDtype::kFp8E4m3;
    const hipError_t status = mlakv::LaunchCopyBlocks(args, static_cast<hipStream_t>(stream));
    MOE_HIP_REQUIRE(status == hipSuccess, "compaction copy launch failed: " << hipGetErrorString(status));
  }
  // On the host backend only the bookkeeping above happens: bytes are moved by the HIP
  // kernel or not at all.
  return moves;
}

PagedAttentionStats KvCacheManager::stats() const {
  PagedAttentionStats out;
  out.total_blocks_allocated = static_cast<uint64_t>(pool_blocks_ * config_.num_layers);
  uint64_t active = 0;
  for (int64_t s = 0; s < config_.max_batch; ++s) {
    if (pool_->seq_len(s) > 0) active += static_cast<uint64_t>(pool_->seq_len(s));
  }
  out.active_context_tokens = active;
  out.block_size = static_cast<uint64_t>(config_.block_size);
  out.kv_cache_utilization = static_cast<double>(active) / static_cast<double>(pool_blocks_ * config_.block_size);
  return out;
}

}  // namespace moe_hip
