// ref_boundary_probe -- the REFERENCE's own callers of the operator boundary (StaticMemoryArena,
// AclDeviceOps, OpTable, PlanAclnnOp, StaticOpSlot: compiled by oracle/Makefile from the reference
// sources where they lie, against include/compat instead of the CANN headers) linked to
// libmoe_kv_hip.so and driven through the two stages of the KV-cache path the way
// Dsv4Pipeline does (src/pipeline/pipeline.cpp:226-249 plan, :390-416 per layer, :515-519 per step).
// TEST INFRASTRUCTURE ONLY: it proves that the library is a drop-in for those callers (it links
// with no symbol left undefined, and on a GPU the reference's code drives the HIP kernels); the
// product never links it, and nothing of the reference is copied here.
//
//   ref_boundary_probe <in.bin> <out.bin> <layers> <steps> <block_size> <max_context> <live> <table>
//     in.bin   bf16 bits: per step and layer, one kv_a row [576] then one q_b row [64 * 576]
//     out.bin  bf16 bits: per step and layer, attn_out [64][512]
//     live     1: the kv length of every launch is the live context (aclnnMlaKvSetSeqLens, this
//                 library's extension); 0: as the reference plans it, the reserved context
//     table    1: identity block table; 0: the zero-filled table the reference leaves behind
// Prints one JSON line with what the reference's bookkeeping saw.
#include <cinttypes>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "moe/core/config.hpp"
#include "moe/core/device_ops.hpp"
#include "moe/core/error.hpp"
#include "moe/core/op_table.hpp"
#include "moe/memory/static_arena.hpp"

using namespace ascend_moe;

namespace {

constexpr int64_t kHeads = 64, kLatent = 512, kRope = 64, kRow = kLatent + kRope;
char kLayoutTnd[] = "TND";
char kCacheModeNorm[] = "Norm";

std::vector<uint16_t> ReadAll(const char* path) {
  std::FILE* file = std::fopen(path, "rb");
  if (file == nullptr) throw Dsv4Error(std::string("cannot open ") + path);
  std::fseek(file, 0, SEEK_END);
  const long bytes = std::ftell(file);
  std::fseek(file, 0, SEEK_SET);
  std::vector<uint16_t> data(static_cast<size_t>(bytes) / 2);
  if (std::fread(data.data(), 2, data.size(), file) != data.size()) throw Dsv4Error("short read");
  std::fclose(file);
  return data;
}

int Run(int argc, char** argv) {
  if (argc != 9) {
    std::fprintf(stderr, "usage: ref_boundary_probe in.bin out.bin layers steps block_size max_context live table\n");
    return 2;
  }
  const int64_t layers = std::atoll(argv[3]), steps = std::atoll(argv[4]), block_size = std::atoll(argv[5]);
  const int64_t max_context = std::atoll(argv[6]);
  const bool live = std::atoi(argv[7]) != 0, identity_table = std::atoi(argv[8]) != 0;
  const int64_t num_blocks = (max_context + block_size - 1) / block_size;
  const std::vector<uint16_t> input = ReadAll(argv[1]);
  const size_t per_item = static_cast<size_t>(kRow + kHeads * kRow);
  if (input.size() != per_item * static_cast<size_t>(layers * steps)) throw Dsv4Error("input size does not match layers x steps");

  AclDeviceOps device(0);                 // aclInit, aclrtSetDevice, aclrtCreateContext
  StaticMemoryArena arena(device);
  // RESERVE: the KV reservations of ReserveActivations / ReserveBackbone
  // (src/memory/static_arena_manager.cpp:298-300, :315-318) and the activations of the two stages.
  const ArenaHandle h_table = arena.Reserve("kv.block_table", sizeof(int32_t) * static_cast<size_t>(num_blocks));
  const ArenaHandle h_slot = arena.Reserve("kv.slot_mapping", sizeof(int32_t));
  const ArenaHandle h_normed = arena.Reserve("act.kv_latent_normed", 2 * kLatent);
  const ArenaHandle h_kv_a = arena.Reserve("act.kv_a", 2 * kRow);
  const ArenaHandle h_q_b = arena.Reserve("act.q_b", 2 * kHeads * kRow);
  const ArenaHandle h_out = arena.Reserve("act.attn_out", 2 * kHeads * kLatent);
  const ArenaHandle h_lse = arena.Reserve("act.softmax_lse", 4 * kHeads);
  const size_t latent_stride = static_cast<size_t>(2 * num_blocks * block_size * kLatent);
  const size_t rope_stride = static_cast<size_t>(2 * num_blocks * block_size * kRope);
  const ArenaHandle h_latent = arena.Reserve("kv.latent_cache", latent_stride * static_cast<size_t>(layers));
  const ArenaHandle h_rope = arena.Reserve("kv.rope_cache", rope_stride * static_cast<size_t>(layers));
  arena.Commit();                         // ONE device allocation, zero-filled
  const uint64_t allocations_after_commit = device.DeviceAllocationCount();

  // Descriptors as CreateDescriptors makes them (src/memory/static_arena_manager.cpp:480-497, :567-588).
  uint8_t* q_b_base = arena.AddressAs<uint8_t>(h_q_b);
  uint8_t* kv_a_base = arena.AddressAs<uint8_t>(h_kv_a);
  aclTensor* q_latent = arena.CreateTensor("q_latent", {1, kHeads, kLatent}, kAclBf16, q_b_base);
  aclTensor* q_rope = arena.CreateTensor("q_rope", {1, kHeads, kRope}, kAclBf16, q_b_base + 2 * kLatent);
  aclTensor* k_rope = arena.CreateTensor("k_rope", {1, 1, kRope}, kAclBf16, kv_a_base + 2 * kLatent);
  aclTensor* kv_latent_normed = arena.CreateTensor("kv_latent_normed", {1, kLatent}, kAclBf16, arena.Address(h_normed));
  aclTensor* attn_out = arena.CreateTensor("attn_out", {1, kHeads, kLatent}, kAclBf16, arena.Address(h_out));
  aclTensor* softmax_lse = arena.CreateTensor("softmax_lse", {1, kHeads, 1}, kAclFloat32, arena.Address(h_lse));
  aclTensor* kv_latent_cache =
      arena.CreateTensor("kv_latent_cache", {num_blocks, block_size, 1, kLatent}, kAclBf16, arena.Address(h_latent));
  aclTensor* kv_rope_cache = arena.CreateTensor("kv_rope_cache", {num_blocks, block_size, 1, kRope}, kAclBf16, arena.Address(h_rope));
  aclTensor* key_rope_cache_view =
      arena.CreateTensor("key_rope_cache_view", {num_blocks, block_size, 1, kRope}, kAclBf16, arena.Address(h_rope));
  aclTensorList* key_list = arena.CreateTensorList("fia_key_list", {kv_latent_cache});
  aclTensorList* value_list = arena.CreateTensorList("fia_value_list", {kv_latent_cache});
  aclTensor* block_table = arena.CreateTensor("block_table", {1, num_blocks}, kAclInt32, arena.Address(h_table));
  aclTensor* slot_mapping = arena.CreateTensor("slot_mapping", {1}, kAclInt32, arena.Address(h_slot));
  aclIntArray* actual_seq_q = arena.CreateIntArray("actual_seq_q", {1});
  aclIntArray* actual_seq_kv = arena.CreateIntArray("actual_seq_kv", {max_context});

  // Plan once (src/pipeline/pipeline.cpp:226-249), adopt into repeatable slots.
  OpTable ops;
  StaticOpSlot scatter, attention;
  aclOpExecutor* executor = nullptr;
  uint64_t workspace = PlanAclnnOp<ScatterPaKvCachePlanFn>(ops, OpId::kScatterPaKvCache, &executor, kv_latent_normed, kv_latent_cache,
                                                           slot_mapping, k_rope, kv_rope_cache, nullptr, nullptr, nullptr,
                                                           kCacheModeNorm, nullptr, nullptr, nullptr);
  scatter.Adopt(OpId::kScatterPaKvCache, "kv_cache_write", workspace, executor);
  arena.NoteWorkspace(workspace);
  const double scale = 1.0 / std::sqrt(192.0);
  workspace = PlanAclnnOp<FusedInferAttentionScoreV5PlanFn>(
      ops, OpId::kFusedInferAttentionScoreV5, &executor, q_latent, key_list, value_list, nullptr, nullptr, actual_seq_q, actual_seq_kv,
      nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, block_table, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
      nullptr, nullptr, nullptr, q_rope, key_rope_cache_view, nullptr, nullptr, nullptr, nullptr, nullptr, kHeads, scale,
      kFiaPreTokensAll, kFiaNextTokensCausal, kLayoutTnd, 1, kFiaSparseModeBand, kFiaInnerPreciseHighPrecision, block_size,
      kFiaAntiquantModeNone, false, kFiaAntiquantModeNone, kFiaAntiquantModeNone, kFiaQueryQuantModeNone, kFiaPseTypeNone, attn_out,
      softmax_lse);
  attention.Adopt(OpId::kFusedInferAttentionScoreV5, "attention", workspace, executor);
  aclOpExecutor* attention_executor = executor;
  arena.NoteWorkspace(workspace);
  arena.CommitWorkspace();                // the second and last allocation
  arena.Seal();
  const uint64_t allocations_after_build = device.DeviceAllocationCount();

  DeviceStream stream = device.CreateStream();
  if (identity_table) {  // the reference never writes the table; a paged read needs it
    std::vector<int32_t> identity(static_cast<size_t>(num_blocks));
    for (int64_t i = 0; i < num_blocks; ++i) identity[static_cast<size_t>(i)] = static_cast<int32_t>(i);
    device.MemcpySync(arena.Address(h_table), arena.Bytes(h_table), identity.data(), identity.size() * 4, MemcpyKind::kHostToDevice);
  }
  int32_t* slot_mailbox = static_cast<int32_t*>(device.HostPinnedMalloc(sizeof(int32_t) * static_cast<size_t>(steps)));
  uint16_t* staging = static_cast<uint16_t*>(device.HostPinnedMalloc(input.size() * 2));
  std::memcpy(staging, input.data(), input.size() * 2);
  std::vector<uint16_t> output(static_cast<size_t>(layers * steps * kHeads * kLatent));
  uint16_t* out_staging = static_cast<uint16_t*>(device.HostPinnedMalloc(output.size() * 2));

  for (int64_t position = 0; position < steps; ++position) {
    // slot of this token: the pinned mailbox is the DMA source (pipeline.cpp:515-519); one word
    // per step here, so no word is rewritten while its copy may still be queued
    slot_mailbox[position] = static_cast<int32_t>(position);
    device.MemcpyAsync(arena.Address(h_slot), 4, slot_mailbox + position, 4, MemcpyKind::kHostToDevice, stream);
    if (live) {
      const int64_t length = position + 1;
      if (aclnnMlaKvSetSeqLens(attention_executor, &length, 1) != 0) throw Dsv4Error("aclnnMlaKvSetSeqLens refused");
    }
    for (int64_t layer = 0; layer < layers; ++layer) {
      const uint16_t* item = staging + per_item * static_cast<size_t>(position * layers + layer);
      // what the stages before the cache write leave behind: kv_a (latent | rope), its normed
      // latent (here: the latent itself) and q_b
      device.MemcpyAsync(kv_a_base, 2 * kRow, item, 2 * kRow, MemcpyKind::kHostToDevice, stream);
      device.MemcpyAsync(arena.Address(h_normed), 2 * kLatent, item, 2 * kLatent, MemcpyKind::kHostToDevice, stream);
      device.MemcpyAsync(q_b_base, 2 * kHeads * kRow, item + kRow, 2 * kHeads * kRow, MemcpyKind::kHostToDevice, stream);
      // this layer's slice of the paged cache (pipeline.cpp:390-400)
      uint8_t* latent = arena.AddressAs<uint8_t>(h_latent) + latent_stride * static_cast<size_t>(layer);
      uint8_t* rope = arena.AddressAs<uint8_t>(h_rope) + rope_stride * static_cast<size_t>(layer);
      scatter.SetAddress(1, kv_latent_cache, latent);
      scatter.SetAddress(4, kv_rope_cache, rope);
      attention.SetTensorListAddress(1, 0, key_list, latent);
      attention.SetTensorListAddress(2, 0, value_list, latent);
      attention.SetAddress(25, key_rope_cache_view, rope);
      scatter.Launch(ops, arena.workspace(), stream);
      attention.Launch(ops, arena.workspace(), stream);
      device.MemcpyAsync(out_staging + static_cast<size_t>((position * layers + layer) * kHeads * kLatent), 2 * kHeads * kLatent,
                         arena.Address(h_out), 2 * kHeads * kLatent, MemcpyKind::kDeviceToHost, stream);
    }
  }
  device.SynchronizeStream(stream);
  const uint64_t allocations_after_steps = device.DeviceAllocationCount();
  std::memcpy(output.data(), out_staging, output.size() * 2);
  std::FILE* file = std::fopen(argv[2], "wb");
  if (file == nullptr || std::fwrite(output.data(), 2, output.size(), file) != output.size()) throw Dsv4Error("cannot write the output");
  std::fclose(file);
  device.DestroyStream(stream);
  device.HostPinnedFree(slot_mailbox);
  device.HostPinnedFree(staging);
  device.HostPinnedFree(out_staging);
  std::printf("{\"backend\": \"%s\", \"soc\": \"%s\", \"arena_bytes\": %zu, \"reservations\": %zu, \"workspace_bytes\": %" PRIu64
              ", \"allocations_after_commit\": %" PRIu64 ", \"allocations_after_build\": %" PRIu64 ", \"allocations_after_steps\": %" PRIu64
              ", \"scatter_found\": %d, \"attention_found\": %d, \"rms_norm_found\": %d}\n",
              device.backend_name(), device.soc_name().c_str(), arena.arena_bytes(), arena.reservations().size(),
              arena.workspace_bytes(), allocations_after_commit, allocations_after_build, allocations_after_steps,
              ops.op(OpId::kScatterPaKvCache).available() ? 1 : 0, ops.op(OpId::kFusedInferAttentionScoreV5).available() ? 1 : 0,
              ops.op(OpId::kRmsNorm).available() ? 1 : 0);
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    return Run(argc, argv);
  } catch (const std::exception& error) {
    std::fprintf(stderr, "ref_boundary_probe: %s\n", error.what());
    return 1;
  }
}
