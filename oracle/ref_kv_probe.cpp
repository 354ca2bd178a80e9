// ref_kv_probe -- a small driver around the REFERENCE's own host classes, built by
// oracle/Makefile from the reference sources where they lie (never copied here).
// TEST INFRASTRUCTURE ONLY: it exists to validate the CPU oracle and to write the
// golden ledger fixture; the product never links it.
//
// Commands (all output is JSON on stdout):
//   ledger <block_size> <max_context>     the reference StaticArenaManager reserves its
//                                         activations + backbone and commits on the mock
//                                         runtime; prints the KV reservations, arena size,
//                                         num_blocks, BackboneDeviceBytes and the KV
//                                         diagnostics at Build time
//   arena-script <n> <bytes,align>...     replays Reserve calls on the reference
//                                         StaticMemoryArena over SimulatedDeviceOps, then
//                                         Commit; prints offsets / refusals / arena size
//   arena-contract                        the phase-latch sequence of the reference's own
//                                         TestStaticArena, one outcome per line
//   stats <block_size> <max_context> <position>   the pipeline's KV diagnostics arithmetic
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "moe/core/config.hpp"
#include "moe/core/device_ops.hpp"
#include "moe/core/error.hpp"
#include "moe/memory/static_arena.hpp"
#include "moe/memory/static_arena_manager.hpp"

using namespace ascend_moe;

namespace {

bool Refuses(const std::function<void()>& action) {
  try {
    action();
  } catch (const Dsv4Error&) {
    return true;
  }
  return false;
}

int Ledger(int64_t block_size, int64_t max_context) {
  RuntimeConfig config;
  config.block_size = block_size;
  config.max_context_len = max_context;
  config.synthetic_weights = true;
  AclDeviceOps device(0);
  StaticArenaManager manager(device, device, config);
  manager.ReserveActivations();
  manager.ReserveBackbone();
  manager.Commit();
  const StaticMemoryArena& arena = manager.arena();
  std::printf("{\"block_size\": %" PRId64 ", \"max_context\": %" PRId64 ", \"num_blocks\": %" PRId64
              ", \"arena_bytes\": %zu, \"reservations\": %zu, \"backbone_device_bytes\": %zu, "
              "\"total_blocks_allocated\": %" PRId64 ", \"kv\": {",
              block_size, max_context, manager.num_blocks(), arena.arena_bytes(), arena.reservations().size(),
              StaticArenaManager::BackboneDeviceBytes(config.mla, block_size, max_context),
              manager.num_blocks() * kNumLayers);
  bool first = true;
  for (const ArenaReservation& reservation : arena.reservations()) {
    const bool wanted = std::strncmp(reservation.name, "kv.", 3) == 0 || std::strcmp(reservation.name, "w.rope_cos") == 0 ||
                        std::strcmp(reservation.name, "w.rope_sin") == 0;
    if (!wanted) continue;
    std::printf("%s\"%s\": {\"offset\": %zu, \"bytes\": %zu, \"align\": %zu}", first ? "" : ", ", reservation.name,
                reservation.offset, reservation.bytes, reservation.align);
    first = false;
  }
  std::printf("}}\n");
  return 0;
}

int ArenaScript(int argc, char** argv) {
  const int count = std::atoi(argv[2]);
  SimulatedDeviceOps device(1ull << 30);
  StaticMemoryArena arena(device);
  std::printf("{\"steps\": [");
  for (int index = 0; index < count; ++index) {
    size_t bytes = 0, align = 0;
    if (std::sscanf(argv[3 + index], "%zu,%zu", &bytes, &align) != 2) return 2;
    ArenaHandle handle = kInvalidArenaHandle;
    const bool refused = Refuses([&] { handle = arena.Reserve("probe", bytes, align); });
    if (refused) {
      std::printf("%s{\"refused\": true}", index ? ", " : "");
    } else {
      std::printf("%s{\"refused\": false, \"handle\": %zu, \"offset\": %zu}", index ? ", " : "", handle,
                  arena.reservations()[handle].offset);
    }
  }
  const bool commit_refused = Refuses([&] { arena.Commit(); });
  std::printf("], \"commit_refused\": %s, \"reserved_bytes\": %zu, \"arena_bytes\": %zu, \"device_allocations\": %" PRIu64
              ", \"base_mod_4096\": %zu}\n",
              commit_refused ? "true" : "false", arena.reserved_bytes(), arena.arena_bytes(),
              device.counters().device_allocations,
              static_cast<size_t>(reinterpret_cast<uintptr_t>(arena.arena_base()) % 4096));
  return 0;
}

// The same calls, in the same order, as the reference's TestStaticArena
// (tests/mock_contract_smoke.cpp:533-584); prints each observable.
int ArenaContract() {
  SimulatedDeviceOps device(1ull << 30);
  StaticMemoryArena arena(device);
  const ArenaHandle first = arena.Reserve("a.small", 100);
  const ArenaHandle second = arena.Reserve("b.aligned", 4096, 4096);
  const ArenaHandle third = arena.Reserve("c.tail", 7);
  std::printf("{");
  std::printf("\"address_before_commit_refused\": %d, ", Refuses([&] { arena.Address(first); }));
  std::printf("\"zero_byte_refused\": %d, ", Refuses([&] { arena.Reserve("d.zero", 0); }));
  std::printf("\"odd_align_refused\": %d, ", Refuses([&] { arena.Reserve("e.odd-align", 64, 3); }));
  arena.Commit();
  std::printf("\"allocations_after_commit\": %" PRIu64 ", ", device.counters().device_allocations);
  std::printf("\"offsets\": [%zu, %zu, %zu], ", arena.reservations()[first].offset, arena.reservations()[second].offset,
              arena.reservations()[third].offset);
  std::printf("\"arena_bytes\": %zu, ", arena.arena_bytes());
  std::printf("\"second_abs_mod_4096\": %zu, ",
              static_cast<size_t>(reinterpret_cast<uintptr_t>(arena.Address(second)) % 4096));
  std::printf("\"late_reserve_refused\": %d, ", Refuses([&] { arena.Reserve("f.late", 8); }));
  arena.NoteWorkspace(1024);
  arena.NoteWorkspace(4096);
  arena.NoteWorkspace(2048);
  arena.CommitWorkspace();
  std::printf("\"workspace_bytes\": %" PRIu64 ", ", arena.workspace_bytes());
  std::printf("\"fits_4096_refused\": %d, ", Refuses([&] { arena.AssertWorkspaceFits(4096, "probe"); }));
  std::printf("\"fits_4097_refused\": %d, ", Refuses([&] { arena.AssertWorkspaceFits(4097, "probe"); }));
  std::printf("\"allocations_after_workspace\": %" PRIu64 ", ", device.counters().device_allocations);
  arena.Seal();
  std::printf("\"sealed\": %d, ", arena.sealed() ? 1 : 0);
  std::printf("\"sealed_reserve_refused\": %d, ", Refuses([&] { arena.Reserve("g.sealed", 8); }));
  std::printf("\"sealed_descriptor_refused\": %d, ", Refuses([&] { arena.CreateIntArray("h.sealed", {1, 2}); }));
  std::printf("\"sealed_workspace_refused\": %d", Refuses([&] { arena.CommitWorkspace(); }));
  std::printf("}\n");
  return 0;
}

// src/pipeline/pipeline.cpp:134-136 and :532-534, evaluated with the reference's own
// StaticArenaManager::num_blocks().
int Stats(int64_t block_size, int64_t max_context, int64_t position) {
  RuntimeConfig config;
  config.block_size = block_size;
  config.max_context_len = max_context;
  SimulatedDeviceOps device(1ull << 20);
  int64_t num_blocks = -1;
  const bool refused = Refuses([&] {
    StaticArenaManager manager(device, device, config);
    num_blocks = manager.num_blocks();
  });
  if (refused) {
    std::printf("{\"refused\": true}\n");
    return 0;
  }
  const double utilization = static_cast<double>(position + 1) / static_cast<double>(num_blocks * config.block_size);
  std::printf("{\"refused\": false, \"num_blocks\": %" PRId64 ", \"total_blocks_allocated\": %" PRId64
              ", \"active_context_tokens\": %" PRId64 ", \"kv_cache_utilization\": %.17g}\n",
              num_blocks, num_blocks * kNumLayers, position + 1, utilization);
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    if (argc >= 4 && std::strcmp(argv[1], "ledger") == 0) return Ledger(std::atoll(argv[2]), std::atoll(argv[3]));
    if (argc >= 3 && std::strcmp(argv[1], "arena-script") == 0 && argc == 3 + std::atoi(argv[2])) return ArenaScript(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "arena-contract") == 0) return ArenaContract();
    if (argc >= 5 && std::strcmp(argv[1], "stats") == 0) return Stats(std::atoll(argv[2]), std::atoll(argv[3]), std::atoll(argv[4]));
  } catch (const std::exception& error) {
    std::fprintf(stderr, "ref_kv_probe: %s\n", error.what());
    return 1;
  }
  std::fprintf(stderr, "usage: ref_kv_probe ledger|arena-script|arena-contract|stats ...\n");
  return 2;
}
