// Three-phase single-allocation device arena (RESERVE -> BUILD -> SEALED).
//
// Same public calls, ordering rules and refusals as the reference's StaticMemoryArena
// (include/moe/memory/static_arena.hpp:79-181; src/memory/static_arena.cpp):
//   Reserve            :88-102   bump offset = AlignUp(cursor, align); refused when sealed,
//                                committed, empty, or align not a power of two
//   Commit             :108-118  ONE DeviceMalloc of AlignUp(cursor, 512), zero-fill, validate
//   Address / Bytes    :120-129
//   NoteWorkspace / CommitWorkspace / AssertWorkspaceFits   :270-295  shared workspace sized by
//                                the high-water mark over every planned operator
//   Seal               :301-304  one-way latch
//   ValidateAlignment  :310-332
//   DescribeLedger     :334-348
// The descriptor factory of the reference class (aclCreateTensor and friends) lives with
// the operator shim, not here: this arena only owns memory.
#pragma once

#include <string>
#include <vector>

#include "moe_hip/core.hpp"

namespace moe_hip {

using ArenaHandle = size_t;
inline constexpr ArenaHandle kInvalidArenaHandle = static_cast<ArenaHandle>(-1);

struct ArenaReservation {
  std::string name;
  size_t offset = 0;
  size_t bytes = 0;
  size_t align = kArenaAlignBytes;
};

class StaticMemoryArena {
 public:
  explicit StaticMemoryArena(IDeviceBackend& backend);
  ~StaticMemoryArena();
  StaticMemoryArena(const StaticMemoryArena&) = delete;
  StaticMemoryArena& operator=(const StaticMemoryArena&) = delete;

  ArenaHandle Reserve(const char* name, size_t bytes, size_t align = kArenaAlignBytes);
  size_t reserved_bytes() const { return next_offset_; }

  void Commit();
  bool committed() const { return phase_ != Phase::kReserve; }
  void* Address(ArenaHandle handle) const;
  template <typename T>
  T* AddressAs(ArenaHandle handle) const {
    return static_cast<T*>(Address(handle));
  }
  size_t Bytes(ArenaHandle handle) const;
  size_t Offset(ArenaHandle handle) const;

  void NoteWorkspace(uint64_t bytes);
  void CommitWorkspace();
  void* workspace() const { return scratch_.base; }
  uint64_t workspace_bytes() const { return scratch_.bytes; }
  void AssertWorkspaceFits(uint64_t bytes, const char* what) const;

  void Seal();
  bool sealed() const { return phase_ == Phase::kSealed; }

  const std::vector<ArenaReservation>& reservations() const { return ledger_; }
  size_t arena_bytes() const { return pool_.bytes; }
  const void* arena_base() const { return pool_.base; }
  IDeviceBackend& backend() const { return backend_; }

  void ValidateAlignment() const;
  std::string DescribeLedger() const;

 private:
  // RESERVE until Commit, BUILD until Seal, SEALED for good: one value instead of a latch per edge.
  enum class Phase { kReserve, kBuild, kSealed };
  // One device allocation owned by the arena.
  struct Block {
    void* base = nullptr;
    size_t bytes = 0;
  };
  void CheckNotSealed(const char* call) const;  // throws in Phase::kSealed
  void CheckBuilt(const char* call) const;      // throws in Phase::kReserve
  const ArenaReservation& Entry(ArenaHandle handle) const;

  IDeviceBackend& backend_;
  Phase phase_ = Phase::kReserve;
  std::vector<ArenaReservation> ledger_;  // in request order; a handle is an index into it
  size_t next_offset_ = 0;                // where the next reservation would start, before alignment
  Block pool_;                            // what Commit allocated
  Block scratch_;                         // the operators' shared workspace (CommitWorkspace)
  uint64_t scratch_wanted_ = 0;           // largest NoteWorkspace so far
};

}  // namespace moe_hip
