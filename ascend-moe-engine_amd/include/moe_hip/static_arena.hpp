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
  size_t reserved_bytes() const { return cursor_; }

  void Commit();
  bool committed() const { return arena_ != nullptr; }
  void* Address(ArenaHandle handle) const;
  template <typename T>
  T* AddressAs(ArenaHandle handle) const {
    return static_cast<T*>(Address(handle));
  }
  size_t Bytes(ArenaHandle handle) const;
  size_t Offset(ArenaHandle handle) const;

  void NoteWorkspace(uint64_t bytes);
  void CommitWorkspace();
  void* workspace() const { return workspace_; }
  uint64_t workspace_bytes() const { return workspace_bytes_; }
  void AssertWorkspaceFits(uint64_t bytes, const char* what) const;

  void Seal();
  bool sealed() const { return sealed_; }

  const std::vector<ArenaReservation>& reservations() const { return reservations_; }
  size_t arena_bytes() const { return arena_bytes_; }
  const void* arena_base() const { return arena_; }
  IDeviceBackend& backend() const { return backend_; }

  void ValidateAlignment() const;
  std::string DescribeLedger() const;

 private:
  void RefuseIfSealed(const char* what) const;
  void RequireCommitted(const char* what) const;

  IDeviceBackend& backend_;
  std::vector<ArenaReservation> reservations_;
  size_t cursor_ = 0;
  void* arena_ = nullptr;
  size_t arena_bytes_ = 0;
  void* workspace_ = nullptr;
  uint64_t workspace_bytes_ = 0;
  uint64_t workspace_high_water_ = 0;
  bool sealed_ = false;
};

}  // namespace moe_hip
