// Host-side foundation of the MI355X paged MLA KV-cache path: error type, geometry
// constants and the device backend contract.
//
// Mirrors, for this path only, the reference engine's
//   include/moe/core/error.hpp:38-77          (Dsv4Error / DSV4_REQUIRE  -> KvError / MOE_HIP_REQUIRE)
//   include/moe/core/config.hpp:38-51, :78-109, :237   (topology, MlaGeometry, arena alignment)
//   include/moe/core/device_allocator.hpp:32-60        (IDeviceAllocator)
//   include/moe/core/stream_engine.hpp:35-56           (the ordered-copy part of IStreamEngine)
#pragma once

#include <cstddef>
#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>

namespace moe_hip {

class KvError : public std::runtime_error {
 public:
  explicit KvError(const std::string& message) : std::runtime_error(message) {}
};

#define MOE_HIP_REQUIRE(condition, message)                                                      \
  do {                                                                                           \
    if (!(condition)) {                                                                          \
      std::ostringstream moe_hip_msg_;                                                           \
      moe_hip_msg_ << message << " [" << #condition << " at " << __FILE__ << ":" << __LINE__ << "]"; \
      throw ::moe_hip::KvError(moe_hip_msg_.str());                                              \
    }                                                                                            \
  } while (false)

// Topology constants of the model the reference serves.
inline constexpr int64_t kNumLayers = 43;
inline constexpr int64_t kNumAttentionHeads = 64;
inline constexpr int64_t kDefaultKvLoraRank = 512;
inline constexpr int64_t kDefaultQkRopeHeadDim = 64;
inline constexpr int64_t kDefaultQkNopeHeadDim = 128;
inline constexpr size_t kArenaAlignBytes = 512;
inline constexpr size_t kDeviceAllocAlignBytes = 4096;

struct MlaGeometry {
  int64_t kv_lora_rank = kDefaultKvLoraRank;
  int64_t qk_rope_head_dim = kDefaultQkRopeHeadDim;
  int64_t qk_nope_head_dim = kDefaultQkNopeHeadDim;
  int64_t kv_row_elements() const { return kv_lora_rank + qk_rope_head_dim; }
  int64_t q_head_dim() const { return qk_nope_head_dim + qk_rope_head_dim; }
};

size_t AlignUp(size_t value, size_t alignment);
int64_t DivideUp(int64_t value, int64_t divisor);

enum class CopyKind { kHostToDevice, kDeviceToHost, kDeviceToDevice };

// What the arena and the KV cache manager need from a device: memory, a fill, an
// allocation counter (the zero-allocation-per-step invariant is enforced by watching it)
// and stream-ordered copies for the per-step metadata.
class IDeviceBackend {
 public:
  virtual ~IDeviceBackend() = default;
  virtual void* DeviceMalloc(size_t bytes) = 0;
  virtual void DeviceFree(void* pointer) = 0;
  virtual void* HostPinnedMalloc(size_t bytes) = 0;
  virtual void HostPinnedFree(void* pointer) = 0;
  virtual void DeviceMemset(void* pointer, size_t capacity, int value, size_t count) = 0;
  virtual uint64_t DeviceAllocationCount() const = 0;
  virtual bool QueryDeviceMemory(size_t* free_bytes, size_t* total_bytes) = 0;
  virtual void MemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count,
                           CopyKind kind, void* stream) = 0;
  virtual void SynchronizeStream(void* stream) = 0;
  // Events order the reuse of pinned staging buffers behind the copies that read them.
  virtual void* CreateEvent() = 0;
  virtual void DestroyEvent(void* event) = 0;
  virtual void RecordEvent(void* event, void* stream) = 0;
  virtual void SynchronizeEvent(void* event) = 0;
  // True when kernels can run on memory from this backend.
  virtual bool runs_kernels() const = 0;
  virtual const char* backend_name() const = 0;
};

// hipMalloc / hipHostMalloc / hipMemcpyAsync on the current device.
class HipDeviceBackend final : public IDeviceBackend {
 public:
  HipDeviceBackend();
  void* DeviceMalloc(size_t bytes) override;
  void DeviceFree(void* pointer) override;
  void* HostPinnedMalloc(size_t bytes) override;
  void HostPinnedFree(void* pointer) override;
  void DeviceMemset(void* pointer, size_t capacity, int value, size_t count) override;
  uint64_t DeviceAllocationCount() const override { return allocations_; }
  bool QueryDeviceMemory(size_t* free_bytes, size_t* total_bytes) override;
  void MemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count, CopyKind kind,
                   void* stream) override;
  void SynchronizeStream(void* stream) override;
  void* CreateEvent() override;
  void DestroyEvent(void* event) override;
  void RecordEvent(void* event, void* stream) override;
  void SynchronizeEvent(void* event) override;
  bool runs_kernels() const override { return true; }
  const char* backend_name() const override { return "hip"; }

 private:
  uint64_t allocations_ = 0;
};

// 4096-aligned host memory and immediate copies: the counterpart of the reference's
// SimulatedDeviceOps (src/core/device_ops.cpp:268-440). It lets the arena, the block pool
// and the descriptor plumbing be exercised on a machine without a GPU. No kernel ever
// runs on it: every launch entry point refuses memory it cannot reach from the device.
class HostDeviceBackend final : public IDeviceBackend {
 public:
  void* DeviceMalloc(size_t bytes) override;
  void DeviceFree(void* pointer) override;
  void* HostPinnedMalloc(size_t bytes) override;
  void HostPinnedFree(void* pointer) override;
  void DeviceMemset(void* pointer, size_t capacity, int value, size_t count) override;
  uint64_t DeviceAllocationCount() const override { return allocations_; }
  bool QueryDeviceMemory(size_t* free_bytes, size_t* total_bytes) override;
  void MemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count, CopyKind kind,
                   void* stream) override;
  void SynchronizeStream(void* stream) override;
  void* CreateEvent() override;
  void DestroyEvent(void* event) override;
  void RecordEvent(void* event, void* stream) override;
  void SynchronizeEvent(void* event) override;
  bool runs_kernels() const override { return false; }
  const char* backend_name() const override { return "host"; }

 private:
  uint64_t allocations_ = 0;
};

}  // namespace moe_hip
