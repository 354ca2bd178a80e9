// Device backends: HIP (hipMalloc / pinned host / stream-ordered copies) and plain host memory.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>

#include "moe_hip/core.hpp"

namespace moe_hip {

size_t AlignUp(size_t value, size_t alignment) { return (value + alignment - 1) & ~(alignment - 1); }
int64_t DivideUp(int64_t value, int64_t divisor) { return (value + divisor - 1) / divisor; }

namespace {
void CheckHip(hipError_t status, const char* call) {
  if (status != hipSuccess) {
    throw KvError(std::string(call) + " failed: " + hipGetErrorString(status));
  }
}
#define MOE_HIP_CHECK(expr) CheckHip((expr), #expr)

hipMemcpyKind ToHip(CopyKind kind) {
  switch (kind) {
    case CopyKind::kHostToDevice:
      return hipMemcpyHostToDevice;
    case CopyKind::kDeviceToHost:
      return hipMemcpyDeviceToHost;
    default:
      return hipMemcpyDeviceToDevice;
  }
}
}  // namespace

// ---- HIP ------------------------------------------------------------------------

HipDeviceBackend::HipDeviceBackend() {
  int count = 0;
  const hipError_t status = hipGetDeviceCount(&count);
  MOE_HIP_REQUIRE(status == hipSuccess && count > 0,
                  "no HIP device is visible; the HIP backend cannot be created (status " << static_cast<int>(status) << ")");
}

void* HipDeviceBackend::DeviceMalloc(size_t bytes) {
  MOE_HIP_REQUIRE(bytes > 0, "zero-byte device allocation");
  void* pointer = nullptr;
  MOE_HIP_CHECK(hipMalloc(&pointer, bytes));
  ++allocations_;
  return pointer;
}

void HipDeviceBackend::DeviceFree(void* pointer) {
  if (pointer != nullptr) (void)hipFree(pointer);
}

void* HipDeviceBackend::HostPinnedMalloc(size_t bytes) {
  MOE_HIP_REQUIRE(bytes > 0, "zero-byte pinned allocation");
  void* pointer = nullptr;
  MOE_HIP_CHECK(hipHostMalloc(&pointer, bytes, hipHostMallocDefault));
  return pointer;
}

void HipDeviceBackend::HostPinnedFree(void* pointer) {
  if (pointer != nullptr) (void)hipHostFree(pointer);
}

void HipDeviceBackend::DeviceMemset(void* pointer, size_t capacity, int value, size_t count) {
  MOE_HIP_REQUIRE(count <= capacity, "memset of " << count << " bytes into " << capacity);
  MOE_HIP_CHECK(hipMemset(pointer, value, count));
  MOE_HIP_CHECK(hipDeviceSynchronize());
}

bool HipDeviceBackend::QueryDeviceMemory(size_t* free_bytes, size_t* total_bytes) {
  return hipMemGetInfo(free_bytes, total_bytes) == hipSuccess;
}

void HipDeviceBackend::MemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count,
                                   CopyKind kind, void* stream) {
  MOE_HIP_REQUIRE(count <= destination_capacity, "copy of " << count << " bytes into " << destination_capacity);
  if (count == 0) return;
  MOE_HIP_CHECK(hipMemcpyAsync(destination, source, count, ToHip(kind), static_cast<hipStream_t>(stream)));
}

void HipDeviceBackend::SynchronizeStream(void* stream) {
  MOE_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

void* HipDeviceBackend::CreateEvent() {
  hipEvent_t event = nullptr;
  MOE_HIP_CHECK(hipEventCreateWithFlags(&event, hipEventDisableTiming));
  return event;
}

void HipDeviceBackend::DestroyEvent(void* event) {
  if (event != nullptr) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}

void HipDeviceBackend::RecordEvent(void* event, void* stream) {
  MOE_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}

void HipDeviceBackend::SynchronizeEvent(void* event) {
  MOE_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}

// ---- host -------------------------------------------------------------------------

void* HostDeviceBackend::DeviceMalloc(size_t bytes) {
  MOE_HIP_REQUIRE(bytes > 0, "zero-byte device allocation");
  void* pointer = std::aligned_alloc(kDeviceAllocAlignBytes, AlignUp(bytes, kDeviceAllocAlignBytes));
  MOE_HIP_REQUIRE(pointer != nullptr, "host backend could not allocate " << bytes << " bytes");
  ++allocations_;
  return pointer;
}

void HostDeviceBackend::DeviceFree(void* pointer) { std::free(pointer); }

void* HostDeviceBackend::HostPinnedMalloc(size_t bytes) {
  MOE_HIP_REQUIRE(bytes > 0, "zero-byte pinned allocation");
  void* pointer = std::aligned_alloc(kDeviceAllocAlignBytes, AlignUp(bytes, kDeviceAllocAlignBytes));
  MOE_HIP_REQUIRE(pointer != nullptr, "host backend could not allocate " << bytes << " bytes");
  return pointer;
}

void HostDeviceBackend::HostPinnedFree(void* pointer) { std::free(pointer); }

void HostDeviceBackend::DeviceMemset(void* pointer, size_t capacity, int value, size_t count) {
  MOE_HIP_REQUIRE(count <= capacity, "memset of " << count << " bytes into " << capacity);
  std::memset(pointer, value, count);
}

bool HostDeviceBackend::QueryDeviceMemory(size_t*, size_t*) { return false; }

void HostDeviceBackend::MemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count,
                                    CopyKind, void*) {
  MOE_HIP_REQUIRE(count <= destination_capacity, "copy of " << count << " bytes into " << destination_capacity);
  std::memcpy(destination, source, count);
}

void HostDeviceBackend::SynchronizeStream(void*) {}
void* HostDeviceBackend::CreateEvent() { return this; }
void HostDeviceBackend::DestroyEvent(void*) {}
void HostDeviceBackend::RecordEvent(void*, void*) {}
void HostDeviceBackend::SynchronizeEvent(void*) {}

}  // namespace moe_hip
