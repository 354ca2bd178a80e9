// The aclnn-compatible half of the C ABI (include/aclnn_hip.h): descriptor engine, aclrt
// runtime over HIP, and the two-phase operators of the KV-cache path. Operators validate the
// plan-time contract, capture their arguments in IR order and, at launch, hand plain pointers
// and strides to the thin kernel ABI (include/mlakv.h).
#include "aclnn_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_set>
#include <vector>

#include "../kernels/kernels.h"
#include "abi_common.h"
#include "mlakv.h"

using mlakv_abi::Fail;

namespace {

// ---- handle registry -------------------------------------------------------------------
// Every descriptor handed out is remembered, so a stale or foreign pointer is answered with
// a status instead of being dereferenced.
std::mutex g_registry_mutex;
std::unordered_set<const void*> g_live;

void Register(const void* handle) {
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  g_live.insert(handle);
}
bool Unregister(const void* handle) {
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  return g_live.erase(handle) != 0;
}
bool IsLive(const void* handle) {
  if (handle == nullptr) return false;
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  return g_live.count(handle) != 0;
}

size_t ElementBytes(aclDataType dtype) {
  switch (dtype) {
    case ACL_FLOAT32: case ACL_INT32: return 4;
    case ACL_FLOAT16: case ACL_BF16: case ACL_INT16: case ACL_UINT16: return 2;
    case ACL_INT64: case ACL_UINT64: case ACL_FLOAT64: return 8;
    case ACL_INT8: case ACL_UINT8: case ACL_BOOL: case ACL_FLOAT8_E5M2: case ACL_FLOAT8_E4M3FN: case ACL_FLOAT8_E8M0:
    case ACL_FP4X2_E2M1: return 1;
    default: return 0;
  }
}

}  // namespace

struct aclTensor {
  std::vector<int64_t> dims, strides, storage;
  int64_t offset = 0;
  aclDataType dtype = ACL_DT_UNDEFINED;
  aclFormat format = ACL_FORMAT_ND;
  void* data = nullptr;
  int64_t numel() const {
    int64_t n = 1;
    for (int64_t d : dims) n *= d;
    return n;
  }
  bool contiguous() const {
    int64_t expected = 1;
    for (size_t i = dims.size(); i-- > 0;) {
      if (dims[i] != 1 && strides[i] != expected) return false;
      expected *= dims[i];
    }
    return true;
  }
};
struct aclTensorList { std::vector<aclTensor*> items; };
// The values are copied at creation, as the reference's own implementation of the call does
// (mock/mock_descriptor.cpp:249-256): callers build arrays from temporaries.
struct aclIntArray { std::vector<int64_t> storage; const int64_t* values = nullptr; uint64_t size = 0; };
struct aclScalar { void* value = nullptr; aclDataType dtype = ACL_DT_UNDEFINED; };

namespace {

enum class OpKind { kScatter, kAttention, kGather, kMxQuant, kIndexer };
enum class SlotKind { kNull, kTensor, kList, kIntArray };

struct Slot {
  SlotKind kind = SlotKind::kNull;
  const void* handle = nullptr;
  std::vector<void*> addresses;  // one per tensor (lists: one per item), view offset applied
};

void* EffectiveAddress(const aclTensor* t, void* base) {
  return base == nullptr ? nullptr : static_cast<char*>(base) + t->offset * static_cast<int64_t>(ElementBytes(t->dtype));
}

Slot TensorSlot(const aclTensor* t) {
  Slot s;
  if (t == nullptr) return s;
  s.kind = SlotKind::kTensor;
  s.handle = t;
  s.addresses.push_back(EffectiveAddress(t, t->data));
  return s;
}
Slot ListSlot(const aclTensorList* l) {
  Slot s;
  if (l == nullptr) return s;
  s.kind = SlotKind::kList;
  s.handle = l;
  for (const aclTensor* t : l->items) s.addresses.push_back(EffectiveAddress(t, t->data));
  return s;
}
Slot ArraySlot(const aclIntArray* a) {
  Slot s;
  if (a == nullptr) return s;
  s.kind = SlotKind::kIntArray;
  s.handle = a;
  return s;
}

}  // namespace

struct aclOpExecutor {
  OpKind kind;
  bool repeatable = false;
  bool launched = false;
  std::vector<Slot> slots;  // IR order
  // scatter / gather / attention geometry frozen at plan time
  int32_t tokens = 0, heads = 0, num_blocks = 0, block_size = 0, table_width = 0, batch = 0, max_seq_len = 0;
  int64_t key_row_stride = 0, value_row_stride = 0;                  // bytes, token rows outside the cache
  int64_t key_block_stride = 0, key_slot_stride = 0;                 // bytes, latent plane
  int64_t value_block_stride = 0, value_slot_stride = 0;             // bytes, rope plane
  int64_t q_token_stride = 0, q_head_stride = 0, qr_token_stride = 0, qr_head_stride = 0;
  int64_t out_token_stride = 0, out_head_stride = 0;
  double scale = 0.0;
  bool want_lse = false;
  mlakvAttnPlan plan{};
  int64_t aux_stride[4] = {0, 0, 0, 0};  // indexer: weights / query scale / key scale block / output strides
  int32_t sparse_count = 0;
  uint64_t workspace_bytes = 0;
  uint64_t lens_offset = 0;  // attention: where the int32 lengths live inside the workspace
  const int32_t* bound_lens = nullptr;
  int32_t bound_longest = -1;  // the caller's word for the longest of the bound lengths; -1: none given
  std::vector<int32_t> host_lens;  // plan-time kv lengths, or those of the latest aclnnMlaKvSetSeqLens
};

namespace {

const aclTensor* AsTensor(const aclTensor* t) { return IsLive(t) ? t : nullptr; }
const aclTensorList* AsList(const aclTensorList* l) { return IsLive(l) ? l : nullptr; }
const aclIntArray* AsArray(const aclIntArray* a) { return IsLive(a) ? a : nullptr; }
aclOpExecutor* AsExecutor(aclOpExecutor* e) { return IsLive(e) ? e : nullptr; }

aclError RtFail(hipError_t status, const char* who) {
  Fail(ACL_ERROR_RT_FAILURE, "%s: %s", who, hipGetErrorString(status));
  return ACL_ERROR_RT_FAILURE;
}

#define SHIM_REQUIRE(cond, code, ...) \
  do {                                \
    if (!(cond)) return Fail(code, __VA_ARGS__); \
  } while (false)

// A paged cache descriptor [blocks, block, 1, dim] (or [blocks, block, dim]) whose rows are dense.
bool PagedCacheShape(const aclTensor* t, int64_t dim, int64_t* blocks, int64_t* block_size, int64_t* block_stride,
                     int64_t* slot_stride) {
  const size_t n = t->dims.size();
  if (n != 3 && n != 4) return false;
  if (t->dims[n - 1] != dim || t->strides[n - 1] != 1) return false;
  if (n == 4 && t->dims[2] != 1) return false;
  *blocks = t->dims[0];
  *block_size = t->dims[1];
  *block_stride = t->strides[0];
  *slot_stride = t->strides[1];
  return *blocks > 0 && *block_size > 0 && *slot_stride >= dim && *block_stride >= *slot_stride * *block_size;
}

// Token rows [T, dim] or [T, 1, dim] with a dense last axis.
bool TokenRows(const aclTensor* t, int64_t dim, int64_t* tokens, int64_t* row_stride) {
  const size_t n = t->dims.size();
  if (n != 2 && n != 3) return false;
  if (t->dims[n - 1] != dim || t->strides[n - 1] != 1) return false;
  if (n == 3 && t->dims[1] != 1) return false;
  *tokens = t->dims[0];
  *row_stride = t->strides[0];
  return *tokens > 0 && (*row_stride >= dim || *tokens == 1);
}

aclOpExecutor* NewExecutor(OpKind kind, std::vector<Slot> slots) {
  auto* executor = new aclOpExecutor();
  executor->kind = kind;
  executor->slots = std::move(slots);
  Register(executor);
  return executor;
}

}  // namespace

extern "C" {

// ---- runtime ------------------------------------------------------------------------------

aclError aclInit(const char*) { return ACL_SUCCESS; }
aclError aclFinalize(void) { return ACL_SUCCESS; }
aclnnStatus aclnnInit(const char*) { return ACLNN_SUCCESS; }
aclnnStatus aclnnFinalize(void) { return ACLNN_SUCCESS; }
const char* aclGetRecentErrMsg(void) { return mlakv_abi::LastError(); }

aclError aclrtSetDevice(int32_t device_id) {
  const hipError_t status = hipSetDevice(device_id);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtSetDevice");
}
aclError aclrtResetDevice(int32_t device_id) {
  // The HIP primary context is shared with every other user of the device in this process
  // (for one, the framework that owns the caller's tensors); draining is the safe equivalent.
  if (hipSetDevice(device_id) != hipSuccess) return Fail(ACL_ERROR_INVALID_PARAM, "aclrtResetDevice: no device %d", device_id);
  const hipError_t status = hipDeviceSynchronize();
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtResetDevice");
}
aclError aclrtCreateContext(aclrtContext* context, int32_t device_id) {
  SHIM_REQUIRE(context != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtCreateContext: null output");
  const hipError_t status = hipSetDevice(device_id);
  if (status != hipSuccess) return RtFail(status, "aclrtCreateContext");
  *context = reinterpret_cast<aclrtContext>(static_cast<intptr_t>(device_id) + 1);  // HIP uses the primary context
  return ACL_SUCCESS;
}
aclError aclrtDestroyContext(aclrtContext) { return ACL_SUCCESS; }
aclError aclrtSetCurrentContext(aclrtContext context) {
  SHIM_REQUIRE(context != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtSetCurrentContext: null context");
  const hipError_t status = hipSetDevice(static_cast<int>(reinterpret_cast<intptr_t>(context)) - 1);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtSetCurrentContext");
}
aclError aclrtGetDeviceCount(uint32_t* device_count) {
  SHIM_REQUIRE(device_count != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtGetDeviceCount: null output");
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess) count = 0;
  *device_count = static_cast<uint32_t>(count);
  return ACL_SUCCESS;
}
const char* aclrtGetSocName(void) {
  static const std::string name = [] {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess) {
      std::string arch = prop.gcnArchName;
      return arch.substr(0, arch.find(':'));
    }
    return std::string("gfx950");
  }();
  return name.c_str();
}

aclError aclrtMalloc(void** device_ptr, size_t size, aclrtMemMallocPolicy) {
  SHIM_REQUIRE(device_ptr != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtMalloc: null output");
  SHIM_REQUIRE(size > 0, ACL_ERROR_INVALID_PARAM, "aclrtMalloc: zero bytes");
  const hipError_t status = hipMalloc(device_ptr, size);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtMalloc");
}
aclError aclrtFree(void* device_ptr) {
  const hipError_t status = hipFree(device_ptr);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtFree");
}
aclError aclrtMallocHost(void** host_ptr, size_t size) {
  SHIM_REQUIRE(host_ptr != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtMallocHost: null output");
  SHIM_REQUIRE(size > 0, ACL_ERROR_INVALID_PARAM, "aclrtMallocHost: zero bytes");
  const hipError_t status = hipHostMalloc(host_ptr, size, hipHostMallocDefault);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtMallocHost");
}
aclError aclrtFreeHost(void* host_ptr) {
  const hipError_t status = hipHostFree(host_ptr);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtFreeHost");
}

static hipMemcpyKind ToHipKind(aclrtMemcpyKind kind) {
  switch (kind) {
    case ACL_MEMCPY_HOST_TO_HOST: return hipMemcpyHostToHost;
    case ACL_MEMCPY_HOST_TO_DEVICE: return hipMemcpyHostToDevice;
    case ACL_MEMCPY_DEVICE_TO_HOST: return hipMemcpyDeviceToHost;
    default: return hipMemcpyDeviceToDevice;
  }
}

aclError aclrtMemcpy(void* destination, size_t destination_capacity, const void* source, size_t count, aclrtMemcpyKind kind) {
  SHIM_REQUIRE(destination != nullptr && source != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtMemcpy: null pointer");
  SHIM_REQUIRE(count <= destination_capacity, ACL_ERROR_INVALID_PARAM, "aclrtMemcpy: %zu bytes into %zu", count, destination_capacity);
  if (count == 0) return ACL_SUCCESS;
  const hipError_t status = hipMemcpy(destination, source, count, ToHipKind(kind));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtMemcpy");
}
aclError aclrtMemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count,
                          aclrtMemcpyKind kind, aclrtStream stream) {
  SHIM_REQUIRE(destination != nullptr && source != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtMemcpyAsync: null pointer");
  SHIM_REQUIRE(count <= destination_capacity, ACL_ERROR_INVALID_PARAM, "aclrtMemcpyAsync: %zu bytes into %zu", count, destination_capacity);
  if (count == 0) return ACL_SUCCESS;
  const hipError_t status = hipMemcpyAsync(destination, source, count, ToHipKind(kind), static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtMemcpyAsync");
}
aclError aclrtMemset(void* destination, size_t destination_capacity, int32_t value, size_t count) {
  SHIM_REQUIRE(destination != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtMemset: null pointer");
  SHIM_REQUIRE(count <= destination_capacity, ACL_ERROR_INVALID_PARAM, "aclrtMemset: %zu bytes into %zu", count, destination_capacity);
  hipError_t status = hipMemset(destination, value, count);
  if (status == hipSuccess) status = hipDeviceSynchronize();
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtMemset");
}

aclError aclrtCreateStream(aclrtStream* stream) {
  SHIM_REQUIRE(stream != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtCreateStream: null output");
  hipStream_t s = nullptr;
  const hipError_t status = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
  if (status != hipSuccess) return RtFail(status, "aclrtCreateStream");
  *stream = s;
  return ACL_SUCCESS;
}
aclError aclrtDestroyStream(aclrtStream stream) {
  hipError_t status = hipStreamSynchronize(static_cast<hipStream_t>(stream));
  if (status == hipSuccess) status = hipStreamDestroy(static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtDestroyStream");
}
aclError aclrtDestroyStreamForce(aclrtStream stream) {
  const hipError_t status = hipStreamDestroy(static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtDestroyStreamForce");
}
aclError aclrtCreateEventExWithFlag(aclrtEvent* event, uint32_t) {
  SHIM_REQUIRE(event != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtCreateEventExWithFlag: null output");
  hipEvent_t e = nullptr;
  const hipError_t status = hipEventCreateWithFlags(&e, hipEventDisableTiming);
  if (status != hipSuccess) return RtFail(status, "aclrtCreateEventExWithFlag");
  *event = e;
  return ACL_SUCCESS;
}
aclError aclrtDestroyEvent(aclrtEvent event) {
  const hipError_t status = hipEventDestroy(static_cast<hipEvent_t>(event));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtDestroyEvent");
}
aclError aclrtRecordEvent(aclrtEvent event, aclrtStream stream) {
  const hipError_t status = hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtRecordEvent");
}
aclError aclrtStreamWaitEvent(aclrtStream stream, aclrtEvent event) {
  const hipError_t status = hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtStreamWaitEvent");
}
aclError aclrtSynchronizeStream(aclrtStream stream) {
  const hipError_t status = hipStreamSynchronize(static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtSynchronizeStream");
}
aclError aclrtSynchronizeStreamWithTimeout(aclrtStream stream, int32_t timeout_ms) {
  if (timeout_ms < 0) return aclrtSynchronizeStream(stream);
  const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(timeout_ms);
  for (;;) {
    const hipError_t status = hipStreamQuery(static_cast<hipStream_t>(stream));
    if (status == hipSuccess) return ACL_SUCCESS;
    if (status != hipErrorNotReady) return RtFail(status, "aclrtSynchronizeStreamWithTimeout");
    if (std::chrono::steady_clock::now() >= deadline) {
      return Fail(ACL_ERROR_RT_STREAM_SYNC_TIMEOUT, "aclrtSynchronizeStreamWithTimeout: stream still busy after %d ms", timeout_ms);
    }
    std::this_thread::sleep_for(std::chrono::microseconds(50));
  }
}
aclError aclrtSynchronizeEvent(aclrtEvent event) {
  const hipError_t status = hipEventSynchronize(static_cast<hipEvent_t>(event));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtSynchronizeEvent");
}
aclError aclrtGetMemInfo(aclrtMemAttr, size_t* free_bytes, size_t* total_bytes) {
  SHIM_REQUIRE(free_bytes != nullptr && total_bytes != nullptr, ACL_ERROR_INVALID_PARAM, "aclrtGetMemInfo: null output");
  const hipError_t status = hipMemGetInfo(free_bytes, total_bytes);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclrtGetMemInfo");
}

// ---- stream capture ------------------------------------------------------------------------

aclError aclmdlRICaptureBegin(aclrtStream stream, aclmdlRICaptureMode mode) {
  SHIM_REQUIRE(stream != nullptr, ACL_ERROR_INVALID_PARAM, "aclmdlRICaptureBegin: a stream of its own is needed (not the null stream)");
  hipStreamCaptureMode hip_mode;
  switch (mode) {
    case ACL_MODEL_RI_CAPTURE_MODE_GLOBAL: hip_mode = hipStreamCaptureModeGlobal; break;
    case ACL_MODEL_RI_CAPTURE_MODE_THREAD_LOCAL: hip_mode = hipStreamCaptureModeThreadLocal; break;
    case ACL_MODEL_RI_CAPTURE_MODE_RELAXED: hip_mode = hipStreamCaptureModeRelaxed; break;
    default: return Fail(ACL_ERROR_INVALID_PARAM, "aclmdlRICaptureBegin: unknown capture mode %d", static_cast<int>(mode));
  }
  const hipError_t status = hipStreamBeginCapture(static_cast<hipStream_t>(stream), hip_mode);
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclmdlRICaptureBegin");
}
aclError aclmdlRICaptureEnd(aclrtStream stream, aclmdlRI* model_ri) {
  SHIM_REQUIRE(stream != nullptr && model_ri != nullptr, ACL_ERROR_INVALID_PARAM, "aclmdlRICaptureEnd: null stream or output");
  *model_ri = nullptr;
  hipGraph_t graph = nullptr;
  hipError_t status = hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph);
  if (status != hipSuccess || graph == nullptr) return RtFail(status == hipSuccess ? hipErrorUnknown : status, "aclmdlRICaptureEnd");
  hipGraphExec_t exec = nullptr;
  status = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (status != hipSuccess) return RtFail(status, "aclmdlRICaptureEnd (instantiate)");
  *model_ri = exec;
  return ACL_SUCCESS;
}
aclError aclmdlRIExecuteAsync(aclmdlRI model_ri, aclrtStream stream) {
  SHIM_REQUIRE(model_ri != nullptr, ACL_ERROR_INVALID_PARAM, "aclmdlRIExecuteAsync: null recording");
  const hipError_t status = hipGraphLaunch(static_cast<hipGraphExec_t>(model_ri), static_cast<hipStream_t>(stream));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclmdlRIExecuteAsync");
}
aclError aclmdlRIDestroy(aclmdlRI model_ri) {
  if (model_ri == nullptr) return ACL_SUCCESS;
  const hipError_t status = hipGraphExecDestroy(static_cast<hipGraphExec_t>(model_ri));
  return status == hipSuccess ? ACL_SUCCESS : RtFail(status, "aclmdlRIDestroy");
}

// ---- descriptor engine ------------------------------------------------------------------

aclTensor* aclCreateTensor(const int64_t* view_dims, uint64_t view_dims_num, aclDataType dtype, const int64_t* view_strides,
                           int64_t storage_offset, aclFormat format, const int64_t* storage_dims,
                           uint64_t storage_dims_num, void* device_data) {
  if (view_dims == nullptr || view_dims_num == 0 || view_dims_num > 8 || ElementBytes(dtype) == 0 || storage_offset < 0) {
    Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateTensor: needs 1..8 dims, a known dtype and a non-negative offset");
    return nullptr;
  }
  auto* t = new aclTensor();
  t->dims.assign(view_dims, view_dims + view_dims_num);
  if (view_strides != nullptr) {
    t->strides.assign(view_strides, view_strides + view_dims_num);
  } else {
    t->strides.assign(view_dims_num, 1);
    for (size_t i = view_dims_num; i-- > 1;) t->strides[i - 1] = t->strides[i] * t->dims[i];
  }
  for (uint64_t i = 0; i < view_dims_num; ++i) {
    if (t->dims[i] < 0 || t->strides[i] < 0) {
      delete t;
      Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateTensor: negative dimension or stride");
      return nullptr;
    }
  }
  if (storage_dims != nullptr && storage_dims_num > 0) t->storage.assign(storage_dims, storage_dims + storage_dims_num);
  else t->storage = t->dims;
  t->offset = storage_offset;
  t->dtype = dtype;
  t->format = format;
  t->data = device_data;
  Register(t);
  return t;
}

aclnnStatus aclDestroyTensor(const aclTensor* tensor) {
  if (tensor == nullptr) return ACLNN_SUCCESS;
  SHIM_REQUIRE(Unregister(tensor), ACLNN_ERR_PARAM_INVALID, "aclDestroyTensor: not a live tensor handle");
  delete tensor;
  return ACLNN_SUCCESS;
}

static aclnnStatus CopyOut(const std::vector<int64_t>& values, int64_t** out, uint64_t* count) {
  *out = new int64_t[values.size() ? values.size() : 1];
  for (size_t i = 0; i < values.size(); ++i) (*out)[i] = values[i];
  *count = values.size();
  return ACLNN_SUCCESS;
}
#define SHIM_TENSOR(t, who)                                                                  \
  SHIM_REQUIRE((t) != nullptr, ACLNN_ERR_PARAM_NULLPTR, who ": null tensor");                \
  SHIM_REQUIRE(IsLive(t), ACLNN_ERR_PARAM_INVALID, who ": not a live tensor handle")

aclnnStatus aclGetViewShape(const aclTensor* tensor, int64_t** dims, uint64_t* count) {
  SHIM_TENSOR(tensor, "aclGetViewShape");
  SHIM_REQUIRE(dims && count, ACLNN_ERR_PARAM_NULLPTR, "aclGetViewShape: null output");
  return CopyOut(tensor->dims, dims, count);
}
aclnnStatus aclGetStorageShape(const aclTensor* tensor, int64_t** dims, uint64_t* count) {
  SHIM_TENSOR(tensor, "aclGetStorageShape");
  SHIM_REQUIRE(dims && count, ACLNN_ERR_PARAM_NULLPTR, "aclGetStorageShape: null output");
  return CopyOut(tensor->storage, dims, count);
}
aclnnStatus aclGetViewStrides(const aclTensor* tensor, int64_t** strides, uint64_t* count) {
  SHIM_TENSOR(tensor, "aclGetViewStrides");
  SHIM_REQUIRE(strides && count, ACLNN_ERR_PARAM_NULLPTR, "aclGetViewStrides: null output");
  return CopyOut(tensor->strides, strides, count);
}
aclnnStatus aclGetDataType(const aclTensor* tensor, aclDataType* dtype) {
  SHIM_TENSOR(tensor, "aclGetDataType");
  SHIM_REQUIRE(dtype, ACLNN_ERR_PARAM_NULLPTR, "aclGetDataType: null output");
  *dtype = tensor->dtype;
  return ACLNN_SUCCESS;
}
aclnnStatus aclGetFormat(const aclTensor* tensor, aclFormat* format) {
  SHIM_TENSOR(tensor, "aclGetFormat");
  SHIM_REQUIRE(format, ACLNN_ERR_PARAM_NULLPTR, "aclGetFormat: null output");
  *format = tensor->format;
  return ACLNN_SUCCESS;
}
aclnnStatus aclGetRawTensorAddr(const aclTensor* tensor, void** address) {
  SHIM_TENSOR(tensor, "aclGetRawTensorAddr");
  SHIM_REQUIRE(address, ACLNN_ERR_PARAM_NULLPTR, "aclGetRawTensorAddr: null output");
  *address = tensor->data;
  return ACLNN_SUCCESS;
}
aclnnStatus aclGetViewOffset(const aclTensor* tensor, int64_t* offset) {
  SHIM_TENSOR(tensor, "aclGetViewOffset");
  SHIM_REQUIRE(offset, ACLNN_ERR_PARAM_NULLPTR, "aclGetViewOffset: null output");
  *offset = tensor->offset;
  return ACLNN_SUCCESS;
}

aclTensorList* aclCreateTensorList(const aclTensor* const* tensors, uint64_t size) {
  if (tensors == nullptr || size == 0) {
    Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateTensorList: an empty list");
    return nullptr;
  }
  for (uint64_t i = 0; i < size; ++i) {
    if (!IsLive(tensors[i])) {
      Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateTensorList: item %llu is not a live tensor handle", static_cast<unsigned long long>(i));
      return nullptr;
    }
  }
  auto* list = new aclTensorList();
  for (uint64_t i = 0; i < size; ++i) list->items.push_back(const_cast<aclTensor*>(tensors[i]));
  Register(list);
  return list;
}
aclnnStatus aclDestroyTensorList(const aclTensorList* tensor_list) {
  if (tensor_list == nullptr) return ACLNN_SUCCESS;
  SHIM_REQUIRE(Unregister(tensor_list), ACLNN_ERR_PARAM_INVALID, "aclDestroyTensorList: not a live list handle");
  for (aclTensor* item : tensor_list->items) {  // the list owns its tensors
    if (Unregister(item)) delete item;
  }
  delete tensor_list;
  return ACLNN_SUCCESS;
}

aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size) {
  if (value == nullptr || size == 0) {
    Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateIntArray: an empty array");
    return nullptr;
  }
  auto* array = new aclIntArray();
  array->storage.assign(value, value + size);
  array->values = array->storage.data();
  array->size = size;
  Register(array);
  return array;
}
aclnnStatus aclDestroyIntArray(const aclIntArray* array) {
  if (array == nullptr) return ACLNN_SUCCESS;
  SHIM_REQUIRE(Unregister(array), ACLNN_ERR_PARAM_INVALID, "aclDestroyIntArray: not a live array handle");
  delete array;
  return ACLNN_SUCCESS;
}
aclScalar* aclCreateScalar(void* value, aclDataType dtype) {
  if (value == nullptr || ElementBytes(dtype) == 0) {
    Fail(ACLNN_ERR_PARAM_INVALID, "aclCreateScalar: null value or unknown dtype");
    return nullptr;
  }
  auto* scalar = new aclScalar();
  scalar->value = value;
  scalar->dtype = dtype;
  Register(scalar);
  return scalar;
}
aclnnStatus aclDestroyScalar(const aclScalar* scalar) {
  if (scalar == nullptr) return ACLNN_SUCCESS;
  SHIM_REQUIRE(Unregister(scalar), ACLNN_ERR_PARAM_INVALID, "aclDestroyScalar: not a live scalar handle");
  delete scalar;
  return ACLNN_SUCCESS;
}

aclnnStatus aclSetTensorAddr(aclOpExecutor* executor, uint64_t index, const aclTensor* tensor, void* address) {
  SHIM_REQUIRE(executor && tensor && address, ACLNN_ERR_PARAM_NULLPTR, "aclSetTensorAddr: null argument");
  SHIM_REQUIRE(AsExecutor(executor), ACLNN_ERR_PARAM_INVALID, "aclSetTensorAddr: not a live executor");
  SHIM_REQUIRE(AsTensor(tensor), ACLNN_ERR_PARAM_INVALID, "aclSetTensorAddr: not a live tensor handle");
  SHIM_REQUIRE(index < executor->slots.size(), ACLNN_ERR_PARAM_INVALID, "aclSetTensorAddr: IR index %llu outside the %zu captured arguments",
               static_cast<unsigned long long>(index), executor->slots.size());
  Slot& slot = executor->slots[index];
  SHIM_REQUIRE(slot.kind == SlotKind::kTensor, ACLNN_ERR_PARAM_INVALID,
               "aclSetTensorAddr: IR index %llu was bound as %s at plan time", static_cast<unsigned long long>(index),
               slot.kind == SlotKind::kNull ? "null" : "a list or array");
  const aclTensor* planned = static_cast<const aclTensor*>(slot.handle);
  SHIM_REQUIRE(planned == tensor || (planned->dims == tensor->dims && planned->dtype == tensor->dtype && planned->strides == tensor->strides),
               ACLNN_ERR_PARAM_INVALID, "aclSetTensorAddr: the tensor does not match the one planned at IR index %llu (shape, dtype and strides are frozen)",
               static_cast<unsigned long long>(index));
  slot.addresses[0] = EffectiveAddress(planned, address);
  return ACLNN_SUCCESS;
}

aclnnStatus aclSetDynamicTensorAddr(aclOpExecutor* executor, uint64_t ir_index, uint64_t relative_index,
                                    const aclTensorList* tensor_list, void* address) {
  SHIM_REQUIRE(executor && tensor_list && address, ACLNN_ERR_PARAM_NULLPTR, "aclSetDynamicTensorAddr: null argument");
  SHIM_REQUIRE(AsExecutor(executor), ACLNN_ERR_PARAM_INVALID, "aclSetDynamicTensorAddr: not a live executor");
  SHIM_REQUIRE(AsList(tensor_list), ACLNN_ERR_PARAM_INVALID, "aclSetDynamicTensorAddr: not a live list handle");
  SHIM_REQUIRE(ir_index < executor->slots.size(), ACLNN_ERR_PARAM_INVALID, "aclSetDynamicTensorAddr: IR index %llu outside the %zu captured arguments",
               static_cast<unsigned long long>(ir_index), executor->slots.size());
  Slot& slot = executor->slots[ir_index];
  SHIM_REQUIRE(slot.kind == SlotKind::kList && slot.handle == tensor_list, ACLNN_ERR_PARAM_INVALID,
               "aclSetDynamicTensorAddr: IR index %llu does not hold this tensor list", static_cast<unsigned long long>(ir_index));
  SHIM_REQUIRE(relative_index < slot.addresses.size(), ACLNN_ERR_PARAM_INVALID, "aclSetDynamicTensorAddr: item %llu of a %zu-item list",
               static_cast<unsigned long long>(relative_index), slot.addresses.size());
  slot.addresses[relative_index] = EffectiveAddress(tensor_list->items[relative_index], address);
  return ACLNN_SUCCESS;
}

aclnnStatus aclSetAclOpExecutorRepeatable(aclOpExecutor* executor) {
  SHIM_REQUIRE(executor, ACLNN_ERR_PARAM_NULLPTR, "aclSetAclOpExecutorRepeatable: null executor");
  SHIM_REQUIRE(AsExecutor(executor), ACLNN_ERR_PARAM_INVALID, "aclSetAclOpExecutorRepeatable: not a live executor");
  executor->repeatable = true;
  return ACLNN_SUCCESS;
}
aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor) {
  if (executor == nullptr) return ACLNN_SUCCESS;
  SHIM_REQUIRE(Unregister(executor), ACLNN_ERR_PARAM_INVALID, "aclDestroyAclOpExecutor: not a live executor");
  delete executor;
  return ACLNN_SUCCESS;
}

// ---- aclnnScatterPaKvCache -----------------------------------------------------------------

aclnnStatus aclnnScatterPaKvCacheGetWorkspaceSize(const aclTensor* key, aclTensor* key_cache_ref, const aclTensor* slot_mapping,
                                                  const aclTensor* value, aclTensor* value_cache_ref,
                                                  const aclTensor* compress_lens_optional,
                                                  const aclTensor* compress_seq_offset_optional,
                                                  const aclTensor* seq_lens_optional, char* cache_mode_optional,
                                                  char* scatter_mode_optional, const aclIntArray* strides_optional,
                                                  const aclIntArray* offsets_optional, uint64_t* workspace_size,
                                                  aclOpExecutor** executor) {
  SHIM_REQUIRE(workspace_size && executor, ACLNN_ERR_PARAM_NULLPTR, "ScatterPaKvCache: null workspace_size / executor output");
  *executor = nullptr;
  SHIM_REQUIRE(key && key_cache_ref && slot_mapping && value && value_cache_ref, ACLNN_ERR_PARAM_NULLPTR,
               "ScatterPaKvCache: key, caches, slot mapping and value are required");
  SHIM_REQUIRE(AsTensor(key) && AsTensor(key_cache_ref) && AsTensor(slot_mapping) && AsTensor(value) && AsTensor(value_cache_ref),
               ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: bad tensor handle");
  SHIM_REQUIRE(!compress_lens_optional && !compress_seq_offset_optional && !seq_lens_optional && !strides_optional && !offsets_optional,
               ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: compression / stride arguments are not served (the decode path passes null)");
  SHIM_REQUIRE(cache_mode_optional == nullptr || std::strcmp(cache_mode_optional, "Norm") == 0, ACLNN_ERR_PARAM_INVALID,
               "ScatterPaKvCache: cache mode '%s' is not served; the engine uses \"Norm\"", cache_mode_optional);
  SHIM_REQUIRE(scatter_mode_optional == nullptr, ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: scatter mode is not served");
  SHIM_REQUIRE(key->dtype == ACL_BF16 && value->dtype == ACL_BF16 && key_cache_ref->dtype == ACL_BF16 && value_cache_ref->dtype == ACL_BF16,
               ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: BF16 token rows and caches expected");
  SHIM_REQUIRE(slot_mapping->dtype == ACL_INT32, ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: slot mapping must be INT32");
  int64_t tokens = 0, value_tokens = 0, key_row = 0, value_row = 0;
  SHIM_REQUIRE(TokenRows(key, 512, &tokens, &key_row), ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: key must be [T, 512] with a dense last axis");
  SHIM_REQUIRE(TokenRows(value, 64, &value_tokens, &value_row) && value_tokens == tokens, ACLNN_ERR_PARAM_INVALID,
               "ScatterPaKvCache: value must be [T, 1, 64] with the key's T");
  SHIM_REQUIRE(slot_mapping->numel() == tokens && slot_mapping->contiguous(), ACLNN_ERR_PARAM_INVALID,
               "ScatterPaKvCache: slot mapping must hold one dense INT32 per token");
  int64_t blocks = 0, block_size = 0, kb = 0, ks = 0, vblocks = 0, vblock_size = 0, vb = 0, vs = 0;
  SHIM_REQUIRE(PagedCacheShape(key_cache_ref, 512, &blocks, &block_size, &kb, &ks), ACLNN_ERR_PARAM_INVALID,
               "ScatterPaKvCache: the key cache is paged [blocks, block, 1, 512]");
  SHIM_REQUIRE(PagedCacheShape(value_cache_ref, 64, &vblocks, &vblock_size, &vb, &vs) && vblocks == blocks && vblock_size == block_size,
               ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: the value cache is paged [blocks, block, 1, 64] with the key cache's geometry");
  SHIM_REQUIRE(blocks <= INT32_MAX / block_size && tokens <= INT32_MAX, ACLNN_ERR_PARAM_INVALID, "ScatterPaKvCache: sizes overflow INT32 slots");
  aclOpExecutor* e = NewExecutor(OpKind::kScatter, {TensorSlot(key), TensorSlot(key_cache_ref), TensorSlot(slot_mapping), TensorSlot(value),
                                                    TensorSlot(value_cache_ref), Slot(), Slot(), Slot(), Slot(), Slot()});
  e->tokens = static_cast<int32_t>(tokens);
  e->num_blocks = static_cast<int32_t>(blocks);
  e->block_size = static_cast<int32_t>(block_size);
  e->key_row_stride = key_row * 2;
  e->value_row_stride = value_row * 2;
  e->key_block_stride = kb * 2;
  e->key_slot_stride = ks * 2;
  e->value_block_stride = vb * 2;
  e->value_slot_stride = vs * 2;
  e->workspace_bytes = 0;
  *workspace_size = 0;
  *executor = e;
  return ACLNN_SUCCESS;
}

static aclnnStatus BeginLaunch(aclOpExecutor* executor, OpKind kind, void* workspace, uint64_t workspace_size, const char* who) {
  SHIM_REQUIRE(executor, ACLNN_ERR_PARAM_NULLPTR, "%s: null executor", who);
  SHIM_REQUIRE(AsExecutor(executor) && executor->kind == kind, ACLNN_ERR_PARAM_INVALID, "%s: not an executor planned by this operator", who);
  SHIM_REQUIRE(executor->repeatable || !executor->launched, ACLNN_ERR_PARAM_INVALID,
               "%s: the executor was consumed by its first launch; call aclSetAclOpExecutorRepeatable after planning", who);
  SHIM_REQUIRE(workspace_size >= executor->workspace_bytes && (executor->workspace_bytes == 0 || workspace != nullptr),
               ACLNN_ERR_PARAM_INVALID, "%s: planned %llu workspace bytes, given %llu", who,
               static_cast<unsigned long long>(executor->workspace_bytes), static_cast<unsigned long long>(workspace_size));
  return ACLNN_SUCCESS;
}

static void FillView(mlakvCacheView* view, const aclOpExecutor* e, void* latent, void* rope) {
  std::memset(view, 0, sizeof(*view));
  view->latent = latent;
  view->latent_block_stride = e->key_block_stride;
  view->latent_row_stride = e->key_slot_stride;
  view->rope = rope;
  view->rope_block_stride = e->value_block_stride;
  view->rope_row_stride = e->value_slot_stride;
  view->num_layers = 1;
  view->num_blocks = e->num_blocks;
  view->block_size = e->block_size;
  view->latent_dim = 512;
  view->rope_dim = 64;
  view->dtype = MLAKV_DTYPE_BF16;
}

aclnnStatus aclnnScatterPaKvCache(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream) {
  if (aclnnStatus s = BeginLaunch(executor, OpKind::kScatter, workspace, workspace_size, "aclnnScatterPaKvCache")) return s;
  mlakvCacheView view;
  FillView(&view, executor, executor->slots[1].addresses[0], executor->slots[4].addresses[0]);
  const mlakvStatus status = mlakvAppend(&view, 0, 1, executor->slots[0].addresses[0], 0, executor->key_row_stride,
                                         executor->slots[3].addresses[0], 0, executor->value_row_stride,
                                         static_cast<const int32_t*>(executor->slots[2].addresses[0]), executor->tokens, stream);
  if (status == MLAKV_SUCCESS) executor->launched = true;
  return status;
}

// ---- aclnnDynamicMxQuant ----------------------------------------------------------------------

aclnnStatus aclnnDynamicMxQuantGetWorkspaceSize(const aclTensor* x, int64_t axis, char* round_mode_optional, int64_t dst_type,
                                                int64_t blocksize, int64_t scale_alg, const aclTensor* y_out,
                                                const aclTensor* mxscale_out, uint64_t* workspace_size, aclOpExecutor** executor) {
  SHIM_REQUIRE(workspace_size && executor, ACLNN_ERR_PARAM_NULLPTR, "DynamicMxQuant: null workspace_size / executor output");
  *executor = nullptr;
  SHIM_REQUIRE(x && y_out && mxscale_out, ACLNN_ERR_PARAM_NULLPTR, "DynamicMxQuant: x, y and mxscale are required");
  SHIM_REQUIRE(AsTensor(x) && AsTensor(y_out) && AsTensor(mxscale_out), ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: bad tensor handle");
  const int64_t rank = static_cast<int64_t>(x->dims.size());
  SHIM_REQUIRE(rank == 2, ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: x must be [rows, cols] (the engine quantizes flat activations)");
  SHIM_REQUIRE(axis == -1 || axis == rank - 1, ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: only the last axis is served, got %lld",
               static_cast<long long>(axis));
  SHIM_REQUIRE(round_mode_optional == nullptr || std::strcmp(round_mode_optional, "rint") == 0, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: round mode '%s' is not served; the engine uses \"rint\"", round_mode_optional);
  SHIM_REQUIRE(dst_type == ACL_FLOAT8_E4M3FN, ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: dst_type %lld is not served; the engine uses E4M3 (36)",
               static_cast<long long>(dst_type));
  SHIM_REQUIRE(blocksize == 32, ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: the microscale block is 32, got %lld", static_cast<long long>(blocksize));
  SHIM_REQUIRE(scale_alg == 0, ACLNN_ERR_PARAM_INVALID, "DynamicMxQuant: only the OCP scale algorithm (0) is served");
  SHIM_REQUIRE(x->dtype == ACL_BF16 && y_out->dtype == ACL_FLOAT8_E4M3FN && mxscale_out->dtype == ACL_FLOAT8_E8M0, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: BF16 input, E4M3 values and E8M0 scales expected");
  const int64_t rows = x->dims[0], cols = x->dims[1];
  SHIM_REQUIRE(rows > 0 && cols > 0 && cols % 32 == 0 && cols <= INT32_MAX, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: %lld columns are not a whole number of blocks of 32", static_cast<long long>(cols));
  SHIM_REQUIRE(y_out->dims.size() == 2 && y_out->dims[0] == rows && y_out->dims[1] == cols, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: y must have the shape of x");
  SHIM_REQUIRE(mxscale_out->dims.size() == 2 && mxscale_out->dims[0] == rows && mxscale_out->dims[1] == cols / 32, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: mxscale must be [rows, cols / 32]");
  SHIM_REQUIRE(x->strides[1] == 1 && y_out->strides[1] == 1 && mxscale_out->strides[1] == 1, ACLNN_ERR_PARAM_INVALID,
               "DynamicMxQuant: the last axis must be dense");
  aclOpExecutor* e = NewExecutor(OpKind::kMxQuant, {TensorSlot(x), TensorSlot(y_out), TensorSlot(mxscale_out)});
  e->tokens = static_cast<int32_t>(cols);  // columns
  e->key_row_stride = x->strides[0] * 2;
  e->value_row_stride = y_out->strides[0];
  e->key_block_stride = mxscale_out->strides[0];
  e->q_token_stride = rows;
  e->workspace_bytes = 0;
  *workspace_size = 0;
  *executor = e;
  return ACLNN_SUCCESS;
}

// ---- aclnnQuantLightningIndexer ---------------------------------------------------------------

aclnnStatus aclnnQuantLightningIndexerGetWorkspaceSize(const aclTensor* query, const aclTensor* key, const aclTensor* weights,
                                                       const aclTensor* query_dequant_scale, const aclTensor* key_dequant_scale,
                                                       const aclTensor* actual_seq_lengths_query_optional,
                                                       const aclTensor* actual_seq_lengths_key_optional,
                                                       const aclTensor* block_table_optional, int64_t query_quant_mode,
                                                       int64_t key_quant_mode, char* layout_query_optional,
                                                       char* layout_key_optional, int64_t sparse_count, int64_t sparse_mode,
                                                       int64_t pre_tokens, int64_t next_tokens, const aclTensor* out,
                                                       uint64_t* workspace_size, aclOpExecutor** executor) {
  const char* who = "QuantLightningIndexer";
  SHIM_REQUIRE(workspace_size && executor, ACLNN_ERR_PARAM_NULLPTR, "%s: null workspace_size / executor output", who);
  *executor = nullptr;
  SHIM_REQUIRE(query && key && weights && query_dequant_scale && key_dequant_scale && out, ACLNN_ERR_PARAM_NULLPTR,
               "%s: query, key, weights, both dequant scales and out are required", who);
  SHIM_REQUIRE(actual_seq_lengths_key_optional && block_table_optional, ACLNN_ERR_PARAM_NULLPTR,
               "%s: the paged key layout needs actual_seq_lengths_key and block_table", who);
  SHIM_REQUIRE(AsTensor(query) && AsTensor(key) && AsTensor(weights) && AsTensor(query_dequant_scale) && AsTensor(key_dequant_scale) &&
                   AsTensor(actual_seq_lengths_key_optional) && AsTensor(block_table_optional) && AsTensor(out) &&
                   (actual_seq_lengths_query_optional == nullptr || AsTensor(actual_seq_lengths_query_optional)),
               ACLNN_ERR_PARAM_INVALID, "%s: bad tensor handle", who);
  SHIM_REQUIRE(query_quant_mode == 0 && key_quant_mode == 0, ACLNN_ERR_PARAM_INVALID, "%s: only per-token-head quantization (mode 0) is served", who);
  SHIM_REQUIRE(layout_query_optional == nullptr || std::strcmp(layout_query_optional, "BSND") == 0, ACLNN_ERR_PARAM_INVALID,
               "%s: query layout '%s' is not served; decode uses \"BSND\"", who, layout_query_optional);
  SHIM_REQUIRE(layout_key_optional != nullptr && std::strcmp(layout_key_optional, "PA_BSND") == 0, ACLNN_ERR_PARAM_INVALID,
               "%s: only the paged key layout \"PA_BSND\" is served", who);
  SHIM_REQUIRE(sparse_count >= 1 && sparse_count <= 2048, ACLNN_ERR_PARAM_INVALID, "%s: sparse_count %lld outside [1, 2048]", who,
               static_cast<long long>(sparse_count));
  SHIM_REQUIRE(sparse_mode == 0 || sparse_mode == 3, ACLNN_ERR_PARAM_INVALID, "%s: sparse_mode %lld is not one of 0, 3", who,
               static_cast<long long>(sparse_mode));
  SHIM_REQUIRE(pre_tokens == INT64_MAX && next_tokens == INT64_MAX, ACLNN_ERR_PARAM_INVALID, "%s: only the unrestricted window is served", who);
  SHIM_REQUIRE(query->dtype == ACL_FLOAT8_E4M3FN && key->dtype == ACL_FLOAT8_E4M3FN, ACLNN_ERR_PARAM_INVALID, "%s: E4M3 query and key expected", who);
  SHIM_REQUIRE(weights->dtype == ACL_BF16 && query_dequant_scale->dtype == ACL_FLOAT32 && key_dequant_scale->dtype == ACL_FLOAT32,
               ACLNN_ERR_PARAM_INVALID, "%s: BF16 weights and FP32 dequant scales expected", who);
  SHIM_REQUIRE(block_table_optional->dtype == ACL_INT32 && actual_seq_lengths_key_optional->dtype == ACL_INT32 && out->dtype == ACL_INT32,
               ACLNN_ERR_PARAM_INVALID, "%s: block table, key lengths and out must be INT32", who);
  // query [B, 1, N1, 128]: one decode token per sequence
  SHIM_REQUIRE(query->dims.size() == 4 && query->dims[1] == 1 && query->dims[3] == 128 && query->strides[3] == 1, ACLNN_ERR_PARAM_INVALID,
               "%s: query must be [B, 1, N1, 128] (one decode token per sequence)", who);
  const int64_t batch = query->dims[0], heads = query->dims[2];
  SHIM_REQUIRE(batch > 0 && batch <= 65535 && (heads == 16 || heads == 32 || heads == 48 || heads == 64), ACLNN_ERR_PARAM_INVALID,
               "%s: N1 = %lld is not one of 16, 32, 48, 64", who, static_cast<long long>(heads));
  int64_t blocks = 0, bs = 0, kb = 0, ks = 0;
  SHIM_REQUIRE(PagedCacheShape(key, 128, &blocks, &bs, &kb, &ks), ACLNN_ERR_PARAM_INVALID, "%s: key must be paged [blocks, block, 1, 128]", who);
  SHIM_REQUIRE(weights->dims.size() == 3 && weights->dims[0] == batch && weights->dims[1] == 1 && weights->dims[2] == heads && weights->strides[2] == 1 &&
                   query_dequant_scale->dims.size() == 3 && query_dequant_scale->dims[0] == batch && query_dequant_scale->dims[2] == heads &&
                   query_dequant_scale->strides[2] == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: weights and query_dequant_scale must be [B, 1, N1]", who);
  SHIM_REQUIRE(key_dequant_scale->dims.size() == 3 && key_dequant_scale->dims[0] == blocks && key_dequant_scale->dims[1] == bs &&
                   key_dequant_scale->dims[2] == 1 && key_dequant_scale->strides[1] == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: key_dequant_scale must be [blocks, block, 1] with dense slots", who);
  SHIM_REQUIRE(block_table_optional->dims.size() == 2 && block_table_optional->dims[0] == batch && block_table_optional->contiguous() &&
                   actual_seq_lengths_key_optional->numel() == batch && actual_seq_lengths_key_optional->contiguous(),
               ACLNN_ERR_PARAM_INVALID, "%s: block table [B, W] and key lengths [B] must be dense", who);
  SHIM_REQUIRE(out->dims.size() == 4 && out->dims[0] == batch && out->dims[1] == 1 && out->dims[2] == 1 && out->dims[3] == sparse_count &&
                   out->strides[3] == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: out must be [B, 1, 1, sparse_count]", who);
  const int64_t width = block_table_optional->dims[1];
  SHIM_REQUIRE(width * bs <= INT32_MAX && blocks <= INT32_MAX, ACLNN_ERR_PARAM_INVALID, "%s: sizes overflow INT32", who);
  aclOpExecutor* e = NewExecutor(OpKind::kIndexer, {TensorSlot(query), TensorSlot(key), TensorSlot(weights), TensorSlot(query_dequant_scale),
                                                    TensorSlot(key_dequant_scale), TensorSlot(actual_seq_lengths_query_optional),
                                                    TensorSlot(actual_seq_lengths_key_optional), TensorSlot(block_table_optional),
                                                    TensorSlot(out)});
  e->batch = static_cast<int32_t>(batch);
  e->heads = static_cast<int32_t>(heads);
  e->num_blocks = static_cast<int32_t>(blocks);
  e->block_size = static_cast<int32_t>(bs);
  e->table_width = static_cast<int32_t>(width);
  e->max_seq_len = static_cast<int32_t>(width * bs);  // every length the table can address
  e->sparse_count = static_cast<int32_t>(sparse_count);
  e->key_block_stride = kb;
  e->key_slot_stride = ks;
  e->q_token_stride = query->strides[0];
  e->q_head_stride = query->strides[2];
  e->aux_stride[0] = weights->strides[0] * 2;
  e->aux_stride[1] = query_dequant_scale->strides[0];
  e->aux_stride[2] = key_dequant_scale->strides[0];
  e->aux_stride[3] = out->strides[0];
  e->workspace_bytes = mlakvIndexerWorkspaceBytes(e->batch, e->max_seq_len);
  *workspace_size = e->workspace_bytes;
  *executor = e;
  return ACLNN_SUCCESS;
}

// ---- aclnnFusedInferAttentionScoreV5 ------------------------------------------------------------

aclnnStatus aclnnFusedInferAttentionScoreV5GetWorkspaceSize(
    const aclTensor* query, const aclTensorList* key, const aclTensorList* value, const aclTensor* pse_shift,
    const aclTensor* atten_mask, const aclIntArray* actual_seq_lengths, const aclIntArray* actual_seq_lengths_kv,
    const aclTensor* deq_scale1, const aclTensor* quant_scale1, const aclTensor* deq_scale2, const aclTensor* quant_scale2,
    const aclTensor* quant_offset2, const aclTensor* antiquant_scale, const aclTensor* antiquant_offset,
    const aclTensor* block_table, const aclTensor* query_padding_size, const aclTensor* kv_padding_size,
    const aclTensor* key_antiquant_scale, const aclTensor* key_antiquant_offset, const aclTensor* value_antiquant_scale,
    const aclTensor* value_antiquant_offset, const aclTensor* key_shared_prefix, const aclTensor* value_shared_prefix,
    const aclIntArray* actual_shared_prefix_len, const aclTensor* query_rope, const aclTensor* key_rope,
    const aclTensor* key_rope_antiquant_scale, const aclTensor* dequant_scale_query, const aclTensor* learnable_sink,
    const aclIntArray* q_start_idx, const aclIntArray* kv_start_idx, int64_t num_heads, double scale_value,
    int64_t pre_tokens, int64_t next_tokens, char* input_layout, int64_t num_key_value_heads, int64_t sparse_mode,
    int64_t inner_precise, int64_t block_size, int64_t antiquant_mode, bool softmax_lse_flag, int64_t key_antiquant_mode,
    int64_t value_antiquant_mode, int64_t query_quant_mode, int64_t pse_type, const aclTensor* attention_out,
    const aclTensor* softmax_lse, uint64_t* workspace_size, aclOpExecutor** executor) {
  const char* who = "FusedInferAttentionScoreV5";
  SHIM_REQUIRE(workspace_size && executor, ACLNN_ERR_PARAM_NULLPTR, "%s: null workspace_size / executor output", who);
  *executor = nullptr;
  SHIM_REQUIRE(query && key && value && block_table && query_rope && key_rope && attention_out && actual_seq_lengths_kv,
               ACLNN_ERR_PARAM_NULLPTR, "%s: query, key/value lists, block table, rope tensors, kv lengths and output are required", who);
  SHIM_REQUIRE(AsTensor(query) && AsList(key) && AsList(value) && AsTensor(block_table) && AsTensor(query_rope) && AsTensor(key_rope) &&
                   AsTensor(attention_out) && AsArray(actual_seq_lengths_kv),
               ACLNN_ERR_PARAM_INVALID, "%s: bad tensor handle", who);
  SHIM_REQUIRE(actual_seq_lengths == nullptr || AsArray(actual_seq_lengths), ACLNN_ERR_PARAM_INVALID, "%s: bad query-length array", who);
  SHIM_REQUIRE(!pse_shift && !atten_mask && !deq_scale1 && !quant_scale1 && !deq_scale2 && !quant_scale2 && !quant_offset2 &&
                   !antiquant_scale && !antiquant_offset && !query_padding_size && !kv_padding_size && !key_antiquant_scale &&
                   !key_antiquant_offset && !value_antiquant_scale && !value_antiquant_offset && !key_shared_prefix &&
                   !value_shared_prefix && !actual_shared_prefix_len && !key_rope_antiquant_scale && !dequant_scale_query &&
                   !learnable_sink && !q_start_idx && !kv_start_idx,
               ACLNN_ERR_PARAM_INVALID, "%s: masks, position terms, quantisation, padding, prefix and sink arguments are not served "
               "(the decode path passes null)", who);
  SHIM_REQUIRE(antiquant_mode == 0 && key_antiquant_mode == 0 && value_antiquant_mode == 0 && query_quant_mode == 0 && pse_type == 0,
               ACLNN_ERR_PARAM_INVALID, "%s: quantisation / pse modes must be 0", who);
  SHIM_REQUIRE(input_layout != nullptr && std::strcmp(input_layout, "TND") == 0, ACLNN_ERR_PARAM_INVALID, "%s: layout \"TND\" expected", who);
  SHIM_REQUIRE(num_key_value_heads == 1, ACLNN_ERR_PARAM_INVALID, "%s: absorbed MLA has one key/value head, got %lld", who,
               static_cast<long long>(num_key_value_heads));
  SHIM_REQUIRE(sparse_mode == 0 || sparse_mode == 3, ACLNN_ERR_PARAM_INVALID, "%s: sparse mode %lld is not served", who, static_cast<long long>(sparse_mode));
  SHIM_REQUIRE(inner_precise == 0 || inner_precise == 1, ACLNN_ERR_PARAM_INVALID, "%s: inner_precise must be 0 or 1", who);
  SHIM_REQUIRE(pre_tokens >= 0 && next_tokens >= 0, ACLNN_ERR_PARAM_INVALID, "%s: negative attention window", who);
  SHIM_REQUIRE(scale_value > 0.0, ACLNN_ERR_PARAM_INVALID, "%s: a positive softmax scale is required", who);
  SHIM_REQUIRE(key->items.size() == 1 && value->items.size() == 1, ACLNN_ERR_PARAM_INVALID, "%s: one key and one value tensor expected", who);
  const aclTensor* k = key->items[0];
  const aclTensor* v = value->items[0];
  SHIM_REQUIRE(query->dtype == ACL_BF16 && query_rope->dtype == ACL_BF16 && k->dtype == ACL_BF16 && v->dtype == ACL_BF16 &&
                   key_rope->dtype == ACL_BF16 && attention_out->dtype == ACL_BF16,
               ACLNN_ERR_PARAM_INVALID, "%s: BF16 query, cache and output expected", who);
  SHIM_REQUIRE(block_table->dtype == ACL_INT32 && block_table->dims.size() == 2 && block_table->contiguous(), ACLNN_ERR_PARAM_INVALID,
               "%s: block table must be a dense INT32 [T, W]", who);
  SHIM_REQUIRE(query->dims.size() == 3 && query->dims[2] == 512 && query->strides[2] == 1, ACLNN_ERR_PARAM_INVALID,
               "%s: query must be [T, N, 512] with a dense last axis", who);
  const int64_t tokens = query->dims[0], heads = query->dims[1];
  SHIM_REQUIRE(heads == num_heads, ACLNN_ERR_PARAM_INVALID, "%s: num_heads %lld but the query has %lld heads", who,
               static_cast<long long>(num_heads), static_cast<long long>(heads));
  SHIM_REQUIRE(query_rope->dims.size() == 3 && query_rope->dims[0] == tokens && query_rope->dims[1] == heads && query_rope->dims[2] == 64 &&
                   query_rope->strides[2] == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: query_rope must be [T, N, 64] with a dense last axis", who);
  SHIM_REQUIRE(attention_out->dims.size() == 3 && attention_out->dims[0] == tokens && attention_out->dims[1] == heads &&
                   attention_out->dims[2] == 512 && attention_out->strides[2] == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: attention_out must be [T, N, 512] with a dense last axis", who);
  SHIM_REQUIRE(block_table->dims[0] == tokens, ACLNN_ERR_PARAM_INVALID, "%s: one block-table row per query token (decode) expected", who);
  SHIM_REQUIRE(actual_seq_lengths_kv->size == static_cast<uint64_t>(tokens), ACLNN_ERR_PARAM_INVALID,
               "%s: actual_seq_lengths_kv must hold one length per sequence (%lld)", who, static_cast<long long>(tokens));
  SHIM_REQUIRE(actual_seq_lengths == nullptr || actual_seq_lengths->size == static_cast<uint64_t>(tokens) || actual_seq_lengths->size == 1,
               ACLNN_ERR_PARAM_INVALID, "%s: actual_seq_lengths must hold one entry per sequence", who);
  int64_t blocks = 0, bs = 0, kb = 0, ks = 0, rblocks = 0, rbs = 0, rb = 0, rs = 0, vblocks = 0, vbs = 0, vb = 0, vs = 0;
  SHIM_REQUIRE(PagedCacheShape(k, 512, &blocks, &bs, &kb, &ks), ACLNN_ERR_PARAM_INVALID, "%s: the key cache is paged [blocks, block, 1, 512]", who);
  SHIM_REQUIRE(PagedCacheShape(v, 512, &vblocks, &vbs, &vb, &vs) && vblocks == blocks && vbs == bs && vb == kb && vs == ks,
               ACLNN_ERR_PARAM_INVALID, "%s: the value cache must have the key cache's geometry (K and V alias the latent cache)", who);
  SHIM_REQUIRE(PagedCacheShape(key_rope, 64, &rblocks, &rbs, &rb, &rs) && rblocks == blocks && rbs == bs, ACLNN_ERR_PARAM_INVALID,
               "%s: key_rope is paged [blocks, block, 1, 64] with the key cache's geometry", who);
  SHIM_REQUIRE(block_size == bs, ACLNN_ERR_PARAM_INVALID, "%s: block_size %lld but the cache has %lld slots per block", who,
               static_cast<long long>(block_size), static_cast<long long>(bs));
  if (softmax_lse_flag) {
    SHIM_REQUIRE(softmax_lse != nullptr && AsTensor(softmax_lse) && softmax_lse->dtype == ACL_FLOAT32 && softmax_lse->numel() == tokens * heads &&
                     softmax_lse->contiguous(),
                 ACLNN_ERR_PARAM_INVALID, "%s: softmax_lse must be a dense FP32 [T, N, 1] when requested", who);
  }
  const int64_t width = block_table->dims[1];
  SHIM_REQUIRE(tokens <= 65535 && width * bs <= INT32_MAX && blocks <= INT32_MAX / bs, ACLNN_ERR_PARAM_INVALID, "%s: sizes exceed the launch limits", who);
  for (int64_t b = 0; b < tokens; ++b) {
    const int64_t len = actual_seq_lengths_kv->values[b];
    SHIM_REQUIRE(len >= 0 && len <= width * bs, ACLNN_ERR_PARAM_INVALID, "%s: kv length %lld of sequence %lld outside [0, %lld]", who,
                 static_cast<long long>(len), static_cast<long long>(b), static_cast<long long>(width * bs));
  }
  mlakvAttnPlan plan;
  if (mlakvStatus s = mlakvAttnPlanInit(static_cast<int32_t>(tokens), static_cast<int32_t>(heads), static_cast<int32_t>(width * bs),
                                        static_cast<int32_t>(bs), MLAKV_DTYPE_BF16, &plan)) {
    return s;
  }
  std::vector<Slot> slots = {
      TensorSlot(query), ListSlot(key), ListSlot(value), TensorSlot(pse_shift), TensorSlot(atten_mask), ArraySlot(actual_seq_lengths),
      ArraySlot(actual_seq_lengths_kv), TensorSlot(deq_scale1), TensorSlot(quant_scale1), TensorSlot(deq_scale2), TensorSlot(quant_scale2),
      TensorSlot(quant_offset2), TensorSlot(antiquant_scale), TensorSlot(antiquant_offset), TensorSlot(block_table),
      TensorSlot(query_padding_size), TensorSlot(kv_padding_size), TensorSlot(key_antiquant_scale), TensorSlot(key_antiquant_offset),
      TensorSlot(value_antiquant_scale), TensorSlot(value_antiquant_offset), TensorSlot(key_shared_prefix), TensorSlot(value_shared_prefix),
      ArraySlot(actual_shared_prefix_len), TensorSlot(query_rope), TensorSlot(key_rope), TensorSlot(key_rope_antiquant_scale),
      TensorSlot(dequant_scale_query), TensorSlot(learnable_sink), ArraySlot(q_start_idx), ArraySlot(kv_start_idx),
      TensorSlot(attention_out), TensorSlot(softmax_lse)};
  aclOpExecutor* e = NewExecutor(OpKind::kAttention, std::move(slots));
  e->tokens = e->batch = static_cast<int32_t>(tokens);
  e->heads = static_cast<int32_t>(heads);
  e->num_blocks = static_cast<int32_t>(blocks);
  e->block_size = static_cast<int32_t>(bs);
  e->table_width = static_cast<int32_t>(width);
  e->max_seq_len = static_cast<int32_t>(width * bs);
  e->key_block_stride = kb * 2;
  e->key_slot_stride = ks * 2;
  e->value_block_stride = rb * 2;  // rope plane
  e->value_slot_stride = rs * 2;
  e->q_token_stride = query->strides[0] * 2;
  e->q_head_stride = query->strides[1] * 2;
  e->qr_token_stride = query_rope->strides[0] * 2;
  e->qr_head_stride = query_rope->strides[1] * 2;
  e->out_token_stride = attention_out->strides[0] * 2;
  e->out_head_stride = attention_out->strides[1] * 2;
  e->scale = scale_value;
  e->want_lse = softmax_lse_flag;
  e->plan = plan;
  e->lens_offset = (plan.workspace_bytes + 255) & ~255ull;
  e->workspace_bytes = e->lens_offset + ((static_cast<uint64_t>(tokens) * sizeof(int32_t) + 255) & ~255ull);
  e->host_lens.resize(static_cast<size_t>(tokens));
  for (int64_t b = 0; b < tokens; ++b) e->host_lens[static_cast<size_t>(b)] = static_cast<int32_t>(actual_seq_lengths_kv->values[b]);
  *workspace_size = e->workspace_bytes;
  *executor = e;
  return ACLNN_SUCCESS;
}

aclnnStatus aclnnQuantLightningIndexer(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream) {
  if (aclnnStatus s = BeginLaunch(executor, OpKind::kIndexer, workspace, workspace_size, "aclnnQuantLightningIndexer")) return s;
  aclOpExecutor* e = executor;
  mlakvIndexKeyView keys{};
  keys.keys = e->slots[1].addresses[0];
  keys.block_stride = e->key_block_stride;
  keys.row_stride = e->key_slot_stride;
  keys.scales = static_cast<const float*>(e->slots[4].addresses[0]);
  keys.scale_block_stride = e->aux_stride[2];
  keys.num_blocks = e->num_blocks;
  keys.block_size = e->block_size;
  keys.dim = 128;
  const mlakvStatus status = mlakvLightningIndexer(
      &keys, e->slots[0].addresses[0], e->q_token_stride, e->q_head_stride, e->slots[2].addresses[0], e->aux_stride[0],
      static_cast<const float*>(e->slots[3].addresses[0]), e->aux_stride[1], e->heads, static_cast<const int32_t*>(e->slots[7].addresses[0]),
      e->table_width, static_cast<const int32_t*>(e->slots[6].addresses[0]), e->batch, e->max_seq_len, e->sparse_count,
      static_cast<int32_t*>(e->slots[8].addresses[0]), e->aux_stride[3], workspace, workspace_size, stream);
  if (status == MLAKV_SUCCESS) e->launched = true;
  return status;
}

aclnnStatus aclnnDynamicMxQuant(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream) {
  if (aclnnStatus s = BeginLaunch(executor, OpKind::kMxQuant, workspace, workspace_size, "aclnnDynamicMxQuant")) return s;
  const mlakvStatus status = mlakvDynamicMxQuant(executor->slots[0].addresses[0], executor->key_row_stride, executor->q_token_stride,
                                                 executor->tokens, executor->slots[1].addresses[0], executor->value_row_stride,
                                                 executor->slots[2].addresses[0], executor->key_block_stride, stream);
  if (status == MLAKV_SUCCESS) executor->launched = true;
  return status;
}

aclnnStatus aclnnFusedInferAttentionScoreV5(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream) {
  const char* who = "aclnnFusedInferAttentionScoreV5";
  if (aclnnStatus s = BeginLaunch(executor, OpKind::kAttention, workspace, workspace_size, who)) return s;
  aclOpExecutor* e = executor;
  void* latent = e->slots[1].addresses[0];
  SHIM_REQUIRE(e->slots[2].addresses[0] == latent, ACLNN_ERR_PARAM_INVALID,
               "%s: the value tensor must alias the key tensor (absorbed MLA reads the latent cache as K and V)", who);
  const int32_t* device_lens = e->bound_lens;
  const bool inline_lens = device_lens == nullptr && e->batch <= MLAKV_ATTN_HOST_LENS_MAX;
  if (device_lens == nullptr && !inline_lens) {
    // The lengths travel in the argument block of a one-workgroup kernel: the host vector is free
    // again when the call returns, and nothing is staged or waited for.
    int32_t* staged = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + e->lens_offset);
    for (int32_t first = 0; first < e->batch; first += mlakv::kMaxStoreWords) {
      const int count = std::min<int32_t>(mlakv::kMaxStoreWords, e->batch - first);
      const hipError_t status = mlakv::LaunchStoreWords(e->host_lens.data() + first, count, staged + first, static_cast<hipStream_t>(stream));
      SHIM_REQUIRE(status == hipSuccess, ACLNN_ERR_RUNTIME_ERROR, "%s: length upload failed: %s", who, hipGetErrorString(status));
    }
    device_lens = staged;
  }
  mlakvCacheView view;
  FillView(&view, e, latent, e->slots[25].addresses[0]);
  float* lse = e->want_lse ? static_cast<float*>(e->slots[32].addresses[0]) : nullptr;
  // Up to MLAKV_ATTN_HOST_LENS_MAX sequences (the reference has one): the lengths ride in the
  // attention kernels' own argument block, no launch is spent on them.
  const mlakvStatus status =
      inline_lens ? mlakvAttnDecodeHostLens(&e->plan, &view, 0, e->slots[0].addresses[0], e->q_token_stride, e->q_head_stride,
                                            e->slots[24].addresses[0], e->qr_token_stride, e->qr_head_stride,
                                            static_cast<const int32_t*>(e->slots[14].addresses[0]), e->table_width, e->host_lens.data(),
                                            e->scale, e->slots[31].addresses[0], e->out_token_stride, e->out_head_stride, lse, workspace,
                                            e->plan.workspace_bytes, stream)
                  // (lengths in device memory; a bound the caller gave for them decides the kernels)
                  : mlakvAttnDecodeBounded(&e->plan, &view, 0, e->slots[0].addresses[0], e->q_token_stride, e->q_head_stride,
                                           e->slots[24].addresses[0], e->qr_token_stride, e->qr_head_stride,
                                           static_cast<const int32_t*>(e->slots[14].addresses[0]), e->table_width, device_lens,
                                           e->bound_lens == nullptr ? *std::max_element(e->host_lens.begin(), e->host_lens.end())  // staged from the host values
                                                                    : (e->bound_longest >= 0 ? e->bound_longest : e->max_seq_len),
                                           e->scale,
                                           e->slots[31].addresses[0], e->out_token_stride, e->out_head_stride, lse, workspace,
                                           e->plan.workspace_bytes, stream);
  if (status == MLAKV_SUCCESS) e->launched = true;
  return status;
}

aclnnStatus aclnnMlaKvSetSeqLens(aclOpExecutor* executor, const int64_t* seq_lens, uint64_t count) {
  const char* who = "aclnnMlaKvSetSeqLens";
  SHIM_REQUIRE(executor && seq_lens, ACLNN_ERR_PARAM_NULLPTR, "%s: null executor or lengths", who);
  SHIM_REQUIRE(AsExecutor(executor) && executor->kind == OpKind::kAttention, ACLNN_ERR_PARAM_INVALID, "%s: not an attention executor", who);
  SHIM_REQUIRE(count == static_cast<uint64_t>(executor->batch), ACLNN_ERR_PARAM_INVALID, "%s: %llu lengths for %d sequences", who,
               static_cast<unsigned long long>(count), executor->batch);
  for (uint64_t b = 0; b < count; ++b) {
    SHIM_REQUIRE(seq_lens[b] >= 0 && seq_lens[b] <= executor->max_seq_len, ACLNN_ERR_PARAM_INVALID,
                 "%s: kv length %lld of sequence %llu outside [0, %d]", who, static_cast<long long>(seq_lens[b]),
                 static_cast<unsigned long long>(b), executor->max_seq_len);
  }
  for (uint64_t b = 0; b < count; ++b) executor->host_lens[b] = static_cast<int32_t>(seq_lens[b]);
  return ACLNN_SUCCESS;
}

aclnnStatus aclnnMlaKvBindSeqLens(aclOpExecutor* executor, const int32_t* device_seq_lens) {
  SHIM_REQUIRE(executor, ACLNN_ERR_PARAM_NULLPTR, "aclnnMlaKvBindSeqLens: null executor");
  SHIM_REQUIRE(AsExecutor(executor) && executor->kind == OpKind::kAttention, ACLNN_ERR_PARAM_INVALID,
               "aclnnMlaKvBindSeqLens: not an attention executor");
  executor->bound_lens = device_seq_lens;
  executor->bound_longest = -1;
  return ACLNN_SUCCESS;
}

aclnnStatus aclnnMlaKvSetSeqLenBound(aclOpExecutor* executor, int64_t longest) {
  const char* who = "aclnnMlaKvSetSeqLenBound";
  SHIM_REQUIRE(executor, ACLNN_ERR_PARAM_NULLPTR, "%s: null executor", who);
  SHIM_REQUIRE(AsExecutor(executor) && executor->kind == OpKind::kAttention, ACLNN_ERR_PARAM_INVALID, "%s: not an attention executor", who);
  SHIM_REQUIRE(longest >= -1 && longest <= executor->max_seq_len, ACLNN_ERR_PARAM_INVALID, "%s: bound %lld outside [-1, %d]", who,
               static_cast<long long>(longest), executor->max_seq_len);
  executor->bound_longest = static_cast<int32_t>(longest);
  return ACLNN_SUCCESS;
}

// ---- aclnnGatherPaKvCache ------------------------------------------------------------------------

aclnnStatus aclnnGatherPaKvCacheGetWorkspaceSize(const aclTensor* key_cache, const aclTensor* value_cache,
                                                 const aclTensor* block_table, const aclTensor* seq_lens,
                                                 const aclTensor* cu_seq_lens, aclTensor* key_out, aclTensor* value_out,
                                                 int64_t max_seq_len, uint64_t* workspace_size, aclOpExecutor** executor) {
  const char* who = "GatherPaKvCache";
  SHIM_REQUIRE(workspace_size && executor, ACLNN_ERR_PARAM_NULLPTR, "%s: null workspace_size / executor output", who);
  *executor = nullptr;
  SHIM_REQUIRE(key_cache && value_cache && block_table && seq_lens && cu_seq_lens && key_out && value_out, ACLNN_ERR_PARAM_NULLPTR,
               "%s: every tensor argument is required", who);
  SHIM_REQUIRE(AsTensor(key_cache) && AsTensor(value_cache) && AsTensor(block_table) && AsTensor(seq_lens) && AsTensor(cu_seq_lens) &&
                   AsTensor(key_out) && AsTensor(value_out),
               ACLNN_ERR_PARAM_INVALID, "%s: bad tensor handle", who);
  SHIM_REQUIRE(key_cache->dtype == ACL_BF16 && value_cache->dtype == ACL_BF16 && key_out->dtype == ACL_BF16 && value_out->dtype == ACL_BF16,
               ACLNN_ERR_PARAM_INVALID, "%s: BF16 caches and outputs expected", who);
  SHIM_REQUIRE(block_table->dtype == ACL_INT32 && seq_lens->dtype == ACL_INT32 && cu_seq_lens->dtype == ACL_INT32, ACLNN_ERR_PARAM_INVALID,
               "%s: block table and lengths must be INT32", who);
  SHIM_REQUIRE(block_table->dims.size() == 2 && block_table->contiguous() && seq_lens->contiguous() && cu_seq_lens->contiguous(),
               ACLNN_ERR_PARAM_INVALID, "%s: block table [B, W] and dense length vectors expected", who);
  const int64_t batch = block_table->dims[0], width = block_table->dims[1];
  SHIM_REQUIRE(seq_lens->numel() == batch && cu_seq_lens->numel() == batch + 1, ACLNN_ERR_PARAM_INVALID,
               "%s: seq_lens [B] and cu_seq_lens [B+1] expected", who);
  int64_t blocks = 0, bs = 0, kb = 0, ks = 0, vblocks = 0, vbs = 0, vb = 0, vs = 0, rows = 0, vrows = 0, key_row = 0, value_row = 0;
  SHIM_REQUIRE(PagedCacheShape(key_cache, 512, &blocks, &bs, &kb, &ks), ACLNN_ERR_PARAM_INVALID, "%s: the key cache is paged [blocks, block, 1, 512]", who);
  SHIM_REQUIRE(PagedCacheShape(value_cache, 64, &vblocks, &vbs, &vb, &vs) && vblocks == blocks && vbs == bs, ACLNN_ERR_PARAM_INVALID,
               "%s: the value cache is paged [blocks, block, 1, 64] with the key cache's geometry", who);
  SHIM_REQUIRE(TokenRows(key_out, 512, &rows, &key_row) && TokenRows(value_out, 64, &vrows, &value_row) && rows == vrows, ACLNN_ERR_PARAM_INVALID,
               "%s: outputs must be [total, 512] and [total, 1, 64]", who);
  SHIM_REQUIRE(max_seq_len > 0 && max_seq_len <= width * bs && batch <= 65535, ACLNN_ERR_PARAM_INVALID, "%s: max_seq_len outside (0, W * block]", who);
  aclOpExecutor* e = NewExecutor(OpKind::kGather, {TensorSlot(key_cache), TensorSlot(value_cache), TensorSlot(block_table), TensorSlot(seq_lens),
                                                   TensorSlot(cu_seq_lens), TensorSlot(key_out), TensorSlot(value_out)});
  e->batch = static_cast<int32_t>(batch);
  e->num_blocks = static_cast<int32_t>(blocks);
  e->block_size = static_cast<int32_t>(bs);
  e->table_width = static_cast<int32_t>(width);
  e->max_seq_len = static_cast<int32_t>(max_seq_len);
  e->key_block_stride = kb * 2;
  e->key_slot_stride = ks * 2;
  e->value_block_stride = vb * 2;
  e->value_slot_stride = vs * 2;
  e->key_row_stride = key_row * 2;
  e->value_row_stride = value_row * 2;
  *workspace_size = 0;
  *executor = e;
  return ACLNN_SUCCESS;
}

aclnnStatus aclnnGatherPaKvCache(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream) {
  if (aclnnStatus s = BeginLaunch(executor, OpKind::kGather, workspace, workspace_size, "aclnnGatherPaKvCache")) return s;
  aclOpExecutor* e = executor;
  mlakvCacheView view;
  FillView(&view, e, e->slots[0].addresses[0], e->slots[1].addresses[0]);
  const mlakvStatus status = mlakvGather(&view, 0, 1, static_cast<const int32_t*>(e->slots[2].addresses[0]), e->table_width,
                                         static_cast<const int32_t*>(e->slots[3].addresses[0]),
                                         static_cast<const int32_t*>(e->slots[4].addresses[0]), e->batch, e->max_seq_len,
                                         e->slots[5].addresses[0], 0, e->key_row_stride, e->slots[6].addresses[0], 0,
                                         e->value_row_stride, stream);
  if (status == MLAKV_SUCCESS) e->launched = true;
  return status;
}

}  // extern "C"
