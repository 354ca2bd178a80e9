/*
 * aclnn_hip.h -- the operator boundary of the reference engine, served by HIP on MI355X.
 *
 * The reference (fxslava/ascend-moe-engine) reaches its device through three C surfaces, all
 * resolved by name at run time or link time:
 *   - the two-phase aclnn operator ABI  (include/moe/core/op_table.hpp:339-454, launch ABI :1022;
 *     resolution by dlsym, src/core/op_table.cpp:95-121)
 *   - the descriptor engine            (mock/include/aclnn/acl_meta.h:59-90; used by
 *     src/memory/static_arena.cpp:131-268 and src/core/op_table.cpp:230-270)
 *   - the aclrt runtime                (mock/include/acl/acl.h:32-72; used by src/core/device_ops.cpp)
 * libmoe_kv_hip.so exports the symbols below with the same names, argument order and types,
 * so the engine's StaticMemoryArena / StaticOpSlot / PlanAclnnOp code drives the HIP kernels
 * unchanged for the two operators of the KV-cache path:
 *     aclnnScatterPaKvCache            stage "kv_cache_write"  (src/pipeline/pipeline.cpp:226-234)
 *     aclnnFusedInferAttentionScoreV5  stage "attention"       (src/pipeline/pipeline.cpp:235-249)
 * The other operators of the engine are not part of this library.
 *
 * Status convention (include/moe/core/op_table.hpp:142-147): 0 success, 161001 null
 * parameter, 161002 invalid parameter, 361001 runtime error. A launch returning 0 means
 * "enqueued"; asynchronous failures surface at synchronisation. No function throws.
 */
#ifndef ACLNN_HIP_H_
#define ACLNN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- base types (values as in the CANN headers the reference compiles against;
 *      mock/include/acl/acl_base.h:33-60, mock/include/aclnn/acl_meta.h:31-50) ---- */
typedef int32_t aclError;
typedef int32_t aclnnStatus;

#define ACL_SUCCESS 0
#define ACL_ERROR_INVALID_PARAM 100000
#define ACL_ERROR_REPEAT_INITIALIZE 100031
#define ACL_ERROR_RT_FAILURE 107000
#define ACL_ERROR_RT_STREAM_SYNC_TIMEOUT 107020
#define ACLNN_SUCCESS 0
#define ACLNN_ERR_PARAM_NULLPTR 161001
#define ACLNN_ERR_PARAM_INVALID 161002
#define ACLNN_ERR_RUNTIME_ERROR 361001

typedef enum aclDataType {
  ACL_FLOAT32 = 0, ACL_FLOAT16 = 1, ACL_INT8 = 2, ACL_INT32 = 3, ACL_UINT8 = 4, ACL_INT16 = 6, ACL_UINT16 = 7,
  ACL_INT64 = 9, ACL_UINT64 = 10, ACL_FLOAT64 = 11, ACL_BOOL = 12, ACL_DT_UNDEFINED = 17, ACL_BF16 = 27,
  ACL_FLOAT8_E5M2 = 35, ACL_FLOAT8_E4M3FN = 36, ACL_FLOAT8_E8M0 = 37, ACL_FP4X2_E2M1 = 40
} aclDataType;
typedef enum aclFormat { ACL_FORMAT_ND = 2 } aclFormat;
typedef enum aclrtMemcpyKind {
  ACL_MEMCPY_HOST_TO_HOST = 0, ACL_MEMCPY_HOST_TO_DEVICE = 1, ACL_MEMCPY_DEVICE_TO_HOST = 2, ACL_MEMCPY_DEVICE_TO_DEVICE = 3
} aclrtMemcpyKind;
typedef enum aclrtMemMallocPolicy {
  ACL_MEM_MALLOC_HUGE_FIRST = 0, ACL_MEM_MALLOC_HUGE_ONLY = 1, ACL_MEM_MALLOC_NORMAL_FIRST = 2, ACL_MEM_MALLOC_NORMAL_ONLY = 3
} aclrtMemMallocPolicy;
typedef enum aclrtMemAttr { ACL_HBM_MEM = 0, ACL_DDR_MEM = 1 } aclrtMemAttr;
#define ACL_EVENT_SYNC 0x0

typedef void* aclrtStream;  /* a hipStream_t */
typedef void* aclrtEvent;   /* a hipEvent_t */
typedef void* aclrtContext;

typedef struct aclOpExecutor aclOpExecutor;
typedef struct aclTensor aclTensor;
typedef struct aclScalar aclScalar;
typedef struct aclIntArray aclIntArray;
typedef struct aclTensorList aclTensorList;

/* ---- runtime (mock/include/acl/acl.h:32-72; callers: src/core/device_ops.cpp AclDeviceOps,
 *      src/core/acl_guard.cpp:22-46) ---- */
aclError aclInit(const char* config_path);
aclError aclFinalize(void);
aclnnStatus aclnnInit(const char* config_path);
aclnnStatus aclnnFinalize(void);
const char* aclGetRecentErrMsg(void);
aclError aclrtSetDevice(int32_t device_id);
aclError aclrtResetDevice(int32_t device_id);
aclError aclrtCreateContext(aclrtContext* context, int32_t device_id);
aclError aclrtDestroyContext(aclrtContext context);
aclError aclrtSetCurrentContext(aclrtContext context);
aclError aclrtGetDeviceCount(uint32_t* device_count);
const char* aclrtGetSocName(void);
/* Device memory is at least 4096-byte aligned, as the reference requires of every backend
 * (include/moe/core/device_allocator.hpp:36-39). */
aclError aclrtMalloc(void** device_ptr, size_t size, aclrtMemMallocPolicy policy);
aclError aclrtFree(void* device_ptr);
aclError aclrtMallocHost(void** host_ptr, size_t size); /* pinned */
aclError aclrtFreeHost(void* host_ptr);
/* destination_capacity is the caller's proof of room; count > capacity is refused. */
aclError aclrtMemcpy(void* destination, size_t destination_capacity, const void* source, size_t count, aclrtMemcpyKind kind);
aclError aclrtMemcpyAsync(void* destination, size_t destination_capacity, const void* source, size_t count,
                          aclrtMemcpyKind kind, aclrtStream stream);
aclError aclrtMemset(void* destination, size_t destination_capacity, int32_t value, size_t count);
aclError aclrtCreateStream(aclrtStream* stream);
aclError aclrtDestroyStream(aclrtStream stream);
aclError aclrtDestroyStreamForce(aclrtStream stream);
aclError aclrtCreateEventExWithFlag(aclrtEvent* event, uint32_t flag);
aclError aclrtDestroyEvent(aclrtEvent event);
aclError aclrtRecordEvent(aclrtEvent event, aclrtStream stream);
aclError aclrtStreamWaitEvent(aclrtStream stream, aclrtEvent event);
aclError aclrtSynchronizeStream(aclrtStream stream);
aclError aclrtSynchronizeStreamWithTimeout(aclrtStream stream, int32_t timeout_ms);
aclError aclrtSynchronizeEvent(aclrtEvent event);
aclError aclrtGetMemInfo(aclrtMemAttr attr, size_t* free_bytes, size_t* total_bytes);

/* ---- stream capture: a step enqueued once, replayed as one launch ----
 * Named after CANN's stream-capture entry points (aclmdlRICaptureBegin / CaptureEnd / ExecuteAsync /
 * Destroy; CANN is not installed here, so the match with its headers is unchecked). The reference
 * does not call them (its loop enqueues every operator every step, src/pipeline/pipeline.cpp:390-416),
 * so nothing of the reference binds to these. Served by a
 * HIP graph: everything enqueued on `stream` between Begin and End (operator launches, asynchronous
 * copies to or from pinned host memory) is recorded instead of run; ExecuteAsync enqueues the whole
 * recording on a stream. Addresses and host-side arguments are those of the recording; what changes
 * from replay to replay has to live in memory the recording reads (a pinned host word copied by a
 * recorded aclrtMemcpyAsync, device lengths bound with aclnnMlaKvBindSeqLens). The first launch of
 * every operator on a device must have happened before Begin (it sets up the kernels). */
typedef void* aclmdlRI;
typedef enum {
  ACL_MODEL_RI_CAPTURE_MODE_GLOBAL = 0,
  ACL_MODEL_RI_CAPTURE_MODE_THREAD_LOCAL = 1,
  ACL_MODEL_RI_CAPTURE_MODE_RELAXED = 2
} aclmdlRICaptureMode;
aclError aclmdlRICaptureBegin(aclrtStream stream, aclmdlRICaptureMode mode);
aclError aclmdlRICaptureEnd(aclrtStream stream, aclmdlRI* model_ri);
aclError aclmdlRIExecuteAsync(aclmdlRI model_ri, aclrtStream stream);
aclError aclmdlRIDestroy(aclmdlRI model_ri);

/* ---- descriptor engine (mock/include/aclnn/acl_meta.h:59-90) ----
 * Dims and strides count ELEMENTS. The getters return arrays allocated with new[]; the
 * caller releases them with delete[] (src/memory/static_arena.cpp:181-188). A tensor list owns
 * the tensor handles it was built from; destroying the list destroys them
 * (src/memory/static_arena.cpp:172-208). */
aclTensor* aclCreateTensor(const int64_t* view_dims, uint64_t view_dims_num, aclDataType dtype, const int64_t* view_strides,
                           int64_t storage_offset, aclFormat format, const int64_t* storage_dims,
                           uint64_t storage_dims_num, void* device_data);
aclnnStatus aclDestroyTensor(const aclTensor* tensor);
aclnnStatus aclGetViewShape(const aclTensor* tensor, int64_t** dims, uint64_t* count);
aclnnStatus aclGetStorageShape(const aclTensor* tensor, int64_t** dims, uint64_t* count);
aclnnStatus aclGetViewStrides(const aclTensor* tensor, int64_t** strides, uint64_t* count);
aclnnStatus aclGetDataType(const aclTensor* tensor, aclDataType* dtype);
aclnnStatus aclGetFormat(const aclTensor* tensor, aclFormat* format);
aclnnStatus aclGetRawTensorAddr(const aclTensor* tensor, void** address);
aclnnStatus aclGetViewOffset(const aclTensor* tensor, int64_t* offset);
aclTensorList* aclCreateTensorList(const aclTensor* const* tensors, uint64_t size);
aclnnStatus aclDestroyTensorList(const aclTensorList* tensor_list);
aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size); /* copies the values */
aclnnStatus aclDestroyIntArray(const aclIntArray* array);
aclScalar* aclCreateScalar(void* value, aclDataType dtype);
aclnnStatus aclDestroyScalar(const aclScalar* scalar);
/* Address swaps on a planned executor (src/core/op_table.cpp:245-258). `index` is the IR
 * index of the argument: its position among the tensor / tensor-list / int-array arguments
 * of the plan call, nulls included (include/moe/pipeline/pipeline.hpp:176-184:
 * scatter keyCacheRef = 1, valueCacheRef = 4; attention key[] = 1, value[] = 2, keyRope = 25). */
aclnnStatus aclSetTensorAddr(aclOpExecutor* executor, uint64_t index, const aclTensor* tensor, void* address);
aclnnStatus aclSetDynamicTensorAddr(aclOpExecutor* executor, uint64_t ir_index, uint64_t relative_index,
                                    const aclTensorList* tensor_list, void* address);
aclnnStatus aclSetAclOpExecutorRepeatable(aclOpExecutor* executor);
aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor);

/* ---- operators ---- */

/* include/moe/core/op_table.hpp:365-372 (ScatterPaKvCachePlanFn). Served subset, which is the
 * reference's call (src/pipeline/pipeline.cpp:229-233): key [T,512] and value [T,1,64] bf16,
 * caches [blocks, block, 1, dim] bf16, slot mapping int32 [T], cache mode "Norm", every
 * compression argument null. Returns workspace 0. */
aclnnStatus aclnnScatterPaKvCacheGetWorkspaceSize(const aclTensor* key, aclTensor* key_cache_ref, const aclTensor* slot_mapping,
                                                  const aclTensor* value, aclTensor* value_cache_ref,
                                                  const aclTensor* compress_lens_optional,
                                                  const aclTensor* compress_seq_offset_optional,
                                                  const aclTensor* seq_lens_optional, char* cache_mode_optional,
                                                  char* scatter_mode_optional, const aclIntArray* strides_optional,
                                                  const aclIntArray* offsets_optional, uint64_t* workspace_size,
                                                  aclOpExecutor** executor);
/* include/moe/core/op_table.hpp:1022 (AclnnLaunchFn) */
aclnnStatus aclnnScatterPaKvCache(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream);

/* include/moe/core/op_table.hpp:438-454 (FusedInferAttentionScoreV5PlanFn). Served subset, the
 * reference's call (src/pipeline/pipeline.cpp:237-248): query [T,N,512] and query_rope [T,N,64]
 * bf16 views (any element strides), one key tensor and one value tensor that alias the same
 * paged latent cache [blocks, block, 1, 512], key_rope [blocks, block, 1, 64], block_table
 * int32 [T, W], one query token per sequence, layout "TND", num_key_value_heads 1, no masks,
 * no quantisation arguments. actual_seq_lengths_kv holds one length per sequence; its values
 * are copied at plan time (the reference fixes them there, src/memory/static_arena_manager.cpp:
 * 584-588). A caller that attends over the live context, not the reserved one, updates them
 * with aclnnMlaKvSetSeqLens (host values) or aclnnMlaKvBindSeqLens (a device array). The
 * workspace covers the partials of sequences split over several workgroups and the lengths. */
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
    const aclTensor* softmax_lse, uint64_t* workspace_size, aclOpExecutor** executor);
aclnnStatus aclnnFusedInferAttentionScoreV5(void* workspace, uint64_t workspace_size, aclOpExecutor* executor,
                                            aclrtStream stream);

/* aclnnDynamicMxQuant, as the reference plans and launches it behind the attention (stage
 * `attn_quant`, src/pipeline/pipeline.cpp:251-258; contract include/moe/core/op_table.hpp:205-233):
 * x bf16 [rows, cols] (cols a multiple of 32, dense last axis) -> y E4M3 [rows, cols] and
 * mxscale E8M0 [rows, cols / 32]; axis -1, round mode "rint" (or null), dst_type 36, blocksize
 * 32, scale_alg 0 (OCP). IR indices: x 0, y 1, mxscale 2. No workspace. */
aclnnStatus aclnnDynamicMxQuantGetWorkspaceSize(const aclTensor* x, int64_t axis, char* round_mode_optional, int64_t dst_type,
                                                int64_t blocksize, int64_t scale_alg, const aclTensor* y_out,
                                                const aclTensor* mxscale_out, uint64_t* workspace_size, aclOpExecutor** executor);
aclnnStatus aclnnDynamicMxQuant(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream);

/* aclnnQuantLightningIndexer for decode (contract include/moe/core/op_table.hpp:964-1006; the
 * reference's op table requires the symbol, src/core/op_table.cpp:87-88): query E4M3
 * [B, 1, N1, 128] with N1 in {16, 32, 48, 64}; key E4M3 paged [blocks, block, 1, 128] (layout
 * "PA_BSND"); weights BF16 [B, 1, N1]; query_dequant_scale FP32 [B, 1, N1]; key_dequant_scale FP32
 * [blocks, block, 1]; actual_seq_lengths_key INT32 [B] and block_table INT32 [B, W] (device
 * tensors, both required); quant modes 0; layout_query "BSND" or null; sparse_count in [1, 2048];
 * sparse_mode 0 or 3 (the same thing for one query token); pre/next tokens INT64_MAX; out INT32
 * [B, 1, 1, sparse_count]. IR indices: query 0, key 1, weights 2, query_dequant_scale 3,
 * key_dequant_scale 4, actual_seq_lengths_query 5, actual_seq_lengths_key 6, block_table 7,
 * out 8. The workspace holds the 16-bit scores of W * block tokens per sequence. */
aclnnStatus aclnnQuantLightningIndexerGetWorkspaceSize(const aclTensor* query, const aclTensor* key, const aclTensor* weights,
                                                       const aclTensor* query_dequant_scale, const aclTensor* key_dequant_scale,
                                                       const aclTensor* actual_seq_lengths_query_optional,
                                                       const aclTensor* actual_seq_lengths_key_optional,
                                                       const aclTensor* block_table_optional, int64_t query_quant_mode,
                                                       int64_t key_quant_mode, char* layout_query_optional,
                                                       char* layout_key_optional, int64_t sparse_count, int64_t sparse_mode,
                                                       int64_t pre_tokens, int64_t next_tokens, const aclTensor* out,
                                                       uint64_t* workspace_size, aclOpExecutor** executor);
aclnnStatus aclnnQuantLightningIndexer(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream);

/* EXTENSION (the reference has no such operator: its paged read is implicit in the attention
 * operator). Block-table gather as a two-phase operator, for callers that want the paged read the
 * reference leaves inside its attention operator (addressing as in third_party/ops_transformer/
 * attention/quant_lightning_indexer/op_kernel/arch35/quant_lightning_indexer_service_cube.h:243-270).
 * key_cache / value_cache [blocks, block, 1, dim] bf16; block_table int32 [B, W]; seq_lens and
 * cu_seq_lens int32 device tensors [B] and [B+1]; key_out [total, 512] and value_out
 * [total, 1, 64] bf16 views (any row stride). IR indices: key_cache 0, value_cache 1,
 * block_table 2, seq_lens 3, cu_seq_lens 4, key_out 5, value_out 6. */
aclnnStatus aclnnGatherPaKvCacheGetWorkspaceSize(const aclTensor* key_cache, const aclTensor* value_cache,
                                                 const aclTensor* block_table, const aclTensor* seq_lens,
                                                 const aclTensor* cu_seq_lens, aclTensor* key_out, aclTensor* value_out,
                                                 int64_t max_seq_len, uint64_t* workspace_size, aclOpExecutor** executor);
aclnnStatus aclnnGatherPaKvCache(void* workspace, uint64_t workspace_size, aclOpExecutor* executor, aclrtStream stream);

/* EXTENSION (no reference counterpart: the reference fixes the length at build time,
 * src/memory/static_arena_manager.cpp:584-588). Replaces the kv lengths of a planned attention
 * executor by `count` = T host values, each in [0, table width * block size]; they are copied, and
 * every later launch carries them in the attention kernels' own argument block (T <= 64) or sends
 * them to the device in the argument block of a small kernel in front of it. */
aclnnStatus aclnnMlaKvSetSeqLens(aclOpExecutor* executor, const int64_t* seq_lens, uint64_t count);
/* EXTENSION (no reference counterpart, as above). Binds a device int32 array [T] of live context
 * lengths to a planned attention executor; it then replaces the host values, with no per-launch
 * copy. NULL unbinds. */
aclnnStatus aclnnMlaKvBindSeqLens(aclOpExecutor* executor, const int32_t* device_seq_lens);
/* EXTENSION (no reference counterpart, as above). With lengths bound to device memory the launch
 * cannot see them and chooses its kernels for the reserved context. A caller that knows a bound the
 * lengths stay under (a recorded step's loop knows its position) says so here: `longest` then
 * decides the kernels (short contexts have faster ones), and a device length above it is read as
 * `longest`. -1 withdraws the bound; binding another array withdraws it too. */
aclnnStatus aclnnMlaKvSetSeqLenBound(aclOpExecutor* executor, int64_t longest);

#ifdef __cplusplus
}
#endif
#endif /* ACLNN_HIP_H_ */
