// The thin C ABI (include/mlakv.h): argument validation, status codes and error text around
// the kernel launchers and the host classes. Nothing here touches data.
#include "mlakv.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>

#include "../kernels/kernels.h"
#include "abi_common.h"
#include "moe_hip/kv_cache_manager.hpp"
#include "moe_hip/static_arena.hpp"

static_assert(MLAKV_NOALLOC_SCRATCH_BYTES == mlakv::kAttnStaticScratchBytes, "header and kernel file agree on the scratch size");

namespace mlakv_abi {

static thread_local std::string g_last_error;

mlakvStatus Fail(mlakvStatus code, const char* format, ...) {
  char buffer[1024];
  va_list args;
  va_start(args, format);
  std::vsnprintf(buffer, sizeof(buffer), format, args);
  va_end(args);
  g_last_error = buffer;
  return code;
}

mlakvStatus FailText(mlakvStatus code, const std::string& text) {
  g_last_error = text;
  return code;
}

const char* LastError() { return g_last_error.c_str(); }

int ComputeUnits() {
  static const int units = [] {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return 256;  // MI355X figure, for planning without a device
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return 256;
    return prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }();
  return units;
}

mlakvStatus CheckView(const mlakvCacheView* cache, const char* who) {
  if (cache == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: cache view is null", who);
  if (cache->latent == nullptr || cache->rope == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: cache planes are null", who);
  if (cache->latent_dim != mlakv::kLatentDim || cache->rope_dim != mlakv::kRopeDim) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: kernels are built for latent %d + rope %d, got %d + %d", who, mlakv::kLatentDim,
                mlakv::kRopeDim, cache->latent_dim, cache->rope_dim);
  }
  if (cache->dtype != MLAKV_DTYPE_BF16 && cache->dtype != MLAKV_DTYPE_FP8_E4M3) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: unknown cache dtype %d", who, cache->dtype);
  }
  if (cache->dtype == MLAKV_DTYPE_FP8_E4M3 && cache->scale == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: an FP8 cache needs its scale plane", who);
  }
  if (cache->block_size <= 0 || cache->num_blocks <= 0 || cache->num_layers <= 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: block_size %d, num_blocks %d, num_layers %d must be positive", who,
                cache->block_size, cache->num_blocks, cache->num_layers);
  }
  const int64_t strides[] = {cache->latent_layer_stride, cache->latent_block_stride, cache->latent_row_stride,
                             cache->rope_layer_stride,   cache->rope_block_stride,   cache->rope_row_stride};
  for (int64_t stride : strides) {
    if (stride % 16 != 0) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: cache stride %lld is not a multiple of 16 bytes", who, static_cast<long long>(stride));
    }
  }
  if (reinterpret_cast<uintptr_t>(cache->latent) % 16 != 0 || reinterpret_cast<uintptr_t>(cache->rope) % 16 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: cache plane addresses must be 16-byte aligned", who);
  }
  if (cache->scale != nullptr && (reinterpret_cast<uintptr_t>(cache->scale) % 4 != 0 || cache->scale_layer_stride % 4 != 0 ||
                                  cache->scale_block_stride % 4 != 0)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: scale plane must be 4-byte aligned", who);
  }
  return MLAKV_SUCCESS;
}

mlakvStatus CheckLayers(const mlakvCacheView* cache, int32_t begin, int32_t count, const char* who) {
  if (begin < 0 || count < 0 || begin + count > cache->num_layers) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: layers [%d, %d) outside the cache's %d layers", who, begin, begin + count,
                cache->num_layers);
  }
  return MLAKV_SUCCESS;
}

mlakv::Plane PlaneAt(void* base, int64_t layer_stride, int64_t block_stride, int64_t row_stride, int32_t layer) {
  mlakv::Plane plane;
  plane.base = base == nullptr ? nullptr : static_cast<char*>(base) + static_cast<int64_t>(layer) * layer_stride;
  plane.layer_stride = layer_stride;
  plane.block_stride = block_stride;
  plane.row_stride = row_stride;
  return plane;
}

void FillPlanes(const mlakvCacheView* cache, int32_t layer, mlakv::Plane* latent, mlakv::Plane* rope, mlakv::Plane* scale) {
  *latent = PlaneAt(cache->latent, cache->latent_layer_stride, cache->latent_block_stride, cache->latent_row_stride, layer);
  *rope = PlaneAt(cache->rope, cache->rope_layer_stride, cache->rope_block_stride, cache->rope_row_stride, layer);
  *scale = PlaneAt(cache->scale, cache->scale_layer_stride, cache->scale_block_stride, 4, layer);
}

mlakvStatus HipFail(hipError_t status, const char* who) {
  return Fail(MLAKV_ERR_RUNTIME, "%s: %s", who, hipGetErrorString(status));
}

bool Aligned16(const void* pointer) { return reinterpret_cast<uintptr_t>(pointer) % 16 == 0; }

}  // namespace mlakv_abi

using namespace mlakv_abi;

extern "C" {

const char* mlakvGetLastError(void) { return LastError(); }

mlakvStatus mlakvPrepare(void) {
  for (hipError_t (*prepare)() : {mlakv::PrepareAttnKernels, mlakv::PreparePagedCopyKernels, mlakv::PrepareIndexerKernels,
                                   mlakv::PrepareMxQuantKernels}) {
    if (const hipError_t status = prepare(); status != hipSuccess) return HipFail(status, "mlakvPrepare");
  }
  return MLAKV_SUCCESS;
}

int32_t mlakvDeviceCount(void) {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess) return 0;
  return count;
}

// ---- kernels ----------------------------------------------------------------------

mlakvStatus mlakvAppend(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count, const void* latent_src,
                        int64_t latent_src_layer_stride, int64_t latent_src_row_stride, const void* rope_src,
                        int64_t rope_src_layer_stride, int64_t rope_src_row_stride, const int32_t* slot_mapping,
                        int32_t num_tokens, void* stream) {
  if (mlakvStatus s = CheckView(cache, "mlakvAppend")) return s;
  if (mlakvStatus s = CheckLayers(cache, layer_begin, layer_count, "mlakvAppend")) return s;
  if (num_tokens < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvAppend: negative token count");
  if (num_tokens == 0 || layer_count == 0) return MLAKV_SUCCESS;
  if (latent_src == nullptr || rope_src == nullptr || slot_mapping == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvAppend: source rows and slot mapping are required");
  }
  if (!Aligned16(latent_src) || !Aligned16(rope_src) || latent_src_row_stride % 16 != 0 || rope_src_row_stride % 16 != 0 ||
      latent_src_layer_stride % 16 != 0 || rope_src_layer_stride % 16 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvAppend: source rows must be 16-byte aligned with 16-byte-multiple strides");
  }
  mlakv::AppendArgs args{};
  FillPlanes(cache, layer_begin, &args.latent, &args.rope, &args.scale);
  args.latent_src = {const_cast<char*>(static_cast<const char*>(latent_src)), latent_src_layer_stride, latent_src_row_stride};
  args.rope_src = {const_cast<char*>(static_cast<const char*>(rope_src)), rope_src_layer_stride, rope_src_row_stride};
  args.slots = slot_mapping;
  args.num_tokens = num_tokens;
  args.num_layers = layer_count;
  args.num_blocks = cache->num_blocks;
  args.block_size = cache->block_size;
  args.fp8 = cache->dtype == MLAKV_DTYPE_FP8_E4M3;
  const hipError_t status = mlakv::LaunchAppend(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, "mlakvAppend");
}

mlakvStatus mlakvNormRopeAppend(const mlakvCacheView* cache, int32_t layer, const void* kv_a, int64_t kv_a_row_stride,
                                const void* gamma, double epsilon, const void* rope_cos, const void* rope_sin,
                                int64_t rope_table_row_stride, const int32_t* positions, const int32_t* slot_mapping,
                                int32_t num_tokens, void* latent_normed_out, int64_t latent_normed_row_stride,
                                void* rope_out, int64_t rope_out_row_stride, void* q_rope, int64_t q_rope_token_stride,
                                int64_t q_rope_head_stride, int32_t num_heads, void* stream) {
  const char* who = "mlakvNormRopeAppend";
  if (mlakvStatus s = CheckView(cache, who)) return s;
  if (mlakvStatus s = CheckLayers(cache, layer, 1, who)) return s;
  if (num_tokens < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: negative token count", who);
  if (num_tokens == 0) return MLAKV_SUCCESS;
  if (kv_a == nullptr || gamma == nullptr || rope_cos == nullptr || rope_sin == nullptr || positions == nullptr ||
      slot_mapping == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: rows, gamma, rope tables, positions and slot mapping are required", who);
  }
  if (!(epsilon > 0.0) || !std::isfinite(epsilon)) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a positive epsilon is required", who);
  if (!Aligned16(kv_a) || kv_a_row_stride % 16 != 0 || !Aligned16(gamma)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: kv_a rows and gamma must be 16-byte aligned, the row stride a multiple of 16", who);
  }
  if (kv_a_row_stride < (cache->latent_dim + cache->rope_dim) * 2) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a kv_a row holds latent and rope, %d bytes", who, (cache->latent_dim + cache->rope_dim) * 2);
  }
  if (rope_table_row_stride % 2 != 0 || rope_table_row_stride < cache->rope_dim * 2 ||
      reinterpret_cast<uintptr_t>(rope_cos) % 2 != 0 || reinterpret_cast<uintptr_t>(rope_sin) % 2 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: rope table rows hold %d bf16 values", who, cache->rope_dim);
  }
  if ((latent_normed_out != nullptr && (!Aligned16(latent_normed_out) || latent_normed_row_stride % 16 != 0)) ||
      (rope_out != nullptr && (reinterpret_cast<uintptr_t>(rope_out) % 2 != 0 || rope_out_row_stride % 2 != 0))) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: optional outputs must be aligned to their element groups (16 / 2 bytes)", who);
  }
  if (q_rope != nullptr) {
    if (num_heads <= 0 || num_heads > 4096) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: query rope needs a head count in [1, 4096]", who);
    if (!Aligned16(q_rope) || q_rope_token_stride % 16 != 0 || q_rope_head_stride % 16 != 0 ||
        q_rope_head_stride < cache->rope_dim * 2 || q_rope_token_stride < q_rope_head_stride * num_heads) {
      return Fail(MLAKV_ERR_PARAM_INVALID,
                  "%s: query rope slices must be 16-byte aligned with strides that are multiples of 16 and do not overlap", who);
    }
    if (!Aligned16(rope_cos) || !Aligned16(rope_sin) || rope_table_row_stride % 16 != 0) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: with query rope the table rows must be 16-byte aligned", who);
    }
    if (static_cast<int64_t>(num_tokens) * (1 + (num_heads + 7) / 8) > (int64_t{1} << 30)) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: too many (token, head group) items for one launch", who);
    }
  }
  mlakv::NormRopeAppendArgs args{};
  FillPlanes(cache, layer, &args.append.latent, &args.append.rope, &args.append.scale);
  args.append.slots = slot_mapping;
  args.append.num_tokens = num_tokens;
  args.append.num_layers = 1;
  args.append.num_blocks = cache->num_blocks;
  args.append.block_size = cache->block_size;
  args.append.fp8 = cache->dtype == MLAKV_DTYPE_FP8_E4M3;
  args.kv_a = static_cast<const char*>(kv_a);
  args.kv_a_row_stride = kv_a_row_stride;
  args.gamma = static_cast<const char*>(gamma);
  args.epsilon = static_cast<float>(epsilon);
  args.rope_cos = static_cast<const char*>(rope_cos);
  args.rope_sin = static_cast<const char*>(rope_sin);
  args.rope_table_row_stride = rope_table_row_stride;
  args.positions = positions;
  args.latent_out = static_cast<char*>(latent_normed_out);
  args.latent_out_row_stride = latent_normed_row_stride;
  args.rope_out = static_cast<char*>(rope_out);
  args.rope_out_row_stride = rope_out_row_stride;
  args.q_rope = static_cast<char*>(q_rope);
  args.q_rope_token_stride = q_rope_token_stride;
  args.q_rope_head_stride = q_rope_head_stride;
  args.num_heads = q_rope != nullptr ? num_heads : 0;
  const hipError_t status = mlakv::LaunchNormRopeAppend(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
}

static mlakvStatus GatherImpl(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count, const int32_t* block_table,
                              int32_t table_stride, const int32_t* seq_lens, const int32_t* cu_seq_lens, int32_t batch,
                              int32_t max_seq_len, void* latent_dst, int64_t latent_dst_layer_stride,
                              int64_t latent_dst_row_stride, void* rope_dst, int64_t rope_dst_layer_stride,
                              int64_t rope_dst_row_stride, void* stream, void* start_event, void* stop_event) {
  if (mlakvStatus s = CheckView(cache, "mlakvGather")) return s;
  if (mlakvStatus s = CheckLayers(cache, layer_begin, layer_count, "mlakvGather")) return s;
  if (batch < 0 || max_seq_len < 0 || table_stride < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvGather: negative size");
  if (batch == 0 || layer_count == 0 || max_seq_len == 0) return MLAKV_SUCCESS;
  if (block_table == nullptr || seq_lens == nullptr || cu_seq_lens == nullptr || latent_dst == nullptr || rope_dst == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvGather: block table, lengths and destinations are required");
  }
  if (static_cast<int64_t>(table_stride) * cache->block_size < max_seq_len) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvGather: a table row of %d blocks cannot address %d tokens", table_stride, max_seq_len);
  }
  if (batch > 65535 || layer_count > 65535) return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvGather: batch/layers exceed the launch grid");
  if (!Aligned16(latent_dst) || !Aligned16(rope_dst) || latent_dst_row_stride % 16 != 0 || rope_dst_row_stride % 16 != 0 ||
      latent_dst_layer_stride % 16 != 0 || rope_dst_layer_stride % 16 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvGather: destination rows must be 16-byte aligned with 16-byte-multiple strides");
  }
  mlakv::GatherArgs args{};
  FillPlanes(cache, layer_begin, &args.latent, &args.rope, &args.scale);
  args.latent_dst = {static_cast<char*>(latent_dst), latent_dst_layer_stride, latent_dst_row_stride};
  args.rope_dst = {static_cast<char*>(rope_dst), rope_dst_layer_stride, rope_dst_row_stride};
  args.block_table = block_table;
  args.table_stride = table_stride;
  args.seq_lens = seq_lens;
  args.cu_seq_lens = cu_seq_lens;
  args.batch = batch;
  args.max_seq_len = max_seq_len;
  args.num_layers = layer_count;
  args.num_blocks = cache->num_blocks;
  args.block_size = cache->block_size;
  args.fp8 = cache->dtype == MLAKV_DTYPE_FP8_E4M3;
  const hipError_t status = mlakv::LaunchGather(args, static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(start_event),
                                                static_cast<hipEvent_t>(stop_event));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, "mlakvGather");
}

mlakvStatus mlakvGather(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count, const int32_t* block_table,
                        int32_t table_stride, const int32_t* seq_lens, const int32_t* cu_seq_lens, int32_t batch,
                        int32_t max_seq_len, void* latent_dst, int64_t latent_dst_layer_stride,
                        int64_t latent_dst_row_stride, void* rope_dst, int64_t rope_dst_layer_stride,
                        int64_t rope_dst_row_stride, void* stream) {
  return GatherImpl(cache, layer_begin, layer_count, block_table, table_stride, seq_lens, cu_seq_lens, batch, max_seq_len, latent_dst,
                    latent_dst_layer_stride, latent_dst_row_stride, rope_dst, rope_dst_layer_stride, rope_dst_row_stride, stream,
                    nullptr, nullptr);
}

mlakvStatus mlakvGatherTimed(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count, const int32_t* block_table,
                             int32_t table_stride, const int32_t* seq_lens, const int32_t* cu_seq_lens, int32_t batch,
                             int32_t max_seq_len, void* latent_dst, int64_t latent_dst_layer_stride,
                             int64_t latent_dst_row_stride, void* rope_dst, int64_t rope_dst_layer_stride,
                             int64_t rope_dst_row_stride, void* stream, void* start_event, void* stop_event) {
  if (start_event == nullptr || stop_event == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvGatherTimed: both events are required");
  }
  if (batch == 0 || layer_count == 0 || max_seq_len == 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvGatherTimed: an empty gather launches nothing, so there is nothing to time");
  }
  return GatherImpl(cache, layer_begin, layer_count, block_table, table_stride, seq_lens, cu_seq_lens, batch, max_seq_len, latent_dst,
                    latent_dst_layer_stride, latent_dst_row_stride, rope_dst, rope_dst_layer_stride, rope_dst_row_stride, stream,
                    start_event, stop_event);
}

mlakvStatus mlakvCopyBlocks(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count, const int32_t* moves,
                            int32_t num_moves, void* stream) {
  if (mlakvStatus s = CheckView(cache, "mlakvCopyBlocks")) return s;
  if (mlakvStatus s = CheckLayers(cache, layer_begin, layer_count, "mlakvCopyBlocks")) return s;
  if (num_moves < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvCopyBlocks: negative move count");
  if (num_moves == 0 || layer_count == 0) return MLAKV_SUCCESS;
  if (moves == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvCopyBlocks: moves is null");
  if (layer_count > 65535) return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvCopyBlocks: layers exceed the launch grid");
  mlakv::CopyBlocksArgs args{};
  FillPlanes(cache, layer_begin, &args.latent, &args.rope, &args.scale);
  args.moves = moves;
  args.num_moves = num_moves;
  args.num_layers = layer_count;
  args.num_blocks = cache->num_blocks;
  args.block_size = cache->block_size;
  const int32_t element = cache->dtype == MLAKV_DTYPE_BF16 ? 2 : 1;
  args.latent_row_bytes = element * cache->latent_dim;
  args.rope_row_bytes = element * cache->rope_dim;
  args.has_scale = cache->dtype == MLAKV_DTYPE_FP8_E4M3;
  const hipError_t status = mlakv::LaunchCopyBlocks(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, "mlakvCopyBlocks");
}

}  // extern "C"

namespace {

constexpr int32_t kDefaultMergeSpinUs = 50;
static_assert(MLAKV_ATTN_HEAD_BLOCK_TOKENS == mlakv::kAttnHeadBlockTokens, "the header states the kernel's staging size");

// The largest unit (in tiles) whose block-table entries fit the kernel's LDS staging whatever
// the unit's offset inside a block; a selection stages one entry per selected token.
int64_t CapUnitTiles(int32_t block_size, bool sparse) {
  if (sparse) return mlakv::kAttnTableEntries / mlakv::kTileTokens;
  const int64_t cap = ((static_cast<int64_t>(mlakv::kAttnTableEntries) - 2) * block_size + 2) / mlakv::kTileTokens;
  return cap < 1 ? 1 : cap;
}

struct PlanShape {
  int64_t max_tiles, head_groups, cap, units;
  uint64_t workspace;
};

// What follows from a plan's own fields; the launch recomputes it to refuse a plan that was not
// made by the init functions.
PlanShape ShapeOf(int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size, bool sparse, int32_t chunk_tiles,
                  int32_t work_groups, bool halved_units) {
  PlanShape shape;
  shape.max_tiles = (static_cast<int64_t>(max_seq_len) + mlakv::kTileTokens - 1) / mlakv::kTileTokens;
  shape.head_groups = (heads + 63) / 64;
  shape.cap = CapUnitTiles(block_size, sparse);
  // the longest flat axis a launch can see: every sequence full, each with its idle positions in front
  const int64_t total = static_cast<int64_t>(batch) * (shape.max_tiles + mlakv::kAttnBoundaryTiles);
  if (chunk_tiles > 0) {
    shape.units = (total + chunk_tiles - 1) / chunk_tiles;
  } else {
    const int64_t capped = (total + shape.cap - 1) / shape.cap;
    shape.units = capped > work_groups ? capped : work_groups;
  }
  const uint64_t rows = static_cast<uint64_t>(shape.head_groups) * static_cast<uint64_t>(shape.units + batch) * 64;
  // bf16 partial outputs, then fp32 partial log-sum-exps
  shape.workspace = rows * mlakv::kLatentDim * 2 + ((rows * sizeof(float) + 255) & ~255ull);
  // Halved whole-selection units: two partials of 16 rows per (sequence, 16 heads) and, behind the
  // rows of all of them, their LSEs (2 x 4 x 16 floats each).
  const uint64_t halved = static_cast<uint64_t>(batch) * (heads / 16) * (32 * mlakv::kLatentDim * 2 + 2 * 4 * 16 * sizeof(float));
  if (halved_units && halved > shape.workspace) shape.workspace = halved;
  return shape;
}

// How a whole-context launch whose longest context is `bound` tokens cuts its work: 0 = the
// 64-head kernel's flat cut, 1 = one workgroup per (sequence, 16 heads), 2 = two. Measured on
// MI355X, bf16 and FP8 caches alike (64 heads unless said; us, 64-head kernel / one workgroup per
// unit / two): batch 1 .. 32 (and 16 x 128, 64 x 16 heads), 128 tokens 14.5-16.8 / 8.3-8.5 / 8.7-9.9;
// 256: 17.0-19.2 / 10.3-11.4 / 10.1-11.6; 512: 16.4-21.4 / 15.4-17.7 / 12.8-15.0; 768: 16.5-22.5 /
// 20.8-24.0 / 15.5-18.7; 1024: 16.7-25.6 / 26.1-29.6 / 18.3-22.9. Batch 48, 64 (32 x 128): 256:
// 21.1-22.9 / 12.0-12.8; 512: 21.3-23.9 / 17.9-20.3; 768: 23.7-26.8 / 24.4-37.5. Batch 96, 128
// (64 x 128), two rounds of units: 256: 24.8-27.6 / 21.1-24.6; 384: 27.5-30.4 / 27.2-32.1. Batch 256:
// 128: 29.0 / 31.8.
int32_t ShortContextUnits(const mlakvAttnPlan* plan, int32_t bound) {
  if (plan->selection_units == MLAKV_ATTN_UNITS_SPLIT || bound > MLAKV_ATTN_HEAD_BLOCK_TOKENS) return 0;
  if (plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK) return 1;
  if (plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES) return 2;
  const int64_t pairs = static_cast<int64_t>(plan->batch) * (plan->heads / 16);
  if (2 * pairs <= ComputeUnits()) return bound <= 256 ? 1 : (bound <= 768 ? 2 : 0);
  if (pairs <= ComputeUnits()) return bound <= 512 ? 1 : 0;
  if (pairs <= 2 * ComputeUnits()) return bound <= 256 ? 1 : 0;
  return 0;
}

mlakvStatus AttnPlanImpl(const char* who, int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size,
                         int32_t dtype, bool sparse, const mlakvAttnPlanOptions* options, mlakvAttnPlan* plan) {
  if (plan == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: plan is null", who);
  if (batch <= 0 || batch > 65535) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: batch %d outside [1, 65535]", who, batch);
  if (heads <= 0 || heads % 16 != 0 || heads > 128) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: heads %d must be a multiple of 16 up to 128", who, heads);
  }
  if (max_seq_len <= 0 || block_size <= 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: sizes must be positive", who);
  if (dtype != MLAKV_DTYPE_BF16 && dtype != MLAKV_DTYPE_FP8_E4M3) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: unknown cache dtype %d", who, dtype);
  }
  mlakvAttnPlanOptions chosen{};
  if (options != nullptr) chosen = *options;
  if (chosen.chunk_tiles < 0 || chosen.work_groups < 0 || chosen.work_groups > 65535 || chosen.merge_mode < 0 ||
      chosen.merge_mode > MLAKV_ATTN_MERGE_SECOND_LAUNCH || chosen.merge_spin_us > 1000000 || chosen.selection_units < 0 ||
      chosen.selection_units > MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: options outside their ranges", who);
  }
  const int64_t head_groups = (heads + 63) / 64;
  const int64_t cap = CapUnitTiles(block_size, sparse);
  int32_t work_groups = chosen.work_groups;
  if (work_groups == 0) {
    // One workgroup occupies a whole CU (a ring of four 36 KB tile buffers).
    work_groups = static_cast<int32_t>(ComputeUnits() / head_groups);
    if (work_groups < 1) work_groups = 1;
  }
  int32_t chunk_tiles = chosen.chunk_tiles;
  if (chunk_tiles > cap) chunk_tiles = static_cast<int32_t>(cap);
  PlanShape shape = ShapeOf(batch, heads, max_seq_len, block_size, sparse, chunk_tiles, work_groups, false);
  if (shape.units > (int64_t{1} << 30)) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: too many work units (%lld)", who, static_cast<long long>(shape.units));
  plan->batch = batch;
  plan->heads = heads;
  plan->max_seq_len = max_seq_len;
  plan->block_size = block_size;
  plan->dtype = dtype;
  plan->chunk_tiles = chunk_tiles;
  plan->work_groups = work_groups;
  plan->max_units = static_cast<int32_t>(shape.units);
  // The in-launch merge meets on counters the library holds for kAttnSyncSequences (head group,
  // sequence) pairs; beyond that the merge is a launch of its own.
  // (and a sequence's partials are counted in 16 bits)
  const bool fits = static_cast<int64_t>(batch) * head_groups <= mlakv::kAttnSyncSequences && shape.units < 65535;
  // Measured on MI355X: announcing and polling at agent scope costs about as much as the second
  // launch it replaces (a counter round trip is ~2 us, as is the partial read), so the second
  // launch, which needs no counters, is the default.
  plan->merge_mode = chosen.merge_mode == MLAKV_ATTN_MERGE_IN_LAUNCH && fits ? MLAKV_ATTN_MERGE_IN_LAUNCH : MLAKV_ATTN_MERGE_SECOND_LAUNCH;
  plan->merge_spin_us = chosen.merge_spin_us == 0 ? kDefaultMergeSpinUs : (chosen.merge_spin_us < 0 ? -1 : chosen.merge_spin_us);
  plan->reserved = sparse ? 1 : 0;
  // Whole-selection units of 16 heads where they apply, unless the caller asked for properties of
  // the split (a unit size, a workgroup count, a merge).
  const bool head_block_fits = sparse && max_seq_len <= MLAKV_ATTN_HEAD_BLOCK_TOKENS;
  const bool head_block_asked = chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK || chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES;
  if (sparse && head_block_asked && !head_block_fits) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: whole-selection units of 16 heads take up to %d selected tokens", who,
                MLAKV_ATTN_HEAD_BLOCK_TOKENS);
  }
  // Halved units leave two partials of 16 rows (and their LSEs, another half row) per (sequence,
  // 16 heads) in the workspace and meet on four of the library's counters each.
  const int64_t pairs = static_cast<int64_t>(batch) * (heads / 16);
  const bool halves_fit = head_block_fits && pairs * 4 <= 2 * mlakv::kAttnSyncSequences;
  if (sparse && chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES && !halves_fit) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: halved whole-selection units take up to %d (sequence, 16 heads) pairs", who,
                mlakv::kAttnSyncSequences / 2);
  }
  const bool split_asked = chosen.chunk_tiles != 0 || chosen.work_groups != 0 || chosen.merge_mode != 0;
  // Measured on MI355X (batch 4 .. 128, 64 and 128 heads): a whole-selection unit streams a tile per
  // 0.7 us after 5.5 us of set-up, so with one unit per CU it is ahead of the split up to 512
  // selected tokens (8.5 against 12 us at 64, 12 against 19 us at 256, level at 512), with two
  // units per CU up to 256, and behind beyond that. While two workgroups per unit still fit the CUs
  // once, halving the units pays from 257 selected tokens (the exchange costs what four tiles do:
  // 11.5 us either way at 256) to 768 (15.2 against 17.5 us at 512, 18.9 against 21.0 us for the
  // split at 768; the split is ahead again at 1024).
  const int64_t rounds = (static_cast<int64_t>(batch) * (heads / 16) + ComputeUnits() - 1) / ComputeUnits();
  // FP8 caches (same shapes): the split converts every K tile in four waves and is behind the whole
  // units at every measured size (batch 64, 512 selected tokens: 26.6 against 19.2 us; batch 128,
  // 1024: 63.8 against 63.1), the halved units ahead of both from 257 tokens on (batch 32, 512:
  // 19.7 / 17.3 / 15.2 us; 1024: 24.7 / 28.6 / 22.1).
  const bool fp8 = dtype == MLAKV_DTYPE_FP8_E4M3;
  const bool head_block_pays = fp8 ? (rounds <= 4 || max_seq_len <= 256)
                                   : ((rounds <= 1 && max_seq_len <= 512) || (rounds <= 2 && max_seq_len <= 256));
  const bool head_block = head_block_fits && (chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK ||
                                              (chosen.selection_units == MLAKV_ATTN_UNITS_AUTO && !split_asked && head_block_pays));
  const bool halves_pay = 2 * pairs <= ComputeUnits() && max_seq_len > 256 && (fp8 || max_seq_len <= 768);
  const bool halves = sparse && (chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES ||
                                 (chosen.selection_units == MLAKV_ATTN_UNITS_AUTO && !split_asked && halves_fit && halves_pay));
  if (sparse) {
    plan->selection_units = halves ? MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES : (head_block ? MLAKV_ATTN_UNITS_HEAD_BLOCK : MLAKV_ATTN_UNITS_SPLIT);
  } else {
    // A whole-context plan keeps what was asked for: AUTO lets every launch choose by the lengths it
    // can see (ShortContextUnits), SPLIT keeps the 64-head kernel, the other two need a context the
    // units can stage. Properties of the split pin the split.
    if ((chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK || chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES) &&
        (max_seq_len > MLAKV_ATTN_HEAD_BLOCK_TOKENS || (chosen.selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES && pairs * 4 > 2 * mlakv::kAttnSyncSequences))) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: whole-context units of 16 heads take contexts of up to %d tokens", who, MLAKV_ATTN_HEAD_BLOCK_TOKENS);
    }
    plan->selection_units = chosen.selection_units == MLAKV_ATTN_UNITS_AUTO && split_asked ? MLAKV_ATTN_UNITS_SPLIT : chosen.selection_units;
  }
  if (halves) shape = ShapeOf(batch, heads, max_seq_len, block_size, sparse, chunk_tiles, work_groups, true);
  plan->workspace_bytes = shape.workspace;
  return MLAKV_SUCCESS;
}

}  // namespace

extern "C" {

mlakvStatus mlakvAttnPlanInit(int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size, int32_t dtype,
                              mlakvAttnPlan* plan) {
  return AttnPlanImpl("mlakvAttnPlanInit", batch, heads, max_seq_len, block_size, dtype, false, nullptr, plan);
}

mlakvStatus mlakvAttnPlanInitEx(int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size, int32_t dtype,
                                const mlakvAttnPlanOptions* options, mlakvAttnPlan* plan) {
  const bool selection = options != nullptr && options->selection != 0;
  if (options != nullptr && (options->selection < 0 || options->selection > 1 || options->reserved[0] != 0 ||
                             options->reserved[1] != 0)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvAttnPlanInitEx: options outside their ranges");
  }
  if (selection && (max_seq_len <= 0 || max_seq_len > 2048)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvAttnPlanInitEx: sparse_count %d outside [1, 2048]", max_seq_len);
  }
  return AttnPlanImpl("mlakvAttnPlanInitEx", batch, heads, max_seq_len, block_size, dtype, selection, options, plan);
}

mlakvStatus mlakvAttnSparsePlanInit(int32_t batch, int32_t heads, int32_t sparse_count, int32_t block_size, int32_t dtype,
                                    mlakvAttnPlan* plan) {
  if (sparse_count <= 0 || sparse_count > 2048) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvAttnSparsePlanInit: sparse_count %d outside [1, 2048]", sparse_count);
  }
  return AttnPlanImpl("mlakvAttnSparsePlanInit", batch, heads, sparse_count, block_size, dtype, true, nullptr, plan);
}

}  // extern "C"

namespace {
mlakvStatus AttnDecodeImpl(const char* who, const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                           const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                           int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                           int32_t table_stride, const int32_t* seq_lens, double scale, void* out, int64_t out_seq_stride,
                           int64_t out_head_stride, const mlakvMxQuantOut* quant, const int32_t* sparse_indices,
                           int64_t sparse_indices_seq_stride, float* lse, void* workspace, uint64_t workspace_bytes,
                           void* stream, const int32_t* host_lens = nullptr, int32_t longest = -1) {
  if (plan == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: plan is null", who);
  if (host_lens != nullptr) {
    if (plan->batch > mlakv::kAttnInlineLens) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: host lengths ride in the argument block for up to %d sequences, the plan has %d", who,
                  mlakv::kAttnInlineLens, plan->batch);
    }
    seq_lens = host_lens;  // (only its being non-null matters below)
  }
  if (mlakvStatus s = CheckView(cache, who)) return s;
  if (mlakvStatus s = CheckLayers(cache, layer, 1, who)) return s;
  if (q_latent == nullptr || q_rope == nullptr || block_table == nullptr || seq_lens == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: query, block table and lengths are required", who);
  }
  if (out == nullptr && quant == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: an output is required", who);
  if (quant != nullptr) {
    if (quant->codes == nullptr || quant->scales == nullptr) {
      return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the quantised output needs codes and scales", who);
    }
    if (!Aligned16(quant->codes) || quant->codes_seq_stride % 16 != 0 || quant->codes_head_stride % 16 != 0 ||
        quant->codes_head_stride < mlakv::kLatentDim || !Aligned16(quant->scales) || quant->scales_seq_stride % 16 != 0 ||
        quant->scales_head_stride % 16 != 0 || quant->scales_head_stride < mlakv::kLatentDim / 32) {
      return Fail(MLAKV_ERR_PARAM_INVALID,
                  "%s: codes (512 per head) and scales (16 per head) must be 16-byte aligned with 16-byte-multiple strides", who);
    }
  }
  if (plan->dtype != cache->dtype || plan->block_size != cache->block_size) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the plan was made for dtype %d / block %d, the cache has %d / %d", who,
                plan->dtype, plan->block_size, cache->dtype, cache->block_size);
  }
  if (!(scale > 0.0) || !std::isfinite(scale)) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a positive softmax scale is required", who);
  // The kernels size their LDS staging, their grid and their partial slots from the plan: a plan
  // that was not made by the init functions (or was altered since) is refused here instead of
  // faulting there.
  {
    const bool fields = plan->batch > 0 && plan->batch <= 65535 && plan->heads > 0 && plan->heads % 16 == 0 && plan->heads <= 128 &&
                        plan->max_seq_len > 0 && plan->block_size > 0 && plan->chunk_tiles >= 0 && plan->work_groups >= 1 &&
                        plan->work_groups <= 65535 && (plan->reserved == 0 || plan->reserved == 1) &&
                        (plan->reserved == 0 ? (plan->selection_units == MLAKV_ATTN_UNITS_AUTO || plan->selection_units == MLAKV_ATTN_UNITS_SPLIT ||
                                                ((plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK ||
                                                  plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES) &&
                                                 plan->max_seq_len <= MLAKV_ATTN_HEAD_BLOCK_TOKENS))
                                             : (plan->selection_units == MLAKV_ATTN_UNITS_SPLIT ||
                                                ((plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK ||
                                                  plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES) &&
                                                 plan->max_seq_len <= MLAKV_ATTN_HEAD_BLOCK_TOKENS))) &&
                        (plan->reserved == 0 || plan->max_seq_len <= 2048) &&
                        (plan->merge_mode == MLAKV_ATTN_MERGE_IN_LAUNCH || plan->merge_mode == MLAKV_ATTN_MERGE_SECOND_LAUNCH) &&
                        (plan->merge_spin_us == -1 || (plan->merge_spin_us > 0 && plan->merge_spin_us <= 1000000));
    bool sane = fields;
    if (fields) {
      const PlanShape shape = ShapeOf(plan->batch, plan->heads, plan->max_seq_len, plan->block_size, plan->reserved == 1,
                                      plan->chunk_tiles, plan->work_groups,
                                      plan->reserved == 1 && plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES);
      sane = plan->chunk_tiles <= shape.cap && plan->max_units == shape.units && plan->workspace_bytes == shape.workspace &&
             (plan->merge_mode != MLAKV_ATTN_MERGE_IN_LAUNCH ||
              (static_cast<int64_t>(plan->batch) * shape.head_groups <= mlakv::kAttnSyncSequences && shape.units < 65535));
    }
    if (!sane) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the plan is not one made by mlakvAttnPlanInit / mlakvAttnSparsePlanInit", who);
    }
  }
  const bool sparse = sparse_indices != nullptr;
  if (sparse != (plan->reserved == 1)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the plan was made by %s", who,
                plan->reserved == 1 ? "mlakvAttnSparsePlanInit (selected-token attention)" : "mlakvAttnPlanInit (whole-context attention)");
  }
  if (sparse && (sparse_indices_seq_stride < plan->max_seq_len || reinterpret_cast<uintptr_t>(sparse_indices) % 4 != 0)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a row of the selection holds %d int32 entries", who, plan->max_seq_len);
  }
  if (sparse) {
    // The kernel stages a selected token as (block << ceil(log2(block_size))) | slot in 31 bits.
    int slot_bits = 0;
    while ((int64_t{1} << slot_bits) < cache->block_size) ++slot_bits;
    if ((static_cast<int64_t>(cache->num_blocks) << slot_bits) > (int64_t{1} << 31)) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: %d blocks of %d slots exceed the 2^31 pool slots selected-token attention addresses", who,
                  cache->num_blocks, cache->block_size);
    }
  }
  if (table_stride <= 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the block table needs at least one column", who);
  if (!sparse && static_cast<int64_t>(table_stride) * cache->block_size < plan->max_seq_len) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a table row of %d blocks cannot address %d tokens", who, table_stride,
                plan->max_seq_len);
  }
  if (!Aligned16(q_latent) || !Aligned16(q_rope) || q_latent_seq_stride % 16 != 0 || q_latent_head_stride % 16 != 0 ||
      q_rope_seq_stride % 16 != 0 || q_rope_head_stride % 16 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: query rows must be 16-byte aligned with 16-byte-multiple strides", who);
  }
  if (out != nullptr && (!Aligned16(out) || out_seq_stride % 16 != 0 || out_head_stride % 16 != 0)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: output rows must be 16-byte aligned with 16-byte-multiple strides", who);
  }
  if (workspace == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the plan needs %llu workspace bytes", who,
                                        static_cast<unsigned long long>(plan->workspace_bytes));
  if (workspace_bytes < plan->workspace_bytes || !Aligned16(workspace)) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: workspace of %llu bytes (16-byte aligned) needed, %llu given", who,
                static_cast<unsigned long long>(plan->workspace_bytes), static_cast<unsigned long long>(workspace_bytes));
  }
  mlakv::AttnArgs args{};
  FillPlanes(cache, layer, &args.latent, &args.rope, &args.scale);
  args.q_latent = static_cast<const char*>(q_latent);
  args.q_latent_seq_stride = q_latent_seq_stride;
  args.q_latent_head_stride = q_latent_head_stride;
  args.q_rope = static_cast<const char*>(q_rope);
  args.q_rope_seq_stride = q_rope_seq_stride;
  args.q_rope_head_stride = q_rope_head_stride;
  args.block_table = block_table;
  args.table_stride = table_stride;
  args.seq_lens = host_lens != nullptr ? nullptr : seq_lens;
  if (host_lens != nullptr) {
    args.inline_count = plan->batch;
    for (int32_t i = 0; i < plan->batch; ++i) args.inline_lens[i] = host_lens[i];
  }
  args.out = static_cast<char*>(out);
  args.out_seq_stride = out_seq_stride;
  args.out_head_stride = out_head_stride;
  args.lse = lse;
  args.sparse_indices = sparse_indices;
  args.sparse_seq_stride = sparse_indices_seq_stride;
  args.sparse_count = sparse ? plan->max_seq_len : 0;
  if (quant != nullptr) {
    args.out_codes = static_cast<char*>(quant->codes);
    args.out_codes_seq_stride = quant->codes_seq_stride;
    args.out_codes_head_stride = quant->codes_head_stride;
    args.out_scales = static_cast<char*>(quant->scales);
    args.out_scales_seq_stride = quant->scales_seq_stride;
    args.out_scales_head_stride = quant->scales_head_stride;
  }
  const uint64_t rows = static_cast<uint64_t>((plan->heads + 63) / 64) * (static_cast<uint64_t>(plan->max_units) + plan->batch) * 64;
  args.partial_out = static_cast<char*>(workspace);
  args.partial_lse = reinterpret_cast<float*>(static_cast<char*>(workspace) + rows * mlakv::kLatentDim * 2);
  args.scale_log2 = static_cast<float>(scale * 1.4426950408889634);
  args.batch = plan->batch;
  args.heads = plan->heads;
  args.num_blocks = cache->num_blocks;
  args.block_size = cache->block_size;
  {
    const int64_t addressable = static_cast<int64_t>(table_stride) * cache->block_size;
    args.max_tokens = sparse ? plan->max_seq_len : static_cast<int32_t>(addressable < plan->max_seq_len ? addressable : plan->max_seq_len);
  }
  args.work_groups = plan->work_groups;
  args.max_units = plan->max_units;
  args.forced_unit_tiles = plan->chunk_tiles;
  // Amortise the query load over at least 128 tokens; a selection is short and latency-bound, where
  // 64-token units measured faster.
  args.min_unit_tiles = sparse ? 2 : 4;
  args.cap_unit_tiles = static_cast<int32_t>(CapUnitTiles(plan->block_size, sparse));
  args.spin_ticks = plan->merge_spin_us < 0 ? 0 : plan->merge_spin_us * 100;
  args.merge_in_launch = plan->merge_mode == MLAKV_ATTN_MERGE_IN_LAUNCH;
  args.fp8 = cache->dtype == MLAKV_DTYPE_FP8_E4M3;
  args.head_block_units = plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK ? 1 : (plan->selection_units == MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES ? 2 : 0);
  if (!sparse) {
    // A whole context that is short: the units of the selected-token attention (one workgroup, or
    // two, per sequence and 16 heads; no selection, every position of the context) are ahead of the
    // 64-head kernel, whose work units are all fixed cost at that size. What the launch can see of
    // the lengths decides: the values themselves when they ride in the argument block, else the
    // plan's bound.
    int32_t bound = longest >= 0 ? std::min(longest, args.max_tokens) : args.max_tokens;  // (the caller's word for lengths in device memory)
    if (host_lens != nullptr) {
      bound = 0;
      for (int32_t i = 0; i < plan->batch; ++i) bound = std::max(bound, std::min(std::max(host_lens[i], 0), args.max_tokens));
    }
    args.head_block_units = ShortContextUnits(plan, bound);
    const uint64_t halved = static_cast<uint64_t>(plan->batch) * (plan->heads / 16) * (32 * mlakv::kLatentDim * 2 + 2 * 4 * 16 * sizeof(float));
    if (args.head_block_units == 2 && halved > plan->workspace_bytes) args.head_block_units = 1;  // (the halves' partials must fit what the plan sized for the split)
    if (quant != nullptr && args.head_block_units != 0) {
      // The units have no quantising epilogue: they write bf16 rows (the caller's, or rows of the
      // workspace behind the halves' partials) and the standalone quantiser follows in the same
      // stream; its codes are those of the fused epilogue, by construction of both from the bf16 rows.
      const uint64_t rows_offset = args.head_block_units == 2 ? ((halved + 255) & ~255ull) : 0;
      const uint64_t rows_bytes = static_cast<uint64_t>(plan->batch) * plan->heads * mlakv::kLatentDim * 2;
      const bool own_rows = out == nullptr;
      const bool uniform = (own_rows || out_seq_stride == plan->heads * out_head_stride) &&
                           quant->codes_seq_stride == plan->heads * quant->codes_head_stride &&
                           quant->scales_seq_stride == plan->heads * quant->scales_head_stride;
      if (!uniform || (own_rows && rows_offset + rows_bytes > plan->workspace_bytes)) {
        args.head_block_units = 0;
      } else {
        if (own_rows) {
          args.out = static_cast<char*>(workspace) + rows_offset;
          args.out_seq_stride = static_cast<int64_t>(plan->heads) * mlakv::kLatentDim * 2;
          args.out_head_stride = mlakv::kLatentDim * 2;
        }
        args.out_codes = nullptr;
        args.out_scales = nullptr;
        args.sparse_count = std::max(bound, 1);
        hipError_t status = mlakv::LaunchAttnDecode(args, static_cast<hipStream_t>(stream));
        if (status != hipSuccess) return HipFail(status, who);
        mlakv::MxQuantArgs quantise{};
        quantise.x = args.out;
        quantise.x_row_stride = args.out_head_stride;
        quantise.codes = static_cast<char*>(quant->codes);
        quantise.codes_row_stride = quant->codes_head_stride;
        quantise.scales = static_cast<char*>(quant->scales);
        quantise.scales_row_stride = quant->scales_head_stride;
        quantise.rows = static_cast<int64_t>(plan->batch) * plan->heads;
        quantise.cols = mlakv::kLatentDim;
        status = mlakv::LaunchMxQuant(quantise, static_cast<hipStream_t>(stream));
        return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
      }
    }
    args.sparse_count = args.head_block_units != 0 ? std::max(bound, 1) : 0;
  }
  const hipError_t status = mlakv::LaunchAttnDecode(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
}

}  // namespace

extern "C" {

mlakvStatus mlakvAttnDecode(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                            int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                            int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                            int32_t table_stride, const int32_t* seq_lens, double scale, void* out, int64_t out_seq_stride,
                            int64_t out_head_stride, float* lse, void* workspace, uint64_t workspace_bytes, void* stream) {
  if (out == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvAttnDecode: the output is required");
  return AttnDecodeImpl("mlakvAttnDecode", plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope,
                        q_rope_seq_stride, q_rope_head_stride, block_table, table_stride, seq_lens, scale, out, out_seq_stride,
                        out_head_stride, nullptr, nullptr, 0, lse, workspace, workspace_bytes, stream);
}

mlakvStatus mlakvAttnDecodeBounded(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                                   int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                                   int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                                   int32_t table_stride, const int32_t* seq_lens, int32_t longest, double scale, void* out,
                                   int64_t out_seq_stride, int64_t out_head_stride, float* lse, void* workspace,
                                   uint64_t workspace_bytes, void* stream) {
  const char* who = "mlakvAttnDecodeBounded";
  if (out == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the output is required", who);
  if (longest < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the bound of the lengths must not be negative", who);
  return AttnDecodeImpl(who, plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope, q_rope_seq_stride,
                        q_rope_head_stride, block_table, table_stride, seq_lens, scale, out, out_seq_stride, out_head_stride, nullptr,
                        nullptr, 0, lse, workspace, workspace_bytes, stream, nullptr, longest);
}

mlakvStatus mlakvAttnDecodeHostLens(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                                    int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                                    int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                                    int32_t table_stride, const int32_t* host_seq_lens, double scale, void* out,
                                    int64_t out_seq_stride, int64_t out_head_stride, float* lse, void* workspace,
                                    uint64_t workspace_bytes, void* stream) {
  const char* who = "mlakvAttnDecodeHostLens";
  if (out == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the output is required", who);
  if (host_seq_lens == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the lengths are required", who);
  return AttnDecodeImpl(who, plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope, q_rope_seq_stride,
                        q_rope_head_stride, block_table, table_stride, nullptr, scale, out, out_seq_stride, out_head_stride, nullptr,
                        nullptr, 0, lse, workspace, workspace_bytes, stream, host_seq_lens);
}

mlakvStatus mlakvAttnDecodeNoAlloc(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                                   int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                                   int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                                   int32_t table_stride, const int32_t* seq_lens, double scale, void* out, int64_t out_seq_stride,
                                   int64_t out_head_stride, float* lse, void* stream) {
  const char* who = "mlakvAttnDecodeNoAlloc";
  if (plan == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: plan is null", who);
  if (out == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the output is required", who);
  if (plan->workspace_bytes > MLAKV_NOALLOC_SCRATCH_BYTES) {
    return Fail(MLAKV_ERR_PARAM_INVALID,
                "%s: the plan needs %llu bytes of split-KV partials, the library's static scratch holds %llu; use "
                "mlakvAttnDecode with a workspace of the caller's",
                who, static_cast<unsigned long long>(plan->workspace_bytes),
                static_cast<unsigned long long>(MLAKV_NOALLOC_SCRATCH_BYTES));
  }
  char* scratch = nullptr;
  const hipError_t resolved = mlakv::AttnStaticScratch(&scratch);
  if (resolved != hipSuccess) return HipFail(resolved, who);
  return AttnDecodeImpl(who, plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope, q_rope_seq_stride,
                        q_rope_head_stride, block_table, table_stride, seq_lens, scale, out, out_seq_stride, out_head_stride,
                        nullptr, nullptr, 0, lse, scratch, mlakv::kAttnStaticScratchBytes, stream);
}

mlakvStatus mlakvAttnDecodeSparse(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                                  int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                                  int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                                  int32_t table_stride, const int32_t* seq_lens, const int32_t* sparse_indices,
                                  int64_t sparse_indices_seq_stride, double scale, void* out, int64_t out_seq_stride,
                                  int64_t out_head_stride, float* lse, void* workspace, uint64_t workspace_bytes,
                                  void* stream) {
  if (out == nullptr || sparse_indices == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvAttnDecodeSparse: the output and the selection are required");
  }
  return AttnDecodeImpl("mlakvAttnDecodeSparse", plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope,
                        q_rope_seq_stride, q_rope_head_stride, block_table, table_stride, seq_lens, scale, out, out_seq_stride,
                        out_head_stride, nullptr, sparse_indices, sparse_indices_seq_stride, lse, workspace, workspace_bytes,
                        stream);
}

mlakvStatus mlakvAttnDecodeMxQuant(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer, const void* q_latent,
                                   int64_t q_latent_seq_stride, int64_t q_latent_head_stride, const void* q_rope,
                                   int64_t q_rope_seq_stride, int64_t q_rope_head_stride, const int32_t* block_table,
                                   int32_t table_stride, const int32_t* seq_lens, double scale, void* out, int64_t out_seq_stride,
                                   int64_t out_head_stride, const mlakvMxQuantOut* quant, float* lse, void* workspace,
                                   uint64_t workspace_bytes, void* stream) {
  if (quant == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvAttnDecodeMxQuant: the quantised output is required");
  return AttnDecodeImpl("mlakvAttnDecodeMxQuant", plan, cache, layer, q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope,
                        q_rope_seq_stride, q_rope_head_stride, block_table, table_stride, seq_lens, scale, out, out_seq_stride,
                        out_head_stride, quant, nullptr, 0, lse, workspace, workspace_bytes, stream);
}

uint64_t mlakvIndexerWorkspaceBytes(int32_t batch, int32_t max_seq_len) {
  if (batch <= 0 || max_seq_len <= 0) return 0;
  const uint64_t row = (static_cast<uint64_t>(max_seq_len) + 127) & ~127ull;  // 16-bit keys, rows 256-byte aligned
  return static_cast<uint64_t>(batch) * row * 2;
}

mlakvStatus mlakvLightningIndexer(const mlakvIndexKeyView* keys, const void* query, int64_t query_seq_stride,
                                  int64_t query_head_stride, const void* weights, int64_t weights_seq_stride,
                                  const float* query_dequant_scale, int64_t query_scale_seq_stride, int32_t heads,
                                  const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, int32_t batch,
                                  int32_t max_seq_len, int32_t sparse_count, int32_t* sparse_indices,
                                  int64_t sparse_indices_seq_stride, void* workspace, uint64_t workspace_bytes, void* stream) {
  const char* who = "mlakvLightningIndexer";
  if (keys == nullptr || keys->keys == nullptr || keys->scales == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the index key pool is required", who);
  if (batch < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: negative batch", who);
  if (batch == 0) return MLAKV_SUCCESS;
  if (query == nullptr || weights == nullptr || query_dequant_scale == nullptr || block_table == nullptr || seq_lens == nullptr ||
      sparse_indices == nullptr) {
    return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: query, weights, scales, block table, lengths and output are required", who);
  }
  if (keys->dim != 128) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: index keys have 128 elements, not %d", who, keys->dim);
  if (heads <= 0 || heads % 16 != 0 || heads > 64) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: heads %d must be 16, 32, 48 or 64", who, heads);
  }
  if (sparse_count <= 0 || sparse_count > 2048) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: sparse_count %d outside [1, 2048]", who, sparse_count);
  if (keys->num_blocks <= 0 || keys->block_size <= 0 || max_seq_len <= 0 || batch > 65535) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: sizes must be positive (batch at most 65535)", who);
  }
  if (static_cast<int64_t>(table_stride) * keys->block_size < max_seq_len) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: a table row of %d blocks cannot address %d tokens", who, table_stride, max_seq_len);
  }
  if (!Aligned16(keys->keys) || keys->row_stride % 16 != 0 || keys->block_stride % 16 != 0 || keys->row_stride < 128 ||
      reinterpret_cast<uintptr_t>(keys->scales) % 4 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: key rows must be 16-byte aligned and hold 128 bytes", who);
  }
  if (!Aligned16(query) || query_seq_stride % 16 != 0 || query_head_stride % 16 != 0 || query_head_stride < 128 ||
      reinterpret_cast<uintptr_t>(weights) % 2 != 0 || weights_seq_stride % 2 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: query rows must be 16-byte aligned and hold 128 bytes; weights are bf16", who);
  }
  if (sparse_indices_seq_stride < sparse_count) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: an output row holds %d entries", who, sparse_count);
  const uint64_t needed = max_seq_len > sparse_count ? mlakvIndexerWorkspaceBytes(batch, max_seq_len) : 0;
  if (needed > 0) {
    if (workspace == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: %llu workspace bytes are needed", who, static_cast<unsigned long long>(needed));
    if (workspace_bytes < needed || !Aligned16(workspace)) {
      return Fail(MLAKV_ERR_PARAM_INVALID, "%s: workspace of %llu bytes (16-byte aligned) needed, %llu given", who,
                  static_cast<unsigned long long>(needed), static_cast<unsigned long long>(workspace_bytes));
    }
  }
  mlakv::IndexerArgs args{};
  args.query = static_cast<const char*>(query);
  args.query_seq_stride = query_seq_stride;
  args.query_head_stride = query_head_stride;
  args.weights = static_cast<const char*>(weights);
  args.weights_seq_stride = weights_seq_stride;
  args.query_scale = query_dequant_scale;
  args.query_scale_seq_stride = query_scale_seq_stride;
  args.key_base = static_cast<const char*>(keys->keys);
  args.key_block_stride = keys->block_stride;
  args.key_row_stride = keys->row_stride;
  args.key_scale_base = keys->scales;
  args.key_scale_block_stride = keys->scale_block_stride;
  args.block_table = block_table;
  args.table_stride = table_stride;
  args.seq_lens = seq_lens;
  args.keys = static_cast<unsigned short*>(workspace);
  args.keys_stride = static_cast<int64_t>((static_cast<uint64_t>(max_seq_len) + 127) & ~127ull);
  args.indices_out = sparse_indices;
  args.indices_seq_stride = sparse_indices_seq_stride;
  args.batch = batch;
  args.heads = heads;
  args.num_blocks = keys->num_blocks;
  args.block_size = keys->block_size;
  args.max_seq_len = max_seq_len;
  args.sparse_count = sparse_count;
  const hipError_t status = mlakv::LaunchIndexer(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
}

mlakvStatus mlakvIndexKeyAppend(const mlakvIndexKeyView* keys, const void* k, int64_t k_row_stride,
                                const int32_t* slot_mapping, int32_t num_tokens, void* stream) {
  const char* who = "mlakvIndexKeyAppend";
  if (keys == nullptr || keys->keys == nullptr || keys->scales == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: the index key pool is required", who);
  if (num_tokens < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: negative num_tokens", who);
  if (num_tokens == 0) return MLAKV_SUCCESS;
  if (k == nullptr || slot_mapping == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: rows and slot mapping are required", who);
  if (keys->dim != 128) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: index keys have 128 elements, not %d", who, keys->dim);
  if (keys->num_blocks <= 0 || keys->block_size <= 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: the pool needs blocks of a positive size", who);
  if (!Aligned16(keys->keys) || keys->row_stride % 16 != 0 || keys->block_stride % 16 != 0 || keys->row_stride < 128 ||
      reinterpret_cast<uintptr_t>(keys->scales) % 4 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: key rows must be 16-byte aligned and hold 128 bytes", who);
  }
  if (!Aligned16(k) || k_row_stride % 16 != 0 || k_row_stride < 256) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: source rows must be 16-byte aligned and hold 128 bf16 values", who);
  }
  mlakv::IndexKeyAppendArgs args{};
  args.key_base = static_cast<char*>(const_cast<void*>(keys->keys));
  args.key_block_stride = keys->block_stride;
  args.key_row_stride = keys->row_stride;
  args.key_scale_base = const_cast<float*>(keys->scales);
  args.key_scale_block_stride = keys->scale_block_stride;
  args.num_blocks = keys->num_blocks;
  args.block_size = keys->block_size;
  args.src = static_cast<const char*>(k);
  args.src_row_stride = k_row_stride;
  args.slots = slot_mapping;
  args.num_tokens = num_tokens;
  const hipError_t status = mlakv::LaunchIndexKeyAppend(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
}

mlakvStatus mlakvDynamicMxQuant(const void* x, int64_t x_row_stride, int64_t rows, int32_t cols, void* codes,
                                int64_t codes_row_stride, void* scales, int64_t scales_row_stride, void* stream) {
  const char* who = "mlakvDynamicMxQuant";
  if (rows < 0 || cols < 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: negative shape", who);
  if (rows == 0 || cols == 0) return MLAKV_SUCCESS;
  if (x == nullptr || codes == nullptr || scales == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: input, codes and scales are required", who);
  if (cols % 32 != 0) return Fail(MLAKV_ERR_PARAM_INVALID, "%s: %d columns are not a whole number of blocks of 32", who, cols);
  if (!Aligned16(x) || x_row_stride % 16 != 0 || x_row_stride < static_cast<int64_t>(cols) * 2) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: input rows must be 16-byte aligned and hold %d bf16 values", who, cols);
  }
  if (reinterpret_cast<uintptr_t>(codes) % 8 != 0 || codes_row_stride % 8 != 0 || codes_row_stride < cols ||
      scales_row_stride < cols / 32) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: code rows must be 8-byte aligned and hold %d bytes, scale rows %d", who, cols, cols / 32);
  }
  mlakv::MxQuantArgs args{};
  args.x = static_cast<const char*>(x);
  args.x_row_stride = x_row_stride;
  args.codes = static_cast<char*>(codes);
  args.codes_row_stride = codes_row_stride;
  args.scales = static_cast<char*>(scales);
  args.scales_row_stride = scales_row_stride;
  args.rows = rows;
  args.cols = cols;
  const hipError_t status = mlakv::LaunchMxQuant(args, static_cast<hipStream_t>(stream));
  return status == hipSuccess ? MLAKV_SUCCESS : HipFail(status, who);
}

}  // extern "C"

// ---- arena and KV cache handles -------------------------------------------------------

struct mlakvArena {
  std::unique_ptr<moe_hip::IDeviceBackend> backend;
  std::unique_ptr<moe_hip::StaticMemoryArena> arena;
  // Caches hold a reference to the arena: destroying the arena while some are alive only marks
  // it, and the last cache to go takes the arena with it.
  int live_caches = 0;
  bool destroy_requested = false;
};

struct mlakvKvCache {
  mlakvArena* owner = nullptr;
  std::unique_ptr<moe_hip::KvCacheManager> manager;
};

namespace {
// Runs `body`, mapping a contract refusal (KvError) to MLAKV_ERR_CONTRACT.
template <typename Body>
mlakvStatus Guard(const char* who, Body body) {
  try {
    body();
    return MLAKV_SUCCESS;
  } catch (const moe_hip::KvError& error) {
    return FailText(MLAKV_ERR_CONTRACT, std::string(who) + ": " + error.what());
  } catch (const std::exception& error) {
    return FailText(MLAKV_ERR_RUNTIME, std::string(who) + ": " + error.what());
  }
}
}  // namespace

extern "C" {

mlakvStatus mlakvArenaCreate(int32_t backend, mlakvArena** arena) {
  if (arena == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "mlakvArenaCreate: output is null");
  *arena = nullptr;
  if (backend != MLAKV_BACKEND_HIP && backend != MLAKV_BACKEND_HOST) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvArenaCreate: unknown backend %d", backend);
  }
  auto handle = std::make_unique<mlakvArena>();
  const mlakvStatus status = Guard("mlakvArenaCreate", [&] {
    if (backend == MLAKV_BACKEND_HIP) handle->backend = std::make_unique<moe_hip::HipDeviceBackend>();
    else handle->backend = std::make_unique<moe_hip::HostDeviceBackend>();
    handle->arena = std::make_unique<moe_hip::StaticMemoryArena>(*handle->backend);
  });
  if (status != MLAKV_SUCCESS) return status == MLAKV_ERR_CONTRACT ? MLAKV_ERR_RUNTIME : status;
  *arena = handle.release();
  return MLAKV_SUCCESS;
}

void mlakvArenaDestroy(mlakvArena* arena) {
  if (arena == nullptr) return;
  if (arena->live_caches > 0) {
    arena->destroy_requested = true;
    return;
  }
  arena->arena.reset();
  arena->backend.reset();
  delete arena;
}

#define MLAKV_NEED(pointer, who) \
  if ((pointer) == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, who ": null argument")

mlakvStatus mlakvArenaReserve(mlakvArena* arena, const char* name, size_t bytes, size_t align, size_t* handle) {
  MLAKV_NEED(arena, "mlakvArenaReserve");
  MLAKV_NEED(name, "mlakvArenaReserve");
  return Guard("mlakvArenaReserve", [&] {
    const size_t h = arena->arena->Reserve(name, bytes, align);
    if (handle != nullptr) *handle = h;
  });
}

mlakvStatus mlakvArenaCommit(mlakvArena* arena) {
  MLAKV_NEED(arena, "mlakvArenaCommit");
  return Guard("mlakvArenaCommit", [&] { arena->arena->Commit(); });
}

mlakvStatus mlakvArenaAddress(const mlakvArena* arena, size_t handle, void** address) {
  MLAKV_NEED(arena, "mlakvArenaAddress");
  MLAKV_NEED(address, "mlakvArenaAddress");
  return Guard("mlakvArenaAddress", [&] { *address = arena->arena->Address(handle); });
}

mlakvStatus mlakvArenaBytes(const mlakvArena* arena, size_t handle, size_t* bytes) {
  MLAKV_NEED(arena, "mlakvArenaBytes");
  MLAKV_NEED(bytes, "mlakvArenaBytes");
  return Guard("mlakvArenaBytes", [&] { *bytes = arena->arena->Bytes(handle); });
}

mlakvStatus mlakvArenaOffset(const mlakvArena* arena, size_t handle, size_t* offset) {
  MLAKV_NEED(arena, "mlakvArenaOffset");
  MLAKV_NEED(offset, "mlakvArenaOffset");
  return Guard("mlakvArenaOffset", [&] { *offset = arena->arena->Offset(handle); });
}

mlakvStatus mlakvArenaNoteWorkspace(mlakvArena* arena, uint64_t bytes) {
  MLAKV_NEED(arena, "mlakvArenaNoteWorkspace");
  return Guard("mlakvArenaNoteWorkspace", [&] { arena->arena->NoteWorkspace(bytes); });
}

mlakvStatus mlakvArenaCommitWorkspace(mlakvArena* arena) {
  MLAKV_NEED(arena, "mlakvArenaCommitWorkspace");
  return Guard("mlakvArenaCommitWorkspace", [&] { arena->arena->CommitWorkspace(); });
}

mlakvStatus mlakvArenaAssertWorkspaceFits(const mlakvArena* arena, uint64_t bytes, const char* what) {
  MLAKV_NEED(arena, "mlakvArenaAssertWorkspaceFits");
  return Guard("mlakvArenaAssertWorkspaceFits", [&] { arena->arena->AssertWorkspaceFits(bytes, what ? what : "plan"); });
}

mlakvStatus mlakvArenaSeal(mlakvArena* arena) {
  MLAKV_NEED(arena, "mlakvArenaSeal");
  return Guard("mlakvArenaSeal", [&] { arena->arena->Seal(); });
}

mlakvStatus mlakvArenaValidateAlignment(const mlakvArena* arena) {
  MLAKV_NEED(arena, "mlakvArenaValidateAlignment");
  return Guard("mlakvArenaValidateAlignment", [&] {
    MOE_HIP_REQUIRE(arena->arena->committed(), "ValidateAlignment needs the arena to be committed first");
    arena->arena->ValidateAlignment();
  });
}

void* mlakvArenaWorkspace(const mlakvArena* arena) { return arena ? arena->arena->workspace() : nullptr; }
uint64_t mlakvArenaWorkspaceBytes(const mlakvArena* arena) { return arena ? arena->arena->workspace_bytes() : 0; }
size_t mlakvArenaTotalBytes(const mlakvArena* arena) { return arena ? arena->arena->arena_bytes() : 0; }
size_t mlakvArenaReservedBytes(const mlakvArena* arena) { return arena ? arena->arena->reserved_bytes() : 0; }
size_t mlakvArenaReservationCount(const mlakvArena* arena) { return arena ? arena->arena->reservations().size() : 0; }
int32_t mlakvArenaSealed(const mlakvArena* arena) { return arena && arena->arena->sealed() ? 1 : 0; }
uint64_t mlakvArenaDeviceAllocationCount(const mlakvArena* arena) { return arena ? arena->backend->DeviceAllocationCount() : 0; }

size_t mlakvArenaDescribeLedger(const mlakvArena* arena, char* buffer, size_t capacity) {
  if (arena == nullptr) return 0;
  const std::string text = arena->arena->DescribeLedger();
  if (buffer != nullptr && capacity > 0) {
    const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
    std::memcpy(buffer, text.data(), n);
    buffer[n] = '\0';
  }
  return text.size();
}

// ---- KV cache manager ---------------------------------------------------------------

mlakvStatus mlakvKvCacheCreate(mlakvArena* arena, const mlakvKvConfig* config, mlakvKvCache** cache) {
  MLAKV_NEED(arena, "mlakvKvCacheCreate");
  MLAKV_NEED(config, "mlakvKvCacheCreate");
  MLAKV_NEED(cache, "mlakvKvCacheCreate");
  *cache = nullptr;
  if (config->dtype != MLAKV_DTYPE_BF16 && config->dtype != MLAKV_DTYPE_FP8_E4M3) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "mlakvKvCacheCreate: unknown cache dtype %d", config->dtype);
  }
  auto handle = std::make_unique<mlakvKvCache>();
  handle->owner = arena;
  const mlakvStatus status = Guard("mlakvKvCacheCreate", [&] {
    moe_hip::KvCacheConfig c;
    c.num_layers = config->num_layers;
    c.block_size = config->block_size;
    c.max_context_len = config->max_context_len;
    c.max_batch = config->max_batch;
    c.pool_blocks = config->pool_blocks;
    c.mla.kv_lora_rank = config->kv_lora_rank;
    c.mla.qk_rope_head_dim = config->qk_rope_head_dim;
    c.dtype = static_cast<moe_hip::KvDtype>(config->dtype);
    c.fused_rows = config->fused_rows != 0;
    c.seed = config->seed;
    c.shuffle = config->shuffle != 0;
    handle->manager = std::make_unique<moe_hip::KvCacheManager>(*arena->arena, c);
  });
  if (status != MLAKV_SUCCESS) return status;
  ++arena->live_caches;
  *cache = handle.release();
  return MLAKV_SUCCESS;
}

void mlakvKvCacheDestroy(mlakvKvCache* cache) {
  if (cache == nullptr) return;
  mlakvArena* owner = cache->owner;
  delete cache;
  if (owner != nullptr && --owner->live_caches == 0 && owner->destroy_requested) mlakvArenaDestroy(owner);
}

mlakvStatus mlakvKvCacheBind(mlakvKvCache* cache) {
  MLAKV_NEED(cache, "mlakvKvCacheBind");
  return Guard("mlakvKvCacheBind", [&] { cache->manager->Bind(); });
}

mlakvStatus mlakvKvCacheGetView(const mlakvKvCache* cache, mlakvCacheView* view) {
  MLAKV_NEED(cache, "mlakvKvCacheGetView");
  MLAKV_NEED(view, "mlakvKvCacheGetView");
  if (!cache->manager->bound()) return Fail(MLAKV_ERR_CONTRACT, "mlakvKvCacheGetView: the cache is not bound yet");
  const moe_hip::KvCacheView& v = cache->manager->view();
  view->latent = v.latent.base;
  view->latent_layer_stride = v.latent.layer_stride;
  view->latent_block_stride = v.latent.block_stride;
  view->latent_row_stride = v.latent.row_stride;
  view->rope = v.rope.base;
  view->rope_layer_stride = v.rope.layer_stride;
  view->rope_block_stride = v.rope.block_stride;
  view->rope_row_stride = v.rope.row_stride;
  view->scale = v.scale.base;
  view->scale_layer_stride = v.scale.layer_stride;
  view->scale_block_stride = v.scale.block_stride;
  view->num_layers = v.num_layers;
  view->num_blocks = v.num_blocks;
  view->block_size = v.block_size;
  view->latent_dim = v.latent_dim;
  view->rope_dim = v.rope_dim;
  view->dtype = static_cast<int32_t>(v.dtype);
  return MLAKV_SUCCESS;
}

int64_t mlakvKvCacheNumBlocks(const mlakvKvCache* cache) { return cache ? cache->manager->num_blocks() : 0; }
int64_t mlakvKvCachePoolBlocks(const mlakvKvCache* cache) { return cache ? cache->manager->pool_blocks() : 0; }

mlakvStatus mlakvKvCacheAddSequence(mlakvKvCache* cache, int64_t seq, int64_t context_len) {
  MLAKV_NEED(cache, "mlakvKvCacheAddSequence");
  return Guard("mlakvKvCacheAddSequence", [&] { cache->manager->AddSequence(seq, context_len); });
}

mlakvStatus mlakvKvCacheAppendToken(mlakvKvCache* cache, int64_t seq, int32_t* slot) {
  MLAKV_NEED(cache, "mlakvKvCacheAppendToken");
  return Guard("mlakvKvCacheAppendToken", [&] {
    const int32_t s = cache->manager->AppendToken(seq);
    if (slot != nullptr) *slot = s;
  });
}

mlakvStatus mlakvKvCacheAppendTokenAll(mlakvKvCache* cache, int32_t* slots, int64_t* appended) {
  MLAKV_NEED(cache, "mlakvKvCacheAppendTokenAll");
  return Guard("mlakvKvCacheAppendTokenAll", [&] {
    const int64_t n = cache->manager->AppendTokenAll(slots);
    if (appended != nullptr) *appended = n;
  });
}

mlakvStatus mlakvKvCacheFreeSequence(mlakvKvCache* cache, int64_t seq) {
  MLAKV_NEED(cache, "mlakvKvCacheFreeSequence");
  return Guard("mlakvKvCacheFreeSequence", [&] { cache->manager->FreeSequence(seq); });
}

mlakvStatus mlakvKvCacheCompact(mlakvKvCache* cache, int32_t* moves, int64_t* num_moves, void* stream) {
  MLAKV_NEED(cache, "mlakvKvCacheCompact");
  return Guard("mlakvKvCacheCompact", [&] {
    const auto planned = cache->manager->Compact(stream);
    if (moves != nullptr) {
      for (size_t i = 0; i < planned.size(); ++i) {
        moves[2 * i] = planned[i].first;
        moves[2 * i + 1] = planned[i].second;
      }
    }
    if (num_moves != nullptr) *num_moves = static_cast<int64_t>(planned.size());
  });
}

mlakvStatus mlakvKvCacheUploadStep(mlakvKvCache* cache, void* stream) {
  MLAKV_NEED(cache, "mlakvKvCacheUploadStep");
  return Guard("mlakvKvCacheUploadStep", [&] { cache->manager->UploadStep(stream); });
}

mlakvStatus mlakvKvCacheUploadStepAndAppend(mlakvKvCache* cache, int32_t layer_begin, int32_t layer_count, const void* latent_src,
                                            int64_t latent_src_layer_stride, int64_t latent_src_row_stride, const void* rope_src,
                                            int64_t rope_src_layer_stride, int64_t rope_src_row_stride, void* stream) {
  MLAKV_NEED(cache, "mlakvKvCacheUploadStepAndAppend");
  const char* who = "mlakvKvCacheUploadStepAndAppend";
  if (latent_src == nullptr || rope_src == nullptr) return Fail(MLAKV_ERR_PARAM_NULLPTR, "%s: source rows are required", who);
  if (!Aligned16(latent_src) || !Aligned16(rope_src) || latent_src_row_stride % 16 != 0 || rope_src_row_stride % 16 != 0 ||
      latent_src_layer_stride % 16 != 0 || rope_src_layer_stride % 16 != 0) {
    return Fail(MLAKV_ERR_PARAM_INVALID, "%s: source rows must be 16-byte aligned with 16-byte-multiple strides", who);
  }
  return Guard(who, [&] {
    cache->manager->UploadStepAndAppend(latent_src, latent_src_layer_stride, latent_src_row_stride, rope_src, rope_src_layer_stride,
                                        rope_src_row_stride, layer_begin, layer_count, stream);
  });
}

mlakvStatus mlakvKvCacheGetStats(const mlakvKvCache* cache, mlakvKvStats* stats) {
  MLAKV_NEED(cache, "mlakvKvCacheGetStats");
  MLAKV_NEED(stats, "mlakvKvCacheGetStats");
  const moe_hip::PagedAttentionStats s = cache->manager->stats();
  stats->total_blocks_allocated = s.total_blocks_allocated;
  stats->active_context_tokens = s.active_context_tokens;
  stats->block_size = s.block_size;
  stats->kv_cache_utilization = s.kv_cache_utilization;
  return MLAKV_SUCCESS;
}

int64_t mlakvKvStatsFormatJson(const mlakvKvStats* stats, char* buffer, size_t capacity) {
  if (stats == nullptr) return -1;
  // %.12g is what an ostream at precision 12 in the classic locale prints for a double; a
  // non-finite utilisation is written as null.
  char utilization[40];
  if (std::isfinite(stats->kv_cache_utilization)) {
    std::snprintf(utilization, sizeof utilization, "%.12g", stats->kv_cache_utilization);
    for (char* c = utilization; *c != 0; ++c) {
      if (*c == ',') *c = '.';  // a process-wide locale with a decimal comma must not leak into JSON
    }
  } else {
    std::snprintf(utilization, sizeof utilization, "null");
  }
  const int needed = std::snprintf(buffer, buffer == nullptr ? 0 : capacity,
                                   "  \"paged_attention\": {\n"
                                   "    \"total_blocks_allocated\": %llu,\n"
                                   "    \"active_context_tokens\": %llu,\n"
                                   "    \"block_size\": %llu,\n"
                                   "    \"kv_cache_utilization\": %s\n"
                                   "  }",
                                   static_cast<unsigned long long>(stats->total_blocks_allocated),
                                   static_cast<unsigned long long>(stats->active_context_tokens),
                                   static_cast<unsigned long long>(stats->block_size), utilization);
  return needed;
}

const int32_t* mlakvKvCacheHostBlockTable(const mlakvKvCache* cache) { return cache ? cache->manager->host_block_table() : nullptr; }
const int32_t* mlakvKvCacheHostSlotMapping(const mlakvKvCache* cache) { return cache ? cache->manager->host_slot_mapping() : nullptr; }
const int32_t* mlakvKvCacheHostSeqLens(const mlakvKvCache* cache) { return cache ? cache->manager->host_seq_lens() : nullptr; }
int64_t mlakvKvCacheFreeBlocks(const mlakvKvCache* cache) { return cache ? cache->manager->pool().free_blocks() : 0; }

int64_t mlakvKvCacheFreeList(const mlakvKvCache* cache, int32_t* out) {
  if (cache == nullptr) return 0;
  const std::vector<int32_t> list = cache->manager->pool().FreeList();
  if (out != nullptr && !list.empty()) std::memcpy(out, list.data(), list.size() * sizeof(int32_t));
  return static_cast<int64_t>(list.size());
}

int32_t* mlakvKvCacheDeviceBlockTable(const mlakvKvCache* cache) { return cache ? cache->manager->device_block_table() : nullptr; }
int32_t* mlakvKvCacheDeviceSlotMapping(const mlakvKvCache* cache) { return cache ? cache->manager->device_slot_mapping() : nullptr; }
int32_t* mlakvKvCacheDeviceSeqLens(const mlakvKvCache* cache) { return cache ? cache->manager->device_seq_lens() : nullptr; }
int32_t* mlakvKvCacheDeviceCuSeqLens(const mlakvKvCache* cache) { return cache ? cache->manager->device_cu_seq_lens() : nullptr; }

int64_t mlakvNumBlocks(int64_t max_context_len, int64_t block_size) {
  if (block_size <= 0 || max_context_len < block_size) return -1;
  return moe_hip::DivideUp(max_context_len, block_size);
}

uint64_t mlakvBackboneDeviceBytes(int64_t kv_lora_rank, int64_t qk_rope_head_dim, int64_t block_size, int64_t max_context_len) {
  moe_hip::MlaGeometry mla;
  mla.kv_lora_rank = kv_lora_rank;
  mla.qk_rope_head_dim = qk_rope_head_dim;
  return moe_hip::BackboneDeviceBytes(mla, block_size, max_context_len);
}

}  // extern "C"
