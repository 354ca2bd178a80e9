/*
 * mlakv.h -- thin C ABI over the gfx950 HIP kernels of the paged MLA KV-cache path:
 * static-arena block reservation, per-layer latent KV append, block-table gather,
 * compaction copy and absorbed-MLA decode attention.
 *
 * Plain pointers and sizes only. Every device pointer is an address the caller owns
 * (the arena below hands them out); `stream` is a hipStream_t passed as void*.
 * All strides are in BYTES unless a parameter says otherwise. Every function returns
 * a status and never throws; mlakvGetLastError() returns the text of the most recent
 * failure on the calling thread.
 *
 * Each entry point cites the interface of the reference engine (fxslava/ascend-moe-engine,
 * paths relative to its tree) that it stands in for.
 */
#ifndef MLAKV_H_
#define MLAKV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t mlakvStatus;
/* Status codes follow the aclnn convention the reference checks against
 * (include/moe/core/op_table.hpp:142-147). */
#define MLAKV_SUCCESS 0
#define MLAKV_ERR_PARAM_NULLPTR 161001
#define MLAKV_ERR_PARAM_INVALID 161002
#define MLAKV_ERR_RUNTIME 361001
/* A refusal of the arena's phase contract (the reference throws Dsv4Error,
 * include/moe/core/error.hpp:38-77; the mock's contract code, mock/mock_descriptor.cpp:40-44). */
#define MLAKV_ERR_CONTRACT 100001

#define MLAKV_DTYPE_BF16 0
#define MLAKV_DTYPE_FP8_E4M3 1

const char* mlakvGetLastError(void);
/* Number of HIP devices visible; 0 without a GPU. Never fails. */
int32_t mlakvDeviceCount(void);
/* Warm-up for the current device: loads every kernel of the library onto it and sets the kernel
 * attributes the launches need (dynamic LDS above 64 KB), so that the first launch of each
 * operator inside a serving loop costs what the later ones cost. Optional (every launch makes
 * sure of its own kernels), idempotent, allocates no device memory, enqueues nothing. The
 * counterpart of what the reference pays once in aclInit / aclnnInit (src/core/acl_guard.cpp:22-46). */
mlakvStatus mlakvPrepare(void);

/* ------------------------------------------------------------------------- */
/* Paged cache geometry                                                       */
/* ------------------------------------------------------------------------- */

/* One paged MLA cache: a latent plane and a rope plane, each
 * [layer][physical block][slot][dim] (src/memory/static_arena_manager.cpp:315-318, :571-578),
 * plus, for FP8 rows, one fp32 scale per slot. A fused 576-element row is the special
 * case rope = latent + latent_dim elements with both row strides equal to the fused row. */
typedef struct mlakvCacheView {
  void* latent;
  int64_t latent_layer_stride, latent_block_stride, latent_row_stride;
  void* rope;
  int64_t rope_layer_stride, rope_block_stride, rope_row_stride;
  void* scale; /* fp32 [layer][block][slot]; NULL for bf16 */
  int64_t scale_layer_stride, scale_block_stride;
  int32_t num_layers;
  int32_t num_blocks; /* physical blocks per layer */
  int32_t block_size; /* token slots per block */
  int32_t latent_dim; /* 512: kv_lora_rank, include/moe/core/config.hpp:78-109 */
  int32_t rope_dim;   /* 64: qk_rope_head_dim */
  int32_t dtype;      /* MLAKV_DTYPE_* */
} mlakvCacheView;

/* ------------------------------------------------------------------------- */
/* Kernels                                                                    */
/* ------------------------------------------------------------------------- */

/* Append: replaces the launch of stage `kv_cache_write` = aclnnScatterPaKvCache
 * (src/pipeline/pipeline.cpp:226-234, :415; contract include/moe/core/op_table.hpp:339-372).
 * For every layer l in [layer_begin, layer_begin+layer_count) and token t with
 * slot_mapping[t] >= 0:  cache[l][slot/bs][slot%bs] = (latent_src[l][t], rope_src[l][t]).
 * Sources are bf16; an FP8 cache quantizes on append (E4M3, one fp32 scale per row =
 * absmax/448, 1 for a zero row). The reference launches one layer per call
 * (layer_count = 1); the batched form exists because 43 launches of 36 KB are
 * launch-bound. */
mlakvStatus mlakvAppend(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count,
                        const void* latent_src, int64_t latent_src_layer_stride, int64_t latent_src_row_stride,
                        const void* rope_src, int64_t rope_src_layer_stride, int64_t rope_src_row_stride,
                        const int32_t* slot_mapping, int32_t num_tokens, void* stream);

/* Fused latent RMSNorm + RoPE (key and, optionally, query slices) + append of one layer: the
 * stages `kv_a_norm`, `rope` and `kv_cache_write` that the reference launches back to back
 * (src/pipeline/pipeline.cpp:213-234; operator contracts include/moe/core/op_table.hpp:151-170
 * aclnnRmsNorm "y = x * gamma / sqrt(mean(x*x) + epsilon)", :315-337 aclnnApplyRotaryPosEmbV2 with
 * "half" rotation, :339-372 aclnnScatterPaKvCache; epsilon = kRmsNormEpsilon, config.hpp:56).
 * kv_a holds bf16 rows [latent 512 | rope 64] as the reference lays out act.kv_a
 * (src/memory/static_arena_manager.cpp:488-490); gamma is the layer's bf16 [512] weight;
 * rope_cos / rope_sin are bf16 tables [position][64] (row = position, pipeline.cpp:403-406);
 * positions and slot_mapping are device int32 [num_tokens]. For token t with p = positions[t]:
 *   y[d]    = bf16(x[d] * gamma[d] / sqrt(mean(x^2) + epsilon))
 *   r'[i]   = bf16(r[i] cos[p][i] - r[i+32] sin[p][i]),  r'[i+32] = bf16(r[i+32] cos[p][i+32] + r[i] sin[p][i+32])
 *   cache[layer][slot_mapping[t]] = (y, r')        (skipped when slot_mapping[t] < 0)
 * Arithmetic in fp32, one rounding to bf16; an FP8 cache quantizes the bf16 values as mlakvAppend
 * does. latent_normed_out (bf16 [num_tokens][512]) and rope_out (bf16 [num_tokens][64]) are
 * optional copies of y and r' (the reference's act.kv_latent_normed and the rotated k_rope;
 * rope_out may be the rope columns of kv_a itself, which is the reference's in-place rotation).
 * q_rope, when not null, is the query's rope slices bf16 [num_tokens][num_heads][64] at the given
 * byte strides (the reference's view into q_b, static_arena_manager.cpp:481-485: head stride
 * 576 * 2); they are rotated in place with the same table row, as the reference's one
 * aclnnApplyRotaryPosEmbV2 call rotates q_rope and k_rope together (pipeline.cpp:219-225). With
 * q_rope the table rows must be 16-byte aligned. */
mlakvStatus mlakvNormRopeAppend(const mlakvCacheView* cache, int32_t layer, const void* kv_a, int64_t kv_a_row_stride,
                                const void* gamma, double epsilon, const void* rope_cos, const void* rope_sin,
                                int64_t rope_table_row_stride, const int32_t* positions, const int32_t* slot_mapping,
                                int32_t num_tokens, void* latent_normed_out, int64_t latent_normed_row_stride,
                                void* rope_out, int64_t rope_out_row_stride, void* q_rope, int64_t q_rope_token_stride,
                                int64_t q_rope_head_stride, int32_t num_heads, void* stream);

/* Gather: the paged read that the reference leaves implicit inside its attention
 * operator (addressing as in third_party/ops_transformer/attention/quant_lightning_indexer/
 * op_kernel/arch35/quant_lightning_indexer_service_cube.h:243-270):
 *   dst[l][cu_seq_lens[b] + i] = cache[l][block_table[b][i / bs]][i % bs],  i < seq_lens[b].
 * Output rows are bf16 (FP8 caches are dequantized: e4m3 * scale). cu_seq_lens has
 * batch+1 entries (exclusive prefix sum of seq_lens); max_seq_len bounds every seq_lens[b]
 * and sizes the launch. table_stride is in int32 elements. */
mlakvStatus mlakvGather(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count,
                        const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens,
                        const int32_t* cu_seq_lens, int32_t batch, int32_t max_seq_len, void* latent_dst,
                        int64_t latent_dst_layer_stride, int64_t latent_dst_row_stride, void* rope_dst,
                        int64_t rope_dst_layer_stride, int64_t rope_dst_row_stride, void* stream);

/* mlakvGather that also times itself: the launch stamps its own start and end into the two
 * hipEvent_t (created by the caller with timing enabled); hipEventElapsedTime(start, stop) after
 * the stream has passed the launch is the kernel's duration. Unlike events recorded around a launch
 * these put no marker packets into the queue (measured: two recorded events cost a 0.7 ms step
 * 4 to 5 us). No counterpart in the reference; it is for benchmarks and profilers. An empty gather
 * launches nothing and is refused. */
mlakvStatus mlakvGatherTimed(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count,
                             const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens,
                             const int32_t* cu_seq_lens, int32_t batch, int32_t max_seq_len, void* latent_dst,
                             int64_t latent_dst_layer_stride, int64_t latent_dst_row_stride, void* rope_dst,
                             int64_t rope_dst_layer_stride, int64_t rope_dst_row_stride, void* stream,
                             void* start_event, void* stop_event);

/* Compaction copy: cache[l][dst_block] = cache[l][src_block] for every (src, dst) pair
 * in `moves` (device int32[2 * num_moves]) and every layer. Sources and destinations must
 * be disjoint sets, which the block pool's plan guarantees. No reference counterpart
 * (the reference never recycles a block). */
mlakvStatus mlakvCopyBlocks(const mlakvCacheView* cache, int32_t layer_begin, int32_t layer_count,
                            const int32_t* moves, int32_t num_moves, void* stream);

/* Decode attention: replaces the plan + launch of stage `attention` =
 * aclnnFusedInferAttentionScoreV5 (src/pipeline/pipeline.cpp:235-249, :416; contract
 * include/moe/core/op_table.hpp:375-454; constants include/moe/core/config.hpp:193-201).
 *   s_i = scale * (q_latent[b,h] . c_i + q_rope[b,h] . r_i), p = softmax_i(s),
 *   out[b,h] = sum_i p_i c_i     over the seq_lens[b] cached rows of sequence b,
 * one query token per sequence, `heads` query heads sharing one latent KV head.
 * The plan fixes shapes and the workspace; the launch only enqueues.
 *
 * How the work is cut: the contexts of the batch, counted in 32-token tiles and laid end to end,
 * are divided into equal work units, one per workgroup (one workgroup per CU and group of 64
 * heads), at every launch from the live seq_lens on the device; a sequence shorter than
 * its neighbours costs its own tiles and no more. A unit that holds a whole sequence writes that
 * sequence's output; the others leave partial results in the workspace, which a second small
 * launch merges (MLAKV_ATTN_MERGE_SECOND_LAUNCH, the default) or the same launch does
 * (MLAKV_ATTN_MERGE_IN_LAUNCH: contributors meet on counters the library keeps in a static device
 * array, with a bounded wait; measured no faster on MI355X, kept for callers that want one
 * launch). seq_lens[b] is read as min(max(seq_lens[b], 0), max_seq_len).
 * Limits of MLAKV_ATTN_MERGE_IN_LAUNCH: the counters are 16 regions per GPU, handed to the launches
 * of a process in turn. Launches that are ordered (one stream, or streams joined by events) can be
 * of any number; of launches that may run side by side on unordered streams at most 16 may be in
 * flight on one GPU, or two of them share counters and merge wrongly. A region's words are zero
 * between launches because the last contributor of every sequence clears them: a launch that is
 * torn down midway (device reset, process kill) leaves them as they are for the next user of that
 * region in the same process. The second-launch merge has neither limit. */
#define MLAKV_ATTN_MERGE_AUTO 0
#define MLAKV_ATTN_MERGE_IN_LAUNCH 1
#define MLAKV_ATTN_MERGE_SECOND_LAUNCH 2
typedef struct mlakvAttnPlan {
  int32_t batch;
  int32_t heads;           /* multiple of 16, at most 128 */
  int32_t max_seq_len;
  int32_t block_size;
  int32_t dtype;           /* cache dtype */
  int32_t chunk_tiles;     /* tiles per work unit when fixed by mlakvAttnPlanInitEx; 0: from the live lengths */
  int32_t work_groups;     /* workgroups per group of 64 heads */
  int32_t max_units;       /* bound on the work units of one launch (sizes the workspace) */
  int32_t merge_mode;      /* MLAKV_ATTN_MERGE_IN_LAUNCH or _SECOND_LAUNCH */
  int32_t merge_spin_us;   /* bound of the in-launch merge's wait for a sequence's other partials */
  int32_t reserved;        /* 1: made by mlakvAttnSparsePlanInit (max_seq_len holds sparse_count) */
  int32_t selection_units; /* selected-token plans: MLAKV_ATTN_UNITS_SPLIT, _HEAD_BLOCK or _HEAD_BLOCK_HALVES, fixed by the plan;
                            * whole-context plans: what the options asked for, MLAKV_ATTN_UNITS_AUTO = every launch chooses */
  uint64_t workspace_bytes;
} mlakvAttnPlan;

mlakvStatus mlakvAttnPlanInit(int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size, int32_t dtype,
                              mlakvAttnPlan* plan);

/* The same with the planner's choices spelled out (tests and measurements use it to force many
 * small units, a single unit per sequence, the second-launch merge or a wait that gives up at
 * once); a zero field keeps the default. No reference counterpart. */
/* How a selected-token launch cuts its work.
 * SPLIT: the selections of the batch laid end to end and cut into one unit per CU, 64 heads per
 *   unit; units that hold part of a selection leave partials that a merge puts together.
 * HEAD_BLOCK: one unit = the whole selection of one sequence for 16 heads; nothing to merge and the
 *   workspace stays untouched. sparse_count up to MLAKV_ATTN_HEAD_BLOCK_TOKENS.
 * HEAD_BLOCK_HALVES: the same unit taken by two workgroups, half of the selection's tiles each; each
 *   leaves a partial (16 rows) in the workspace and counts itself on a word of the library's
 *   counters (those of MLAKV_ATTN_MERGE_IN_LAUNCH, with their limit on launches in flight); the
 *   second to finish combines the two inside the launch, nobody waits. Up to 2048 (sequence, 16
 *   heads) pairs.
 * AUTO, unless chunk_tiles, work_groups or merge_mode ask for properties of the split, takes what
 * was measured ahead. bf16 caches: HEAD_BLOCK_HALVES from 257 to 768 selected tokens while two
 * workgroups per unit fit the CUs once; else HEAD_BLOCK up to 512 selected tokens while batch x
 * heads / 16 units fit the CUs once and up to 256 while they fit twice; else SPLIT. FP8 caches:
 * HEAD_BLOCK_HALVES from 257 selected tokens while two workgroups per unit fit the CUs once; else
 * HEAD_BLOCK while the units fit the CUs four times (beyond that up to 256 selected tokens); else
 * SPLIT.
 * Whole-context plans (mlakvAttnPlanInit[Ex] without `selection`) use the same units for short
 * contexts: a unit then takes every position of its sequence. AUTO decides at every launch from
 * the longest context the launch can see -- the lengths themselves with mlakvAttnDecodeHostLens,
 * the plan's max_seq_len with lengths in device memory: while two workgroups per unit fit the CUs
 * once, HEAD_BLOCK up to 256 tokens and HEAD_BLOCK_HALVES up to 768; while one per unit fits,
 * HEAD_BLOCK up to 512; while they fit twice, up to 256; the 64-head kernel otherwise and whenever
 * chunk_tiles, work_groups or merge_mode ask for properties of the split. SPLIT keeps the 64-head
 * kernel always; HEAD_BLOCK and HEAD_BLOCK_HALVES ask for the units (max_seq_len up to
 * MLAKV_ATTN_HEAD_BLOCK_TOKENS). The two kinds of kernel round differently (both inside the stated
 * tolerance), so launches of one plan that see different lengths may differ in the last bits. */
#define MLAKV_ATTN_UNITS_AUTO 0
#define MLAKV_ATTN_UNITS_SPLIT 1
#define MLAKV_ATTN_UNITS_HEAD_BLOCK 2
#define MLAKV_ATTN_UNITS_HEAD_BLOCK_HALVES 3
#define MLAKV_ATTN_HEAD_BLOCK_TOKENS 1024
typedef struct mlakvAttnPlanOptions {
  int32_t chunk_tiles;    /* tiles per work unit, fixed instead of derived from the live lengths */
  int32_t work_groups;    /* workgroups per group of 64 heads (default: CUs / head groups) */
  int32_t merge_mode;     /* MLAKV_ATTN_MERGE_* */
  int32_t merge_spin_us;  /* > 0: microseconds; < 0: do not wait at all (the last contributor merges) */
  int32_t selection;      /* 1: a plan for mlakvAttnDecodeSparse; max_seq_len then holds sparse_count */
  int32_t selection_units; /* MLAKV_ATTN_UNITS_* */
  int32_t reserved[2];    /* zero */
} mlakvAttnPlanOptions;
mlakvStatus mlakvAttnPlanInitEx(int32_t batch, int32_t heads, int32_t max_seq_len, int32_t block_size, int32_t dtype,
                                const mlakvAttnPlanOptions* options, mlakvAttnPlan* plan);

/* q strides: bytes between sequences / between heads. out is bf16 [batch, heads, latent_dim]
 * with its own strides; lse (optional) is fp32 [batch, heads], natural log of the softmax
 * denominator. workspace must hold plan->workspace_bytes. */
mlakvStatus mlakvAttnDecode(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                            const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                            const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                            const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, double scale,
                            void* out, int64_t out_seq_stride, int64_t out_head_stride, float* lse, void* workspace,
                            uint64_t workspace_bytes, void* stream);

/* mlakvAttnDecode for a caller that keeps the lengths in device memory (a recorded step reads them
 * there) and still knows, on the host, a bound they stay under: `longest` >= seq_lens[b] for every
 * sequence when the launch runs. The launch chooses its kernels by `longest` as
 * mlakvAttnDecodeHostLens does by the lengths themselves (short contexts: the units of 16 heads).
 * The bound is the caller's word: a length above it is read as `longest`. No reference
 * counterpart. */
mlakvStatus mlakvAttnDecodeBounded(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                                   const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                                   const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                                   const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, int32_t longest,
                                   double scale, void* out, int64_t out_seq_stride, int64_t out_head_stride, float* lse,
                                   void* workspace, uint64_t workspace_bytes, void* stream);

/* mlakvAttnDecode for a caller that knows the live lengths on the host (the engine's decode loop
 * does: src/pipeline/pipeline.cpp:515-519 derives the position on the host): host_seq_lens holds
 * plan->batch values, at most MLAKV_ATTN_HOST_LENS_MAX; they are copied into the kernels' argument
 * block, so nothing is uploaded and the buffer is free again on return. A larger batch is refused
 * with MLAKV_ERR_PARAM_INVALID: upload the lengths and call mlakvAttnDecode. */
#define MLAKV_ATTN_HOST_LENS_MAX 64
mlakvStatus mlakvAttnDecodeHostLens(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                                    const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                                    const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                                    const int32_t* block_table, int32_t table_stride, const int32_t* host_seq_lens,
                                    double scale, void* out, int64_t out_seq_stride, int64_t out_head_stride, float* lse,
                                    void* workspace, uint64_t workspace_bytes, void* stream);

/* mlakvAttnDecode for callers that cannot allocate device memory and have no workspace to pass
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference, whose operators always receive the arena's shared workspace
 * (src/memory/static_arena.cpp:270-295). The split-KV partials go to a static device array of
 * MLAKV_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process
 * ends; the call allocates nothing (no hipMalloc / hipFree, no allocating library routine) and
 * otherwise behaves like mlakvAttnDecode: same arguments without the workspace pair, same
 * results bit for bit. A plan whose workspace_bytes exceeds MLAKV_NOALLOC_SCRATCH_BYTES is
 * refused with MLAKV_ERR_PARAM_INVALID. The first call on a device resolves the array's address
 * (make it outside any stream capture). All calls on one GPU share the array: launches that may
 * overlap there (different streams without an ordering between them) race on the partials. */
#define MLAKV_NOALLOC_SCRATCH_BYTES (24ull << 20)
mlakvStatus mlakvAttnDecodeNoAlloc(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                                   const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                                   const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                                   const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, double scale,
                                   void* out, int64_t out_seq_stride, int64_t out_head_stride, float* lse, void* stream);

/* Block-32 MX quantization of bf16 rows along the last axis: replaces the plan + launch of
 * aclnnDynamicMxQuant (contract include/moe/core/op_table.hpp:205-233; the reference's stages
 * `attn_quant` src/pipeline/pipeline.cpp:251-258 and `shared_act_quant`), with the reference's
 * fixed attributes: axis -1, round mode rint, dst E4M3, blocksize 32, OCP scale algorithm
 * (OCP Microscaling Formats v1.0, 6.3):
 *   shared_exp = floor(log2(max |v|)) - 8 clamped to [-127, 127], scale byte = shared_exp + 127 (E8M0)
 *   code       = e4m3(v * 2^-shared_exp), nearest even, saturating at +-448
 * A block of zeros gets scale byte 0 and zero codes; a block holding Inf/NaN gets scale 0xff and
 * NaN codes. x is bf16 [rows][cols] (cols a multiple of 32), codes E4M3 [rows][cols], scales
 * E8M0 [rows][cols / 32]; strides in bytes. */
mlakvStatus mlakvDynamicMxQuant(const void* x, int64_t x_row_stride, int64_t rows, int32_t cols, void* codes,
                                int64_t codes_row_stride, void* scales, int64_t scales_row_stride, void* stream);

/* Where the quantized attention output goes: codes E4M3 [batch][heads][512] and scales E8M0
 * [batch][heads][16] at byte strides (the reference's act.attn_fp8 [tokens][heads * 512] and
 * act.attn_mx_scale [tokens][heads * 16], src/memory/static_arena_manager.cpp:493-496). */
typedef struct mlakvMxQuantOut {
  void* codes;
  int64_t codes_seq_stride, codes_head_stride;
  void* scales;
  int64_t scales_seq_stride, scales_head_stride;
} mlakvMxQuantOut;

/* Decode attention with the quantization of its output fused into the epilogue: the stages
 * `attention` and `attn_quant` that the reference launches back to back
 * (src/pipeline/pipeline.cpp:235-258, :416-417) in one call. The codes and scales are those
 * mlakvDynamicMxQuant gives on the bf16 output of mlakvAttnDecode, bit for bit; `out` (bf16) is
 * optional here and, when given, receives that output as well. */
mlakvStatus mlakvAttnDecodeMxQuant(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                                   const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                                   const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                                   const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, double scale,
                                   void* out, int64_t out_seq_stride, int64_t out_head_stride, const mlakvMxQuantOut* quant,
                                   float* lse, void* workspace, uint64_t workspace_bytes, void* stream);

/* Selected-token decode attention: the consumer of the Lightning Indexer's output, i.e. the same
 * attention over the k best tokens of each sequence instead of its whole context (the model's
 * long-context mechanism: index_topk = kIndexTopK = 512, include/moe/core/config.hpp:49-51;
 * selection contract aclnnQuantLightningIndexer, include/moe/core/op_table.hpp:964-1006: INT32
 * indices [B, S1, N2, k], sparse_count in [1, 2048]; the vendored kernel writes the valid indices
 * first and fills the rest with -1, third_party/ops_transformer/attention/quant_lightning_indexer/
 * op_kernel/arch35/quant_lightning_indexer_service_vector.h:446-541). The reference's pipeline does
 * not launch a sparse attention yet (src/pipeline/pipeline.cpp:576-578 reports it as not
 * applied), so this entry has no stage to replace; it reads the same paged pool through the same
 * block table.
 *   sparse_indices: device int32 [batch][sparse_count] at `sparse_indices_seq_stride` elements per
 *   sequence; sequence b attends to the cached rows at positions sparse_indices[b][0 .. n-1], where
 *   n is the number of entries before the first one that is negative or >= seq_lens[b]
 *   (n = 0: zeros, lse = -inf). Order does not matter; repeated positions count repeatedly.
 * The plan comes from mlakvAttnSparsePlanInit (sparse_count takes the place of max_seq_len); how
 * it cuts the work (plan->selection_units) is described with MLAKV_ATTN_UNITS_* above. The
 * workspace is required either way; whole-selection units leave it untouched, halved ones use
 * its first 2112 bytes x batch x heads. */
mlakvStatus mlakvAttnSparsePlanInit(int32_t batch, int32_t heads, int32_t sparse_count, int32_t block_size, int32_t dtype,
                                    mlakvAttnPlan* plan);
mlakvStatus mlakvAttnDecodeSparse(const mlakvAttnPlan* plan, const mlakvCacheView* cache, int32_t layer,
                                  const void* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                                  const void* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                                  const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens,
                                  const int32_t* sparse_indices, int64_t sparse_indices_seq_stride, double scale,
                                  void* out, int64_t out_seq_stride, int64_t out_head_stride, float* lse, void* workspace,
                                  uint64_t workspace_bytes, void* stream);

/* Lightning Indexer for decode (one query token per sequence): replaces the plan + launch of
 * aclnnQuantLightningIndexer (contract include/moe/core/op_table.hpp:964-1006; kernel vendored
 * under third_party/ops_transformer/attention/quant_lightning_indexer, formula in its README.md)
 * with the engine's fixed attributes: E4M3 query and key, per-token-head quantization (mode 0),
 * key layout PA_BSND with N2 = 1 and D = 128, causal sparse mode (for one query token: every
 * cached token is eligible).
 *   score[b][t] = key_scale[t] * sum_h (weights[b][h] * query_dequant_scale[b][h]) * ReLU(q[b][h] . k[t])
 *   sparse_indices[b] = the sparse_count positions with the largest scores
 * Scores are compared as bf16 (fp32 arithmetic in the vendored kernel's order, rounded with ties
 * away from zero); equal scores go to the lower position. Output per sequence, as the vendored
 * kernel writes it: a sequence no longer than sparse_count yields 0 .. len-1; otherwise the
 * positions above the k-th score in increasing order, then those equal to it; the rest is -1.
 * This is the list mlakvAttnDecodeSparse takes.
 *   keys: the paged pool of index keys, E4M3 [block][slot][128] with one fp32 dequantization scale
 *   per row, addressed through the same block table as the KV cache.
 *   query E4M3 [batch][heads][128] (strides in bytes), weights bf16 [batch][heads] (byte stride),
 *   query_dequant_scale fp32 [batch][heads] (element stride); heads in {16, 32, 48, 64}.
 *   workspace: mlakvIndexerWorkspaceBytes(batch, max_seq_len) bytes (the 16-bit scores). */
typedef struct mlakvIndexKeyView {
  const void* keys;
  int64_t block_stride, row_stride;  /* bytes */
  const float* scales;
  int64_t scale_block_stride;        /* elements */
  int32_t num_blocks, block_size, dim, reserved;
} mlakvIndexKeyView;
uint64_t mlakvIndexerWorkspaceBytes(int32_t batch, int32_t max_seq_len);
/* Writes index keys into that pool: row t of `k` (bf16 [num_tokens][128], stride in bytes) is
 * quantised like a row of the FP8 KV cache (scale = absmax / 448 in fp32, 1.0 for a zero row;
 * code = E4M3 of the correctly rounded x / scale, saturating) and lands at slot_mapping[t] =
 * block * block_size + slot of the pool (`keys->keys` and `keys->scales` are written through); a
 * negative slot or a block outside the pool skips the row, as in mlakvAppend. The reference has no
 * such stage (it reserves no index-key pool, src/pipeline/pipeline.cpp:576-578): the write side of
 * the vendored operator's key input (third_party/ops_transformer/attention/quant_lightning_indexer,
 * key + key_dequant_scale, "PA_BSND"), for callers that keep the keys paged beside the KV cache. */
mlakvStatus mlakvIndexKeyAppend(const mlakvIndexKeyView* keys, const void* k, int64_t k_row_stride,
                                const int32_t* slot_mapping, int32_t num_tokens, void* stream);
mlakvStatus mlakvLightningIndexer(const mlakvIndexKeyView* keys, const void* query, int64_t query_seq_stride,
                                  int64_t query_head_stride, const void* weights, int64_t weights_seq_stride,
                                  const float* query_dequant_scale, int64_t query_scale_seq_stride, int32_t heads,
                                  const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens, int32_t batch,
                                  int32_t max_seq_len, int32_t sparse_count, int32_t* sparse_indices,
                                  int64_t sparse_indices_seq_stride, void* workspace, uint64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* Static arena (host)                                                        */
/* ------------------------------------------------------------------------- */

/* The three-phase single-allocation arena, same calls and refusals as the reference's
 * StaticMemoryArena (include/moe/memory/static_arena.hpp:79-181, src/memory/static_arena.cpp):
 * Reserve :88-102, Commit :108-118, Address/Bytes :120-129, NoteWorkspace/CommitWorkspace/
 * AssertWorkspaceFits :270-295, Seal :301-304, ValidateAlignment :310-332, DescribeLedger :334-348.
 * A refusal returns MLAKV_ERR_CONTRACT where the reference throws. */
typedef struct mlakvArena mlakvArena;
#define MLAKV_BACKEND_HIP 0   /* hipMalloc / hipMemset on the current device */
#define MLAKV_BACKEND_HOST 1  /* 4096-aligned host memory: the counterpart of the reference's
                                 SimulatedDeviceOps (src/core/device_ops.cpp:268-440), for
                                 exercising the arena and block pool without a GPU. Kernels
                                 never run on it. */
mlakvStatus mlakvArenaCreate(int32_t backend, mlakvArena** arena);
void mlakvArenaDestroy(mlakvArena* arena);
mlakvStatus mlakvArenaReserve(mlakvArena* arena, const char* name, size_t bytes, size_t align, size_t* handle);
mlakvStatus mlakvArenaCommit(mlakvArena* arena);
mlakvStatus mlakvArenaAddress(const mlakvArena* arena, size_t handle, void** address);
mlakvStatus mlakvArenaBytes(const mlakvArena* arena, size_t handle, size_t* bytes);
mlakvStatus mlakvArenaOffset(const mlakvArena* arena, size_t handle, size_t* offset);
mlakvStatus mlakvArenaNoteWorkspace(mlakvArena* arena, uint64_t bytes);
mlakvStatus mlakvArenaCommitWorkspace(mlakvArena* arena);
mlakvStatus mlakvArenaAssertWorkspaceFits(const mlakvArena* arena, uint64_t bytes, const char* what);
mlakvStatus mlakvArenaSeal(mlakvArena* arena);
mlakvStatus mlakvArenaValidateAlignment(const mlakvArena* arena);
void* mlakvArenaWorkspace(const mlakvArena* arena);
uint64_t mlakvArenaWorkspaceBytes(const mlakvArena* arena);
size_t mlakvArenaTotalBytes(const mlakvArena* arena);
size_t mlakvArenaReservedBytes(const mlakvArena* arena);
size_t mlakvArenaReservationCount(const mlakvArena* arena);
int32_t mlakvArenaSealed(const mlakvArena* arena);
/* Device allocations served so far by the arena's backend; the zero-allocation-per-step
 * invariant is checked by watching it (include/moe/core/device_allocator.hpp:47-50). */
uint64_t mlakvArenaDeviceAllocationCount(const mlakvArena* arena);
/* Writes the ledger text (NUL-terminated, truncated to capacity); returns the full length. */
size_t mlakvArenaDescribeLedger(const mlakvArena* arena, char* buffer, size_t capacity);

/* ------------------------------------------------------------------------- */
/* KV cache manager (host): reservations, block pool, per-step metadata       */
/* ------------------------------------------------------------------------- */

/* The KV part of the reference's StaticArenaManager (src/memory/static_arena_manager.cpp:
 * num_blocks :192-201, reservations :298-300 and :315-318, per-layer strides
 * src/pipeline/pipeline.cpp:390-395, slot mapping :515-519, diagnostics :134-136 and :532-534),
 * generalised from one sequence with identity paging to a batch over a shared pool of
 * physical blocks with a free list, recycling and compaction. */
typedef struct mlakvKvConfig {
  int64_t num_layers;       /* 43: include/moe/core/config.hpp:38 */
  int64_t block_size;       /* RuntimeConfig::block_size */
  int64_t max_context_len;  /* RuntimeConfig::max_context_len */
  int64_t max_batch;        /* 1 in the reference (kTokensPerStep) */
  int64_t pool_blocks;      /* physical blocks per layer; 0 = max_batch * ceil(max_context_len / block_size) */
  int64_t kv_lora_rank;     /* 512 */
  int64_t qk_rope_head_dim; /* 64 */
  int32_t dtype;            /* MLAKV_DTYPE_* */
  int32_t fused_rows;       /* 0: two planes as in the reference; 1: one plane of 576-element rows */
  uint64_t seed;            /* free-list shuffle seed */
  int32_t shuffle;          /* 0: free list in id order (identity paging for one sequence) */
  int32_t reserved;
} mlakvKvConfig;

typedef struct mlakvKvStats { /* include/moe/diagnostics/inference_stats.hpp:21-28 */
  uint64_t total_blocks_allocated;
  uint64_t active_context_tokens;
  uint64_t block_size;
  double kv_cache_utilization;
} mlakvKvStats;

typedef struct mlakvKvCache mlakvKvCache;
/* RESERVE phase: records kv.block_table, kv.slot_mapping, kv.seq_lens, kv.cu_seq_lens,
 * kv.compaction_moves, kv.latent_cache, kv.rope_cache (and kv.scale_cache for FP8) in `arena`. */
mlakvStatus mlakvKvCacheCreate(mlakvArena* arena, const mlakvKvConfig* config, mlakvKvCache** cache);
void mlakvKvCacheDestroy(mlakvKvCache* cache);
/* After mlakvArenaCommit: resolves the reservations to addresses. */
mlakvStatus mlakvKvCacheBind(mlakvKvCache* cache);
mlakvStatus mlakvKvCacheGetView(const mlakvKvCache* cache, mlakvCacheView* view);
int64_t mlakvKvCacheNumBlocks(const mlakvKvCache* cache);      /* per sequence: ceil(max_ctx / bs) */
int64_t mlakvKvCachePoolBlocks(const mlakvKvCache* cache);
mlakvStatus mlakvKvCacheAddSequence(mlakvKvCache* cache, int64_t seq, int64_t context_len);
/* Bookkeeping for one decode step of sequence `seq`: the slot of its next token
 * (slot = table[pos / bs] * bs + pos % bs; identity paging gives slot = position,
 * src/pipeline/pipeline.cpp:517). */
mlakvStatus mlakvKvCacheAppendToken(mlakvKvCache* cache, int64_t seq, int32_t* slot);
/* The same for every live sequence in one call (the batched decode step): slots, when not NULL,
 * receives max_batch entries, -1 for an unused sequence; appended receives the count. The slot
 * mapping that mlakvKvCacheUploadStep sends holds one entry per sequence, the slot of its latest
 * token: a caller that appends several tokens of one sequence between uploads (a prefill) keeps
 * the slots these calls return and passes them to mlakvAppend itself. */
mlakvStatus mlakvKvCacheAppendTokenAll(mlakvKvCache* cache, int32_t* slots, int64_t* appended);
mlakvStatus mlakvKvCacheFreeSequence(mlakvKvCache* cache, int64_t seq);
/* Plans the defragmentation (live blocks to ids [0, n_live)), rewrites the host tables and
 * free list, writes the (src, dst) pairs to `moves` (capacity 2 * pool_blocks, may be NULL)
 * and, when the arena is on the HIP backend, uploads them and enqueues the copy kernel. May be
 * called between mlakvKvCacheAppendToken and mlakvKvCacheUploadStep: the slots of tokens that
 * wait for the upload follow their blocks. */
mlakvStatus mlakvKvCacheCompact(mlakvKvCache* cache, int32_t* moves, int64_t* num_moves, void* stream);
/* Enqueues the H2D copy of this step's metadata (block table, slot mapping, seq_lens,
 * cu_seq_lens) from the pinned mirror; the batched form of the reference's 4-byte
 * slot mailbox copy (src/pipeline/pipeline.cpp:515-519). On the host backend it is a memcpy. */
mlakvStatus mlakvKvCacheUploadStep(mlakvKvCache* cache, void* stream);
/* mlakvKvCacheUploadStep followed by mlakvAppend of one row per sequence with the cache's own slot
 * mapping (the per-step pair of src/pipeline/pipeline.cpp:515-519 and :399-404, for all layers
 * [layer_begin, layer_begin + layer_count) at once): the row of sequence s of layer l is at
 * src + l * layer_stride + s * row_stride (bf16, 16-byte aligned, strides multiples of 16);
 * sequences without a token this step are skipped. When the step's metadata fits the argument
 * block of one kernel (the usual decode step) both happen in ONE launch; otherwise it is the
 * two calls. HIP backend only. */
mlakvStatus mlakvKvCacheUploadStepAndAppend(mlakvKvCache* cache, int32_t layer_begin, int32_t layer_count, const void* latent_src,
                                            int64_t latent_src_layer_stride, int64_t latent_src_row_stride, const void* rope_src,
                                            int64_t rope_src_layer_stride, int64_t rope_src_row_stride, void* stream);
mlakvStatus mlakvKvCacheGetStats(const mlakvKvCache* cache, mlakvKvStats* stats);
/* The "paged_attention" member of the reference's --diag-json file, byte for byte as
 * InferenceDiagnostics::DumpJson writes it (src/diagnostics/inference_stats.cpp:42-47: two-space
 * member indent, numbers at 12 significant digits, null for a non-finite utilization; sample
 * docs/examples/inference_diagnostics_dry_run.json), without a trailing comma or newline, for a
 * harness that assembles that file. Returns the length needed excluding the terminator (call with
 * buffer NULL to size it), or -1 for a null stats pointer; writes at most `capacity` bytes. */
int64_t mlakvKvStatsFormatJson(const mlakvKvStats* stats, char* buffer, size_t capacity);
/* Host mirrors (valid until the cache is destroyed). */
const int32_t* mlakvKvCacheHostBlockTable(const mlakvKvCache* cache);  /* [max_batch][num_blocks] */
const int32_t* mlakvKvCacheHostSlotMapping(const mlakvKvCache* cache); /* [max_batch], -1 = no token this step */
const int32_t* mlakvKvCacheHostSeqLens(const mlakvKvCache* cache);     /* [max_batch], 0 for unused */
int64_t mlakvKvCacheFreeBlocks(const mlakvKvCache* cache);
int64_t mlakvKvCacheFreeList(const mlakvKvCache* cache, int32_t* out); /* head first; returns length */
/* Device addresses inside the arena (NULL before Bind). */
int32_t* mlakvKvCacheDeviceBlockTable(const mlakvKvCache* cache);
int32_t* mlakvKvCacheDeviceSlotMapping(const mlakvKvCache* cache);
int32_t* mlakvKvCacheDeviceSeqLens(const mlakvKvCache* cache);
int32_t* mlakvKvCacheDeviceCuSeqLens(const mlakvKvCache* cache);

/* Pure arithmetic mirrors, usable without any allocation. */
int64_t mlakvNumBlocks(int64_t max_context_len, int64_t block_size); /* -1 = refused */
uint64_t mlakvBackboneDeviceBytes(int64_t kv_lora_rank, int64_t qk_rope_head_dim, int64_t block_size,
                                  int64_t max_context_len); /* static_arena_manager.cpp:205-241 */

#ifdef __cplusplus
}
#endif
#endif /* MLAKV_H_ */
