/*
 * kv_oracle.h -- CPU restatement of the paged MLA KV-cache path. TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker for the HIP implementation. Nothing in the shipped
 * product may link, load or call it: only the test suite, the smoke entry and the
 * cpu_baseline leg of the benchmark do, and there only to produce expected values
 * or a CPU timing.
 *
 * Every function names the reference file:line it follows (paths relative to the
 * reference tree). Where the reference has no counterpart (batched block pool,
 * FP8 rows, compaction, attention numerics -- its operators are closed binaries and
 * its mock executes nothing) the header says so and names what pins the function
 * instead.
 *
 * PARITY STATUS
 *   pinned by the reference itself (oracle/_ref probe + golden ledger):
 *     kvo_align_up, kvo_divide_up, kvo_num_blocks, kvo_backbone_device_bytes,
 *     kvo_kv_reservation_bytes, kvo_arena_*, kvo_kv_stats
 *   pinned by closed form / brute force / library routine (no reference numerics exist):
 *     kvo_slot, kvo_append_rows, kvo_gather_rows (memcpy identities),
 *     kvo_splitmix64 (published known answers), kvo_pool_* (invariants, brute force),
 *     kvo_e4m3_* and kvo_bf16_* (torch CPU casts, exhaustive decode table),
 *     kvo_mla_decode (float64 torch softmax on small inputs, special cases)
 *   parity unpinned against the reference's device results: append bytes, gathered
 *     bytes and attention values as produced by CANN's aclnnScatterPaKvCache /
 *     aclnnFusedInferAttentionScoreV5 (CANN 9.2.0-beta.2, closed, absent).
 */
#ifndef KV_ORACLE_H_
#define KV_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVO_OK 0
#define KVO_REFUSED 1

#define KVO_DTYPE_BF16 0
#define KVO_DTYPE_FP8_E4M3 1

/* ---- layout arithmetic --------------------------------------------------- */

/* src/memory/expert_layout.cpp:27 */
size_t kvo_align_up(size_t value, size_t alignment);
/* src/memory/static_arena_manager.cpp:183 */
int64_t kvo_divide_up(int64_t value, int64_t divisor);
/* src/memory/static_arena_manager.cpp:192-201; -1 when the reference constructor refuses. */
int64_t kvo_num_blocks(int64_t max_context_len, int64_t block_size);
/* src/memory/static_arena_manager.cpp:205-241 */
uint64_t kvo_backbone_device_bytes(int64_t kv_lora_rank, int64_t qk_rope_head_dim, int64_t block_size,
                                   int64_t max_context_len);

/* Sizes of the four KV reservations, src/memory/static_arena_manager.cpp:298-300, :315-318.
 * `tokens_per_step` is 1 in the reference (kTokensPerStep); a batch generalises it. */
typedef struct kvo_kv_reservation_bytes_t {
  uint64_t block_table;
  uint64_t slot_mapping;
  uint64_t latent_cache;
  uint64_t rope_cache;
} kvo_kv_reservation_bytes_t;
void kvo_kv_reservation_bytes(int64_t num_layers, int64_t tokens_per_step, int64_t num_blocks, int64_t block_size,
                              int64_t kv_lora_rank, int64_t qk_rope_head_dim, kvo_kv_reservation_bytes_t* out);

/* KV diagnostics, src/pipeline/pipeline.cpp:134-136 and :532-534. */
typedef struct kvo_kv_stats_t {
  uint64_t total_blocks_allocated;
  uint64_t active_context_tokens;
  uint64_t block_size;
  double kv_cache_utilization;
} kvo_kv_stats_t;
void kvo_kv_stats(int64_t num_layers, int64_t num_blocks, int64_t block_size, int64_t position, kvo_kv_stats_t* out);

/* ---- static arena (src/memory/static_arena.cpp) -------------------------- */

typedef struct kvo_arena kvo_arena;
kvo_arena* kvo_arena_new(void);
void kvo_arena_delete(kvo_arena* arena);
/* :88-102 */
int kvo_arena_reserve(kvo_arena* arena, const char* name, size_t bytes, size_t align, size_t* handle);
/* :108-118; `base` plays the address the single device allocation returned. */
int kvo_arena_commit(kvo_arena* arena, uintptr_t base);
/* :120-129 */
int kvo_arena_address(const kvo_arena* arena, size_t handle, uintptr_t* address);
int kvo_arena_bytes(const kvo_arena* arena, size_t handle, size_t* bytes);
int kvo_arena_offset(const kvo_arena* arena, size_t handle, size_t* offset);
/* :270-295 */
int kvo_arena_note_workspace(kvo_arena* arena, uint64_t bytes);
int kvo_arena_commit_workspace(kvo_arena* arena);
int kvo_arena_workspace_fits(const kvo_arena* arena, uint64_t bytes);
uint64_t kvo_arena_workspace_bytes(const kvo_arena* arena);
/* :301-304 */
int kvo_arena_seal(kvo_arena* arena);
int kvo_arena_sealed(const kvo_arena* arena);
/* :310-332 */
int kvo_arena_validate(const kvo_arena* arena);
size_t kvo_arena_total_bytes(const kvo_arena* arena);
size_t kvo_arena_reserved_bytes(const kvo_arena* arena);
size_t kvo_arena_count(const kvo_arena* arena);
int kvo_arena_allocations(const kvo_arena* arena);

/* ---- paged addressing ---------------------------------------------------- */

/* slot = table[pos / bs] * bs + pos % bs. Paged addressing as in
 * third_party/ops_transformer/attention/quant_lightning_indexer/op_kernel/arch35/
 * quant_lightning_indexer_service_cube.h:243-270; with an identity table this is the
 * reference's slot = position (src/pipeline/pipeline.cpp:517). */
int64_t kvo_slot(const int32_t* table_row, int64_t position, int64_t block_size);

/* Scatter of token rows into one plane of one layer: for each t with slots[t] >= 0,
 * plane[slot/bs][slot%bs][:] = src[t][:] (contract of aclnnScatterPaKvCache mode "Norm",
 * include/moe/core/op_table.hpp:339-372). All strides in bytes. */
void kvo_append_rows(uint8_t* plane, int64_t block_stride, int64_t row_stride, int64_t block_size,
                     const uint8_t* src, int64_t src_row_stride, int64_t row_bytes, const int32_t* slots,
                     int64_t num_tokens);

/* Block-table gather of one plane of one layer into packed per-sequence rows:
 * dst[cu(b) + i][:] = plane[table[b][i/bs]][i%bs][:], i < seq_lens[b]. */
void kvo_gather_rows(const uint8_t* plane, int64_t block_stride, int64_t row_stride, int64_t block_size,
                     const int32_t* table, int64_t table_stride, const int32_t* seq_lens, int64_t batch,
                     uint8_t* dst, int64_t dst_row_stride, int64_t row_bytes);

/* Block copy used by compaction: plane[dst_block] = plane[src_block] for each move. */
void kvo_copy_blocks(uint8_t* plane, int64_t block_stride, int64_t block_bytes, const int32_t* moves,
                     int64_t num_moves);

/* ---- number formats ------------------------------------------------------ */

uint16_t kvo_bf16_from_f32(float value); /* round to nearest even; NaN stays NaN */
float kvo_bf16_to_f32(uint16_t bits);
/* OCP FP8 E4M3FN: bias 7, no infinities, 0x7f/0xff NaN, max finite 448
 * (reference constant kSwigluMaxDtypeValue, include/moe/core/config.hpp:191). Encode rounds
 * to nearest even and saturates finite inputs to +-448. */
uint8_t kvo_e4m3_from_f32(float value);
float kvo_e4m3_to_f32(uint8_t code);
/* scale = absmax(row)/448 in fp32; 1.0 for an all-zero row. */
float kvo_fp8_row_scale(const uint16_t* latent_bf16, int64_t latent_dim, const uint16_t* rope_bf16,
                        int64_t rope_dim);

/* Latent RMSNorm and key RoPE of the two stages in front of the cache write
 * (reference src/pipeline/pipeline.cpp:213-225; operator contracts include/moe/core/op_table.hpp:151-170
 * "y = x * gamma / sqrt(mean(x*x) + epsilon)" and :315-337 "half rotation"; rope table row = position
 * (pipeline.cpp:403-406)). Evaluated in double, rounded once to bf16 (nearest even):
 *   latent_out[t][d] = bf16(x[t][d] * gamma[d] / sqrt(mean_d x[t][d]^2 + epsilon))
 *   rope_out[t][i]        = bf16(r[t][i] cos[p][i] - r[t][i+h] sin[p][i])          i < h = rope_dim / 2
 *   rope_out[t][i+h]      = bf16(r[t][i+h] cos[p][i+h] + r[t][i] sin[p][i+h])
 * kv_a rows hold [latent | rope] bf16 (reference static_arena_manager.cpp:488-490).
 * Parity with CANN's rounding is unpinned (no reference numerics); pinned by closed forms in
 * tests/test_oracle_norm_rope.py. */
void kvo_norm_rope_rows(const uint16_t* kv_a, int64_t kv_a_row_stride, const uint16_t* gamma, double epsilon,
                        const uint16_t* rope_cos, const uint16_t* rope_sin, int64_t rope_table_row_stride,
                        const int32_t* positions, int64_t num_tokens, int64_t latent_dim, int64_t rope_dim,
                        uint16_t* latent_out, int64_t latent_out_row_stride, uint16_t* rope_out,
                        int64_t rope_out_row_stride);

/* The rotation alone, for rows that share a position in groups of rows_per_position consecutive
 * rows (the query's rope slices: one row per head, reference q_rope view
 * static_arena_manager.cpp:481-485, rotated by the same aclnnApplyRotaryPosEmbV2 call as k_rope,
 * pipeline.cpp:219-225): row t uses table row positions[t / rows_per_position]. */
void kvo_rope_rows(const uint16_t* rows, int64_t row_stride, const uint16_t* rope_cos, const uint16_t* rope_sin,
                   int64_t rope_table_row_stride, const int32_t* positions, int64_t rows_per_position, int64_t num_rows,
                   int64_t rope_dim, uint16_t* out, int64_t out_row_stride);

/* Block-32 MX quantization of bf16 rows along the last axis: the stage `attn_quant` behind the
 * attention (reference src/pipeline/pipeline.cpp:251-258: aclnnDynamicMxQuant, axis -1, round mode
 * rint, dst E4M3, blocksize kRoutedScaleBlock = 32, scale algorithm OCP; contract
 * include/moe/core/op_table.hpp:205-233). The operator's kernel is closed (CANN); this restates the
 * published algorithm it names, OCP Microscaling Formats (MX) v1.0 section 6.3:
 *   shared_exp = floor(log2(max_i |v_i|)) - 8          (8 = emax of E4M3), clamped to [-127, 127]
 *   scale code = shared_exp + 127                        (E8M0; 0xff = NaN)
 *   code_i     = e4m3(v_i / 2^shared_exp)                (round to nearest even, saturating at +-448)
 * A block of zeros takes the smallest scale (code 0) and zero elements; a block holding an Inf or
 * NaN takes the NaN scale and NaN elements. A trailing block shorter than 32 is quantized over
 * the elements it has. Parity with CANN on the zero and non-finite blocks is unpinned. */
void kvo_mx_quant_rows(const uint16_t* x, int64_t x_row_stride, int64_t rows, int64_t cols, uint8_t* codes,
                       int64_t codes_row_stride, uint8_t* scales, int64_t scales_row_stride);

/* Quantize-on-append: one fp32 scale per token row over latent+rope, code = e4m3(x / scale). */
void kvo_append_rows_fp8(uint8_t* latent_plane, int64_t latent_block_stride, int64_t latent_row_stride,
                         uint8_t* rope_plane, int64_t rope_block_stride, int64_t rope_row_stride,
                         float* scale_plane, int64_t scale_block_stride /* in floats */, int64_t block_size,
                         const uint16_t* latent_src, int64_t latent_src_row_stride /* elements */,
                         const uint16_t* rope_src, int64_t rope_src_row_stride /* elements */, int64_t latent_dim,
                         int64_t rope_dim, const int32_t* slots, int64_t num_tokens);

/* Dequantizing gather: bf16(e4m3_to_f32(code) * scale). */
void kvo_gather_rows_fp8(const uint8_t* latent_plane, int64_t latent_block_stride, int64_t latent_row_stride,
                         const uint8_t* rope_plane, int64_t rope_block_stride, int64_t rope_row_stride,
                         const float* scale_plane, int64_t scale_block_stride, int64_t block_size,
                         const int32_t* table, int64_t table_stride, const int32_t* seq_lens, int64_t batch,
                         uint16_t* latent_dst, int64_t latent_dst_row_stride /* elements */, uint16_t* rope_dst,
                         int64_t rope_dst_row_stride /* elements */, int64_t latent_dim, int64_t rope_dim);

/* ---- absorbed-MLA decode attention --------------------------------------- */

/* Per sequence b and head h (contract of aclnnFusedInferAttentionScoreV5 as the reference
 * plans it, src/pipeline/pipeline.cpp:235-249; include/moe/core/op_table.hpp:375-454):
 *   s_i = scale * (q_lat[b,h] . c_i + q_rope[b,h] . r_i),  p = softmax_i(s),  o[b,h] = sum_i p_i c_i
 * with c_i the latent row (K and V alias it) and r_i the rope row of token i < seq_lens[b],
 * reached through the block table. Accumulation in double (accum_f32 == 0) or float.
 * q strides in elements. out is fp32 [batch, heads, latent_dim]; lse (optional) is
 * log(sum exp(s_i)) per (b,h). A sequence of length 0 yields zeros and lse = -inf. */
typedef struct kvo_cache_view_t {
  const void* latent;      /* layer base */
  int64_t latent_block_stride, latent_row_stride; /* bytes */
  const void* rope;
  int64_t rope_block_stride, rope_row_stride;     /* bytes */
  const float* scale;      /* fp8 only */
  int64_t scale_block_stride;                     /* floats */
  int64_t block_size;
  int64_t latent_dim, rope_dim;
  int32_t dtype;           /* KVO_DTYPE_* */
} kvo_cache_view_t;

void kvo_mla_decode(const uint16_t* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                    const uint16_t* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                    const kvo_cache_view_t* cache, const int32_t* table, int64_t table_stride,
                    const int32_t* seq_lens, int64_t batch, int64_t heads, double scale, float* out, float* lse,
                    int accum_f32);

/* The same attention over selected tokens only: the consumer of the Lightning Indexer's output
 * (reference include/moe/core/op_table.hpp:964-1006: INT32 indices [B, S1, N2, k] of the k best
 * tokens, k = kIndexTopK = 512, include/moe/core/config.hpp:49; the vendored kernel writes the
 * valid indices first and fills the rest with -1,
 * third_party/ops_transformer/attention/quant_lightning_indexer/op_kernel/arch35/
 * quant_lightning_indexer_service_vector.h:446-541). Sequence b attends to the cached rows at
 * positions sparse_indices[b][0 .. n-1], n = number of entries before the first that is negative
 * or >= seq_lens[b]; softmax and output as in kvo_mla_decode (double accumulation). The
 * reference's pipeline does not launch a sparse attention yet (src/pipeline/pipeline.cpp:576-578
 * says so); pinned by reduction to the dense routine: indices 0..n-1 give the dense result bit
 * for bit, and any selection equals the dense routine on a cache holding just those rows. */
void kvo_mla_decode_sparse(const uint16_t* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                           const uint16_t* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                           const kvo_cache_view_t* cache, const int32_t* table, int64_t table_stride,
                           const int32_t* seq_lens, const int32_t* sparse_indices, int64_t sparse_count,
                           int64_t sparse_stride, int64_t batch, int64_t heads, double scale, float* out, float* lse);

/* Lightning Indexer (aclnnQuantLightningIndexer; contract include/moe/core/op_table.hpp:964-1006,
 * kernel vendored under third_party/ops_transformer/attention/quant_lightning_indexer): for one
 * query token of one sequence, the score of cached token t over the g = `heads` index heads
 *   score[t] = key_scale[t] * sum_h (W[h] * query_scale[h]) * ReLU(q_h . k_t)
 * (README.md "计算公式"), evaluated in the order of the vendored arch35 kernel
 * (op_kernel/arch35/vf/quant_lightning_indexer_vector1.h:288-330): w[h] = W[h] * query_scale[h] in
 * fp32; two fp32 accumulators, even and odd heads, one multiply-add per head; their sum times the
 * key scale; rounded to bf16 with ties away from zero (CAST_ROUND) and mapped to an order-preserving
 * 16-bit key (:66-96). q_h . k_t is the exact dot product of the E4M3 values rounded once to
 * fp32 (the NPU's and the GPU's matrix units accumulate in fp32 in an order of their own, so a
 * key may differ by one bf16 step from this restatement; parity with CANN unpinned).
 * query: E4M3 [heads][dim]; weights bf16 [heads]; query_scale fp32 [heads]; key_plane E4M3
 * [block][slot][dim] with key_scale_plane fp32 [block][slot] (layout PA_BSND, N2 = 1). */
void kvo_indexer_scores(const uint8_t* query, const uint16_t* weights, const float* query_scale, int64_t heads,
                        int64_t dim, const uint8_t* key_plane, int64_t key_block_stride, int64_t key_row_stride,
                        const float* key_scale_plane, int64_t scale_block_stride, int64_t block_size,
                        const int32_t* row_table, int64_t seq_len, uint16_t* keys_out);

/* Top-k over the 16-bit keys as the vendored kernel selects (op_kernel/arch35/
 * quant_lightning_indexer_service_vector.h:446-541, vf/vf_topk.h:634-670): a sequence no longer
 * than sparse_count yields 0 .. seq_len-1; otherwise every token whose key is above the k-th
 * largest key, in index order, followed by the lowest-indexed tokens whose key equals it; the rest
 * of the sparse_count entries is -1. (The vendored kernel processes long sequences in trunks, which
 * keeps the same set and may order it differently.) */
void kvo_indexer_topk(const uint16_t* keys, int64_t seq_len, int64_t sparse_count, int32_t* indices_out);

/* ---- block pool: free list, block tables, recycling, compaction ---------- */
/* No reference counterpart (the reference is one sequence with identity paging and
 * never writes its block table, src/memory/static_arena_manager.cpp:298). Semantics:
 *   - the free list is a FIFO queue over physical block ids, initialised 0..P-1 and,
 *     when `shuffle` is set, permuted by Fisher-Yates driven by SplitMix64(seed):
 *     for i = P-1 .. 1: j = next() % (i+1); swap(list[i], list[j]);
 *   - a sequence takes blocks from the head in logical order; freeing a sequence
 *     returns its blocks to the tail in logical order;
 *   - unused table entries are 0 (the arena is zero-filled);
 *   - compaction moves every live block with id >= n_live into the free ids < n_live,
 *     pairing the highest live id with the lowest hole; afterwards the free list is
 *     n_live..P-1 ascending. */
uint64_t kvo_splitmix64(uint64_t* state);

typedef struct kvo_pool kvo_pool;
kvo_pool* kvo_pool_new(int64_t num_blocks, int64_t block_size, int64_t max_seqs, int64_t max_blocks_per_seq,
                       uint64_t seed, int shuffle);
void kvo_pool_delete(kvo_pool* pool);
int kvo_pool_add_sequence(kvo_pool* pool, int64_t seq, int64_t context_len);
int kvo_pool_append_token(kvo_pool* pool, int64_t seq, int32_t* slot);
int kvo_pool_free_sequence(kvo_pool* pool, int64_t seq);
/* moves = (src, dst) pairs, capacity 2 * num_blocks int32. */
int kvo_pool_compact(kvo_pool* pool, int32_t* moves, int64_t* num_moves);
const int32_t* kvo_pool_table(const kvo_pool* pool);
int64_t kvo_pool_seq_len(const kvo_pool* pool, int64_t seq);
int64_t kvo_pool_free_blocks(const kvo_pool* pool);
int64_t kvo_pool_live_blocks(const kvo_pool* pool);
/* free list snapshot, head first; returns its length. */
int64_t kvo_pool_free_list(const kvo_pool* pool, int32_t* out);

#ifdef __cplusplus
}
#endif
#endif /* KV_ORACLE_H_ */
