/*
 * kv_oracle.c -- CPU restatement of the paged MLA KV-cache path. TEST INFRASTRUCTURE ONLY;
 * see kv_oracle.h for the rules on who may call it and for what pins each function.
 */
#include "kv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* layout arithmetic                                                          */
/* ------------------------------------------------------------------------- */

/* src/memory/expert_layout.cpp:27 -- power-of-two alignment only. */
size_t kvo_align_up(size_t value, size_t alignment) { return (value + alignment - 1) & ~(alignment - 1); }

/* src/memory/static_arena_manager.cpp:183 */
int64_t kvo_divide_up(int64_t value, int64_t divisor) { return (value + divisor - 1) / divisor; }

/* src/memory/static_arena_manager.cpp:192-201: block_size > 0 and max_ctx >= block_size or refuse. */
int64_t kvo_num_blocks(int64_t max_context_len, int64_t block_size) {
  if (block_size <= 0) return -1;
  if (max_context_len < block_size) return -1;
  return kvo_divide_up(max_context_len, block_size);
}

/* Model constants, include/moe/core/config.hpp:38-51. */
enum {
  kNumLayers = 43,
  kHiddenSize = 4096,
  kMoeIntermediateSize = 2048,
  kNumRoutedExperts = 256,
  kNumSharedExperts = 1,
  kVocabSize = 129280,
  kNumAttentionHeads = 64,
  kQLoraRank = 1024,
  kDenseScaleBlock = 128 /* block-128 weight scales along K */
};

static uint64_t fp8_bytes(int64_t n) { return (uint64_t)n; }
static uint64_t bf16_bytes(int64_t n) { return (uint64_t)n * 2u; }
static uint64_t fp32_bytes(int64_t n) { return (uint64_t)n * 4u; }
static uint64_t int32_bytes(int64_t n) { return (uint64_t)n * 4u; }
static int64_t dense_scale_cols(int64_t k) { return kvo_divide_up(k, kDenseScaleBlock); }

/* src/memory/static_arena_manager.cpp:205-241, term by term. */
uint64_t kvo_backbone_device_bytes(int64_t kv_lora_rank, int64_t qk_rope_head_dim, int64_t block_size,
                                   int64_t max_context_len) {
  const int64_t kv_row = kv_lora_rank + qk_rope_head_dim; /* config.hpp:92-95 */
  const int64_t q_b_width = kNumAttentionHeads * kv_row;
  const int64_t o_input = kNumAttentionHeads * kv_lora_rank;
  const int64_t shared_inter = (int64_t)kMoeIntermediateSize * kNumSharedExperts;
  uint64_t per_layer = 0;
  per_layer += bf16_bytes(kHiddenSize);
  per_layer += fp8_bytes((int64_t)kQLoraRank * kHiddenSize);
  per_layer += fp8_bytes(kQLoraRank * dense_scale_cols(kHiddenSize));
  per_layer += bf16_bytes(kQLoraRank);
  per_layer += fp8_bytes(q_b_width * kQLoraRank);
  per_layer += fp8_bytes(q_b_width * dense_scale_cols(kQLoraRank));
  per_layer += fp8_bytes(kv_row * kHiddenSize);
  per_layer += fp8_bytes(kv_row * dense_scale_cols(kHiddenSize));
  per_layer += bf16_bytes(kv_lora_rank);
  per_layer += fp8_bytes(kHiddenSize * o_input);
  per_layer += fp8_bytes(kHiddenSize * dense_scale_cols(o_input));
  per_layer += bf16_bytes(kHiddenSize);
  per_layer += bf16_bytes((int64_t)kNumRoutedExperts * kHiddenSize);
  per_layer += fp32_bytes(kNumRoutedExperts);
  per_layer += fp8_bytes(2 * shared_inter * kHiddenSize);
  per_layer += fp8_bytes(2 * shared_inter * dense_scale_cols(kHiddenSize));
  per_layer += fp8_bytes(kHiddenSize * shared_inter);
  per_layer += fp8_bytes(kHiddenSize * dense_scale_cols(shared_inter));

  const int64_t blocks = kvo_divide_up(max_context_len, block_size);
  uint64_t total = per_layer * (uint64_t)kNumLayers;
  total += bf16_bytes((int64_t)kVocabSize * kHiddenSize) * 2u;
  total += bf16_bytes(kHiddenSize);
  total += bf16_bytes(max_context_len * qk_rope_head_dim) * 2u;
  total += bf16_bytes(blocks * block_size * kv_lora_rank) * (uint64_t)kNumLayers;
  total += bf16_bytes(blocks * block_size * qk_rope_head_dim) * (uint64_t)kNumLayers;
  return total;
}

/* src/memory/static_arena_manager.cpp:298-300 (table, slot mapping), :315-318 (planes). */
void kvo_kv_reservation_bytes(int64_t num_layers, int64_t tokens_per_step, int64_t num_blocks, int64_t block_size,
                              int64_t kv_lora_rank, int64_t qk_rope_head_dim, kvo_kv_reservation_bytes_t* out) {
  out->block_table = int32_bytes(tokens_per_step * num_blocks);
  out->slot_mapping = int32_bytes(tokens_per_step);
  out->latent_cache = bf16_bytes(num_layers * num_blocks * block_size * kv_lora_rank);
  out->rope_cache = bf16_bytes(num_layers * num_blocks * block_size * qk_rope_head_dim);
}

/* src/pipeline/pipeline.cpp:134-136 (blocks x layers at Build), :532-534 (per step). */
void kvo_kv_stats(int64_t num_layers, int64_t num_blocks, int64_t block_size, int64_t position, kvo_kv_stats_t* out) {
  out->total_blocks_allocated = (uint64_t)(num_blocks * num_layers);
  out->active_context_tokens = (uint64_t)(position + 1);
  out->block_size = (uint64_t)block_size;
  out->kv_cache_utilization = (double)(position + 1) / (double)(num_blocks * block_size);
}

/* ------------------------------------------------------------------------- */
/* static arena                                                               */
/* ------------------------------------------------------------------------- */

#define KVO_ARENA_ALIGN 512u /* include/moe/core/config.hpp:237 */

typedef struct kvo_reservation {
  const char* name;
  size_t offset;
  size_t bytes;
  size_t align;
} kvo_reservation;

struct kvo_arena {
  kvo_reservation* items;
  size_t count, capacity;
  size_t cursor;
  int committed;
  uintptr_t base;
  size_t arena_bytes;
  int allocations;
  uint64_t workspace_high_water, workspace_bytes;
  int workspace_committed;
  int sealed;
};

kvo_arena* kvo_arena_new(void) { return (kvo_arena*)calloc(1, sizeof(kvo_arena)); }

void kvo_arena_delete(kvo_arena* arena) {
  if (arena == NULL) return;
  free(arena->items);
  free(arena);
}

/* static_arena.cpp:88-102. Refusals (sealed, committed, empty, non-power-of-two) in the
 * reference's order. */
int kvo_arena_reserve(kvo_arena* arena, const char* name, size_t bytes, size_t align, size_t* handle) {
  if (arena->sealed) return KVO_REFUSED;
  if (arena->committed) return KVO_REFUSED;
  if (bytes == 0) return KVO_REFUSED;
  if (align == 0 || (align & (align - 1)) != 0) return KVO_REFUSED;
  if (arena->count == arena->capacity) {
    size_t capacity = arena->capacity ? arena->capacity * 2 : 16;
    kvo_reservation* grown = (kvo_reservation*)realloc(arena->items, capacity * sizeof(kvo_reservation));
    if (grown == NULL) return KVO_REFUSED;
    arena->items = grown;
    arena->capacity = capacity;
  }
  kvo_reservation* r = &arena->items[arena->count];
  r->name = name;
  r->bytes = bytes;
  r->align = align;
  r->offset = kvo_align_up(arena->cursor, align);
  arena->cursor = r->offset + bytes;
  if (handle) *handle = arena->count;
  arena->count++;
  return KVO_OK;
}

/* static_arena.cpp:310-332 */
int kvo_arena_validate(const kvo_arena* arena) {
  size_t previous_end = 0;
  for (size_t i = 0; i < arena->count; ++i) {
    const kvo_reservation* r = &arena->items[i];
    if (r->offset % r->align != 0) return KVO_REFUSED;
    if (r->offset < previous_end) return KVO_REFUSED;
    if (r->offset + r->bytes > arena->arena_bytes) return KVO_REFUSED;
    previous_end = r->offset + r->bytes;
  }
  if (arena->base % KVO_ARENA_ALIGN != 0) return KVO_REFUSED;
  return KVO_OK;
}

/* static_arena.cpp:108-118: one allocation of AlignUp(cursor, 512), then validation. */
int kvo_arena_commit(kvo_arena* arena, uintptr_t base) {
  if (arena->sealed) return KVO_REFUSED;
  if (arena->committed) return KVO_REFUSED;
  if (arena->count == 0) return KVO_REFUSED;
  arena->arena_bytes = kvo_align_up(arena->cursor, KVO_ARENA_ALIGN);
  arena->base = base;
  arena->committed = 1;
  arena->allocations += 1;
  return kvo_arena_validate(arena);
}

/* static_arena.cpp:120-124 */
int kvo_arena_address(const kvo_arena* arena, size_t handle, uintptr_t* address) {
  if (!arena->committed) return KVO_REFUSED;
  if (handle >= arena->count) return KVO_REFUSED;
  *address = arena->base + arena->items[handle].offset;
  return KVO_OK;
}

/* static_arena.cpp:126-129 */
int kvo_arena_bytes(const kvo_arena* arena, size_t handle, size_t* bytes) {
  if (handle >= arena->count) return KVO_REFUSED;
  *bytes = arena->items[handle].bytes;
  return KVO_OK;
}

int kvo_arena_offset(const kvo_arena* arena, size_t handle, size_t* offset) {
  if (handle >= arena->count) return KVO_REFUSED;
  *offset = arena->items[handle].offset;
  return KVO_OK;
}

/* static_arena.cpp:270-273 */
int kvo_arena_note_workspace(kvo_arena* arena, uint64_t bytes) {
  if (arena->sealed) return KVO_REFUSED;
  if (bytes > arena->workspace_high_water) arena->workspace_high_water = bytes;
  return KVO_OK;
}

/* static_arena.cpp:275-288: second and last allocation; none when every plan asked for zero. */
int kvo_arena_commit_workspace(kvo_arena* arena) {
  if (arena->sealed) return KVO_REFUSED;
  if (arena->workspace_committed) return KVO_REFUSED;
  arena->workspace_bytes = arena->workspace_high_water;
  if (arena->workspace_bytes == 0) return KVO_OK;
  arena->workspace_committed = 1;
  arena->allocations += 1;
  return KVO_OK;
}

/* static_arena.cpp:290-295 */
int kvo_arena_workspace_fits(const kvo_arena* arena, uint64_t bytes) {
  return bytes <= arena->workspace_bytes ? KVO_OK : KVO_REFUSED;
}

uint64_t kvo_arena_workspace_bytes(const kvo_arena* arena) { return arena->workspace_bytes; }

/* static_arena.cpp:301-304 */
int kvo_arena_seal(kvo_arena* arena) {
  if (!arena->committed) return KVO_REFUSED;
  arena->sealed = 1;
  return KVO_OK;
}

int kvo_arena_sealed(const kvo_arena* arena) { return arena->sealed; }
size_t kvo_arena_total_bytes(const kvo_arena* arena) { return arena->arena_bytes; }
size_t kvo_arena_reserved_bytes(const kvo_arena* arena) { return arena->cursor; }
size_t kvo_arena_count(const kvo_arena* arena) { return arena->count; }
int kvo_arena_allocations(const kvo_arena* arena) { return arena->allocations; }

/* ------------------------------------------------------------------------- */
/* paged addressing, append, gather, block copy                               */
/* ------------------------------------------------------------------------- */

int64_t kvo_slot(const int32_t* table_row, int64_t position, int64_t block_size) {
  const int64_t logical_block = position / block_size;
  const int64_t in_block = position % block_size;
  return (int64_t)table_row[logical_block] * block_size + in_block;
}

void kvo_append_rows(uint8_t* plane, int64_t block_stride, int64_t row_stride, int64_t block_size,
                     const uint8_t* src, int64_t src_row_stride, int64_t row_bytes, const int32_t* slots,
                     int64_t num_tokens) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t slot = slots[t];
    if (slot < 0) continue;
    uint8_t* row = plane + (slot / block_size) * block_stride + (slot % block_size) * row_stride;
    memcpy(row, src + t * src_row_stride, (size_t)row_bytes);
  }
}

void kvo_gather_rows(const uint8_t* plane, int64_t block_stride, int64_t row_stride, int64_t block_size,
                     const int32_t* table, int64_t table_stride, const int32_t* seq_lens, int64_t batch,
                     uint8_t* dst, int64_t dst_row_stride, int64_t row_bytes) {
  int64_t out_row = 0;
  for (int64_t b = 0; b < batch; ++b) {
    const int32_t* row_table = table + b * table_stride;
    for (int64_t i = 0; i < seq_lens[b]; ++i, ++out_row) {
      const int64_t slot = kvo_slot(row_table, i, block_size);
      const uint8_t* row = plane + (slot / block_size) * block_stride + (slot % block_size) * row_stride;
      memcpy(dst + out_row * dst_row_stride, row, (size_t)row_bytes);
    }
  }
}

void kvo_copy_blocks(uint8_t* plane, int64_t block_stride, int64_t block_bytes, const int32_t* moves,
                     int64_t num_moves) {
  for (int64_t m = 0; m < num_moves; ++m) {
    const int64_t src = moves[2 * m], dst = moves[2 * m + 1];
    memcpy(plane + dst * block_stride, plane + src * block_stride, (size_t)block_bytes);
  }
}

/* ------------------------------------------------------------------------- */
/* number formats                                                             */
/* ------------------------------------------------------------------------- */

static uint32_t f32_bits(float value) {
  uint32_t bits;
  memcpy(&bits, &value, 4);
  return bits;
}

static float bits_f32(uint32_t bits) {
  float value;
  memcpy(&value, &bits, 4);
  return value;
}

uint16_t kvo_bf16_from_f32(float value) {
  uint32_t bits = f32_bits(value);
  if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x0040u); /* quiet NaN */
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

float kvo_bf16_to_f32(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

float kvo_e4m3_to_f32(uint8_t code) {
  const int sign = code >> 7, exponent = (code >> 3) & 15, mantissa = code & 7;
  float magnitude;
  if (exponent == 15 && mantissa == 7) return bits_f32(0x7fc00000u | ((uint32_t)sign << 31));
  if (exponent == 0) magnitude = ldexpf((float)mantissa, -9);               /* subnormal: m/8 * 2^-6 */
  else magnitude = ldexpf(1.0f + (float)mantissa / 8.0f, exponent - 7);
  return sign ? -magnitude : magnitude;
}

/* Round to nearest even onto the E4M3FN grid, saturating to 448. Works on the fp32 bit
 * pattern: values below 2^-6 land on the subnormal grid of spacing 2^-9. */
uint8_t kvo_e4m3_from_f32(float value) {
  const uint32_t bits = f32_bits(value);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
  const uint32_t magnitude_bits = bits & 0x7fffffffu;
  if (magnitude_bits > 0x7f800000u) return (uint8_t)(sign | 0x7fu); /* NaN */
  const float magnitude = bits_f32(magnitude_bits);
  if (magnitude >= 448.0f) return (uint8_t)(sign | 0x7eu);          /* saturate (also +-inf) */
  if (magnitude < 0.015625f) {                                       /* below 2^-6: subnormal grid */
    /* magnitude * 512 is exact in fp32; rint rounds half to even (default rounding mode). */
    const float scaled = magnitude * 512.0f;
    const int q = (int)rintf(scaled);                                /* 0..8; 8 == smallest normal */
    return (uint8_t)(sign | (uint8_t)q);
  }
  /* normal: keep 3 mantissa bits of the fp32 mantissa with RNE */
  uint32_t rounded = magnitude_bits + 0x7ffffu + ((magnitude_bits >> 20) & 1u);
  const int exponent = (int)(rounded >> 23) - 127 + 7;               /* e4m3 biased exponent */
  const uint32_t mantissa = (rounded >> 20) & 7u;
  if (exponent > 15 || (exponent == 15 && mantissa == 7)) return (uint8_t)(sign | 0x7eu);
  return (uint8_t)(sign | (uint8_t)(exponent << 3) | (uint8_t)mantissa);
}

float kvo_fp8_row_scale(const uint16_t* latent_bf16, int64_t latent_dim, const uint16_t* rope_bf16,
                        int64_t rope_dim) {
  float absmax = 0.0f;
  for (int64_t i = 0; i < latent_dim; ++i) {
    const float v = fabsf(kvo_bf16_to_f32(latent_bf16[i]));
    if (v > absmax) absmax = v;
  }
  for (int64_t i = 0; i < rope_dim; ++i) {
    const float v = fabsf(kvo_bf16_to_f32(rope_bf16[i]));
    if (v > absmax) absmax = v;
  }
  if (absmax == 0.0f) return 1.0f;
  return absmax / 448.0f;
}

void kvo_append_rows_fp8(uint8_t* latent_plane, int64_t latent_block_stride, int64_t latent_row_stride,
                         uint8_t* rope_plane, int64_t rope_block_stride, int64_t rope_row_stride,
                         float* scale_plane, int64_t scale_block_stride, int64_t block_size,
                         const uint16_t* latent_src, int64_t latent_src_row_stride, const uint16_t* rope_src,
                         int64_t rope_src_row_stride, int64_t latent_dim, int64_t rope_dim, const int32_t* slots,
                         int64_t num_tokens) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t slot = slots[t];
    if (slot < 0) continue;
    const int64_t block = slot / block_size, in_block = slot % block_size;
    const uint16_t* latent = latent_src + t * latent_src_row_stride;
    const uint16_t* rope = rope_src + t * rope_src_row_stride;
    const float scale = kvo_fp8_row_scale(latent, latent_dim, rope, rope_dim);
    uint8_t* latent_row = latent_plane + block * latent_block_stride + in_block * latent_row_stride;
    uint8_t* rope_row = rope_plane + block * rope_block_stride + in_block * rope_row_stride;
    for (int64_t i = 0; i < latent_dim; ++i) latent_row[i] = kvo_e4m3_from_f32(kvo_bf16_to_f32(latent[i]) / scale);
    for (int64_t i = 0; i < rope_dim; ++i) rope_row[i] = kvo_e4m3_from_f32(kvo_bf16_to_f32(rope[i]) / scale);
    scale_plane[block * scale_block_stride + in_block] = scale;
  }
}

void kvo_gather_rows_fp8(const uint8_t* latent_plane, int64_t latent_block_stride, int64_t latent_row_stride,
                         const uint8_t* rope_plane, int64_t rope_block_stride, int64_t rope_row_stride,
                         const float* scale_plane, int64_t scale_block_stride, int64_t block_size,
                         const int32_t* table, int64_t table_stride, const int32_t* seq_lens, int64_t batch,
                         uint16_t* latent_dst, int64_t latent_dst_row_stride, uint16_t* rope_dst,
                         int64_t rope_dst_row_stride, int64_t latent_dim, int64_t rope_dim) {
  int64_t out_row = 0;
  for (int64_t b = 0; b < batch; ++b) {
    const int32_t* row_table = table + b * table_stride;
    for (int64_t i = 0; i < seq_lens[b]; ++i, ++out_row) {
      const int64_t slot = kvo_slot(row_table, i, block_size);
      const int64_t block = slot / block_size, in_block = slot % block_size;
      const float scale = scale_plane[block * scale_block_stride + in_block];
      const uint8_t* latent_row = latent_plane + block * latent_block_stride + in_block * latent_row_stride;
      const uint8_t* rope_row = rope_plane + block * rope_block_stride + in_block * rope_row_stride;
      uint16_t* latent_out = latent_dst + out_row * latent_dst_row_stride;
      uint16_t* rope_out = rope_dst + out_row * rope_dst_row_stride;
      for (int64_t d = 0; d < latent_dim; ++d) latent_out[d] = kvo_bf16_from_f32(kvo_e4m3_to_f32(latent_row[d]) * scale);
      for (int64_t d = 0; d < rope_dim; ++d) rope_out[d] = kvo_bf16_from_f32(kvo_e4m3_to_f32(rope_row[d]) * scale);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* latent RMSNorm + key RoPE (the stages in front of the cache write)          */
/* ------------------------------------------------------------------------- */

/* One rounding, nearest even, straight from double: going through float first would round twice
 * when the double lies just off a bf16 midpoint (which a float represents exactly). */
static uint16_t bf16_from_double(double v) {
  float f = (float)v;
  uint32_t bits;
  memcpy(&bits, &f, sizeof bits);
  if ((bits & 0xffffu) == 0x8000u && (double)f != v) {
    bits += fabs(v) > fabs((double)f) ? 1u : 0xffffffffu;  /* off the midpoint, on the side v is on */
    memcpy(&f, &bits, sizeof f);
  }
  return kvo_bf16_from_f32(f);
}

void kvo_rope_rows(const uint16_t* rows, int64_t row_stride, const uint16_t* rope_cos, const uint16_t* rope_sin,
                   int64_t rope_table_row_stride, const int32_t* positions, int64_t rows_per_position, int64_t num_rows,
                   int64_t rope_dim, uint16_t* out, int64_t out_row_stride) {
  const int64_t half = rope_dim / 2;
  for (int64_t t = 0; t < num_rows; ++t) {
    const uint16_t* r = rows + t * row_stride;
    const int64_t position = positions[t / rows_per_position];
    const uint16_t* c = rope_cos + position * rope_table_row_stride;
    const uint16_t* s = rope_sin + position * rope_table_row_stride;
    for (int64_t i = 0; i < half; ++i) {
      const double lo = (double)kvo_bf16_to_f32(r[i]), hi = (double)kvo_bf16_to_f32(r[i + half]);
      out[t * out_row_stride + i] = bf16_from_double(lo * (double)kvo_bf16_to_f32(c[i]) - hi * (double)kvo_bf16_to_f32(s[i]));
      out[t * out_row_stride + i + half] =
          bf16_from_double(hi * (double)kvo_bf16_to_f32(c[i + half]) + lo * (double)kvo_bf16_to_f32(s[i + half]));
    }
  }
}

void kvo_norm_rope_rows(const uint16_t* kv_a, int64_t kv_a_row_stride, const uint16_t* gamma, double epsilon,
                        const uint16_t* rope_cos, const uint16_t* rope_sin, int64_t rope_table_row_stride,
                        const int32_t* positions, int64_t num_tokens, int64_t latent_dim, int64_t rope_dim,
                        uint16_t* latent_out, int64_t latent_out_row_stride, uint16_t* rope_out,
                        int64_t rope_out_row_stride) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const uint16_t* x = kv_a + t * kv_a_row_stride;
    double sum_squares = 0.0;
    for (int64_t d = 0; d < latent_dim; ++d) {
      const double v = (double)kvo_bf16_to_f32(x[d]);
      sum_squares += v * v;
    }
    const double rstd = 1.0 / sqrt(sum_squares / (double)latent_dim + epsilon);
    for (int64_t d = 0; d < latent_dim; ++d) {
      latent_out[t * latent_out_row_stride + d] =
          bf16_from_double((double)kvo_bf16_to_f32(x[d]) * rstd * (double)kvo_bf16_to_f32(gamma[d]));
    }
  }
  kvo_rope_rows(kv_a + latent_dim, kv_a_row_stride, rope_cos, rope_sin, rope_table_row_stride, positions, 1, num_tokens,
                rope_dim, rope_out, rope_out_row_stride);
}

/* ------------------------------------------------------------------------- */
/* OCP microscaling (MX) quantization of the attention output                 */
/* ------------------------------------------------------------------------- */

void kvo_mx_quant_rows(const uint16_t* x, int64_t x_row_stride, int64_t rows, int64_t cols, uint8_t* codes,
                       int64_t codes_row_stride, uint8_t* scales, int64_t scales_row_stride) {
  const int64_t block = 32;
  const int element_emax = 8; /* E4M3: largest power of two is 2^8 (448 = 1.75 * 2^8) */
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t b0 = 0; b0 < cols; b0 += block) {
      const int64_t n = cols - b0 < block ? cols - b0 : block;
      const uint16_t* v = x + r * x_row_stride + b0;
      float absmax = 0.0f;
      int special = 0;
      for (int64_t i = 0; i < n; ++i) {
        const float f = kvo_bf16_to_f32(v[i]);
        if (isnan(f) || isinf(f)) special = 1;
        else if (fabsf(f) > absmax) absmax = fabsf(f);
      }
      uint8_t* out = codes + r * codes_row_stride + b0;
      uint8_t* scale_code = scales + r * scales_row_stride + b0 / block;
      if (special) { /* the shared scale is NaN and so is every element */
        *scale_code = 0xffu;
        for (int64_t i = 0; i < n; ++i) out[i] = (uint8_t)((v[i] >> 8 & 0x80u) | 0x7fu);
        continue;
      }
      int shared_exp = -127;
      if (absmax > 0.0f) {
        int e;
        (void)frexpf(absmax, &e); /* absmax = m * 2^e, m in [0.5, 1): floor(log2 absmax) = e - 1 */
        shared_exp = e - 1 - element_emax;
        if (shared_exp < -127) shared_exp = -127;
        if (shared_exp > 127) shared_exp = 127;
      }
      *scale_code = (uint8_t)(shared_exp + 127);
      for (int64_t i = 0; i < n; ++i) {
        /* v * 2^-shared_exp in double is exact; the float cast is exact too unless the value is
         * far below the element grid, where it rounds to zero either way. */
        const double scaled = ldexp((double)kvo_bf16_to_f32(v[i]), -shared_exp);
        out[i] = kvo_e4m3_from_f32((float)scaled);
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* absorbed-MLA decode attention                                              */
/* ------------------------------------------------------------------------- */

static void load_row_f32(const kvo_cache_view_t* cache, int64_t slot, float* latent, float* rope) {
  const int64_t block = slot / cache->block_size, in_block = slot % cache->block_size;
  const uint8_t* latent_row = (const uint8_t*)cache->latent + block * cache->latent_block_stride +
                              in_block * cache->latent_row_stride;
  const uint8_t* rope_row = (const uint8_t*)cache->rope + block * cache->rope_block_stride +
                            in_block * cache->rope_row_stride;
  if (cache->dtype == KVO_DTYPE_BF16) {
    const uint16_t* l = (const uint16_t*)latent_row;
    const uint16_t* r = (const uint16_t*)rope_row;
    for (int64_t d = 0; d < cache->latent_dim; ++d) latent[d] = kvo_bf16_to_f32(l[d]);
    for (int64_t d = 0; d < cache->rope_dim; ++d) rope[d] = kvo_bf16_to_f32(r[d]);
  } else {
    const float scale = cache->scale[block * cache->scale_block_stride + in_block];
    for (int64_t d = 0; d < cache->latent_dim; ++d) latent[d] = kvo_e4m3_to_f32(latent_row[d]) * scale;
    for (int64_t d = 0; d < cache->rope_dim; ++d) rope[d] = kvo_e4m3_to_f32(rope_row[d]) * scale;
  }
}

/* Dense (sparse_indices == NULL: positions 0 .. seq_lens[b]-1) or selected-token attention
 * (positions sparse_indices[b][0 .. n-1], n = the number of entries before the first one that is
 * negative or not below seq_lens[b], at most sparse_count). */
static void mla_decode_rows(const uint16_t* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                            const uint16_t* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                            const kvo_cache_view_t* cache, const int32_t* table, int64_t table_stride,
                            const int32_t* seq_lens, const int32_t* sparse_indices, int64_t sparse_count,
                            int64_t sparse_stride, int64_t batch, int64_t heads, double scale, float* out, float* lse,
                            int accum_f32) {
  const int64_t dl = cache->latent_dim, dr = cache->rope_dim;
  for (int64_t b = 0; b < batch; ++b) {
    int64_t n = seq_lens[b];
    const int32_t* selected = sparse_indices ? sparse_indices + b * sparse_stride : NULL;
    if (selected) {
      int64_t count = 0;
      while (count < sparse_count && selected[count] >= 0 && selected[count] < seq_lens[b]) ++count;
      n = count;
    }
    float* out_b = out + b * heads * dl;
    if (n <= 0) {
      memset(out_b, 0, (size_t)(heads * dl) * sizeof(float));
      if (lse) for (int64_t h = 0; h < heads; ++h) lse[b * heads + h] = -INFINITY;
      continue;
    }
    /* decode this sequence's rows once */
    float* latent = (float*)malloc((size_t)(n * dl) * sizeof(float));
    float* rope = (float*)malloc((size_t)(n * dr) * sizeof(float));
    double* scores = (double*)malloc((size_t)n * sizeof(double));
    const int32_t* row_table = table + b * table_stride;
    for (int64_t i = 0; i < n; ++i) {
      const int64_t position = selected ? selected[i] : i;
      load_row_f32(cache, kvo_slot(row_table, position, cache->block_size), latent + i * dl, rope + i * dr);
    }
    for (int64_t h = 0; h < heads; ++h) {
      const uint16_t* ql = q_latent + b * q_latent_seq_stride + h * q_latent_head_stride;
      const uint16_t* qr = q_rope + b * q_rope_seq_stride + h * q_rope_head_stride;
      double max_score = -INFINITY;
      for (int64_t i = 0; i < n; ++i) {
        double s;
        if (accum_f32) {
          float acc = 0.0f;
          for (int64_t d = 0; d < dl; ++d) acc += kvo_bf16_to_f32(ql[d]) * latent[i * dl + d];
          for (int64_t d = 0; d < dr; ++d) acc += kvo_bf16_to_f32(qr[d]) * rope[i * dr + d];
          s = (double)(acc * (float)scale);
        } else {
          double acc = 0.0;
          for (int64_t d = 0; d < dl; ++d) acc += (double)kvo_bf16_to_f32(ql[d]) * (double)latent[i * dl + d];
          for (int64_t d = 0; d < dr; ++d) acc += (double)kvo_bf16_to_f32(qr[d]) * (double)rope[i * dr + d];
          s = acc * scale;
        }
        scores[i] = s;
        if (s > max_score) max_score = s;
      }
      double denom = 0.0;
      for (int64_t i = 0; i < n; ++i) {
        scores[i] = accum_f32 ? (double)expf((float)(scores[i] - max_score)) : exp(scores[i] - max_score);
        denom += scores[i];
      }
      float* o = out_b + h * dl;
      if (accum_f32) {
        for (int64_t d = 0; d < dl; ++d) {
          float acc = 0.0f;
          for (int64_t i = 0; i < n; ++i) acc += (float)scores[i] * latent[i * dl + d];
          o[d] = acc / (float)denom;
        }
      } else {
        for (int64_t d = 0; d < dl; ++d) {
          double acc = 0.0;
          for (int64_t i = 0; i < n; ++i) acc += scores[i] * (double)latent[i * dl + d];
          o[d] = (float)(acc / denom);
        }
      }
      if (lse) lse[b * heads + h] = (float)(max_score + log(denom));
    }
    free(latent);
    free(rope);
    free(scores);
  }
}

void kvo_mla_decode(const uint16_t* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                    const uint16_t* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                    const kvo_cache_view_t* cache, const int32_t* table, int64_t table_stride,
                    const int32_t* seq_lens, int64_t batch, int64_t heads, double scale, float* out, float* lse,
                    int accum_f32) {
  mla_decode_rows(q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope, q_rope_seq_stride, q_rope_head_stride, cache,
                  table, table_stride, seq_lens, NULL, 0, 0, batch, heads, scale, out, lse, accum_f32);
}

void kvo_mla_decode_sparse(const uint16_t* q_latent, int64_t q_latent_seq_stride, int64_t q_latent_head_stride,
                           const uint16_t* q_rope, int64_t q_rope_seq_stride, int64_t q_rope_head_stride,
                           const kvo_cache_view_t* cache, const int32_t* table, int64_t table_stride,
                           const int32_t* seq_lens, const int32_t* sparse_indices, int64_t sparse_count,
                           int64_t sparse_stride, int64_t batch, int64_t heads, double scale, float* out, float* lse) {
  mla_decode_rows(q_latent, q_latent_seq_stride, q_latent_head_stride, q_rope, q_rope_seq_stride, q_rope_head_stride, cache,
                  table, table_stride, seq_lens, sparse_indices, sparse_count, sparse_stride, batch, heads, scale, out, lse, 0);
}

/* ------------------------------------------------------------------------- */
/* Lightning Indexer: scores and top-k selection                               */
/* ------------------------------------------------------------------------- */

/* fp32 -> bf16 rounding to nearest with ties away from zero, then the order-preserving 16-bit key:
 * a NaN gets the lowest key, a negative value has all bits inverted, any other value its sign bit
 * set. */
static uint16_t indexer_key(float score) {
  uint32_t bits = f32_bits(score);
  uint16_t b;
  if ((bits & 0x7fffffffu) > 0x7f800000u) {
    b = 0x7fc0u;
  } else {
    b = (uint16_t)((bits + 0x8000u) >> 16); /* magnitude + half, truncated: ties go away from zero */
  }
  if (b == 0x7fc0u) return 0x0000u;
  return (b & 0x8000u) ? (uint16_t)~b : (uint16_t)(b | 0x8000u);
}

void kvo_indexer_scores(const uint8_t* query, const uint16_t* weights, const float* query_scale, int64_t heads,
                        int64_t dim, const uint8_t* key_plane, int64_t key_block_stride, int64_t key_row_stride,
                        const float* key_scale_plane, int64_t scale_block_stride, int64_t block_size,
                        const int32_t* row_table, int64_t seq_len, uint16_t* keys_out) {
  float* w = (float*)malloc((size_t)heads * sizeof(float));
  for (int64_t h = 0; h < heads; ++h) w[h] = kvo_bf16_to_f32(weights[h]) * query_scale[h];
  for (int64_t t = 0; t < seq_len; ++t) {
    const int64_t slot = kvo_slot(row_table, t, block_size);
    const int64_t block = slot / block_size, in_block = slot % block_size;
    const uint8_t* k = key_plane + block * key_block_stride + in_block * key_row_stride;
    float sum[2] = {0.0f, 0.0f}; /* even and odd heads, one fused multiply-add per head each */
    for (int64_t h = 0; h < heads; ++h) {
      /* every product of two E4M3 values is exact in double, and so is the sum of 128 of them */
      double dot = 0.0;
      for (int64_t d = 0; d < dim; ++d) dot += (double)kvo_e4m3_to_f32(query[h * dim + d]) * (double)kvo_e4m3_to_f32(k[d]);
      float qk = (float)dot;
      if (!(qk > 0.0f)) qk = 0.0f;
      sum[h & 1] = fmaf(qk, w[h], sum[h & 1]);
    }
    const float score = (sum[0] + sum[1]) * key_scale_plane[block * scale_block_stride + in_block];
    keys_out[t] = indexer_key(score);
  }
  free(w);
}

void kvo_indexer_topk(const uint16_t* keys, int64_t seq_len, int64_t sparse_count, int32_t* indices_out) {
  int64_t written = 0;
  if (seq_len <= sparse_count) {
    for (int64_t t = 0; t < seq_len; ++t) indices_out[written++] = (int32_t)t;
  } else {
    /* the k-th largest key by counting, then everything above it in index order, then the lowest
     * indices among the keys equal to it */
    int64_t histogram[65536];
    memset(histogram, 0, sizeof histogram);
    for (int64_t t = 0; t < seq_len; ++t) ++histogram[keys[t]];
    int64_t above = 0;
    int32_t threshold = 65535;
    while (above + histogram[threshold] < sparse_count) above += histogram[threshold--];
    for (int64_t t = 0; t < seq_len; ++t) {
      if (keys[t] > threshold) indices_out[written++] = (int32_t)t;
    }
    for (int64_t t = 0; t < seq_len && written < sparse_count; ++t) {
      if (keys[t] == threshold) indices_out[written++] = (int32_t)t;
    }
  }
  for (; written < sparse_count; ++written) indices_out[written] = -1;
}

/* ------------------------------------------------------------------------- */
/* block pool                                                                 */
/* ------------------------------------------------------------------------- */

/* SplitMix64 (Steele, Lea, Flood 2014; Vigna's public-domain splitmix64.c). */
uint64_t kvo_splitmix64(uint64_t* state) {
  uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct kvo_pool {
  int64_t num_blocks, block_size, max_seqs, max_blocks_per_seq;
  int32_t* ring;      /* FIFO of free ids, capacity num_blocks */
  int64_t head, count;
  int32_t* table;     /* [max_seqs][max_blocks_per_seq] */
  int64_t* seq_len;   /* -1 = slot unused */
  int64_t* seq_blocks;
};

kvo_pool* kvo_pool_new(int64_t num_blocks, int64_t block_size, int64_t max_seqs, int64_t max_blocks_per_seq,
                       uint64_t seed, int shuffle) {
  if (num_blocks <= 0 || block_size <= 0 || max_seqs <= 0 || max_blocks_per_seq <= 0) return NULL;
  kvo_pool* pool = (kvo_pool*)calloc(1, sizeof(kvo_pool));
  pool->num_blocks = num_blocks;
  pool->block_size = block_size;
  pool->max_seqs = max_seqs;
  pool->max_blocks_per_seq = max_blocks_per_seq;
  pool->ring = (int32_t*)malloc((size_t)num_blocks * sizeof(int32_t));
  pool->table = (int32_t*)calloc((size_t)(max_seqs * max_blocks_per_seq), sizeof(int32_t));
  pool->seq_len = (int64_t*)malloc((size_t)max_seqs * sizeof(int64_t));
  pool->seq_blocks = (int64_t*)calloc((size_t)max_seqs, sizeof(int64_t));
  for (int64_t i = 0; i < num_blocks; ++i) pool->ring[i] = (int32_t)i;
  for (int64_t s = 0; s < max_seqs; ++s) pool->seq_len[s] = -1;
  if (shuffle) {
    uint64_t state = seed;
    for (int64_t i = num_blocks - 1; i >= 1; --i) {
      const int64_t j = (int64_t)(kvo_splitmix64(&state) % (uint64_t)(i + 1));
      const int32_t tmp = pool->ring[i];
      pool->ring[i] = pool->ring[j];
      pool->ring[j] = tmp;
    }
  }
  pool->head = 0;
  pool->count = num_blocks;
  return pool;
}

void kvo_pool_delete(kvo_pool* pool) {
  if (pool == NULL) return;
  free(pool->ring);
  free(pool->table);
  free(pool->seq_len);
  free(pool->seq_blocks);
  free(pool);
}

static int32_t pool_pop(kvo_pool* pool) {
  const int32_t id = pool->ring[pool->head];
  pool->head = (pool->head + 1) % pool->num_blocks;
  pool->count--;
  return id;
}

static void pool_push(kvo_pool* pool, int32_t id) {
  pool->ring[(pool->head + pool->count) % pool->num_blocks] = id;
  pool->count++;
}

int kvo_pool_add_sequence(kvo_pool* pool, int64_t seq, int64_t context_len) {
  if (seq < 0 || seq >= pool->max_seqs || pool->seq_len[seq] >= 0 || context_len < 0) return KVO_REFUSED;
  const int64_t need = kvo_divide_up(context_len, pool->block_size);
  if (need > pool->max_blocks_per_seq || need > pool->count) return KVO_REFUSED;
  int32_t* row = pool->table + seq * pool->max_blocks_per_seq;
  for (int64_t i = 0; i < need; ++i) row[i] = pool_pop(pool);
  pool->seq_len[seq] = context_len;
  pool->seq_blocks[seq] = need;
  return KVO_OK;
}

int kvo_pool_append_token(kvo_pool* pool, int64_t seq, int32_t* slot) {
  if (seq < 0 || seq >= pool->max_seqs || pool->seq_len[seq] < 0) return KVO_REFUSED;
  const int64_t position = pool->seq_len[seq];
  int32_t* row = pool->table + seq * pool->max_blocks_per_seq;
  if (position % pool->block_size == 0) { /* first token of a new logical block */
    if (pool->seq_blocks[seq] >= pool->max_blocks_per_seq || pool->count == 0) return KVO_REFUSED;
    row[pool->seq_blocks[seq]++] = pool_pop(pool);
  }
  *slot = (int32_t)kvo_slot(row, position, pool->block_size);
  pool->seq_len[seq] = position + 1;
  return KVO_OK;
}

int kvo_pool_free_sequence(kvo_pool* pool, int64_t seq) {
  if (seq < 0 || seq >= pool->max_seqs || pool->seq_len[seq] < 0) return KVO_REFUSED;
  int32_t* row = pool->table + seq * pool->max_blocks_per_seq;
  for (int64_t i = 0; i < pool->seq_blocks[seq]; ++i) {
    pool_push(pool, row[i]);
    row[i] = 0;
  }
  pool->seq_len[seq] = -1;
  pool->seq_blocks[seq] = 0;
  return KVO_OK;
}

int kvo_pool_compact(kvo_pool* pool, int32_t* moves, int64_t* num_moves) {
  const int64_t live = pool->num_blocks - pool->count;
  /* owner[id] = seq * max_blocks + logical index, or -1 when free */
  int64_t* owner = (int64_t*)malloc((size_t)pool->num_blocks * sizeof(int64_t));
  for (int64_t i = 0; i < pool->num_blocks; ++i) owner[i] = -1;
  for (int64_t s = 0; s < pool->max_seqs; ++s) {
    if (pool->seq_len[s] < 0) continue;
    for (int64_t i = 0; i < pool->seq_blocks[s]; ++i) owner[pool->table[s * pool->max_blocks_per_seq + i]] = s * pool->max_blocks_per_seq + i;
  }
  int64_t n = 0;
  int64_t hole = 0;
  for (int64_t src = pool->num_blocks - 1; src >= live; --src) {
    if (owner[src] < 0) continue;
    while (owner[hole] >= 0) ++hole; /* a hole below `live` exists for every live block above it */
    moves[2 * n] = (int32_t)src;
    moves[2 * n + 1] = (int32_t)hole;
    ++n;
    pool->table[owner[src]] = (int32_t)hole;
    owner[hole] = owner[src];
    owner[src] = -1;
  }
  free(owner);
  pool->head = 0;
  pool->count = pool->num_blocks - live;
  for (int64_t i = 0; i < pool->count; ++i) pool->ring[i] = (int32_t)(live + i);
  *num_moves = n;
  return KVO_OK;
}

const int32_t* kvo_pool_table(const kvo_pool* pool) { return pool->table; }
int64_t kvo_pool_seq_len(const kvo_pool* pool, int64_t seq) { return pool->seq_len[seq]; }
int64_t kvo_pool_free_blocks(const kvo_pool* pool) { return pool->count; }
int64_t kvo_pool_live_blocks(const kvo_pool* pool) { return pool->num_blocks - pool->count; }

int64_t kvo_pool_free_list(const kvo_pool* pool, int32_t* out) {
  for (int64_t i = 0; i < pool->count; ++i) out[i] = pool->ring[(pool->head + i) % pool->num_blocks];
  return pool->count;
}
