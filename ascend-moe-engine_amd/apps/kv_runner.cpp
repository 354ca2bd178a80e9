// kv_runner -- the KV-cache path of the reference's decode loop, driven through the operator
// boundary (include/aclnn_hip.h) exactly as the reference's runner drives it:
//   apps/moe_runner.cpp:434-447       prefill as single-token steps, then max_new_tokens - 1 more
//   src/pipeline/pipeline.cpp:119-137 Build: reserve, one allocation, descriptors, plan once, seal
//   src/pipeline/pipeline.cpp:515-519 per step: the slot of the token through a pinned mailbox
//   src/pipeline/pipeline.cpp:390-416 per layer: five address swaps, kv_cache_write, attention
// The stages around them (projections, norms, rope, MoE, LM head) are not this library's; their
// outputs -- the kv_a row and the q_b row of every layer and step -- are seeded N(0,1) values
// (SplitMix64 + Box-Muller, rounded to bf16). After the last step every layer's rows are read
// back through the block table (aclnnGatherPaKvCache) and compared byte for byte with what was
// appended. Reports use the reference's field names (--diag-json: src/diagnostics/
// inference_stats.cpp:18-55; --stats-json: apps/moe_runner.cpp:483-514); members that belong to
// the expert hierarchy or the LM head are written with their idle values.
#include <chrono>
#include <cinttypes>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "aclnn_hip.h"
#include "mlakv.h"

namespace {

constexpr int64_t kHeads = 64, kLatent = 512, kRope = 64, kRow = kLatent + kRope;

struct Options {
  int64_t block_size = 128;      // RuntimeConfig defaults, include/moe/core/config.hpp:271-308
  int64_t max_context = 8192;
  int64_t prompt_tokens = 128;   // when neither --prompt-tokens nor --prompt-ids is given
  int64_t max_new_tokens = 1;
  int64_t layers = 43;
  int64_t qk_nope_head_dim = 128;  // only the softmax scale depends on it: 1 / sqrt(nope + rope), pipeline.cpp:238
  int32_t device = 0;
  uint64_t seed = 20251125;
  std::string diag_json, stats_json, report_path;
  std::vector<std::string> ignored;  // flags of stages this runner does not have, accepted for the reference's harness
  bool prompt_from_ids = false;
  bool verbose = false;
  bool dry_run = false;
  bool graph = false;  // decode steps after the first token replay one recorded step
  bool help = false;
};

[[noreturn]] void Die(const std::string& what) { throw std::runtime_error(what); }

void Check(int status, const char* call) {
  if (status != 0) {
    std::ostringstream text;
    text << call << " failed with status " << status << ": " << aclGetRecentErrMsg();
    Die(text.str());
  }
}
#define RUNNER_CHECK(call) Check((call), #call)

// Strict decimal integer, as the reference's ParseInt (apps/moe_runner.cpp:108-113).
int64_t Integer(const std::string& text, const std::string& flag) {
  char* end = nullptr;
  const long long parsed = std::strtoll(text.c_str(), &end, 10);
  if (text.empty() || end == nullptr || *end != '\0') Die(flag + " expects an integer, got '" + text + "'");
  return static_cast<int64_t>(parsed);
}

void PrintUsage() {
  std::printf(
      "kv_runner -- the KV-cache path of the decode loop (append + decode attention per layer) on one GPU\n"
      "\n"
      "  --prompt-ids a,b,c        prompt token ids: their count is the prompt length (the ids themselves\n"
      "                            feed an embedding this runner does not have and are otherwise unused)\n"
      "  --prompt-tokens <n>       prompt length without ids (default 128; not together with --prompt-ids)\n"
      "  --max-new-tokens <n>      tokens to generate (default 1)\n"
      "  --block-size <n>          paged KV block size (default 128)\n"
      "  --max-context <n>         reserved context length (default 8192)\n"
      "  --kv-lora-rank <n>        must be 512, --qk-rope-head-dim <n> must be 64, --v-head-dim <n> must be 128:\n"
      "                            the kernels are compiled for that geometry\n"
      "  --qk-nope-head-dim <n>    enters the softmax scale 1/sqrt(nope + rope) only (default 128)\n"
      "  --layers <n>              layers per step (default 43)\n"
      "  --device <id>             GPU (default 0)\n"
      "  --seed <n>                seed of the synthetic stage outputs\n"
      "  --dry-run                 size and report, decode nothing\n"
      "  --graph                   record one decode step (stream capture) after the first token and\n"
      "                            replay it for every later token: one launch per step for the host\n"
      "  --report <path>           write the report there as well as to stdout\n"
      "  --diag-json <path>        structured diagnostics (also for dry runs)\n"
      "  --stats-json <path>       machine-readable run stats after a decode\n"
      "  --verbose\n"
      "  --synthetic-weights       accepted: the only kind of input this runner has\n"
      "  --weights --config --prompt --vram-slots --moe-path --moe-backend --gating-norm-type\n"
      "  --dense-group-size --routed-coverage <value>\n"
      "                            accepted and ignored: they configure stages (weights, MoE, GEMMs)\n"
      "                            that are not part of the KV path; the report lists them\n");
}

// The reference runner's command line (apps/moe_runner.cpp:137-218), so that a driver written for it
// (python/benchmarks/bench_runner.py:55-71 always passes --prompt-ids, --max-new-tokens, --stats-json
// and --synthetic-weights or --weights, optionally --config) starts this binary unchanged.
Options Parse(int argc, char** argv) {
  Options o;
  bool prompt_tokens_given = false;
  for (int i = 1; i < argc; ++i) {
    const std::string flag = argv[i];
    const auto value = [&]() -> std::string {
      if (i + 1 >= argc) Die(flag + " needs a value");
      return argv[++i];
    };
    const auto geometry = [&](int64_t compiled) {
      const int64_t asked = Integer(value(), flag);
      if (asked != compiled) {
        Die(flag + " " + std::to_string(asked) + " refused: the kernels are compiled for kv_lora_rank 512, qk_rope_head_dim 64, "
            "v_head_dim 128 (" + flag + " must be " + std::to_string(compiled) + ")");
      }
    };
    if (flag == "--help" || flag == "-h") o.help = true;
    else if (flag == "--block-size") o.block_size = Integer(value(), flag);
    else if (flag == "--max-context") o.max_context = Integer(value(), flag);
    else if (flag == "--prompt-tokens") {
      o.prompt_tokens = Integer(value(), flag);
      if (o.prompt_tokens <= 0) Die("--prompt-tokens must be positive");
      prompt_tokens_given = true;
    } else if (flag == "--prompt-ids") {
      // ParseIdList (apps/moe_runner.cpp:115-125): comma-separated integers, empty pieces skipped
      const std::string list = value();
      int64_t count = 0;
      std::stringstream pieces(list);
      std::string piece;
      while (std::getline(pieces, piece, ',')) {
        if (piece.empty()) continue;
        Integer(piece, flag);
        ++count;
      }
      o.prompt_tokens = count;
      o.prompt_from_ids = true;
    }
    else if (flag == "--max-new-tokens") o.max_new_tokens = Integer(value(), flag);
    else if (flag == "--layers") o.layers = Integer(value(), flag);
    else if (flag == "--device") o.device = static_cast<int32_t>(Integer(value(), flag));
    else if (flag == "--seed") o.seed = std::stoull(value());
    else if (flag == "--kv-lora-rank") geometry(kLatent);
    else if (flag == "--qk-rope-head-dim") geometry(kRope);
    else if (flag == "--v-head-dim") geometry(128);
    else if (flag == "--qk-nope-head-dim") {
      o.qk_nope_head_dim = Integer(value(), flag);
      if (o.qk_nope_head_dim <= 0) Die("--qk-nope-head-dim must be positive");
    }
    else if (flag == "--diag-json") o.diag_json = value();
    else if (flag == "--stats-json") o.stats_json = value();
    else if (flag == "--report") o.report_path = value();
    else if (flag == "--verbose") o.verbose = true;
    else if (flag == "--dry-run") o.dry_run = true;
    else if (flag == "--graph") o.graph = true;
    else if (flag == "--synthetic-weights") {}  // the only kind of input this runner has
    else if (flag == "--weights" || flag == "--config" || flag == "--prompt" || flag == "--vram-slots" || flag == "--moe-path" ||
             flag == "--moe-backend" || flag == "--gating-norm-type" || flag == "--dense-group-size" || flag == "--routed-coverage") {
      o.ignored.push_back(flag + " " + value());
    }
    else Die("unknown flag: " + flag + " (--help lists the flags)");
  }
  if (prompt_tokens_given && o.prompt_from_ids) Die("--prompt-tokens cannot be combined with --prompt-ids");
  if (o.block_size <= 0 || o.max_context <= 0) Die("context length and block size must be positive");
  if (o.max_context < o.block_size) Die("block size must not be above the context");
  if (o.max_new_tokens <= 0) Die("--max-new-tokens must be positive");
  if (o.layers < 1) Die("--layers must be at least 1");
  if (o.prompt_from_ids && o.prompt_tokens == 0 && !o.dry_run) Die("--prompt-ids is empty: there is nothing to decode");
  if (o.prompt_tokens > o.max_context) Die("prompt exceeds context capacity");
  return o;
}

// SplitMix64 (Steele, Lea, Flood 2014) and Box-Muller: the same values on every host.
struct Generator {
  uint64_t state;
  uint64_t Next() {
    uint64_t z = (state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
  }
  double Uniform() { return (static_cast<double>(Next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
  double Normal() { return std::sqrt(-2.0 * std::log(Uniform())) * std::cos(6.283185307179586 * Uniform()); }
};

uint16_t ToBf16(float value) {  // round to nearest even
  uint32_t bits;
  std::memcpy(&bits, &value, 4);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return static_cast<uint16_t>(bits >> 16);
}

void Number(std::ostream& out, double value) {  // as the reference writes optional numbers
  if (std::isfinite(value)) out << value;
  else out << "null";
}

struct Diagnostics {
  uint64_t prompt_tokens = 0, generated_tokens = 0, decoded_steps = 0;
  double ttft_ms = NAN, tpot_ms = NAN;
  mlakvKvStats paged{};
};

void DumpDiagJson(const std::string& path, const Options& o, const Diagnostics& d) {
  std::ofstream out(path);
  if (!out.is_open()) Die("cannot write inference diagnostics to " + path);
  out.imbue(std::locale::classic());
  out << std::setprecision(12) << std::boolalpha;
  out << "{\n  \"schema_version\": 1,\n"
      << "  \"mock_runtime\": false,\n"
      << "  \"synthetic_weights\": true,\n"
      << "  \"dry_run\": " << o.dry_run << ",\n"
      << "  \"prompt_tokens\": " << d.prompt_tokens << ",\n"
      << "  \"generated_tokens\": " << d.generated_tokens << ",\n"
      << "  \"decoded_steps\": " << d.decoded_steps << ",\n  \"ttft_ms\": ";
  Number(out, d.ttft_ms);
  out << ",\n  \"tpot_ms\": ";
  Number(out, d.tpot_ms);
  out << ",\n  \"perplexity\": null,\n  \"moe_cache\": {\n"
      << "    \"total_expert_requests\": 0,\n    \"hbm_slot_hits\": 0,\n    \"host_promotions\": 0,\n"
      << "    \"evictions_to_host\": 0,\n    \"hit_rate\": 0\n  },\n";
  std::vector<char> member(static_cast<size_t>(mlakvKvStatsFormatJson(&d.paged, nullptr, 0)) + 1);
  mlakvKvStatsFormatJson(&d.paged, member.data(), member.size());
  out << member.data();
  out << ",\n  \"attention\": {\n    \"mode\": \"dense_mla\",\n    \"attention_entropy\": null,\n    \"sparsity_ratio\": 0\n  }\n}\n";
  out.close();
  if (!out) Die("failed writing inference diagnostics to " + path);
}

int Run(int argc, char** argv) {
  const Options o = Parse(argc, argv);
  if (o.help) {
    PrintUsage();
    return 0;
  }
  const int64_t num_blocks = (o.max_context + o.block_size - 1) / o.block_size;  // static_arena_manager.cpp:192-201
  const int64_t steps = std::min(o.prompt_tokens + o.max_new_tokens - 1, o.max_context);
  Diagnostics diag;
  diag.prompt_tokens = static_cast<uint64_t>(o.prompt_tokens);
  diag.paged.total_blocks_allocated = static_cast<uint64_t>(num_blocks * o.layers);  // pipeline.cpp:134-136
  diag.paged.block_size = static_cast<uint64_t>(o.block_size);
  std::ostringstream report;
  report << "kv_runner: " << o.layers << " layers, block " << o.block_size << ", context " << o.max_context << " (" << num_blocks
         << " blocks per layer), " << o.prompt_tokens << " prompt + " << o.max_new_tokens << " new tokens = " << steps << " steps\n";
  if (o.prompt_from_ids) report << "prompt length taken from --prompt-ids (" << o.prompt_tokens << " ids; their values are not used)\n";
  for (const std::string& flag : o.ignored) report << "ignored (not a flag of the KV path): " << flag << "\n";
  const auto emit_report = [&]() {
    std::cout << report.str();
    if (!o.report_path.empty()) {
      std::ofstream file(o.report_path);
      if (!file.is_open()) Die("cannot write the report to " + o.report_path);
      file << report.str();
    }
  };
  if (o.dry_run) {
    if (!o.diag_json.empty()) DumpDiagJson(o.diag_json, o, diag);
    report << "--dry-run: sized and reported; no token was decoded.\n";
    emit_report();
    return 0;
  }

  RUNNER_CHECK(aclInit(nullptr));
  RUNNER_CHECK(aclnnInit(nullptr));
  RUNNER_CHECK(aclrtSetDevice(o.device));
  aclrtStream stream = nullptr;
  RUNNER_CHECK(aclrtCreateStream(&stream));

  // RESERVE + COMMIT: one allocation for everything the path touches, 512-byte aligned pieces in
  // request order, zero-filled (src/memory/static_arena.cpp:88-118).
  const auto align_up = [](size_t value) { return (value + 511) & ~size_t{511}; };
  size_t cursor = 0;
  const auto reserve = [&](size_t bytes) {
    const size_t offset = align_up(cursor);
    cursor = offset + bytes;
    return offset;
  };
  const size_t latent_stride = static_cast<size_t>(2 * num_blocks * o.block_size * kLatent);  // pipeline.cpp:391-392
  const size_t rope_stride = static_cast<size_t>(2 * num_blocks * o.block_size * kRope);
  const size_t off_table = reserve(4 * static_cast<size_t>(num_blocks));
  const size_t off_slot = reserve(4);
  const size_t off_lens = reserve(4);
  const size_t off_cu = reserve(8);
  // kv_latent_normed, kv_a and q_b sit back to back so that one copy stands in for the stages that write them
  const size_t off_normed = reserve(2 * (kLatent + kRow + kHeads * kRow));
  const size_t off_kv_a = off_normed + 2 * kLatent;
  const size_t off_q_b = off_kv_a + 2 * kRow;
  const size_t off_out = reserve(2 * kHeads * kLatent);
  const size_t off_gather_latent = reserve(2 * static_cast<size_t>(steps) * kLatent);
  const size_t off_gather_rope = reserve(2 * static_cast<size_t>(steps) * kRope);
  const size_t off_latent = reserve(latent_stride * static_cast<size_t>(o.layers));
  const size_t off_rope = reserve(rope_stride * static_cast<size_t>(o.layers));
  const size_t off_live = reserve(4);  // the live length as the attention reads it when steps are replayed
  const size_t arena_bytes = align_up(cursor);
  char* arena = nullptr;
  uint64_t device_allocations = 0;
  RUNNER_CHECK(aclrtMalloc(reinterpret_cast<void**>(&arena), arena_bytes, ACL_MEM_MALLOC_HUGE_FIRST));
  ++device_allocations;
  RUNNER_CHECK(aclrtMemset(arena, arena_bytes, 0, arena_bytes));

  // Descriptors, one layer's view each, pointed at layer 0 (static_arena_manager.cpp:480-497, :567-588).
  std::vector<std::vector<int64_t>> keep_dims;
  const auto tensor = [&](std::vector<int64_t> dims, aclDataType dtype, void* data, std::vector<int64_t> strides = {}) {
    if (strides.empty()) {
      strides.assign(dims.size(), 1);
      for (int64_t i = static_cast<int64_t>(dims.size()) - 2; i >= 0; --i) strides[i] = strides[i + 1] * dims[i + 1];
    }
    keep_dims.push_back(dims);
    const std::vector<int64_t>& d = keep_dims.back();
    keep_dims.push_back(strides);
    const std::vector<int64_t>& s = keep_dims.back();
    aclTensor* t = aclCreateTensor(d.data(), d.size(), dtype, s.data(), 0, ACL_FORMAT_ND, d.data(), d.size(), data);
    if (t == nullptr) Die(std::string("aclCreateTensor: ") + aclGetRecentErrMsg());
    return t;
  };
  keep_dims.reserve(64);
  char* q_b = arena + off_q_b;
  char* kv_a = arena + off_kv_a;
  // q_b holds, per head, [latent 512 | rope 64]: the two query operands are views at the stride of
  // the whole row (static_arena_manager.cpp:481-485 describes them so)
  aclTensor* q_latent = tensor({1, kHeads, kLatent}, ACL_BF16, q_b, {kHeads * kRow, kRow, 1});
  aclTensor* q_rope = tensor({1, kHeads, kRope}, ACL_BF16, q_b + 2 * kLatent, {kHeads * kRow, kRow, 1});
  aclTensor* k_rope = tensor({1, 1, kRope}, ACL_BF16, kv_a + 2 * kLatent);
  aclTensor* kv_latent_normed = tensor({1, kLatent}, ACL_BF16, arena + off_normed);
  aclTensor* attn_out = tensor({1, kHeads, kLatent}, ACL_BF16, arena + off_out);
  aclTensor* latent_cache = tensor({num_blocks, o.block_size, 1, kLatent}, ACL_BF16, arena + off_latent);
  aclTensor* rope_cache = tensor({num_blocks, o.block_size, 1, kRope}, ACL_BF16, arena + off_rope);
  aclTensor* rope_cache_view = tensor({num_blocks, o.block_size, 1, kRope}, ACL_BF16, arena + off_rope);
  aclTensor* key_member = tensor({num_blocks, o.block_size, 1, kLatent}, ACL_BF16, arena + off_latent);
  aclTensor* value_member = tensor({num_blocks, o.block_size, 1, kLatent}, ACL_BF16, arena + off_latent);
  aclTensorList* key_list = aclCreateTensorList(&key_member, 1);
  aclTensorList* value_list = aclCreateTensorList(&value_member, 1);
  aclTensor* block_table = tensor({1, num_blocks}, ACL_INT32, arena + off_table);
  aclTensor* slot_mapping = tensor({1}, ACL_INT32, arena + off_slot);
  aclTensor* seq_lens = tensor({1}, ACL_INT32, arena + off_lens);
  aclTensor* cu_seq_lens = tensor({2}, ACL_INT32, arena + off_cu);
  aclTensor* gather_latent = tensor({steps, kLatent}, ACL_BF16, arena + off_gather_latent);
  aclTensor* gather_rope = tensor({steps, 1, kRope}, ACL_BF16, arena + off_gather_rope);
  const int64_t one = 1;
  aclIntArray* actual_seq_q = aclCreateIntArray(&one, 1);
  aclIntArray* actual_seq_kv = aclCreateIntArray(&o.max_context, 1);
  if (!key_list || !value_list || !actual_seq_q || !actual_seq_kv) Die(std::string("descriptor creation: ") + aclGetRecentErrMsg());

  // Plan once (pipeline.cpp:226-249); the executors are made repeatable as StaticOpSlot::Adopt does.
  char cache_mode[] = "Norm", layout[] = "TND";
  uint64_t ws_scatter = 0, ws_attention = 0, ws_gather = 0;
  aclOpExecutor *ex_scatter = nullptr, *ex_attention = nullptr, *ex_gather = nullptr;
  RUNNER_CHECK(aclnnScatterPaKvCacheGetWorkspaceSize(kv_latent_normed, latent_cache, slot_mapping, k_rope, rope_cache, nullptr, nullptr,
                                                     nullptr, cache_mode, nullptr, nullptr, nullptr, &ws_scatter, &ex_scatter));
  RUNNER_CHECK(aclnnFusedInferAttentionScoreV5GetWorkspaceSize(
      q_latent, key_list, value_list, nullptr, nullptr, actual_seq_q, actual_seq_kv, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
      nullptr, block_table, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, q_rope, rope_cache_view,
      nullptr, nullptr, nullptr, nullptr, nullptr, kHeads, 1.0 / std::sqrt(static_cast<double>(o.qk_nope_head_dim + kRope)), 65536, 0, layout, 1, 3, 0, o.block_size, 0, false, 0, 0,
      0, 0, attn_out, nullptr, &ws_attention, &ex_attention));
  RUNNER_CHECK(aclnnGatherPaKvCacheGetWorkspaceSize(latent_cache, rope_cache, block_table, seq_lens, cu_seq_lens, gather_latent, gather_rope,
                                                    o.max_context, &ws_gather, &ex_gather));
  RUNNER_CHECK(aclSetAclOpExecutorRepeatable(ex_scatter));
  RUNNER_CHECK(aclSetAclOpExecutorRepeatable(ex_attention));
  RUNNER_CHECK(aclSetAclOpExecutorRepeatable(ex_gather));
  const uint64_t workspace_bytes = std::max(ws_scatter, std::max(ws_attention, ws_gather));  // the shared high-water mark
  void* workspace = nullptr;
  if (workspace_bytes > 0) {
    RUNNER_CHECK(aclrtMalloc(&workspace, workspace_bytes, ACL_MEM_MALLOC_HUGE_FIRST));  // the second and last allocation
    ++device_allocations;
  }
  const uint64_t allocations_at_seal = device_allocations;

  // The block table: identity paging for the one sequence (the reference leaves it zero).
  std::vector<int32_t> identity(static_cast<size_t>(num_blocks));
  for (int64_t i = 0; i < num_blocks; ++i) identity[static_cast<size_t>(i)] = static_cast<int32_t>(i);
  RUNNER_CHECK(aclrtMemcpy(arena + off_table, 4 * identity.size(), identity.data(), 4 * identity.size(), ACL_MEMCPY_HOST_TO_DEVICE));

  // The other stages' outputs for every step and layer, pinned so the copies can be asynchronous.
  // Per item: [normed latent 512 | kv_a row 576 (the same latent, then the rope part) | q_b 64 x 576].
  const size_t per_item = static_cast<size_t>(kLatent + kRow + kHeads * kRow);
  const size_t items = static_cast<size_t>(steps * o.layers);
  uint16_t* inputs = nullptr;
  RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&inputs), 2 * per_item * items));
  Generator generator{o.seed};
  for (size_t item = 0; item < items; ++item) {
    uint16_t* row = inputs + per_item * item;
    for (size_t i = static_cast<size_t>(kLatent); i < per_item; ++i) row[i] = ToBf16(static_cast<float>(generator.Normal()));
    std::memcpy(row, row + kLatent, 2 * kLatent);
  }
  int32_t* mailbox = nullptr;
  RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&mailbox), 4 * static_cast<size_t>(steps)));
  uint16_t* readback = nullptr;
  RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&readback), 2 * kHeads * kLatent));

  // Replayed steps: a recorded step cannot take its position, its length or its input rows from
  // host arguments, so the length is read from device memory (a word of the arena, written by a
  // copy from a pinned word as the slot is) and the step's inputs come from one pinned staging area.
  int32_t* live_words = nullptr;   // a word per step (eager steps), like the slot mailbox
  int32_t* replay_words = nullptr; // [slot, length] of the step being replayed
  uint16_t* replay_inputs = nullptr;
  if (o.graph) {
    RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&live_words), 4 * static_cast<size_t>(steps)));
    RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&replay_words), 8));
    RUNNER_CHECK(aclrtMallocHost(reinterpret_cast<void**>(&replay_inputs), 2 * per_item * static_cast<size_t>(o.layers)));
    RUNNER_CHECK(aclnnMlaKvBindSeqLens(ex_attention, reinterpret_cast<const int32_t*>(arena + off_live)));
  }

  uint64_t launches = 0, host_synchronizations = 0, generated = 0, replayed_steps = 0;
  double enqueue_seconds = 0.0, replay_host_seconds = 0.0;
  // One step's work on the stream; `slot_word`, `live_word` and `step_inputs` are pinned host memory.
  const auto enqueue_step = [&](const int32_t* slot_word, const int32_t* live_word, const uint16_t* step_inputs) {
    RUNNER_CHECK(aclrtMemcpyAsync(arena + off_slot, 4, slot_word, 4, ACL_MEMCPY_HOST_TO_DEVICE, stream));
    if (live_word != nullptr) RUNNER_CHECK(aclrtMemcpyAsync(arena + off_live, 4, live_word, 4, ACL_MEMCPY_HOST_TO_DEVICE, stream));
    for (int64_t layer = 0; layer < o.layers; ++layer) {
      const uint16_t* item = step_inputs + per_item * static_cast<size_t>(layer);
      RUNNER_CHECK(aclrtMemcpyAsync(arena + off_normed, 2 * per_item, item, 2 * per_item, ACL_MEMCPY_HOST_TO_DEVICE, stream));
      char* latent = arena + off_latent + latent_stride * static_cast<size_t>(layer);
      char* rope = arena + off_rope + rope_stride * static_cast<size_t>(layer);
      RUNNER_CHECK(aclSetTensorAddr(ex_scatter, 1, latent_cache, latent));            // kScatterKeyCache
      RUNNER_CHECK(aclSetTensorAddr(ex_scatter, 4, rope_cache, rope));                // kScatterValueCache
      RUNNER_CHECK(aclSetDynamicTensorAddr(ex_attention, 1, 0, key_list, latent));    // kFiaKeyList
      RUNNER_CHECK(aclSetDynamicTensorAddr(ex_attention, 2, 0, value_list, latent));  // kFiaValueList
      RUNNER_CHECK(aclSetTensorAddr(ex_attention, 25, rope_cache_view, rope));        // kFiaKeyRope
      RUNNER_CHECK(aclnnScatterPaKvCache(workspace, ws_scatter, ex_scatter, stream));
      RUNNER_CHECK(aclnnFusedInferAttentionScoreV5(workspace, ws_attention, ex_attention, stream));
    }
  };
  uint64_t eager_steps = 0;
  const auto decode_step = [&](int64_t position) {
    const auto begin = std::chrono::steady_clock::now();
    mailbox[position] = static_cast<int32_t>(position);  // slot = position (pipeline.cpp:517); a word per step
    const int64_t live = position + 1;
    if (o.graph) {  // the length lives in device memory; the launch chooses its kernels by the bound it is told
      live_words[position] = static_cast<int32_t>(live);
      RUNNER_CHECK(aclnnMlaKvSetSeqLenBound(ex_attention, live));
    } else {
      RUNNER_CHECK(aclnnMlaKvSetSeqLens(ex_attention, &live, 1));
    }
    enqueue_step(mailbox + position, o.graph ? live_words + position : nullptr, inputs + per_item * static_cast<size_t>(position * o.layers));
    launches += 2 * static_cast<uint64_t>(o.layers);
    ++eager_steps;
    enqueue_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - begin).count();
  };
  aclmdlRI recorded_step = nullptr;
  int64_t recorded_bound = 0;  // the context length the recording's kernels were chosen for
  uint64_t recordings = 0;
  const auto replay_step = [&](int64_t position) {
    const auto begin = std::chrono::steady_clock::now();
    if (recorded_step == nullptr || position + 1 > recorded_bound) {
      // Record: the same calls, from the staging words and rows. A recording fixes the kernels of
      // its launches, and short contexts have faster ones, so it is made for the next size where
      // the choice changes and made again when the context outgrows it.
      if (recorded_step != nullptr) RUNNER_CHECK(aclmdlRIDestroy(recorded_step));
      recorded_step = nullptr;
      recorded_bound = position + 1 <= 256 ? 256 : (position + 1 <= 768 ? 768 : o.max_context);
      recorded_bound = std::min(recorded_bound, o.max_context);
      RUNNER_CHECK(aclnnMlaKvSetSeqLenBound(ex_attention, recorded_bound));
      RUNNER_CHECK(aclmdlRICaptureBegin(stream, ACL_MODEL_RI_CAPTURE_MODE_GLOBAL));
      enqueue_step(replay_words, replay_words + 1, replay_inputs);
      RUNNER_CHECK(aclmdlRICaptureEnd(stream, &recorded_step));
      ++recordings;
    }
    // (the previous step's readback has been waited for: the staging area is free)
    replay_words[0] = static_cast<int32_t>(position);
    replay_words[1] = static_cast<int32_t>(position + 1);
    std::memcpy(replay_inputs, inputs + per_item * static_cast<size_t>(position * o.layers), 2 * per_item * static_cast<size_t>(o.layers));
    RUNNER_CHECK(aclmdlRIExecuteAsync(recorded_step, stream));
    launches += 2 * static_cast<uint64_t>(o.layers);
    ++replayed_steps;
    replay_host_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - begin).count();
  };
  const auto read_token = [&]() {  // where the reference reads the argmax back: one synchronisation per generated token
    RUNNER_CHECK(aclrtMemcpyAsync(readback, 2 * kHeads * kLatent, arena + off_out, 2 * kHeads * kLatent, ACL_MEMCPY_DEVICE_TO_HOST, stream));
    RUNNER_CHECK(aclrtSynchronizeStream(stream));
    ++host_synchronizations;
    ++generated;
  };

  const auto decode_start = std::chrono::steady_clock::now();
  int64_t position = 0;
  for (int64_t i = 0; i < o.prompt_tokens && position < o.max_context; ++i) decode_step(position++);
  read_token();
  const auto first_token_time = std::chrono::steady_clock::now();
  for (int64_t i = 1; i < o.max_new_tokens && position < o.max_context; ++i) {
    if (o.graph) {
      replay_step(position++);
    } else {
      decode_step(position++);
    }
    read_token();
  }
  const auto decode_end = std::chrono::steady_clock::now();
  // The last step's attention output (64 heads x 512 bf16) in two figures: FNV-1a over its bytes
  // (the same for the same seed and flags as long as the same kernels run) and the sum of the
  // magnitudes (which kernels that round differently agree on to a fraction of a percent: a step
  // whose lengths the host passes by value may take the short-context units where a replayed step,
  // whose length lives in device memory, takes the 64-head kernel).
  uint64_t output_hash = 0xcbf29ce484222325ull;
  for (size_t i = 0; i < 2 * static_cast<size_t>(kHeads * kLatent); ++i) {
    output_hash = (output_hash ^ reinterpret_cast<const unsigned char*>(readback)[i]) * 0x100000001b3ull;
  }
  double output_l1 = 0.0;
  for (size_t i = 0; i < static_cast<size_t>(kHeads * kLatent); ++i) {
    const uint32_t bits = static_cast<uint32_t>(readback[i]) << 16;
    float value;
    std::memcpy(&value, &bits, 4);
    output_l1 += std::fabs(static_cast<double>(value));
  }
  const double ttft_seconds = std::chrono::duration<double>(first_token_time - decode_start).count();
  const double decode_span_seconds = std::chrono::duration<double>(decode_end - first_token_time).count();
  const double total_seconds = std::chrono::duration<double>(decode_end - decode_start).count();
  const double tpot_seconds = generated > 1 ? decode_span_seconds / static_cast<double>(generated - 1) : 0.0;
  const uint64_t allocations_in_step = device_allocations - allocations_at_seal;

  // Gather every layer's rows through the block table and compare them with what was appended.
  const int32_t lens_host[1] = {static_cast<int32_t>(position)};
  const int32_t cu_host[2] = {0, static_cast<int32_t>(position)};
  RUNNER_CHECK(aclrtMemcpy(arena + off_lens, 4, lens_host, 4, ACL_MEMCPY_HOST_TO_DEVICE));
  RUNNER_CHECK(aclrtMemcpy(arena + off_cu, 8, cu_host, 8, ACL_MEMCPY_HOST_TO_DEVICE));
  std::vector<uint16_t> rows_latent(static_cast<size_t>(position * kLatent)), rows_rope(static_cast<size_t>(position * kRope));
  uint64_t mismatched_rows = 0;
  for (int64_t layer = 0; layer < o.layers; ++layer) {
    RUNNER_CHECK(aclSetTensorAddr(ex_gather, 0, latent_cache, arena + off_latent + latent_stride * static_cast<size_t>(layer)));
    RUNNER_CHECK(aclSetTensorAddr(ex_gather, 1, rope_cache, arena + off_rope + rope_stride * static_cast<size_t>(layer)));
    RUNNER_CHECK(aclnnGatherPaKvCache(workspace, ws_gather, ex_gather, stream));
    RUNNER_CHECK(aclrtSynchronizeStream(stream));
    RUNNER_CHECK(aclrtMemcpy(rows_latent.data(), 2 * rows_latent.size(), arena + off_gather_latent, 2 * rows_latent.size(), ACL_MEMCPY_DEVICE_TO_HOST));
    RUNNER_CHECK(aclrtMemcpy(rows_rope.data(), 2 * rows_rope.size(), arena + off_gather_rope, 2 * rows_rope.size(), ACL_MEMCPY_DEVICE_TO_HOST));
    for (int64_t p = 0; p < position; ++p) {
      const uint16_t* item = inputs + per_item * static_cast<size_t>(p * o.layers + layer) + kLatent;  // the kv_a row
      if (std::memcmp(rows_latent.data() + p * kLatent, item, 2 * kLatent) != 0 ||
          std::memcmp(rows_rope.data() + p * kRope, item + kLatent, 2 * kRope) != 0) {
        ++mismatched_rows;
      }
    }
  }

  diag.generated_tokens = generated;
  diag.decoded_steps = static_cast<uint64_t>(position);
  diag.ttft_ms = ttft_seconds * 1000.0;
  if (generated > 1) diag.tpot_ms = tpot_seconds * 1000.0;
  diag.paged.active_context_tokens = static_cast<uint64_t>(position);                                       // pipeline.cpp:532-534
  diag.paged.kv_cache_utilization = static_cast<double>(position) / static_cast<double>(num_blocks * o.block_size);
  report << "steps " << position << ", layers " << o.layers << ", launches " << launches << "\n"
         << "timing: ttft " << ttft_seconds << " s (prefill of " << o.prompt_tokens << " single-token steps + first readback), tpot "
         << tpot_seconds << " s, total " << total_seconds << " s\n"
         << "host time per step (enqueue only) " << enqueue_seconds / static_cast<double>(eager_steps) * 1e3 << " ms over "
         << eager_steps << " steps enqueued call by call\n"
         << (replayed_steps > 0 ? "replayed " + std::to_string(replayed_steps) + " steps from " + std::to_string(recordings) +
                                      " recording(s) of a step (one per range of context lengths with kernels of its own): host time per replayed step " +
                                      std::to_string(replay_host_seconds / static_cast<double>(replayed_steps) * 1e3) +
                                      " ms (staging the step's inputs, one launch; recording included)\n"
                                : std::string())
         << "host synchronizations " << host_synchronizations << " (one per generated-token readback)\n"
         << "allocations inside a step " << allocations_in_step << " (must be 0); descriptors 0 (must be 0)\n"
         << "gathered " << position << " rows x " << o.layers << " layers through the block table: " << mismatched_rows
         << " rows differ from what was appended (must be 0)\n"
         << "kv cache: " << diag.paged.total_blocks_allocated << " blocks of " << o.block_size << " tokens, utilization "
         << std::setprecision(12) << diag.paged.kv_cache_utilization << "\n";
  if (!o.stats_json.empty()) {
    std::ofstream stats(o.stats_json);
    if (!stats.is_open()) Die("cannot write the stats to " + o.stats_json);
    stats << "{\n"
          << "  \"generated_tokens\": " << generated << ",\n"
          << "  \"prompt_tokens\": " << o.prompt_tokens << ",\n"
          << "  \"steps\": " << position << ",\n"
          << "  \"layers\": " << o.layers << ",\n"
          << "  \"launches\": " << launches << ",\n"
          << "  \"host_synchronizations\": " << host_synchronizations << ",\n"
          << "  \"expert_slot_hits\": 0,\n  \"expert_slot_misses\": 0,\n"
          << "  \"swap_h2d_bytes\": 0,\n  \"swap_d2h_bytes\": 0,\n  \"swap_d2d_bytes\": 0,\n  \"swap_chunks\": 0,\n"
          << "  \"startup_ingest_bytes\": 0,\n"
          << "  \"device_allocations_in_step\": " << allocations_in_step << ",\n"
          << "  \"descriptors_built_in_step\": 0,\n"
          << "  \"ttft_seconds\": " << ttft_seconds << ",\n"
          << "  \"tpot_seconds\": " << tpot_seconds << ",\n"
          << "  \"decode_span_seconds\": " << decode_span_seconds << ",\n"
          << "  \"total_seconds\": " << total_seconds << ",\n"
          << "  \"device_slots\": 0,\n  \"slot_bytes\": 0,\n"
          << "  \"backbone_bytes\": " << arena_bytes << ",\n"
          << "  \"host_enqueue_seconds_per_step\": " << enqueue_seconds / static_cast<double>(eager_steps) << ",\n"
          << "  \"replayed_steps\": " << replayed_steps << ",\n"
          << "  \"recordings\": " << recordings << ",\n"
          << "  \"host_seconds_per_replayed_step\": " << (replayed_steps > 0 ? replay_host_seconds / static_cast<double>(replayed_steps) : 0.0) << ",\n"
          << "  \"last_output_fnv1a\": \"" << std::hex << output_hash << std::dec << "\",\n"
          << "  \"last_output_l1\": " << std::setprecision(12) << output_l1 << ",\n"
          << "  \"gathered_rows\": " << position * o.layers << ",\n"
          << "  \"gathered_rows_mismatched\": " << mismatched_rows << "\n"
          << "}\n";
    report << "stats written to " << o.stats_json << "\n";
  }
  if (!o.diag_json.empty()) {
    DumpDiagJson(o.diag_json, o, diag);
    report << "diagnostics written to " << o.diag_json << "\n";
  }
  emit_report();

  // Teardown in the reference's order: executors after the streams drain and before descriptors
  // and buffers (include/moe/core/op_table.hpp:131-134; src/memory/static_arena.cpp:50-69).
  RUNNER_CHECK(aclrtSynchronizeStream(stream));
  aclDestroyAclOpExecutor(ex_gather);
  aclDestroyAclOpExecutor(ex_attention);
  aclDestroyAclOpExecutor(ex_scatter);
  aclDestroyTensorList(key_list);
  aclDestroyTensorList(value_list);
  for (aclTensor* t : {q_latent, q_rope, k_rope, kv_latent_normed, attn_out, latent_cache, rope_cache, rope_cache_view, block_table,
                       slot_mapping, seq_lens, cu_seq_lens, gather_latent, gather_rope}) {
    aclDestroyTensor(t);
  }
  aclDestroyIntArray(actual_seq_q);
  aclDestroyIntArray(actual_seq_kv);
  if (recorded_step != nullptr) RUNNER_CHECK(aclmdlRIDestroy(recorded_step));
  if (o.graph) {
    aclrtFreeHost(live_words);
    aclrtFreeHost(replay_words);
    aclrtFreeHost(replay_inputs);
  }
  aclrtFreeHost(readback);
  aclrtFreeHost(mailbox);
  aclrtFreeHost(inputs);
  if (workspace != nullptr) aclrtFree(workspace);
  aclrtFree(arena);
  aclrtDestroyStream(stream);
  aclnnFinalize();
  aclFinalize();
  return allocations_in_step == 0 && mismatched_rows == 0 ? 0 : 1;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    return Run(argc, argv);
  } catch (const std::exception& error) {
    std::cerr << "kv_runner: " << error.what() << "\n";
    return 2;
  }
}
