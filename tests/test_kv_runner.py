"""The first-party runner (ascend-moe-engine_amd/apps/kv_runner.cpp): the KV-cache path of the
reference's decode loop, driven through the aclnn*/aclrt* exports as the reference's pipeline
drives them (src/pipeline/pipeline.cpp:390-416, :515-519; apps/moe_runner.cpp:434-447), with the
reference's flags and report files (--diag-json: src/diagnostics/inference_stats.cpp:18-55;
--stats-json: apps/moe_runner.cpp:483-514).

tests/golden/inference_diagnostics_dry_run.json is the sample the reference holds under
docs/examples/ (a data file, the output of its own dry run)."""
import json
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
RUNNER = os.path.join(ROOT, "ascend-moe-engine_amd", "kv_runner")
SAMPLE = os.path.join(HERE, "golden", "inference_diagnostics_dry_run.json")

# apps/moe_runner.cpp:483-514, in the order written there
STATS_FIELDS = ["generated_tokens", "prompt_tokens", "steps", "layers", "launches", "host_synchronizations", "expert_slot_hits",
                "expert_slot_misses", "swap_h2d_bytes", "swap_d2h_bytes", "swap_d2d_bytes", "swap_chunks", "startup_ingest_bytes",
                "device_allocations_in_step", "descriptors_built_in_step", "ttft_seconds", "tpot_seconds", "decode_span_seconds",
                "total_seconds", "device_slots", "slot_bytes", "backbone_bytes"]
# the reference's runner on its mock runtime (no device work at all), --prompt-tokens 128 --block-size 64, on 8 host cores:
# time to first token 48.9 ms over 128 steps of 43 layers
REFERENCE_HOST_MS_PER_STEP = 0.38


def run(*args, check=True):
    if not os.path.exists(RUNNER):
        pytest.fail("ascend-moe-engine_amd/kv_runner is not built: run `make -C ascend-moe-engine_amd`")
    done = subprocess.run([RUNNER, *map(str, args)], capture_output=True, text=True, timeout=300)
    if check and done.returncode != 0:
        pytest.fail(f"kv_runner exited with {done.returncode}\n{done.stdout}\n{done.stderr}")
    return done


def test_dry_run_writes_the_reference_sample_but_for_the_runtime_line(tmp_path):
    # the reference's defaults (block 128, context 8192, 43 layers) with the sample's 128 prompt tokens
    path = tmp_path / "diag.json"
    run("--dry-run", "--prompt-tokens", 128, "--diag-json", path)
    ours = path.read_text().splitlines()
    sample = open(SAMPLE).read().splitlines()
    assert len(ours) == len(sample)
    different = [(a, b) for a, b in zip(ours, sample) if a != b]
    assert different == [('  "mock_runtime": false,', '  "mock_runtime": true,')]  # this is a real device path
    # the paged_attention member byte for byte
    begin = sample.index('  "paged_attention": {')
    assert ours[begin:begin + 6] == sample[begin:begin + 6]


def test_flags_are_checked_and_a_missing_device_is_an_error(tmp_path):
    assert run("--no-such-flag", check=False).returncode == 2
    assert run("--block-size", 0, check=False).returncode == 2
    assert run("--block-size", 128, "--max-context", 64, check=False).returncode == 2
    import torch
    if not torch.cuda.is_available():
        done = run("--layers", 1, check=False)
        assert done.returncode == 2 and "aclrtSetDevice" in done.stderr  # no CPU path behind the boundary


def harness_argv(prompt_ids, new_tokens, stats_path, weights=None, config=None):
    """The command line the reference's benchmark driver starts its runner with
    (python/benchmarks/bench_runner.py:55-63 and :120-126): --prompt-ids <csv>, --max-new-tokens,
    --stats-json, then --weights <dir> or --synthetic-weights, then --config <file> when given."""
    argv = ["--prompt-ids", ",".join(str(t) for t in prompt_ids), "--max-new-tokens", str(new_tokens), "--stats-json", str(stats_path)]
    argv += ["--weights", weights] if weights else ["--synthetic-weights"]
    if config:
        argv += ["--config", config]
    return argv


def test_the_reference_harness_command_line_is_accepted(tmp_path):
    """What bench_runner.py passes, plus --dry-run so that no device is needed: the prompt length is
    the number of ids; --weights / --config are taken and reported as ignored; the MLA geometry
    flags of apps/moe_runner.cpp:170-181 are accepted at the compiled geometry and refused elsewhere."""
    ids = [(7919 * i + 13) % 129280 for i in range(37)]
    stats, diag = tmp_path / "stats.json", tmp_path / "diag.json"
    done = run(*harness_argv(ids, 32, stats), "--dry-run", "--diag-json", diag)
    assert "37 prompt + 32 new tokens = 68 steps" in done.stdout
    parsed = json.loads(diag.read_text())
    assert parsed["prompt_tokens"] == 37 and parsed["dry_run"] is True and parsed["generated_tokens"] == 0
    assert not stats.exists()                                    # written after a decode only, as the reference does
    done = run(*harness_argv(ids, 4, stats, weights="/models/ckpt", config="/models/ckpt/config.json"), "--dry-run")
    assert "ignored (not a flag of the KV path): --weights /models/ckpt" in done.stdout
    assert "ignored (not a flag of the KV path): --config /models/ckpt/config.json" in done.stdout
    run("--dry-run", "--kv-lora-rank", 512, "--qk-rope-head-dim", 64, "--qk-nope-head-dim", 128, "--v-head-dim", 128, "--prompt-tokens", 8)
    refused = run("--dry-run", "--kv-lora-rank", 256, check=False)
    assert refused.returncode == 2 and "compiled for kv_lora_rank 512, qk_rope_head_dim 64" in refused.stderr
    assert run("--dry-run", "--qk-rope-head-dim", 32, check=False).returncode == 2
    assert run("--dry-run", "--prompt-ids", "1,2", "--prompt-tokens", 2, check=False).returncode == 2   # apps/moe_runner.cpp:281-283
    assert run("--dry-run", "--prompt-ids", "1,x", check=False).returncode == 2
    assert run("--prompt-ids", "", check=False).returncode == 2                                         # nothing to decode
    report = tmp_path / "report.txt"
    done = run("--dry-run", "--prompt-tokens", 5, "--report", report, "--moe-path", "fused", "--vram-slots", 3)
    assert report.read_text() == done.stdout
    assert run("--help").stdout.startswith("kv_runner --")


@pytest.mark.gpu
def test_the_reference_harness_command_line_decodes(tmp_path):
    """The same command line for real: 24 prompt ids + 3 new tokens; the fields the driver reads
    from --stats-json (bench_runner.py:66-69, :74-94) are there and sensible."""
    ids = [(7919 * i + 13) % 129280 for i in range(24)]
    stats = tmp_path / "stats.json"
    run(*harness_argv(ids, 3, stats), "--block-size", 64, "--max-context", 256)
    report = json.loads(stats.read_text())
    assert list(report.keys())[:len(STATS_FIELDS)] == STATS_FIELDS
    assert report["prompt_tokens"] == 24 and report["generated_tokens"] == 3 and report["steps"] == 26
    assert report["ttft_seconds"] > 0 and report["tpot_seconds"] > 0
    assert report["total_seconds"] >= report["ttft_seconds"] + report["decode_span_seconds"] - 1e-6
    assert report["backbone_bytes"] > 43 * 256 * 1152 and report["gathered_rows_mismatched"] == 0


@pytest.mark.gpu
def test_configs0_through_the_operator_boundary(tmp_path):
    """128-token prompt, one more decode token, 43 layers, block 64, context 8192: every row of
    every layer comes back through the block table byte for byte; 129 of 8192 tokens."""
    diag, stats = tmp_path / "diag.json", tmp_path / "stats.json"
    done = run("--block-size", 64, "--max-context", 8192, "--prompt-tokens", 128, "--max-new-tokens", 2, "--diag-json", diag,
               "--stats-json", stats)
    print(done.stdout)
    text = diag.read_text()
    parsed = json.loads(text)
    sample = json.load(open(SAMPLE))
    assert list(parsed.keys()) == list(sample.keys())
    for member in ("moe_cache", "paged_attention", "attention"):
        assert list(parsed[member].keys()) == list(sample[member].keys())
    assert ('  "paged_attention": {\n    "total_blocks_allocated": 5504,\n    "active_context_tokens": 129,\n    "block_size": 64,\n'
            '    "kv_cache_utilization": 0.0157470703125\n  },\n') in text          # docs/preflight-verification.md:42-45
    assert parsed["prompt_tokens"] == 128 and parsed["generated_tokens"] == 2 and parsed["decoded_steps"] == 129
    assert parsed["ttft_ms"] > 0 and parsed["tpot_ms"] > 0 and parsed["mock_runtime"] is False
    report = json.loads(stats.read_text())
    assert list(report.keys())[:len(STATS_FIELDS)] == STATS_FIELDS
    assert report["steps"] == 129 and report["layers"] == 43 and report["launches"] == 129 * 43 * 2
    assert report["host_synchronizations"] == 2                  # one per generated token, as the reference's argmax readback
    assert report["device_allocations_in_step"] == 0 and report["descriptors_built_in_step"] == 0
    assert report["gathered_rows"] == 129 * 43 and report["gathered_rows_mismatched"] == 0
    per_step_ms = report["host_enqueue_seconds_per_step"] * 1e3
    print(f"host time per step: {per_step_ms:.3f} ms over 43 layers (the reference's mock dry run: "
          f"{REFERENCE_HOST_MS_PER_STEP} ms per step, plumbing only)")


@pytest.mark.gpu
def test_replayed_steps_equal_steps_enqueued_call_by_call(tmp_path):
    """--graph records one decode step after the first token (stream capture through the library's
    aclmdlRI* entry points) and replays it for every later token: the slot, the live length and the
    step's input rows reach the recording through pinned staging memory. A recording fixes its
    kernels, so the runner makes one per range of context lengths that has kernels of its own (this
    run crosses 256 tokens: two). Same appended rows (the runner's own gather check), same bits of
    the last step's attention output as without the flag."""
    reports = {}
    for mode in ("calls", "graph"):
        stats = tmp_path / f"stats_{mode}.json"
        done = run("--block-size", 64, "--max-context", 1024, "--prompt-tokens", 240, "--max-new-tokens", 40, "--stats-json", stats,
                   *(["--graph"] if mode == "graph" else []))
        reports[mode] = json.loads(stats.read_text())
        assert reports[mode]["gathered_rows_mismatched"] == 0 and reports[mode]["steps"] == 279
        assert reports[mode]["device_allocations_in_step"] == 0
        print(mode, done.stdout.split("timing: ")[1].splitlines()[0])
    assert reports["calls"]["replayed_steps"] == 0 and reports["graph"]["replayed_steps"] == 39
    assert reports["graph"]["recordings"] == 2
    assert reports["graph"]["last_output_fnv1a"] == reports["calls"]["last_output_fnv1a"]
    assert reports["graph"]["last_output_l1"] == reports["calls"]["last_output_l1"]
    assert reports["graph"]["launches"] == reports["calls"]["launches"] == 279 * 43 * 2
    print(f"tpot: {reports['calls']['tpot_seconds'] * 1e3:.3f} ms call by call (host {reports['calls']['host_enqueue_seconds_per_step'] * 1e3:.3f} ms "
          f"per step), {reports['graph']['tpot_seconds'] * 1e3:.3f} ms replayed (host {reports['graph']['host_seconds_per_replayed_step'] * 1e3:.3f} ms)")


@pytest.mark.gpu
def test_ragged_last_block_and_context_cap(tmp_path):
    # a context that is not a multiple of the block; the loop stops at the context as the reference's does
    stats = tmp_path / "stats.json"
    run("--block-size", 16, "--max-context", 100, "--prompt-tokens", 90, "--max-new-tokens", 40, "--layers", 3, "--stats-json", stats)
    report = json.loads(stats.read_text())
    assert report["steps"] == 100 and report["gathered_rows"] == 300 and report["gathered_rows_mismatched"] == 0
