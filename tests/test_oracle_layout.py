"""Pins the oracle's (and the product's host-side) layout arithmetic to values produced by the
reference's own classes (tests/golden/reference_goldens.json, written by
tests/golden/make_reference_goldens.py) and, when the reference probe is built, to the probe
directly on fresh random inputs."""
import ctypes as C
import json
import os
import random
import subprocess

import pytest

import mlakv_ffi as ffi
import oracle_ffi as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "oracle", "_ref", "ref_kv_probe")


def test_align_up_and_divide_up_closed_forms(oracle):
    for align in (1, 2, 16, 512, 4096):
        for value in list(range(0, 3 * align + 2)) + [10 ** 9 + 7]:
            assert oracle.kvo_align_up(value, align) == -(-value // align) * align
    for divisor in (1, 3, 64, 128):
        for value in range(0, 4 * divisor + 1):
            assert oracle.kvo_divide_up(value, divisor) == -(-value // divisor)


def test_ledger_goldens_sizes_and_blocks(oracle, goldens):
    assert len(goldens["ledger"]) >= 9
    for entry in goldens["ledger"]:
        bs, ctx = entry["block_size"], entry["max_context"]
        assert oracle.kvo_num_blocks(ctx, bs) == entry["num_blocks"]
        assert ffi.load().mlakvNumBlocks(ctx, bs) == entry["num_blocks"]
        sizes = orc.KvReservationBytes()
        oracle.kvo_kv_reservation_bytes(43, 1, entry["num_blocks"], bs, 512, 64, C.byref(sizes))
        assert sizes.block_table == entry["kv"]["kv.block_table"]["bytes"]
        assert sizes.slot_mapping == entry["kv"]["kv.slot_mapping"]["bytes"]
        assert sizes.latent_cache == entry["kv"]["kv.latent_cache"]["bytes"]
        assert sizes.rope_cache == entry["kv"]["kv.rope_cache"]["bytes"]
        assert oracle.kvo_backbone_device_bytes(512, 64, bs, ctx) == entry["backbone_device_bytes"]
        assert ffi.load().mlakvBackboneDeviceBytes(512, 64, bs, ctx) == entry["backbone_device_bytes"]
        assert entry["total_blocks_allocated"] == entry["num_blocks"] * 43
    # values the reference records from its own dry runs (docs/examples/inference_diagnostics_dry_run.json and the arena ledger)
    by_key = {(e["block_size"], e["max_context"]): e for e in goldens["ledger"]}
    assert by_key[(64, 8192)]["kv"]["kv.latent_cache"]["bytes"] == 360710144
    assert by_key[(64, 8192)]["kv"]["kv.rope_cache"]["bytes"] == 45088768
    assert by_key[(64, 8192)]["backbone_device_bytes"] == 11444004864
    assert by_key[(64, 8192)]["total_blocks_allocated"] == 5504
    assert by_key[(128, 8192)]["total_blocks_allocated"] == 2752  # docs/examples/inference_diagnostics_dry_run.json
    assert by_key[(128, 256)]["total_blocks_allocated"] == 86     # tests/mock_pipeline_e2e.cpp:615-618
    assert by_key[(64, 2000)]["num_blocks"] == 32 and by_key[(64, 32768)]["total_blocks_allocated"] == 22016


def test_product_reservations_match_reference_lengths(goldens):
    """One sequence, bf16, two planes: the KV cache manager's reservations have the reference's
    names' sizes, are 512-aligned and laid out in request order."""
    for entry in goldens["ledger"]:
        bs, ctx = entry["block_size"], entry["max_context"]
        if ctx * 43 * 576 * 2 > 1 << 30:
            continue  # host backend really allocates; keep to small arenas
        arena = ffi.Arena(ffi.BACKEND_HOST)
        cache = ffi.KvCache(arena, num_layers=43, block_size=bs, max_context_len=ctx, max_batch=1)
        assert cache.num_blocks == entry["num_blocks"] and cache.pool_blocks == entry["num_blocks"]
        names = {0: "kv.block_table", 1: "kv.slot_mapping", 5: "kv.latent_cache", 6: "kv.rope_cache"}
        for handle, name in names.items():
            assert arena.nbytes(handle) == entry["kv"][name]["bytes"], name
            assert arena.offset(handle) % 512 == 0
        offsets = [arena.offset(h) for h in range(arena.count)]
        assert offsets == sorted(offsets)
        assert "kv.latent_cache" in arena.ledger() and "kv.block_table" in arena.ledger()
        cache.close()
        arena.close()


def _replay_oracle(oracle, script):
    arena = oracle.kvo_arena_new()
    steps = []
    for nbytes, align in script:
        handle = C.c_size_t()
        status = oracle.kvo_arena_reserve(arena, b"probe", nbytes, align, C.byref(handle))
        if status != orc.OK:
            steps.append({"refused": True})
        else:
            offset = C.c_size_t()
            oracle.kvo_arena_offset(arena, handle.value, C.byref(offset))
            steps.append({"refused": False, "handle": handle.value, "offset": offset.value})
    commit_refused = oracle.kvo_arena_commit(arena, 4096 * 7) != orc.OK
    out = {"steps": steps, "commit_refused": commit_refused, "reserved_bytes": oracle.kvo_arena_reserved_bytes(arena),
           "arena_bytes": oracle.kvo_arena_total_bytes(arena), "device_allocations": oracle.kvo_arena_allocations(arena)}
    oracle.kvo_arena_delete(arena)
    return out


def _replay_product(script):
    arena = ffi.Arena(ffi.BACKEND_HOST)
    steps = []
    for nbytes, align in script:
        try:
            handle = arena.reserve("probe", nbytes, align)
            steps.append({"refused": False, "handle": handle, "offset": arena.offset(handle)})
        except ffi.MlakvError as error:
            assert error.status == ffi.ERR_CONTRACT
            steps.append({"refused": True})
    commit_refused = False
    try:
        arena.commit()
    except ffi.MlakvError:
        commit_refused = True
    out = {"steps": steps, "commit_refused": commit_refused, "reserved_bytes": arena.reserved_bytes,
           "arena_bytes": arena.total_bytes, "device_allocations": arena.device_allocations}
    if not commit_refused:
        arena.validate()
        assert arena.address(0) % 4096 == 0
    arena.close()
    return out


def _comparable(result):
    return {k: result[k] for k in ("steps", "commit_refused", "reserved_bytes", "arena_bytes", "device_allocations")}


def test_arena_scripts_match_reference(oracle, goldens):
    assert len(goldens["arena_scripts"]) >= 20
    refused_seen = False
    for case in goldens["arena_scripts"]:
        script = [tuple(step) for step in case["script"]]
        expected = _comparable(case["result"])
        refused_seen |= any(step["refused"] for step in expected["steps"])
        assert _replay_oracle(oracle, script) == expected
        assert _replay_product(script) == expected
    assert refused_seen


@pytest.mark.skipif(not os.path.exists(PROBE), reason="reference probe not built (needs /root/reference)")
def test_arena_scripts_against_live_reference_probe(oracle):
    rng = random.Random(7)
    for _ in range(12):
        script = [(rng.randint(0, 9000), rng.choice([0, 1, 3, 8, 64, 512, 4096, 5000])) for _ in range(rng.randint(1, 10))]
        out = subprocess.run([PROBE, "arena-script", str(len(script)), *[f"{b},{a}" for b, a in script]], check=True,
                             capture_output=True, text=True).stdout
        expected = _comparable(json.loads(out))
        assert _replay_oracle(oracle, script) == expected
        assert _replay_product(script) == expected


def test_arena_phase_contract_matches_reference_test(oracle, goldens):
    """The calls of the reference's TestStaticArena (tests/mock_contract_smoke.cpp:533-584), on the
    oracle arena and on the product arena (host backend), against the reference's outcomes."""
    expected = goldens["arena_contract"]
    assert expected["offsets"] == [0, 4096, 8192] and expected["arena_bytes"] == 8704

    # oracle
    a = oracle.kvo_arena_new()
    handles = [C.c_size_t() for _ in range(3)]
    assert oracle.kvo_arena_reserve(a, b"a.small", 100, 512, C.byref(handles[0])) == orc.OK
    assert oracle.kvo_arena_reserve(a, b"b.aligned", 4096, 4096, C.byref(handles[1])) == orc.OK
    assert oracle.kvo_arena_reserve(a, b"c.tail", 7, 512, C.byref(handles[2])) == orc.OK
    address = C.c_size_t()
    got = {}
    got["address_before_commit_refused"] = int(oracle.kvo_arena_address(a, 0, C.byref(address)) != orc.OK)
    got["zero_byte_refused"] = int(oracle.kvo_arena_reserve(a, b"d.zero", 0, 512, None) != orc.OK)
    got["odd_align_refused"] = int(oracle.kvo_arena_reserve(a, b"e.odd", 64, 3, None) != orc.OK)
    assert oracle.kvo_arena_commit(a, 1 << 20) == orc.OK
    got["allocations_after_commit"] = oracle.kvo_arena_allocations(a)
    offsets = []
    for h in handles:
        off = C.c_size_t()
        oracle.kvo_arena_offset(a, h.value, C.byref(off))
        offsets.append(off.value)
    got["offsets"] = offsets
    got["arena_bytes"] = oracle.kvo_arena_total_bytes(a)
    oracle.kvo_arena_address(a, 1, C.byref(address))
    got["second_abs_mod_4096"] = address.value % 4096
    got["late_reserve_refused"] = int(oracle.kvo_arena_reserve(a, b"f.late", 8, 512, None) != orc.OK)
    for ws in (1024, 4096, 2048):
        assert oracle.kvo_arena_note_workspace(a, ws) == orc.OK
    assert oracle.kvo_arena_commit_workspace(a) == orc.OK
    got["workspace_bytes"] = oracle.kvo_arena_workspace_bytes(a)
    got["fits_4096_refused"] = int(oracle.kvo_arena_workspace_fits(a, 4096) != orc.OK)
    got["fits_4097_refused"] = int(oracle.kvo_arena_workspace_fits(a, 4097) != orc.OK)
    got["allocations_after_workspace"] = oracle.kvo_arena_allocations(a)
    assert oracle.kvo_arena_seal(a) == orc.OK
    got["sealed"] = oracle.kvo_arena_sealed(a)
    got["sealed_reserve_refused"] = int(oracle.kvo_arena_reserve(a, b"g.sealed", 8, 512, None) != orc.OK)
    got["sealed_workspace_refused"] = int(oracle.kvo_arena_commit_workspace(a) != orc.OK)
    oracle.kvo_arena_delete(a)
    for key, value in got.items():
        assert value == expected[key], key

    # product
    def refused(fn):
        try:
            fn()
        except ffi.MlakvError as error:
            assert error.status == ffi.ERR_CONTRACT, error
            return 1
        return 0

    p = ffi.Arena(ffi.BACKEND_HOST)
    first = p.reserve("a.small", 100)
    second = p.reserve("b.aligned", 4096, 4096)
    third = p.reserve("c.tail", 7)
    got = {}
    got["address_before_commit_refused"] = refused(lambda: p.address(first))
    got["zero_byte_refused"] = refused(lambda: p.reserve("d.zero", 0))
    got["odd_align_refused"] = refused(lambda: p.reserve("e.odd-align", 64, 3))
    p.commit()
    got["allocations_after_commit"] = p.device_allocations
    got["offsets"] = [p.offset(first), p.offset(second), p.offset(third)]
    got["arena_bytes"] = p.total_bytes
    got["second_abs_mod_4096"] = p.address(second) % 4096
    assert p.address(third) > p.address(first)
    p.validate()
    got["late_reserve_refused"] = refused(lambda: p.reserve("f.late", 8))
    for ws in (1024, 4096, 2048):
        p.note_workspace(ws)
    p.commit_workspace()
    got["workspace_bytes"] = p.workspace_bytes
    got["fits_4096_refused"] = refused(lambda: p.assert_workspace_fits(4096, "test"))
    got["fits_4097_refused"] = refused(lambda: p.assert_workspace_fits(4097, "test"))
    got["allocations_after_workspace"] = p.device_allocations
    p.seal()
    got["sealed"] = int(p.sealed)
    got["sealed_reserve_refused"] = refused(lambda: p.reserve("g.sealed", 8))
    got["sealed_workspace_refused"] = refused(lambda: p.commit_workspace())
    assert refused(lambda: p.note_workspace(1)) == 1
    assert "SEALED" in p.ledger()
    p.close()
    for key, value in got.items():
        assert value == expected[key], key


def test_kv_diagnostics_goldens(oracle, goldens):
    for case in goldens["stats"]:
        bs, ctx, position = case["block_size"], case["max_context"], case["position"]
        expected = case["result"]
        if expected["refused"]:
            assert oracle.kvo_num_blocks(ctx, bs) == -1
            assert ffi.load().mlakvNumBlocks(ctx, bs) == -1
            arena = ffi.Arena(ffi.BACKEND_HOST)
            with pytest.raises(ffi.MlakvError):
                ffi.KvCache(arena, num_layers=43, block_size=bs, max_context_len=ctx)
            arena.close()
            continue
        blocks = oracle.kvo_num_blocks(ctx, bs)
        stats = orc.KvStats()
        oracle.kvo_kv_stats(43, blocks, bs, position, C.byref(stats))
        assert stats.total_blocks_allocated == expected["total_blocks_allocated"]
        assert stats.active_context_tokens == expected["active_context_tokens"]
        assert stats.kv_cache_utilization == expected["kv_cache_utilization"]
        # product: one sequence with identity paging, `position + 1` decode steps; only the
        # bookkeeping runs (nothing is committed, so no memory is allocated)
        arena = ffi.Arena(ffi.BACKEND_HOST)
        cache = ffi.KvCache(arena, num_layers=43, block_size=bs, max_context_len=ctx, max_batch=1)
        cache.add_sequence(0, 0)
        for step in range(position + 1):
            assert cache.append_token(0) == step  # slot = position, reference pipeline.cpp:517
        got = cache.stats()
        assert got.total_blocks_allocated == expected["total_blocks_allocated"]
        assert got.active_context_tokens == expected["active_context_tokens"]
        assert got.kv_cache_utilization == expected["kv_cache_utilization"]
        assert got.block_size == bs
        cache.close()
        arena.close()
    utilisations = {(c["block_size"], c["max_context"], c["position"]): c["result"].get("kv_cache_utilization")
                    for c in goldens["stats"]}
    assert utilisations[(128, 256, 1)] == 2.0 / 256.0            # tests/mock_pipeline_e2e.cpp:663-666
    assert utilisations[(64, 8192, 128)] == 0.0157470703125      # docs/preflight-verification.md:42-45
    assert utilisations[(64, 8192, 127)] == 0.015625


# The "paged_attention" member of the reference's sample diagnostics file, as it stands there
# (docs/examples/inference_diagnostics_dry_run.json:19-24: 43 layers, block 128, context 8192,
# nothing decoded yet).
_DRY_RUN_PAGED_ATTENTION = (
    '  "paged_attention": {\n'
    '    "total_blocks_allocated": 2752,\n'
    '    "active_context_tokens": 0,\n'
    '    "block_size": 128,\n'
    '    "kv_cache_utilization": 0\n'
    '  }'
)


def test_diag_json_paged_attention_block_matches_the_reference_sample_byte_for_byte():
    lib = ffi.load()
    arena = ffi.Arena(ffi.BACKEND_HOST)
    cache = ffi.KvCache(arena, num_layers=43, block_size=128, max_context_len=8192, max_batch=1)
    stats = cache.stats()
    needed = lib.mlakvKvStatsFormatJson(C.byref(stats), None, 0)
    assert needed == len(_DRY_RUN_PAGED_ATTENTION)
    buffer = C.create_string_buffer(needed + 1)
    assert lib.mlakvKvStatsFormatJson(C.byref(stats), buffer, needed + 1) == needed
    assert buffer.value.decode() == _DRY_RUN_PAGED_ATTENTION
    # spliced into a document it parses, and a truncating buffer is never overrun
    import json
    assert json.loads("{\n" + buffer.value.decode() + "\n}")["paged_attention"]["total_blocks_allocated"] == 2752
    small = C.create_string_buffer(b"\xff" * 16, 16)
    assert lib.mlakvKvStatsFormatJson(C.byref(stats), small, 8) == needed
    assert small.raw[7:8] == b"\x00" and small.raw[8:] == b"\xff" * 8
    # 12 significant digits as an ostream at precision 12 prints them (docs/preflight-verification.md:42-45
    # quotes 0.0157470703125 for 129 tokens of 8192), and null for a non-finite value
    cache.add_sequence(0, 0)
    for _ in range(129):
        cache.append_token(0)
    cache.close()
    arena.close()
    arena = ffi.Arena(ffi.BACKEND_HOST)
    cache = ffi.KvCache(arena, num_layers=43, block_size=64, max_context_len=8192, max_batch=1)
    cache.add_sequence(0, 0)
    for _ in range(129):
        cache.append_token(0)
    stats = cache.stats()
    buffer = C.create_string_buffer(256)
    lib.mlakvKvStatsFormatJson(C.byref(stats), buffer, 256)
    assert '"kv_cache_utilization": 0.0157470703125\n' in buffer.value.decode()
    assert '"active_context_tokens": 129,' in buffer.value.decode()
    stats.kv_cache_utilization = float("nan")
    lib.mlakvKvStatsFormatJson(C.byref(stats), buffer, 256)
    assert '"kv_cache_utilization": null\n' in buffer.value.decode()
    stats.kv_cache_utilization = 1.0 / 3.0
    lib.mlakvKvStatsFormatJson(C.byref(stats), buffer, 256)
    assert '"kv_cache_utilization": 0.333333333333\n' in buffer.value.decode()
    assert lib.mlakvKvStatsFormatJson(None, buffer, 256) == -1
    cache.close()
    arena.close()
