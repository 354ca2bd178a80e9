"""GPU parity: absorbed-MLA decode attention through the C ABI against the CPU oracle
(float64 accumulation). Tolerance, from the target statement: 2e-2 relative for bf16 KV,
6e-2 for FP8 KV, measured as max|gpu - oracle| / max|oracle| per test and element-wise as
|gpu - oracle| <= tol * (|oracle| + max|oracle|)."""
import math

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE
SCALE = 1.0 / math.sqrt(192.0)  # 1/sqrt(qk_nope + qk_rope), reference pipeline.cpp:238
TOL_BF16, TOL_FP8 = 2e-2, 6e-2


def _fill_cache(cache, ctxs, table, seed, outliers=0.0):
    total = sum(ctxs)
    latent_src = kt.randn_bf16((cache.layers, total, LATENT), seed=seed, outlier_fraction=outliers).cuda()
    rope_src = kt.randn_bf16((cache.layers, total, ROPE), seed=seed + 1, outlier_fraction=outliers).cuda()
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(table, ctxs, cache.block_size)))
    torch.cuda.synchronize()
    return latent_src, rope_src


def _assert_close(got_bf16, expected_f32, tol):
    got = got_bf16.float().cpu().numpy()
    assert np.isfinite(got).all()
    peak = np.abs(expected_f32).max()
    err = np.abs(got - expected_f32)
    assert err.max() <= tol * peak, f"max err {err.max():.4g} vs {tol} * {peak:.4g}"
    assert (err <= tol * (np.abs(expected_f32) + peak)).all()
    return err.max() / peak


@pytest.mark.parametrize("bs", [16, 64, 128])
@pytest.mark.parametrize("heads", [16, 64, 128])
def test_attention_matches_oracle_ragged(bs, heads):
    ctxs = [1, 63, 64, 65, 200, 333]
    blocks = sum(-(-c // bs) for c in ctxs) + 4
    pool = kt.build_tables(ctxs, bs, blocks, seed=31)
    table = pool.table()
    cache = kt.PagedCache(2, blocks, bs)
    _fill_cache(cache, ctxs, table, seed=40)
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=50).cuda()
    expected, expected_lse = kt.oracle_attention(cache, 1, q, table, ctxs, SCALE)
    # the planner's choice; units of one tile (every sequence split, several units per workgroup
    # when there are fewer workgroups than units); two tiles; units that each hold whole sequences
    # (written without partials); then the merge inside the launch: contributors that wait for each
    # other, a merge that never waits (the contributor that arrives last does all of it), a wait
    # that mostly gives up (two workgroups take turns over many units)
    in_launch = ffi.ATTN_MERGE_IN_LAUNCH
    for options in ({}, {"chunk_tiles": 1}, {"chunk_tiles": 1, "work_groups": 3}, {"chunk_tiles": 2}, {"chunk_tiles": 100},
                    {"chunk_tiles": 1, "merge_mode": in_launch}, {"merge_mode": in_launch},
                    {"chunk_tiles": 2, "merge_mode": in_launch, "merge_spin_us": -1},
                    {"chunk_tiles": 1, "work_groups": 3, "merge_mode": in_launch},
                    {"chunk_tiles": 3, "work_groups": 2, "merge_mode": in_launch, "merge_spin_us": 1}):
        out, lse, plan = kt.attention(cache, 1, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE, **options)
        _assert_close(out, expected, TOL_BF16)
        assert np.abs(lse.cpu().numpy() - expected_lse).max() <= 2e-2, options


def test_attention_special_cases():
    bs, heads = 64, 64
    # (a) context of one token: softmax is 1, output is exactly that latent row
    # (b) all rows identical: output equals the row
    # (c) one dominant score: output tends to that row
    ctxs = [1, 150, 130]
    blocks = 8
    pool = kt.build_tables(ctxs, bs, blocks, seed=3)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    total = sum(ctxs)
    latent = kt.randn_bf16((1, total, LATENT), seed=60)
    rope = kt.randn_bf16((1, total, ROPE), seed=61)
    latent[0, 1:151] = latent[0, 1]
    rope[0, 1:151] = rope[0, 1]
    q = kt.randn_bf16((3, heads, LATENT + ROPE), seed=62)
    # sequence 2: make token 17 dominate for every head by aligning it with +-q is impossible for all
    # heads at once, so use a shared query for all heads and a row parallel to it.
    q[2, :, :] = q[2, 0, :]
    base = 151
    latent[0, base + 17] = (q[2, 0, :LATENT].float() * 4).to(torch.bfloat16)
    rope[0, base + 17] = (q[2, 0, LATENT:].float() * 4).to(torch.bfloat16)
    latent, rope = latent.cuda(), rope.cuda()
    kt.append(cache, latent, rope, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    out, lse, _ = kt.attention(cache, 0, q.cuda(), kt.dev_i32(table), kt.dev_i32(ctxs), SCALE)
    assert torch.equal(out[0], latent[0, 0].expand(heads, LATENT))  # (a) exact
    assert torch.allclose(out[1].float(), latent[0, 1].float().expand(heads, LATENT), rtol=2 ** -7, atol=1e-6)  # (b)
    dominant = latent[0, base + 17].float()
    assert (out[2].float() - dominant).abs().max() <= 2e-2 * dominant.abs().max()  # (c)
    expected, _ = kt.oracle_attention(cache, 0, q.cuda(), table, ctxs, SCALE)
    _assert_close(out, expected, TOL_BF16)


def test_attention_invariant_under_physical_block_permutation():
    bs, heads = 64, 64
    ctxs = [257, 100]
    blocks = 12
    outs = []
    for seed in (1, 2):
        pool = kt.build_tables(ctxs, bs, blocks, seed=seed)
        table = pool.table()
        cache = kt.PagedCache(1, blocks, bs)
        _fill_cache(cache, ctxs, table, seed=70)
        q = kt.randn_bf16((2, heads, LATENT + ROPE), seed=71).cuda()
        out, lse, _ = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE)
        outs.append((out, lse, table))
    assert not np.array_equal(outs[0][2], outs[1][2])
    assert torch.equal(outs[0][0], outs[1][0])  # same logical order -> bitwise identical
    assert torch.equal(outs[0][1], outs[1][1])


def test_attention_empty_sequence_gives_zeros():
    bs, heads = 64, 64
    ctxs = [0, 70, 0]
    blocks = 4
    pool = kt.build_tables(ctxs, bs, blocks, seed=4)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    _fill_cache(cache, ctxs, table, seed=80)
    q = kt.randn_bf16((3, heads, LATENT + ROPE), seed=81).cuda()
    for chunk_tiles in (1, 100):
        out, lse, _ = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE, max_seq_len=128, chunk_tiles=chunk_tiles)
        assert (out[0] == 0).all() and (out[2] == 0).all()
        assert torch.isinf(lse[0]).all() and (lse[0] < 0).all()
        expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE)
        _assert_close(out, expected, TOL_BF16)


@pytest.mark.parametrize("bs", [16, 64])
def test_attention_fp8_kv_matches_oracle(bs):
    heads = 64
    ctxs = [5, 64, 129, 700]
    blocks = sum(-(-c // bs) for c in ctxs) + 2
    pool = kt.build_tables(ctxs, bs, blocks, seed=9)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs, fp8=True)
    _fill_cache(cache, ctxs, table, seed=90, outliers=0.01)
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=91).cuda()
    out, lse, _ = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE)
    expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE)
    _assert_close(out, expected, TOL_FP8)
    assert np.abs(lse.cpu().numpy() - expected_lse).max() <= 6e-2


def test_config3_full_size_against_oracle_sample_and_torch():
    """BASELINE config 3: batch 32, 64 heads, context 2048, block 64, shuffled table. Every
    sequence is checked against a float32 torch evaluation of the same formula on the GPU
    (library routine); four sequences are checked against the float64 oracle."""
    batch, heads, ctx, bs = 32, 64, 2048, 64
    ctxs = [ctx] * batch
    blocks = batch * (ctx // bs) + 16
    pool = kt.build_tables(ctxs, bs, blocks, seed=77)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    gen = torch.Generator(device="cuda").manual_seed(3)
    latent_src = torch.randn(1, batch * ctx, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
    rope_src = torch.randn(1, batch * ctx, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    q = torch.randn(batch, heads, LATENT + ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    out, lse, plan = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE)
    k = torch.cat([latent_src[0], rope_src[0]], dim=-1).float().view(batch, ctx, LATENT + ROPE)
    v = latent_src[0].float().view(batch, ctx, LATENT)
    scores = torch.einsum("bhd,btd->bht", q.float(), k) * SCALE
    ref = torch.einsum("bht,btd->bhd", torch.softmax(scores, dim=-1), v)
    peak = ref.abs().max().item()
    assert (out.float() - ref).abs().max().item() <= TOL_BF16 * peak
    assert (lse - torch.logsumexp(scores, dim=-1)).abs().max().item() <= 2e-2
    sample = [0, 7, 19, 31]
    expected, _ = kt.oracle_attention(cache, 0, q[sample], table[sample], [ctx] * len(sample), SCALE)
    _assert_close(out[sample], expected, TOL_BF16)


@pytest.mark.parametrize("fp8", [False, True])
def test_maximum_context_single_sequence_many_chunks(fp8):
    """BASELINE's largest context (32768 tokens) for one sequence: the launch cuts it into one unit per
    CU, so the merge runs over many groups of partials. The whole sequence is checked
    against a float32 torch evaluation on the GPU (library routine), 16 heads of it against the
    float64 oracle; a second, short sequence in the same batch shares the last unit."""
    heads, bs = 64, 128
    ctxs = [32768, 200]
    blocks = sum(-(-c // bs) for c in ctxs) + 8
    pool = kt.build_tables(ctxs, bs, blocks, seed=5)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
    gen = torch.Generator(device="cuda").manual_seed(9)
    total = sum(ctxs)
    latent_src = torch.randn(1, total, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
    rope_src = torch.randn(1, total, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    q = torch.randn(len(ctxs), heads, LATENT + ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    out, lse, plan = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE)
    assert plan.work_groups >= 64  # the long sequence is cut over (nearly) all of them
    tol = TOL_FP8 if fp8 else TOL_BF16
    if fp8:  # compare against the values the cache really holds
        lat_rows, rope_rows = kt.gather(cache, kt.dev_i32(table), kt.dev_i32(ctxs))
        lat_rows, rope_rows = lat_rows[0].float(), rope_rows[0].float()
    else:
        lat_rows, rope_rows = latent_src[0].float(), rope_src[0].float()
    start = 0
    for b, n in enumerate(ctxs):
        k = torch.cat([lat_rows[start:start + n], rope_rows[start:start + n]], dim=-1)
        scores = (q[b].float() @ k.T) * SCALE
        ref = torch.softmax(scores, dim=-1) @ lat_rows[start:start + n]
        peak = ref.abs().max().item()
        assert (out[b].float() - ref).abs().max().item() <= tol * peak, (b, n)
        assert (lse[b] - torch.logsumexp(scores, dim=-1)).abs().max().item() <= 2e-2
        start += n
    if not fp8:
        expected, _ = kt.oracle_attention(cache, 0, q[:1, :16].contiguous(), table[:1], ctxs[:1], SCALE)
        _assert_close(out[:1, :16], expected, TOL_BF16)


@pytest.mark.parametrize("fp8", [False, True])
def test_short_whole_contexts_in_units_of_16_heads(fp8):
    """A whole-context launch whose longest context the launch can see is short takes the units of
    the selected-token attention (no selection: every position of the sequence): asked for by the
    plan, chosen by the default plan from its own bound, and chosen by a launch with host-known
    lengths under a plan made for long contexts. Against the oracle, against the 64-head kernel, and
    the quantising entry point (which keeps the 64-head kernel) against its own bf16 output."""
    import ctypes as C
    lib = ffi.load()
    bs, heads = 64, 64
    tol = TOL_FP8 if fp8 else TOL_BF16
    for ctxs in ([1, 0, 250, 64, 33, 256, 65, 129], [300, 512, 1, 0, 97], [1000, 1024, 3]):
        blocks = sum(-(-c // bs) for c in ctxs) + 4
        table = kt.build_tables(ctxs, bs, blocks, seed=91, max_blocks=2048 // bs).table()   # rows wide enough for a 2048-token plan
        cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
        _fill_cache(cache, ctxs, table, seed=92, outliers=0.01 if fp8 else 0.0)
        q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=93).cuda()
        tab, lens = kt.dev_i32(table), kt.dev_i32(ctxs)
        expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE)
        live = np.array(ctxs) > 0
        split, split_lse, plan = kt.attention(cache, 0, q, tab, lens, SCALE, selection_units=ffi.ATTN_UNITS_SPLIT)
        assert plan.selection_units == ffi.ATTN_UNITS_SPLIT
        _assert_close(split, expected, tol)
        peak = np.abs(expected).max()
        for units in (ffi.ATTN_UNITS_AUTO, ffi.ATTN_UNITS_HEAD_BLOCK, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES):
            out, lse, plan = kt.attention(cache, 0, q, tab, lens, SCALE, selection_units=units)
            assert plan.selection_units == units
            _assert_close(out, expected, tol)
            assert np.abs(lse.cpu().numpy()[live] - expected_lse[live]).max() <= tol
            assert not out[~torch.from_numpy(live).cuda()].any() and torch.isneginf(lse[~torch.from_numpy(live).cuda()]).all()
            assert (out.float() - split.float()).abs().max().item() <= 2 ** -5 * peak
            if units != ffi.ATTN_UNITS_AUTO or max(ctxs) <= 768:   # the units ran: not the 64-head kernel's bits
                assert not torch.equal(out, split)
            else:
                assert torch.equal(out, split)
        # a plan for long contexts, the lengths by value: the launch sees that they are short
        long_plan = kt.make_plan(len(ctxs), heads, 2048, bs, fp8)
        ws = torch.empty(int(long_plan.workspace_bytes), dtype=torch.uint8, device="cuda")
        by_value, by_value_lse = torch.full_like(split, float("nan")), torch.full_like(split_lse, float("nan"))
        in_memory = torch.full_like(split, float("nan"))
        host = (C.c_int32 * len(ctxs))(*ctxs)
        row = (LATENT + ROPE) * 2
        head_args = (C.byref(long_plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row, q.data_ptr() + LATENT * 2, heads * row, row,
                     tab.data_ptr(), tab.shape[1])
        ffi.check(lib.mlakvAttnDecodeHostLens(*head_args, C.cast(host, C.c_void_p), SCALE, by_value.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                              by_value_lse.data_ptr(), ws.data_ptr(), ws.numel(), kt.stream_ptr()))
        ffi.check(lib.mlakvAttnDecode(*head_args, lens.data_ptr(), SCALE, in_memory.data_ptr(), heads * LATENT * 2, LATENT * 2, None,
                                      ws.data_ptr(), ws.numel(), kt.stream_ptr()))
        # the lengths in device memory and the caller's word for their bound: as by value
        bounded = torch.full_like(split, float("nan"))
        ffi.check(lib.mlakvAttnDecodeBounded(*head_args, lens.data_ptr(), max(ctxs), SCALE, bounded.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                             None, ws.data_ptr(), ws.numel(), kt.stream_ptr()))
        torch.cuda.synchronize()
        assert torch.equal(bounded, by_value)
        _assert_close(by_value, expected, tol)
        _assert_close(in_memory, expected, tol)
        assert torch.equal(in_memory, split)                       # lengths in device memory: the plan's bound decides
        assert torch.equal(by_value, split) == (max(ctxs) > 768)   # by value: the lengths themselves
        # the quantising entry point makes the same choice and quantises the units' bf16 rows (held in
        # the workspace when the caller wants no bf16 output) with the standalone quantiser
        plain, _, _ = kt.attention(cache, 0, q, tab, lens, SCALE)
        _, _, _, codes, scales = kt.attention(cache, 0, q, tab, lens, SCALE, quant=True, want_out=False)
        with_out, _, _, codes_too, scales_too = kt.attention(cache, 0, q, tab, lens, SCALE, quant=True)
        want_codes, want_scales = orc.mx_quant_rows(kt.bits16(plain).reshape(-1, LATENT))
        assert torch.equal(with_out, plain)
        for got_codes, got_scales in ((codes, scales), (codes_too, scales_too)):
            assert np.array_equal(got_scales.cpu().numpy().reshape(-1, LATENT // 32), want_scales)
            assert np.array_equal(got_codes.cpu().numpy().reshape(-1, LATENT), want_codes)


def test_host_lengths_in_the_argument_block_give_the_same_bits():
    """mlakvAttnDecodeHostLens against mlakvAttnDecode with the same lengths in device memory: the
    kernels only read the lengths from another place, so every output bit agrees; split and
    unsplit sequences, an empty one, bf16 and FP8; more than 64 sequences are refused."""
    import ctypes as C
    lib = ffi.load()
    # the second list leaves every sequence inside one work unit: with the lengths on the host the
    # launcher sees that and does not launch the merge at all
    for fp8, ctxs in ((False, [1, 0, 700, 64, 333, 2048, 65]), (True, [1, 0, 700, 64, 333, 2048, 65]),
                      (False, [100, 0, 128, 64, 1]), (True, [100, 0, 128, 64, 1])):
        bs, heads = 64, 64
        blocks = sum(-(-c // bs) for c in ctxs) + 4
        pool = kt.build_tables(ctxs, bs, blocks, seed=77)
        table = pool.table()
        cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
        _fill_cache(cache, ctxs, table, seed=78, outliers=0.01 if fp8 else 0.0)
        q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=79).cuda()
        tab = kt.dev_i32(table)
        for options in ({}, {"chunk_tiles": 1}, {"chunk_tiles": 3, "merge_mode": ffi.ATTN_MERGE_IN_LAUNCH}):
            want, want_lse, plan = kt.attention(cache, 0, q, tab, kt.dev_i32(ctxs), SCALE, **options)
            ws = torch.empty(int(plan.workspace_bytes), dtype=torch.uint8, device="cuda")
            out = torch.full_like(want, float("nan"))
            lse = torch.full_like(want_lse, float("nan"))
            host = (C.c_int32 * len(ctxs))(*ctxs)
            row = (LATENT + ROPE) * 2
            ffi.check(lib.mlakvAttnDecodeHostLens(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                                  q.data_ptr() + LATENT * 2, heads * row, row, tab.data_ptr(), tab.shape[1],
                                                  C.cast(host, C.c_void_p), SCALE, out.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                                  lse.data_ptr(), ws.data_ptr(), ws.numel(), kt.stream_ptr()))
            host[2] = 5  # the values were copied: changing the buffer after the call changes nothing
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), (fp8, options)
            assert torch.equal(lse, want_lse)
    many = kt.make_plan(65, 64, 64, 64, False)
    assert lib.mlakvAttnDecodeHostLens(C.byref(many), C.byref(cache.view), 0, q.data_ptr(), 1, 1, q.data_ptr(), 1, 1, tab.data_ptr(), 1,
                                       C.cast(host, C.c_void_p), SCALE, out.data_ptr(), 1, 1, None, ws.data_ptr(), ws.numel(),
                                       None) == ffi.ERR_PARAM_INVALID


@pytest.mark.parametrize("seed", range(10))
def test_attention_on_drawn_shapes(seed):
    """Shapes, block sizes (multiples of the 32-token tile and not), cache types, plan options and a
    selection drawn from a seeded generator: dense and selected-token attention against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    bs = int(rng.choice([16, 24, 32, 48, 64, 96, 128]))
    heads = int(rng.choice([16, 32, 48, 64, 80, 128]))
    fp8 = bool(rng.integers(0, 2))
    batch = int(rng.integers(1, 13))
    ctxs = [int(v) for v in rng.integers(0, 600, size=batch)]
    if batch > 2:
        ctxs[int(rng.integers(0, batch))] = 0          # an empty sequence among the others
    ctxs[int(rng.integers(0, batch))] = int(rng.integers(600, 1400))  # and a long one
    blocks = sum(-(-c // bs) for c in ctxs) + 5
    table = kt.build_tables(ctxs, bs, blocks, seed=seed).table()
    cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
    _fill_cache(cache, ctxs, table, seed=2000 + seed, outliers=0.01 if fp8 else 0.0)
    q = kt.randn_bf16((batch, heads, LATENT + ROPE), seed=3000 + seed).cuda()
    tol = TOL_FP8 if fp8 else TOL_BF16
    options = {}
    if rng.integers(0, 2):
        options["chunk_tiles"] = int(rng.choice([1, 2, 5, 40]))
    if rng.integers(0, 2):
        options["work_groups"] = int(rng.choice([1, 7, 300]))
    if rng.integers(0, 3) == 0:
        options["merge_mode"] = ffi.ATTN_MERGE_IN_LAUNCH
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE)
    out, lse, _ = kt.attention(cache, 0, q, table_d, lens_d, SCALE, **options)
    case = dict(bs=bs, heads=heads, fp8=fp8, ctxs=ctxs, options=options)
    live = np.array(ctxs) > 0
    assert np.abs(out.float().cpu().numpy()[~live]).max(initial=0.0) == 0.0, case   # nothing to attend to: zeros
    # the same launch with the lengths in the argument block (the merge is then only launched when
    # the host-side cut splits a sequence): the same bits
    import ctypes as C
    plan = kt.make_plan(batch, heads, max(max(ctxs), 1), bs, fp8, **options)
    ws = torch.empty(max(int(plan.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    out_h = torch.full_like(out, float("nan"))
    host = (C.c_int32 * batch)(*ctxs)
    row = (LATENT + ROPE) * 2
    ffi.check(ffi.load().mlakvAttnDecodeHostLens(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                                 q.data_ptr() + LATENT * 2, heads * row, row, table_d.data_ptr(), table_d.shape[1],
                                                 C.cast(host, C.c_void_p), SCALE, out_h.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                                 None, ws.data_ptr(), ws.numel(), kt.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out_h.view(torch.int16), out.view(torch.int16)), case
    _assert_close(out[torch.as_tensor(live)], expected[live], tol)
    assert np.abs(lse.cpu().numpy()[live] - expected_lse[live]).max() <= (6e-2 if fp8 else 2e-2), case
    # a selection of up to k positions per sequence, shorter lists ended by -1
    k = int(rng.choice([32, 100, 256]))
    selection = np.full((batch, k), -1, dtype=np.int32)
    for b, n in enumerate(ctxs):
        take = min(n, k, int(rng.integers(1, k + 1)))
        selection[b, :take] = rng.permutation(n)[:take]
    expected_s, _ = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=selection)
    out_s, _, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, kt.dev_i32(selection), SCALE)
    _assert_close(out_s[torch.as_tensor(live)], expected_s[live], tol)
