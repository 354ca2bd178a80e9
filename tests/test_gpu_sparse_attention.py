"""GPU parity: selected-token decode attention (mlakvAttnDecodeSparse) through the C ABI against
the CPU oracle (2e-2 of the peak for bf16 KV, 6e-2 for FP8 KV, as for the dense attention), and
through what the definition fixes: selecting every token reproduces the dense entry point,
permuting the selection changes nothing beyond rounding, the selection ends at its first invalid
entry, an empty selection gives zeros."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE
SCALE = 1.0 / math.sqrt(192.0)


def _setup(ctxs, bs, fp8, seed):
    blocks = sum(-(-c // bs) for c in ctxs) + 3
    pool = kt.build_tables(ctxs, bs, blocks, seed=seed)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
    total = sum(ctxs)
    latent = kt.randn_bf16((1, total, LATENT), seed=seed + 1, outlier_fraction=0.01).cuda()
    rope = kt.randn_bf16((1, total, ROPE), seed=seed + 2).cuda()
    kt.append(cache, latent, rope, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    torch.cuda.synchronize()
    return cache, table


def _close(got_bf16, expected, tol):
    got = got_bf16.float().cpu().numpy()
    assert np.isfinite(got).all()
    peak = max(np.abs(expected).max(), 1e-30)
    assert np.abs(got - expected).max() <= tol * peak, np.abs(got - expected).max() / peak


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("bs,k", [(64, 512), (16, 100), (128, 2048), (48, 200)])  # 48: slots packed behind six bits, not all used
def test_selected_tokens_match_oracle(fp8, bs, k):
    heads = 64
    ctxs = [3000, 700, 1, 0, 2049, 130]
    cache, table = _setup(ctxs, bs, fp8, seed=80)
    rng = np.random.default_rng(81)
    selection = np.full((len(ctxs), k), -1, dtype=np.int32)
    for s, n in enumerate(ctxs):
        take = min(n, k)
        if s == 1:
            take = min(n, k) // 2          # fewer than k although the context is long enough
        selection[s, :take] = rng.permutation(n)[:take]
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=82).cuda()
    expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=selection)
    table_d, lens_d, sel_d = kt.dev_i32(table), kt.dev_i32(ctxs), kt.dev_i32(selection)
    # what the default plan does with 24 units, far fewer than CUs: a whole selection for 16 heads up
    # to 256 selected tokens, two workgroups per unit from there to 768 (FP8: to the 1024 a unit can
    # stage), the split beyond
    default_units = (ffi.ATTN_UNITS_SPLIT if k > (1024 if fp8 else 768) else
                     ffi.ATTN_UNITS_HEAD_BLOCK_HALVES if k > 256 else ffi.ATTN_UNITS_HEAD_BLOCK)
    for options in ({}, {"chunk_tiles": 1}, {"chunk_tiles": 100}, {"chunk_tiles": 3, "merge_mode": 1},
                    {"selection_units": ffi.ATTN_UNITS_SPLIT}):
        out, lse, plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE, **options)
        assert plan.chunk_tiles * 32 <= 512  # a unit's selected tokens are staged in LDS, one entry each
        assert plan.selection_units == (ffi.ATTN_UNITS_SPLIT if options else default_units)
        _close(out, expected, 6e-2 if fp8 else 2e-2)
        live = np.array([min(n, k) > 0 for n in ctxs])
        assert np.abs(lse.cpu().numpy()[live] - expected_lse[live]).max() <= (6e-2 if fp8 else 2e-2)
        assert not out[3].any() and torch.isneginf(lse[3]).all()


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("batch,heads,bs,k", [(19, 128, 64, 1024), (8, 16, 16, 33), (3, 32, 48, 512), (9, 64, 128, 96)])
def test_whole_selection_units_of_16_heads(batch, heads, bs, k, fp8):
    """One workgroup per (sequence, 16 heads): selections of every length up to k (0, 1, multiples
    of the 32-token tile and one beside them), more sequences than one round over the XCDs, against
    the oracle and against the split units on the same inputs."""
    rng = np.random.default_rng(700 + batch)
    ctxs = [int(v) for v in rng.integers(1, 2 * k, size=batch)]
    takes = [int(v) for v in rng.integers(0, k + 1, size=batch)]
    takes[:4] = [k, 1, 32, 33][:min(4, batch)]
    if batch > 4:
        takes[4] = 0
    ctxs = [max(c, t) for c, t in zip(ctxs, takes)]
    cache, table = _setup(ctxs, bs, fp8, seed=70 + batch)
    tol = 6e-2 if fp8 else 2e-2
    selection = np.full((batch, k), -1, dtype=np.int32)
    for s, (n, take) in enumerate(zip(ctxs, takes)):
        selection[s, :take] = rng.permutation(n)[:take]
    q = kt.randn_bf16((batch, heads, LATENT + ROPE), seed=71 + batch).cuda()
    expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=selection)
    table_d, lens_d, sel_d = kt.dev_i32(table), kt.dev_i32(ctxs), kt.dev_i32(selection)
    out, lse, plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE, selection_units=ffi.ATTN_UNITS_HEAD_BLOCK)
    assert plan.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK
    _close(out, expected, tol)
    live = np.array(takes) > 0
    assert np.abs(lse.cpu().numpy()[live] - expected_lse[live]).max() <= tol
    assert not out[~torch.from_numpy(live).cuda()].any() and torch.isneginf(lse[~torch.from_numpy(live).cuda()]).all()
    split, split_lse, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE, selection_units=ffi.ATTN_UNITS_SPLIT)
    peak = np.abs(expected).max()
    assert (out.float() - split.float()).abs().max().item() <= 2 ** -6 * peak   # same tokens, same tiles; partials round to bf16 once more
    assert (lse[torch.from_numpy(live).cuda()] - split_lse[torch.from_numpy(live).cuda()]).abs().max().item() <= 1e-3
    # two workgroups per unit, each with half of the tiles, the second to finish combining the two
    halves, halves_lse, halves_plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE,
                                                          selection_units=ffi.ATTN_UNITS_HEAD_BLOCK_HALVES)
    assert halves_plan.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK_HALVES
    _close(halves, expected, tol)
    assert np.abs(halves_lse.cpu().numpy()[live] - expected_lse[live]).max() <= tol
    assert (halves.float() - out.float()).abs().max().item() <= 2 ** -6 * peak
    assert not halves[~torch.from_numpy(live).cuda()].any() and torch.isneginf(halves_lse[~torch.from_numpy(live).cuda()]).all()
    # Launch after launch (more of them than the library has sets of counters), alternating with a
    # shorter selection whose pairs split differently: every pair's counter is back at zero and no
    # partial of an earlier launch is taken for a new one; whichever half finishes second, the
    # result is the same to the bit.
    shorter = selection.copy()
    shorter[:, k // 3:] = -1
    shorter_d = kt.dev_i32(shorter)
    shorter_expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=shorter)
    shorter_first = None
    for launch in range(40):
        if launch % 2 == 0:
            again, again_lse, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE, selection_units=ffi.ATTN_UNITS_HEAD_BLOCK_HALVES)
            assert torch.equal(again, halves) and torch.equal(again_lse, halves_lse), launch
        else:
            again, _, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, shorter_d, SCALE, selection_units=ffi.ATTN_UNITS_HEAD_BLOCK_HALVES)
            if shorter_first is None:
                shorter_first = again
                _close(again, shorter_expected, tol)
            assert torch.equal(again, shorter_first), launch
    # what the option refuses: selections above the staging size
    lib, refused = ffi.load(), ffi.AttnPlan()
    for units in (ffi.ATTN_UNITS_HEAD_BLOCK, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES):
        options = ffi.AttnPlanOptions(0, 0, 0, 0, 1, units)
        assert lib.mlakvAttnPlanInitEx(batch, heads, ffi.ATTN_HEAD_BLOCK_TOKENS + 1, bs, ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16,
                                       C.byref(options), C.byref(refused)) == ffi.ERR_PARAM_INVALID


def test_halved_units_side_by_side_on_two_streams():
    """Launches of halved units on two unordered streams, back to back without a host wait between
    them: each launch has counters of its own (the library hands them out in turn), so the two
    streams' pairs never meet on one word, and every launch gives the bytes its stream's inputs
    give alone."""
    import ctypes as C
    lib = ffi.load()
    bs, heads, k = 64, 64, 512
    ctxs = [4000, 2500, 600, 3000, 513, 1900, 2047, 800]
    cache, table = _setup(ctxs, bs, False, seed=90)
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    rng = np.random.default_rng(91)
    row = (LATENT + ROPE) * 2
    lanes = []
    for lane in range(2):
        selection = np.full((len(ctxs), k), -1, dtype=np.int32)
        for s, n in enumerate(ctxs):
            take = min(n, k) - 7 * lane * s          # the two streams' selections end at different tiles
            selection[s, :take] = rng.permutation(n)[:take]
        q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=92 + lane).cuda()
        sel_d = kt.dev_i32(selection)
        alone, alone_lse, plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, sel_d, SCALE,
                                                     selection_units=ffi.ATTN_UNITS_HEAD_BLOCK_HALVES)
        expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=selection)
        _close(alone, expected, 2e-2)
        lanes.append({"q": q, "sel": sel_d, "alone": alone, "alone_lse": alone_lse, "plan": plan, "stream": torch.cuda.Stream(),
                      "workspace": torch.empty(int(plan.workspace_bytes), dtype=torch.uint8, device="cuda"),
                      "outs": [torch.full_like(alone, float("nan")) for _ in range(24)],
                      "lses": [torch.full_like(alone_lse, float("nan")) for _ in range(24)]})
    torch.cuda.synchronize()
    for launch in range(24):
        for lane in lanes:
            q, plan = lane["q"], lane["plan"]
            ffi.check(lib.mlakvAttnDecodeSparse(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                                q.data_ptr() + LATENT * 2, heads * row, row, table_d.data_ptr(), table_d.shape[1],
                                                lens_d.data_ptr(), lane["sel"].data_ptr(), lane["sel"].stride(0), float(SCALE),
                                                lane["outs"][launch].data_ptr(), heads * LATENT * 2, LATENT * 2,
                                                lane["lses"][launch].data_ptr(), lane["workspace"].data_ptr(),
                                                int(plan.workspace_bytes), C.c_void_p(lane["stream"].cuda_stream)))
    torch.cuda.synchronize()
    for lane in lanes:
        for launch in range(24):
            assert torch.equal(lane["outs"][launch], lane["alone"]), launch
            assert torch.equal(lane["lses"][launch], lane["alone_lse"]), launch


@pytest.mark.parametrize("fp8", [False, True])
def test_table_entries_that_name_no_block_read_as_rows_of_zeros(fp8):
    """A block-table entry outside [0, num_blocks) is never followed: its tokens count as rows of
    zeros (score 0, nothing added to the output), in the whole-context kernel and in both kinds of
    selected-token units. The oracle gets a table that points those entries at a block that was
    never written (the cache starts as zeros)."""
    bs, heads, k = 64, 32, 256
    ctxs = [700, 300, 64]
    cache, table = _setup(ctxs, bs, fp8, seed=60)
    spare = sorted(set(range(cache.blocks)) - {int(b) for s, n in enumerate(ctxs) for b in table[s, :-(-n // bs)]})[0]
    holes = [(0, 3, -1), (0, 10, cache.blocks + 7), (1, 0, 2 ** 31 - 1), (2, 0, -5)]
    broken, zeroed = table.copy(), table.copy()
    for s, logical, value in holes:
        broken[s, logical], zeroed[s, logical] = value, spare
    rng = np.random.default_rng(61)
    selection = np.full((len(ctxs), k), -1, dtype=np.int32)
    for s, n in enumerate(ctxs):
        take = min(n, k)
        selection[s, :take] = rng.permutation(n)[:take]
    selection[0, :8] = 3 * bs + np.arange(8)            # tokens of a hole for certain, a whole tile row group
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=62).cuda()
    tol = 6e-2 if fp8 else 2e-2
    lens_d, sel_d = kt.dev_i32(ctxs), kt.dev_i32(selection)
    expected, expected_lse = kt.oracle_attention(cache, 0, q, zeroed, ctxs, SCALE)
    out, lse, _ = kt.attention(cache, 0, q, kt.dev_i32(broken), lens_d, SCALE)
    _close(out, expected, tol)
    assert np.abs(lse.cpu().numpy() - expected_lse).max() <= tol
    expected, expected_lse = kt.oracle_attention(cache, 0, q, zeroed, ctxs, SCALE, sparse_indices=selection)
    for units in (ffi.ATTN_UNITS_SPLIT, ffi.ATTN_UNITS_HEAD_BLOCK, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES):
        out, lse, plan = kt.sparse_attention(cache, 0, q, kt.dev_i32(broken), lens_d, sel_d, SCALE, selection_units=units)
        assert plan.selection_units == units
        _close(out, expected, tol)
        assert np.abs(lse.cpu().numpy() - expected_lse).max() <= tol


def test_full_selection_equals_dense_and_order_does_not_matter():
    bs, heads, k = 64, 64, 512
    ctxs = [512, 300, 77]
    cache, table = _setup(ctxs, bs, False, seed=90)
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=91).cuda()
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    dense, dense_lse, _ = kt.attention(cache, 0, q, table_d, lens_d, SCALE)
    identity = np.full((len(ctxs), k), -1, dtype=np.int32)
    shuffled = identity.copy()
    rng = np.random.default_rng(92)
    for s, n in enumerate(ctxs):
        identity[s, :n] = np.arange(n)
        shuffled[s, :n] = rng.permutation(n)
    out, lse, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, kt.dev_i32(identity), SCALE)
    peak = dense.float().abs().max().item()
    # same tokens in the same tiles: only the chunking may differ
    assert (out.float() - dense.float()).abs().max().item() <= 2 ** -7 * peak
    assert (lse - dense_lse).abs().max().item() <= 1e-3
    out2, lse2, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, kt.dev_i32(shuffled), SCALE)
    assert (out2.float() - dense.float()).abs().max().item() <= 2e-2 * peak
    assert (lse2 - dense_lse).abs().max().item() <= 1e-3


def test_selection_ends_at_first_invalid_entry_and_argument_checks():
    bs, heads, k = 64, 16, 64
    ctxs = [200, 200]
    cache, table = _setup(ctxs, bs, False, seed=95)
    q = kt.randn_bf16((2, heads, LATENT + ROPE), seed=96).cuda()
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    selection = np.full((2, k), -1, dtype=np.int32)
    selection[0, :10] = np.arange(10) * 7
    selection[1, :10] = np.arange(10) * 7
    selection[1, 10] = 200       # not inside the context: ends the list
    selection[1, 11:20] = 5      # never looked at
    out, lse, plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, kt.dev_i32(selection), SCALE)
    q_same = q.clone()
    q_same[1] = q[0]
    cache2, table2 = cache, table
    # both sequences hold different rows, so compare each with the oracle instead of with each other
    expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE, sparse_indices=selection)
    _close(out, expected, 2e-2)
    lib = ffi.load()
    row = (LATENT + ROPE) * 2
    sel_d = kt.dev_i32(selection)
    dense_plan = ffi.AttnPlan()
    ffi.check(lib.mlakvAttnPlanInit(2, heads, 200, bs, ffi.DTYPE_BF16, C.byref(dense_plan)))
    workspace = torch.zeros(max(int(plan.workspace_bytes), int(dense_plan.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    out_t = torch.zeros(2, heads, LATENT, dtype=torch.bfloat16, device="cuda")

    def sparse_call(p, sel=sel_d.data_ptr(), stride=k, out_ptr=out_t.data_ptr()):
        return lib.mlakvAttnDecodeSparse(C.byref(p), C.byref(cache.view), 0, q.data_ptr(), heads * row, row, q.data_ptr() + LATENT * 2,
                                         heads * row, row, table_d.data_ptr(), table_d.shape[1], lens_d.data_ptr(), sel, stride,
                                         SCALE, out_ptr, heads * LATENT * 2, LATENT * 2, None, workspace.data_ptr(),
                                         workspace.numel(), kt.stream_ptr())

    assert sparse_call(plan) == 0
    assert sparse_call(dense_plan) == ffi.ERR_PARAM_INVALID            # a whole-context plan
    assert sparse_call(plan, sel=None) == ffi.ERR_PARAM_NULLPTR
    assert sparse_call(plan, stride=k - 1) == ffi.ERR_PARAM_INVALID
    assert sparse_call(plan, out_ptr=None) == ffi.ERR_PARAM_NULLPTR
    # a selected token is staged as (block, slot) in 31 bits: a pool beyond that is refused before any launch
    huge = type(cache.view).from_buffer_copy(cache.view)
    huge.num_blocks = 1 << 26
    refused = lib.mlakvAttnDecodeSparse(C.byref(plan), C.byref(huge), 0, q.data_ptr(), heads * row, row, q.data_ptr() + LATENT * 2,
                                        heads * row, row, table_d.data_ptr(), table_d.shape[1], lens_d.data_ptr(), sel_d.data_ptr(), k,
                                        SCALE, out_t.data_ptr(), heads * LATENT * 2, LATENT * 2, None, workspace.data_ptr(),
                                        workspace.numel(), kt.stream_ptr())
    assert refused == ffi.ERR_PARAM_INVALID and b"2^31" in lib.mlakvGetLastError()
    dense_with_sparse_plan = lib.mlakvAttnDecode(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                                 q.data_ptr() + LATENT * 2, heads * row, row, table_d.data_ptr(), table_d.shape[1],
                                                 lens_d.data_ptr(), SCALE, out_t.data_ptr(), heads * LATENT * 2, LATENT * 2, None,
                                                 workspace.data_ptr(), workspace.numel(), kt.stream_ptr())
    assert dense_with_sparse_plan == ffi.ERR_PARAM_INVALID
    bad = ffi.AttnPlan()
    assert lib.mlakvAttnSparsePlanInit(2, heads, 0, bs, ffi.DTYPE_BF16, C.byref(bad)) == ffi.ERR_PARAM_INVALID
    assert lib.mlakvAttnSparsePlanInit(2, heads, 2049, bs, ffi.DTYPE_BF16, C.byref(bad)) == ffi.ERR_PARAM_INVALID
    torch.cuda.synchronize()
