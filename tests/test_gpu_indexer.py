"""GPU parity: Lightning Indexer (mlakvLightningIndexer) through the C ABI against the CPU oracle.
The scores are compared as the values of the 16-bit keys the selection sorts by. The kernel sums
the exact products in fp32 in the matrix unit's order and the head sum in a lane-tree order, the
oracle rounds the exact dot product once and follows the vendored kernel's even/odd order, so a
score may differ by fp32 rounding of a sum that can cancel (weights of either sign): the bound is
one bf16 step of the score plus 1e-5 of the sum of the terms' magnitudes, and at most 0.5 % of the
keys may differ at all. The selection itself is integer work and must be bit-exact on the keys the
GPU produced, in the documented order."""
import ctypes as C

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

D = 128


def _decode_table():
    lib = orc.load()
    return np.array([lib.kvo_e4m3_to_f32(c) for c in range(256)], dtype=np.float64)


_E4M3 = _decode_table()


def _key_value(keys):
    keys = np.asarray(keys, dtype=np.uint16)
    bits = np.where(keys & 0x8000, keys & 0x7FFF, ~keys & 0xFFFF).astype(np.uint32)
    return (bits << 16).view(np.float32).astype(np.float64)


def _codes(rng, shape, spread):
    """Random E4M3 codes without NaN: magnitudes below `spread` exponent steps, either sign."""
    magnitude = rng.integers(0, spread, shape).astype(np.uint8)
    return (magnitude | (rng.integers(0, 2, shape).astype(np.uint8) << 7)).astype(np.uint8)


def _run(seq_lens, bs, heads, k, seed, zero_query=False, row_padding=0):
    rng = np.random.default_rng(seed)
    batch = len(seq_lens)
    max_len = max(max(seq_lens), 1)
    blocks = sum(-(-n // bs) for n in seq_lens) + 5
    pool = kt.build_tables(seq_lens, bs, blocks, seed=seed, max_blocks=-(-max_len // bs))
    table = pool.table()
    key_plane = _codes(rng, (blocks * bs, D), 0x58)
    key_scale = rng.uniform(0.01, 0.05, blocks * bs).astype(np.float32)
    query = np.zeros((batch, heads, D), np.uint8) if zero_query else _codes(rng, (batch, heads, D), 0x58)
    weights = kt.randn_bf16((batch, heads), seed=seed + 1)
    q_scale = rng.uniform(0.01, 0.05, (batch, heads)).astype(np.float32)
    lib = ffi.load()
    keys_d = torch.as_tensor(key_plane, device="cuda")
    scales_d = torch.as_tensor(key_scale, device="cuda")
    view = ffi.IndexKeyView(keys_d.data_ptr(), bs * D, D, scales_d.data_ptr(), bs, blocks, bs, D, 0)
    query_d = torch.as_tensor(query, device="cuda")
    # `row_padding` extra elements behind every sequence's weights and scales: rows that do not
    # start on 8 / 16 bytes take the kernel's element-wise loads
    weights_d = torch.zeros(batch, heads + row_padding, dtype=torch.bfloat16, device="cuda")
    weights_d[:, :heads] = weights.cuda()
    q_scale_d = torch.zeros(batch, heads + row_padding, dtype=torch.float32, device="cuda")
    q_scale_d[:, :heads] = torch.as_tensor(q_scale, device="cuda")
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(seq_lens)
    out = torch.full((batch, k), -7, dtype=torch.int32, device="cuda")
    ws_bytes = int(lib.mlakvIndexerWorkspaceBytes(batch, max_len))
    workspace = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    ffi.check(lib.mlakvLightningIndexer(C.byref(view), query_d.data_ptr(), heads * D, D, weights_d.data_ptr(), (heads + row_padding) * 2,
                                        q_scale_d.data_ptr(), heads + row_padding, heads, table_d.data_ptr(), table.shape[1], lens_d.data_ptr(),
                                        batch, max_len, k, out.data_ptr(), k, workspace.data_ptr(), workspace.numel(),
                                        kt.stream_ptr()))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    row = (max_len + 127) // 128 * 128
    gpu_keys = workspace.view(torch.int16).cpu().numpy().view(np.uint16)[: batch * row].reshape(batch, row)
    differing = total = 0
    for b, n in enumerate(seq_lens):
        if n <= k:
            assert got[b].tolist() == list(range(n)) + [-1] * (k - n)
            continue
        want_keys = orc.indexer_scores(query[b], kt.bits16(weights[b]), q_scale[b], key_plane, key_scale, bs, table[b], n)
        # fp32 rounding in a different order: one bf16 step of the score, plus the fp32 error of a
        # 64-term sum that may cancel (weights of either sign), measured against the sum of magnitudes
        slots = table[b][np.arange(n) // bs].astype(np.int64) * bs + np.arange(n) % bs
        qk = np.maximum(_E4M3[query[b]] @ _E4M3[key_plane[slots]].T, 0.0)
        w = (kt.bits16(weights[b]).astype(np.uint32) << 16).view(np.float32).astype(np.float64) * q_scale[b]
        magnitude = (qk * np.abs(w)[:, None]).sum(axis=0) * key_scale[slots]
        got_f, want_f = _key_value(gpu_keys[b, :n]), _key_value(want_keys)
        tolerance = 2.0 ** -7 * np.abs(want_f) + 1e-5 * magnitude + 1e-30
        assert (np.abs(got_f - want_f) <= tolerance).all(), (b, np.abs(got_f - want_f).max())
        differing += int((gpu_keys[b, :n] != want_keys).sum())
        total += n
        # integer selection: bit-exact on the keys the GPU holds, in the documented order
        assert got[b].tolist() == orc.indexer_topk(gpu_keys[b, :n], k).tolist()
        # and against the oracle's own keys: the same set except where such a key difference
        # moves a token across the threshold
        want = orc.indexer_topk(want_keys, k)
        odd = sorted(set(got[b].tolist()) ^ set(want.tolist()))
        threshold = _key_value(np.sort(want_keys)[-k:])[0]
        assert all(abs(want_f[t] - threshold) <= 2 * tolerance[t] for t in odd), (b, len(odd))
        assert len(odd) <= max(2, k // 50)
    assert total == 0 or differing <= 0.005 * total
    return got


@pytest.mark.parametrize("bs,heads,k", [(64, 64, 512), (16, 32, 100), (128, 16, 2048), (64, 48, 64)])
def test_indexer_matches_oracle_ragged(bs, heads, k):
    _run([3000, 513 if k == 512 else k + 1, 1, 0, 2600, k, 777], bs, heads, k, seed=101)


def test_weight_and_scale_rows_need_no_alignment():
    _run([900, 300, 1200], 64, 32, 128, seed=105, row_padding=1)


@pytest.mark.parametrize("bs", [16, 64])
def test_index_key_append_matches_the_oracle_quantiser(bs):
    """The write side of the key pool: bit-exact with the oracle's E4M3 row quantiser (the one the
    FP8 KV cache is pinned with) at 128 elements per row; untouched slots stay as they were."""
    rng = np.random.default_rng(131)
    tokens, blocks = 203, 9 if bs == 64 else 30
    rows = kt.randn_bf16((tokens, D), seed=132, outlier_fraction=0.02)
    rows[7] = 0                                  # a zero row: scale 1, zero codes
    rows[11, 5] = 1e30                           # one huge value: the rest of the row rounds to zero codes
    slots = rng.permutation(blocks * bs)[:tokens].astype(np.int32)
    slots[3] = -1                                # skipped
    slots[4] = blocks * bs + 5                   # a block outside the pool: skipped
    lib = ffi.load()
    keys_d = torch.full((blocks * bs, D), 0x11, dtype=torch.uint8, device="cuda")
    scales_d = torch.full((blocks * bs,), 7.0, dtype=torch.float32, device="cuda")
    view = ffi.IndexKeyView(keys_d.data_ptr(), bs * D, D, scales_d.data_ptr(), bs, blocks, bs, D, 0)
    rows_d, slots_d = rows.cuda(), kt.dev_i32(slots)
    ffi.check(lib.mlakvIndexKeyAppend(C.byref(view), rows_d.data_ptr(), D * 2, slots_d.data_ptr(), tokens, kt.stream_ptr()))
    torch.cuda.synchronize()
    want_keys = np.full(blocks * bs * D, 0x11, dtype=np.uint8)
    want_scales = np.full(blocks * bs, 7.0, dtype=np.float32)
    live = (slots >= 0) & (slots < blocks * bs)
    unused = np.zeros((tokens, 1), dtype=np.uint16)
    finite = kt.bits16(rows).copy()
    orc.append_rows_fp8(want_keys, np.zeros(1, np.uint8), want_scales, bs, finite[live], unused[live], slots[live],
                        latent_dim=D, rope_dim=0)
    assert np.array_equal(keys_d.cpu().numpy().reshape(-1), want_keys)
    assert np.array_equal(scales_d.cpu().numpy(), want_scales)
    assert lib.mlakvIndexKeyAppend(C.byref(view), None, D * 2, slots_d.data_ptr(), tokens, kt.stream_ptr()) == ffi.ERR_PARAM_NULLPTR
    assert lib.mlakvIndexKeyAppend(C.byref(view), rows_d.data_ptr(), D, slots_d.data_ptr(), tokens, kt.stream_ptr()) == ffi.ERR_PARAM_INVALID
    assert lib.mlakvIndexKeyAppend(C.byref(view), rows_d.data_ptr(), D * 2, slots_d.data_ptr(), 0, kt.stream_ptr()) == 0


def test_all_equal_scores_select_the_first_positions():
    got = _run([1000, 300], 64, 64, 256, seed=102, zero_query=True)
    assert got[0].tolist() == list(range(256)) and got[1].tolist() == list(range(256))


def test_indices_feed_the_selected_token_attention():
    """The two operators chained on one block table: the attention over the indexer's list equals
    the oracle's attention over the same list."""
    import math
    bs, heads, k = 64, 64, 128
    ctxs = [700, 90]
    blocks = sum(-(-c // bs) for c in ctxs) + 2
    pool = kt.build_tables(ctxs, bs, blocks, seed=103)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    total = sum(ctxs)
    kt.append(cache, kt.randn_bf16((1, total, kt.LATENT), seed=104).cuda(), kt.randn_bf16((1, total, kt.ROPE), seed=105).cuda(),
              kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    rng = np.random.default_rng(106)
    keys_d = torch.as_tensor(_codes(rng, (blocks * bs, D), 0x58), device="cuda")
    scales_d = torch.as_tensor(rng.uniform(0.01, 0.05, blocks * bs).astype(np.float32), device="cuda")
    view = ffi.IndexKeyView(keys_d.data_ptr(), bs * D, D, scales_d.data_ptr(), bs, blocks, bs, D, 0)
    iq = torch.as_tensor(_codes(rng, (2, heads, D), 0x58), device="cuda")
    iw = kt.randn_bf16((2, heads), seed=107).cuda()
    iqs = torch.as_tensor(rng.uniform(0.01, 0.05, (2, heads)).astype(np.float32), device="cuda")
    lib = ffi.load()
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    selection = torch.zeros(2, k, dtype=torch.int32, device="cuda")
    workspace = torch.zeros(int(lib.mlakvIndexerWorkspaceBytes(2, 700)), dtype=torch.uint8, device="cuda")
    ffi.check(lib.mlakvLightningIndexer(C.byref(view), iq.data_ptr(), heads * D, D, iw.data_ptr(), heads * 2, iqs.data_ptr(), heads,
                                        heads, table_d.data_ptr(), table.shape[1], lens_d.data_ptr(), 2, 700, k,
                                        selection.data_ptr(), k, workspace.data_ptr(), workspace.numel(), kt.stream_ptr()))
    q = kt.randn_bf16((2, heads, kt.LATENT + kt.ROPE), seed=108).cuda()
    scale = 1.0 / math.sqrt(192.0)
    out, lse, _ = kt.sparse_attention(cache, 0, q, table_d, lens_d, selection, scale)
    chosen = selection.cpu().numpy()
    assert (chosen[0] >= 0).all() and len(set(chosen[0].tolist())) == k
    assert chosen[1].tolist() == list(range(90)) + [-1] * (k - 90)
    expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, scale, sparse_indices=chosen)
    peak = np.abs(expected).max()
    assert np.abs(out.float().cpu().numpy() - expected).max() <= 2e-2 * peak


def test_argument_checks():
    lib = ffi.load()
    keys = torch.zeros(4 * 64, D, dtype=torch.uint8, device="cuda")
    scales = torch.ones(4 * 64, dtype=torch.float32, device="cuda")
    query = torch.zeros(1, 64, D, dtype=torch.uint8, device="cuda")
    weights = torch.ones(1, 64, dtype=torch.bfloat16, device="cuda")
    q_scale = torch.ones(1, 64, dtype=torch.float32, device="cuda")
    table, lens = kt.dev_i32(np.arange(4, dtype=np.int32).reshape(1, 4)), kt.dev_i32([200])
    out = torch.zeros(1, 64, dtype=torch.int32, device="cuda")
    workspace = torch.zeros(int(lib.mlakvIndexerWorkspaceBytes(1, 256)), dtype=torch.uint8, device="cuda")

    def call(view=None, heads=64, k=64, max_len=256, ws=workspace.data_ptr(), ws_bytes=workspace.numel(), q=query.data_ptr(), stride=64):
        view = view or ffi.IndexKeyView(keys.data_ptr(), 64 * D, D, scales.data_ptr(), 64, 4, 64, D, 0)
        return lib.mlakvLightningIndexer(C.byref(view), q, 64 * D, D, weights.data_ptr(), 128, q_scale.data_ptr(), 64, heads,
                                         table.data_ptr(), 4, lens.data_ptr(), 1, max_len, k, out.data_ptr(), stride, ws, ws_bytes,
                                         kt.stream_ptr())

    assert call() == 0
    assert call(heads=24) == ffi.ERR_PARAM_INVALID
    assert call(k=0) == ffi.ERR_PARAM_INVALID and call(k=4096) == ffi.ERR_PARAM_INVALID
    assert call(max_len=257) == ffi.ERR_PARAM_INVALID          # the table row addresses 256 tokens
    assert call(ws=None) == ffi.ERR_PARAM_NULLPTR
    assert call(ws_bytes=16) == ffi.ERR_PARAM_INVALID
    assert call(q=None) == ffi.ERR_PARAM_NULLPTR
    assert call(stride=32) == ffi.ERR_PARAM_INVALID
    assert call(view=ffi.IndexKeyView(keys.data_ptr(), 64 * D, D, scales.data_ptr(), 64, 4, 64, 64, 0)) == ffi.ERR_PARAM_INVALID
    assert call(max_len=64, ws=None, ws_bytes=0) == 0          # nothing longer than k: no scores, no workspace
    torch.cuda.synchronize()


def test_full_size_indexer_and_selected_attention_on_sampled_sequences():
    """The shape the bench times (batch 32, context 8192, 64 index heads, top-512, block 64): the
    indexer's keys and selection for three sampled sequences against the oracle, every sequence's
    list checked for being 512 distinct in-range positions, then the selected-token attention over
    those lists against the oracle for the same three sequences."""
    import math
    bs, heads, k, batch, ctx = 64, 64, 512, 32, 8192
    blocks = batch * (ctx // bs) + 7
    rng = np.random.default_rng(120)
    pool = kt.build_tables([ctx] * batch, bs, blocks, seed=121)
    table = pool.table()
    key_plane = _codes(rng, (blocks * bs, D), 0x58)
    key_scale = rng.uniform(0.01, 0.05, blocks * bs).astype(np.float32)
    query = _codes(rng, (batch, heads, D), 0x58)
    weights = kt.randn_bf16((batch, heads), seed=122)
    q_scale = rng.uniform(0.01, 0.05, (batch, heads)).astype(np.float32)
    lib = ffi.load()
    keys_d, scales_d = torch.as_tensor(key_plane, device="cuda"), torch.as_tensor(key_scale, device="cuda")
    view = ffi.IndexKeyView(keys_d.data_ptr(), bs * D, D, scales_d.data_ptr(), bs, blocks, bs, D, 0)
    query_d, weights_d, q_scale_d = torch.as_tensor(query, device="cuda"), weights.cuda(), torch.as_tensor(q_scale, device="cuda")
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32([ctx] * batch)
    selection = torch.full((batch, k), -7, dtype=torch.int32, device="cuda")
    workspace = torch.zeros(int(lib.mlakvIndexerWorkspaceBytes(batch, ctx)), dtype=torch.uint8, device="cuda")
    ffi.check(lib.mlakvLightningIndexer(C.byref(view), query_d.data_ptr(), heads * D, D, weights_d.data_ptr(), heads * 2,
                                        q_scale_d.data_ptr(), heads, heads, table_d.data_ptr(), table.shape[1], lens_d.data_ptr(),
                                        batch, ctx, k, selection.data_ptr(), k, workspace.data_ptr(), workspace.numel(),
                                        kt.stream_ptr()))
    torch.cuda.synchronize()
    chosen = selection.cpu().numpy()
    assert ((chosen >= 0) & (chosen < ctx)).all()
    assert all(len(set(row.tolist())) == k for row in chosen)
    gpu_keys = workspace.view(torch.int16).cpu().numpy().view(np.uint16).reshape(batch, ctx)
    sample = (0, 13, 31)
    for b in sample:
        want_keys = orc.indexer_scores(query[b], kt.bits16(weights[b]), q_scale[b], key_plane, key_scale, bs, table[b], ctx)
        assert (gpu_keys[b] != want_keys).mean() <= 0.005
        assert chosen[b].tolist() == orc.indexer_topk(gpu_keys[b], k).tolist()
    # the MLA cache behind the same table, filled on the device; attention over the selected lists
    cache = kt.PagedCache(1, blocks, bs)
    cache.latent.copy_(torch.randn(cache.latent.shape, device="cuda", generator=torch.Generator(device="cuda").manual_seed(123)).to(torch.bfloat16))
    cache.rope.copy_(torch.randn(cache.rope.shape, device="cuda", generator=torch.Generator(device="cuda").manual_seed(124)).to(torch.bfloat16))
    q = kt.randn_bf16((batch, 64, kt.LATENT + kt.ROPE), seed=125).cuda()
    scale = 1.0 / math.sqrt(192.0)
    out, lse, plan = kt.sparse_attention(cache, 0, q, table_d, lens_d, selection, scale)
    assert plan.work_groups >= 128
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    for b in sample:
        expected, expected_lse = kt.oracle_attention(cache, 0, q[b:b + 1], table[b:b + 1], [ctx], scale, sparse_indices=chosen[b:b + 1])
        peak = np.abs(expected).max()
        assert np.abs(got[b] - expected[0]).max() <= 2e-2 * peak
        assert np.abs(lse[b].cpu().numpy() - expected_lse[0]).max() <= 2e-2


def test_two_phase_operator_equals_the_direct_entry():
    """aclnnQuantLightningIndexer through plan / launch on descriptors shaped as the operator's
    contract names them, against mlakvLightningIndexer on the same buffers."""
    import acl_ffi as acl
    lib, alib = ffi.load(), acl.load()
    keep = acl.Keep()
    rng = np.random.default_rng(130)
    batch, heads, bs, k = 3, 64, 64, 128
    seq_lens = [900, 64, 333]
    width = -(-max(seq_lens) // bs)
    blocks = sum(-(-n // bs) for n in seq_lens) + 2
    pool = kt.build_tables(seq_lens, bs, blocks, seed=131, max_blocks=width)
    table = pool.table()
    keys_d = torch.as_tensor(_codes(rng, (blocks, bs, 1, D), 0x58), device="cuda")
    scales_d = torch.as_tensor(rng.uniform(0.01, 0.05, (blocks, bs, 1)).astype(np.float32), device="cuda")
    query_d = torch.as_tensor(_codes(rng, (batch, 1, heads, D), 0x58), device="cuda")
    weights_d = kt.randn_bf16((batch, 1, heads), seed=132).cuda()
    q_scale_d = torch.as_tensor(rng.uniform(0.01, 0.05, (batch, 1, heads)).astype(np.float32), device="cuda")
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(seq_lens)
    out_shim = torch.full((batch, 1, 1, k), -7, dtype=torch.int32, device="cuda")
    E8 = acl.ACL_FLOAT8_E4M3FN
    handles = [keep.tensor([batch, 1, heads, D], E8, query_d.data_ptr()), keep.tensor([blocks, bs, 1, D], E8, keys_d.data_ptr()),
               keep.tensor([batch, 1, heads], acl.ACL_BF16, weights_d.data_ptr()),
               keep.tensor([batch, 1, heads], acl.ACL_FLOAT32, q_scale_d.data_ptr()),
               keep.tensor([blocks, bs, 1], acl.ACL_FLOAT32, scales_d.data_ptr())]
    t_lens = keep.tensor([batch], acl.ACL_INT32, lens_d.data_ptr())
    t_table = keep.tensor([batch, width], acl.ACL_INT32, table_d.data_ptr())
    t_out = keep.tensor([batch, 1, 1, k], acl.ACL_INT32, out_shim.data_ptr())
    big = 2 ** 63 - 1
    workspace_bytes, executor = C.c_uint64(0), C.c_void_p()
    assert alib.aclnnQuantLightningIndexerGetWorkspaceSize(*handles, None, t_lens, t_table, 0, 0, b"BSND", b"PA_BSND", k, 3, big, big, t_out,
                                                           C.byref(workspace_bytes), C.byref(executor)) == 0, acl.last_error()
    workspace = torch.zeros(max(workspace_bytes.value, 16), dtype=torch.uint8, device="cuda")
    assert alib.aclnnQuantLightningIndexer(workspace.data_ptr(), workspace.numel(), executor, kt.stream_ptr()) == 0, acl.last_error()
    torch.cuda.synchronize()
    assert alib.aclDestroyAclOpExecutor(executor) == 0
    out_direct = torch.full((batch, k), -7, dtype=torch.int32, device="cuda")
    view = ffi.IndexKeyView(keys_d.data_ptr(), bs * D, D, scales_d.data_ptr(), bs, blocks, bs, D, 0)
    ws2 = torch.zeros(int(lib.mlakvIndexerWorkspaceBytes(batch, width * bs)), dtype=torch.uint8, device="cuda")
    ffi.check(lib.mlakvLightningIndexer(C.byref(view), query_d.data_ptr(), heads * D, D, weights_d.data_ptr(), heads * 2, q_scale_d.data_ptr(),
                                        heads, heads, table_d.data_ptr(), width, lens_d.data_ptr(), batch, width * bs, k,
                                        out_direct.data_ptr(), k, ws2.data_ptr(), ws2.numel(), kt.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out_shim.reshape(batch, k), out_direct)
    got = out_direct.cpu().numpy()
    assert got[1].tolist() == list(range(64)) + [-1] * (k - 64)
    assert (got[0] >= 0).all() and (got[0] < 900).all() and len(set(got[0].tolist())) == k
