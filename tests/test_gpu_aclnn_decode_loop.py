"""GPU parity through the aclnn-compatible boundary, driven the way the reference's pipeline
drives it (src/pipeline/pipeline.cpp:390-416, :515-519): descriptors built once, executors
planned once and made repeatable, per layer the cache-slice addresses are swapped at IR
indices 1/4 (scatter) and 1/2/25 (attention), per step the slot goes through a pinned
mailbox. Device memory, streams and copies go through the aclrt surface."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

import acl_ffi as acl
import kv_testing as kt
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

LATENT, ROPE = 512, 64


def _ok(status):
    assert status == 0, acl.last_error()


def test_reference_shaped_decode_loop_matches_oracle():
    lib = acl.load()
    layers, heads, bs, max_ctx, steps = 2, 64, 64, 256, 70
    blocks = max_ctx // bs
    _ok(lib.aclInit(None))
    _ok(lib.aclrtSetDevice(0))
    count = C.c_uint32()
    _ok(lib.aclrtGetDeviceCount(C.byref(count)))
    assert count.value >= 1 and lib.aclrtGetSocName().decode().startswith("gfx")
    stream = C.c_void_p()
    _ok(lib.aclrtCreateStream(C.byref(stream)))

    def dmalloc(nbytes):
        p = C.c_void_p()
        _ok(lib.aclrtMalloc(C.byref(p), nbytes, 0))
        assert p.value % 4096 == 0
        _ok(lib.aclrtMemset(p, nbytes, 0, nbytes))
        return p.value

    latent_stride, rope_stride = blocks * bs * LATENT * 2, blocks * bs * ROPE * 2
    latent_base, rope_base = dmalloc(layers * latent_stride), dmalloc(layers * rope_stride)
    table_dev, slot_dev = dmalloc(blocks * 4), dmalloc(512)
    q_b, kv_a, kv_normed, attn_out = dmalloc(heads * 576 * 2), dmalloc(576 * 2), dmalloc(LATENT * 2), dmalloc(heads * LATENT * 2)
    mailbox = C.c_void_p()
    _ok(lib.aclrtMallocHost(C.byref(mailbox), 4096))
    table_host = (C.c_int32 * blocks)(*range(blocks))  # identity paging, written once
    _ok(lib.aclrtMemcpy(table_dev, blocks * 4, table_host, blocks * 4, 1))

    keep = acl.Keep()
    q_latent = keep.tensor([1, heads, LATENT], acl.ACL_BF16, q_b, strides=[heads * 576, 576, 1])
    q_rope = keep.tensor([1, heads, ROPE], acl.ACL_BF16, q_b + LATENT * 2, strides=[heads * 576, 576, 1])
    t_normed = keep.tensor([1, LATENT], acl.ACL_BF16, kv_normed)
    t_k_rope = keep.tensor([1, 1, ROPE], acl.ACL_BF16, kv_a + LATENT * 2)
    t_latent_cache = keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, latent_base)
    t_rope_cache = keep.tensor([blocks, bs, 1, ROPE], acl.ACL_BF16, rope_base)
    t_rope_view = keep.tensor([blocks, bs, 1, ROPE], acl.ACL_BF16, rope_base)
    key_list = keep.tensor_list([keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, latent_base)])
    value_list = keep.tensor_list([keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, latent_base)])
    t_table = keep.tensor([1, blocks], acl.ACL_INT32, table_dev)
    t_slot = keep.tensor([1], acl.ACL_INT32, slot_dev)
    seq_q, _ = keep.int_array([1])
    seq_kv, seq_kv_storage = keep.int_array([max_ctx])
    t_out = keep.tensor([1, heads, LATENT], acl.ACL_BF16, attn_out)

    status, ws_scatter, ex_scatter = acl.plan_scatter(t_normed, t_latent_cache, t_slot, t_k_rope, t_rope_cache)
    _ok(status)
    scale = 1.0 / math.sqrt(192.0)
    status, ws_attn, ex_attn = acl.plan_attention(q_latent, key_list, value_list, seq_q, seq_kv, t_table, q_rope, t_rope_view, heads,
                                                  scale, bs, t_out)
    _ok(status)
    _ok(lib.aclSetAclOpExecutorRepeatable(ex_scatter))
    _ok(lib.aclSetAclOpExecutorRepeatable(ex_attn))
    workspace_bytes = max(ws_scatter, ws_attn)
    workspace = dmalloc(workspace_bytes)

    rows = kt.randn_bf16((steps, layers, 576), seed=5).cuda()
    queries = kt.randn_bf16((steps, layers, heads, 576), seed=6).cuda()
    results = torch.zeros(steps, layers, heads, LATENT, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    D2D, H2D = 3, 1
    for position in range(steps):
        C.cast(mailbox, C.POINTER(C.c_int32))[position] = position  # a fresh mailbox word per step: no reuse while in flight
        _ok(lib.aclrtMemcpyAsync(slot_dev, 4, mailbox.value + 4 * position, 4, H2D, stream))
        seq_kv_storage[0] = -7  # the array's values were copied when it was created: the caller's storage is its own again
        live = (C.c_int64 * 1)(position + 1)
        _ok(lib.aclnnMlaKvSetSeqLens(ex_attn, live, 1))  # the live length, copied; `live` may go out of scope
        for layer in range(layers):
            latent, rope = latent_base + layer * latent_stride, rope_base + layer * rope_stride
            _ok(lib.aclSetTensorAddr(ex_scatter, 1, t_latent_cache, latent))
            _ok(lib.aclSetTensorAddr(ex_scatter, 4, t_rope_cache, rope))
            _ok(lib.aclSetDynamicTensorAddr(ex_attn, 1, 0, key_list, latent))
            _ok(lib.aclSetDynamicTensorAddr(ex_attn, 2, 0, value_list, latent))
            _ok(lib.aclSetTensorAddr(ex_attn, 25, t_rope_view, rope))
            row = rows[position, layer]
            _ok(lib.aclrtMemcpyAsync(kv_normed, LATENT * 2, row.data_ptr(), LATENT * 2, D2D, stream))
            _ok(lib.aclrtMemcpyAsync(kv_a, 576 * 2, row.data_ptr(), 576 * 2, D2D, stream))
            _ok(lib.aclrtMemcpyAsync(q_b, heads * 576 * 2, queries[position, layer].data_ptr(), heads * 576 * 2, D2D, stream))
            _ok(lib.aclnnScatterPaKvCache(workspace, workspace_bytes, ex_scatter, stream))
            _ok(lib.aclnnFusedInferAttentionScoreV5(workspace, workspace_bytes, ex_attn, stream))
            _ok(lib.aclrtMemcpyAsync(results[position, layer].data_ptr(), heads * LATENT * 2, attn_out, heads * LATENT * 2, D2D, stream))
    _ok(lib.aclrtSynchronizeStreamWithTimeout(stream, 30000))

    # oracle: identity table, rows appended at slot = position, attention over position + 1 rows
    table = np.arange(blocks, dtype=np.int32).reshape(1, blocks)
    for layer in range(layers):
        lat_plane = np.zeros(blocks * bs * LATENT * 2, dtype=np.uint8)
        rope_plane = np.zeros(blocks * bs * ROPE * 2, dtype=np.uint8)
        src = rows[:, layer].contiguous()
        slots = np.arange(steps, dtype=np.int32)
        orc.append_rows(lat_plane, bs * LATENT * 2, LATENT * 2, bs, kt.u8(src[:, :LATENT].contiguous()).reshape(-1), LATENT * 2, LATENT * 2, slots)
        orc.append_rows(rope_plane, bs * ROPE * 2, ROPE * 2, bs, kt.u8(src[:, LATENT:].contiguous()).reshape(-1), ROPE * 2, ROPE * 2, slots)
        # the cache bytes on the device equal the oracle's
        got = torch.zeros(blocks * bs * LATENT, dtype=torch.bfloat16, device="cuda")
        _ok(lib.aclrtMemcpy(got.data_ptr(), got.numel() * 2, latent_base + layer * latent_stride, got.numel() * 2, D2D))
        assert kt.u8(got).tobytes() == lat_plane.tobytes()
        for position in (0, 1, 63, 64, steps - 1):
            qb = kt.bits16(queries[position, layer]).reshape(1, heads, 576)
            expected, _ = orc.mla_decode(np.ascontiguousarray(qb[..., :LATENT]), np.ascontiguousarray(qb[..., LATENT:]),
                                         lat_plane.view(np.uint16), rope_plane.view(np.uint16), bs, table, [position + 1], scale)
            got_out = results[position, layer].float().cpu().numpy()
            peak = np.abs(expected).max()
            assert np.abs(got_out - expected[0]).max() <= 2e-2 * peak, (layer, position)

    # a consumed executor: without aclSetAclOpExecutorRepeatable the second launch is refused
    status, _, once = acl.plan_scatter(t_normed, t_latent_cache, t_slot, t_k_rope, t_rope_cache)
    _ok(status)
    _ok(lib.aclnnScatterPaKvCache(None, 0, once, stream))
    assert lib.aclnnScatterPaKvCache(None, 0, once, stream) == 161002
    assert "consumed" in acl.last_error()
    # too small a workspace is refused before anything is enqueued
    assert lib.aclnnFusedInferAttentionScoreV5(workspace, 16, ex_attn, stream) == 161002
    # value list no longer aliasing the key list is refused
    _ok(lib.aclSetDynamicTensorAddr(ex_attn, 2, 0, value_list, latent_base + 4096))
    assert lib.aclnnFusedInferAttentionScoreV5(workspace, workspace_bytes, ex_attn, stream) == 161002
    _ok(lib.aclrtSynchronizeStream(stream))
    for executor in (once, ex_scatter, ex_attn):
        _ok(lib.aclDestroyAclOpExecutor(executor))
    for pointer in (latent_base, rope_base, table_dev, slot_dev, q_b, kv_a, kv_normed, attn_out, workspace):
        _ok(lib.aclrtFree(pointer))
    _ok(lib.aclrtFreeHost(mailbox))
    _ok(lib.aclrtDestroyStream(stream))


def test_gather_operator_and_bound_device_lengths():
    lib = acl.load()
    bs, heads = 64, 64
    ctxs = [100, 3, 64]
    blocks = 8
    pool = kt.build_tables(ctxs, bs, blocks, seed=17)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    total = sum(ctxs)
    latent = kt.randn_bf16((1, total, LATENT), seed=7).cuda()
    rope = kt.randn_bf16((1, total, ROPE), seed=8).cuda()
    kt.append(cache, latent, rope, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    keep = acl.Keep()
    t_lat = keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, cache.latent.data_ptr())
    t_rope = keep.tensor([blocks, bs, 1, ROPE], acl.ACL_BF16, cache.rope.data_ptr())
    table_dev, lens_dev = kt.dev_i32(table), kt.dev_i32(ctxs)
    cu_dev = kt.dev_i32(np.concatenate([[0], np.cumsum(ctxs)]))
    out = torch.zeros(total, 576, dtype=torch.bfloat16, device="cuda")  # fused 576-element rows
    t_table = keep.tensor(list(table.shape), acl.ACL_INT32, table_dev.data_ptr())
    t_lens = keep.tensor([3], acl.ACL_INT32, lens_dev.data_ptr())
    t_cu = keep.tensor([4], acl.ACL_INT32, cu_dev.data_ptr())
    t_key_out = keep.tensor([total, LATENT], acl.ACL_BF16, out.data_ptr(), strides=[576, 1])
    t_value_out = keep.tensor([total, 1, ROPE], acl.ACL_BF16, out.data_ptr(), strides=[576, 64, 1], offset=LATENT)
    ws, ex = C.c_uint64(), C.c_void_p()
    _ok(lib.aclnnGatherPaKvCacheGetWorkspaceSize(t_lat, t_rope, t_table, t_lens, t_cu, t_key_out, t_value_out, 128, C.byref(ws), C.byref(ex)))
    _ok(lib.aclnnGatherPaKvCache(None, 0, ex, kt.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out[:, :LATENT], latent[0]) and torch.equal(out[:, LATENT:], rope[0])
    _ok(lib.aclDestroyAclOpExecutor(ex))
    # attention with device-resident lengths bound to the executor
    q = kt.randn_bf16((3, heads, 576), seed=9).cuda()
    t_q = keep.tensor([3, heads, LATENT], acl.ACL_BF16, q.data_ptr(), strides=[heads * 576, 576, 1])
    t_qr = keep.tensor([3, heads, ROPE], acl.ACL_BF16, q.data_ptr(), strides=[heads * 576, 576, 1], offset=LATENT)
    klist = keep.tensor_list([keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, cache.latent.data_ptr())])
    vlist = keep.tensor_list([keep.tensor([blocks, bs, 1, LATENT], acl.ACL_BF16, cache.latent.data_ptr())])
    seq_kv, _ = keep.int_array([0, 0, 0])  # stale plan-time lengths; the bound device array wins
    result = torch.zeros(3, heads, LATENT, dtype=torch.bfloat16, device="cuda")
    t_res = keep.tensor([3, heads, LATENT], acl.ACL_BF16, result.data_ptr())
    scale = 1.0 / math.sqrt(192.0)
    status, ws_bytes, ex = acl.plan_attention(t_q, klist, vlist, None, seq_kv, t_table, t_qr, t_rope, heads, scale, bs, t_res)
    _ok(status)
    _ok(lib.aclnnMlaKvBindSeqLens(ex, lens_dev.data_ptr()))
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    _ok(lib.aclnnFusedInferAttentionScoreV5(workspace.data_ptr(), ws_bytes, ex, kt.stream_ptr()))
    torch.cuda.synchronize()
    expected, _ = kt.oracle_attention(cache, 0, q, table, ctxs, scale)
    got = result.float().cpu().numpy()
    assert np.abs(got - expected).max() <= 2e-2 * np.abs(expected).max()
    _ok(lib.aclDestroyAclOpExecutor(ex))
