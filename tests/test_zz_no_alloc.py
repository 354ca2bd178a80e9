"""GPU: the allocation-free attention entry point (mlakvAttnDecodeNoAlloc: split-KV partials in
the library's static device array) against mlakvAttnDecode with a caller workspace, bit for
bit, on two calls in a row, the second with a smaller input. Collected last on purpose."""
import ctypes as C
import math

import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE
SCALE = 1.0 / math.sqrt(192.0)


def _case(ctxs, heads, bs, seed):
    blocks = sum(-(-c // bs) for c in ctxs) + 3
    pool = kt.build_tables(ctxs, bs, blocks, seed=seed)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    total = sum(ctxs)
    latent = kt.randn_bf16((1, total, LATENT), seed=seed + 1).cuda()
    rope = kt.randn_bf16((1, total, ROPE), seed=seed + 2).cuda()
    kt.append(cache, latent, rope, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=seed + 3).cuda()
    return cache, q, kt.dev_i32(table), kt.dev_i32(ctxs)


def _no_alloc(cache, q, table, lens, max_seq_len):
    lib = ffi.load()
    batch, heads = q.shape[0], q.shape[1]
    plan = ffi.AttnPlan()
    ffi.check(lib.mlakvAttnPlanInit(batch, heads, max_seq_len, cache.block_size, ffi.DTYPE_BF16, C.byref(plan)))
    out = torch.full((batch, heads, LATENT), float("nan"), dtype=torch.bfloat16, device="cuda")
    lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device="cuda")
    row = (LATENT + ROPE) * 2
    def call():
        ffi.check(lib.mlakvAttnDecodeNoAlloc(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                             q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), table.shape[1],
                                             lens.data_ptr(), float(SCALE), out.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                             lse.data_ptr(), kt.stream_ptr()))
    # Once untimed: the kernels are loaded onto the device and the static array's address is resolved
    # (one-time set-up, which may take device memory for the code). Then the call is bracketed with
    # the driver's own count of free device memory (hipMemGetInfo): a hipMalloc inside the library
    # would lower it, whatever torch's allocator knows; torch's counter is watched as well.
    ffi.check(lib.mlakvPrepare())
    call()
    torch.cuda.synchronize()
    out.fill_(float("nan"))
    lse.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    allocated_before = torch.cuda.memory_allocated()
    call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"free device memory went from {free_before} to {free_after} bytes across the call"
    assert torch.cuda.memory_allocated() == allocated_before
    return out, lse, plan


def test_no_alloc_entry_matches_workspace_entry_twice():
    # first call: several chunks per sequence (partials fill a good part of the scratch);
    # second call: a smaller batch with shorter contexts, which must not see the first call's partials
    for ctxs, heads in (([1500, 2048, 700, 64, 1, 1999], 64), ([130, 300], 32)):
        cache, q, table, lens = _case(ctxs, heads, 64, seed=len(ctxs))
        expected, expected_lse, plan = kt.attention(cache, 0, q, table, lens, SCALE, max_seq_len=max(ctxs))
        got, got_lse, plan2 = _no_alloc(cache, q, table, lens, max(ctxs))
        assert plan2.max_units == plan.max_units and plan2.workspace_bytes == plan.workspace_bytes
        assert torch.equal(got, expected)
        assert torch.equal(got_lse, expected_lse)


def test_no_alloc_entry_refuses_a_plan_beyond_its_scratch():
    lib = ffi.load()
    cache, q, table, lens = _case([100], 64, 64, seed=9)
    plan = ffi.AttnPlan()
    # 4096 sequences of 16384 tokens: far more partial rows than the static array holds
    ffi.check(lib.mlakvAttnPlanInit(4096, 128, 1 << 20, 64, ffi.DTYPE_BF16, C.byref(plan)))
    assert plan.workspace_bytes > 24 << 20
    status = lib.mlakvAttnDecodeNoAlloc(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), 64 * 1152, 1152,
                                        q.data_ptr() + 1024, 64 * 1152, 1152, table.data_ptr(), table.shape[1],
                                        lens.data_ptr(), float(SCALE), q.data_ptr(), 64 * 1024, 1024, None, kt.stream_ptr())
    assert status == ffi.ERR_PARAM_INVALID
    assert b"static scratch" in lib.mlakvGetLastError()
