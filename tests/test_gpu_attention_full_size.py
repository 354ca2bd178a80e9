"""GPU parity of the decode attention at the full size of the ragged configurations, on the very
length draws bench.py times (same generator, same seed):
  configs[3]: batch 64, contexts uniform in [512, 8192], FP8 latent KV, N(0,1) rows with 1 % of the
              elements x20, 64 heads;
  configs[4]: batch 128, contexts lognormal (median 4096, sigma 1.0, capped at 32768), bf16, 64 heads;
and of the batch walk in windows of 64 sequences on cheap shapes (65 .. 130 short sequences with
empty ones among them, forced unit lengths and workgroup counts, both merges).
Every sequence is checked against a float32 torch evaluation of the formula on the GPU (a library
routine; for FP8 on the rows the cache really holds, as the dequantising gather returns them), a
sample that includes the shortest and the longest against the float64 oracle. Tolerances from the
target statement: 2e-2 of the peak for bf16 KV, 6e-2 for FP8 KV.
Operator contract: include/moe/core/op_table.hpp:375-454; stage src/pipeline/pipeline.cpp:235-249."""
import ctypes as C
import math
import os
import sys

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402  (draw_contexts and CONTEXT_SEED: the lengths the benchmark times)

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE
SCALE = 1.0 / math.sqrt(192.0)
TOL_BF16, TOL_FP8 = 2e-2, 6e-2


def _fill(cache, table, ctxs, seed, outlier_fraction):
    """N(0,1) rows (optionally 1 % of the elements x20) into every live slot, through the append
    kernel (an FP8 cache quantises on the way), in pieces of 128k rows."""
    slots = kt.dev_i32(kt.slots_for(table, ctxs, cache.block_size))
    gen = torch.Generator(device="cuda").manual_seed(seed)
    piece = 128 * 1024
    for start in range(0, slots.numel(), piece):
        rows = min(piece, slots.numel() - start)
        x = torch.randn(rows, LATENT + ROPE, generator=gen, device="cuda")
        if outlier_fraction > 0:
            x = torch.where(torch.rand(rows, LATENT + ROPE, generator=gen, device="cuda") < outlier_fraction, x * 20.0, x)
        x = x.to(torch.bfloat16)
        kt.append(cache, x[None, :, :LATENT], x[None, :, LATENT:], slots[start:start + rows])
        torch.cuda.synchronize()


def _torch_check(out, lse, q, lat_rows, rope_rows, ctxs, tol):
    """Every sequence against softmax(q k^T scale) v in float32 on the GPU."""
    worst, start = 0.0, 0
    for b, n in enumerate(ctxs):
        lat, rope = lat_rows[start:start + n].float(), rope_rows[start:start + n].float()
        scores = (q[b, :, :LATENT].float() @ lat.T + q[b, :, LATENT:].float() @ rope.T) * SCALE
        ref = torch.softmax(scores, dim=-1) @ lat
        peak = ref.abs().max().item()
        err = (out[b].float() - ref).abs().max().item()
        assert err <= tol * peak, (b, n, err, peak)
        assert (lse[b] - torch.logsumexp(scores, dim=-1)).abs().max().item() <= (6e-2 if tol == TOL_FP8 else 2e-2), (b, n)
        worst = max(worst, err / peak)
        start += n
    return worst


def _oracle_check(cache, out, q, table, ctxs, sample, tol):
    for b in sample:
        heads = q.shape[1] if ctxs[b] <= 8192 else 16   # the float64 loop over 32768 tokens: a quarter of the heads
        expected, _ = kt.oracle_attention(cache, 0, q[b:b + 1, :heads].contiguous(), table[b:b + 1], [ctxs[b]], SCALE)
        got = out[b:b + 1, :heads].float().cpu().numpy()
        peak = np.abs(expected).max()
        assert np.abs(got - expected).max() <= tol * peak, (b, ctxs[b])


def _host_lens_launch(plan, cache, q, table_d, ctxs):
    heads, row = q.shape[1], (LATENT + ROPE) * 2
    ws = torch.empty(int(plan.workspace_bytes), dtype=torch.uint8, device="cuda")
    out = torch.full((len(ctxs), heads, LATENT), float("nan"), dtype=torch.bfloat16, device="cuda")
    host = (C.c_int32 * len(ctxs))(*ctxs)
    ffi.check(ffi.load().mlakvAttnDecodeHostLens(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                                 q.data_ptr() + LATENT * 2, heads * row, row, table_d.data_ptr(), table_d.shape[1],
                                                 C.cast(host, C.c_void_p), SCALE, out.data_ptr(), heads * LATENT * 2, LATENT * 2,
                                                 None, ws.data_ptr(), ws.numel(), kt.stream_ptr()))
    torch.cuda.synchronize()
    return out


def _sample(ctxs):
    order = np.argsort(ctxs)
    return sorted({int(order[0]), int(order[-1]), int(order[len(order) // 2]), int(order[len(order) // 4])})


def test_configs3_full_size_fp8_ragged():
    bs, heads = 64, 64
    ctxs = bench.draw_contexts(np, "uniform_512_8192", 64, bench.CONTEXT_SEED)
    assert len(ctxs) == 64 and min(ctxs) >= 512 and max(ctxs) <= 8192
    blocks = sum(-(-c // bs) for c in ctxs) + 8
    table = kt.build_tables(ctxs, bs, blocks, seed=7).table()
    cache = kt.PagedCache(1, blocks, bs, fp8=True)
    _fill(cache, table, ctxs, seed=2, outlier_fraction=0.01)
    q = torch.randn(64, heads, LATENT + ROPE, generator=torch.Generator(device="cuda").manual_seed(3), device="cuda").to(torch.bfloat16)
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    out, lse, plan = kt.attention(cache, 0, q, table_d, lens_d, SCALE)
    assert plan.work_groups >= 64 and plan.merge_mode == ffi.ATTN_MERGE_SECOND_LAUNCH
    lat_rows, rope_rows = kt.gather(cache, table_d, lens_d)      # what the cache holds, dequantised
    worst = _torch_check(out, lse, q, lat_rows[0], rope_rows[0], ctxs, TOL_FP8)
    _oracle_check(cache, out, q, table, ctxs, _sample(ctxs), TOL_FP8)
    # the same launch with the lengths in the argument block, and with the merge inside the launch
    assert torch.equal(_host_lens_launch(plan, cache, q, table_d, ctxs).view(torch.int16), out.view(torch.int16))
    merged, lse_m, _ = kt.attention(cache, 0, q, table_d, lens_d, SCALE, merge_mode=ffi.ATTN_MERGE_IN_LAUNCH)
    assert torch.equal(merged.view(torch.int16), out.view(torch.int16)) and torch.equal(lse_m, lse)
    print(f"configs[3] full size: {sum(ctxs)} tokens, worst error {worst:.2e} of the peak (tolerance {TOL_FP8})")


def test_configs4_full_size_bf16_lognormal():
    bs, heads = 64, 64
    ctxs = bench.draw_contexts(np, "lognormal_4096_cap_32768", 128, bench.CONTEXT_SEED)
    assert len(ctxs) == 128 and max(ctxs) <= 32768
    blocks = sum(-(-c // bs) for c in ctxs) + 8
    table = kt.build_tables(ctxs, bs, blocks, seed=7).table()
    cache = kt.PagedCache(1, blocks, bs)
    _fill(cache, table, ctxs, seed=2, outlier_fraction=0.0)
    q = torch.randn(128, heads, LATENT + ROPE, generator=torch.Generator(device="cuda").manual_seed(3), device="cuda").to(torch.bfloat16)
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    out, lse, plan = kt.attention(cache, 0, q, table_d, lens_d, SCALE)   # two windows of 64 sequences
    lat_rows, rope_rows = kt.gather(cache, table_d, lens_d)
    worst = _torch_check(out, lse, q, lat_rows[0], rope_rows[0], ctxs, TOL_BF16)
    del lat_rows, rope_rows
    _oracle_check(cache, out, q, table, ctxs, _sample(ctxs), TOL_BF16)
    merged, lse_m, _ = kt.attention(cache, 0, q, table_d, lens_d, SCALE, merge_mode=ffi.ATTN_MERGE_IN_LAUNCH)
    assert torch.equal(merged.view(torch.int16), out.view(torch.int16)) and torch.equal(lse_m, lse)
    print(f"configs[4] full size: {sum(ctxs)} tokens, longest {max(ctxs)}, worst error {worst:.2e} of the peak (tolerance {TOL_BF16})")


@pytest.mark.parametrize("batch,fp8,options", [
    (65, False, {}),
    (97, True, {"chunk_tiles": 1, "work_groups": 5}),
    (130, False, {"chunk_tiles": 3, "work_groups": 64}),
    (130, True, {"chunk_tiles": 2, "work_groups": 7, "merge_mode": ffi.ATTN_MERGE_IN_LAUNCH}),
    (128, False, {"chunk_tiles": 1, "merge_mode": ffi.ATTN_MERGE_IN_LAUNCH, "merge_spin_us": -1}),
    (129, False, {"work_groups": 3}),
])
def test_more_than_one_window_of_sequences(batch, fp8, options):
    """The kernels walk the batch 64 sequences at a time; here the units, the empty sequences and
    the merges cross those windows. Everything against the float64 oracle."""
    bs, heads = 64, 32
    rng = np.random.default_rng(500 + batch)
    ctxs = [int(v) for v in rng.integers(1, 200, size=batch)]
    for b in rng.choice(batch, size=batch // 8, replace=False):
        ctxs[int(b)] = 0                                   # empty sequences, some at the window edges
    ctxs[63], ctxs[64] = 0, 190
    ctxs[batch - 1] = 170
    blocks = sum(-(-c // bs) for c in ctxs) + 4
    table = kt.build_tables(ctxs, bs, blocks, seed=batch).table()
    cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
    _fill(cache, table, ctxs, seed=batch + 1, outlier_fraction=0.01 if fp8 else 0.0)
    q = kt.randn_bf16((batch, heads, LATENT + ROPE), seed=batch + 2).cuda()
    out, lse, _ = kt.attention(cache, 0, q, kt.dev_i32(table), kt.dev_i32(ctxs), SCALE, **options)
    expected, expected_lse = kt.oracle_attention(cache, 0, q, table, ctxs, SCALE)
    live = np.array(ctxs) > 0
    got = out.float().cpu().numpy()
    assert np.abs(got[~live]).max() == 0.0
    tol = TOL_FP8 if fp8 else TOL_BF16
    peak = np.abs(expected[live]).max()
    assert np.abs(got[live] - expected[live]).max() <= tol * peak
    assert np.abs(lse.cpu().numpy()[live] - expected_lse[live]).max() <= (6e-2 if fp8 else 2e-2)
