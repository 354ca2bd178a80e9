"""A decode step captured once as a HIP graph and replayed: the append of one row per sequence, the
whole-context attention (decode kernel + merge launch) and the selected-token attention in halved
whole-selection units (whose workgroups meet on the library's counters). Every replay runs on new
inputs written into the captured buffers, with eager work and a device synchronisation between
replays, and is compared with the same calls made eagerly: bit for bit, since every kernel here is
deterministic. The library's entry points only enqueue kernels, so nothing else may appear in the
graph (no memset nodes, no copies)."""
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


def _calls(lib, cache, state, stream):
    """The step: append, whole-context attention, selected-token attention; on `stream`."""
    heads, row = state["heads"], (LATENT + ROPE) * 2
    q, table, lens = state["q"], state["table"], state["lens"]
    ffi.check(lib.mlakvAppend(C.byref(cache.view), 0, 1, state["new_latent"].data_ptr(), state["new_latent"].stride(0) * 2,
                              state["new_latent"].stride(1) * 2, state["new_rope"].data_ptr(), state["new_rope"].stride(0) * 2,
                              state["new_rope"].stride(1) * 2, state["slots"].data_ptr(), state["slots"].numel(), stream))
    ffi.check(lib.mlakvAttnDecode(C.byref(state["plan"]), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                  q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), table.shape[1], lens.data_ptr(),
                                  float(SCALE), state["out"].data_ptr(), heads * LATENT * 2, LATENT * 2, state["lse"].data_ptr(),
                                  state["workspace"].data_ptr(), int(state["plan"].workspace_bytes), stream))
    ffi.check(lib.mlakvAttnDecodeSparse(C.byref(state["sparse_plan"]), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                        q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), table.shape[1],
                                        lens.data_ptr(), state["selection"].data_ptr(), state["selection"].stride(0), float(SCALE),
                                        state["sparse_out"].data_ptr(), heads * LATENT * 2, LATENT * 2, state["sparse_lse"].data_ptr(),
                                        state["sparse_workspace"].data_ptr(), int(state["sparse_plan"].workspace_bytes), stream))


def test_a_captured_decode_step_replays_like_eager_calls():
    lib = ffi.load()
    bs, heads, k = 64, 64, 512
    ctxs = [1500, 700, 2047, 64, 1, 900, 1300, 513]
    batch = len(ctxs)
    blocks = sum(-(-(n + 8) // bs) for n in ctxs) + 4
    pool = kt.build_tables([n + 8 for n in ctxs], bs, blocks, seed=11)   # room for the rows the replays append
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs)
    total = sum(ctxs)
    kt.append(cache, kt.randn_bf16((1, total, LATENT), seed=12).cuda(), kt.randn_bf16((1, total, ROPE), seed=13).cuda(),
              kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    torch.cuda.synchronize()
    twin = kt.PagedCache(1, blocks, bs)        # the eager calls get a cache of their own with the same bytes
    twin.latent.copy_(cache.latent)
    twin.rope.copy_(cache.rope)

    def make_state():
        plan = kt.make_plan(batch, heads, 2048 + 8, bs, False)
        sparse_plan = kt.make_plan(batch, heads, k, bs, False, selection=True)
        assert sparse_plan.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK_HALVES
        return {"heads": heads, "plan": plan, "sparse_plan": sparse_plan,
                "q": torch.zeros(batch, heads, LATENT + ROPE, dtype=torch.bfloat16, device="cuda"),
                "table": kt.dev_i32(table), "lens": torch.zeros(batch, dtype=torch.int32, device="cuda"),
                "slots": torch.zeros(batch, dtype=torch.int32, device="cuda"),
                "new_latent": torch.zeros(1, batch, LATENT, dtype=torch.bfloat16, device="cuda"),
                "new_rope": torch.zeros(1, batch, ROPE, dtype=torch.bfloat16, device="cuda"),
                "selection": torch.full((batch, k), -1, dtype=torch.int32, device="cuda"),
                "out": torch.zeros(batch, heads, LATENT, dtype=torch.bfloat16, device="cuda"),
                "lse": torch.zeros(batch, heads, dtype=torch.float32, device="cuda"),
                "sparse_out": torch.zeros(batch, heads, LATENT, dtype=torch.bfloat16, device="cuda"),
                "sparse_lse": torch.zeros(batch, heads, dtype=torch.float32, device="cuda"),
                "workspace": torch.empty(int(plan.workspace_bytes), dtype=torch.uint8, device="cuda"),
                "sparse_workspace": torch.empty(int(sparse_plan.workspace_bytes), dtype=torch.uint8, device="cuda")}

    def set_inputs(state, step):
        """Step `step`: every sequence gets one more row; new query, new selection."""
        lens = [n + step + 1 for n in ctxs]
        rng = np.random.default_rng(100 + step)
        selection = np.full((batch, k), -1, dtype=np.int32)
        for s, n in enumerate(lens):
            take = min(n, k)
            selection[s, :take] = rng.permutation(n)[:take]
        slots = [int(table[s, (n - 1) // bs]) * bs + (n - 1) % bs for s, n in enumerate(lens)]
        state["q"].copy_(kt.randn_bf16((batch, heads, LATENT + ROPE), seed=200 + step).cuda())
        state["new_latent"].copy_(kt.randn_bf16((1, batch, LATENT), seed=300 + step).cuda())
        state["new_rope"].copy_(kt.randn_bf16((1, batch, ROPE), seed=400 + step).cuda())
        state["lens"].copy_(kt.dev_i32(lens))
        state["slots"].copy_(kt.dev_i32(slots))
        state["selection"].copy_(kt.dev_i32(selection))
        for name in ("out", "sparse_out"):
            state[name].fill_(float("nan"))
        return lens, selection

    captured, eager = make_state(), make_state()
    side = torch.cuda.Stream()
    # Everything the library sets up on first use (kernel attributes, the counters' address) happens in
    # eager calls before the capture.
    set_inputs(eager, 0)
    _calls(lib, twin, eager, kt.stream_ptr())
    torch.cuda.synchronize()
    twin.latent.copy_(cache.latent)
    twin.rope.copy_(cache.rope)

    set_inputs(captured, 0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _calls(lib, cache, captured, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    cache.latent.copy_(twin.latent)       # (the capture itself runs nothing; keep the two caches equal whatever it did)
    cache.rope.copy_(twin.rope)

    for step in range(5):
        lens, selection = set_inputs(captured, step)
        set_inputs(eager, step)
        graph.replay()
        _calls(lib, twin, eager, kt.stream_ptr())
        torch.cuda.synchronize()
        assert torch.equal(cache.latent, twin.latent) and torch.equal(cache.rope, twin.rope), step
        for name in ("out", "lse", "sparse_out", "sparse_lse"):
            assert torch.equal(captured[name], eager[name]), (step, name)
        if step in (0, 4):                 # and the eager calls are right
            expected, _ = kt.oracle_attention(twin, 0, eager["q"], table, lens, SCALE)
            got = eager["out"].float().cpu().numpy()
            assert np.abs(got - expected).max() <= 2e-2 * np.abs(expected).max()
            expected, _ = kt.oracle_attention(twin, 0, eager["q"], table, lens, SCALE, sparse_indices=selection)
            got = eager["sparse_out"].float().cpu().numpy()
            assert np.abs(got - expected).max() <= 2e-2 * np.abs(expected).max()
        # eager work of the program's own between replays
        torch.zeros(1 << 20, device="cuda").sum().item()
