#!/usr/bin/env python3
"""Benchmark of the paged MLA KV-cache hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input, for the workload the
headline metric is quoted on (BASELINE.json configs[1]):
    43 layers, batch 32, contexts uniform in [128, 2048], block 64, seeded-shuffled free list,
    bf16 rows of 576 elements (512 latent + 64 rope); per step: host block-pool bookkeeping,
    metadata upload, append of one row per sequence per layer, gather of every sequence's
    full context into contiguous [sum ctx, 576] rows per layer.
`value` is algorithmic bytes per step / wall time per step with all inputs resident in HBM.
The decode-attention configuration (configs[2]: batch 32, 64 heads, context 2048) is timed in
the same run and reported under "attention" (us per launch and fraction of the HBM roofline);
launches rotate over 8 layer slices (604 MB) so the 256 MB Infinity Cache cannot hold the KV.

Prints ONE JSON line. Everything goes through the C ABI (include/mlakv.h); the CPU oracle is
used only for the cpu_baseline leg.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ascend-moe-engine_amd", "python"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

# HBM bytes per algorithmic byte of the gather kernel, from two rocprofv3 --pmc runs of this file
# (FETCH_SIZE scaled by 2.000, WRITE_SIZE by 1.000, the factors a plain 1 GiB copy gives):
# (1956.8 + 1956.7) MB measured per dispatch against 3912.4 MB algorithmic.
GATHER_TRAFFIC_PER_ALGORITHMIC_BYTE = 1.0003
HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0
LATENT, ROPE, ROW = 512, 64, 576
ROW_BYTES = ROW * 2


def sustained_us(torch, fn, min_iters, warm_ms=250.0, timed_ms=100.0):
    """Average microseconds per fn(i) launch once the device has settled: launches get faster for
    some 100 ms of sustained load (the long attention shape measured 284 us per launch over 2
    launches, 254 over 32, 227 over 512; most likely clock and power management), so the launches
    run back to back for `warm_ms` before the timed ones, which then cover at least `timed_ms`."""
    def run(n):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(n):
            fn(i)
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1e3 / n
    rough = run(16)
    run(max(16, int(warm_ms * 1e3 / rough)))
    return run(max(min_iters, int(timed_ms * 1e3 / rough)))


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=60)
    p.add_argument("--warmup", type=int, default=60)
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-attention", action="store_true")
    p.add_argument("--side-only", action="store_true", help="development aid: time only the FP8 append/gather and compaction kernels")
    p.add_argument("--attention-only", action="store_true", help="development aid: time only the attention configurations")
    p.add_argument("--split-out", action="store_true", help="gather into separate latent/rope planes instead of 576-wide rows")
    return p.parse_args()


def stream_ptr(torch):
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def bench_append_gather(args, torch, np, ffi):
    lib = ffi.load()
    layers, batch, bs = 43, 32, 64
    rng = np.random.default_rng(20251125)
    ctxs = [int(v) for v in rng.integers(128, 2049, size=batch)]
    total_steps = args.warmup + args.steps
    max_ctx = 2048 + max(128, -(-total_steps // bs) * bs)  # every sequence grows by one token per step
    pool_blocks = sum(-(-(c + total_steps) // bs) for c in ctxs) + 32
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=max_ctx, max_batch=batch,
                        pool_blocks=pool_blocks, seed=20251125, shuffle=1)
    arena.commit()
    cache.bind()
    arena.seal()
    view = cache.view()
    for s, n in enumerate(ctxs):
        cache.add_sequence(s, n)
    gen = torch.Generator(device="cuda").manual_seed(1)
    # prefill the pool with N(0,1) rows so the gather reads real data
    total = sum(ctxs)
    table = cache.host_block_table()
    slots = np.concatenate([table[s, np.arange(n) // bs].astype(np.int64) * bs + np.arange(n) % bs
                            for s, n in enumerate(ctxs)]).astype(np.int32)
    slots_dev = torch.as_tensor(slots, device="cuda")
    for layer in range(layers):
        lat = torch.randn(total, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
        rop = torch.randn(total, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
        ffi.check(lib.mlakvAppend(C.byref(view), layer, 1, lat.data_ptr(), 0, LATENT * 2, rop.data_ptr(), 0, ROPE * 2,
                                  slots_dev.data_ptr(), total, stream_ptr(torch)))
        torch.cuda.synchronize()
    step_latent = torch.randn(layers, batch, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
    step_rope = torch.randn(layers, batch, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    rows_cap = total + batch * total_steps
    if args.split_out:
        out_latent = torch.empty(layers, rows_cap, LATENT, dtype=torch.bfloat16, device="cuda")
        out_rope = torch.empty(layers, rows_cap, ROPE, dtype=torch.bfloat16, device="cuda")
        dst = (out_latent.data_ptr(), rows_cap * LATENT * 2, LATENT * 2, out_rope.data_ptr(), rows_cap * ROPE * 2, ROPE * 2)
    else:
        out = torch.empty(layers, rows_cap, ROW, dtype=torch.bfloat16, device="cuda")
        dst = (out.data_ptr(), rows_cap * ROW_BYTES, ROW_BYTES, out.data_ptr() + LATENT * 2, rows_cap * ROW_BYTES, ROW_BYTES)
    allocations_before = arena.device_allocations
    gather_events = []

    def step(timed):
        for s in range(batch):
            cache.append_token(s)
        cache.upload_step(stream_ptr(torch))
        # events bracket the gather only: every record is a barrier packet in the queue, and a third
        # one in front of the 4-us append cost more than the append itself
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)] if timed else None
        ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, step_latent.data_ptr(), batch * LATENT * 2, LATENT * 2,
                                  step_rope.data_ptr(), batch * ROPE * 2, ROPE * 2, cache.device_slot_mapping, batch,
                                  stream_ptr(torch)))
        if timed:
            ev[0].record()
        ffi.check(lib.mlakvGather(C.byref(view), 0, layers, cache.device_block_table, cache.num_blocks,
                                  cache.device_seq_lens, cache.device_cu_seq_lens, batch, max_ctx, dst[0], dst[1], dst[2],
                                  dst[3], dst[4], dst[5], stream_ptr(torch)))
        if timed:
            ev[1].record()
            gather_events.append((ev[0], ev[1]))

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    rows_per_step = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(True)
        rows_per_step.append(total + batch * (args.warmup + i + 1))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert arena.device_allocations == allocations_before, "a step allocated device memory"

    blocks_per_step = []
    lens = cache.host_seq_lens()
    # algorithmic bytes: append 2*R*row + 4*R; gather 2*sum(ctx)*row + 4*sum(ceil(ctx/bs)), per layer
    def gather_bytes(rows, final_lens, back):
        nblk = sum(-(-(int(l) - back) // bs) for l in final_lens)
        return layers * (2 * rows * ROW_BYTES + 4 * nblk)
    append_bytes = layers * (2 * batch * ROW_BYTES + 4 * batch)
    g_bytes = [gather_bytes(rows_per_step[i], lens, args.steps - 1 - i) for i in range(args.steps)]
    total_bytes = sum(g_bytes) + append_bytes * args.steps
    gather_ms = [a.elapsed_time(b) for a, b in gather_events]
    # the append launch on its own, after the timed region: the same rows to the same slots again,
    # 64 launches back to back between two events (one launch between two events times the events)
    def append_again():
        ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, step_latent.data_ptr(), batch * LATENT * 2, LATENT * 2,
                                  step_rope.data_ptr(), batch * ROPE * 2, ROPE * 2, cache.device_slot_mapping, batch,
                                  stream_ptr(torch)))
    for _ in range(8):
        append_again()
    torch.cuda.synchronize()
    pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    pair[0].record()
    for _ in range(64):
        append_again()
    pair[1].record()
    torch.cuda.synchronize()
    append_ms = [pair[0].elapsed_time(pair[1]) / 64]
    gather_gbps = sum(g_bytes) / (sum(gather_ms) * 1e-3) / 1e9
    result = {
        "value": total_bytes / elapsed / 1e9,
        "ms_per_step": elapsed / args.steps * 1e3,
        "gather_ms": sum(gather_ms) / len(gather_ms),
        "append_ms": sum(append_ms) / len(append_ms),
        "gather_gbps": gather_gbps,
        "append_gbps": append_bytes / (sum(append_ms) / len(append_ms) * 1e-3) / 1e9,
        "bytes_per_step": total_bytes / args.steps,
        "gather_bytes_per_launch": sum(g_bytes) / args.steps,
        "mean_ctx": sum(rows_per_step) / len(rows_per_step) / batch,
        "ctxs": ctxs, "pool_blocks": pool_blocks, "seed": 20251125,
    }
    cache.close()
    arena.close()
    return result


def bench_attention(args, torch, np, ffi, fp8=False, batch=32, ctx=2048, heads=64, slices=8, iters=None, label=None,
                    mx_quant=False, sparse_k=None):
    lib = ffi.load()
    bs = 64
    slices = int(os.environ.get("MLAKV_BENCH_SLICES", slices))  # development aid: 1 keeps the KV cache-resident
    blocks_per_seq = -(-ctx // bs)
    pool_blocks = batch * blocks_per_seq + 8
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=slices, block_size=bs, max_context_len=ctx, max_batch=batch,
                        pool_blocks=pool_blocks, seed=7, shuffle=int(os.environ.get("MLAKV_BENCH_SHUFFLE", "1")),
                        dtype=ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16)
    plan = ffi.AttnPlan()
    if sparse_k:
        ffi.check(lib.mlakvAttnSparsePlanInit(batch, heads, sparse_k, bs, cache.config.dtype, C.byref(plan)))
    else:
        ffi.check(lib.mlakvAttnPlanInit(batch, heads, ctx, bs, cache.config.dtype, C.byref(plan)))
    arena.note_workspace(int(plan.workspace_bytes))
    arena.commit()
    arena.commit_workspace()
    cache.bind()
    arena.seal()
    view = cache.view()
    for s in range(batch):
        cache.add_sequence(s, ctx)
    cache.upload_step(stream_ptr(torch))
    table = cache.host_block_table()
    slots = np.concatenate([table[s, np.arange(ctx) // bs].astype(np.int64) * bs + np.arange(ctx) % bs
                            for s in range(batch)]).astype(np.int32)
    slots_dev = torch.as_tensor(slots, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(2)
    for layer in range(slices):
        lat = torch.randn(batch * ctx, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
        rop = torch.randn(batch * ctx, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
        ffi.check(lib.mlakvAppend(C.byref(view), layer, 1, lat.data_ptr(), 0, LATENT * 2, rop.data_ptr(), 0, ROPE * 2,
                                  slots_dev.data_ptr(), batch * ctx, stream_ptr(torch)))
        torch.cuda.synchronize()
    q = torch.randn(slices, batch, heads, ROW, generator=gen, device="cuda").to(torch.bfloat16)
    out = torch.empty(slices, batch, heads, LATENT, dtype=torch.bfloat16, device="cuda")

    selection = None
    if sparse_k:
        # every sequence attends to sparse_k distinct random positions of its context (what a
        # top-k selection looks like to the memory system), a fresh draw per layer slice
        rng = np.random.default_rng(5)
        selection = torch.as_tensor(np.stack([np.stack([rng.permutation(ctx)[:sparse_k] for _ in range(batch)])
                                              for _ in range(slices)]).astype(np.int32), device="cuda")

    def launch_sparse(i):
        k = i % slices
        ffi.check(lib.mlakvAttnDecodeSparse(C.byref(plan), C.byref(view), k, q[k].data_ptr(), heads * ROW_BYTES, ROW_BYTES,
                                            q[k].data_ptr() + LATENT * 2, heads * ROW_BYTES, ROW_BYTES,
                                            cache.device_block_table, cache.num_blocks, cache.device_seq_lens,
                                            selection[k].data_ptr(), sparse_k, 1.0 / math.sqrt(192.0), out[k].data_ptr(),
                                            heads * LATENT * 2, LATENT * 2, None, arena.workspace, arena.workspace_bytes,
                                            stream_ptr(torch)))

    def launch(i):
        if sparse_k:
            return launch_sparse(i)
        k = i % slices
        ffi.check(lib.mlakvAttnDecode(C.byref(plan), C.byref(view), k, q[k].data_ptr(), heads * ROW_BYTES, ROW_BYTES,
                                      q[k].data_ptr() + LATENT * 2, heads * ROW_BYTES, ROW_BYTES,
                                      cache.device_block_table, cache.num_blocks, cache.device_seq_lens,
                                      1.0 / math.sqrt(192.0), out[k].data_ptr(), heads * LATENT * 2, LATENT * 2, None,
                                      arena.workspace, arena.workspace_bytes, stream_ptr(torch)))

    iters = iters or max(args.steps * 8, 64)

    def timed_us(fn):
        return sustained_us(torch, fn, iters)

    us = timed_us(launch)
    mx = None
    if mx_quant:
        # the reference's next stage, block-32 MX quantisation of the output: fused into the
        # attention epilogue, against attention followed by the standalone operator
        codes = torch.empty(slices, batch, heads, LATENT, dtype=torch.uint8, device="cuda")
        scales = torch.empty(slices, batch, heads, LATENT // 32, dtype=torch.uint8, device="cuda")
        targets = [ffi.MxQuantOut(codes[k].data_ptr(), heads * LATENT, LATENT, scales[k].data_ptr(), heads * (LATENT // 32),
                                  LATENT // 32) for k in range(slices)]

        def fused(i):
            k = i % slices
            ffi.check(lib.mlakvAttnDecodeMxQuant(C.byref(plan), C.byref(view), k, q[k].data_ptr(), heads * ROW_BYTES, ROW_BYTES,
                                                 q[k].data_ptr() + LATENT * 2, heads * ROW_BYTES, ROW_BYTES,
                                                 cache.device_block_table, cache.num_blocks, cache.device_seq_lens,
                                                 1.0 / math.sqrt(192.0), None, 0, 0, C.byref(targets[k]), None,
                                                 arena.workspace, arena.workspace_bytes, stream_ptr(torch)))

        def unfused(i):
            k = i % slices
            launch(i)
            ffi.check(lib.mlakvDynamicMxQuant(out[k].data_ptr(), LATENT * 2, batch * heads, LATENT, codes[k].data_ptr(), LATENT,
                                              scales[k].data_ptr(), LATENT // 32, stream_ptr(torch)))

        mx = {"us_fused_epilogue": timed_us(fused), "us_attention_then_quant": timed_us(unfused)}
    kv_row = 580 if fp8 else ROW_BYTES
    attended = sparse_k or ctx
    algorithmic = batch * attended * kv_row + batch * heads * ROW * 2 + batch * heads * LATENT * 2 + 4 * batch * blocks_per_seq
    if sparse_k:
        algorithmic += 4 * batch * sparse_k
    flops = 2.0 * batch * heads * attended * (ROW + LATENT)
    result = {
        "us_per_step": us,
        "workload": f"{label or ('configs[3]-shape' if fp8 else 'configs[2]-shape')}: 1 layer per launch, batch {batch}, {heads} heads, ctx {ctx}, block 64, "
                    f"{'fp8 e4m3 + fp32 row scale' if fp8 else 'bf16'} KV, shuffled table, {slices} rotating layer slices"
                    + (f", {sparse_k} selected tokens per sequence" if sparse_k else ""),
        "roofline": {"bound": "hbm", "achieved": algorithmic / (us * 1e-6) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": algorithmic / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, "traffic": None},
        "algorithmic_bytes": algorithmic,
        "mfma_tflops": flops / (us * 1e-6) / 1e12,
        "mfma_frac_of_bf16_peak": flops / (us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "work_groups": int(plan.work_groups), "max_units": int(plan.max_units),
        "merge": "in launch" if plan.merge_mode == ffi.ATTN_MERGE_IN_LAUNCH else "second launch",
        "workspace_bytes": int(plan.workspace_bytes), "timing": "250 ms of back-to-back launches untimed, then at least 100 ms of them timed",
    }
    if mx is not None:
        result["mx_quant_output"] = mx
    cache.close()
    arena.close()
    return result


def bench_indexer(args, torch, np, ffi, batch=32, ctx=8192, heads=64, k=512, bs=64, slices=4):
    """Lightning Indexer at the shape the selected-token attention is timed on: FP8 index keys
    (128 + 4 bytes per cached token) scored against one query token per sequence, top-k selected.
    HIP-event time of the operator (score kernel + selection kernel) over rotating key pools."""
    lib = ffi.load()
    blocks = batch * (ctx // bs)
    rng = np.random.default_rng(9)
    keys = [torch.randint(0, 0x58, (blocks * bs, 128), dtype=torch.uint8, device="cuda") for _ in range(slices)]
    scales = torch.rand(blocks * bs, device="cuda") * 0.04 + 0.01
    table = torch.as_tensor(rng.permutation(blocks).astype(np.int32).reshape(batch, ctx // bs), device="cuda")
    lens = torch.full((batch,), ctx, dtype=torch.int32, device="cuda")
    query = torch.randint(0, 0x58, (batch, heads, 128), dtype=torch.uint8, device="cuda")
    weights = torch.randn(batch, heads, device="cuda").to(torch.bfloat16)
    q_scale = torch.rand(batch, heads, device="cuda") * 0.04 + 0.01
    out = torch.empty(batch, k, dtype=torch.int32, device="cuda")
    workspace = torch.empty(int(lib.mlakvIndexerWorkspaceBytes(batch, ctx)), dtype=torch.uint8, device="cuda")
    views = [ffi.IndexKeyView(kp.data_ptr(), bs * 128, 128, scales.data_ptr(), bs, blocks, bs, 128, 0) for kp in keys]

    def launch(i):
        ffi.check(lib.mlakvLightningIndexer(C.byref(views[i % slices]), query.data_ptr(), heads * 128, 128, weights.data_ptr(),
                                            heads * 2, q_scale.data_ptr(), heads, heads, table.data_ptr(), ctx // bs, lens.data_ptr(),
                                            batch, ctx, k, out.data_ptr(), k, workspace.data_ptr(), workspace.numel(),
                                            stream_ptr(torch)))
    us = sustained_us(torch, launch, 64)
    algorithmic = batch * ctx * (128 + 4) + batch * heads * (128 + 2 + 4) + 4 * batch * (ctx // bs) + 4 * batch * k
    return {"us_per_step": us,
            "workload": f"batch {batch}, ctx {ctx}, {heads} index heads x 128, top-{k}, block {bs}, e4m3 keys + fp32 row scale, "
                        f"shuffled table, {slices} rotating key pools",
            "roofline": {"bound": "hbm", "achieved": algorithmic / (us * 1e-6) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": algorithmic / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, "traffic": None},
            "algorithmic_bytes": algorithmic, "timing": "250 ms of back-to-back launches untimed, then at least 100 ms of them timed"}


def bench_side_kernels(args, torch, np, ffi):
    """The other data-movement kernels of the path at configs[3]/[4]-like sizes (8 layers to bound
    memory): FP8 quantize-on-append, FP8 dequantising gather, bf16 compaction copy. HIP-event
    time per launch against algorithmic bytes."""
    lib = ffi.load()
    bs, layers, batch, max_ctx = 64, 8, 64, 8192
    rng = np.random.default_rng(11)
    ctxs = [int(v) for v in rng.integers(512, 8193, size=batch)]
    total = sum(ctxs)
    blocks = sum(-(-c // bs) for c in ctxs)
    out = {}

    def timed(fn, reps=5):
        return sustained_us(torch, lambda i: fn(), reps, warm_ms=100.0, timed_ms=50.0) * 1e-3

    gen = torch.Generator(device="cuda").manual_seed(5)
    lat = torch.randn(layers, total, LATENT, generator=gen, device="cuda").to(torch.bfloat16)
    rop = torch.randn(layers, total, ROPE, generator=gen, device="cuda").to(torch.bfloat16)
    for fp8 in (True, False):
        arena = ffi.Arena(ffi.BACKEND_HIP)
        cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=max_ctx, max_batch=batch,
                            pool_blocks=blocks + 16, seed=3, shuffle=1, dtype=ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16)
        arena.commit()
        cache.bind()
        arena.seal()
        view = cache.view()
        for s, n in enumerate(ctxs):
            cache.add_sequence(s, n)
        cache.upload_step(stream_ptr(torch))
        table = cache.host_block_table()
        slots = torch.as_tensor(np.concatenate([table[s, np.arange(n) // bs].astype(np.int64) * bs + np.arange(n) % bs
                                                for s, n in enumerate(ctxs)]).astype(np.int32), device="cuda")

        def append():
            ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, lat.data_ptr(), total * LATENT * 2, LATENT * 2, rop.data_ptr(),
                                      total * ROPE * 2, ROPE * 2, slots.data_ptr(), total, stream_ptr(torch)))
        ms = timed(append)
        if fp8:
            nbytes = layers * (total * (ROW_BYTES + 580) + 4 * total)
            out["append_fp8"] = {"ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9, "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                 "rows": total, "layers": layers}
            dst = torch.empty(layers, total, ROW, dtype=torch.bfloat16, device="cuda")

            def gather():
                ffi.check(lib.mlakvGather(C.byref(view), 0, layers, cache.device_block_table, cache.num_blocks,
                                          cache.device_seq_lens, cache.device_cu_seq_lens, batch, max_ctx, dst.data_ptr(),
                                          total * ROW_BYTES, ROW_BYTES, dst.data_ptr() + LATENT * 2, total * ROW_BYTES, ROW_BYTES,
                                          stream_ptr(torch)))
            ms = timed(gather)
            nbytes = layers * (total * (580 + ROW_BYTES) + 4 * blocks)
            out["gather_fp8"] = {"ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9, "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                 "rows": total, "layers": layers}
            del dst
        else:
            # fused latent RMSNorm + key RoPE + append of one layer over every row (prefill-sized launch)
            kv_a = torch.cat([lat[0], rop[0]], dim=1).contiguous()
            gamma = torch.ones(LATENT, dtype=torch.bfloat16, device="cuda")
            ang = torch.outer(torch.arange(max_ctx, dtype=torch.float32, device="cuda"),
                              10000.0 ** (-torch.arange(0, ROPE // 2, dtype=torch.float32, device="cuda") * 2 / ROPE))
            cos = torch.cat([ang.cos(), ang.cos()], dim=1).to(torch.bfloat16)
            sin = torch.cat([ang.sin(), ang.sin()], dim=1).to(torch.bfloat16)
            positions = torch.as_tensor(np.concatenate([np.arange(n) for n in ctxs]).astype(np.int32), device="cuda")

            def fused():
                ffi.check(lib.mlakvNormRopeAppend(C.byref(view), 0, kv_a.data_ptr(), ROW_BYTES, gamma.data_ptr(), 1e-6, cos.data_ptr(),
                                                  sin.data_ptr(), ROPE * 2, positions.data_ptr(), slots.data_ptr(), total, None, 0,
                                                  None, 0, None, 0, 0, 0, stream_ptr(torch)))
            ms = timed(fused)
            nbytes = total * (2 * ROW_BYTES + 8)
            out["norm_rope_append_bf16"] = {"ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9,
                                            "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "rows": total, "layers": 1}
            # the same with the query's rope slices (64 heads, 128 of every 1152 bytes) rotated in place
            q_tokens, heads = min(total, 32768), 64
            q = torch.randn(q_tokens, heads, ROW, device="cuda").to(torch.bfloat16)

            def fused_with_query():
                ffi.check(lib.mlakvNormRopeAppend(C.byref(view), 0, kv_a.data_ptr(), ROW_BYTES, gamma.data_ptr(), 1e-6, cos.data_ptr(),
                                                  sin.data_ptr(), ROPE * 2, positions.data_ptr(), slots.data_ptr(), q_tokens, None, 0,
                                                  None, 0, q.data_ptr() + LATENT * 2, heads * ROW_BYTES, ROW_BYTES, heads,
                                                  stream_ptr(torch)))
            ms = timed(fused_with_query)
            nbytes = q_tokens * (2 * ROW_BYTES + 8 + heads * 2 * ROPE * 2)
            out["norm_rope_append_query_rope_bf16"] = {"ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9,
                                                       "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "rows": q_tokens,
                                                       "heads": heads, "layers": 1}
            del q
            del kv_a
            # free every other sequence, then compact: the device copies each moved block in every layer
            for s in range(0, batch, 2):
                cache.free_sequence(s)
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            moves = cache.compact(stream_ptr(torch))
            stop.record()
            torch.cuda.synchronize()
            whole_ms = start.elapsed_time(stop)
            # the copy kernel alone, replaying the same move list from device memory
            moves_dev = torch.as_tensor(np.asarray(moves, dtype=np.int32).reshape(-1), device="cuda")

            def copy():
                ffi.check(lib.mlakvCopyBlocks(C.byref(view), 0, layers, moves_dev.data_ptr(), len(moves), stream_ptr(torch)))
            ms = timed(copy)
            nbytes = 2 * len(moves) * bs * ROW_BYTES * layers
            out["compaction_bf16"] = {"ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9, "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                      "moved_blocks": len(moves), "layers": layers,
                                      "ms_with_host_plan_and_upload": whole_ms}
        cache.close()
        arena.close()
    return out


def cpu_baseline(np, ag):
    """The CPU oracle (a port: the reference has no CPU numerics for this path) on one core, on a
    bounded sample of the same workload: the append+gather step of all 43 layers, 12 times."""
    import oracle_ffi as orc
    bs, batch = 64, len(ag["ctxs"])
    sample_layers = 43
    ctxs = [c + 1 for c in ag["ctxs"]]
    pool = orc.Pool(ag["pool_blocks"], bs, batch, 40, seed=ag["seed"], shuffle=True)
    for s, n in enumerate(ctxs):
        pool.add_sequence(s, n)
    table = pool.table()
    rng = np.random.default_rng(3)
    plane0 = rng.integers(0, 255, size=ag["pool_blocks"] * bs * ROW_BYTES, dtype=np.uint8)
    planes = [plane0.copy() for _ in range(sample_layers)]  # distinct memory per layer, same bytes
    rows = rng.integers(0, 255, size=(sample_layers, batch * ROW_BYTES), dtype=np.uint8)
    slots = np.array([int(table[s, (n - 1) // bs]) * bs + (n - 1) % bs for s, n in enumerate(ctxs)], dtype=np.int32)
    times = []
    for rep in range(13):
        t0 = time.perf_counter()
        for layer in range(sample_layers):
            orc.append_rows(planes[layer], bs * ROW_BYTES, ROW_BYTES, bs, rows[layer], ROW_BYTES, ROW_BYTES, slots)
            orc.gather_rows(planes[layer], bs * ROW_BYTES, ROW_BYTES, bs, table, ctxs, ROW_BYTES)
        times.append(time.perf_counter() - t0)
    times = sorted(times[1:])
    median = times[len(times) // 2]
    nbytes = sample_layers * (2 * sum(ctxs) * ROW_BYTES + 2 * batch * ROW_BYTES)
    return {"value": nbytes / median / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"append+gather of {sample_layers} of 43 layers of the same workload (fused 576-element rows), "
                      f"median of 12 runs after one warm-up, host cores visible: {os.cpu_count()}"}


def cpu_attention_baseline(np):
    import oracle_ffi as orc
    bs, heads, ctx, batch = 64, 64, 2048, 1
    sample = 32  # every sequence, one after the other (about 10 s on one core)
    rng = np.random.default_rng(4)
    blocks = ctx // bs
    latent = orc.bf16_to_f32(np.zeros(1, np.uint16))  # warm the library
    latent_plane = (rng.standard_normal(blocks * bs * LATENT).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    rope_plane = (rng.standard_normal(blocks * bs * ROPE).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    q_lat = (rng.standard_normal((batch, heads, LATENT)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    q_rope = (rng.standard_normal((batch, heads, ROPE)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    table = np.arange(blocks, dtype=np.int32).reshape(1, blocks)
    t0 = time.perf_counter()
    for _ in range(sample):
        orc.mla_decode(q_lat, q_rope, latent_plane, rope_plane, bs, table, [ctx], 1 / math.sqrt(192.0), accum_f32=True)
    seconds = time.perf_counter() - t0
    return {"value": seconds * 32 / sample * 1e6, "unit": "us/step", "cores": 1, "kind": "port",
            "sample": f"{sample} of 32 sequences (64 heads, ctx 2048, fp32 accumulate), time scaled by {32 // sample}"}


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py measures one GPU: this path has no multi-GPU leg (sequences shard with no exchange); "
                         "run with --gpus 1\n")
        return 2
    import numpy as np
    import torch

    import mlakv_ffi as ffi
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU: the HIP library has no CPU fallback\n")
        return 3
    torch.cuda.set_device(0)
    # A plain 1 GiB device copy of known size: the reference point that scales rocprofv3's
    # FETCH_SIZE / WRITE_SIZE readings for the kernels below.
    calib_src = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
    calib_dst = torch.empty_like(calib_src)
    calib_dst.copy_(calib_src)
    torch.cuda.synchronize()
    del calib_src, calib_dst
    if args.side_only:
        print(json.dumps({"side_kernels": bench_side_kernels(args, torch, np, ffi)}))
        return 0
    if args.attention_only:
        print(json.dumps({"attention": bench_attention(args, torch, np, ffi, mx_quant=True),
                          "attention_fp8": bench_attention(args, torch, np, ffi, fp8=True, batch=64, ctx=4352, iters=64),
                          "attention_long": bench_attention(args, torch, np, ffi, batch=128, ctx=8192, slices=2, iters=16,
                                                            label="configs[4]-scale decode shape (one workgroup per sequence)"),
                          "attention_sparse": bench_attention(args, torch, np, ffi, batch=32, ctx=8192, slices=4, sparse_k=512,
                                                              label="selected-token decode (index_topk 512 of 8192)"),
                          "indexer": bench_indexer(args, torch, np, ffi)}))
        return 0
    ag = bench_append_gather(args, torch, np, ffi)
    line = {
        "metric": "paged-KV append+gather GB/s; MLA decode attn us/step (% HBM roofline)",
        "value": ag["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ag["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1]: paged append+gather, 43 layers, batch 32, ctx uniform [128,2048] "
                               f"(mean {ag['mean_ctx']:.0f} in the timed steps), block 64, seeded-shuffled free list, bf16 rows "
                               "of 576 elements, 1 row appended per sequence per layer then full-context gather into "
                               + ("separate latent/rope planes" if args.split_out else "contiguous 576-element rows"),
                   "bytes_per_step": ag["bytes_per_step"], "frac_of_hbm_peak": ag["value"] / HBM_PEAK_GBPS},
        "roofline": {"bound": "hbm", "achieved": ag["gather_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": ag["gather_gbps"] / HBM_PEAK_GBPS,
                     "traffic": ag["gather_bytes_per_launch"] * GATHER_TRAFFIC_PER_ALGORITHMIC_BYTE,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE x2.000 + WRITE_SIZE x1.000 per gather dispatch of this "
                                       "command, applied as a ratio to the algorithmic bytes of the timed launches",
                     "kernel": "GatherBf16TileKernel",
                     "avg_launch_ms": ag["gather_ms"], "algorithmic_bytes_per_launch": ag["gather_bytes_per_launch"]},
        "append": {"avg_launch_ms": ag["append_ms"], "achieved_gbps": ag["append_gbps"],
                   "note": "interval between 64 back-to-back launches of the 32-row x 43-layer append (2.9 MB): "
                           "bound by the launch rate, the kernel itself runs about 4 us in the rocprofv3 trace"},
    }
    if not args.no_attention:
        line["attention"] = bench_attention(args, torch, np, ffi, mx_quant=True)
        line["attention_fp8"] = bench_attention(args, torch, np, ffi, fp8=True, batch=64, ctx=4352, iters=64)
        line["attention_long"] = bench_attention(args, torch, np, ffi, batch=128, ctx=8192, slices=2, iters=16,
                                                 label="configs[4]-scale decode shape (one workgroup per sequence)")
        line["attention_sparse"] = bench_attention(args, torch, np, ffi, batch=32, ctx=8192, slices=4, sparse_k=512,
                                                   label="selected-token decode (index_topk 512 of 8192)")
        line["indexer"] = bench_indexer(args, torch, np, ffi)
        line["side_kernels"] = bench_side_kernels(args, torch, np, ffi)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(np, ag)
        if not args.no_attention:
            line["attention"]["cpu_baseline"] = cpu_attention_baseline(np)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
