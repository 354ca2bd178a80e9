"""GPU parity: a continuous-batching loop in the shape of configs[4] (scaled down): sequences
with seeded lengths and finish times share one block pool; every step appends one row per live
sequence and layer, runs decode attention for every live sequence, recycles finished sequences
into new prompts and periodically compacts the pool on the device. Checked against the CPU
oracle: block tables and free list after every pool operation (bit-exact), attention values
(2e-2 of the peak, bf16 KV), and the gathered bytes of every live sequence across compaction."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE
SCALE = 1.0 / math.sqrt(192.0)


def _lognormal_lengths(rng, count, median, sigma, cap):
    return [int(min(cap, max(1, round(math.exp(math.log(median) + sigma * rng.standard_normal()))))) for _ in range(count)]


def test_recycle_compact_attend_every_step():
    bs, layers, batch, heads = 64, 2, 8, 64
    max_ctx, pool_blocks, steps = 1024, 72, 40
    rng = np.random.default_rng(2025)
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=max_ctx, max_batch=batch,
                        pool_blocks=pool_blocks, seed=5, shuffle=1)
    lib = ffi.load()
    plan = ffi.AttnPlan()
    ffi.check(lib.mlakvAttnPlanInit(batch, heads, max_ctx, bs, ffi.DTYPE_BF16, C.byref(plan)))
    arena.note_workspace(int(plan.workspace_bytes))
    arena.commit()
    arena.commit_workspace()
    cache.bind()
    arena.seal()
    view = cache.view()
    pool = orc.Pool(pool_blocks, bs, batch, max_ctx // bs, seed=5, shuffle=True)

    # host mirror of every live sequence's rows, per layer: the logical KV the cache must hold
    mirror = [None] * batch
    finish_at = [0] * batch
    seed_counter = [100]

    def new_rows(count):
        seed_counter[0] += 2
        lat = kt.randn_bf16((layers, count, LATENT), seed=seed_counter[0])
        rop = kt.randn_bf16((layers, count, ROPE), seed=seed_counter[0] + 1)
        return lat, rop

    def write_rows(lat, rop, slots):
        count = lat.shape[1]
        lat_d, rop_d = lat.cuda(), rop.cuda()
        ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, lat_d.data_ptr(), count * LATENT * 2, LATENT * 2,
                                  rop_d.data_ptr(), count * ROPE * 2, ROPE * 2, kt.dev_i32(slots).data_ptr(), count,
                                  kt.stream_ptr()))
        torch.cuda.synchronize()

    def admit(seq, step):
        prompt = _lognormal_lengths(rng, 1, 160, 0.8, max_ctx - steps - 1)[0]
        status = pool.add_sequence(seq, prompt)
        if status != orc.OK:  # pool exhausted: the product must refuse as well, and nothing changes
            with pytest.raises(ffi.MlakvError):
                cache.add_sequence(seq, prompt)
            return False
        cache.add_sequence(seq, prompt)
        table = pool.table()
        slots = [int(table[seq, i // bs]) * bs + i % bs for i in range(prompt)]
        lat, rop = new_rows(prompt)
        write_rows(lat, rop, slots)
        mirror[seq] = [lat, rop]
        finish_at[seq] = step + int(rng.integers(3, 25))
        return True

    for s in range(batch):
        assert admit(s, 0)
    assert np.array_equal(cache.host_block_table(), pool.table())

    compactions = 0
    for step in range(1, steps + 1):
        # finished sequences leave, new prompts take their place
        for s in range(batch):
            if mirror[s] is not None and finish_at[s] <= step:
                cache.free_sequence(s)
                pool.free_sequence(s)
                mirror[s] = None
            if mirror[s] is None:
                admit(s, step)
        if step % 7 == 0:
            before = {s: _gather_one(lib, view, cache, s, layers, batch, max_ctx) for s in range(batch) if mirror[s] is not None}
            moves = cache.compact(kt.stream_ptr())
            assert moves == pool.compact()
            compactions += len(moves) > 0
            cache.upload_step(kt.stream_ptr())
            for s, rows in before.items():
                after = _gather_one(lib, view, cache, s, layers, batch, max_ctx)
                assert torch.equal(rows[0], after[0]) and torch.equal(rows[1], after[1])
            live_blocks = sum(-(-mirror[s][0].shape[1] // bs) for s in range(batch) if mirror[s] is not None)
            table = pool.table()
            used = sorted(int(table[s, b]) for s in range(batch) if mirror[s] is not None
                          for b in range(-(-mirror[s][0].shape[1] // bs)))
            assert used == list(range(live_blocks))  # live blocks occupy [0, n_live)
        # decode: one new row per live sequence and layer
        live = [s for s in range(batch) if mirror[s] is not None]
        slots, lat_new, rop_new = [], [], []
        for s in live:
            slot = cache.append_token(s)
            assert (orc.OK, slot) == pool.append_token(s)
            slots.append(slot)
            lat, rop = new_rows(1)
            lat_new.append(lat)
            rop_new.append(rop)
            mirror[s][0] = torch.cat([mirror[s][0], lat], dim=1)
            mirror[s][1] = torch.cat([mirror[s][1], rop], dim=1)
        write_rows(torch.cat(lat_new, dim=1), torch.cat(rop_new, dim=1), slots)
        cache.upload_step(kt.stream_ptr())
        assert np.array_equal(cache.host_block_table(), pool.table())
        assert cache.free_list() == pool.free_list()
        lens = [mirror[s][0].shape[1] if mirror[s] is not None else 0 for s in range(batch)]
        assert list(cache.host_seq_lens()) == lens

        # attention for the whole batch on the last layer, against the oracle fed from the mirror
        layer = layers - 1
        q = kt.randn_bf16((batch, heads, LATENT + ROPE), seed=7000 + step).cuda()
        out = torch.full((batch, heads, LATENT), float("nan"), dtype=torch.bfloat16, device="cuda")
        row = (LATENT + ROPE) * 2
        ffi.check(lib.mlakvAttnDecode(C.byref(plan), C.byref(view), layer, q.data_ptr(), heads * row, row,
                                      q.data_ptr() + LATENT * 2, heads * row, row, cache.device_block_table,
                                      cache.num_blocks, cache.device_seq_lens, SCALE, out.data_ptr(), heads * LATENT * 2,
                                      LATENT * 2, None, arena.workspace, arena.workspace_bytes, kt.stream_ptr()))
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        assert np.isfinite(got).all()
        if step % 4 == 0 or step == steps:
            for s in range(batch):
                if mirror[s] is None:
                    assert not got[s].any()  # an empty slot of the batch yields zeros
                    continue
                n = lens[s]
                identity = np.arange(-(-n // bs), dtype=np.int32).reshape(1, -1)
                lat_plane = np.zeros((identity.shape[1] * bs, LATENT), dtype=np.uint16)
                rope_plane = np.zeros((identity.shape[1] * bs, ROPE), dtype=np.uint16)
                lat_plane[:n] = kt.bits16(mirror[s][0][layer])
                rope_plane[:n] = kt.bits16(mirror[s][1][layer])
                qb = kt.bits16(q[s:s + 1])
                expected, _ = orc.mla_decode(np.ascontiguousarray(qb[..., :LATENT]), np.ascontiguousarray(qb[..., LATENT:]),
                                             lat_plane.reshape(-1), rope_plane.reshape(-1), bs, identity, [n], SCALE)
                peak = np.abs(expected).max()
                assert np.abs(got[s] - expected[0]).max() <= 2e-2 * peak, (step, s, n)
    assert compactions >= 1
    assert cache.free_blocks == pool_blocks - sum(-(-mirror[s][0].shape[1] // bs) for s in range(batch) if mirror[s] is not None)
    assert cache.free_blocks == pool.free_blocks
    cache.close()
    arena.close()


def _gather_one(lib, view, cache, seq, layers, batch, max_ctx):
    """Gathered latent and rope rows of every live sequence (the whole batch is gathered; the
    caller compares its own sequence through the cumulative offsets)."""
    lens = np.array(cache.host_seq_lens(), dtype=np.int64)
    total = int(lens.sum())
    latent_out = torch.zeros(layers, total, LATENT, dtype=torch.bfloat16, device="cuda")
    rope_out = torch.zeros(layers, total, ROPE, dtype=torch.bfloat16, device="cuda")
    ffi.check(lib.mlakvGather(C.byref(view), 0, layers, cache.device_block_table, cache.num_blocks, cache.device_seq_lens,
                              cache.device_cu_seq_lens, batch, max_ctx, latent_out.data_ptr(), total * LATENT * 2,
                              LATENT * 2, rope_out.data_ptr(), total * ROPE * 2, ROPE * 2, kt.stream_ptr()))
    torch.cuda.synchronize()
    start = int(lens[:seq].sum())
    return latent_out[:, start:start + int(lens[seq])].clone(), rope_out[:, start:start + int(lens[seq])].clone()
