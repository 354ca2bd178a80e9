"""GPU parity: append / gather / compaction through the C ABI against the CPU oracle.
Bit-exact for block tables, append offsets and gathered bytes (bf16 and FP8 codes/scales)."""
import ctypes as C

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

LATENT, ROPE = kt.LATENT, kt.ROPE


def _oracle_planes(layers, blocks, bs, fp8=False):
    e = 1 if fp8 else 2
    latent = [np.zeros(blocks * bs * LATENT * e, dtype=np.uint8) for _ in range(layers)]
    rope = [np.zeros(blocks * bs * ROPE * e, dtype=np.uint8) for _ in range(layers)]
    scale = [np.zeros(blocks * bs, dtype=np.float32) for _ in range(layers)] if fp8 else None
    return latent, rope, scale


def _oracle_append_bf16(latent, rope, bs, latent_src, rope_src, slots):
    for layer in range(len(latent)):
        ls = kt.u8(latent_src[layer]).reshape(-1)
        rs = kt.u8(rope_src[layer]).reshape(-1)
        orc.append_rows(latent[layer], bs * LATENT * 2, LATENT * 2, bs, ls, LATENT * 2, LATENT * 2, slots)
        orc.append_rows(rope[layer], bs * ROPE * 2, ROPE * 2, bs, rs, ROPE * 2, ROPE * 2, slots)


def test_config1_identity_paging_append_then_gather():
    """BASELINE config 1: one layer, block 64, one sequence with identity paging; 128 prompt rows
    appended one per step, one decode row, gather of all 129 rows, byte comparison. Runs on the
    arena + KV cache manager (HIP backend), so the reservations and diagnostics are exercised too."""
    bs, max_ctx = 64, 8192
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=1, block_size=bs, max_context_len=max_ctx, max_batch=1)
    arena.commit()
    assert arena.device_allocations == 1
    cache.bind()
    arena.seal()
    view = cache.view()
    lib = ffi.load()
    cache.add_sequence(0, 0)
    rows = kt.randn_bf16((129, LATENT + ROPE), seed=1).cuda()
    latent_src = rows[:, :LATENT].contiguous()
    rope_src = rows[:, LATENT:].contiguous()
    allocations_before = arena.device_allocations
    for position in range(129):
        slot = cache.append_token(0)
        assert slot == position  # identity paging: slot = position (reference pipeline.cpp:517)
        cache.upload_step(kt.stream_ptr())
        ffi.check(lib.mlakvAppend(C.byref(view), 0, 1, latent_src[position].data_ptr(), 0, LATENT * 2,
                                  rope_src[position].data_ptr(), 0, ROPE * 2, cache.device_slot_mapping, 1,
                                  kt.stream_ptr()))
    assert arena.device_allocations == allocations_before  # zero allocations inside the steps
    torch.cuda.synchronize()
    stats = cache.stats()
    assert stats.active_context_tokens == 129
    assert stats.kv_cache_utilization == 0.0157470703125  # reference docs/preflight-verification.md:42-45
    assert stats.total_blocks_allocated == 128
    latent_out = torch.zeros(129, LATENT, dtype=torch.bfloat16, device="cuda")
    rope_out = torch.zeros(129, ROPE, dtype=torch.bfloat16, device="cuda")
    ffi.check(lib.mlakvGather(C.byref(view), 0, 1, cache.device_block_table, cache.num_blocks, cache.device_seq_lens,
                              cache.device_cu_seq_lens, 1, 129, latent_out.data_ptr(), 0, LATENT * 2,
                              rope_out.data_ptr(), 0, ROPE * 2, kt.stream_ptr()))
    torch.cuda.synchronize()
    # oracle: memcpy append at slot = position into a zeroed plane, then gather through the table
    blocks = cache.pool_blocks
    lat, rop, _ = _oracle_planes(1, blocks, bs)
    slots = np.arange(129, dtype=np.int32)
    orc.append_rows(lat[0], bs * LATENT * 2, LATENT * 2, bs, kt.u8(latent_src).reshape(-1), LATENT * 2, LATENT * 2, slots)
    orc.append_rows(rop[0], bs * ROPE * 2, ROPE * 2, bs, kt.u8(rope_src).reshape(-1), ROPE * 2, ROPE * 2, slots)
    table = cache.host_block_table()
    assert list(table[0, :3]) == [0, 1, 2]
    exp_latent = orc.gather_rows(lat[0], bs * LATENT * 2, LATENT * 2, bs, table, [129], LATENT * 2)
    exp_rope = orc.gather_rows(rop[0], bs * ROPE * 2, ROPE * 2, bs, table, [129], ROPE * 2)
    assert kt.u8(latent_out).reshape(-1).tobytes() == exp_latent.tobytes()
    assert kt.u8(rope_out).reshape(-1).tobytes() == exp_rope.tobytes()
    assert kt.u8(latent_out).reshape(-1).tobytes() == kt.u8(latent_src).reshape(-1).tobytes()
    cache.close()
    arena.close()


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("bs", [16, 64, 128])
def test_append_gather_shuffled_ragged_batch(fused, bs):
    layers = 3
    ctxs = [0, 1, bs - 1, bs, bs + 1, 3 * bs + 7, 5 * bs]
    need = sum(-(-c // bs) for c in ctxs)
    blocks = need + 5
    pool = kt.build_tables(ctxs, bs, blocks, seed=7)
    table = pool.table()
    total = sum(ctxs)
    cache = kt.PagedCache(layers, blocks, bs, fused=fused)
    latent_src = kt.randn_bf16((layers, total, LATENT), seed=2).cuda()
    rope_src = kt.randn_bf16((layers, total, ROPE), seed=3).cuda()
    slots = kt.slots_for(table, ctxs, bs)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(slots))
    torch.cuda.synchronize()
    lat, rop, _ = _oracle_planes(layers, blocks, bs)
    _oracle_append_bf16(lat, rop, bs, latent_src, rope_src, slots)
    for layer in range(layers):  # planes bit-exact, including the untouched (zero) slots
        assert kt.u8(cache.latent[layer].contiguous()).reshape(-1).tobytes() == lat[layer].tobytes()
        assert kt.u8(cache.rope[layer].contiguous()).reshape(-1).tobytes() == rop[layer].tobytes()
    for fused_out in (False, True):
        got_latent, got_rope = kt.gather(cache, kt.dev_i32(table), kt.dev_i32(ctxs), fused_out=fused_out)
        for layer in range(layers):
            exp_latent = orc.gather_rows(lat[layer], bs * LATENT * 2, LATENT * 2, bs, table, ctxs, LATENT * 2)
            exp_rope = orc.gather_rows(rop[layer], bs * ROPE * 2, ROPE * 2, bs, table, ctxs, ROPE * 2)
            assert kt.u8(got_latent[layer].contiguous()).reshape(-1).tobytes() == exp_latent.tobytes()
            assert kt.u8(got_rope[layer].contiguous()).reshape(-1).tobytes() == exp_rope.tobytes()
        # gather o append = identity on the logical sequences
        assert torch.equal(got_latent.contiguous(), latent_src)
        assert torch.equal(got_rope.contiguous(), rope_src)


def test_append_skips_negative_slots_and_layer_window():
    layers, bs, blocks = 4, 64, 6
    cache = kt.PagedCache(layers, blocks, bs)
    latent_src = kt.randn_bf16((2, 5, LATENT), seed=4).cuda()
    rope_src = kt.randn_bf16((2, 5, ROPE), seed=5).cuda()
    slots = np.array([3, -1, 200, -1, 64], dtype=np.int32)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(slots), layer_begin=1, layer_count=2)
    torch.cuda.synchronize()
    lat, rop, _ = _oracle_planes(layers, blocks, bs)
    _oracle_append_bf16(lat[1:3], rop[1:3], bs, latent_src, rope_src, slots)
    for layer in range(layers):
        assert kt.u8(cache.latent[layer].contiguous()).reshape(-1).tobytes() == lat[layer].tobytes()
        assert kt.u8(cache.rope[layer].contiguous()).reshape(-1).tobytes() == rop[layer].tobytes()


def test_compaction_copy_keeps_gathered_bytes():
    layers, bs = 2, 64
    ctxs = [130, 64, 300, 17, 200]
    blocks = 24
    pool = kt.build_tables(ctxs, bs, blocks, seed=11)
    cache = kt.PagedCache(layers, blocks, bs)
    total = sum(ctxs)
    latent_src = kt.randn_bf16((layers, total, LATENT), seed=6).cuda()
    rope_src = kt.randn_bf16((layers, total, ROPE), seed=7).cuda()
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(pool.table(), ctxs, bs)))
    # sequences 1 and 3 finish; their blocks return to the free list
    assert pool.free_sequence(1) == orc.OK and pool.free_sequence(3) == orc.OK
    live_ctxs = [130, 0, 300, 0, 200]
    before_latent, before_rope = kt.gather(cache, kt.dev_i32(pool.table()), kt.dev_i32(live_ctxs))
    lat = [kt.u8(cache.latent[l].contiguous()).reshape(-1).copy() for l in range(layers)]
    moves = pool.compact()
    assert moves, "the shuffled pool must need moves"
    live = pool.live_blocks
    table = pool.table()
    used = sorted(int(table[s, i]) for s, n in enumerate(live_ctxs) for i in range(-(-n // bs)))
    assert used == list(range(live))  # live blocks occupy [0, n_live)
    lib = ffi.load()
    moves_dev = kt.dev_i32(np.asarray(moves, dtype=np.int32).reshape(-1))
    ffi.check(lib.mlakvCopyBlocks(C.byref(cache.view), 0, layers, moves_dev.data_ptr(), len(moves), kt.stream_ptr()))
    torch.cuda.synchronize()
    for l in range(layers):  # plane equals the oracle's block copies
        orc.copy_blocks(lat[l], bs * LATENT * 2, bs * LATENT * 2, moves)
        assert kt.u8(cache.latent[l].contiguous()).reshape(-1).tobytes() == lat[l].tobytes()
    after_latent, after_rope = kt.gather(cache, kt.dev_i32(table), kt.dev_i32(live_ctxs))
    assert torch.equal(before_latent, after_latent) and torch.equal(before_rope, after_rope)


def test_kv_cache_manager_matches_oracle_pool_and_compacts_on_device():
    bs, layers, batch = 64, 2, 6
    ctxs = [100, 64, 129, 1, 250, 63]
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=512, max_batch=batch, pool_blocks=20,
                        seed=99, shuffle=1)
    arena.commit()
    cache.bind()
    view = cache.view()
    pool = orc.Pool(20, bs, batch, 8, seed=99, shuffle=True)
    for s, n in enumerate(ctxs):
        cache.add_sequence(s, n)
        assert pool.add_sequence(s, n) == orc.OK
    assert np.array_equal(cache.host_block_table(), pool.table())
    total = sum(ctxs)
    latent_src = kt.randn_bf16((layers, total, LATENT), seed=8).cuda()
    rope_src = kt.randn_bf16((layers, total, ROPE), seed=9).cuda()
    lib = ffi.load()
    slots = kt.dev_i32(kt.slots_for(pool.table(), ctxs, bs))
    ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, latent_src.data_ptr(), total * LATENT * 2, LATENT * 2,
                              rope_src.data_ptr(), total * ROPE * 2, ROPE * 2, slots.data_ptr(), total, kt.stream_ptr()))
    cache.free_sequence(2)
    cache.free_sequence(5)
    pool.free_sequence(2)
    pool.free_sequence(5)
    moves = cache.compact(kt.stream_ptr())
    assert moves == pool.compact()
    assert np.array_equal(cache.host_block_table(), pool.table())
    assert cache.free_list() == pool.free_list()
    cache.upload_step(kt.stream_ptr())
    live = [100, 64, 0, 1, 250, 0]
    rows = sum(live)
    latent_out = torch.zeros(layers, rows, LATENT, dtype=torch.bfloat16, device="cuda")
    rope_out = torch.zeros(layers, rows, ROPE, dtype=torch.bfloat16, device="cuda")
    ffi.check(lib.mlakvGather(C.byref(view), 0, layers, cache.device_block_table, cache.num_blocks,
                              cache.device_seq_lens, cache.device_cu_seq_lens, batch, 512, latent_out.data_ptr(),
                              rows * LATENT * 2, LATENT * 2, rope_out.data_ptr(), rows * ROPE * 2, ROPE * 2,
                              kt.stream_ptr()))
    torch.cuda.synchronize()
    starts = np.concatenate([[0], np.cumsum(ctxs)])
    keep = np.concatenate([np.arange(starts[s], starts[s] + ctxs[s]) for s in (0, 1, 3, 4)])
    assert torch.equal(latent_out, latent_src[:, keep]) and torch.equal(rope_out, rope_src[:, keep])
    cache.close()
    arena.close()


# ---- FP8 rows ---------------------------------------------------------------------------


@pytest.mark.parametrize("bs", [16, 64])
def test_fp8_quantize_on_append_and_dequant_gather_bit_exact(bs):
    layers = 2
    ctxs = [1, bs + 3, 4 * bs, 0, 77]
    blocks = sum(-(-c // bs) for c in ctxs) + 3
    pool = kt.build_tables(ctxs, bs, blocks, seed=21)
    table = pool.table()
    total = sum(ctxs)
    cache = kt.PagedCache(layers, blocks, bs, fp8=True)
    latent_src = kt.randn_bf16((layers, total, LATENT), seed=10, outlier_fraction=0.01).cuda()
    rope_src = kt.randn_bf16((layers, total, ROPE), seed=11, outlier_fraction=0.01).cuda()
    latent_src[0, 0] = 0  # an all-zero row: scale must be 1, codes 0
    rope_src[0, 0] = 0
    slots = kt.slots_for(table, ctxs, bs)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(slots))
    torch.cuda.synchronize()
    lat, rop, scl = _oracle_planes(layers, blocks, bs, fp8=True)
    for layer in range(layers):
        orc.append_rows_fp8(lat[layer], rop[layer], scl[layer], bs, kt.bits16(latent_src[layer]),
                            kt.bits16(rope_src[layer]), slots)
        assert cache.scale_np(layer).tobytes() == scl[layer].tobytes()
        assert cache.latent_np(layer).tobytes() == lat[layer].tobytes()
        assert cache.rope_np(layer).tobytes() == rop[layer].tobytes()
    assert scl[0][slots[0]] == 1.0
    got_latent, got_rope = kt.gather(cache, kt.dev_i32(table), kt.dev_i32(ctxs))
    for layer in range(layers):
        exp_latent, exp_rope = orc.gather_rows_fp8(lat[layer], rop[layer], scl[layer], bs, table, ctxs)
        assert kt.bits16(got_latent[layer]).tobytes() == exp_latent.tobytes()
        assert kt.bits16(got_rope[layer]).tobytes() == exp_rope.tobytes()
    # round-trip bound: |x - dequant| <= scale * 2^-4 * 448 / ... per element; e4m3 keeps 3 mantissa
    # bits, so the relative error of a normal code is at most 2^-4 and the absolute error in the
    # subnormal range at most scale * 2^-10 (plus the bf16 rounding of the result, 2^-9 relative).
    x = latent_src.float()
    y = got_latent.float()
    scale = (torch.maximum(latent_src.float().abs().amax(-1), rope_src.float().abs().amax(-1)) / 448.0).unsqueeze(-1)
    bound = torch.maximum(x.abs() * (2.0 ** -4 + 2.0 ** -8), scale * 2.0 ** -9)
    assert bool(((x - y).abs() <= bound).all())


def test_fp8_quantize_rows_at_the_edges_of_the_arithmetic_bit_exact():
    """Rows where the quantiser's shortcuts do not apply or must not matter, against the oracle bit
    for bit: magnitudes so small that the scale's reciprocal leaves the normal range (every lane
    divides), subnormal bf16 values, NaNs beside finite values (a NaN never becomes the row's
    maximum), a row of nothing but NaNs, infinities, quotients that sit exactly on rounding
    boundaries of the E4M3 grid (ties go to even), the largest finite bf16."""
    bs, layers = 16, 1
    rng = np.random.default_rng(33)
    rows = []
    base = rng.standard_normal((LATENT + ROPE,)).astype(np.float32)
    rows.append(base * np.float32(2.0 ** -112))                      # reciprocal of the scale overflows
    rows.append(base * np.float32(2.0 ** -101))                      # just below the switch
    rows.append(base * np.float32(2.0 ** -99))                       # just above it
    rows.append(base * np.float32(2.0 ** -130))                      # subnormal values
    with_nan = base.copy(); with_nan[[0, 513]] = np.nan; with_nan[[5, 575]] = np.copysign(np.nan, -1.0)   # both signs
    rows.append(with_nan)
    rows.append(np.full(LATENT + ROPE, np.nan, dtype=np.float32))
    with_inf = base.copy(); with_inf[[7, 520]] = [np.inf, -np.inf]
    rows.append(with_inf)
    ties = np.zeros(LATENT + ROPE, dtype=np.float32)                  # absmax 448: scale exactly 1
    grid = np.array([17, 19, 21, 23, 25, 27, 29, 31, 34, 36, 44, 52, 1.0625, 0.9375, 2.0 ** -9 * 1.5, 2.0 ** -9 * 2.5, 2.0 ** -10,
                     3 * 2.0 ** -10, 416 + 16, 448], dtype=np.float32)
    ties[:len(grid)] = grid; ties[100:100 + len(grid)] = -grid; ties[LATENT + 3] = 448.0; ties[LATENT + 4] = 17.0
    rows.append(ties)
    rows.append(ties * np.float32(3.0))                               # the same quotients behind a scale that is not a power of two
    rows.append(base / np.abs(base).max() * np.float32(3.3895314e38))  # absmax = the largest finite bf16
    data = torch.from_numpy(np.stack(rows)).to(torch.bfloat16)
    total = data.shape[0]
    blocks = -(-total // bs) + 1
    table = kt.build_tables([total], bs, blocks, seed=5).table()
    cache = kt.PagedCache(layers, blocks, bs, fp8=True)
    latent_src, rope_src = data[None, :, :LATENT].contiguous().cuda(), data[None, :, LATENT:].contiguous().cuda()
    slots = kt.slots_for(table, [total], bs)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(slots))
    torch.cuda.synchronize()
    lat, rop, scl = _oracle_planes(layers, blocks, bs, fp8=True)
    orc.append_rows_fp8(lat[0], rop[0], scl[0], bs, kt.bits16(latent_src[0]), kt.bits16(rope_src[0]), slots)
    assert cache.scale_np(0).tobytes() == scl[0].tobytes()
    got_lat, got_rope = cache.latent_np(0).reshape(-1, LATENT), cache.rope_np(0).reshape(-1, ROPE)
    for r, slot in enumerate(slots):
        assert got_lat[slot].tobytes() == lat[0].reshape(-1, LATENT)[slot].tobytes(), r
        assert got_rope[slot].tobytes() == rop[0].reshape(-1, ROPE)[slot].tobytes(), r
    assert scl[0][slots[5]] == 1.0                                    # nothing but NaNs: absmax 0
    # and back through the dequantising gather: bit for bit where the oracle's value is a number, a NaN
    # where it is one (0 x inf has the sign of the machine's default NaN, which differs between the two)
    table_d = kt.dev_i32(table)
    got_latent, got_rope = kt.gather(cache, table_d, kt.dev_i32([total]))
    exp_latent, exp_rope = orc.gather_rows_fp8(lat[0], rop[0], scl[0], bs, table, [total])
    for got, expected in ((kt.bits16(got_latent[0]), exp_latent), (kt.bits16(got_rope[0]), exp_rope)):
        got, expected = got.reshape(-1), expected.reshape(-1)
        is_nan = (expected & 0x7FFF) > 0x7F80
        assert np.array_equal(got[~is_nan], expected[~is_nan])
        assert ((got[is_nan] & 0x7FFF) > 0x7F80).all() and is_nan.sum() >= 4


def test_fp8_scale_of_every_bf16_maximum_bit_exact():
    """One row per positive finite bf16 value (and zero), that value its only non-zero element at a
    varying column: the stored scale is the oracle's absmax / 448 for every possible maximum, and
    the codes are the oracle's (the element itself encodes as 448)."""
    bs = 64
    values = np.arange(0, 0x7F80, dtype=np.uint32)             # bf16 bit patterns 0 .. largest finite
    total = len(values)
    data = np.zeros((total, LATENT + ROPE), dtype=np.uint16)
    data[np.arange(total), (np.arange(total) * 37) % (LATENT + ROPE)] = values.astype(np.uint16)
    src = torch.from_numpy(data.view(np.int16)).view(torch.bfloat16)
    blocks = -(-total // bs) + 1
    table = kt.build_tables([total], bs, blocks, seed=9).table()
    cache = kt.PagedCache(1, blocks, bs, fp8=True)
    latent_src, rope_src = src[None, :, :LATENT].contiguous().cuda(), src[None, :, LATENT:].contiguous().cuda()
    slots = kt.slots_for(table, [total], bs)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(slots))
    torch.cuda.synchronize()
    lat, rop, scl = _oracle_planes(1, blocks, bs, fp8=True)
    orc.append_rows_fp8(lat[0], rop[0], scl[0], bs, kt.bits16(latent_src[0]), kt.bits16(rope_src[0]), slots)
    assert cache.scale_np(0).tobytes() == scl[0].tobytes()
    assert cache.latent_np(0).tobytes() == lat[0].tobytes()
    assert cache.rope_np(0).tobytes() == rop[0].tobytes()


def test_fp8_compaction_moves_codes_and_scales():
    layers, bs, blocks = 2, 64, 12
    ctxs = [100, 64, 129]
    pool = kt.build_tables(ctxs, bs, blocks, seed=5)
    cache = kt.PagedCache(layers, blocks, bs, fp8=True)
    total = sum(ctxs)
    latent_src = kt.randn_bf16((layers, total, LATENT), seed=12).cuda()
    rope_src = kt.randn_bf16((layers, total, ROPE), seed=13).cuda()
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(pool.table(), ctxs, bs)))
    pool.free_sequence(1)
    live = [100, 0, 129]
    before = kt.gather(cache, kt.dev_i32(pool.table()), kt.dev_i32(live))
    moves = pool.compact()
    lib = ffi.load()
    moves_dev = kt.dev_i32(np.asarray(moves, dtype=np.int32).reshape(-1))
    ffi.check(lib.mlakvCopyBlocks(C.byref(cache.view), 0, layers, moves_dev.data_ptr(), len(moves), kt.stream_ptr()))
    after = kt.gather(cache, kt.dev_i32(pool.table()), kt.dev_i32(live))
    assert torch.equal(before[0], after[0]) and torch.equal(before[1], after[1])


# ---- full-size property checks (BASELINE config 2 shape) ---------------------------------------


def test_config2_full_size_round_trip():
    """43 layers, batch 32, contexts uniform in [128, 2048], block 64, shuffled free list: the
    gathered rows must equal the appended rows for every layer (gather o append = identity)."""
    layers, batch, bs = 43, 32, 64
    rng = np.random.default_rng(2)
    ctxs = [int(v) for v in rng.integers(128, 2049, size=batch)]
    blocks = sum(-(-(c + 1) // bs) for c in ctxs) + 64
    pool = kt.build_tables(ctxs, bs, blocks, seed=1234, max_blocks=33)
    cache = kt.PagedCache(layers, blocks, bs)
    total = sum(ctxs)
    gen = torch.Generator(device="cuda").manual_seed(5)
    latent_src = torch.randn(layers, total, LATENT, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    rope_src = torch.randn(layers, total, ROPE, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(pool.table(), ctxs, bs)))
    # one decode step: one more row per sequence per layer
    step_latent = torch.randn(layers, batch, LATENT, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    step_rope = torch.randn(layers, batch, ROPE, generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    step_slots = []
    for s in range(batch):
        status, slot = pool.append_token(s)
        assert status == orc.OK
        step_slots.append(slot)
    kt.append(cache, step_latent, step_rope, kt.dev_i32(step_slots))
    new_ctxs = [c + 1 for c in ctxs]
    got_latent, got_rope = kt.gather(cache, kt.dev_i32(pool.table()), kt.dev_i32(new_ctxs))
    starts = np.concatenate([[0], np.cumsum(new_ctxs)])
    old_starts = np.concatenate([[0], np.cumsum(ctxs)])
    for s in range(batch):
        a, b = int(starts[s]), int(starts[s + 1])
        oa, ob = int(old_starts[s]), int(old_starts[s + 1])
        assert torch.equal(got_latent[:, a:b - 1], latent_src[:, oa:ob])
        assert torch.equal(got_rope[:, a:b - 1], rope_src[:, oa:ob])
        assert torch.equal(got_latent[:, b - 1], step_latent[:, s])
        assert torch.equal(got_rope[:, b - 1], step_rope[:, s])
    # slots never written stay zero: checksum of the whole pool equals checksum of the sources
    pool_sum = cache.latent.view(torch.int16).to(torch.int64).sum().item()
    src_sum = latent_src.view(torch.int16).to(torch.int64).sum().item() + step_latent.view(torch.int16).to(torch.int64).sum().item()
    assert pool_sum == src_sum


_HIP = None


def _device_i32(pointer, count):
    """`count` int32 values at a raw device address (the C ABI hands out addresses, not tensors)."""
    global _HIP
    if _HIP is None:
        _HIP = C.CDLL("libamdhip64.so")
        _HIP.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _HIP.hipMemcpy.restype = C.c_int
    out = np.empty(count, dtype=np.int32)
    torch.cuda.synchronize()
    assert _HIP.hipMemcpy(out.ctypes.data, pointer, count * 4, 2) == 0  # hipMemcpyDeviceToHost
    return out


@pytest.mark.parametrize("fp8", [False, True])
def test_one_launch_step_equals_upload_then_append(fp8):
    """mlakvKvCacheUploadStepAndAppend against mlakvKvCacheUploadStep + mlakvAppend on a twin cache:
    the same planes, and the device metadata equal to the host mirrors, over steps that open
    blocks (entries sent as pairs), steps after a sequence left or joined (whole table copied:
    the two-call fallback) and steps where some sequences have no token."""
    bs, layers, batch, max_ctx = 16, 3, 6, 160
    lib = ffi.load()
    twins = []
    for _ in range(2):
        arena = ffi.Arena(ffi.BACKEND_HIP)
        cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=max_ctx, max_batch=batch, pool_blocks=48,
                            seed=9, shuffle=1, dtype=ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16)
        arena.commit()
        cache.bind()
        arena.seal()
        twins.append((arena, cache, cache.view()))
    for _, cache, _ in twins:
        for seq, n in enumerate([5, 15, 16, 0, 31]):  # sequence 5 stays unused
            cache.add_sequence(seq, n)
        cache.upload_step(kt.stream_ptr())
    width = twins[0][1].num_blocks
    for step in range(40):
        latent = kt.randn_bf16((layers, batch, LATENT), seed=1000 + 2 * step, outlier_fraction=0.01 if fp8 else 0.0).cuda()
        rope = kt.randn_bf16((layers, batch, ROPE), seed=1001 + 2 * step).cuda()
        for which, (_, cache, view) in enumerate(twins):
            if step == 12:
                cache.free_sequence(1)
            if step == 20:
                cache.add_sequence(1, 7)
            if step % 5 == 3:   # only some sequences get a token
                for seq in (0, 4):
                    cache.append_token(seq)
            else:
                cache.append_token_all()
            if which == 0:
                cache.upload_step(kt.stream_ptr())
                ffi.check(lib.mlakvAppend(C.byref(view), 0, layers, latent.data_ptr(), batch * LATENT * 2, LATENT * 2, rope.data_ptr(),
                                          batch * ROPE * 2, ROPE * 2, cache.device_slot_mapping, batch, kt.stream_ptr()))
            else:
                cache.upload_step_and_append(0, layers, latent.data_ptr(), batch * LATENT * 2, LATENT * 2, rope.data_ptr(),
                                             batch * ROPE * 2, ROPE * 2, kt.stream_ptr())
        torch.cuda.synchronize()
        fused = twins[1][1]
        assert np.array_equal(_device_i32(fused.device_block_table, batch * width).reshape(batch, width), fused.host_block_table())
        assert np.array_equal(_device_i32(fused.device_seq_lens, batch), fused.host_seq_lens())
        lens = fused.host_seq_lens()
        assert np.array_equal(_device_i32(fused.device_cu_seq_lens, batch + 1), np.concatenate([[0], np.cumsum(lens)]))
        assert np.array_equal(_device_i32(fused.device_slot_mapping, batch), _device_i32(twins[0][1].device_slot_mapping, batch))
    # the planes of the twins hold the same bytes
    for name in ("latent", "rope", "scale"):
        pointers = [getattr(view, name) for _, _, view in twins]
        if not pointers[0]:
            continue
        stride = getattr(twins[0][2], name + "_layer_stride")
        a, b = (_device_i32(p, layers * stride // 4) for p in pointers)
        assert np.array_equal(a, b)
    # a layer window, and refusals
    _, cache, view = twins[1]
    cache.append_token_all()
    cache.upload_step_and_append(1, 2, latent.data_ptr(), batch * LATENT * 2, LATENT * 2, rope.data_ptr(), batch * ROPE * 2, ROPE * 2,
                                 kt.stream_ptr())
    torch.cuda.synchronize()
    assert lib.mlakvKvCacheUploadStepAndAppend(cache.handle, 2, 2, latent.data_ptr(), 0, LATENT * 2, rope.data_ptr(), 0, ROPE * 2,
                                               None) == ffi.ERR_CONTRACT  # layers outside the cache: the manager refuses
    assert lib.mlakvKvCacheUploadStepAndAppend(cache.handle, 0, 1, None, 0, LATENT * 2, rope.data_ptr(), 0, ROPE * 2,
                                               None) == ffi.ERR_PARAM_NULLPTR
    assert lib.mlakvKvCacheUploadStepAndAppend(cache.handle, 0, 1, latent.data_ptr() + 2, 0, LATENT * 2, rope.data_ptr(), 0, ROPE * 2,
                                               None) == ffi.ERR_PARAM_INVALID
    for arena, cache, _ in twins:
        cache.close()
        arena.close()


@pytest.mark.parametrize("fp8,bs", [(False, 64), (False, 12), (True, 64)])  # the tiled, the generic and the FP8 kernel
def test_gather_that_times_itself_moves_the_same_bytes(fp8, bs):
    """mlakvGatherTimed: the plain gather's bytes, and a kernel duration in the caller's two events."""
    layers = 4
    ctxs = [300, 0, 77, 1000]
    blocks = sum(-(-c // bs) for c in ctxs) + 3
    table = kt.build_tables(ctxs, bs, blocks, seed=11).table()
    total = sum(ctxs)
    cache = kt.PagedCache(layers, blocks, bs, fp8=fp8)
    kt.append(cache, kt.randn_bf16((layers, total, LATENT), seed=12).cuda(), kt.randn_bf16((layers, total, ROPE), seed=13).cuda(),
              kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    want_latent, want_rope = kt.gather(cache, table_d, lens_d)

    hip = C.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipEventDestroy.argtypes = [C.c_void_p]
    hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
    start, stop = C.c_void_p(), C.c_void_p()
    assert hip.hipEventCreate(C.byref(start)) == 0 and hip.hipEventCreate(C.byref(stop)) == 0
    lib = ffi.load()
    cu = kt.dev_i32(np.concatenate([[0], np.cumsum(ctxs)]))
    latent = torch.zeros(layers, total, LATENT, dtype=torch.bfloat16, device="cuda")
    rope = torch.zeros(layers, total, ROPE, dtype=torch.bfloat16, device="cuda")

    def timed(first, second, batch=len(ctxs)):
        return lib.mlakvGatherTimed(C.byref(cache.view), 0, layers, table_d.data_ptr(), table_d.shape[1], lens_d.data_ptr(),
                                    cu.data_ptr(), batch, max(ctxs), latent.data_ptr(), total * LATENT * 2, LATENT * 2,
                                    rope.data_ptr(), total * ROPE * 2, ROPE * 2, kt.stream_ptr(), first, second)

    outer = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    outer[0].record()
    assert timed(start, stop) == 0
    outer[1].record()
    torch.cuda.synchronize()
    assert torch.equal(latent, want_latent) and torch.equal(rope, want_rope)
    ms = C.c_float(-1.0)
    assert hip.hipEventElapsedTime(C.byref(ms), start, stop) == 0
    # the kernel's own duration: positive, and inside the interval that recorded events bracket
    assert 0.0 < ms.value <= outer[0].elapsed_time(outer[1]) + 1e-3, (ms.value, outer[0].elapsed_time(outer[1]))
    assert timed(None, stop) == ffi.ERR_PARAM_NULLPTR and timed(start, None) == ffi.ERR_PARAM_NULLPTR
    assert timed(start, stop, batch=0) == ffi.ERR_PARAM_INVALID  # nothing would be launched, so nothing to time
    hip.hipEventDestroy(start)
    hip.hipEventDestroy(stop)


@pytest.mark.parametrize("seed", range(8))
def test_append_and_gather_on_drawn_shapes(seed):
    """Layers, block sizes (with and without the 8-row tile), context lengths, cache type and plane
    layout drawn from a seeded generator: the cache planes and the gathered rows, bit for bit."""
    rng = np.random.default_rng(500 + seed)
    fp8 = bool(rng.integers(0, 2))
    bs = int(rng.choice([4, 8, 12, 16, 40, 64, 128]))
    layers = int(rng.integers(1, 6))
    batch = int(rng.integers(1, 10))
    ctxs = [int(v) for v in rng.integers(0, 5 * bs + 9, size=batch)]
    ctxs[int(rng.integers(0, batch))] = 0
    blocks = sum(-(-c // bs) for c in ctxs) + int(rng.integers(1, 6))
    table = kt.build_tables(ctxs, bs, blocks, seed=seed).table()
    total = sum(ctxs)
    fused = (not fp8) and bool(rng.integers(0, 2))
    cache = kt.PagedCache(layers, blocks, bs, fp8=fp8, fused=fused) if not fp8 else kt.PagedCache(layers, blocks, bs, fp8=True)
    latent_src = kt.randn_bf16((layers, max(total, 1), LATENT), seed=600 + seed, outlier_fraction=0.01)[:, :total].contiguous().cuda()
    rope_src = kt.randn_bf16((layers, max(total, 1), ROPE), seed=700 + seed, outlier_fraction=0.01)[:, :total].contiguous().cuda()
    slots = kt.slots_for(table, ctxs, bs)
    case = dict(fp8=fp8, bs=bs, layers=layers, ctxs=ctxs, fused=fused)
    if total:
        kt.append(cache, latent_src, rope_src, kt.dev_i32(slots))
    torch.cuda.synchronize()
    lat, rop, scl = _oracle_planes(layers, blocks, bs, fp8=fp8)
    if fp8:
        for layer in range(layers):
            if total:
                orc.append_rows_fp8(lat[layer], rop[layer], scl[layer], bs, kt.bits16(latent_src[layer]), kt.bits16(rope_src[layer]), slots)
            assert cache.scale_np(layer).tobytes() == scl[layer].tobytes(), case
            assert cache.latent_np(layer).tobytes() == lat[layer].tobytes(), case
            assert cache.rope_np(layer).tobytes() == rop[layer].tobytes(), case
    else:
        if total:
            _oracle_append_bf16(lat, rop, bs, latent_src, rope_src, slots)
        for layer in range(layers):
            assert kt.u8(cache.latent[layer].contiguous()).reshape(-1).tobytes() == lat[layer].tobytes(), case
            assert kt.u8(cache.rope[layer].contiguous()).reshape(-1).tobytes() == rop[layer].tobytes(), case
    if total == 0:
        return
    first = int(rng.integers(0, layers))
    count = int(rng.integers(1, layers - first + 1))
    got_latent, got_rope = kt.gather(cache, kt.dev_i32(table), kt.dev_i32(ctxs), fused_out=bool(rng.integers(0, 2)),
                                     layer_begin=first, layer_count=count)
    for i in range(count):
        layer = first + i
        if fp8:
            exp_latent, exp_rope = orc.gather_rows_fp8(lat[layer], rop[layer], scl[layer], bs, table, ctxs)
            assert kt.bits16(got_latent[i]).tobytes() == exp_latent.tobytes(), case
            assert kt.bits16(got_rope[i]).tobytes() == exp_rope.tobytes(), case
        else:
            assert torch.equal(got_latent[i].contiguous(), latent_src[layer]), case
            assert torch.equal(got_rope[i].contiguous(), rope_src[layer]), case
