"""GPU parity with pools whose byte offsets do not fit 32 bits: one layer plane above 4 GiB, and
a layer offset (layer x layer stride) above 4 GiB. Append, gather, decode attention and the
compaction copy run on blocks on both sides of the 4 GiB line and on the last block of the pool.

The oracle never sees the big pool: it works on a compact pool that holds only the touched
blocks (every physical block index replaced by its rank among the touched ones), from the same
source rows. Block contents, gathered rows (bit-exact) and attention outputs (2e-2, 6e-2 for FP8)
must agree, and nothing outside the touched blocks may have been written."""
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
FOUR_GIB = 1 << 32


@pytest.fixture(autouse=True)
def _give_the_pool_back():
    """These pools are 5 to 10 GB each: they go back to the driver when their test ends, not when the
    process does (launches that follow the release of that much memory ran 2 % slower for some ten
    seconds on the box)."""
    yield
    import gc
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


class Compact:
    """The oracle's pool: the touched blocks of one layer, in rank order."""

    def __init__(self, touched, bs, fp8):
        self.rank = {block: i for i, block in enumerate(touched)}
        self.touched, self.bs, self.fp8 = touched, bs, fp8
        e = 1 if fp8 else 2
        self.e = e
        self.latent = np.zeros(len(touched) * bs * LATENT * e, dtype=np.uint8)
        self.rope = np.zeros(len(touched) * bs * ROPE * e, dtype=np.uint8)
        self.scale = np.zeros(len(touched) * bs, dtype=np.float32) if fp8 else None

    def table(self, real_table):
        return np.vectorize(lambda b: self.rank.get(int(b), 0))(real_table).astype(np.int32)

    def append(self, latent_src, rope_src, slots):
        bs, e = self.bs, self.e
        if self.fp8:
            orc.append_rows_fp8(self.latent, self.rope, self.scale, bs, kt.bits16(latent_src), kt.bits16(rope_src), slots)
        else:
            orc.append_rows(self.latent, bs * LATENT * e, LATENT * e, bs, kt.u8(latent_src).reshape(-1), LATENT * e, LATENT * e, slots)
            orc.append_rows(self.rope, bs * ROPE * e, ROPE * e, bs, kt.u8(rope_src).reshape(-1), ROPE * e, ROPE * e, slots)

    def copy(self, moves):
        bs, e = self.bs, self.e
        orc.copy_blocks(self.latent, bs * LATENT * e, bs * LATENT * e, moves)
        orc.copy_blocks(self.rope, bs * ROPE * e, bs * ROPE * e, moves)
        if self.fp8:
            orc.copy_blocks(self.scale.view(np.uint8), bs * 4, bs * 4, moves)


def _assert_blocks_equal(cache, layer, compact):
    """Every touched block holds the oracle's bytes, and the layer holds nothing else."""
    index = torch.as_tensor(compact.touched, device="cuda")
    got_latent = kt.u8(cache.latent[layer].index_select(0, index)).reshape(-1)
    got_rope = kt.u8(cache.rope[layer].index_select(0, index)).reshape(-1)
    assert got_latent.tobytes() == compact.latent.tobytes()
    assert got_rope.tobytes() == compact.rope.tobytes()
    raw = torch.uint8 if cache.fp8 else torch.int16
    assert int(torch.count_nonzero(cache.latent[layer].view(raw))) == int(np.count_nonzero(compact.latent.view(np.uint8 if cache.fp8 else np.int16)))
    assert int(torch.count_nonzero(cache.rope[layer].view(raw))) == int(np.count_nonzero(compact.rope.view(np.uint8 if cache.fp8 else np.int16)))
    if cache.fp8:
        got_scale = cache.scale[layer].index_select(0, index).cpu().numpy().reshape(-1)
        assert got_scale.tobytes() == compact.scale.tobytes()
        assert int(torch.count_nonzero(cache.scale[layer])) == int(np.count_nonzero(compact.scale))


def _assert_attention_close(got_bf16, expected, tol):
    got = got_bf16.float().cpu().numpy()
    assert np.isfinite(got).all()
    peak = np.abs(expected).max()
    assert np.abs(got - expected).max() <= tol * peak


def _run(layers, blocks, bs, fp8, layer, seq_blocks, ctxs, move_pairs, seed):
    """seq_blocks: physical blocks of each sequence, in logical order; move_pairs: (source, destination)
    block moves applied after the first round of checks (destinations untouched until then)."""
    e = 1 if fp8 else 2
    cache = kt.PagedCache(layers, blocks, bs, fp8=fp8)
    width = max(len(b) for b in seq_blocks)
    table = np.zeros((len(seq_blocks), width), dtype=np.int32)
    for s, row in enumerate(seq_blocks):
        table[s, :len(row)] = row
    touched = sorted({b for row in seq_blocks for b in row} | {dst for _, dst in move_pairs})
    compact = Compact(touched, bs, fp8)
    small_table = compact.table(table)
    # the offsets this case is about
    plane_bytes = blocks * bs * LATENT * e
    top = max(touched)
    assert layer * plane_bytes + top * bs * LATENT * e > FOUR_GIB
    print(f"layer {layer} of {layers}, {blocks} blocks of {bs} tokens, fp8={fp8}: latent plane {plane_bytes / 2**30:.2f} GiB, "
          f"highest touched byte offset {(layer * plane_bytes + (top + 1) * bs * LATENT * e) / 2**30:.2f} GiB", flush=True)

    total = sum(ctxs)
    latent_src = kt.randn_bf16((1, total, LATENT), seed=seed, outlier_fraction=0.01 if fp8 else 0.0).cuda()
    rope_src = kt.randn_bf16((1, total, ROPE), seed=seed + 1).cuda()
    kt.append(cache, latent_src, rope_src, kt.dev_i32(kt.slots_for(table, ctxs, bs)), layer_begin=layer, layer_count=1)
    torch.cuda.synchronize()
    compact.append(latent_src[0], rope_src[0], kt.slots_for(small_table, ctxs, bs))
    _assert_blocks_equal(cache, layer, compact)
    for other in range(layers):  # the other layers stay zero
        if other != layer:
            assert int(torch.count_nonzero(cache.latent[other].view(torch.uint8 if fp8 else torch.int16))) == 0

    def check_reads(real_table, small):
        got_latent, got_rope = kt.gather(cache, kt.dev_i32(real_table), kt.dev_i32(ctxs), layer_begin=layer, layer_count=1)
        if fp8:
            want_latent, want_rope = orc.gather_rows_fp8(compact.latent, compact.rope, compact.scale, bs, small, ctxs)
            assert kt.bits16(got_latent[0]).tobytes() == np.asarray(want_latent).tobytes()
            assert kt.bits16(got_rope[0]).tobytes() == np.asarray(want_rope).tobytes()
        else:
            want_latent = orc.gather_rows(compact.latent, bs * LATENT * 2, LATENT * 2, bs, small, ctxs, LATENT * 2)
            want_rope = orc.gather_rows(compact.rope, bs * ROPE * 2, ROPE * 2, bs, small, ctxs, ROPE * 2)
            assert kt.u8(got_latent[0]).reshape(-1).tobytes() == want_latent.tobytes()
            assert kt.u8(got_rope[0]).reshape(-1).tobytes() == want_rope.tobytes()
        q = kt.randn_bf16((len(ctxs), 64, LATENT + ROPE), seed=seed + 2).cuda()
        qb = kt.bits16(q)
        expected, expected_lse = orc.mla_decode(np.ascontiguousarray(qb[..., :LATENT]), np.ascontiguousarray(qb[..., LATENT:]),
                                                compact.latent if fp8 else compact.latent.view(np.uint16),
                                                compact.rope if fp8 else compact.rope.view(np.uint16), bs, small,
                                                np.asarray(ctxs, dtype=np.int32), SCALE, scale_plane=compact.scale)
        for options in ({}, {"chunk_tiles": 1}):
            out, lse, _ = kt.attention(cache, layer, q, kt.dev_i32(real_table), kt.dev_i32(ctxs), SCALE, **options)
            _assert_attention_close(out, expected, 6e-2 if fp8 else 2e-2)
            assert np.abs(lse.cpu().numpy() - expected_lse).max() <= (6e-2 if fp8 else 2e-2)

    check_reads(table, small_table)

    # compaction copies across the line, then the same reads through the moved table
    moves = np.asarray(move_pairs, dtype=np.int32)
    lib = ffi.load()
    moves_dev = kt.dev_i32(moves.reshape(-1))
    ffi.check(lib.mlakvCopyBlocks(C.byref(cache.view), layer, 1, moves_dev.data_ptr(), len(moves), kt.stream_ptr()))
    torch.cuda.synchronize()
    compact.copy([(compact.rank[int(s)], compact.rank[int(d)]) for s, d in moves])
    _assert_blocks_equal(cache, layer, compact)
    moved = table.copy()
    for source, destination in move_pairs:
        moved[table == source] = destination
    check_reads(moved, compact.table(moved))


@pytest.mark.parametrize("fp8", [False, True])
def test_one_layer_plane_above_4_gib(fp8):
    bs = 64
    block_bytes = bs * LATENT * (1 if fp8 else 2)
    line = FOUR_GIB // block_bytes              # first block that starts at or above 4 GiB
    blocks = line + 4500                        # 4.27 GiB of latent rows in the one layer
    last = blocks - 1
    # sequence 0 walks across the line and ends in the last block; sequence 1 starts in the last
    # block but one, jumps to block 0 and ends just above the line; sequence 2 stays below it
    seq_blocks = [[line - 2, line - 1, line, line + 1, last], [last - 1, 0, line + 2], [7, line - 3]]
    ctxs = [4 * bs + 37, 2 * bs + 1, bs + 64]
    # one move down across the line, one up across it, one from the last block
    move_pairs = [(line + 1, 11), (line - 3, line + 100), (last, line - 10)]
    _run(1, blocks, bs, fp8, 0, seq_blocks, ctxs, move_pairs, seed=300 + int(fp8))


def test_layer_offset_above_4_gib():
    bs = 64
    blocks = 30000                               # 1.83 GiB of latent rows per layer, 3 layers
    layers, layer = 3, 2                         # layer 2 starts at 3.66 GiB and crosses the line inside
    block_bytes = bs * LATENT * 2
    line = (FOUR_GIB - layer * blocks * block_bytes) // block_bytes  # first block of layer 2 at or above 4 GiB
    assert 0 < line < blocks - 10
    last = blocks - 1
    seq_blocks = [[line - 1, line, line + 1, last], [3, last - 1, line + 2]]
    ctxs = [3 * bs + 5, 2 * bs + 64]
    move_pairs = [(line + 1, 17), (3, last - 5)]
    _run(layers, blocks, bs, False, layer, seq_blocks, ctxs, move_pairs, seed=310)


def test_arena_commit_of_a_pool_above_4_gib_is_zero_filled_and_addressed_in_64_bits():
    """RESERVE / COMMIT of a KV pool above 4 GiB per layer on the HIP backend: the view's strides are
    the 64-bit products, the last block of the last layer is writable through the manager's own
    slot mapping, and the commit's zero-fill reached the end of the allocation."""
    import time
    bs, layers, pool = 64, 2, 70000
    arena = ffi.Arena(ffi.BACKEND_HIP)
    cache = ffi.KvCache(arena, num_layers=layers, block_size=bs, max_context_len=bs * 8, max_batch=2, pool_blocks=pool)
    begin = time.perf_counter()
    arena.commit()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - begin
    cache.bind()
    arena.seal()
    view = cache.view()
    assert view.latent_layer_stride == pool * bs * LATENT * 2 > FOUR_GIB
    assert view.latent_block_stride == bs * LATENT * 2
    total = arena.committed_bytes if hasattr(arena, "committed_bytes") else None
    print(f"arena commit of {layers} x {pool} blocks ({layers * pool * bs * (LATENT + ROPE) * 2 / 1e9:.1f} GB): {seconds * 1e3:.1f} ms"
          f" (allocation + zero-fill){'' if total is None else f', {total} bytes'}", flush=True)
    lib = ffi.load()
    # a token in the last block of the pool, last layer
    last_slot = (pool - 1) * bs + (bs - 1)
    row = kt.randn_bf16((1, 1, LATENT + ROPE), seed=5).cuda()
    latent_src, rope_src = row[..., :LATENT].contiguous(), row[..., LATENT:].contiguous()
    slots = kt.dev_i32([last_slot])
    ffi.check(lib.mlakvAppend(C.byref(view), layers - 1, 1, latent_src.data_ptr(), 0, LATENT * 2, rope_src.data_ptr(), 0, ROPE * 2,
                              slots.data_ptr(), 1, kt.stream_ptr()))
    table = kt.dev_i32(np.asarray([[pool - 1]], dtype=np.int32))
    lens, cu = kt.dev_i32([bs]), kt.dev_i32([0, bs])
    out_latent = torch.full((bs, LATENT), 7.0, dtype=torch.bfloat16, device="cuda")
    out_rope = torch.full((bs, ROPE), 7.0, dtype=torch.bfloat16, device="cuda")
    ffi.check(lib.mlakvGather(C.byref(view), layers - 1, 1, table.data_ptr(), 1, lens.data_ptr(), cu.data_ptr(), 1, bs,
                              out_latent.data_ptr(), bs * LATENT * 2, LATENT * 2, out_rope.data_ptr(), bs * ROPE * 2, ROPE * 2,
                              kt.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out_latent[bs - 1], latent_src[0, 0]) and torch.equal(out_rope[bs - 1], rope_src[0, 0])
    assert int(torch.count_nonzero(out_latent[: bs - 1].view(torch.int16))) == 0  # the rest of the block is the commit's zeros
    assert int(torch.count_nonzero(out_rope[: bs - 1].view(torch.int16))) == 0
    cache.close()
    arena.close()
