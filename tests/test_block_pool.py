"""Block pool: the oracle's pool pinned by an independent pure-Python model, invariants and
brute force; the product's pool (KV cache manager, host backend, bookkeeping only) must
agree with the oracle bit for bit on tables, slots, free lists and compaction moves."""
import random

import ctypes as C

import numpy as np
import pytest

import mlakv_ffi as ffi
import oracle_ffi as orc

MASK = (1 << 64) - 1


def splitmix64(state):
    state = (state + 0x9E3779B97F4A7C15) & MASK
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return state, z ^ (z >> 31)


class ModelPool:
    """Pure-Python restatement of the documented semantics (FIFO free list, Fisher-Yates by
    SplitMix64, logical-order allocate and free, highest-live-to-lowest-hole compaction)."""

    def __init__(self, blocks, bs, seqs, width, seed, shuffle):
        self.blocks, self.bs, self.width = blocks, bs, width
        self.free = list(range(blocks))
        if shuffle:
            state = seed
            for i in range(blocks - 1, 0, -1):
                state, r = splitmix64(state)
                j = r % (i + 1)
                self.free[i], self.free[j] = self.free[j], self.free[i]
        self.table = [[] for _ in range(seqs)]
        self.len = [-1] * seqs

    def add(self, s, n):
        need = -(-n // self.bs)
        if self.len[s] >= 0 or need > self.width or need > len(self.free):
            return False
        self.table[s] = [self.free.pop(0) for _ in range(need)]
        self.len[s] = n
        return True

    def append(self, s):
        if self.len[s] < 0:
            return None
        p = self.len[s]
        if p % self.bs == 0:
            if len(self.table[s]) >= self.width or not self.free:
                return None
            self.table[s].append(self.free.pop(0))
        self.len[s] = p + 1
        return self.table[s][p // self.bs] * self.bs + p % self.bs

    def release(self, s):
        if self.len[s] < 0:
            return False
        self.free.extend(self.table[s])
        self.table[s] = []
        self.len[s] = -1
        return True

    def compact(self):
        live = self.blocks - len(self.free)
        owner = {}
        for s, row in enumerate(self.table):
            for i, b in enumerate(row):
                owner[b] = (s, i)
        holes = [b for b in range(live) if b not in owner]
        moves = []
        for src in range(self.blocks - 1, live - 1, -1):
            if src in owner:
                dst = holes.pop(0)
                s, i = owner.pop(src)
                self.table[s][i] = dst
                moves.append((src, dst))
        self.free = list(range(live, self.blocks))
        return moves

    def dense_table(self, seqs):
        out = np.zeros((seqs, self.width), dtype=np.int32)
        for s, row in enumerate(self.table):
            out[s, :len(row)] = row
        return out


def _check_invariants(table, lens, bs, blocks, free_list):
    owned = []
    for s, n in enumerate(lens):
        if n >= 0:
            owned += [int(b) for b in table[s, : -(-n // bs)]]
    assert len(owned) == len(set(owned)), "a physical block has two owners"
    assert not set(owned) & set(free_list)
    assert len(owned) + len(free_list) == blocks
    assert sorted(owned + list(free_list)) == list(range(blocks))


@pytest.mark.parametrize("shuffle", [False, True])
def test_random_operations_oracle_product_and_model_agree(shuffle):
    rng = random.Random(11)
    for trial in range(6):
        bs = rng.choice([4, 16, 64])
        seqs, width = 7, 9
        blocks = rng.randint(12, 40)
        seed = rng.getrandbits(63)
        model = ModelPool(blocks, bs, seqs, width, seed, shuffle)
        oracle_pool = orc.Pool(blocks, bs, seqs, width, seed=seed, shuffle=shuffle)
        arena = ffi.Arena(ffi.BACKEND_HOST)
        product = ffi.KvCache(arena, num_layers=2, block_size=bs, max_context_len=width * bs, max_batch=seqs,
                              pool_blocks=blocks, seed=seed, shuffle=int(shuffle))
        assert oracle_pool.free_list() == model.free == product.free_list()
        for _ in range(300):
            op = rng.random()
            s = rng.randrange(seqs)
            if op < 0.25:
                n = rng.randint(0, width * bs)
                ok = model.add(s, n)
                assert (oracle_pool.add_sequence(s, n) == orc.OK) == ok
                if ok:
                    product.add_sequence(s, n)
                else:
                    with pytest.raises(ffi.MlakvError):
                        product.add_sequence(s, n)
            elif op < 0.75:
                slot = model.append(s)
                status, oslot = oracle_pool.append_token(s)
                assert (status == orc.OK) == (slot is not None)
                if slot is not None:
                    assert oslot == slot == product.append_token(s)
                else:
                    with pytest.raises(ffi.MlakvError):
                        product.append_token(s)
            elif op < 0.9:
                ok = model.release(s)
                assert (oracle_pool.free_sequence(s) == orc.OK) == ok
                if ok:
                    product.free_sequence(s)
                else:
                    with pytest.raises(ffi.MlakvError):
                        product.free_sequence(s)
            else:
                moves = model.compact()
                assert oracle_pool.compact() == moves == product.compact()
                live = blocks - len(model.free)
                assert all(src >= live > dst for src, dst in moves)
                assert len({src for src, _ in moves} | {dst for _, dst in moves}) == 2 * len(moves)
            table = oracle_pool.table()
            assert np.array_equal(table, model.dense_table(seqs))
            assert np.array_equal(table, product.host_block_table())
            assert oracle_pool.free_list() == model.free == product.free_list()
            lens = [oracle_pool.seq_len(i) for i in range(seqs)]
            assert lens == model.len
            assert list(product.host_seq_lens()) == [0] * seqs  # refreshed only at upload
            _check_invariants(table, lens, bs, blocks, model.free)
        product.close()
        arena.close()


def test_slot_closed_form_brute_force(oracle):
    import ctypes as C
    for bs in (16, 64, 128):
        identity = np.arange(4, dtype=np.int32)
        shuffled = np.array([3, 0, 2, 1], dtype=np.int32)
        for pos in range(3 * bs + 1):
            assert oracle.kvo_slot(identity.ctypes.data_as(C.c_void_p), pos, bs) == pos  # reference: slot = position
            expected = int(shuffled[pos // bs]) * bs + pos % bs
            assert oracle.kvo_slot(shuffled.ctypes.data_as(C.c_void_p), pos, bs) == expected


def test_gather_of_append_is_identity_and_survives_compaction():
    bs, blocks, row = 8, 20, 48
    rng = np.random.default_rng(5)
    pool = orc.Pool(blocks, bs, 4, 6, seed=123, shuffle=True)
    ctxs = [13, 8, 30, 1]
    for s, n in enumerate(ctxs):
        assert pool.add_sequence(s, n) == orc.OK
    table = pool.table()
    plane = np.zeros(blocks * bs * row, dtype=np.uint8)
    src = rng.integers(0, 256, size=(sum(ctxs), row), dtype=np.uint8)
    slots = np.concatenate([table[s, np.arange(n) // bs] * bs + np.arange(n) % bs for s, n in enumerate(ctxs)]).astype(np.int32)
    orc.append_rows(plane, bs * row, row, bs, src.reshape(-1), row, row, slots)
    written = np.zeros(blocks * bs, dtype=bool)
    written[slots] = True
    assert (plane.reshape(-1, row)[~written] == 0).all()  # untouched slots stay zero
    assert np.array_equal(orc.gather_rows(plane, bs * row, row, bs, table, ctxs, row).reshape(-1, row), src)
    pool.free_sequence(1)
    live_ctxs = [13, 0, 30, 1]
    before = orc.gather_rows(plane, bs * row, row, bs, pool.table(), live_ctxs, row)
    moves = pool.compact()
    orc.copy_blocks(plane, bs * row, bs * row, moves)
    after = orc.gather_rows(plane, bs * row, row, bs, pool.table(), live_ctxs, row)
    assert np.array_equal(before, after)
    used = sorted(int(pool.table()[s, i]) for s, n in enumerate(live_ctxs) for i in range(-(-n // bs)))
    assert used == list(range(pool.live_blocks))
    assert pool.free_list() == list(range(pool.live_blocks, blocks))


def test_upload_step_refreshes_lengths_and_resets_slot_mapping():
    arena = ffi.Arena(ffi.BACKEND_HOST)
    cache = ffi.KvCache(arena, num_layers=1, block_size=16, max_context_len=64, max_batch=3)
    arena.commit()
    cache.bind()
    cache.add_sequence(0, 5)
    cache.add_sequence(2, 16)
    s0, s2 = cache.append_token(0), cache.append_token(2)
    assert list(cache.host_slot_mapping()) == [s0, -1, s2]
    before = arena.device_allocations
    cache.upload_step(None)
    assert arena.device_allocations == before
    assert list(cache.host_seq_lens()) == [6, 0, 17]
    assert list(cache.host_slot_mapping()) == [-1, -1, -1]
    # the "device" side of the host backend is ordinary memory: the upload landed there
    import ctypes as C
    lens = (C.c_int32 * 3).from_address(cache.device_seq_lens)
    cu = (C.c_int32 * 4).from_address(cache.device_cu_seq_lens)
    slots = (C.c_int32 * 3).from_address(cache.device_slot_mapping)
    assert list(lens) == [6, 0, 17] and list(cu) == [0, 6, 6, 23] and list(slots) == [s0, -1, s2]
    table = (C.c_int32 * 12).from_address(cache.device_block_table)
    assert list(table) == list(cache.host_block_table().reshape(-1))
    # a later step that opens a block (position 16 of sequence 0 after ten more tokens) reaches the table too
    for _ in range(10):
        cache.append_token(0)
        cache.upload_step(None)
    assert list(cache.host_seq_lens()) == [16, 0, 17]
    cache.append_token(0)
    cache.upload_step(None)
    assert list(table) == list(cache.host_block_table().reshape(-1)) and table[1] == cache.host_block_table()[0, 1]
    # the one-launch step needs kernels: the bookkeeping backend refuses it and says why
    lib = ffi.load()
    rows = (C.c_uint16 * (3 * 576))()
    status = lib.mlakvKvCacheUploadStepAndAppend(cache.handle, 0, 1, C.addressof(rows), 0, 1152, C.addressof(rows), 0, 1152, None)
    assert status == ffi.ERR_CONTRACT and b"kernels" in lib.mlakvGetLastError()
    cache.close()
    arena.close()


def test_compaction_between_append_and_upload_moves_the_pending_slots():
    """A token whose slot waits for the upload sits in a block that compaction moves: the slot
    has to follow the block, or the append kernel would write the row into a freed block. The
    oracle pool, driven through the same operations, gives the expected slots."""
    bs, blocks = 16, 12
    arena = ffi.Arena(ffi.BACKEND_HOST)
    cache = ffi.KvCache(arena, num_layers=1, block_size=bs, max_context_len=64, max_batch=4, pool_blocks=blocks, seed=5, shuffle=1)
    arena.commit()
    cache.bind()
    pool = orc.Pool(blocks, bs, 4, 4, seed=5, shuffle=True)
    for s, n in enumerate([20, 33, 16, 47]):
        cache.add_sequence(s, n)
        assert pool.add_sequence(s, n) == orc.OK
    cache.upload_step(None)
    cache.free_sequence(0)
    cache.free_sequence(2)
    pool.free_sequence(0)
    pool.free_sequence(2)
    assert cache.append_token_all() == 2          # sequences 1 and 3 (3 opens a new block: 48 tokens)
    want_before = {s: pool.append_token(s)[1] for s in (1, 3)}
    assert [int(v) for v in cache.host_slot_mapping()] == [-1, want_before[1], -1, want_before[3]]
    moves = cache.compact(None)
    want_moves = pool.compact()
    assert [tuple(m) for m in moves] == [tuple(m) for m in want_moves] and len(moves) > 0
    table = pool.table()
    expected = [-1, -1, -1, -1]
    for s in (1, 3):
        pos = pool.seq_len(s) - 1
        expected[s] = int(table[s, pos // bs]) * bs + pos % bs
    assert [int(v) for v in cache.host_slot_mapping()] == expected
    assert expected != [-1, want_before[1], -1, want_before[3]]   # at least one pending slot did move
    assert np.array_equal(cache.host_block_table(), table)
    cache.close()
    arena.close()


def test_arena_outlives_its_caches_whatever_the_order_of_destruction():
    arena = ffi.Arena(ffi.BACKEND_HOST)
    cache = ffi.KvCache(arena, num_layers=1, block_size=16, max_context_len=64, max_batch=2)
    arena.commit()
    cache.bind()
    cache.add_sequence(0, 3)
    lib = ffi.load()
    handle, arena_handle = cache.handle, arena.handle
    arena.handle = None                     # the wrapper must not destroy it a second time
    lib.mlakvArenaDestroy(arena_handle)     # deferred: the cache still refers to the arena
    slot = C.c_int32()
    assert lib.mlakvKvCacheAppendToken(handle, 0, C.byref(slot)) == 0 and slot.value >= 0
    assert lib.mlakvKvCacheUploadStep(handle, None) == 0
    cache.handle = None
    lib.mlakvKvCacheDestroy(handle)         # the last cache takes the arena with it
