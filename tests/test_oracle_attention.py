"""Pins the oracle's decode attention: against torch's float64 softmax(q k^T * scale) v on small
inputs (a library routine, not the reference), and through the special cases the
mathematics fixes. A dropped rope term, a wrong scale, a transposed operand or a
table-indexing slip fails at least one of these."""
import math

import numpy as np
import torch

import oracle_ffi as orc

LATENT, ROPE = 512, 64
SCALE = 1.0 / math.sqrt(192.0)


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _case(seed, ctxs, bs, heads, blocks):
    gen = torch.Generator().manual_seed(seed)
    perm = torch.randperm(blocks, generator=gen).numpy()
    width = max(1, max(-(-c // bs) for c in ctxs))
    table = np.zeros((len(ctxs), width), dtype=np.int32)
    cursor = 0
    for s, n in enumerate(ctxs):
        need = -(-n // bs)
        table[s, :need] = perm[cursor:cursor + need]
        cursor += need
    latent = torch.zeros(blocks * bs, LATENT, dtype=torch.bfloat16)
    rope = torch.zeros(blocks * bs, ROPE, dtype=torch.bfloat16)
    rows = []
    for s, n in enumerate(ctxs):
        pos = np.arange(n)
        slots = table[s, pos // bs] * bs + pos % bs
        l = torch.randn(n, LATENT, generator=gen).to(torch.bfloat16)
        r = torch.randn(n, ROPE, generator=gen).to(torch.bfloat16)
        latent[slots] = l
        rope[slots] = r
        rows.append((l, r))
    q = torch.randn(len(ctxs), heads, LATENT + ROPE, generator=gen).to(torch.bfloat16)
    return q, latent, rope, table, rows


def _torch_reference(q, rows, scale):
    outs, lses = [], []
    for s, (l, r) in enumerate(rows):
        k = torch.cat([l, r], dim=-1).double()
        scores = q[s].double() @ k.T * scale
        outs.append(torch.softmax(scores, dim=-1) @ l.double())
        lses.append(torch.logsumexp(scores, dim=-1))
    return torch.stack(outs).numpy(), torch.stack(lses).numpy()


def test_matches_torch_float64_on_small_inputs():
    for seed, bs in ((0, 4), (1, 16), (2, 64)):
        ctxs = [1, bs - 1, bs, bs + 1, 3 * bs + 2]
        q, latent, rope, table, rows = _case(seed, ctxs, bs, heads=5, blocks=12)
        out, lse = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1),
                                  _bits(rope).reshape(-1), bs, table, ctxs, SCALE)
        ref, ref_lse = _torch_reference(q, rows, SCALE)
        assert np.abs(out - ref).max() <= 1e-6
        assert np.abs(lse - ref_lse).max() <= 1e-5
        out32, _ = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1),
                                  _bits(rope).reshape(-1), bs, table, ctxs, SCALE, accum_f32=True)
        assert np.abs(out32 - ref).max() <= 1e-4


def test_special_cases():
    bs = 8
    # context of one token: output is that latent row exactly
    q, latent, rope, table, rows = _case(3, [1], bs, heads=3, blocks=2)
    out, lse = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1),
                              _bits(rope).reshape(-1), bs, table, [1], SCALE)
    assert np.array_equal(out[0], np.broadcast_to(rows[0][0].float().numpy(), (3, LATENT)))
    # lse of one token is its score: scale * (q_lat . c + q_rope . r) -- pins the scale and both terms
    k = torch.cat(rows[0], dim=-1).double()[0]
    assert np.allclose(lse[0], (q[0].double() @ k * SCALE).numpy(), rtol=0, atol=1e-5)
    # identical rows: output equals the row, lse = score + log(n)
    n = 19
    q, latent, rope, table, rows = _case(4, [n], bs, heads=2, blocks=4)
    latent[:] = latent[table[0, 0] * bs]
    rope[:] = rope[table[0, 0] * bs]
    out, lse = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1),
                              _bits(rope).reshape(-1), bs, table, [n], SCALE)
    row = latent[0].float().numpy()
    assert np.abs(out[0] - row).max() <= 1e-6
    score = (q[0].double() @ torch.cat([latent[0], rope[0]]).double() * SCALE).numpy()
    assert np.allclose(lse[0], score + math.log(n), atol=1e-5)
    # empty sequence: zeros and lse = -inf
    out, lse = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1),
                              _bits(rope).reshape(-1), bs, table, [0], SCALE)
    assert (out == 0).all() and np.isneginf(lse).all()


def test_rope_term_and_scale_matter_and_block_permutation_does_not():
    bs, ctxs = 16, [50, 33]
    q, latent, rope, table, rows = _case(5, ctxs, bs, heads=4, blocks=8)
    args = (_bits(q[..., :LATENT]), _bits(q[..., LATENT:]))
    base, _ = orc.mla_decode(*args, _bits(latent).reshape(-1), _bits(rope).reshape(-1), bs, table, ctxs, SCALE)
    no_rope, _ = orc.mla_decode(*args, _bits(latent).reshape(-1), np.zeros(rope.numel(), np.uint16), bs, table, ctxs, SCALE)
    assert np.abs(base - no_rope).max() > 1e-3
    other_scale, _ = orc.mla_decode(*args, _bits(latent).reshape(-1), _bits(rope).reshape(-1), bs, table, ctxs, 1 / math.sqrt(576))
    assert np.abs(base - other_scale).max() > 1e-3
    # move the physical blocks, keep the logical order: identical output
    perm = np.array([3, 7, 0, 5, 1, 6, 2, 4])
    latent2 = latent.view(8, bs, LATENT)[np.argsort(perm)].reshape(-1, LATENT)
    rope2 = rope.view(8, bs, ROPE)[np.argsort(perm)].reshape(-1, ROPE)
    table2 = perm[table].astype(np.int32)
    table2[table == 0] = perm[0]
    moved, _ = orc.mla_decode(*args, _bits(latent2).reshape(-1), _bits(rope2).reshape(-1), bs, table2, ctxs, SCALE)
    assert np.array_equal(base, moved)


def test_fp8_cache_matches_torch_on_dequantized_rows():
    bs, ctxs = 16, [40, 7]
    q, latent, rope, table, rows = _case(6, ctxs, bs, heads=3, blocks=6)
    lat_plane = np.zeros(6 * bs * LATENT, dtype=np.uint8)
    rope_plane = np.zeros(6 * bs * ROPE, dtype=np.uint8)
    scale_plane = np.zeros(6 * bs, dtype=np.float32)
    deq = []
    for s, (l, r) in enumerate(rows):
        pos = np.arange(ctxs[s])
        slots = (table[s, pos // bs] * bs + pos % bs).astype(np.int32)
        orc.append_rows_fp8(lat_plane, rope_plane, scale_plane, bs, _bits(l), _bits(r), slots)
        scale = torch.maximum(l.float().abs().amax(-1), r.float().abs().amax(-1)).unsqueeze(-1) / 448.0
        dl = (l.float() / scale).to(torch.float8_e4m3fn).float() * scale
        dr = (r.float() / scale).to(torch.float8_e4m3fn).float() * scale
        deq.append((dl, dr))
    out, _ = orc.mla_decode(_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), lat_plane, rope_plane, bs, table, ctxs, SCALE,
                            scale_plane=scale_plane)
    ref, _ = _torch_reference(q, deq, SCALE)
    assert np.abs(out - ref).max() <= 1e-5


def test_sparse_selection_reduces_to_the_dense_routine_and_to_torch():
    """The selected-token variant: (a) indices 0..n-1 reproduce the dense result bit for bit;
    (b) any selection equals torch's float64 softmax over exactly the selected rows, in the order
    given; (c) the list ends at the first negative entry or entry beyond the sequence; (d) an
    empty selection gives zeros and lse = -inf; (e) the result does not depend on the order of
    the selection beyond float64 rounding."""
    bs, heads = 16, 3
    ctxs = [40, 7, 65, 33]
    q, latent, rope, table, rows = _case(5, ctxs, bs, heads=heads, blocks=14)
    args = (_bits(q[..., :LATENT]), _bits(q[..., LATENT:]), _bits(latent).reshape(-1), _bits(rope).reshape(-1), bs, table, ctxs, SCALE)
    dense, dense_lse = orc.mla_decode(*args)
    k = 48
    identity = np.full((len(ctxs), k), -1, dtype=np.int32)
    for s, n in enumerate(ctxs):
        identity[s, :min(n, k)] = np.arange(min(n, k))
    out, lse = orc.mla_decode(*args, sparse_indices=identity)
    for s, n in enumerate(ctxs):
        if n <= k:  # the whole sequence is selected
            assert np.array_equal(out[s], dense[s]) and np.array_equal(lse[s], dense_lse[s])
    rng = np.random.default_rng(6)
    picks = np.full((len(ctxs), k), -1, dtype=np.int32)
    counts = [25, 0, 48, 10]
    for s, n in enumerate(ctxs):
        picks[s, :counts[s]] = rng.permutation(n)[:counts[s]]
    picks[3, 10] = 33          # == seq_len: ends the list like a negative entry
    picks[3, 11] = 2           # after the end: ignored
    out, lse = orc.mla_decode(*args, sparse_indices=picks)
    for s in range(len(ctxs)):
        chosen = picks[s, :counts[s]]
        if counts[s] == 0:
            assert not out[s].any() and np.isneginf(lse[s]).all()
            continue
        l, r = rows[s]
        sub = [(l[chosen], r[chosen])]
        want, want_lse = _torch_reference(q[s:s + 1], sub, SCALE)
        assert np.abs(out[s] - want[0]).max() <= 1e-6 * max(1.0, np.abs(want).max())
        assert np.abs(lse[s] - want_lse[0]).max() <= 1e-5
    shuffled = picks.copy()
    shuffled[0, :25] = picks[0, :25][::-1]
    out2, lse2 = orc.mla_decode(*args, sparse_indices=shuffled)
    assert np.abs(out2[0] - out[0]).max() <= 1e-6 and np.abs(lse2[0] - lse[0]).max() <= 1e-6
