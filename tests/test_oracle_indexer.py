"""Pins the oracle's Lightning Indexer restatement (kvo_indexer_scores / kvo_indexer_topk) by what
the published formula and the vendored kernel's selection rule fix: closed forms for the score
(ReLU before the head weights, both scales applied, even/odd head order irrelevant on exactly
representable sums), the bf16 rounding with ties away from zero, the order-preserving key, an
independent float64 numpy evaluation, and a brute-force stable sort for the top-k including ties,
short sequences and k = n. The reference holds no vectors for this operator."""
import numpy as np

import oracle_ffi as orc

D = 128


def e4m3(values):
    lib = orc.load()
    return np.array([lib.kvo_e4m3_from_f32(float(v)) for v in np.asarray(values, dtype=np.float32).reshape(-1)],
                    dtype=np.uint8).reshape(np.shape(values))


def e4m3_values(codes):
    lib = orc.load()
    table = np.array([lib.kvo_e4m3_to_f32(c) for c in range(256)], dtype=np.float64)
    return table[codes]


def bf16_bits(values):
    lib = orc.load()
    return np.array([lib.kvo_bf16_from_f32(float(v)) for v in np.asarray(values, dtype=np.float32).reshape(-1)], dtype=np.uint16)


def key_to_float(keys):
    keys = np.asarray(keys, dtype=np.uint16)
    bits = np.where(keys & 0x8000, keys & 0x7FFF, ~keys & 0xFFFF).astype(np.uint32)
    return (bits << 16).view(np.float32)


def _identity_table(tokens, bs):
    return np.arange(-(-tokens // bs), dtype=np.int32)


def test_closed_forms_relu_scales_and_rounding():
    bs, tokens, heads = 16, 8, 4
    q = np.zeros((heads, D)); q[:, 0] = [1.0, 1.0, 2.0, 1.0]
    k = np.zeros((tokens, D)); k[:, 0] = [1.0, -1.0, 0.5, 3.0, -3.0, 0.0, 2.0, 4.0]
    weights = np.array([1.0, 1.0, 1.0, -0.5])
    q_scale = np.array([1.0, 2.0, 0.25, 1.0], dtype=np.float32)
    k_scale = np.array([1.0, 1.0, 2.0, 1.0, 1.0, 1.0, 0.5, 1.0], dtype=np.float32)
    planes = np.zeros((bs, D), dtype=np.uint8); planes[:tokens] = e4m3(k)
    scales = np.zeros(bs, dtype=np.float32); scales[:tokens] = k_scale
    keys = orc.indexer_scores(e4m3(q), bf16_bits(weights), q_scale, planes, scales, bs, _identity_table(tokens, bs), tokens)
    # per token: relu(q_h k) summed with w_h * qscale_h = [1, 2, 0.25 (on 2k), -0.5] -> (1 + 2 + 0.5 - 0.5) relu(k) = 3 relu(k)
    expect = 3.0 * np.maximum(k[:, 0], 0.0) * k_scale
    assert np.array_equal(key_to_float(keys), expect.astype(np.float32))
    # ties away from zero: 1 + 2^-8 lies halfway between two bf16 values
    q1 = np.zeros((1, D)); q1[0, 0] = 1.0
    k1 = np.zeros((bs, D)); k1[0, 0] = 1.0
    halfway = np.float32(1.0 + 2.0 ** -8)
    keys = orc.indexer_scores(e4m3(q1), bf16_bits([1.0]), np.array([halfway], np.float32), e4m3(k1), np.ones(bs, np.float32), bs,
                              _identity_table(1, bs), 1)
    assert key_to_float(keys)[0] == np.float32(1.0 + 2.0 ** -7)     # nearest-even would give 1.0
    keys = orc.indexer_scores(e4m3(q1), bf16_bits([-1.0]), np.array([halfway], np.float32), e4m3(k1), np.ones(bs, np.float32), bs,
                              _identity_table(1, bs), 1)
    assert key_to_float(keys)[0] == np.float32(-(1.0 + 2.0 ** -7))


def test_key_order_is_the_order_of_the_values():
    values = np.array([-3.0, -1.0, -2.0 ** -120, -0.0, 0.0, 2.0 ** -120, 0.5, 1.0, 1.0078125, 300.0, 3e38], dtype=np.float32)
    q1 = np.zeros((1, D)); q1[0, 0] = 1.0
    bs = 16
    k1 = np.zeros((bs, D)); k1[:len(values), 0] = 1.0
    scales = np.zeros(bs, np.float32); scales[:len(values)] = values
    keys = orc.indexer_scores(e4m3(q1), bf16_bits([1.0]), np.ones(1, np.float32), e4m3(k1), scales, bs, _identity_table(len(values), bs),
                              len(values)).astype(np.int64)
    assert (np.diff(keys) >= 0).all() and keys[3] < keys[4]           # -0 sorts below +0, as its bits do
    assert np.array_equal(key_to_float(keys.astype(np.uint16)), (bf16_bits(values).astype(np.uint32) << 16).view(np.float32))


def test_scores_against_float64_numpy_through_a_shuffled_table():
    rng = np.random.default_rng(7)
    bs, tokens, heads, blocks = 16, 70, 64, 8
    q = e4m3(rng.standard_normal((heads, D)) * 2)
    k = e4m3(rng.standard_normal((tokens, D)) * 2)
    weights = bf16_bits(rng.standard_normal(heads) * 0.1)
    q_scale = rng.uniform(0.01, 0.1, heads).astype(np.float32)
    k_scale = rng.uniform(0.01, 0.1, tokens).astype(np.float32)
    table = rng.permutation(blocks)[: -(-tokens // bs)].astype(np.int32)
    planes = np.zeros((blocks * bs, D), dtype=np.uint8)
    scales = np.zeros(blocks * bs, dtype=np.float32)
    slots = table[np.arange(tokens) // bs] * bs + np.arange(tokens) % bs
    planes[slots] = k
    scales[slots] = k_scale
    keys = orc.indexer_scores(q, weights, q_scale, planes, scales, bs, table, tokens)
    w = (weights.astype(np.uint32) << 16).view(np.float32).astype(np.float64) * q_scale
    qk = e4m3_values(q) @ e4m3_values(k).T                              # [H, T], exact in float64
    want = (np.maximum(qk, 0.0) * w[:, None]).sum(axis=0) * k_scale
    got = key_to_float(keys).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 1e-30))) - 7)
    assert (np.abs(got - want) <= 0.5 * step * 1.01 + 1e-6 * np.abs(want)).all()  # bf16 rounding of an fp32 evaluation


def test_topk_against_a_stable_sort_with_ties_and_short_sequences():
    rng = np.random.default_rng(8)
    for n, k, spread in ((1000, 64, 50), (1000, 512, 4), (300, 300, 10), (10, 64, 3), (0, 8, 1), (2048, 2048, 5), (5000, 2048, 2)):
        keys = rng.integers(0, spread, n).astype(np.uint16) + 0x8000
        got = orc.indexer_topk(keys, k)
        if n <= k:
            assert list(got[:n]) == list(range(n)) and (got[n:] == -1).all()
            continue
        order = np.argsort(-keys.astype(np.int64), kind="stable")[:k]   # descending key, ties by lower index
        assert set(got.tolist()) == set(order.tolist())
        threshold = keys[order[-1]]
        greater = [t for t in range(n) if keys[t] > threshold]
        equal = [t for t in range(n) if keys[t] == threshold][: k - len(greater)]
        assert got.tolist() == greater + equal                          # the documented order
