"""Pins the oracle's latent RMSNorm + key RoPE (kvo_norm_rope_rows) without the reference's
numerics (none exist on CPU): closed forms and special cases chosen so that a dropped epsilon, a
missing gamma, a mean taken as a sum, a wrong rotation sign or a swapped half each fails one of
them, plus an independent float64 numpy evaluation and exact single rounding to bf16."""
import math

import numpy as np

import oracle_ffi as orc

LATENT, ROPE, EPS = 512, 64, 1e-6


def bf16(values):
    """float64/32 array -> bf16 bit patterns, round to nearest even (via the oracle's scalar routine)."""
    lib = orc.load()
    flat = np.asarray(values, dtype=np.float32).reshape(-1)
    return np.array([lib.kvo_bf16_from_f32(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(values))


def f32(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32)


def tables(positions, theta=10000.0):
    inv = theta ** (-np.arange(0, ROPE // 2, dtype=np.float64) * 2 / ROPE)
    ang = np.outer(np.arange(positions, dtype=np.float64), inv)
    return bf16(np.concatenate([np.cos(ang), np.cos(ang)], axis=1)), bf16(np.concatenate([np.sin(ang), np.sin(ang)], axis=1))


def test_constant_row_normalises_to_gamma():
    # x = c everywhere: mean(x^2) = c^2, y = gamma * c / sqrt(c^2 + eps). A sum instead of a mean
    # would give gamma / sqrt(512); a dropped gamma would give 1.
    cos, sin = tables(4)
    gamma = bf16(np.linspace(0.5, 2.0, LATENT))
    for c in (2.0, -0.75):
        kv = np.concatenate([bf16(np.full(LATENT, c)), bf16(np.zeros(ROPE))])[None]
        latent, rope = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, [1])
        expect = bf16(f32(gamma).astype(np.float64) * c / math.sqrt(c * c + EPS))
        assert np.array_equal(latent[0], expect)
        assert not rope.any()


def test_epsilon_dominates_a_zero_row_and_tiny_rows():
    cos, sin = tables(2)
    gamma = bf16(np.ones(LATENT))
    kv = np.zeros((1, LATENT + ROPE), dtype=np.uint16)
    latent, _ = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, [0])
    assert not latent.any()  # 0 * rstd, and rstd = 1/sqrt(eps) is finite
    tiny = 2.0 ** -20  # x^2 << eps: y = x / sqrt(x^2 + eps) ~ x * 1000, not x / |x|
    kv = np.concatenate([bf16(np.full(LATENT, tiny)), bf16(np.zeros(ROPE))])[None]
    latent, _ = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, [0])
    assert np.array_equal(latent[0], bf16(np.full(LATENT, tiny / math.sqrt(tiny * tiny + EPS))))


def test_rope_position_zero_is_identity_and_quarter_turn_swaps_halves():
    gamma = bf16(np.ones(LATENT))
    rng = np.random.default_rng(1)
    r = bf16(rng.standard_normal(ROPE))
    kv = np.concatenate([bf16(np.ones(LATENT)), r])[None]
    cos, sin = tables(3)
    _, rope = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, [0])
    assert np.array_equal(rope[0], r)  # cos = 1, sin = 0
    # hand-made table row: cos = 0, sin = 1 -> out[i] = -r[i+32], out[i+32] = +r[i]
    cos_q, sin_q = np.zeros((1, ROPE), np.uint16), bf16(np.ones((1, ROPE)))
    _, rope = orc.norm_rope_rows(kv, gamma, EPS, cos_q, sin_q, [0])
    assert np.array_equal(f32(rope[0][:32]), -f32(r[32:]))
    assert np.array_equal(f32(rope[0][32:]), f32(r[:32]))


def test_rope_preserves_pair_norms_and_uses_the_row_of_the_position():
    gamma = bf16(np.ones(LATENT))
    rng = np.random.default_rng(2)
    cos, sin = tables(64)
    kv = np.concatenate([bf16(rng.standard_normal((5, LATENT))), bf16(rng.standard_normal((5, ROPE)))], axis=1)
    positions = [63, 0, 17, 17, 5]
    _, rope = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, positions)
    r, out = f32(kv[:, LATENT:]).astype(np.float64), f32(rope).astype(np.float64)
    before = r[:, :32] ** 2 + r[:, 32:] ** 2
    after = out[:, :32] ** 2 + out[:, 32:] ** 2
    assert np.allclose(after, before, rtol=2e-2, atol=1e-3)  # a rotation, up to bf16 rounding of table and result
    for t, p in enumerate(positions):
        c, s = f32(cos[p]).astype(np.float64), f32(sin[p]).astype(np.float64)
        expect = np.concatenate([r[t, :32] * c[:32] - r[t, 32:] * s[:32], r[t, 32:] * c[32:] + r[t, :32] * s[32:]])
        assert np.array_equal(rope[t], bf16(expect.astype(np.float32))) or np.abs(f32(rope[t]) - expect).max() <= 2.0 ** -8 * np.abs(expect).max()


def test_matches_independent_float64_numpy_evaluation_with_one_rounding():
    rng = np.random.default_rng(3)
    n = 64
    kv = np.concatenate([bf16(rng.standard_normal((n, LATENT)) * 3), bf16(rng.standard_normal((n, ROPE)))], axis=1)
    gamma = bf16(rng.uniform(0.2, 1.8, LATENT))
    cos, sin = tables(128)
    positions = rng.integers(0, 128, n)
    latent, rope = orc.norm_rope_rows(kv, gamma, EPS, cos, sin, positions)
    x = f32(kv[:, :LATENT]).astype(np.float64)
    y = x * f32(gamma).astype(np.float64) / np.sqrt((x * x).mean(axis=1, keepdims=True) + EPS)
    # exact single rounding: the oracle's bits must be one of the two bf16 neighbours of y, and the nearer one
    got = f32(latent).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(y), 1e-30))) - 7)
    assert (np.abs(got - y) <= ulp / 2 * (1 + 1e-12)).all()
    r = f32(kv[:, LATENT:]).astype(np.float64)
    c, s = f32(cos[positions]).astype(np.float64), f32(sin[positions]).astype(np.float64)
    expect = np.concatenate([r[:, :32] * c[:, :32] - r[:, 32:] * s[:, :32], r[:, 32:] * c[:, 32:] + r[:, :32] * s[:, 32:]], axis=1)
    got = f32(rope).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(expect), 1e-30))) - 7)
    assert (np.abs(got - expect) <= ulp / 2 * (1 + 1e-12)).all()


def test_rope_rows_share_a_position_per_group_and_agree_with_the_fused_routine():
    # kvo_rope_rows on H rows per position == kvo_norm_rope_rows' rotation applied to each row with
    # the position repeated; position 0 leaves every row of its group untouched.
    rng = np.random.default_rng(4)
    tokens, heads = 6, 5
    cos, sin = tables(32)
    rows = bf16(rng.standard_normal((tokens * heads, ROPE)))
    positions = np.array([0, 31, 7, 7, 1, 19], dtype=np.int32)
    got = orc.rope_rows(rows, cos, sin, positions, heads)
    kv = np.concatenate([np.zeros((tokens * heads, LATENT), np.uint16), rows], axis=1)
    _, want = orc.norm_rope_rows(kv, bf16(np.ones(LATENT)), EPS, cos, sin, np.repeat(positions, heads))
    assert np.array_equal(got, want)
    assert np.array_equal(got[:heads], rows[:heads])
    assert not np.array_equal(got[heads:2 * heads], rows[heads:2 * heads])
