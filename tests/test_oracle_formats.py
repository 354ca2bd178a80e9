"""Pins the oracle's number formats and PRNG: bf16 and E4M3 against torch's CPU casts (a library
routine), the full E4M3 decode table, tie cases, saturation, and SplitMix64's published
known answers."""
import ctypes as C

import numpy as np
import torch

import oracle_ffi as orc


def test_bf16_round_to_nearest_even_matches_torch(oracle):
    gen = torch.Generator().manual_seed(0)
    values = torch.cat([torch.randn(4000, generator=gen) * 10 ** torch.randint(-6, 6, (4000,), generator=gen).float(),
                        torch.tensor([0.0, -0.0, 1.0, -1.0, 3.3895314e38, 1e-40, 65504.0])])
    # exact ties: bf16 value + half an ulp, both parities
    base = torch.tensor([1.0, 1.0078125, 2.0, 2.015625, 0.5, 0.50390625])
    ties = (base.view(torch.int32) + 0x8000).view(torch.float32)
    values = torch.cat([values, ties])
    expected = values.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.kvo_bf16_from_f32(float(v)) for v in values.numpy()], dtype=np.uint16)
    assert np.array_equal(got, expected)
    back = np.array([oracle.kvo_bf16_to_f32(int(b)) for b in got], dtype=np.float32)
    assert np.array_equal(back, values.to(torch.bfloat16).float().numpy())


def test_e4m3_decode_table_matches_torch(oracle):
    codes = torch.arange(256, dtype=torch.uint8)
    expected = codes.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([oracle.kvo_e4m3_to_f32(c) for c in range(256)], dtype=np.float32)
    for c in range(256):
        if np.isnan(expected[c]):
            assert c in (0x7f, 0xff) and np.isnan(got[c])
        else:
            assert got[c] == expected[c], hex(c)
    assert got[0x7e] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def test_e4m3_encode_matches_torch_within_range_and_saturates(oracle):
    gen = torch.Generator().manual_seed(1)
    values = torch.cat([
        torch.randn(20000, generator=gen) * 100,
        torch.randn(5000, generator=gen) * 0.01,
        (torch.rand(5000, generator=gen) - 0.5) * 2 * 448,
        torch.tensor([0.0, -0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 2.0 ** -6, 447.9]),
    ])
    # every midpoint between neighbouring representable magnitudes (ties -> even), and just off them
    table = np.array([orc.load().kvo_e4m3_to_f32(c) for c in range(0x7f)], dtype=np.float64)
    mids = (table[:-1] + table[1:]) / 2
    values = torch.cat([values, torch.tensor(mids, dtype=torch.float32),
                        torch.tensor(np.nextafter(mids.astype(np.float32), np.float32(0))),
                        torch.tensor(np.nextafter(mids.astype(np.float32), np.float32(1000)))])
    values = values[values.abs() <= 448.0]
    expected = values.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([oracle.kvo_e4m3_from_f32(float(v)) for v in values.numpy()], dtype=np.uint8)
    assert np.array_equal(got, expected)
    # beyond the finite range the oracle saturates (torch would give NaN): +-448
    for v, code in ((449.0, 0x7e), (1e9, 0x7e), (float("inf"), 0x7e), (-500.0, 0xfe), (464.0, 0x7e), (463.9, 0x7e)):
        assert oracle.kvo_e4m3_from_f32(v) == code
    assert oracle.kvo_e4m3_from_f32(float("nan")) & 0x7f == 0x7f


def test_row_scale_maps_absmax_to_448_and_guards_zero_rows(oracle):
    gen = torch.Generator().manual_seed(2)
    for trial in range(50):
        latent = (torch.randn(512, generator=gen) * (1 + trial)).to(torch.bfloat16)
        rope = torch.randn(64, generator=gen).to(torch.bfloat16)
        if trial % 3 == 0:
            rope[5] = 100.0 * (trial + 1)  # the maximum may sit in the rope part
        lb = latent.view(torch.int16).numpy().view(np.uint16)
        rb = rope.view(torch.int16).numpy().view(np.uint16)
        scale = oracle.kvo_fp8_row_scale(lb.ctypes.data_as(C.c_void_p), 512, rb.ctypes.data_as(C.c_void_p), 64)
        absmax = max(latent.float().abs().max().item(), rope.float().abs().max().item())
        assert scale == np.float32(absmax) / np.float32(448.0)
        assert oracle.kvo_e4m3_from_f32(float(np.float32(absmax) / np.float32(scale))) == 0x7e
    zeros = np.zeros(512, dtype=np.uint16)
    assert oracle.kvo_fp8_row_scale(zeros.ctypes.data_as(C.c_void_p), 512, zeros.ctypes.data_as(C.c_void_p), 64) == 1.0


def test_fp8_append_then_gather_round_trip_bounds():
    bs, blocks, rows = 16, 4, 40
    gen = torch.Generator().manual_seed(3)
    latent = torch.randn(rows, 512, generator=gen)
    latent = torch.where(torch.rand(rows, 512, generator=gen) < 0.01, latent * 20, latent).to(torch.bfloat16)
    rope = torch.randn(rows, 64, generator=gen).to(torch.bfloat16)
    lb = latent.view(torch.int16).numpy().view(np.uint16)
    rb = rope.view(torch.int16).numpy().view(np.uint16)
    lat_plane = np.zeros(blocks * bs * 512, dtype=np.uint8)
    rope_plane = np.zeros(blocks * bs * 64, dtype=np.uint8)
    scale_plane = np.zeros(blocks * bs, dtype=np.float32)
    table = np.array([[2, 0, 3, 1]], dtype=np.int32)
    pos = np.arange(rows)
    slots = (table[0, pos // bs] * bs + pos % bs).astype(np.int32)
    orc.append_rows_fp8(lat_plane, rope_plane, scale_plane, bs, lb, rb, slots)
    # codes equal torch's cast of x / scale (library routine), scales equal absmax / 448
    absmax = torch.maximum(latent.float().abs().amax(-1), rope.float().abs().amax(-1))
    scale = (absmax / 448.0).numpy().astype(np.float32)
    assert np.array_equal(scale_plane[slots], scale)
    expect_codes = (latent.float() / torch.tensor(scale).unsqueeze(-1)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(lat_plane.reshape(-1, 512)[slots], expect_codes)
    got_latent, got_rope = orc.gather_rows_fp8(lat_plane, rope_plane, scale_plane, bs, table, [rows])
    y = orc.bf16_to_f32(got_latent)
    expect_y = (torch.tensor(expect_codes).view(torch.float8_e4m3fn).float() * torch.tensor(scale).unsqueeze(-1)).to(torch.bfloat16)
    assert np.array_equal(got_latent, expect_y.view(torch.int16).numpy().view(np.uint16))
    x = latent.float().numpy()
    bound = np.maximum(np.abs(x) * (2.0 ** -4 + 2.0 ** -8), scale[:, None] * 2.0 ** -9)
    assert (np.abs(x - y) <= bound).all()


def test_splitmix64_known_answers(oracle):
    # Published outputs of Vigna's splitmix64.c for seed 1234567.
    state = C.c_uint64(1234567)
    expected = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
                16408922859458223821]
    assert [oracle.kvo_splitmix64(C.byref(state)) for _ in range(5)] == expected


def test_division_by_448_in_three_fused_steps_is_exact_for_every_bf16_maximum():
    """The FP8 append kernel forms scale = absmax / 448 as q + (absmax - 448 q) y with y = RN(1/448)
    and q = RN(absmax y), one fused multiply-add each (csrc/kernels/paged_copy.hip). absmax is a
    bf16 value, so the claim that this equals the correctly rounded quotient is checked here for
    every bf16 value the kernel sends down that path (2^-100 up to the largest finite one), in exact
    rational arithmetic; the oracle's own scale (a float division) is compared on the way."""
    from fractions import Fraction

    def rn32(value):
        guess = np.float32(float(value))          # correctly rounded to double, then to float: may be one step off
        best = guess
        for cand in (np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))):
            d_cand, d_best = abs(Fraction(float(cand)) - value), abs(Fraction(float(best)) - value)
            if d_cand < d_best or (d_cand == d_best and (int(np.float32(cand).view(np.uint32)) & 1) == 0):
                best = cand
        return np.float32(best)

    y = rn32(Fraction(1, 448))
    assert int(y.view(np.uint32)) == 0x3B124925
    Y = Fraction(float(y))
    checked = 0
    for bits in range(1, 0x7F80):
        a = np.array([bits << 16], dtype=np.uint32).view(np.float32)[0]
        if a < np.float32(2.0 ** -100):
            continue
        A = Fraction(float(a))
        q0 = rn32(A * Y)
        r0 = rn32(A - 448 * Fraction(float(q0)))
        q1 = rn32(Fraction(float(q0)) + Fraction(float(r0)) * Y)
        assert q1 == rn32(A / 448), hex(bits)
        assert q1 == np.float32(a) / np.float32(448.0), hex(bits)     # what the oracle's division gives
        checked += 1
    assert checked == 29184
