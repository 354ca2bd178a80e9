"""Pins the oracle's block-32 MX quantisation (kvo_mx_quant_rows) against what the published
format fixes: closed forms at powers of two and at the saturation edge (a rounded instead of a
floored exponent, or an emax of 7 or 9, fails there), a brute-force nearest-value search over all
E4M3 codes with ties to the even code, block independence, the zero / non-finite / trailing-block
cases and the clamp of the shared exponent. The reference holds no vectors for this operator (its
mock checks shapes and dtypes only, mock/mock_ops.cpp:339-354)."""
import numpy as np

import oracle_ffi as orc


def bf16(values):
    lib = orc.load()
    flat = np.asarray(values, dtype=np.float32).reshape(-1)
    return np.array([lib.kvo_bf16_from_f32(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(values))


def f32(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32)


def e4m3_values():
    lib = orc.load()
    return np.array([lib.kvo_e4m3_to_f32(c) for c in range(256)], dtype=np.float64)


def test_powers_of_two_and_the_saturation_edge():
    for k in (-20, -3, 0, 5, 40):
        codes, scales = orc.mx_quant_rows(bf16(np.full((1, 32), 2.0 ** k)))
        assert scales[0, 0] == k - 8 + 127 and (codes == 0x78).all()          # 2^k = 256 * 2^(k-8)
        codes, scales = orc.mx_quant_rows(bf16(np.full((1, 32), -448.0 * 2.0 ** k)))
        assert scales[0, 0] == k + 127 and (codes == 0xFE).all()              # -448 = largest magnitude
        row = np.full((1, 32), 2.0 ** k)
        row[0, 7] = 480.0 * 2.0 ** k                                          # same binade as 448: floor, then saturate
        codes, scales = orc.mx_quant_rows(bf16(row))
        assert scales[0, 0] == k + 127 and codes[0, 7] == 0x7E
        assert codes[0, 0] == 0x38                                            # 1.0 at scale 2^k
        row[0, 7] = 512.0 * 2.0 ** k                                          # next binade: the scale doubles
        codes, scales = orc.mx_quant_rows(bf16(row))
        assert scales[0, 0] == k + 128 and codes[0, 7] == 0x78 and codes[0, 0] == 0x30


def test_brute_force_nearest_code_per_block():
    rng = np.random.default_rng(11)
    rows, cols = 24, 512
    # every block at its own magnitude, so a scale shared over the wrong span cannot pass
    x = rng.standard_normal((rows, cols)) * np.repeat(2.0 ** rng.integers(-12, 12, (rows, cols // 32)), 32, axis=1)
    x[3, 40:45] = 0.0
    bits = bf16(x)
    codes, scales = orc.mx_quant_rows(bits)
    v = f32(bits).astype(np.float64).reshape(rows, cols // 32, 32)
    table = e4m3_values()
    finite = np.array([c for c in range(256) if not np.isnan(table[c])])
    shared = np.floor(np.log2(np.abs(v).max(axis=2))) - 8
    assert np.array_equal(scales, (shared + 127).astype(np.uint8))
    scaled = v / 2.0 ** shared[..., None]
    got = codes.reshape(rows, cols // 32, 32)
    dist = np.abs(scaled[..., None] - table[finite])                          # [.., 32, 254]
    best = dist.min(axis=-1)
    assert np.array_equal(np.abs(table[got] - scaled), best)                  # a nearest value (448 when beyond)
    tie = (dist == best[..., None]).sum(axis=-1) > 1
    nonzero = scaled != 0
    assert ((got[tie & nonzero] & 1) == 0).all()                              # ties go to the even code
    assert np.array_equal(got >> 7, (np.signbit(scaled)).astype(np.uint8))    # sign kept, also on values rounded to zero


def test_zero_nonfinite_trailing_and_clamped_blocks():
    codes, scales = orc.mx_quant_rows(np.zeros((2, 64), dtype=np.uint16))
    assert not codes.any() and not scales.any()
    row = bf16(np.ones((1, 64)))
    row[0, 40] = 0x7F80                                                       # +inf in the second block only
    codes, scales = orc.mx_quant_rows(row)
    assert scales[0, 0] == 127 - 8 and scales[0, 1] == 0xFF
    assert (codes[0, :32] == 0x78).all() and ((codes[0, 32:] & 0x7F) == 0x7F).all()
    # trailing block of 8: its own maximum
    row = bf16(np.concatenate([np.full(32, 4.0), np.full(8, 0.5)])[None])
    codes, scales = orc.mx_quant_rows(row)
    assert scales.shape == (1, 2) and list(scales[0]) == [2 - 8 + 127, -1 - 8 + 127] and (codes == 0x78).all()
    # smallest normal bf16: the shared exponent clamps at -127, the element keeps the rest
    row = bf16(np.full((1, 32), 2.0 ** -126))
    codes, scales = orc.mx_quant_rows(row)
    assert scales[0, 0] == 0 and (codes == 0x40).all()                        # 2^-126 / 2^-127 = 2


def test_dequantised_error_bound_and_idempotence():
    rng = np.random.default_rng(12)
    bits = bf16(rng.standard_normal((16, 256)) * 3)
    codes, scales = orc.mx_quant_rows(bits)
    table = e4m3_values()
    deq = table[codes] * np.repeat(2.0 ** (scales.astype(np.float64) - 127), 32, axis=1)
    v = f32(bits).astype(np.float64)
    step = np.repeat(2.0 ** (scales.astype(np.float64) - 127), 32, axis=1)
    assert (np.abs(deq - v) <= np.maximum(np.abs(v) / 16, step * 2.0 ** -10) + 32 * step * (np.abs(v) > 448 * step)).all()
    # the dequantised values are bf16-representable (4 significant bits) and quantise to themselves
    codes2, scales2 = orc.mx_quant_rows(bf16(deq))
    same_scale = scales2 == scales                                            # a block whose maximum rounded up a binade may move
    assert same_scale.mean() > 0.9
    assert np.array_equal(codes2[np.repeat(same_scale, 32, axis=1)], codes[np.repeat(same_scale, 32, axis=1)])
