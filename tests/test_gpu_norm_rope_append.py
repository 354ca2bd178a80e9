"""GPU parity: fused latent RMSNorm + key RoPE + append (mlakvNormRopeAppend) against the CPU
oracle. The kernel works in fp32 and rounds once to bf16; the oracle works in float64 and rounds
once, so a value may land on the neighbouring bf16 when it sits within fp32 rounding error of a
bf16 midpoint: the tolerance is one bf16 ulp (2^-7 relative), and at least 99.5 % of the values
must be bit-identical. What the cache receives is then checked bit-exactly against the kernel's
own normalised output (bf16 cache) or against the oracle's quantisation of it (FP8 cache)."""
import ctypes as C

import numpy as np
import pytest
import torch

import kv_testing as kt
import mlakv_ffi as ffi
import oracle_ffi as orc

pytestmark = pytest.mark.gpu

LATENT, ROPE, EPS = kt.LATENT, kt.ROPE, 1e-6


def _tables(positions, theta=10000.0):
    inv = theta ** (-torch.arange(0, ROPE // 2, dtype=torch.float64) * 2 / ROPE)
    ang = torch.outer(torch.arange(positions, dtype=torch.float64), inv)
    cos = torch.cat([ang.cos(), ang.cos()], dim=1).to(torch.bfloat16)
    sin = torch.cat([ang.sin(), ang.sin()], dim=1).to(torch.bfloat16)
    return cos, sin


def _f32(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32)


def _within_one_ulp(got_bits, want_bits):
    got, want = _f32(got_bits).astype(np.float64), _f32(want_bits).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -126))) - 7)
    assert (np.abs(got - want) <= ulp * 1.0001).all(), np.abs(got - want).max()
    assert (got_bits == want_bits).mean() >= 0.995


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("bs", [16, 64])
def test_fused_norm_rope_append_matches_oracle(fp8, bs):
    tokens, layers, max_pos = 77, 3, 4096
    blocks = -(-tokens // bs) + 3
    layer = 1
    cache = kt.PagedCache(layers, blocks, bs, fp8=fp8)
    kv_a = kt.randn_bf16((tokens, LATENT + ROPE), seed=21, outlier_fraction=0.01)
    kv_a[5] = 0  # a zero row: epsilon keeps the normalisation finite
    gamma = (kt.randn_bf16((LATENT,), seed=22).float() * 0.2 + 1.0).to(torch.bfloat16)
    cos, sin = _tables(max_pos)
    rng = np.random.default_rng(23)
    positions = rng.integers(0, max_pos, tokens).astype(np.int32)
    slots = rng.permutation(blocks * bs)[:tokens].astype(np.int32)
    slots[9] = -1  # skipped by the write, still normalised into the optional outputs
    lib = ffi.load()
    kv_d, gamma_d, cos_d, sin_d = kv_a.cuda(), gamma.cuda(), cos.cuda(), sin.cuda()
    latent_out = torch.zeros(tokens, LATENT, dtype=torch.bfloat16, device="cuda")
    rope_out = torch.zeros(tokens, ROPE, dtype=torch.bfloat16, device="cuda")
    positions_d, slots_d = kt.dev_i32(positions), kt.dev_i32(slots)  # kept alive until the launch has run
    ffi.check(lib.mlakvNormRopeAppend(C.byref(cache.view), layer, kv_d.data_ptr(), (LATENT + ROPE) * 2, gamma_d.data_ptr(), EPS,
                                      cos_d.data_ptr(), sin_d.data_ptr(), ROPE * 2, positions_d.data_ptr(),
                                      slots_d.data_ptr(), tokens, latent_out.data_ptr(), LATENT * 2,
                                      rope_out.data_ptr(), ROPE * 2, None, 0, 0, 0, kt.stream_ptr()))
    torch.cuda.synchronize()
    want_latent, want_rope = orc.norm_rope_rows(kt.bits16(kv_a), kt.bits16(gamma), EPS, kt.bits16(cos), kt.bits16(sin), positions)
    got_latent, got_rope = kt.bits16(latent_out), kt.bits16(rope_out)
    _within_one_ulp(got_latent, want_latent)
    _within_one_ulp(got_rope, want_rope)
    assert not got_latent[5].any()

    # what the cache holds: exactly the kernel's own rows at their slots, nothing anywhere else
    live = slots >= 0
    if fp8:
        lat_plane = np.zeros(blocks * bs * LATENT, dtype=np.uint8)
        rope_plane = np.zeros(blocks * bs * ROPE, dtype=np.uint8)
        scale_plane = np.zeros(blocks * bs, dtype=np.float32)
        orc.append_rows_fp8(lat_plane, rope_plane, scale_plane, bs, got_latent[live], got_rope[live], slots[live])
        assert np.array_equal(cache.latent_np(layer), lat_plane)
        assert np.array_equal(cache.rope_np(layer), rope_plane)
        assert np.array_equal(cache.scale_np(layer), scale_plane)
    else:
        lat_plane = np.zeros((blocks * bs, LATENT), dtype=np.uint16)
        rope_plane = np.zeros((blocks * bs, ROPE), dtype=np.uint16)
        lat_plane[slots[live]] = got_latent[live]
        rope_plane[slots[live]] = got_rope[live]
        assert np.array_equal(cache.latent_np(layer), lat_plane.reshape(-1))
        assert np.array_equal(cache.rope_np(layer), rope_plane.reshape(-1))
    for other in (0, 2):
        assert not cache.latent_np(other).any() and not cache.rope_np(other).any()


def test_optional_outputs_and_argument_checks():
    bs, blocks, tokens = 64, 2, 4
    cache = kt.PagedCache(1, blocks, bs)
    lib = ffi.load()
    kv = kt.randn_bf16((tokens, LATENT + ROPE), seed=1).cuda()
    gamma = torch.ones(LATENT, dtype=torch.bfloat16, device="cuda")
    cos, sin = _tables(8)
    cos, sin = cos.cuda(), sin.cuda()
    pos, slots = kt.dev_i32([0, 1, 2, 3]), kt.dev_i32([3, 2, 1, 0])

    def call(**over):
        args = dict(view=C.byref(cache.view), layer=0, kv=kv.data_ptr(), stride=(LATENT + ROPE) * 2, gamma=gamma.data_ptr(), eps=EPS,
                    cos=cos.data_ptr(), sin=sin.data_ptr(), tstride=ROPE * 2, pos=pos.data_ptr(), slots=slots.data_ptr(), n=tokens,
                    lo=None, lo_stride=0, ro=None, ro_stride=0, q=None, q_token=0, q_head=0, heads=0)
        args.update(over)
        return lib.mlakvNormRopeAppend(args["view"], args["layer"], args["kv"], args["stride"], args["gamma"], args["eps"],
                                       args["cos"], args["sin"], args["tstride"], args["pos"], args["slots"], args["n"],
                                       args["lo"], args["lo_stride"], args["ro"], args["ro_stride"], args["q"], args["q_token"],
                                       args["q_head"], args["heads"], kt.stream_ptr())

    assert call() == 0  # no optional outputs
    torch.cuda.synchronize()
    assert cache.latent[0, 0, :4].abs().sum().item() > 0
    assert call(n=0) == 0
    assert call(kv=None) == ffi.ERR_PARAM_NULLPTR
    assert call(gamma=None) == ffi.ERR_PARAM_NULLPTR
    assert call(eps=0.0) == ffi.ERR_PARAM_INVALID
    assert call(stride=LATENT * 2) == ffi.ERR_PARAM_INVALID      # the row must hold latent and rope
    assert call(kv=kv.data_ptr() + 2) == ffi.ERR_PARAM_INVALID   # alignment
    assert call(layer=1) == ffi.ERR_PARAM_INVALID
    assert call(n=-1) == ffi.ERR_PARAM_INVALID
    q = torch.zeros(tokens, 4, LATENT + ROPE, dtype=torch.bfloat16, device="cuda")
    row = (LATENT + ROPE) * 2
    q_rope = q.data_ptr() + LATENT * 2
    assert call(q=q_rope, q_token=4 * row, q_head=row, heads=4) == 0
    assert call(q=q_rope, q_token=4 * row, q_head=row, heads=0) == ffi.ERR_PARAM_INVALID
    assert call(q=q_rope + 2, q_token=4 * row, q_head=row, heads=4) == ffi.ERR_PARAM_INVALID
    assert call(q=q_rope, q_token=3 * row, q_head=row, heads=4) == ffi.ERR_PARAM_INVALID  # heads overlap the next token
    assert call(q=q_rope, q_token=4 * row, q_head=row, heads=4, cos=cos.data_ptr() + 2) == ffi.ERR_PARAM_INVALID
    torch.cuda.synchronize()


@pytest.mark.parametrize("heads", [64, 13])
def test_query_rope_slices_rotate_in_place_with_the_key(heads):
    """The reference rotates q_rope and k_rope in one operator call; q_rope is a strided view into
    the per-head [latent | rope] query rows. The latent parts of the query must stay untouched, the
    key's rope columns of kv_a are rotated in place (rope_out aliases them)."""
    tokens, bs, max_pos = 37, 32, 512
    blocks = -(-tokens // bs) + 1
    cache = kt.PagedCache(1, blocks, bs)
    lib = ffi.load()
    kv_a = kt.randn_bf16((tokens, LATENT + ROPE), seed=31)
    q = kt.randn_bf16((tokens, heads, LATENT + ROPE), seed=32)
    gamma = torch.ones(LATENT, dtype=torch.bfloat16)
    cos, sin = _tables(max_pos)
    rng = np.random.default_rng(33)
    positions = rng.integers(0, max_pos, tokens).astype(np.int32)
    slots = rng.permutation(blocks * bs)[:tokens].astype(np.int32)
    kv_d, q_d, gamma_d, cos_d, sin_d = kv_a.cuda(), q.cuda(), gamma.cuda(), cos.cuda(), sin.cuda()
    positions_d, slots_d = kt.dev_i32(positions), kt.dev_i32(slots)
    row = (LATENT + ROPE) * 2
    ffi.check(lib.mlakvNormRopeAppend(C.byref(cache.view), 0, kv_d.data_ptr(), row, gamma_d.data_ptr(), EPS, cos_d.data_ptr(),
                                      sin_d.data_ptr(), ROPE * 2, positions_d.data_ptr(), slots_d.data_ptr(), tokens,
                                      None, 0, kv_d.data_ptr() + LATENT * 2, row, q_d.data_ptr() + LATENT * 2, heads * row, row,
                                      heads, kt.stream_ptr()))
    torch.cuda.synchronize()
    q_bits, got_q = kt.bits16(q), kt.bits16(q_d)
    assert np.array_equal(got_q[..., :LATENT], q_bits[..., :LATENT])
    want_q = orc.rope_rows(q_bits[..., LATENT:].reshape(tokens * heads, ROPE), kt.bits16(cos), kt.bits16(sin), positions, heads)
    _within_one_ulp(got_q[..., LATENT:].reshape(tokens * heads, ROPE), want_q)
    _, want_k = orc.norm_rope_rows(kt.bits16(kv_a), kt.bits16(gamma), EPS, kt.bits16(cos), kt.bits16(sin), positions)
    got_kv = kt.bits16(kv_d)
    assert np.array_equal(got_kv[:, :LATENT], kt.bits16(kv_a)[:, :LATENT])  # no latent output was asked for
    _within_one_ulp(got_kv[:, LATENT:], want_k)
    rope_plane = np.zeros((blocks * bs, ROPE), dtype=np.uint16)
    rope_plane[slots] = got_kv[:, LATENT:]
    assert np.array_equal(cache.rope_np(0), rope_plane.reshape(-1))
