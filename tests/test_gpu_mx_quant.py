"""GPU parity, bit-exact: block-32 MX quantisation (E4M3 codes, E8M0 scales) through the C ABI
against the CPU oracle, standalone (mlakvDynamicMxQuant) and as the epilogue of the decode
attention (mlakvAttnDecodeMxQuant), whose codes and scales must equal the standalone operator
applied to the bf16 output of mlakvAttnDecode on the same inputs, in the split-KV case (merge
kernel epilogue), the single-chunk case (attention kernel epilogue) and for an empty sequence."""
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


def _quant(x, x_stride=None, codes_stride=None, scales_stride=None):
    rows, cols = x.shape
    lib = ffi.load()
    codes_stride = codes_stride or cols
    scales_stride = scales_stride or cols // 32
    codes = torch.full((rows, codes_stride), 0xAA, dtype=torch.uint8, device="cuda")
    scales = torch.full((rows, scales_stride), 0xAA, dtype=torch.uint8, device="cuda")
    ffi.check(lib.mlakvDynamicMxQuant(x.data_ptr(), x_stride or x.stride(0) * 2, rows, cols, codes.data_ptr(), codes_stride,
                                      scales.data_ptr(), scales_stride, kt.stream_ptr()))
    torch.cuda.synchronize()
    return codes.cpu().numpy(), scales.cpu().numpy()


def test_standalone_matches_oracle_on_random_outlier_zero_and_nonfinite_blocks():
    rows, cols = 333, 512
    x = kt.randn_bf16((rows, cols), seed=70, outlier_fraction=0.02)
    magnitude = torch.from_numpy(2.0 ** np.random.default_rng(71).integers(-30, 30, (rows, cols // 32)).astype(np.float32))
    x = (x.float() * magnitude.repeat_interleave(32, dim=1)).to(torch.bfloat16)
    x[1, 64:96] = 0
    x[2, 5] = float("inf")
    x[3, 100] = float("nan")
    x[4, 32:64] = 2.0 ** -130      # bf16 subnormals: the scale clamps at the smallest
    x[5, 0:32] = 3.0e38            # close to the largest bf16
    x[6, 0:32] = -448.0
    x[7, 0:32] = 480.0
    codes, scales = _quant(x.cuda())
    want_codes, want_scales = orc.mx_quant_rows(kt.bits16(x))
    assert np.array_equal(scales, want_scales)
    assert np.array_equal(codes, want_codes)


def test_standalone_strided_rows_ragged_row_count_and_argument_checks():
    rows, cols = 37, 96             # 37 * 12 items: the last workgroup is partly idle
    wide = kt.randn_bf16((rows, 160), seed=72).cuda()
    codes, scales = _quant(wide[:, :cols], x_stride=160 * 2, codes_stride=104, scales_stride=5)
    want_codes, want_scales = orc.mx_quant_rows(kt.bits16(wide[:, :cols].contiguous()))
    assert np.array_equal(codes[:, :cols], want_codes) and (codes[:, cols:] == 0xAA).all()
    assert np.array_equal(scales[:, :3], want_scales) and (scales[:, 3:] == 0xAA).all()
    lib = ffi.load()
    x = wide
    y = torch.zeros(rows, 160, dtype=torch.uint8, device="cuda")
    s = torch.zeros(rows, 8, dtype=torch.uint8, device="cuda")

    def call(xp=x.data_ptr(), xs=320, r=rows, c=cols, yp=y.data_ptr(), ys=160, sp=s.data_ptr(), ss=8):
        return lib.mlakvDynamicMxQuant(xp, xs, r, c, yp, ys, sp, ss, kt.stream_ptr())

    assert call() == 0
    assert call(r=0) == 0
    assert call(xp=None) == ffi.ERR_PARAM_NULLPTR
    assert call(sp=None) == ffi.ERR_PARAM_NULLPTR
    assert call(c=40) == ffi.ERR_PARAM_INVALID       # not whole blocks
    assert call(xs=64) == ffi.ERR_PARAM_INVALID      # row shorter than its columns
    assert call(xp=x.data_ptr() + 2) == ffi.ERR_PARAM_INVALID
    assert call(ys=64) == ffi.ERR_PARAM_INVALID
    assert call(ss=2) == ffi.ERR_PARAM_INVALID
    assert call(r=-1) == ffi.ERR_PARAM_INVALID
    torch.cuda.synchronize()


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("options", [{}, {"chunk_tiles": 2}, {"chunk_tiles": 100}, {"chunk_tiles": 1, "merge_mode": 1}])
def test_attention_epilogue_equals_quantising_the_bf16_output(fp8, options):
    bs, heads = 64, 64
    ctxs = [1, 0, 65, 200, 333, 32]   # one empty sequence: zero codes under scale byte 0
    blocks = sum(-(-c // bs) for c in ctxs) + 3
    pool = kt.build_tables(ctxs, bs, blocks, seed=73)
    table = pool.table()
    cache = kt.PagedCache(1, blocks, bs, fp8=fp8)
    total = sum(ctxs)
    latent = kt.randn_bf16((1, total, LATENT), seed=74, outlier_fraction=0.01).cuda()
    rope = kt.randn_bf16((1, total, ROPE), seed=75).cuda()
    kt.append(cache, latent, rope, kt.dev_i32(kt.slots_for(table, ctxs, bs)))
    q = kt.randn_bf16((len(ctxs), heads, LATENT + ROPE), seed=76).cuda()
    # planner's choice; sequences split over units (the merge quantises); whole sequences per unit
    # (the kernel's own epilogue quantises); the merge inside the launch
    table_d, lens_d = kt.dev_i32(table), kt.dev_i32(ctxs)
    # (with the planner's choice, contexts this short go to the units of 16 heads in both entry points;
    # the quantising one then runs the standalone quantiser behind them)
    out, lse, plan = kt.attention(cache, 0, q, table_d, lens_d, SCALE, **options)
    out_q, lse_q, _, codes, scales = kt.attention(cache, 0, q, table_d, lens_d, SCALE, quant=True, **options)
    assert torch.equal(out_q, out) and torch.equal(lse_q, lse)       # the bf16 output is unchanged by the epilogue
    want_codes, want_scales = orc.mx_quant_rows(kt.bits16(out).reshape(-1, LATENT))
    assert np.array_equal(scales.cpu().numpy().reshape(-1, LATENT // 32), want_scales)
    assert np.array_equal(codes.cpu().numpy().reshape(-1, LATENT), want_codes)
    assert not codes[1].any() and not scales[1].any()
    # the standalone operator on the device output agrees as well
    alone_codes, alone_scales = _quant(out.reshape(-1, LATENT))
    assert np.array_equal(alone_codes, want_codes) and np.array_equal(alone_scales, want_scales)
    # without the bf16 output
    none_out, _, _, codes2, scales2 = kt.attention(cache, 0, q, table_d, lens_d, SCALE, quant=True, want_out=False, want_lse=False,
                                                   **options)
    assert none_out is None and torch.equal(codes2, codes) and torch.equal(scales2, scales)


def test_fused_entry_argument_checks():
    bs, heads = 64, 16
    cache = kt.PagedCache(1, 4, bs)
    lib = ffi.load()
    plan = ffi.AttnPlan()
    ffi.check(lib.mlakvAttnPlanInit(1, heads, 64, bs, ffi.DTYPE_BF16, C.byref(plan)))
    q = torch.zeros(1, heads, LATENT + ROPE, dtype=torch.bfloat16, device="cuda")
    table, lens = kt.dev_i32(np.zeros((1, 1), np.int32)), kt.dev_i32([0])
    codes = torch.zeros(1, heads, LATENT, dtype=torch.uint8, device="cuda")
    scales = torch.zeros(1, heads, 16, dtype=torch.uint8, device="cuda")
    workspace = torch.zeros(max(int(plan.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    row = (LATENT + ROPE) * 2

    def call(target):
        return lib.mlakvAttnDecodeMxQuant(C.byref(plan), C.byref(cache.view), 0, q.data_ptr(), heads * row, row,
                                          q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), 1, lens.data_ptr(), SCALE,
                                          None, 0, 0, target, None, workspace.data_ptr(), int(plan.workspace_bytes), kt.stream_ptr())

    good = ffi.MxQuantOut(codes.data_ptr(), heads * LATENT, LATENT, scales.data_ptr(), heads * 16, 16)
    assert call(C.byref(good)) == 0
    assert call(None) == ffi.ERR_PARAM_NULLPTR
    assert call(C.byref(ffi.MxQuantOut(None, heads * LATENT, LATENT, scales.data_ptr(), heads * 16, 16))) == ffi.ERR_PARAM_NULLPTR
    assert call(C.byref(ffi.MxQuantOut(codes.data_ptr() + 4, heads * LATENT, LATENT, scales.data_ptr(), heads * 16, 16))) == ffi.ERR_PARAM_INVALID
    assert call(C.byref(ffi.MxQuantOut(codes.data_ptr(), heads * LATENT, 256, scales.data_ptr(), heads * 16, 16))) == ffi.ERR_PARAM_INVALID
    assert call(C.byref(ffi.MxQuantOut(codes.data_ptr(), heads * LATENT, LATENT, scales.data_ptr(), heads * 16, 8))) == ffi.ERR_PARAM_INVALID
    torch.cuda.synchronize()


def test_two_phase_operator_matches_oracle_and_supports_address_swaps():
    """aclnnDynamicMxQuant through the plan / launch boundary, as the reference drives stage
    `attn_quant`: planned once on descriptors, made repeatable, launched with the tensors' addresses
    and again after aclSetTensorAddr moved the input."""
    import acl_ffi as acl
    lib = acl.load()
    keep = acl.Keep()
    rows, cols = 5, 64 * 512
    x = kt.randn_bf16((rows, cols), seed=77, outlier_fraction=0.01).cuda()
    x2 = kt.randn_bf16((rows, cols), seed=78).cuda()
    y = torch.zeros(rows, cols, dtype=torch.uint8, device="cuda")
    scales = torch.zeros(rows, cols // 32, dtype=torch.uint8, device="cuda")
    tx = keep.tensor([rows, cols], acl.ACL_BF16, x.data_ptr())
    ty = keep.tensor([rows, cols], acl.ACL_FLOAT8_E4M3FN, y.data_ptr())
    ts = keep.tensor([rows, cols // 32], 37, scales.data_ptr())
    workspace, executor = C.c_uint64(1), C.c_void_p()
    assert lib.aclnnDynamicMxQuantGetWorkspaceSize(tx, -1, b"rint", 36, 32, 0, ty, ts, C.byref(workspace), C.byref(executor)) == 0
    assert workspace.value == 0
    assert lib.aclSetAclOpExecutorRepeatable(executor) == 0
    assert lib.aclnnDynamicMxQuant(None, 0, executor, kt.stream_ptr()) == 0
    torch.cuda.synchronize()
    want_codes, want_scales = orc.mx_quant_rows(kt.bits16(x))
    assert np.array_equal(y.cpu().numpy(), want_codes) and np.array_equal(scales.cpu().numpy(), want_scales)
    assert lib.aclSetTensorAddr(executor, 0, tx, x2.data_ptr()) == 0
    assert lib.aclnnDynamicMxQuant(None, 0, executor, kt.stream_ptr()) == 0
    torch.cuda.synchronize()
    want_codes, want_scales = orc.mx_quant_rows(kt.bits16(x2))
    assert np.array_equal(y.cpu().numpy(), want_codes) and np.array_equal(scales.cpu().numpy(), want_scales)
    assert lib.aclDestroyAclOpExecutor(executor) == 0
