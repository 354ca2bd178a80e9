"""Shared helpers for the test-suite: seeded bf16 inputs, cache views over torch tensors,
and the calls into the C ABI. Torch is used for device memory and streams only."""
import ctypes as C

import numpy as np
import torch

import mlakv_ffi as ffi
import oracle_ffi as orc

LATENT, ROPE = 512, 64


def randn_bf16(shape, seed, outlier_fraction=0.0, outlier_scale=20.0):
    """N(0,1) rounded to bf16 (torch CPU cast = round to nearest even); returns a CPU bf16 tensor."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=gen, dtype=torch.float32)
    if outlier_fraction > 0:
        mask = torch.rand(shape, generator=gen) < outlier_fraction
        x = torch.where(mask, x * outlier_scale, x)
    return x.to(torch.bfloat16)


def bits16(t):
    """bf16 tensor (any device) -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


class PagedCache:
    """A paged MLA cache held in torch device tensors, with the mlakvCacheView over it."""

    def __init__(self, layers, blocks, block_size, fp8=False, fused=False, device="cuda"):
        self.layers, self.blocks, self.block_size, self.fp8, self.fused = layers, blocks, block_size, fp8, fused
        dt = torch.uint8 if fp8 else torch.bfloat16
        e = 1 if fp8 else 2
        self.element = e
        if fused:
            self.kv = torch.zeros(layers, blocks, block_size, LATENT + ROPE, dtype=dt, device=device)
            self.latent = self.kv[..., :LATENT]
            self.rope = self.kv[..., LATENT:]
            latent_row = rope_row = (LATENT + ROPE) * e
            latent_ptr = self.kv.data_ptr()
            rope_ptr = latent_ptr + LATENT * e
        else:
            self.latent = torch.zeros(layers, blocks, block_size, LATENT, dtype=dt, device=device)
            self.rope = torch.zeros(layers, blocks, block_size, ROPE, dtype=dt, device=device)
            latent_row, rope_row = LATENT * e, ROPE * e
            latent_ptr, rope_ptr = self.latent.data_ptr(), self.rope.data_ptr()
        self.scale = torch.zeros(layers, blocks, block_size, dtype=torch.float32, device=device) if fp8 else None
        self.view = ffi.CacheView(
            latent=latent_ptr, latent_layer_stride=blocks * block_size * latent_row,
            latent_block_stride=block_size * latent_row, latent_row_stride=latent_row,
            rope=rope_ptr, rope_layer_stride=blocks * block_size * rope_row, rope_block_stride=block_size * rope_row,
            rope_row_stride=rope_row,
            scale=self.scale.data_ptr() if fp8 else None, scale_layer_stride=blocks * block_size * 4,
            scale_block_stride=block_size * 4,
            num_layers=layers, num_blocks=blocks, block_size=block_size, latent_dim=LATENT, rope_dim=ROPE,
            dtype=ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16)

    # numpy copies of one layer's planes, contiguous [blocks*bs, dim]
    def latent_np(self, layer):
        t = self.latent[layer].contiguous()
        return u8(t).reshape(-1) if self.fp8 else bits16(t).reshape(-1)

    def rope_np(self, layer):
        t = self.rope[layer].contiguous()
        return u8(t).reshape(-1) if self.fp8 else bits16(t).reshape(-1)

    def scale_np(self, layer):
        return self.scale[layer].detach().cpu().contiguous().numpy().reshape(-1)


def stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def dev_i32(values):
    return torch.as_tensor(np.asarray(values, dtype=np.int32), device="cuda")


def append(cache, latent_src, rope_src, slots, layer_begin=0, layer_count=None):
    """latent_src [L, T, 512] bf16 cuda, rope_src [L, T, 64] bf16 cuda, slots int32 cuda [T]."""
    lib = ffi.load()
    layer_count = cache.layers if layer_count is None else layer_count
    ffi.check(lib.mlakvAppend(C.byref(cache.view), layer_begin, layer_count, latent_src.data_ptr(),
                              latent_src.stride(0) * 2, latent_src.stride(1) * 2, rope_src.data_ptr(),
                              rope_src.stride(0) * 2, rope_src.stride(1) * 2, slots.data_ptr(), slots.numel(),
                              stream_ptr()))


def gather(cache, table, seq_lens, fused_out=False, layer_begin=0, layer_count=None, max_seq_len=None):
    """table int32 cuda [B, W]; seq_lens int32 cuda [B]. Returns (latent [L, total, 512], rope [L, total, 64]) bf16."""
    lib = ffi.load()
    layer_count = cache.layers if layer_count is None else layer_count
    lens = seq_lens.cpu().numpy()
    total = int(lens.sum())
    cu = dev_i32(np.concatenate([[0], np.cumsum(lens)]))
    max_seq_len = int(lens.max()) if max_seq_len is None else max_seq_len
    rows = max(total, 1)
    if fused_out:
        out = torch.zeros(layer_count, rows, LATENT + ROPE, dtype=torch.bfloat16, device="cuda")
        latent_out, rope_out = out[..., :LATENT], out[..., LATENT:]
        latent_ptr, rope_ptr = out.data_ptr(), out.data_ptr() + LATENT * 2
        layer_stride_l = layer_stride_r = rows * (LATENT + ROPE) * 2
        row_l = row_r = (LATENT + ROPE) * 2
    else:
        latent_out = torch.zeros(layer_count, rows, LATENT, dtype=torch.bfloat16, device="cuda")
        rope_out = torch.zeros(layer_count, rows, ROPE, dtype=torch.bfloat16, device="cuda")
        latent_ptr, rope_ptr = latent_out.data_ptr(), rope_out.data_ptr()
        layer_stride_l, layer_stride_r = rows * LATENT * 2, rows * ROPE * 2
        row_l, row_r = LATENT * 2, ROPE * 2
    ffi.check(lib.mlakvGather(C.byref(cache.view), layer_begin, layer_count, table.data_ptr(), table.shape[1],
                              seq_lens.data_ptr(), cu.data_ptr(), table.shape[0], max_seq_len, latent_ptr,
                              layer_stride_l, row_l, rope_ptr, layer_stride_r, row_r, stream_ptr()))
    torch.cuda.synchronize()
    return latent_out[:, :total], rope_out[:, :total]


def make_plan(batch, heads, max_seq_len, block_size, fp8, chunk_tiles=0, work_groups=0, merge_mode=0, merge_spin_us=0,
              selection=False, selection_units=0):
    """The default plan, or one with the planner's choices forced (mlakvAttnPlanInitEx). With
    selection=True, max_seq_len is the length of the selection (mlakvAttnSparsePlanInit)."""
    lib = ffi.load()
    plan = ffi.AttnPlan()
    dtype = ffi.DTYPE_FP8_E4M3 if fp8 else ffi.DTYPE_BF16
    if chunk_tiles or work_groups or merge_mode or merge_spin_us or selection_units:
        options = ffi.AttnPlanOptions(chunk_tiles, work_groups, merge_mode, merge_spin_us, 1 if selection else 0, selection_units)
        ffi.check(lib.mlakvAttnPlanInitEx(batch, heads, max_seq_len, block_size, dtype, C.byref(options), C.byref(plan)))
    elif selection:
        ffi.check(lib.mlakvAttnSparsePlanInit(batch, heads, max_seq_len, block_size, dtype, C.byref(plan)))
    else:
        ffi.check(lib.mlakvAttnPlanInit(batch, heads, max_seq_len, block_size, dtype, C.byref(plan)))
    return plan


def attention(cache, layer, q, table, seq_lens, scale, max_seq_len=None, want_lse=True, quant=False, want_out=True, **plan_options):
    """q [B, H, 576] bf16 cuda (latent | rope per head). Returns (out [B,H,512] bf16, lse [B,H] f32, plan);
    with quant=True through the fused entry point, returning (out or None, lse, plan, codes [B,H,512] u8,
    scales [B,H,16] u8)."""
    lib = ffi.load()
    batch, heads = q.shape[0], q.shape[1]
    lens = seq_lens.cpu().numpy()
    max_seq_len = max(int(lens.max()), 1) if max_seq_len is None else max_seq_len
    plan = make_plan(batch, heads, max_seq_len, cache.block_size, cache.fp8, **plan_options)
    workspace = torch.empty(max(int(plan.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    out = torch.full((batch, heads, LATENT), float("nan"), dtype=torch.bfloat16, device="cuda") if want_out else None
    lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device="cuda") if want_lse else None
    row = (LATENT + ROPE) * 2
    head_args = (C.byref(plan), C.byref(cache.view), layer, q.data_ptr(), heads * row, row,
                 q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), table.shape[1],
                 seq_lens.data_ptr(), float(scale), out.data_ptr() if want_out else None, heads * LATENT * 2, LATENT * 2)
    tail_args = (lse.data_ptr() if want_lse else None, workspace.data_ptr(), int(plan.workspace_bytes), stream_ptr())
    if not quant:
        ffi.check(lib.mlakvAttnDecode(*head_args, *tail_args))
        torch.cuda.synchronize()
        return out, lse, plan
    codes = torch.full((batch, heads, LATENT), 0xAA, dtype=torch.uint8, device="cuda")
    scales = torch.full((batch, heads, LATENT // 32), 0xAA, dtype=torch.uint8, device="cuda")
    target = ffi.MxQuantOut(codes.data_ptr(), heads * LATENT, LATENT, scales.data_ptr(), heads * (LATENT // 32), LATENT // 32)
    ffi.check(lib.mlakvAttnDecodeMxQuant(*head_args, C.byref(target), *tail_args))
    torch.cuda.synchronize()
    return out, lse, plan, codes, scales


def sparse_attention(cache, layer, q, table, seq_lens, selection, scale, want_lse=True, **plan_options):
    """Selected-token attention: `selection` int32 cuda [B, k]. Returns (out, lse, plan)."""
    lib = ffi.load()
    batch, heads = q.shape[0], q.shape[1]
    plan = make_plan(batch, heads, selection.shape[1], cache.block_size, cache.fp8, selection=True, **plan_options)
    workspace = torch.empty(max(int(plan.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    out = torch.full((batch, heads, LATENT), float("nan"), dtype=torch.bfloat16, device="cuda")
    lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device="cuda") if want_lse else None
    row = (LATENT + ROPE) * 2
    ffi.check(lib.mlakvAttnDecodeSparse(C.byref(plan), C.byref(cache.view), layer, q.data_ptr(), heads * row, row,
                                        q.data_ptr() + LATENT * 2, heads * row, row, table.data_ptr(), table.shape[1],
                                        seq_lens.data_ptr(), selection.data_ptr(), selection.stride(0), float(scale),
                                        out.data_ptr(), heads * LATENT * 2, LATENT * 2, lse.data_ptr() if want_lse else None,
                                        workspace.data_ptr(), int(plan.workspace_bytes), stream_ptr()))
    torch.cuda.synchronize()
    return out, lse, plan


def oracle_attention(cache, layer, q, table_np, lens_np, scale, accum_f32=False, sparse_indices=None):
    qb = bits16(q)
    q_lat = np.ascontiguousarray(qb[..., :LATENT])
    q_rope = np.ascontiguousarray(qb[..., LATENT:])
    return orc.mla_decode(q_lat, q_rope, cache.latent_np(layer), cache.rope_np(layer), cache.block_size, table_np,
                          lens_np, scale, scale_plane=cache.scale_np(layer) if cache.fp8 else None, accum_f32=accum_f32,
                          sparse_indices=sparse_indices)


def build_tables(ctxs, block_size, pool_blocks, seed, shuffle=True, max_blocks=None):
    """Block tables from the ORACLE pool (first-fit from a shuffled free list)."""
    max_blocks = max_blocks or max(1, -(-max(max(ctxs), 1) // block_size))
    pool = orc.Pool(pool_blocks, block_size, len(ctxs), max_blocks, seed=seed, shuffle=shuffle)
    for s, n in enumerate(ctxs):
        assert pool.add_sequence(s, n) == orc.OK
    return pool


def slots_for(table_np, ctxs, block_size):
    """Slot of every token of every sequence, in packed sequence order."""
    out = []
    for s, n in enumerate(ctxs):
        pos = np.arange(n)
        out.append(table_np[s, pos // block_size].astype(np.int64) * block_size + pos % block_size)
    return np.concatenate(out).astype(np.int32) if out else np.zeros(0, np.int32)
