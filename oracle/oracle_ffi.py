"""ctypes loader for the CPU oracle (oracle/libkv_oracle.so). TEST INFRASTRUCTURE ONLY.

Imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py -- as the
checker, never as the thing measured or shipped. The product library never sees it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkv_oracle.so")

OK, REFUSED = 0, 1
DTYPE_BF16, DTYPE_FP8_E4M3 = 0, 1

_i32, _i64, _u64, _sz, _vp = C.c_int32, C.c_int64, C.c_uint64, C.c_size_t, C.c_void_p
_P = C.POINTER


class KvReservationBytes(C.Structure):
    _fields_ = [("block_table", _u64), ("slot_mapping", _u64), ("latent_cache", _u64), ("rope_cache", _u64)]


class KvStats(C.Structure):
    _fields_ = [("total_blocks_allocated", _u64), ("active_context_tokens", _u64), ("block_size", _u64),
                ("kv_cache_utilization", C.c_double)]


class CacheView(C.Structure):
    _fields_ = [("latent", _vp), ("latent_block_stride", _i64), ("latent_row_stride", _i64),
                ("rope", _vp), ("rope_block_stride", _i64), ("rope_row_stride", _i64),
                ("scale", _vp), ("scale_block_stride", _i64), ("block_size", _i64),
                ("latent_dim", _i64), ("rope_dim", _i64), ("dtype", _i32)]


_PROTOTYPES = {
    "kvo_align_up": (_sz, [_sz, _sz]),
    "kvo_divide_up": (_i64, [_i64, _i64]),
    "kvo_num_blocks": (_i64, [_i64, _i64]),
    "kvo_backbone_device_bytes": (_u64, [_i64, _i64, _i64, _i64]),
    "kvo_kv_reservation_bytes": (None, [_i64, _i64, _i64, _i64, _i64, _i64, _P(KvReservationBytes)]),
    "kvo_kv_stats": (None, [_i64, _i64, _i64, _i64, _P(KvStats)]),
    "kvo_arena_new": (_vp, []),
    "kvo_arena_delete": (None, [_vp]),
    "kvo_arena_reserve": (C.c_int, [_vp, C.c_char_p, _sz, _sz, _P(_sz)]),
    "kvo_arena_commit": (C.c_int, [_vp, C.c_size_t]),
    "kvo_arena_address": (C.c_int, [_vp, _sz, _P(C.c_size_t)]),
    "kvo_arena_bytes": (C.c_int, [_vp, _sz, _P(_sz)]),
    "kvo_arena_offset": (C.c_int, [_vp, _sz, _P(_sz)]),
    "kvo_arena_note_workspace": (C.c_int, [_vp, _u64]),
    "kvo_arena_commit_workspace": (C.c_int, [_vp]),
    "kvo_arena_workspace_fits": (C.c_int, [_vp, _u64]),
    "kvo_arena_workspace_bytes": (_u64, [_vp]),
    "kvo_arena_seal": (C.c_int, [_vp]),
    "kvo_arena_sealed": (C.c_int, [_vp]),
    "kvo_arena_validate": (C.c_int, [_vp]),
    "kvo_arena_total_bytes": (_sz, [_vp]),
    "kvo_arena_reserved_bytes": (_sz, [_vp]),
    "kvo_arena_count": (_sz, [_vp]),
    "kvo_arena_allocations": (C.c_int, [_vp]),
    "kvo_slot": (_i64, [_vp, _i64, _i64]),
    "kvo_append_rows": (None, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64]),
    "kvo_gather_rows": (None, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64]),
    "kvo_copy_blocks": (None, [_vp, _i64, _i64, _vp, _i64]),
    "kvo_bf16_from_f32": (C.c_uint16, [C.c_float]),
    "kvo_bf16_to_f32": (C.c_float, [C.c_uint16]),
    "kvo_e4m3_from_f32": (C.c_uint8, [C.c_float]),
    "kvo_e4m3_to_f32": (C.c_float, [C.c_uint8]),
    "kvo_fp8_row_scale": (C.c_float, [_vp, _i64, _vp, _i64]),
    "kvo_append_rows_fp8": (None, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64,
                                   _vp, _i64]),
    "kvo_gather_rows_fp8": (None, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64,
                                   _vp, _i64, _i64, _i64]),
    "kvo_norm_rope_rows": (None, [_vp, _i64, _vp, C.c_double, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64]),
    "kvo_rope_rows": (None, [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _vp, _i64]),
    "kvo_mx_quant_rows": (None, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64]),
    "kvo_mla_decode": (None, [_vp, _i64, _i64, _vp, _i64, _i64, _P(CacheView), _vp, _i64, _vp, _i64, _i64, C.c_double,
                              _vp, _vp, C.c_int]),
    "kvo_mla_decode_sparse": (None, [_vp, _i64, _i64, _vp, _i64, _i64, _P(CacheView), _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64,
                                     C.c_double, _vp, _vp]),
    "kvo_indexer_scores": (None, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _vp]),
    "kvo_indexer_topk": (None, [_vp, _i64, _i64, _vp]),
    "kvo_splitmix64": (_u64, [_P(_u64)]),
    "kvo_pool_new": (_vp, [_i64, _i64, _i64, _i64, _u64, C.c_int]),
    "kvo_pool_delete": (None, [_vp]),
    "kvo_pool_add_sequence": (C.c_int, [_vp, _i64, _i64]),
    "kvo_pool_append_token": (C.c_int, [_vp, _i64, _P(_i32)]),
    "kvo_pool_free_sequence": (C.c_int, [_vp, _i64]),
    "kvo_pool_compact": (C.c_int, [_vp, _P(_i32), _P(_i64)]),
    "kvo_pool_table": (_P(_i32), [_vp]),
    "kvo_pool_seq_len": (_i64, [_vp, _i64]),
    "kvo_pool_free_blocks": (_i64, [_vp]),
    "kvo_pool_live_blocks": (_i64, [_vp]),
    "kvo_pool_free_list": (_i64, [_vp, _P(_i32)]),
}

_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "oracle"], check=True, capture_output=True)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def _ptr(array):
    return array.ctypes.data_as(_vp) if array is not None else None


# ---- numpy-level helpers ------------------------------------------------------------------


def bf16_from_f32(values):
    """float32 array -> uint16 bf16 bit patterns (round to nearest even), via the oracle."""
    lib = load()
    flat = np.ascontiguousarray(values, dtype=np.float32).ravel()
    out = np.empty(flat.shape, dtype=np.uint16)
    for i, v in enumerate(flat):
        out[i] = lib.kvo_bf16_from_f32(float(v))
    return out.reshape(np.shape(values))


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


class Pool:
    def __init__(self, num_blocks, block_size, max_seqs, max_blocks_per_seq, seed=0, shuffle=False):
        self.lib = load()
        self.shape = (max_seqs, max_blocks_per_seq)
        self.num_blocks = num_blocks
        self.handle = self.lib.kvo_pool_new(num_blocks, block_size, max_seqs, max_blocks_per_seq, seed, int(shuffle))
        assert self.handle

    def __del__(self):
        if getattr(self, "handle", None):
            self.lib.kvo_pool_delete(self.handle)
            self.handle = None

    def add_sequence(self, seq, context_len):
        return self.lib.kvo_pool_add_sequence(self.handle, seq, context_len)

    def append_token(self, seq):
        slot = _i32()
        status = self.lib.kvo_pool_append_token(self.handle, seq, C.byref(slot))
        return status, slot.value

    def free_sequence(self, seq):
        return self.lib.kvo_pool_free_sequence(self.handle, seq)

    def compact(self):
        moves = (_i32 * (2 * self.num_blocks))()
        count = _i64()
        self.lib.kvo_pool_compact(self.handle, moves, C.byref(count))
        return [(moves[2 * i], moves[2 * i + 1]) for i in range(count.value)]

    def table(self):
        pointer = self.lib.kvo_pool_table(self.handle)
        return np.ctypeslib.as_array(pointer, shape=(self.shape[0] * self.shape[1],)).reshape(self.shape).copy()

    def seq_len(self, seq):
        return self.lib.kvo_pool_seq_len(self.handle, seq)

    @property
    def free_blocks(self):
        return self.lib.kvo_pool_free_blocks(self.handle)

    @property
    def live_blocks(self):
        return self.lib.kvo_pool_live_blocks(self.handle)

    def free_list(self):
        out = (_i32 * self.num_blocks)()
        n = self.lib.kvo_pool_free_list(self.handle, out)
        return list(out[:n])


def append_rows(plane, block_stride, row_stride, block_size, src, src_row_stride, row_bytes, slots):
    """plane, src: uint8 numpy arrays (plane modified in place)."""
    slots = np.ascontiguousarray(slots, dtype=np.int32)
    load().kvo_append_rows(_ptr(plane), block_stride, row_stride, block_size, _ptr(src), src_row_stride, row_bytes,
                           _ptr(slots), len(slots))


def gather_rows(plane, block_stride, row_stride, block_size, table, seq_lens, row_bytes, dst_row_stride=None):
    table = np.ascontiguousarray(table, dtype=np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    total = int(seq_lens.sum())
    dst_row_stride = dst_row_stride or row_bytes
    dst = np.zeros(max(total, 1) * dst_row_stride, dtype=np.uint8)
    load().kvo_gather_rows(_ptr(plane), block_stride, row_stride, block_size, _ptr(table), table.shape[1],
                           _ptr(seq_lens), len(seq_lens), _ptr(dst), dst_row_stride, row_bytes)
    return dst[: total * dst_row_stride]


def copy_blocks(plane, block_stride, block_bytes, moves):
    moves = np.ascontiguousarray(np.asarray(moves, dtype=np.int32).reshape(-1))
    load().kvo_copy_blocks(_ptr(plane), block_stride, block_bytes, _ptr(moves), len(moves) // 2)


def append_rows_fp8(latent_plane, rope_plane, scale_plane, block_size, latent_src, rope_src, slots, latent_dim=512,
                    rope_dim=64, latent_row_stride=None, rope_row_stride=None):
    """Planes: uint8 [blocks*bs*dim] / float32 [blocks*bs]; sources: uint16 [T, dim] bf16 bits."""
    slots = np.ascontiguousarray(slots, dtype=np.int32)
    latent_row_stride = latent_row_stride or latent_dim
    rope_row_stride = rope_row_stride or rope_dim
    load().kvo_append_rows_fp8(_ptr(latent_plane), latent_row_stride * block_size, latent_row_stride, _ptr(rope_plane),
                               rope_row_stride * block_size, rope_row_stride, _ptr(scale_plane), block_size, block_size,
                               _ptr(latent_src), latent_src.shape[1], _ptr(rope_src), rope_src.shape[1], latent_dim,
                               rope_dim, _ptr(slots), len(slots))


def norm_rope_rows(kv_a, gamma, epsilon, rope_cos, rope_sin, positions, latent_dim=512, rope_dim=64):
    """kv_a uint16 [T, latent+rope] bf16 bits; gamma uint16 [latent]; rope_cos/sin uint16 [P, rope];
    positions int32 [T]. Returns (latent uint16 [T, latent], rope uint16 [T, rope])."""
    kv_a = np.ascontiguousarray(kv_a, dtype=np.uint16)
    gamma = np.ascontiguousarray(gamma, dtype=np.uint16)
    rope_cos = np.ascontiguousarray(rope_cos, dtype=np.uint16)
    rope_sin = np.ascontiguousarray(rope_sin, dtype=np.uint16)
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    n = kv_a.shape[0]
    latent = np.zeros((n, latent_dim), dtype=np.uint16)
    rope = np.zeros((n, rope_dim), dtype=np.uint16)
    load().kvo_norm_rope_rows(_ptr(kv_a), kv_a.shape[1], _ptr(gamma), float(epsilon), _ptr(rope_cos), _ptr(rope_sin), rope_cos.shape[1],
                              _ptr(positions), n, latent_dim, rope_dim, _ptr(latent), latent_dim, _ptr(rope), rope_dim)
    return latent, rope


def rope_rows(rows, rope_cos, rope_sin, positions, rows_per_position=1):
    """rows uint16 [N, rope] bf16 bits (N = len(positions) * rows_per_position). Returns the rotated rows."""
    rows = np.ascontiguousarray(rows, dtype=np.uint16)
    rope_cos = np.ascontiguousarray(rope_cos, dtype=np.uint16)
    rope_sin = np.ascontiguousarray(rope_sin, dtype=np.uint16)
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    assert rows.shape[0] == len(positions) * rows_per_position
    out = np.zeros_like(rows)
    load().kvo_rope_rows(_ptr(rows), rows.shape[1], _ptr(rope_cos), _ptr(rope_sin), rope_cos.shape[1], _ptr(positions),
                         rows_per_position, rows.shape[0], rows.shape[1], _ptr(out), rows.shape[1])
    return out


def mx_quant_rows(x):
    """x uint16 [rows, cols] bf16 bits. Returns (codes uint8 [rows, cols], scales uint8 [rows, ceil(cols/32)])."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    rows, cols = x.shape
    codes = np.zeros((rows, cols), dtype=np.uint8)
    scales = np.zeros((rows, -(-cols // 32)), dtype=np.uint8)
    load().kvo_mx_quant_rows(_ptr(x), cols, rows, cols, _ptr(codes), cols, _ptr(scales), scales.shape[1])
    return codes, scales


def indexer_scores(query, weights, query_scale, key_plane, key_scale_plane, block_size, row_table, seq_len):
    """One sequence: query uint8 [H, D] (E4M3 codes), weights uint16 [H] (bf16 bits), query_scale float32 [H],
    key_plane uint8 [blocks*bs, D], key_scale_plane float32 [blocks*bs], row_table int32 [max_blocks].
    Returns the 16-bit order-preserving score keys, uint16 [seq_len]."""
    query = np.ascontiguousarray(query, dtype=np.uint8)
    weights = np.ascontiguousarray(weights, dtype=np.uint16)
    query_scale = np.ascontiguousarray(query_scale, dtype=np.float32)
    key_plane = np.ascontiguousarray(key_plane, dtype=np.uint8)
    key_scale_plane = np.ascontiguousarray(key_scale_plane, dtype=np.float32)
    row_table = np.ascontiguousarray(row_table, dtype=np.int32)
    heads, dim = query.shape
    keys = np.zeros(max(seq_len, 1), dtype=np.uint16)
    load().kvo_indexer_scores(_ptr(query), _ptr(weights), _ptr(query_scale), heads, dim, _ptr(key_plane), block_size * dim, dim,
                              _ptr(key_scale_plane), block_size, block_size, _ptr(row_table), seq_len, _ptr(keys))
    return keys[:seq_len]


def indexer_topk(keys, sparse_count):
    keys = np.ascontiguousarray(keys, dtype=np.uint16)
    out = np.zeros(sparse_count, dtype=np.int32)
    load().kvo_indexer_topk(_ptr(keys), len(keys), sparse_count, _ptr(out))
    return out


def gather_rows_fp8(latent_plane, rope_plane, scale_plane, block_size, table, seq_lens, latent_dim=512, rope_dim=64):
    table = np.ascontiguousarray(table, dtype=np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    total = int(seq_lens.sum())
    latent = np.zeros((max(total, 1), latent_dim), dtype=np.uint16)
    rope = np.zeros((max(total, 1), rope_dim), dtype=np.uint16)
    load().kvo_gather_rows_fp8(_ptr(latent_plane), latent_dim * block_size, latent_dim, _ptr(rope_plane),
                               rope_dim * block_size, rope_dim, _ptr(scale_plane), block_size, block_size, _ptr(table),
                               table.shape[1], _ptr(seq_lens), len(seq_lens), _ptr(latent), latent_dim, _ptr(rope),
                               rope_dim, latent_dim, rope_dim)
    return latent[:total], rope[:total]


def mla_decode(q_latent, q_rope, latent_plane, rope_plane, block_size, table, seq_lens, scale, scale_plane=None,
               accum_f32=False, latent_row_stride=None, rope_row_stride=None, sparse_indices=None):
    """q_latent [B,H,512], q_rope [B,H,64]: uint16 bf16 bits, contiguous. Planes for ONE layer:
    bf16 -> uint16 arrays, fp8 -> uint8 arrays with scale_plane float32 [blocks*bs].
    Returns (out float32 [B,H,512], lse float32 [B,H])."""
    lib = load()
    fp8 = scale_plane is not None
    element = 1 if fp8 else 2
    latent_dim, rope_dim = q_latent.shape[2], q_rope.shape[2]
    latent_row_stride = latent_row_stride or latent_dim * element
    rope_row_stride = rope_row_stride or rope_dim * element
    view = CacheView(latent=_ptr(latent_plane), latent_block_stride=latent_row_stride * block_size,
                     latent_row_stride=latent_row_stride, rope=_ptr(rope_plane),
                     rope_block_stride=rope_row_stride * block_size, rope_row_stride=rope_row_stride,
                     scale=_ptr(scale_plane) if fp8 else None, scale_block_stride=block_size, block_size=block_size,
                     latent_dim=latent_dim, rope_dim=rope_dim, dtype=DTYPE_FP8_E4M3 if fp8 else DTYPE_BF16)
    table = np.ascontiguousarray(table, dtype=np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    q_latent = np.ascontiguousarray(q_latent, dtype=np.uint16)
    q_rope = np.ascontiguousarray(q_rope, dtype=np.uint16)
    batch, heads = q_latent.shape[0], q_latent.shape[1]
    out = np.zeros((batch, heads, latent_dim), dtype=np.float32)
    lse = np.zeros((batch, heads), dtype=np.float32)
    if sparse_indices is not None:
        # int32 [B, k]: the positions each sequence attends to, valid entries first, -1 after them
        sparse_indices = np.ascontiguousarray(sparse_indices, dtype=np.int32)
        assert sparse_indices.shape[0] == batch and not accum_f32
        lib.kvo_mla_decode_sparse(_ptr(q_latent), heads * latent_dim, latent_dim, _ptr(q_rope), heads * rope_dim, rope_dim,
                                  C.byref(view), _ptr(table), table.shape[1], _ptr(seq_lens), _ptr(sparse_indices),
                                  sparse_indices.shape[1], sparse_indices.shape[1], batch, heads, float(scale), _ptr(out),
                                  _ptr(lse))
        return out, lse
    lib.kvo_mla_decode(_ptr(q_latent), heads * latent_dim, latent_dim, _ptr(q_rope), heads * rope_dim, rope_dim,
                       C.byref(view), _ptr(table), table.shape[1], _ptr(seq_lens), batch, heads, float(scale), _ptr(out),
                       _ptr(lse), int(accum_f32))
    return out, lse
