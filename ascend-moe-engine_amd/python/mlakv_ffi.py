"""ctypes binding of libmoe_kv_hip.so (include/mlakv.h), used by the tests, the smoke entry
and the benchmark. It only declares prototypes and turns non-zero statuses into exceptions;
there is no Python implementation of anything behind it, and loading fails loudly when the
library has not been built.
"""
import ctypes as C
import weakref
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
PACKAGE_DIR = os.path.dirname(_HERE)
LIB_PATH = os.path.join(PACKAGE_DIR, "libmoe_kv_hip.so")

SUCCESS = 0
ERR_PARAM_NULLPTR = 161001
ERR_PARAM_INVALID = 161002
ERR_RUNTIME = 361001
ERR_CONTRACT = 100001
DTYPE_BF16 = 0
DTYPE_FP8_E4M3 = 1
BACKEND_HIP = 0
BACKEND_HOST = 1


class MlakvError(RuntimeError):
    def __init__(self, status, text):
        super().__init__(f"status {status}: {text}")
        self.status = status


class CacheView(C.Structure):
    _fields_ = [
        ("latent", C.c_void_p), ("latent_layer_stride", C.c_int64), ("latent_block_stride", C.c_int64),
        ("latent_row_stride", C.c_int64),
        ("rope", C.c_void_p), ("rope_layer_stride", C.c_int64), ("rope_block_stride", C.c_int64),
        ("rope_row_stride", C.c_int64),
        ("scale", C.c_void_p), ("scale_layer_stride", C.c_int64), ("scale_block_stride", C.c_int64),
        ("num_layers", C.c_int32), ("num_blocks", C.c_int32), ("block_size", C.c_int32), ("latent_dim", C.c_int32),
        ("rope_dim", C.c_int32), ("dtype", C.c_int32),
    ]


class MxQuantOut(C.Structure):
    _fields_ = [("codes", C.c_void_p), ("codes_seq_stride", C.c_int64), ("codes_head_stride", C.c_int64),
                ("scales", C.c_void_p), ("scales_seq_stride", C.c_int64), ("scales_head_stride", C.c_int64)]


class IndexKeyView(C.Structure):
    _fields_ = [("keys", C.c_void_p), ("block_stride", C.c_int64), ("row_stride", C.c_int64), ("scales", C.c_void_p),
                ("scale_block_stride", C.c_int64), ("num_blocks", C.c_int32), ("block_size", C.c_int32), ("dim", C.c_int32),
                ("reserved", C.c_int32)]


class AttnPlan(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("heads", C.c_int32), ("max_seq_len", C.c_int32), ("block_size", C.c_int32),
        ("dtype", C.c_int32), ("chunk_tiles", C.c_int32), ("work_groups", C.c_int32), ("max_units", C.c_int32),
        ("merge_mode", C.c_int32), ("merge_spin_us", C.c_int32), ("reserved", C.c_int32), ("selection_units", C.c_int32),
        ("workspace_bytes", C.c_uint64),
    ]


class AttnPlanOptions(C.Structure):
    _fields_ = [("chunk_tiles", C.c_int32), ("work_groups", C.c_int32), ("merge_mode", C.c_int32), ("merge_spin_us", C.c_int32),
                ("selection", C.c_int32), ("selection_units", C.c_int32), ("reserved", C.c_int32 * 2)]


ATTN_MERGE_AUTO, ATTN_MERGE_IN_LAUNCH, ATTN_MERGE_SECOND_LAUNCH = 0, 1, 2
ATTN_UNITS_AUTO, ATTN_UNITS_SPLIT, ATTN_UNITS_HEAD_BLOCK, ATTN_UNITS_HEAD_BLOCK_HALVES = 0, 1, 2, 3
ATTN_HEAD_BLOCK_TOKENS = 1024


class KvConfig(C.Structure):
    _fields_ = [
        ("num_layers", C.c_int64), ("block_size", C.c_int64), ("max_context_len", C.c_int64), ("max_batch", C.c_int64),
        ("pool_blocks", C.c_int64), ("kv_lora_rank", C.c_int64), ("qk_rope_head_dim", C.c_int64),
        ("dtype", C.c_int32), ("fused_rows", C.c_int32), ("seed", C.c_uint64), ("shuffle", C.c_int32),
        ("reserved", C.c_int32),
    ]


class KvStats(C.Structure):
    _fields_ = [
        ("total_blocks_allocated", C.c_uint64), ("active_context_tokens", C.c_uint64), ("block_size", C.c_uint64),
        ("kv_cache_utilization", C.c_double),
    ]


_i32, _i64, _u64, _vp, _sz = C.c_int32, C.c_int64, C.c_uint64, C.c_void_p, C.c_size_t
_P = C.POINTER

# name -> (restype, argtypes). Every symbol include/mlakv.h declares appears here.
PROTOTYPES = {
    "mlakvGetLastError": (C.c_char_p, []),
    "mlakvDeviceCount": (_i32, []),
    "mlakvPrepare": (_i32, []),
    "mlakvAppend": (_i32, [_P(CacheView), _i32, _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp]),
    "mlakvNormRopeAppend": (_i32, [_P(CacheView), _i32, _vp, _i64, _vp, C.c_double, _vp, _vp, _i64, _vp, _vp, _i32, _vp, _i64,
                                   _vp, _i64, _vp, _i64, _i64, _i32, _vp]),
    "mlakvGather": (_i32, [_P(CacheView), _i32, _i32, _vp, _i32, _vp, _vp, _i32, _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "mlakvGatherTimed": (_i32, [_P(CacheView), _i32, _i32, _vp, _i32, _vp, _vp, _i32, _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp,
                                _vp, _vp]),
    "mlakvCopyBlocks": (_i32, [_P(CacheView), _i32, _i32, _vp, _i32, _vp]),
    "mlakvAttnPlanInit": (_i32, [_i32, _i32, _i32, _i32, _i32, _P(AttnPlan)]),
    "mlakvAttnPlanInitEx": (_i32, [_i32, _i32, _i32, _i32, _i32, _P(AttnPlanOptions), _P(AttnPlan)]),
    "mlakvAttnDecode": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp,
                               C.c_double, _vp, _i64, _i64, _vp, _vp, _u64, _vp]),
    "mlakvAttnDecodeHostLens": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp,
                                       C.c_double, _vp, _i64, _i64, _vp, _vp, _u64, _vp]),
    "mlakvAttnDecodeBounded": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp, _i32,
                                      C.c_double, _vp, _i64, _i64, _vp, _vp, _u64, _vp]),
    "mlakvAttnDecodeNoAlloc": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp,
                                      C.c_double, _vp, _i64, _i64, _vp, _vp]),
    "mlakvAttnDecodeMxQuant": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp,
                                      C.c_double, _vp, _i64, _i64, _P(MxQuantOut), _vp, _vp, _u64, _vp]),
    "mlakvAttnSparsePlanInit": (_i32, [_i32, _i32, _i32, _i32, _i32, _P(AttnPlan)]),
    "mlakvAttnDecodeSparse": (_i32, [_P(AttnPlan), _P(CacheView), _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i32, _vp, _vp, _i64,
                                     C.c_double, _vp, _i64, _i64, _vp, _vp, _u64, _vp]),
    "mlakvIndexerWorkspaceBytes": (_u64, [_i32, _i32]),
    "mlakvIndexKeyAppend": (_i32, [_P(IndexKeyView), _vp, _i64, _vp, _i32, _vp]),
    "mlakvLightningIndexer": (_i32, [_P(IndexKeyView), _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i32, _vp, _i32, _vp, _i32, _i32, _i32,
                                     _vp, _i64, _vp, _u64, _vp]),
    "mlakvDynamicMxQuant": (_i32, [_vp, _i64, _i64, _i32, _vp, _i64, _vp, _i64, _vp]),
    "mlakvArenaCreate": (_i32, [_i32, _P(_vp)]),
    "mlakvArenaDestroy": (None, [_vp]),
    "mlakvArenaReserve": (_i32, [_vp, C.c_char_p, _sz, _sz, _P(_sz)]),
    "mlakvArenaCommit": (_i32, [_vp]),
    "mlakvArenaAddress": (_i32, [_vp, _sz, _P(_vp)]),
    "mlakvArenaBytes": (_i32, [_vp, _sz, _P(_sz)]),
    "mlakvArenaOffset": (_i32, [_vp, _sz, _P(_sz)]),
    "mlakvArenaNoteWorkspace": (_i32, [_vp, _u64]),
    "mlakvArenaCommitWorkspace": (_i32, [_vp]),
    "mlakvArenaAssertWorkspaceFits": (_i32, [_vp, _u64, C.c_char_p]),
    "mlakvArenaSeal": (_i32, [_vp]),
    "mlakvArenaValidateAlignment": (_i32, [_vp]),
    "mlakvArenaWorkspace": (_vp, [_vp]),
    "mlakvArenaWorkspaceBytes": (_u64, [_vp]),
    "mlakvArenaTotalBytes": (_sz, [_vp]),
    "mlakvArenaReservedBytes": (_sz, [_vp]),
    "mlakvArenaReservationCount": (_sz, [_vp]),
    "mlakvArenaSealed": (_i32, [_vp]),
    "mlakvArenaDeviceAllocationCount": (_u64, [_vp]),
    "mlakvArenaDescribeLedger": (_sz, [_vp, C.c_char_p, _sz]),
    "mlakvKvCacheCreate": (_i32, [_vp, _P(KvConfig), _P(_vp)]),
    "mlakvKvCacheDestroy": (None, [_vp]),
    "mlakvKvCacheBind": (_i32, [_vp]),
    "mlakvKvCacheGetView": (_i32, [_vp, _P(CacheView)]),
    "mlakvKvCacheNumBlocks": (_i64, [_vp]),
    "mlakvKvCachePoolBlocks": (_i64, [_vp]),
    "mlakvKvCacheAddSequence": (_i32, [_vp, _i64, _i64]),
    "mlakvKvCacheAppendToken": (_i32, [_vp, _i64, _P(_i32)]),
    "mlakvKvCacheAppendTokenAll": (_i32, [_vp, _P(_i32), _P(_i64)]),
    "mlakvKvCacheFreeSequence": (_i32, [_vp, _i64]),
    "mlakvKvCacheCompact": (_i32, [_vp, _P(_i32), _P(_i64), _vp]),
    "mlakvKvCacheUploadStep": (_i32, [_vp, _vp]),
    "mlakvKvCacheUploadStepAndAppend": (_i32, [_vp, _i32, _i32, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "mlakvKvCacheGetStats": (_i32, [_vp, _P(KvStats)]),
    "mlakvKvStatsFormatJson": (_i64, [_P(KvStats), C.c_char_p, _sz]),
    "mlakvKvCacheHostBlockTable": (_P(_i32), [_vp]),
    "mlakvKvCacheHostSlotMapping": (_P(_i32), [_vp]),
    "mlakvKvCacheHostSeqLens": (_P(_i32), [_vp]),
    "mlakvKvCacheFreeBlocks": (_i64, [_vp]),
    "mlakvKvCacheFreeList": (_i64, [_vp, _P(_i32)]),
    "mlakvKvCacheDeviceBlockTable": (_vp, [_vp]),
    "mlakvKvCacheDeviceSlotMapping": (_vp, [_vp]),
    "mlakvKvCacheDeviceSeqLens": (_vp, [_vp]),
    "mlakvKvCacheDeviceCuSeqLens": (_vp, [_vp]),
    "mlakvNumBlocks": (_i64, [_i64, _i64]),
    "mlakvBackboneDeviceBytes": (_u64, [_i64, _i64, _i64, _i64]),
}

_lib = None


def load():
    """Returns the loaded library with prototypes applied; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    # PyTorch ships its own copy of the HIP runtime. A process must hold exactly one, so when
    # torch is part of the process it has to be loaded first: this library then binds to the
    # runtime that is already there instead of bringing a second one.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is not built: run `make -C {PACKAGE_DIR}` (or __graft_entry__.build()). "
            "There is no fallback implementation.")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    text = load().mlakvGetLastError()
    return text.decode() if text else ""


def check(status):
    if status != SUCCESS:
        raise MlakvError(status, last_error())


# ---- small object wrappers (host-side handles) ---------------------------------------


class Arena:
    def __init__(self, backend=BACKEND_HIP):
        self.lib = load()
        handle = _vp()
        check(self.lib.mlakvArenaCreate(backend, C.byref(handle)))
        self.handle = handle
        self._caches = weakref.WeakSet()  # KvCache objects built on this arena

    def close(self):
        """Destroys the caches built on this arena first: they hold pinned staging buffers that
        are released through the arena's backend, whatever order the garbage collector picks."""
        if self.handle:
            for cache in list(self._caches):
                cache.close()
            self.lib.mlakvArenaDestroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def reserve(self, name, nbytes, align=512):
        out = _sz()
        check(self.lib.mlakvArenaReserve(self.handle, name.encode(), nbytes, align, C.byref(out)))
        return out.value

    def commit(self):
        check(self.lib.mlakvArenaCommit(self.handle))

    def address(self, handle):
        out = _vp()
        check(self.lib.mlakvArenaAddress(self.handle, handle, C.byref(out)))
        return out.value

    def nbytes(self, handle):
        out = _sz()
        check(self.lib.mlakvArenaBytes(self.handle, handle, C.byref(out)))
        return out.value

    def offset(self, handle):
        out = _sz()
        check(self.lib.mlakvArenaOffset(self.handle, handle, C.byref(out)))
        return out.value

    def note_workspace(self, nbytes):
        check(self.lib.mlakvArenaNoteWorkspace(self.handle, nbytes))

    def commit_workspace(self):
        check(self.lib.mlakvArenaCommitWorkspace(self.handle))

    def assert_workspace_fits(self, nbytes, what="plan"):
        check(self.lib.mlakvArenaAssertWorkspaceFits(self.handle, nbytes, what.encode()))

    def seal(self):
        check(self.lib.mlakvArenaSeal(self.handle))

    def validate(self):
        check(self.lib.mlakvArenaValidateAlignment(self.handle))

    @property
    def workspace(self):
        return self.lib.mlakvArenaWorkspace(self.handle)

    @property
    def workspace_bytes(self):
        return self.lib.mlakvArenaWorkspaceBytes(self.handle)

    @property
    def total_bytes(self):
        return self.lib.mlakvArenaTotalBytes(self.handle)

    @property
    def reserved_bytes(self):
        return self.lib.mlakvArenaReservedBytes(self.handle)

    @property
    def count(self):
        return self.lib.mlakvArenaReservationCount(self.handle)

    @property
    def sealed(self):
        return bool(self.lib.mlakvArenaSealed(self.handle))

    @property
    def device_allocations(self):
        return self.lib.mlakvArenaDeviceAllocationCount(self.handle)

    def ledger(self):
        n = self.lib.mlakvArenaDescribeLedger(self.handle, None, 0)
        buf = C.create_string_buffer(n + 1)
        self.lib.mlakvArenaDescribeLedger(self.handle, buf, n + 1)
        return buf.value.decode()


class KvCache:
    def __init__(self, arena, **config):
        self.lib = load()
        self.arena = arena
        cfg = KvConfig(num_layers=43, block_size=128, max_context_len=8192, max_batch=1, pool_blocks=0,
                       kv_lora_rank=512, qk_rope_head_dim=64, dtype=DTYPE_BF16, fused_rows=0, seed=0, shuffle=0)
        for key, value in config.items():
            setattr(cfg, key, value)
        self.config = cfg
        handle = _vp()
        check(self.lib.mlakvKvCacheCreate(arena.handle, C.byref(cfg), C.byref(handle)))
        self.handle = handle
        arena._caches.add(self)

    def close(self):
        if self.handle:
            self.lib.mlakvKvCacheDestroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def bind(self):
        check(self.lib.mlakvKvCacheBind(self.handle))

    def view(self):
        out = CacheView()
        check(self.lib.mlakvKvCacheGetView(self.handle, C.byref(out)))
        return out

    @property
    def num_blocks(self):
        return self.lib.mlakvKvCacheNumBlocks(self.handle)

    @property
    def pool_blocks(self):
        return self.lib.mlakvKvCachePoolBlocks(self.handle)

    def add_sequence(self, seq, context_len):
        check(self.lib.mlakvKvCacheAddSequence(self.handle, seq, context_len))

    def append_token(self, seq):
        out = _i32()
        check(self.lib.mlakvKvCacheAppendToken(self.handle, seq, C.byref(out)))
        return out.value

    def append_token_all(self):
        """One token for every live sequence; returns the number appended."""
        appended = C.c_int64()
        check(self.lib.mlakvKvCacheAppendTokenAll(self.handle, None, C.byref(appended)))
        return appended.value

    def free_sequence(self, seq):
        check(self.lib.mlakvKvCacheFreeSequence(self.handle, seq))

    def compact(self, stream=None):
        moves = (_i32 * (2 * self.pool_blocks))()
        count = _i64()
        check(self.lib.mlakvKvCacheCompact(self.handle, moves, C.byref(count), stream))
        return [(moves[2 * i], moves[2 * i + 1]) for i in range(count.value)]

    def upload_step(self, stream=None):
        check(self.lib.mlakvKvCacheUploadStep(self.handle, stream))

    def upload_step_and_append(self, layer_begin, layer_count, latent_ptr, latent_layer_stride, latent_row_stride, rope_ptr,
                               rope_layer_stride, rope_row_stride, stream=None):
        check(self.lib.mlakvKvCacheUploadStepAndAppend(self.handle, layer_begin, layer_count, latent_ptr, latent_layer_stride,
                                                       latent_row_stride, rope_ptr, rope_layer_stride, rope_row_stride, stream))

    def stats(self):
        out = KvStats()
        check(self.lib.mlakvKvCacheGetStats(self.handle, C.byref(out)))
        return out

    def host_block_table(self):
        import numpy as np
        rows, cols = self.config.max_batch, self.num_blocks
        pointer = self.lib.mlakvKvCacheHostBlockTable(self.handle)
        return np.ctypeslib.as_array(pointer, shape=(rows * cols,)).reshape(rows, cols).copy()

    def host_slot_mapping(self):
        import numpy as np
        pointer = self.lib.mlakvKvCacheHostSlotMapping(self.handle)
        return np.ctypeslib.as_array(pointer, shape=(self.config.max_batch,)).copy()

    def host_seq_lens(self):
        import numpy as np
        pointer = self.lib.mlakvKvCacheHostSeqLens(self.handle)
        return np.ctypeslib.as_array(pointer, shape=(self.config.max_batch,)).copy()

    @property
    def free_blocks(self):
        return self.lib.mlakvKvCacheFreeBlocks(self.handle)

    def free_list(self):
        out = (_i32 * self.pool_blocks)()
        n = self.lib.mlakvKvCacheFreeList(self.handle, out)
        return list(out[:n])

    @property
    def device_block_table(self):
        return self.lib.mlakvKvCacheDeviceBlockTable(self.handle)

    @property
    def device_slot_mapping(self):
        return self.lib.mlakvKvCacheDeviceSlotMapping(self.handle)

    @property
    def device_seq_lens(self):
        return self.lib.mlakvKvCacheDeviceSeqLens(self.handle)

    @property
    def device_cu_seq_lens(self):
        return self.lib.mlakvKvCacheDeviceCuSeqLens(self.handle)
