"""ctypes prototypes for the aclnn-compatible surface (include/aclnn_hip.h), for the tests."""
import ctypes as C

import mlakv_ffi as ffi

ACL_FLOAT32, ACL_INT32, ACL_INT64, ACL_BF16, ACL_FLOAT8_E4M3FN = 0, 3, 9, 27, 36
ACL_FORMAT_ND = 2
_vp, _i64, _u64, _i32 = C.c_void_p, C.c_int64, C.c_uint64, C.c_int32
_P = C.POINTER

FIA_ARGTYPES = ([_vp] * 31 + [_i64, C.c_double, _i64, _i64, C.c_char_p, _i64, _i64, _i64, _i64, _i64, C.c_bool, _i64, _i64,
                              _i64, _i64, _vp, _vp, _P(_u64), _P(_vp)])

PROTOTYPES = {
    "aclInit": (_i32, [C.c_char_p]), "aclFinalize": (_i32, []), "aclnnInit": (_i32, [C.c_char_p]), "aclnnFinalize": (_i32, []),
    "aclGetRecentErrMsg": (C.c_char_p, []),
    "aclrtSetDevice": (_i32, [_i32]), "aclrtResetDevice": (_i32, [_i32]), "aclrtCreateContext": (_i32, [_P(_vp), _i32]),
    "aclrtDestroyContext": (_i32, [_vp]), "aclrtSetCurrentContext": (_i32, [_vp]), "aclrtGetDeviceCount": (_i32, [_P(C.c_uint32)]),
    "aclrtGetSocName": (C.c_char_p, []),
    "aclrtMalloc": (_i32, [_P(_vp), C.c_size_t, _i32]), "aclrtFree": (_i32, [_vp]),
    "aclrtMallocHost": (_i32, [_P(_vp), C.c_size_t]), "aclrtFreeHost": (_i32, [_vp]),
    "aclrtMemcpy": (_i32, [_vp, C.c_size_t, _vp, C.c_size_t, _i32]),
    "aclrtMemcpyAsync": (_i32, [_vp, C.c_size_t, _vp, C.c_size_t, _i32, _vp]),
    "aclrtMemset": (_i32, [_vp, C.c_size_t, _i32, C.c_size_t]),
    "aclrtCreateStream": (_i32, [_P(_vp)]), "aclrtDestroyStream": (_i32, [_vp]), "aclrtDestroyStreamForce": (_i32, [_vp]),
    "aclrtCreateEventExWithFlag": (_i32, [_P(_vp), C.c_uint32]), "aclrtDestroyEvent": (_i32, [_vp]),
    "aclrtRecordEvent": (_i32, [_vp, _vp]), "aclrtStreamWaitEvent": (_i32, [_vp, _vp]), "aclrtSynchronizeStream": (_i32, [_vp]),
    "aclrtSynchronizeStreamWithTimeout": (_i32, [_vp, _i32]), "aclrtSynchronizeEvent": (_i32, [_vp]),
    "aclrtGetMemInfo": (_i32, [_i32, _P(C.c_size_t), _P(C.c_size_t)]),
    "aclmdlRICaptureBegin": (_i32, [_vp, _i32]), "aclmdlRICaptureEnd": (_i32, [_vp, _P(_vp)]),
    "aclmdlRIExecuteAsync": (_i32, [_vp, _vp]), "aclmdlRIDestroy": (_i32, [_vp]),
    "aclCreateTensor": (_vp, [_P(_i64), _u64, _i32, _P(_i64), _i64, _i32, _P(_i64), _u64, _vp]),
    "aclDestroyTensor": (_i32, [_vp]),
    "aclGetViewShape": (_i32, [_vp, _P(_P(_i64)), _P(_u64)]), "aclGetStorageShape": (_i32, [_vp, _P(_P(_i64)), _P(_u64)]),
    "aclGetViewStrides": (_i32, [_vp, _P(_P(_i64)), _P(_u64)]), "aclGetDataType": (_i32, [_vp, _P(_i32)]),
    "aclGetFormat": (_i32, [_vp, _P(_i32)]), "aclGetRawTensorAddr": (_i32, [_vp, _P(_vp)]), "aclGetViewOffset": (_i32, [_vp, _P(_i64)]),
    "aclCreateTensorList": (_vp, [_P(_vp), _u64]), "aclDestroyTensorList": (_i32, [_vp]),
    "aclCreateIntArray": (_vp, [_P(_i64), _u64]), "aclDestroyIntArray": (_i32, [_vp]),
    "aclCreateScalar": (_vp, [_vp, _i32]), "aclDestroyScalar": (_i32, [_vp]),
    "aclSetTensorAddr": (_i32, [_vp, _u64, _vp, _vp]), "aclSetDynamicTensorAddr": (_i32, [_vp, _u64, _u64, _vp, _vp]),
    "aclSetAclOpExecutorRepeatable": (_i32, [_vp]), "aclDestroyAclOpExecutor": (_i32, [_vp]),
    "aclnnScatterPaKvCacheGetWorkspaceSize": (_i32, [_vp] * 8 + [C.c_char_p, C.c_char_p, _vp, _vp, _P(_u64), _P(_vp)]),
    "aclnnScatterPaKvCache": (_i32, [_vp, _u64, _vp, _vp]),
    "aclnnFusedInferAttentionScoreV5GetWorkspaceSize": (_i32, FIA_ARGTYPES),
    "aclnnFusedInferAttentionScoreV5": (_i32, [_vp, _u64, _vp, _vp]),
    "aclnnGatherPaKvCacheGetWorkspaceSize": (_i32, [_vp] * 7 + [_i64, _P(_u64), _P(_vp)]),
    "aclnnGatherPaKvCache": (_i32, [_vp, _u64, _vp, _vp]),
    "aclnnMlaKvBindSeqLens": (_i32, [_vp, _vp]), "aclnnMlaKvSetSeqLenBound": (_i32, [_vp, _i64]),
    "aclnnMlaKvSetSeqLens": (_i32, [_vp, _vp, _u64]),
    "aclnnDynamicMxQuantGetWorkspaceSize": (_i32, [_vp, _i64, C.c_char_p, _i64, _i64, _i64, _vp, _vp, _P(_u64), _P(_vp)]),
    "aclnnDynamicMxQuant": (_i32, [_vp, _u64, _vp, _vp]),
    "aclnnQuantLightningIndexerGetWorkspaceSize": (_i32, [_vp] * 8 + [_i64, _i64, C.c_char_p, C.c_char_p, _i64, _i64, _i64, _i64, _vp,
                                                          _P(_u64), _P(_vp)]),
    "aclnnQuantLightningIndexer": (_i32, [_vp, _u64, _vp, _vp]),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        lib = C.CDLL(ffi.LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def last_error():
    text = load().aclGetRecentErrMsg()
    return text.decode() if text else ""


class Keep:
    """Keeps dim/stride arrays alive for as long as the descriptors built from them."""

    def __init__(self):
        self.arrays = []

    def tensor(self, dims, dtype, data, strides=None, offset=0):
        lib = load()
        d = (_i64 * len(dims))(*dims)
        s = (_i64 * len(dims))(*strides) if strides is not None else None
        self.arrays += [d, s]
        handle = lib.aclCreateTensor(d, len(dims), dtype, s, offset, ACL_FORMAT_ND, d, len(dims), data)
        assert handle, last_error()
        return handle

    def tensor_list(self, tensors):
        arr = (_vp * len(tensors))(*tensors)
        handle = load().aclCreateTensorList(arr, len(tensors))
        assert handle, last_error()
        return handle

    def int_array(self, values):
        arr = (_i64 * len(values))(*values)
        self.arrays.append(arr)
        handle = load().aclCreateIntArray(arr, len(values))
        assert handle, last_error()
        return handle, arr


def plan_scatter(key, key_cache, slot_mapping, value, value_cache, cache_mode=b"Norm", **overrides):
    lib = load()
    workspace, executor = _u64(123), _vp()
    args = dict(compress_lens=None, compress_seq_offset=None, seq_lens=None, scatter_mode=None, strides=None, offsets=None)
    args.update(overrides)
    status = lib.aclnnScatterPaKvCacheGetWorkspaceSize(key, key_cache, slot_mapping, value, value_cache, args["compress_lens"],
                                                       args["compress_seq_offset"], args["seq_lens"], cache_mode,
                                                       args["scatter_mode"], args["strides"], args["offsets"],
                                                       C.byref(workspace), C.byref(executor))
    return status, workspace.value, executor.value


def plan_attention(query, key_list, value_list, seq_q, seq_kv, block_table, query_rope, key_rope, heads, scale, block_size, out,
                   lse=None, lse_flag=False, layout=b"TND", kv_heads=1, sparse_mode=3, extra=None):
    """Argument order of the reference's call, src/pipeline/pipeline.cpp:237-248."""
    lib = load()
    workspace, executor = _u64(0), _vp()
    tensors = [None] * 31
    tensors[0], tensors[1], tensors[2] = query, key_list, value_list
    tensors[5], tensors[6] = seq_q, seq_kv
    tensors[14] = block_table
    tensors[24], tensors[25] = query_rope, key_rope
    for index, handle in (extra or {}).items():
        tensors[index] = handle
    status = lib.aclnnFusedInferAttentionScoreV5GetWorkspaceSize(
        *tensors, heads, scale, 65536, 0, layout, kv_heads, sparse_mode, 0, block_size, 0, lse_flag, 0, 0, 0, 0, out, lse,
        C.byref(workspace), C.byref(executor))
    return status, workspace.value, executor.value
