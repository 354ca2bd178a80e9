"""The drop-in boundary without a GPU: exported symbols, descriptor engine, plan-time contracts
and IR-index address swaps of the two operators, in the shape the reference engine uses them
(src/memory/static_arena_manager.cpp:567-588, src/pipeline/pipeline.cpp:226-249, :390-400).
No compute call is made here."""
import ctypes as C
import os
import re
import subprocess

import pytest

import acl_ffi as acl
import mlakv_ffi as ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x7F0000000000  # plan-time descriptors only carry addresses; nothing is dereferenced


def _declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:mlakv|acl|aclnn|aclrt)[A-Za-z0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(ffi.LIB_PATH)
    for header, minimum in (("mlakv.h", 45), ("aclnn_hip.h", 55)):
        names = _declared_functions(header)
        assert len(names) >= minimum, (header, len(names))
        for name in names:
            assert hasattr(lib, name), f"{name} declared in include/{header} is not exported"
    assert set(_declared_functions("mlakv.h")) == set(ffi.PROTOTYPES)
    assert set(_declared_functions("aclnn_hip.h")) == set(acl.PROTOTYPES)


def test_signatures_match_the_reference_typedefs(tmp_path):
    """The same technique as the reference (tests/mock_pipeline_e2e.cpp:59-73): static_assert the
    exported declarations against the plan / launch function-pointer types the engine casts
    its dlsym results to (include/moe/core/op_table.hpp:365-372, :438-454, :1022)."""
    source = tmp_path / "signature_check.cpp"
    source.write_text(r'''
#include <type_traits>
#include "aclnn_hip.h"
using ScatterPaKvCachePlanFn = int (*)(const aclTensor*, aclTensor*, const aclTensor*, const aclTensor*, aclTensor*,
                                       const aclTensor*, const aclTensor*, const aclTensor*, char*, char*, const aclIntArray*,
                                       const aclIntArray*, uint64_t*, aclOpExecutor**);
using FusedInferAttentionScoreV5PlanFn = int (*)(
    const aclTensor*, const aclTensorList*, const aclTensorList*, const aclTensor*, const aclTensor*, const aclIntArray*,
    const aclIntArray*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*,
    const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*,
    const aclTensor*, const aclTensor*, const aclTensor*, const aclIntArray*, const aclTensor*, const aclTensor*, const aclTensor*,
    const aclTensor*, const aclTensor*, const aclIntArray*, const aclIntArray*, int64_t, double, int64_t, int64_t, char*, int64_t,
    int64_t, int64_t, int64_t, int64_t, bool, int64_t, int64_t, int64_t, int64_t, const aclTensor*, const aclTensor*, uint64_t*,
    aclOpExecutor**);
using DynamicMxQuantPlanFn = int (*)(const aclTensor*, int64_t, char*, int64_t, int64_t, int64_t, const aclTensor*, const aclTensor*,
                                     uint64_t*, aclOpExecutor**);  // include/moe/core/op_table.hpp:230-233
using QuantLightningIndexerPlanFn = int (*)(const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*, const aclTensor*,
                                            const aclTensor*, const aclTensor*, const aclTensor*, int64_t, int64_t, char*, char*,
                                            int64_t, int64_t, int64_t, int64_t, const aclTensor*, uint64_t*,
                                            aclOpExecutor**);  // include/moe/core/op_table.hpp:998-1006
using AclnnLaunchFn = int (*)(void*, uint64_t, aclOpExecutor*, void*);
static_assert(std::is_same_v<decltype(&aclnnQuantLightningIndexerGetWorkspaceSize), QuantLightningIndexerPlanFn>);
static_assert(std::is_same_v<decltype(&aclnnQuantLightningIndexer), AclnnLaunchFn>);
static_assert(std::is_same_v<decltype(&aclnnDynamicMxQuantGetWorkspaceSize), DynamicMxQuantPlanFn>);
static_assert(std::is_same_v<decltype(&aclnnDynamicMxQuant), AclnnLaunchFn>);
static_assert(std::is_same_v<decltype(&aclnnScatterPaKvCacheGetWorkspaceSize), ScatterPaKvCachePlanFn>);
static_assert(std::is_same_v<decltype(&aclnnFusedInferAttentionScoreV5GetWorkspaceSize), FusedInferAttentionScoreV5PlanFn>);
static_assert(std::is_same_v<decltype(&aclnnScatterPaKvCache), AclnnLaunchFn>);
static_assert(std::is_same_v<decltype(&aclnnFusedInferAttentionScoreV5), AclnnLaunchFn>);
int main() { return 0; }
''')
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(source)], check=True)


def test_descriptor_round_trip_and_list_ownership():
    lib = acl.load()
    keep = acl.Keep()
    t = keep.tensor([128, 64, 1, 512], acl.ACL_BF16, FAKE)
    dims, count = C.POINTER(C.c_int64)(), C.c_uint64()
    assert lib.aclGetViewShape(t, C.byref(dims), C.byref(count)) == 0
    assert [dims[i] for i in range(count.value)] == [128, 64, 1, 512]
    assert lib.aclGetViewStrides(t, C.byref(dims), C.byref(count)) == 0
    assert [dims[i] for i in range(count.value)] == [64 * 512, 512, 512, 1]  # contiguous when strides are omitted
    dtype, fmt, addr, off = C.c_int32(), C.c_int32(), C.c_void_p(), C.c_int64()
    assert lib.aclGetDataType(t, C.byref(dtype)) == 0 and dtype.value == acl.ACL_BF16
    assert lib.aclGetFormat(t, C.byref(fmt)) == 0 and fmt.value == acl.ACL_FORMAT_ND
    assert lib.aclGetRawTensorAddr(t, C.byref(addr)) == 0 and addr.value == FAKE
    assert lib.aclGetViewOffset(t, C.byref(off)) == 0 and off.value == 0
    # a list owns copies of descriptors; destroying it destroys them (reference static_arena.cpp:172-208)
    copy = keep.tensor([128, 64, 1, 512], acl.ACL_BF16, FAKE)
    lst = keep.tensor_list([copy])
    assert lib.aclDestroyTensorList(lst) == 0
    assert lib.aclGetDataType(copy, C.byref(dtype)) == 161002  # gone with its list
    assert lib.aclDestroyTensor(copy) == 161002
    assert lib.aclDestroyTensor(t) == 0
    assert lib.aclDestroyTensor(t) == 161002
    assert lib.aclGetDataType(None, C.byref(dtype)) == 161001
    assert not lib.aclCreateTensorList(None, 0)
    assert not lib.aclCreateIntArray(None, 0)
    assert "empty" in acl.last_error()


class Engine:
    """Descriptors as the reference's CreateDescriptors builds them, for one sequence."""

    def __init__(self, block_size=64, max_context=8192, heads=64):
        self.keep = acl.Keep()
        k = self.keep
        self.bs, self.heads = block_size, heads
        self.blocks = -(-max_context // block_size)
        self.q_b = FAKE + 0x100000
        self.q_latent = k.tensor([1, heads, 512], acl.ACL_BF16, self.q_b, strides=[heads * 576, 576, 1])
        self.q_rope = k.tensor([1, heads, 64], acl.ACL_BF16, self.q_b + 1024, strides=[heads * 576, 576, 1])
        self.kv_latent_normed = k.tensor([1, 512], acl.ACL_BF16, FAKE + 0x200000)
        self.k_rope = k.tensor([1, 1, 64], acl.ACL_BF16, FAKE + 0x201000)
        self.latent_cache = k.tensor([self.blocks, block_size, 1, 512], acl.ACL_BF16, FAKE + 0x1000000)
        self.rope_cache = k.tensor([self.blocks, block_size, 1, 64], acl.ACL_BF16, FAKE + 0x9000000)
        self.rope_cache_view = k.tensor([self.blocks, block_size, 1, 64], acl.ACL_BF16, FAKE + 0x9000000)
        self.key_list = k.tensor_list([k.tensor([self.blocks, block_size, 1, 512], acl.ACL_BF16, FAKE + 0x1000000)])
        self.value_list = k.tensor_list([k.tensor([self.blocks, block_size, 1, 512], acl.ACL_BF16, FAKE + 0x1000000)])
        self.block_table = k.tensor([1, self.blocks], acl.ACL_INT32, FAKE + 0x300000)
        self.slot_mapping = k.tensor([1], acl.ACL_INT32, FAKE + 0x301000)
        self.seq_q, _ = k.int_array([1])
        self.seq_kv, self.seq_kv_storage = k.int_array([max_context])
        self.attn_out = k.tensor([1, heads, 512], acl.ACL_BF16, FAKE + 0x400000)
        self.lse = k.tensor([1, heads, 1], acl.ACL_FLOAT32, FAKE + 0x500000)

    def plan_attention(self, **kw):
        args = dict(heads=self.heads, scale=1.0 / 192 ** 0.5, block_size=self.bs)
        args.update(kw)
        return acl.plan_attention(self.q_latent, self.key_list, self.value_list, self.seq_q, self.seq_kv, self.block_table,
                                  self.q_rope, self.rope_cache_view, out=self.attn_out, lse=self.lse, **args)


def test_scatter_plan_contract_and_address_swaps():
    lib = acl.load()
    e = Engine()
    status, workspace, executor = acl.plan_scatter(e.kv_latent_normed, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache)
    assert status == 0 and executor and workspace == 0, acl.last_error()
    assert lib.aclSetAclOpExecutorRepeatable(executor) == 0
    # per-layer slices: IR indices 1 and 4 (reference pipeline.hpp:176-184)
    assert lib.aclSetTensorAddr(executor, 1, e.latent_cache, FAKE + 0x2000000) == 0
    assert lib.aclSetTensorAddr(executor, 4, e.rope_cache, FAKE + 0xA000000) == 0
    assert lib.aclSetTensorAddr(executor, 5, e.rope_cache, FAKE) == 161002   # bound as null at plan time
    assert lib.aclSetTensorAddr(executor, 40, e.rope_cache, FAKE) == 161002  # outside the captured arguments
    assert lib.aclSetTensorAddr(executor, 1, e.rope_cache, FAKE) == 161002   # shape is frozen after the plan
    assert lib.aclSetTensorAddr(executor, 1, e.latent_cache, None) == 161001
    assert lib.aclSetDynamicTensorAddr(executor, 1, 0, e.key_list, FAKE) == 161002  # slot 1 is a tensor, not a list
    assert lib.aclDestroyAclOpExecutor(executor) == 0
    assert lib.aclSetAclOpExecutorRepeatable(executor) == 161002
    # refusals
    k = e.keep
    assert acl.plan_scatter(None, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache)[0] == 161001
    slots64 = k.tensor([1], acl.ACL_INT64, FAKE)
    assert acl.plan_scatter(e.kv_latent_normed, e.latent_cache, slots64, e.k_rope, e.rope_cache)[0] == 161002
    assert acl.plan_scatter(e.kv_latent_normed, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache, cache_mode=b"PA_NZ")[0] == 161002
    assert acl.plan_scatter(e.kv_latent_normed, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache, seq_lens=e.slot_mapping)[0] == 161002
    assert acl.plan_scatter(e.kv_latent_normed, e.rope_cache, e.slot_mapping, e.k_rope, e.rope_cache)[0] == 161002  # key cache width
    flat = k.tensor([e.blocks * 64 * 512], acl.ACL_BF16, FAKE)
    assert acl.plan_scatter(e.kv_latent_normed, flat, e.slot_mapping, e.k_rope, e.rope_cache)[0] == 161002       # not paged
    status, _, executor = acl.plan_scatter(e.kv_latent_normed, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache, cache_mode=None)
    assert status == 0 and lib.aclDestroyAclOpExecutor(executor) == 0
    assert acl.plan_scatter(123456, e.latent_cache, e.slot_mapping, e.k_rope, e.rope_cache)[0] == 161002          # stale handle


def test_attention_plan_contract_workspace_and_ir_indices():
    lib = acl.load()
    e = Engine()
    status, workspace, executor = e.plan_attention()
    assert status == 0 and executor, acl.last_error()
    plan = ffi.AttnPlan()
    ffi.check(ffi.load().mlakvAttnPlanInit(1, 64, 8192, 64, ffi.DTYPE_BF16, C.byref(plan)))
    assert plan.max_units >= 1 and workspace >= plan.workspace_bytes + 4  # partials of split sequences + the lengths
    assert lib.aclSetAclOpExecutorRepeatable(executor) == 0
    layer_latent, layer_rope = FAKE + 0x3000000, FAKE + 0xB000000
    assert lib.aclSetDynamicTensorAddr(executor, 1, 0, e.key_list, layer_latent) == 0    # kFiaKeyList
    assert lib.aclSetDynamicTensorAddr(executor, 2, 0, e.value_list, layer_latent) == 0  # kFiaValueList
    assert lib.aclSetTensorAddr(executor, 25, e.rope_cache_view, layer_rope) == 0         # kFiaKeyRope
    assert lib.aclSetTensorAddr(executor, 24, e.q_rope, FAKE + 0x600000) == 0
    assert lib.aclSetTensorAddr(executor, 22, e.rope_cache_view, layer_rope) == 161002    # the mock's index is not the IR index
    assert lib.aclSetDynamicTensorAddr(executor, 1, 1, e.key_list, layer_latent) == 161002
    assert lib.aclSetDynamicTensorAddr(executor, 1, 0, e.value_list, layer_latent) == 161002
    assert lib.aclnnMlaKvBindSeqLens(executor, FAKE) == 0 and lib.aclnnMlaKvBindSeqLens(executor, None) == 0
    one = (C.c_int64 * 1)(17)
    assert lib.aclnnMlaKvSetSeqLens(executor, one, 1) == 0
    assert lib.aclnnMlaKvSetSeqLens(executor, one, 2) == 161002          # one length per sequence
    assert lib.aclnnMlaKvSetSeqLens(executor, (C.c_int64 * 1)(-1), 1) == 161002
    assert lib.aclnnMlaKvSetSeqLens(executor, (C.c_int64 * 1)(1 << 40), 1) == 161002
    assert lib.aclnnMlaKvSetSeqLens(executor, None, 1) == 161001
    assert lib.aclDestroyAclOpExecutor(executor) == 0
    # refusals, each naming the contract it breaks
    assert e.plan_attention(heads=32)[0] == 161002
    assert e.plan_attention(scale=0.0)[0] == 161002
    assert e.plan_attention(layout=b"BSND")[0] == 161002
    assert e.plan_attention(kv_heads=64)[0] == 161002
    assert e.plan_attention(block_size=128)[0] == 161002
    assert e.plan_attention(sparse_mode=4)[0] == 161002
    assert e.plan_attention(extra={4: e.block_table})[0] == 161002   # an attention mask
    assert e.plan_attention(extra={12: e.lse})[0] == 161002          # antiquant scale
    k = e.keep
    two, _ = k.int_array([5, 6])
    assert acl.plan_attention(e.q_latent, e.key_list, e.value_list, e.seq_q, two, e.block_table, e.q_rope, e.rope_cache_view, 64,
                              0.07, 64, e.attn_out)[0] == 161002
    assert acl.plan_attention(e.q_latent, e.key_list, e.value_list, e.seq_q, None, e.block_table, e.q_rope, e.rope_cache_view, 64,
                              0.07, 64, e.attn_out)[0] == 161001
    assert acl.plan_attention(e.q_latent, e.key_list, e.value_list, e.seq_q, e.seq_kv, e.block_table, e.q_rope, e.rope_cache_view,
                              64, 0.07, 64, e.attn_out, lse=None, lse_flag=True)[0] == 161002
    status, _, executor = e.plan_attention(lse_flag=True)
    assert status == 0 and lib.aclDestroyAclOpExecutor(executor) == 0
    # the failed plans returned no executor (the caller's partial-executor cleanup has nothing to do)
    assert e.plan_attention(heads=32)[2] is None


def test_thin_abi_argument_validation_without_a_device():
    lib = ffi.load()
    plan = ffi.AttnPlan()
    assert lib.mlakvAttnPlanInit(32, 64, 2048, 64, ffi.DTYPE_BF16, C.byref(plan)) == 0
    # without a device the plan assumes 256 CUs: one workgroup each, units cut from the live lengths at launch
    assert (plan.chunk_tiles, plan.work_groups, plan.max_units) == (0, 256, 256)
    assert (plan.merge_mode, plan.merge_spin_us) == (ffi.ATTN_MERGE_SECOND_LAUNCH, 50)
    # one partial slot per unit and one per sequence: bf16 partial outputs + fp32 partial LSEs
    assert plan.workspace_bytes == (256 + 32) * 64 * 512 * 2 + (256 + 32) * 64 * 4
    options = ffi.AttnPlanOptions(chunk_tiles=2, work_groups=0, merge_mode=ffi.ATTN_MERGE_IN_LAUNCH, merge_spin_us=-5)
    forced = ffi.AttnPlan()
    assert lib.mlakvAttnPlanInitEx(32, 128, 2048, 64, ffi.DTYPE_BF16, C.byref(options), C.byref(forced)) == 0
    assert (forced.chunk_tiles, forced.work_groups, forced.max_units) == (2, 128, 32 * (64 + 4) // 2)
    assert (forced.merge_mode, forced.merge_spin_us) == (ffi.ATTN_MERGE_IN_LAUNCH, -1)
    assert forced.workspace_bytes == 2 * (1088 + 32) * 64 * (1024 + 4)
    options.chunk_tiles = 1 << 20  # clamped to what a segment's staged table entries can address
    assert lib.mlakvAttnPlanInitEx(1, 64, 1 << 20, 16, ffi.DTYPE_BF16, C.byref(options), C.byref(forced)) == 0
    assert forced.chunk_tiles == (510 * 16 + 2) // 32
    options.merge_mode = 3
    assert lib.mlakvAttnPlanInitEx(32, 64, 2048, 64, ffi.DTYPE_BF16, C.byref(options), C.byref(forced)) == ffi.ERR_PARAM_INVALID
    # more (head group, sequence) pairs than the library keeps counters for: the merge stays a second launch
    options.merge_mode = ffi.ATTN_MERGE_IN_LAUNCH
    assert lib.mlakvAttnPlanInitEx(4097, 64, 64, 64, ffi.DTYPE_BF16, C.byref(options), C.byref(forced)) == 0
    assert forced.merge_mode == ffi.ATTN_MERGE_SECOND_LAUNCH
    assert lib.mlakvAttnPlanInit(32, 60, 2048, 64, ffi.DTYPE_BF16, C.byref(plan)) == ffi.ERR_PARAM_INVALID
    assert lib.mlakvAttnPlanInit(32, 64, 2048, 64, 7, C.byref(plan)) == ffi.ERR_PARAM_INVALID
    assert lib.mlakvAttnPlanInit(32, 64, 2048, 64, ffi.DTYPE_BF16, None) == ffi.ERR_PARAM_NULLPTR
    view = ffi.CacheView(latent=FAKE, latent_layer_stride=1 << 20, latent_block_stride=65536, latent_row_stride=1024,
                         rope=FAKE + (1 << 30), rope_layer_stride=1 << 17, rope_block_stride=8192, rope_row_stride=128,
                         num_layers=2, num_blocks=16, block_size=64, latent_dim=512, rope_dim=64, dtype=ffi.DTYPE_BF16)
    assert lib.mlakvAppend(None, 0, 1, FAKE, 0, 1024, FAKE, 0, 128, FAKE, 1, None) == ffi.ERR_PARAM_NULLPTR
    assert lib.mlakvAppend(C.byref(view), 0, 3, FAKE, 0, 1024, FAKE, 0, 128, FAKE, 1, None) == ffi.ERR_PARAM_INVALID   # layers
    assert lib.mlakvAppend(C.byref(view), 0, 1, FAKE + 2, 0, 1024, FAKE, 0, 128, FAKE, 1, None) == ffi.ERR_PARAM_INVALID  # alignment
    assert lib.mlakvAppend(C.byref(view), 0, 1, None, 0, 1024, FAKE, 0, 128, FAKE, 1, None) == ffi.ERR_PARAM_NULLPTR
    assert lib.mlakvAppend(C.byref(view), 0, 1, FAKE, 0, 1024, FAKE, 0, 128, FAKE, 0, None) == 0                       # nothing to do
    bad = ffi.CacheView.from_buffer_copy(view)
    bad.latent_dim = 256
    assert lib.mlakvGather(C.byref(bad), 0, 1, FAKE, 4, FAKE, FAKE, 1, 64, FAKE, 0, 1024, FAKE, 0, 128, None) == ffi.ERR_PARAM_INVALID
    assert "512" in ffi.last_error()
    assert lib.mlakvGather(C.byref(view), 0, 1, FAKE, 1, FAKE, FAKE, 1, 4096, FAKE, 0, 1024, FAKE, 0, 128, None) == ffi.ERR_PARAM_INVALID
    fp8 = ffi.CacheView.from_buffer_copy(view)
    fp8.dtype = ffi.DTYPE_FP8_E4M3
    assert lib.mlakvCopyBlocks(C.byref(fp8), 0, 1, FAKE, 1, None) == ffi.ERR_PARAM_NULLPTR  # FP8 without a scale plane
    # a plan altered after its init call is refused at launch (the kernels size LDS staging from it)
    assert lib.mlakvAttnPlanInit(32, 64, 2048, 64, ffi.DTYPE_BF16, C.byref(plan)) == 0
    row = 1152

    def decode(p):
        return lib.mlakvAttnDecode(C.byref(p), C.byref(view), 0, FAKE, 64 * row, row, FAKE + 1024, 64 * row, row, FAKE, 32, FAKE,
                                   0.07, FAKE, 64 * 1024, 1024, None, None, 0, None)

    assert decode(plan) == ffi.ERR_PARAM_NULLPTR          # everything fine up to the missing workspace
    for field, value in (("chunk_tiles", 4096), ("chunk_tiles", -1), ("max_units", 9), ("heads", 60), ("workspace_bytes", 16),
                         ("reserved", 2), ("batch", 0), ("work_groups", 0), ("merge_mode", 0), ("merge_spin_us", 0)):
        altered = ffi.AttnPlan.from_buffer_copy(plan)
        setattr(altered, field, value)
        assert decode(altered) == ffi.ERR_PARAM_INVALID, field
        assert "not one made by" in ffi.last_error()
    sparse = ffi.AttnPlan()
    assert lib.mlakvAttnSparsePlanInit(32, 64, 512, 64, ffi.DTYPE_BF16, C.byref(sparse)) == 0
    assert sparse.reserved == 1 and sparse.max_seq_len == 512 and sparse.chunk_tiles == 0
    assert decode(sparse) == ffi.ERR_PARAM_INVALID        # a selection plan handed to the whole-context entry
    # how a selection plan cuts its work: whole selections for 16 heads while batch x heads / 16 units
    # fit the CUs once (up to 512 selected tokens) or twice (up to 256), two workgroups per unit from
    # 257 to 768 selected tokens while those fit the CUs once, bf16 only; the split otherwise
    if lib.mlakvDeviceCount() == 0:                       # (planning without a device assumes the 256 CUs of an MI355X)
        for batch, heads, count, dtype, expected in ((32, 64, 512, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (32, 64, 256, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (32, 64, 257, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (32, 64, 768, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (32, 64, 769, ffi.DTYPE_BF16, ffi.ATTN_UNITS_SPLIT),
                                                     (16, 128, 512, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (33, 64, 512, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (64, 64, 512, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (65, 64, 512, ffi.DTYPE_BF16, ffi.ATTN_UNITS_SPLIT),
                                                     (128, 64, 256, ffi.DTYPE_BF16, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (128, 64, 257, ffi.DTYPE_BF16, ffi.ATTN_UNITS_SPLIT),
                                                     (128, 128, 128, ffi.DTYPE_BF16, ffi.ATTN_UNITS_SPLIT),
                                                     (64, 64, 513, ffi.DTYPE_BF16, ffi.ATTN_UNITS_SPLIT),
                                                     (32, 64, 512, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (32, 64, 1024, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES),
                                                     (32, 64, 256, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (128, 64, 1024, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (512, 64, 256, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_HEAD_BLOCK),
                                                     (512, 64, 257, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_SPLIT),
                                                     (32, 64, 1025, ffi.DTYPE_FP8_E4M3, ffi.ATTN_UNITS_SPLIT)):
            assert lib.mlakvAttnSparsePlanInit(batch, heads, count, 64, dtype, C.byref(sparse)) == 0
            assert sparse.selection_units == expected, (batch, heads, count, dtype)
    forced = ffi.AttnPlanOptions(0, 0, 0, 0, 1, ffi.ATTN_UNITS_HEAD_BLOCK)
    assert lib.mlakvAttnPlanInitEx(128, 128, 1024, 64, ffi.DTYPE_BF16, C.byref(forced), C.byref(sparse)) == 0
    assert sparse.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK
    assert lib.mlakvAttnPlanInitEx(32, 64, 1025, 64, ffi.DTYPE_BF16, C.byref(forced), C.byref(sparse)) == ffi.ERR_PARAM_INVALID
    halved = ffi.AttnPlanOptions(0, 0, 0, 0, 1, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES)
    assert lib.mlakvAttnPlanInitEx(128, 128, 64, 64, ffi.DTYPE_BF16, C.byref(halved), C.byref(sparse)) == 0
    assert sparse.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK_HALVES
    assert lib.mlakvAttnPlanInitEx(32, 64, 512, 64, ffi.DTYPE_FP8_E4M3, C.byref(halved), C.byref(sparse)) == 0
    assert sparse.selection_units == ffi.ATTN_UNITS_HEAD_BLOCK_HALVES
    assert lib.mlakvAttnPlanInitEx(32, 64, 1025, 64, ffi.DTYPE_FP8_E4M3, C.byref(halved), C.byref(sparse)) == ffi.ERR_PARAM_INVALID
    assert lib.mlakvAttnPlanInitEx(2048, 128, 64, 64, ffi.DTYPE_BF16, C.byref(halved), C.byref(sparse)) == ffi.ERR_PARAM_INVALID  # more pairs than counters
    for option in ({"chunk_tiles": 2}, {"work_groups": 64}, {"merge_mode": ffi.ATTN_MERGE_SECOND_LAUNCH}):   # properties of the split
        asked = ffi.AttnPlanOptions(option.get("chunk_tiles", 0), option.get("work_groups", 0), option.get("merge_mode", 0), 0, 1, 0)
        assert lib.mlakvAttnPlanInitEx(32, 64, 512, 64, ffi.DTYPE_BF16, C.byref(asked), C.byref(sparse)) == 0
        assert sparse.selection_units == ffi.ATTN_UNITS_SPLIT, option
    # whole-context plans keep what was asked for (AUTO: every launch chooses); the units need a context they can stage
    dense_option = ffi.AttnPlanOptions(0, 0, 0, 0, 0, ffi.ATTN_UNITS_SPLIT)
    assert lib.mlakvAttnPlanInitEx(32, 64, 2048, 64, ffi.DTYPE_BF16, C.byref(dense_option), C.byref(sparse)) == 0
    assert sparse.selection_units == ffi.ATTN_UNITS_SPLIT and sparse.reserved == 0
    for units in (ffi.ATTN_UNITS_HEAD_BLOCK, ffi.ATTN_UNITS_HEAD_BLOCK_HALVES):
        dense_option = ffi.AttnPlanOptions(0, 0, 0, 0, 0, units)
        assert lib.mlakvAttnPlanInitEx(32, 64, 1025, 64, ffi.DTYPE_BF16, C.byref(dense_option), C.byref(sparse)) == ffi.ERR_PARAM_INVALID
        assert lib.mlakvAttnPlanInitEx(32, 64, 1024, 64, ffi.DTYPE_BF16, C.byref(dense_option), C.byref(sparse)) == 0
        assert sparse.selection_units == units
    dense_option = ffi.AttnPlanOptions(2, 0, 0, 0, 0, 0)                      # a property of the split pins the split
    assert lib.mlakvAttnPlanInitEx(32, 64, 256, 64, ffi.DTYPE_BF16, C.byref(dense_option), C.byref(sparse)) == 0
    assert sparse.selection_units == ffi.ATTN_UNITS_SPLIT
    assert lib.mlakvAttnPlanInit(32, 64, 2048, 64, ffi.DTYPE_BF16, C.byref(sparse)) == 0 and sparse.selection_units == 0
    altered = ffi.AttnPlan.from_buffer_copy(sparse)
    altered.selection_units = ffi.ATTN_UNITS_HEAD_BLOCK   # a whole-context plan that claims a selection's units
    assert decode(altered) == ffi.ERR_PARAM_INVALID


@pytest.mark.skipif(ffi.load().mlakvDeviceCount() > 0, reason="checks the no-device behaviour")
def test_no_device_fails_loudly_instead_of_falling_back():
    with pytest.raises(ffi.MlakvError) as info:
        ffi.Arena(ffi.BACKEND_HIP)
    assert "no HIP device" in str(info.value)
    # the warm-up reports the runtime's error as a status; it does not pretend to have prepared anything
    lib = ffi.load()
    assert lib.mlakvPrepare() == ffi.ERR_RUNTIME
    assert b"mlakvPrepare" in lib.mlakvGetLastError()


def test_mx_quant_plan_contract():
    """aclnnDynamicMxQuant plan phase with the attributes the reference passes (src/pipeline/pipeline.cpp:251-258:
    axis -1, "rint", E4M3, block 32, OCP) and refusals for anything else; no device is touched."""
    lib = acl.load()
    keep = acl.Keep()
    rows, cols = 3, 64 * 512
    x = keep.tensor([rows, cols], acl.ACL_BF16, None)
    y = keep.tensor([rows, cols], acl.ACL_FLOAT8_E4M3FN, None)
    scales = keep.tensor([rows, cols // 32], 37, None)

    def plan(x=x, axis=-1, mode=b"rint", dst=36, block=32, alg=0, y=y, scales=scales):
        workspace, executor = C.c_uint64(99), C.c_void_p()
        status = lib.aclnnDynamicMxQuantGetWorkspaceSize(x, axis, mode, dst, block, alg, y, scales, C.byref(workspace), C.byref(executor))
        return status, workspace.value, executor.value

    status, workspace, executor = plan()
    assert status == 0 and workspace == 0 and executor
    assert lib.aclDestroyAclOpExecutor(executor) == 0
    assert plan(axis=1)[0] == 0 and plan(mode=None)[0] == 0
    assert plan(axis=0)[0] == ffi.ERR_PARAM_INVALID
    assert plan(mode=b"round")[0] == ffi.ERR_PARAM_INVALID
    assert plan(dst=35)[0] == ffi.ERR_PARAM_INVALID
    assert plan(block=16)[0] == ffi.ERR_PARAM_INVALID
    assert plan(alg=1)[0] == ffi.ERR_PARAM_INVALID
    assert plan(x=None)[0] == ffi.ERR_PARAM_NULLPTR
    assert plan(y=keep.tensor([rows, cols], acl.ACL_BF16, None))[0] == ffi.ERR_PARAM_INVALID
    assert plan(scales=keep.tensor([rows, cols // 16], 37, None))[0] == ffi.ERR_PARAM_INVALID
    assert plan(x=keep.tensor([rows, 40], acl.ACL_BF16, None), y=keep.tensor([rows, 40], acl.ACL_FLOAT8_E4M3FN, None))[0] == ffi.ERR_PARAM_INVALID
    assert "DynamicMxQuant" in acl.last_error()


def test_indexer_plan_contract():
    """aclnnQuantLightningIndexer plan phase for the decode shape (one query token per sequence, paged E4M3 keys) and
    its refusals; no device is touched."""
    lib = acl.load()
    keep = acl.Keep()
    batch, heads, blocks, bs, width, k = 4, 64, 40, 64, 8, 512
    E8 = acl.ACL_FLOAT8_E4M3FN
    t = dict(query=keep.tensor([batch, 1, heads, 128], E8, None), key=keep.tensor([blocks, bs, 1, 128], E8, None),
             weights=keep.tensor([batch, 1, heads], acl.ACL_BF16, None), q_scale=keep.tensor([batch, 1, heads], acl.ACL_FLOAT32, None),
             k_scale=keep.tensor([blocks, bs, 1], acl.ACL_FLOAT32, None), lens=keep.tensor([batch], acl.ACL_INT32, None),
             table=keep.tensor([batch, width], acl.ACL_INT32, None), out=keep.tensor([batch, 1, 1, k], acl.ACL_INT32, None))
    big = 2 ** 63 - 1

    def plan(qmode=0, kmode=0, lq=b"BSND", lk=b"PA_BSND", count=k, mode=3, pre=big, nxt=big, **over):
        a = dict(t)
        a.update(over)
        workspace, executor = C.c_uint64(7), C.c_void_p()
        status = lib.aclnnQuantLightningIndexerGetWorkspaceSize(a["query"], a["key"], a["weights"], a["q_scale"], a["k_scale"], None, a["lens"],
                                                                a["table"], qmode, kmode, lq, lk, count, mode, pre, nxt, a["out"],
                                                                C.byref(workspace), C.byref(executor))
        return status, workspace.value, executor.value

    status, workspace, executor = plan()
    assert status == 0 and executor and workspace == batch * width * bs * 2      # 16-bit scores of every addressable token
    assert lib.aclDestroyAclOpExecutor(executor) == 0
    assert plan(mode=0)[0] == 0 and plan(lq=None)[0] == 0
    assert plan(qmode=1)[0] == ffi.ERR_PARAM_INVALID
    assert plan(lk=b"BSND")[0] == ffi.ERR_PARAM_INVALID and plan(lk=None)[0] == ffi.ERR_PARAM_INVALID
    assert plan(count=4096)[0] == ffi.ERR_PARAM_INVALID
    assert plan(mode=1)[0] == ffi.ERR_PARAM_INVALID
    assert plan(pre=128)[0] == ffi.ERR_PARAM_INVALID
    assert plan(table=None)[0] == ffi.ERR_PARAM_NULLPTR and plan(lens=None)[0] == ffi.ERR_PARAM_NULLPTR
    assert plan(query=keep.tensor([batch, 2, heads, 128], E8, None))[0] == ffi.ERR_PARAM_INVALID   # more than one query token
    assert plan(query=keep.tensor([batch, 1, 24, 128], E8, None), weights=keep.tensor([batch, 1, 24], acl.ACL_BF16, None),
                q_scale=keep.tensor([batch, 1, 24], acl.ACL_FLOAT32, None))[0] == ffi.ERR_PARAM_INVALID
    assert plan(key=keep.tensor([blocks, bs, 1, 64], E8, None))[0] == ffi.ERR_PARAM_INVALID
    assert plan(out=keep.tensor([batch, 1, 1, k + 1], acl.ACL_INT32, None))[0] == ffi.ERR_PARAM_INVALID
    assert plan(weights=keep.tensor([batch, 1, heads], acl.ACL_FLOAT32, None))[0] == ffi.ERR_PARAM_INVALID
    assert "QuantLightningIndexer" in acl.last_error()
