"""The C-ABI library without a GPU: it loads, exports every symbol the headers declare, and its first-phase entry points
apply the reference's argument rules with the reference's return codes (the phase never touches device memory, so fake
device pointers suffice).  Negative cases mirror the reference's own op_api / tiling unit tests:
  moe/moe_init_routing_v2/tests/utest/ts_moe_init_routing_v2_tc.cpp:59-141
  gmm/grouped_matmul_swiglu_quant/tests/ut/op_host/op_api/test_aclnn_grouped_matmul_swiglu_quant.cpp:38-63
  gmm/grouped_matmul/tests/utest_aclnn/ts_aclnn_grouped_matmul.cpp
  moe/moe_finalize_routing_v2/tests/ut/op_host/test_moe_finalize_routing_v2_tiling.cpp
"""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NULLPTR, INVALID = 161001, 161002


def _declared_symbols():
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "**", "*.h"), recursive=True):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"(?:ACL_API|ACLNN_API|__attribute__\(\(visibility\(\"default\"\)\)\))\s+[\w\s\*]+?\b(\w+)\s*\(", text):
            names.add(m.group(1))
    return sorted(names)


def test_headers_declare_the_expected_entry_points():
    names = _declared_symbols()
    for required in ["aclnnMoeInitRoutingV2GetWorkspaceSize", "aclnnMoeInitRoutingV2",
                     "aclnnMoeInitRoutingV3GetWorkspaceSize", "aclnnMoeInitRoutingV3",
                     "aclnnMoeInitRoutingQuantV2GetWorkspaceSize", "aclnnMoeInitRoutingQuantV2",
                     "aclnnMoeGatingTopKSoftmaxV2GetWorkspaceSize", "aclnnMoeGatingTopKSoftmaxV2",
                     "aclnnGroupedMatmulFinalizeRoutingGetWorkspaceSize", "aclnnGroupedMatmulFinalizeRouting",
                     "aclnnGroupedMatmulFinalizeRoutingV2GetWorkspaceSize", "aclnnGroupedMatmulFinalizeRoutingV2",
                     "aclnnGroupedMatmulFinalizeRoutingV3GetWorkspaceSize", "aclnnGroupedMatmulFinalizeRoutingV3",
                     "aclnnGroupedMatmulFinalizeRoutingWeightNzGetWorkspaceSize", "aclnnGroupedMatmulFinalizeRoutingWeightNz",
                     "aclnnGroupedMatmulFinalizeRoutingWeightNzV2GetWorkspaceSize",
                     "aclnnGroupedMatmulFinalizeRoutingWeightNzV2",
                     "aclnnGroupedMatmulSwigluQuantGetWorkspaceSize", "aclnnGroupedMatmulSwigluQuant",
                     "aclnnGroupedMatmulSwigluQuantWeightNZGetWorkspaceSize", "aclnnGroupedMatmulSwigluQuantWeightNZ",
                     "aclnnGroupedMatmulWeightNzGetWorkspaceSize", "aclnnGroupedMatmulWeightNz",
                     "aclnnGroupedMatmulV4GetWorkspaceSize", "aclnnGroupedMatmulV4",
                     "aclnnGroupedMatmulV5GetWorkspaceSize", "aclnnGroupedMatmulV5",
                     "aclnnMoeFinalizeRoutingV2GetWorkspaceSize", "aclnnMoeFinalizeRoutingV2",
                     "aclCreateTensor", "aclDestroyTensor", "aclCreateTensorList", "aclDestroyTensorList", "aclrtMalloc",
                     "aclrtMemcpy", "aclGetRecentErrMsg", "ResetCacheThreadLocal", "opapiKernelTimerEnable",
                     "opapiKernelTimerReport"]:
        assert required in names, required


def test_library_exports_every_declared_symbol(aclnn):
    lib = ctypes.CDLL(aclnn.library_path())
    missing = [n for n in _declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


# ------------------------------------------------------------------------------------------------ helpers
F32, F16, I8, I32, I64, BOOL, BF16 = 0, 1, 2, 3, 9, 12, 27


class T:
    """Descriptor over a fake device address (phase 1 never dereferences it)."""
    _next = 0x10000

    def __init__(self, aclnn, shape, dtype, strides=None, data=True, fmt=2, storage=None):
        T._next += 0x10000
        self.h = aclnn.create_tensor(list(shape), dtype, T._next if data else 0, strides, 0, fmt, storage)


def _status(aclnn, api, args):
    try:
        return 0, aclnn.workspace_size(api, args)
    except aclnn.AclnnError as e:
        assert e.message, "an error status must come with a message"
        return e.code, e.message


def _tl(aclnn, tensors):
    arr = (ctypes.c_void_p * len(tensors))(*[t.h for t in tensors])
    return aclnn.lib().aclCreateTensorList(arr, len(tensors))


# ------------------------------------------------------------------------------------------------ routing
def _routing_args(aclnn, T_=8, K=2, H=16, E=4, mode=0, C=0, flag=0, before=False, active=0, x_dtype=F32, **over):
    x = T(aclnn, (T_, H), x_dtype)
    idx = T(aclnn, (T_, K), I32)
    if mode == 0:
        rows = T_ * K if active == 0 else min(T_ * K, active)
        ex = T(aclnn, over.get("ex_shape", (rows, H)), x_dtype)
    else:
        ex = T(aclnn, over.get("ex_shape", (E, C, H)), x_dtype)
    ri = T(aclnn, over.get("ri_shape", (T_ * K,)), I32)
    cnt = T(aclnn, over.get("cnt_shape", (E,)), I32) if over.get("with_cnt", flag > 0) else None
    bef = T(aclnn, (E,), I32) if before else None
    return [x.h, idx.h, active, C, E, mode, flag, before, ex.h, ri.h, cnt.h if cnt else None, bef.h if bef else None]


def test_routing_valid_shapes(aclnn):
    for kw in [dict(), dict(flag=1), dict(flag=2), dict(mode=1, C=3, before=True), dict(active=5), dict(x_dtype=I8),
               dict(x_dtype=BF16, flag=1), dict(T_=0)]:
        code, ws = _status(aclnn, "aclnnMoeInitRoutingV2", _routing_args(aclnn, **kw))
        assert code == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    (dict(mode=2), "dropPadMode should be 0 or 1"),
    (dict(flag=3), "should be 0, 1 or 2"),
    (dict(flag=1, E=0, with_cnt=False), "expertNum should be greater than 0"),
    (dict(mode=1, C=0), "greater than 0 when dropPadMode is 1"),
    (dict(mode=1, C=9, T_=8), "cannot be less than expertCapacity"),
    (dict(ex_shape=(15, 16)), "first dim of expandedX"),
    (dict(ex_shape=(16, 17)), "second dim of expandedX"),
    (dict(ri_shape=(15,)), "first dim of expandedRowIdx"),
    (dict(flag=1, cnt_shape=(5,)), "expertTokensCountOrCumsum"),
    (dict(active=-1), "activeNum cannot be less than 0"),
    (dict(E=-1), "expertNum cannot be less than 0"),
])
def test_routing_invalid_arguments(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnMoeInitRoutingV2", _routing_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_routing_null_and_rank_checks(aclnn):
    args = _routing_args(aclnn)
    args[0] = None
    assert _status(aclnn, "aclnnMoeInitRoutingV2", args)[0] == NULLPTR
    args = _routing_args(aclnn, flag=1, with_cnt=False)
    assert _status(aclnn, "aclnnMoeInitRoutingV2", args)[0] == NULLPTR  # count output requested but absent
    x3 = T(aclnn, (2, 2, 2), F32)
    args = _routing_args(aclnn)
    args[0] = x3.h
    code, msg = _status(aclnn, "aclnnMoeInitRoutingV2", args)
    assert code == INVALID and "dim number of x should be 2" in msg


# ------------------------------------------------------------------------------------------------ gating
def _gating_args(aclnn, shape=(6, 16), k=4, renorm=0, flag=False, dtype=F32, finished=False, **over):
    x = T(aclnn, shape, dtype)
    fin = T(aclnn, over.get("fin_shape", shape[:-1]), over.get("fin_dtype", BOOL)) if finished else None
    y = T(aclnn, over.get("y_shape", tuple(shape[:-1]) + (k,)), over.get("y_dtype", dtype))
    idx = T(aclnn, over.get("idx_shape", tuple(shape[:-1]) + (k,)), over.get("idx_dtype", I32))
    sm = T(aclnn, over.get("sm_shape", shape), over.get("sm_dtype", F32)) if over.get("with_sm", flag) else None
    return [x.h, fin.h if fin else None, k, renorm, flag, y.h, idx.h, sm.h if sm else None]


def test_gating_valid(aclnn):
    for kw in [dict(), dict(renorm=1), dict(flag=True), dict(renorm=1, flag=True, with_sm=False), dict(dtype=F16),
               dict(dtype=BF16, finished=True), dict(shape=(2, 3, 16)), dict(shape=(2, 3, 16), finished=True, flag=True),
               dict(shape=(0, 16)), dict(k=16), dict(shape=(4, 32768), k=1024)]:
        code, ws = _status(aclnn, "aclnnMoeGatingTopKSoftmaxV2", _gating_args(aclnn, **kw))
        assert code == 0 and ws == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    # rules and messages of moe/moe_gating_top_k_softmax_v2/op_host/moe_gating_top_k_softmax_v2_tiling_base.cpp:40-260
    (dict(dtype=I8), "only supports float32,half,bf16"),
    (dict(shape=(16,), y_shape=(4,), idx_shape=(4,)), "x shape dim(=1) is not 2 or 3"),
    (dict(shape=(2, 2, 2, 16)), "x shape dim(=4) is not 2 or 3"),
    (dict(shape=(6, 0), k=1), "last dim is zero"),
    (dict(finished=True, fin_dtype=I8), "should be BOOL"),
    (dict(finished=True, fin_shape=(6, 1)), "finished dim num (=2) error, should be (=1)"),
    (dict(finished=True, fin_shape=(5,)), "finished and x shape not equal"),
    (dict(k=0), "attr k(=0) is wrong"),
    (dict(k=17), "attr k(=17) is wrong"),
    (dict(shape=(2, 4096), k=1025), "attr k(=1025) is too large"),
    (dict(renorm=2), "attr renorm(=2) is wrong"),
    (dict(y_dtype=F16), "should be same with x data type"),
    (dict(y_shape=(6, 5)), "with last dim k"),
    (dict(y_shape=(5, 4)), "with last dim k"),
    (dict(idx_dtype=I64), "only supports int32"),
    (dict(idx_shape=(6, 3)), "with last dim k"),
    (dict(flag=True, sm_dtype=F16), "should be float"),
    (dict(flag=True, sm_shape=(6, 15)), "softmaxResult and x shape not equal"),
    (dict(shape=(2, 32769)), "at most 32768 experts"),
])
def test_gating_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnMoeGatingTopKSoftmaxV2", _gating_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_gating_nulls(aclnn):
    for pos in (0, 5, 6):
        args = _gating_args(aclnn)
        args[pos] = None
        assert _status(aclnn, "aclnnMoeGatingTopKSoftmaxV2", args)[0] == NULLPTR, pos
    args = _gating_args(aclnn, flag=True, with_sm=False)       # softmax output requested, no tensor for it
    assert _status(aclnn, "aclnnMoeGatingTopKSoftmaxV2", args)[0] == NULLPTR


# ------------------------------------------------------------------------------------------------ routing QuantV2
def _routing_quant_v2_args(aclnn, T_=8, K=2, H=16, E=4, mode=0, C=0, flag=0, before=False, active=0, x_dtype=BF16, quant=0,
                           with_scale=True, with_offset=True, with_dyn=None, **over):
    x = T(aclnn, (T_, H), x_dtype)
    idx = T(aclnn, (T_, K), I32)
    if quant == 0:
        scale = T(aclnn, over.get("scale_shape", (1,)), over.get("scale_dtype", F32)) if with_scale else None
        offset = T(aclnn, over.get("offset_shape", (1,)), over.get("offset_dtype", F32)) if with_offset else None
    else:
        scale = T(aclnn, over.get("scale_shape", (E, H)), over.get("scale_dtype", F32)) if with_scale else None
        offset = None
    rows = E * C if mode == 1 else (T_ * K if active == 0 else min(T_ * K, active))
    ex = T(aclnn, over.get("ex_shape", (E, C, H) if mode == 1 else (rows, H)), over.get("ex_dtype", I8))
    ri = T(aclnn, (T_ * K,), I32)
    cnt = T(aclnn, (E,), I32) if flag > 0 else None
    bef = T(aclnn, (E,), I32) if before else None
    dyn = None
    if with_dyn if with_dyn is not None else quant == 1:
        dyn = T(aclnn, over.get("dyn_shape", (rows,)), over.get("dyn_dtype", F32))
    return [x.h, idx.h, scale.h if scale else None, offset.h if offset else None, active, C, E, mode, flag, before, quant,
            ex.h, ri.h, cnt.h if cnt else None, bef.h if bef else None, dyn.h if dyn else None]


def test_routing_quant_v2_valid(aclnn):
    for kw in [dict(), dict(x_dtype=F32, flag=1), dict(x_dtype=F16, flag=2), dict(mode=1, C=3, before=True), dict(active=5),
               dict(quant=1), dict(quant=1, scale_shape=(1, 16)), dict(quant=1, with_scale=False),
               dict(quant=1, mode=1, C=3, before=True), dict(quant=1, active=5, flag=1), dict(T_=0), dict(quant=1, T_=0)]:
        code, ws = _status(aclnn, "aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, **kw))
        assert code == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    # rules and messages of moe/moe_init_routing_quant_v2/op_host/moe_init_routing_quant_v2_tiling.cpp:132-219
    (dict(quant=2), "quantMode should be 0 or 1"),
    (dict(quant=-1), "quantMode should be 0 or 1"),
    (dict(x_dtype=I8), "not INT8"),
    (dict(ex_dtype=BF16), "expandedXOut must be INT8"),
    (dict(scale_dtype=F16), "data type of scale should be float"),
    (dict(offset_dtype=F16), "data type of offset should be float"),
    (dict(scale_shape=(1, 1)), "dim number of scale should be 1"),
    (dict(scale_shape=(2,)), "first dim of scale should be 1"),
    (dict(offset_shape=(1, 1)), "dim number of offset should be 1"),
    (dict(offset_shape=(2,)), "first dim of offset should be 1"),
    (dict(quant=1, scale_shape=(16,)), "dim number of scale should be 2"),
    (dict(quant=1, scale_shape=(3, 16)), "first dim of scale should be 1 or expert_num"),
    (dict(quant=1, scale_shape=(4, 15)), "second dim of scale should be 16"),
    (dict(quant=1, scale_dtype=F16), "data type of scale should be float"),
    (dict(quant=1, dyn_shape=(15,)), "first dim of dynamicQuantScale should be 16"),
    (dict(quant=1, dyn_shape=(16, 1)), "dim number of dynamicQuantScale should be 1"),
    (dict(quant=1, dyn_dtype=F16), "dynamicQuantScale should be FLOAT"),
    (dict(quant=1, mode=1, C=3, dyn_shape=(16,)), "first dim of dynamicQuantScale should be 12"),
    (dict(quant=1, active=5, dyn_shape=(16,)), "first dim of dynamicQuantScale should be 5"),
    (dict(mode=2), "dropPadMode should be 0 or 1"),
    (dict(flag=3), "should be 0, 1 or 2"),
    (dict(mode=1, C=0), "greater than 0 when dropPadMode is 1"),
    (dict(mode=1, C=9), "cannot be less than expertCapacity"),
    (dict(ex_shape=(15, 16)), "first dim of expandedX"),
    (dict(active=-1), "activeNum cannot be less than 0"),
])
def test_routing_quant_v2_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_routing_quant_v2_nulls(aclnn):
    for pos in (0, 1, 11, 12):
        args = _routing_quant_v2_args(aclnn)
        args[pos] = None
        assert _status(aclnn, "aclnnMoeInitRoutingQuantV2", args)[0] == NULLPTR, pos
    # static quantisation needs both scale and offset (moe_init_routing_quant_v2_tiling.cpp:179-198)
    assert _status(aclnn, "aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, with_scale=False))[0] == NULLPTR
    assert _status(aclnn, "aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, with_offset=False))[0] == NULLPTR
    # dynamic quantisation always emits its scales (moe_init_routing_quant_v2_tiling.cpp:138-140)
    assert _status(aclnn, "aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, quant=1, with_dyn=False))[0] == NULLPTR
    args = _routing_quant_v2_args(aclnn, flag=1)
    args[13] = None
    assert _status(aclnn, "aclnnMoeInitRoutingQuantV2", args)[0] == NULLPTR


# ------------------------------------------------------------------------------------------------ routing V3
def _routing_v3_args(aclnn, T_=8, K=2, H=16, E=4, rng=None, num_type=1, flag=True, quant=-1, row_idx_type=1, active=-1,
                     mode=0, x_dtype=I8, with_scale=True, **over):
    x = T(aclnn, (T_, H), x_dtype)
    idx = T(aclnn, (T_, K), I32)
    scale = T(aclnn, over.get("scale_shape", (T_,)), F32) if with_scale else None
    start, end = (0, E) if rng is None else rng[:2]
    ex = T(aclnn, over.get("ex_shape", (T_ * K, H)), over.get("ex_dtype", x_dtype))
    ri = T(aclnn, over.get("ri_shape", (T_ * K,)), I32)
    cnt = T(aclnn, over.get("cnt_shape", (E, 2) if num_type == 2 else (max(end - start, 0),)), over.get("cnt_dtype", I64))
    es = T(aclnn, (T_ * K,), F32) if (with_scale or over.get("with_es")) else None
    arr = None if rng is None else aclnn.lib().aclCreateIntArray((ctypes.c_int64 * len(rng))(*rng), len(rng))
    return [x.h, idx.h, scale.h if scale else None, None, active, 0, E, mode, num_type, flag, quant, arr, row_idx_type,
            ex.h, ri.h, cnt.h, es.h if es else None]


def test_routing_v3_valid(aclnn):
    for kw in [dict(), dict(num_type=0), dict(num_type=2), dict(rng=(1, 3)), dict(row_idx_type=0), dict(active=16),
               dict(x_dtype=BF16, with_scale=False), dict(T_=0), dict(E=2048), dict(E=4096, rng=(100, 2147)),
               dict(quant=1, x_dtype=BF16, ex_dtype=I8, scale_shape=(4, 16)),
               dict(quant=1, x_dtype=F32, ex_dtype=I8, rng=(1, 3), scale_shape=(2, 16)),
               dict(quant=1, x_dtype=F16, ex_dtype=I8, with_scale=False, with_es=True)]:
        code, ws = _status(aclnn, "aclnnMoeInitRoutingV3", _routing_v3_args(aclnn, **kw))
        assert code == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    # attribute rules and messages of moe/moe_init_routing_v3/op_host/moe_init_routing_v3_tiling.cpp:233-352
    (dict(active=-2), "active_num should be greater than or equal to -1"),
    (dict(active=5), "active_num currently should equal to 16"),
    (dict(E=0, cnt_shape=(1,)), "expert_num should be greater than 0"),
    (dict(mode=1), "drop_pad_mode currently support 0"),
    (dict(num_type=3), "expert_tokens_num_type currently not support 3"),
    (dict(flag=False), "expert_tokens_num_flag currently support True"),
    (dict(rng=(-1, 3)), "expert_start should be greater than or equal to 0"),
    (dict(rng=(3, 3)), "expert_start should be less than expert_end"),
    (dict(rng=(0, 5)), "expert_end should be less than or equal to 4"),
    (dict(rng=(0, 1, 2)), "dim number of expert_range should be 2"),
    (dict(quant=0), "quant_mode currently support -1 or 1"),
    (dict(quant=1), "not INT8"),                                   # dynamic quantisation needs float rows
    (dict(quant=1, x_dtype=BF16, ex_dtype=BF16, scale_shape=(4, 16)), "expandedXOut must be INT8"),
    (dict(quant=1, x_dtype=BF16, ex_dtype=I8, scale_shape=(8,)), "dim number of scale should be 2"),
    (dict(quant=1, x_dtype=BF16, ex_dtype=I8, scale_shape=(3, 16)), "first dim of scale should be 4"),
    (dict(quant=1, x_dtype=BF16, ex_dtype=I8, scale_shape=(4, 15)), "second dim of scale should be 16"),
    (dict(row_idx_type=2), "row_idx_type currently support 1 or 0"),
    (dict(scale_shape=(9,)), "first dim of scale should be 8"),
    (dict(scale_shape=(8, 1)), "dim number of scale should be 1"),
    (dict(ex_shape=(15, 16)), "expandedXOut must be [16, 16]"),
    (dict(ex_dtype=F32), "expandedXOut dtype"),
    (dict(ri_shape=(15,)), "expandedRowIdxOut must be INT32 [16]"),
    (dict(cnt_dtype=I32), "must be INT64"),
    (dict(cnt_shape=(5,)), "expertTokensCountOrCumsumOut must be [4]"),
    (dict(num_type=2, cnt_shape=(4,)), "[4, 2] in KEY_VALUE mode"),
    (dict(E=4096), "at most 2048 active experts"),
])
def test_routing_v3_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnMoeInitRoutingV3", _routing_v3_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_routing_v3_nulls(aclnn):
    for pos in (0, 1, 13, 14, 15):
        args = _routing_v3_args(aclnn)
        args[pos] = None
        assert _status(aclnn, "aclnnMoeInitRoutingV3", args)[0] == NULLPTR, pos
    args = _routing_v3_args(aclnn)
    args[16] = None                      # scale given, no place for the routed scales
    assert _status(aclnn, "aclnnMoeInitRoutingV3", args)[0] == NULLPTR
    args = _routing_v3_args(aclnn, quant=1, x_dtype=BF16, ex_dtype=I8, with_scale=False)   # quantisation always emits scales
    assert _status(aclnn, "aclnnMoeInitRoutingV3", args)[0] == NULLPTR


# ------------------------------------------------------------------------------------------------ SwiGLU quant
def _swiglu_args(aclnn, M=192, K=2048, N=2048, E=4, **over):
    x = T(aclnn, over.get("x_shape", (M, K)), over.get("x_dtype", I8))
    w = T(aclnn, over.get("w_shape", (E, K, N)), over.get("w_dtype", I8), over.get("w_strides"), fmt=over.get("w_fmt", 2),
          storage=over.get("w_storage"))
    ws = T(aclnn, over.get("ws_shape", (E, N)), over.get("ws_dtype", F32))
    xs = T(aclnn, over.get("xs_shape", (M,)), F32)
    gl = T(aclnn, (over.get("gl_len", E),), over.get("gl_dtype", I64))
    out = T(aclnn, over.get("out_shape", (M, N // 2)), I8)
    outs = T(aclnn, (M,), F32)
    return [x.h, w.h, None, None, ws.h, xs.h, gl.h, out.h, outs.h, None]


def test_swiglu_valid(aclnn):
    # shape of the reference op_api unit test, plus the widenings of this build
    for kw in [dict(), dict(ws_dtype=BF16), dict(ws_dtype=F16), dict(gl_dtype=I32), dict(N=28672, K=4096, M=64, E=2),
               dict(w_strides=[2048 * 2048, 1, 2048]), dict(gl_len=3)]:
        code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, **kw))
        assert code == 0, (kw, ws)
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=16, K=256, N=512, E=4))
    assert code == 0 and ws >= 16 * 256 * 4  # S workspace [M, N/2] fp32 plus tables


def test_swiglu_workspace_is_capped(aclnn, monkeypatch):
    """The fp32 SwiGLU workspace holds one band of rows: 512 MiB of it at most by default, whatever M is, and what
    OPAPI_SWIGLU_WORKSPACE_MB says otherwise (never less than one tile of rows)."""
    M, N = 1 << 20, 8192                                   # S for every row at once would be 16 GiB
    tables = M * 4 * (N // 256) + (M // 32 + 8) * 16 + (1 << 16)   # row maxima per n-tile, m-tile table, header
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=M, K=1024, N=N, E=8))
    assert code == 0 and (512 << 20) - 256 * (N // 2) * 4 <= ws <= (512 << 20) + tables
    monkeypatch.setenv("OPAPI_SWIGLU_WORKSPACE_MB", "64")
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=M, K=1024, N=N, E=8))
    assert code == 0 and (64 << 20) - 256 * (N // 2) * 4 <= ws <= (64 << 20) + tables
    monkeypatch.setenv("OPAPI_SWIGLU_WORKSPACE_MB", "1")   # less than one tile of rows: one tile of rows it is
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=4096, K=1024, N=28672, E=2))
    assert code == 0 and ws >= 32 * (28672 // 2) * 4
    small = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=16, K=256, N=512, E=4))[1]
    monkeypatch.delenv("OPAPI_SWIGLU_WORKSPACE_MB")
    assert small == _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=16, K=256, N=512, E=4))[1]


@pytest.mark.parametrize("kw,fragment", [
    (dict(x_dtype=F16), "A8W8"),
    (dict(w_fmt=29), "storageShape for second input (weight) must be 5"),          # NZ format over plain 3-D storage
    (dict(w_fmt=29, w_shape=(4, 64, 128, 16, 16)), "last two dims (16, 32)"),
    (dict(w_fmt=29, w_shape=(4, 64, 127, 16, 32)), "does not match x"),
    (dict(w_fmt=29, w_storage=(4, 64, 127, 16, 32)), "blocked weight storage must be [4, 64, 128, 16, 32]"),
    (dict(w_fmt=4), "ND or FRACTAL_NZ"),
    (dict(N=2047, out_shape=(192, 1023), ws_shape=(4, 2047)), "must even number"),
    (dict(ws_shape=(4, 2046)), "weightScale must be"),
    (dict(xs_shape=(191,)), "xScale must be"),
    (dict(out_shape=(192, 2048)), "output must be"),
    (dict(gl_len=5), "Length of 'groupList' out of range"),
    (dict(K=65536, w_shape=(4, 65536, 2048)), "need lower than"),
    (dict(w_shape=(4, 1024, 2048)), "does not match x"),
    (dict(w_strides=[2048 * 2048, 4096, 2]), "contiguous"),
])
def test_swiglu_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_swiglu_nz_weight_forms(aclnn):
    """The FRACTAL_NZ weight of the reference: 5-D [E, N/32, K/16, 16, 32], or a 3-D view over such storage; through the
    WeightNZ entry point the format field does not matter but the storage shape must be the blocked one."""
    nz5 = dict(w_fmt=29, w_shape=(4, 64, 128, 16, 32))
    nz3 = dict(w_fmt=29, w_storage=(4, 64, 128, 16, 32))
    for api, kw in [("aclnnGroupedMatmulSwigluQuant", nz5), ("aclnnGroupedMatmulSwigluQuant", nz3),
                    ("aclnnGroupedMatmulSwigluQuantWeightNZ", dict(nz5, w_fmt=2)),
                    ("aclnnGroupedMatmulSwigluQuantWeightNZ", dict(nz3, w_fmt=2))]:
        code, ws = _status(aclnn, api, _swiglu_args(aclnn, **kw))
        assert code == 0, (api, kw, ws)
    code, msg = _status(aclnn, "aclnnGroupedMatmulSwigluQuantWeightNZ", _swiglu_args(aclnn))     # plain ND storage
    assert code == INVALID and "storageShape" in msg


def test_swiglu_null_and_empty(aclnn):
    args = _swiglu_args(aclnn)
    args[4] = None
    assert _status(aclnn, "aclnnGroupedMatmulSwigluQuant", args)[0] == NULLPTR
    # an empty groupList is a successful no-op with no workspace
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, gl_len=0))
    assert code == 0 and ws == 0


# ------------------------------------------------------------------------------------------------ grouped matmul V4
def _gmm_args(aclnn, M=64, K=256, N=128, E=4, scale_dtype=F32, out_dtype=BF16, per_token=True, **over):
    x = _tl(aclnn, [T(aclnn, (M, K), over.get("x_dtype", I8))])
    w = _tl(aclnn, [T(aclnn, over.get("w_shape", (E, K, N)), I8)])
    scale = _tl(aclnn, [T(aclnn, (E, N), scale_dtype)]) if scale_dtype is not None else None
    pt = _tl(aclnn, [T(aclnn, over.get("pt_shape", (M,)), F32)]) if per_token else None
    gl = T(aclnn, over.get("gl_shape", (over.get("gl_len", E),)), over.get("gl_dtype", I64))
    out = _tl(aclnn, [T(aclnn, over.get("out_shape", (M, N)), out_dtype)])
    args = [x, w, over.get("bias"), scale, over.get("offset"), None, None, pt, gl.h if over.get("with_gl", True) else None,
            over.get("act_in"), None, None, over.get("split_item", 3), over.get("group_type", 0),
            over.get("group_list_type", 0), over.get("act_type", 0), out, None, None]
    return args


def test_gmm_valid(aclnn):
    for kw in [dict(), dict(scale_dtype=BF16), dict(out_dtype=F16), dict(scale_dtype=None, out_dtype=I32, per_token=False),
               dict(group_list_type=1), dict(split_item=2), dict(gl_dtype=I32), dict(per_token=False),
               dict(group_list_type=2, gl_shape=(4, 2))]:
        code, ws = _status(aclnn, "aclnnGroupedMatmulV4", _gmm_args(aclnn, **kw))
        assert code == 0, (kw, ws)


def test_gmm_empty_optional_means_absent(aclnn):
    # a shape-[0] per-token scale inside a list is "absent" (the reference's graph bridge passes it that way)
    args = _gmm_args(aclnn, per_token=False)
    args[7] = _tl(aclnn, [T(aclnn, (0,), F32)])
    assert _status(aclnn, "aclnnGroupedMatmulV4", args)[0] == 0


@pytest.mark.parametrize("kw,fragment", [
    (dict(x_dtype=F16), "INT8"),
    (dict(scale_dtype=BF16, out_dtype=F16), "scale/output dtype pair"),
    (dict(scale_dtype=None, out_dtype=BF16, per_token=False), "must be INT32"),
    (dict(group_type=2), "groupType 0"),
    (dict(split_item=0), "splitItem 2 or 3"),
    (dict(group_list_type=2), "groupList dim only support 1 or 2(only when groupListType is 2)"),
    (dict(group_list_type=2, gl_shape=(4, 3)), "[e, 2] pairs"),
    (dict(group_list_type=1, gl_shape=(4, 2)), "groupList dim only support 1 or 2(only when groupListType is 2)"),
    (dict(group_list_type=3), "groupListType"),
    (dict(act_type=3), "GELU_ERR_FUNC"),
    (dict(act_type=1), "actType 1"),
    (dict(gl_len=3), "should be equal to weight dim 0"),
    (dict(pt_shape=(63,)), "perTokenScale must be"),
    (dict(out_shape=(64, 127)), "y must be"),
    (dict(with_gl=False), "groupListOptional(tensor) is required"),
])
def test_gmm_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnGroupedMatmulV4", _gmm_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_gmm_reserved_arguments_and_nulls(aclnn):
    args = _gmm_args(aclnn)
    args[9] = _tl(aclnn, [T(aclnn, (4,), F32)])
    code, msg = _status(aclnn, "aclnnGroupedMatmulV4", args)
    assert code == INVALID and "activationInputOptional must be nullptr" in msg
    args = _gmm_args(aclnn)
    args[0] = None
    assert _status(aclnn, "aclnnGroupedMatmulV4", args)[0] == NULLPTR
    args = _gmm_args(aclnn)
    args[16] = None
    assert _status(aclnn, "aclnnGroupedMatmulV4", args)[0] == NULLPTR


def test_gmm_v5_takes_a_tuning_hint(aclnn):
    """V5 = V4 + tuningConfigOptional (absent, empty or a positive expected-rows hint); same validation as V4."""
    lib = aclnn.lib()
    for values in (None, [], [64], [4096, 1]):
        args = _gmm_args(aclnn)
        arr = None
        if values is not None:
            buf = (ctypes.c_int64 * max(len(values), 1))(*values)
            arr = lib.aclCreateIntArray(buf, len(values))
        args = args[:16] + [arr] + args[16:]
        code, ws = _status(aclnn, "aclnnGroupedMatmulV5", args)
        assert code == 0 and ws > 0, (values, ws)
    args = _gmm_args(aclnn, group_type=2)
    args = args[:16] + [None] + args[16:]
    code, msg = _status(aclnn, "aclnnGroupedMatmulV5", args)
    assert code == INVALID and "groupType 0" in msg


# ------------------------------------------------------------------------------------------------ fused combine
def _combine_args(aclnn, M=64, K=256, N=128, E=4, batch=16, version=3, **over):
    x = T(aclnn, (M, K), over.get("x_dtype", I8))
    w = T(aclnn, over.get("w_shape", (E, K, N)), over.get("w_dtype", I8), fmt=over.get("w_fmt", 2))
    scale = T(aclnn, over.get("scale_shape", (E, N)), over.get("scale_dtype", F32))
    bias = T(aclnn, over.get("bias_shape", (E, N)), over.get("bias_dtype", BF16)) if over.get("with_bias", True) else None
    pt = T(aclnn, over.get("pt_shape", (M,)), F32) if over.get("with_pt", True) else None
    gl = T(aclnn, (over.get("gl_len", E),), over.get("gl_dtype", I64))
    shared = T(aclnn, over.get("shared_shape", (4, N)), over.get("shared_dtype", BF16)) if over.get("with_shared", True) else None
    logit = T(aclnn, over.get("logit_shape", (M,)), F32) if over.get("with_logit", True) else None
    ri = T(aclnn, over.get("ri_shape", (M,)), over.get("ri_dtype", I64))
    out = T(aclnn, over.get("out_shape", (batch, N)), over.get("out_dtype", F32))
    head = [x.h, w.h, scale.h, bias.h if bias else None]
    tail = [pt.h if pt else None, gl.h, shared.h if shared else None, logit.h if logit else None, ri.h,
            over.get("dtype", 0), 1.0, over.get("shared_offset", 0), over.get("tx", False), over.get("tw", False),
            over.get("group_list_type", 1)]
    extra = [over.get("offset"), over.get("anti"), None]
    if version == 1:
        return "aclnnGroupedMatmulFinalizeRouting", head + tail + [out.h]
    if version == 2:
        return "aclnnGroupedMatmulFinalizeRoutingV2", head + extra + tail + [out.h]
    tuning = over.get("tuning")
    arr = None if tuning is None else aclnn.lib().aclCreateIntArray((ctypes.c_int64 * len(tuning))(*tuning), len(tuning))
    return "aclnnGroupedMatmulFinalizeRoutingV3", head + extra + tail + [arr, out.h]


def test_combine_valid(aclnn):
    for kw in [dict(), dict(version=1), dict(version=2), dict(scale_dtype=BF16), dict(scale_shape=(4, 1, 128)),
               dict(with_bias=False, with_pt=False, with_shared=False, with_logit=False), dict(bias_dtype=F32),
               dict(ri_dtype=I32), dict(gl_dtype=I32), dict(group_list_type=0), dict(shared_dtype=F16, shared_offset=12),
               dict(tuning=[16]), dict(batch=64), dict(batch=0, with_shared=False)]:
        api, args = _combine_args(aclnn, **kw)
        code, ws = _status(aclnn, api, args)
        assert code == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    # rules of gmm/grouped_matmul_finalize_routing/op_host/op_api/aclnn_grouped_matmul_finalize_routing.cpp
    (dict(dtype=1), "dtype must be 0"),
    (dict(tx=True), "transpose should be false"),
    (dict(tw=True), "transpose should be false"),
    (dict(w_dtype=I32, w_shape=(4, 256, 16)), "INT4 weights"),
    (dict(w_fmt=29), "x2's format is not NZ"),                     # NZ format over plain 3-D storage
    (dict(w_fmt=4), "format should be ND or FRACTAL_NZ"),
    (dict(x_dtype=BF16), "x1 must be INT8"),
    (dict(scale_dtype=I64), "scale must be FLOAT or BF16"),
    (dict(scale_shape=(3, 128)), "Scale fisrt dim should equal to weight EDim 4, but actual is 3"),
    (dict(bias_shape=(4, 127)), "bias's dim value should be (e, n)"),
    (dict(pt_shape=(63,)), "pertokenScale fisrt dim should equal to x MDim 64"),
    (dict(gl_len=5), "groupList fisrt dim should equal to weight EDim 4"),
    (dict(logit_shape=(65,)), "logit fisrt dim should equal to x MDim 64"),
    (dict(ri_shape=(60,)), "rowIndex fisrt dim should equal to x MDim 64"),
    (dict(ri_dtype=F32), "rowIndex must be INT64 or INT32"),
    (dict(batch=65), "Out 1st dim should be less than or equal to x MDim"),
    (dict(out_shape=(16, 64)), "Out 2nd dim"),
    (dict(out_dtype=BF16), "out must be FLOAT"),
    (dict(shared_offset=-1), "sharedInputOffset should bigger than or equal to 0"),
    (dict(shared_offset=13), "exceeds outputBS 16"),
    (dict(shared_shape=(17, 128)), "less than or equal to outputBS 16"),
    (dict(group_list_type=2), "groupListType should be 0 or 1"),
    (dict(w_shape=(4, 255, 128)), "k dim"),
    (dict(tuning=[-1]), "Invalid tuningConfigOptional (-1)"),
    (dict(version=2, offset=1), "offset belongs to the INT4 case"),
])
def test_combine_invalid(aclnn, kw, fragment):
    if kw.get("offset") == 1:
        kw = dict(kw, offset=T(aclnn, (4, 1, 128), F32).h)
    api, args = _combine_args(aclnn, **kw)
    code, msg = _status(aclnn, api, args)
    assert code == INVALID and fragment in msg, (code, msg)


def test_combine_nulls(aclnn):
    for pos in (0, 1, 2):
        api, args = _combine_args(aclnn)
        args[pos] = None
        assert _status(aclnn, api, args)[0] == NULLPTR, pos
    api, args = _combine_args(aclnn)
    args[-1] = None                                             # out
    assert _status(aclnn, api, args)[0] == NULLPTR
    api, args = _combine_args(aclnn, version=2, anti=T(aclnn, (4, 128), F32).h)   # antiquant arguments are not enabled
    assert _status(aclnn, api, args)[0] == NULLPTR


def test_reference_examples_compile_and_link_unmodified():
    """The reference's example programs for the operators built here build against include/ and link to
    libcust_opapi.so without a change (needs the reference checkout; the binaries are run by the GPU tests)."""
    import subprocess
    if not os.path.isdir("/root/reference/moe/moe_init_routing_v2/examples"):
        pytest.skip("reference sources are not present on this machine")
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-B", "ref_examples"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout
    for name in ("test_aclnn_moe_init_routing_v2", "test_aclnn_grouped_matmul_swiglu_quant", "test_aclnn_grouped_matmul",
                 "test_aclnn_moe_finalize_routing_v2", "test_aclnn_moe_init_routing_v3",
                 "test_aclnn_moe_gating_top_k_softmax_v2", "test_aclnn_moe_init_routing_quant_v2"):
        assert os.access(os.path.join(ROOT, "oracle", "_ref", "examples", name), os.X_OK), name


# ------------------------------------------------------------------------------------------------ finalize
def _fin_args(aclnn, T_=12, K=2, H=7, E=3, mode=0, dtype=F32, **over):
    ex = T(aclnn, over.get("ex_shape", (T_ * K, H) if mode in (0, 2) else (E, 4, H)), dtype)
    idx = T(aclnn, over.get("idx_shape", (T_ * K,)), I32)
    x1 = T(aclnn, over.get("x1_shape", (T_, H)), dtype) if over.get("x1", True) else None
    x2 = T(aclnn, (T_, H), dtype) if over.get("x2", True) else None
    bias = T(aclnn, over.get("bias_shape", (E, H)), dtype) if over.get("bias", True) else None
    scales = T(aclnn, (T_, K), over.get("scale_dtype", dtype)) if over.get("scales", True) else None
    eidx = T(aclnn, over.get("eidx_shape", (T_, K)), I32) if over.get("eidx", True) else None
    out = T(aclnn, over.get("out_shape", (T_, H)), over.get("out_dtype", dtype))
    return [ex.h, idx.h, x1.h if x1 else None, x2.h if x2 else None, bias.h if bias else None,
            scales.h if scales else None, eidx.h if eidx else None, mode, out.h]


def test_finalize_valid(aclnn):
    for kw in [dict(), dict(mode=2), dict(mode=1), dict(mode=3), dict(dtype=BF16), dict(dtype=BF16, scale_dtype=F32),
               dict(dtype=F16), dict(x1=False, x2=False, bias=False, eidx=False), dict(scales=False, K=1),
               dict(T_=1024, K=4, H=30, E=10)]:
        code, ws = _status(aclnn, "aclnnMoeFinalizeRoutingV2", _fin_args(aclnn, **kw))
        assert code == 0 and ws == 0, (kw, ws)


@pytest.mark.parametrize("kw,fragment", [
    (dict(mode=4), "drop_pad_mode should be [0,3]"),
    (dict(mode=0, ex_shape=(3, 4, 7)), "2D tensor when drop_pad_mode is 0 or 2"),
    (dict(mode=1, ex_shape=(24, 7)), "3D tensor when drop_pad_mode is 1 or 3"),
    (dict(x1=False), "x2 parameter can't be inputted either"),
    (dict(eidx=False), "expert_idx must exist when bias exist"),
    (dict(x1_shape=(11, 7)), "dim 0 of x1"),
    (dict(bias_shape=(3, 8)), "dim 1 of bias"),
    (dict(bias_shape=(1, 7)), "E should be larger than or equal to K"),
    (dict(eidx_shape=(12, 3)), "dim 1 of expert_idx"),
    (dict(out_dtype=F16), "dtype of y should be same"),
    (dict(out_shape=(12, 8)), "dim 1 of output"),
    (dict(dtype=F16, scale_dtype=F32), "scales dtype"),
])
def test_finalize_invalid(aclnn, kw, fragment):
    code, msg = _status(aclnn, "aclnnMoeFinalizeRoutingV2", _fin_args(aclnn, **kw))
    assert code == INVALID and fragment in msg, (code, msg)


def test_second_phase_rejects_bad_workspace(aclnn):
    """Phase 2 checks its arguments before touching the device."""
    lib = aclnn.lib()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = lib.aclnnMoeInitRoutingV2GetWorkspaceSize(*_routing_args(aclnn, flag=1), ctypes.byref(ws), ctypes.byref(ex))
    assert st == 0 and ws.value > 0
    st = lib.aclnnMoeInitRoutingV2(None, ws.value, ex, None)   # null workspace although bytes are required
    assert st == NULLPTR
    assert lib.aclnnMoeInitRoutingV2(None, 0, None, None) == NULLPTR  # null executor


# ------------------------------------------------------------------------------------------------ negative extents
def test_negative_extents_are_rejected_everywhere(aclnn):
    """Shapes are caller data: a set of tensors that agree with each other on a negative extent is still refused."""
    cases = [
        ("aclnnMoeInitRoutingV2", _routing_args(aclnn, T_=-4)),
        ("aclnnMoeInitRoutingQuantV2", _routing_quant_v2_args(aclnn, T_=-4)),
        ("aclnnMoeInitRoutingV3", _routing_v3_args(aclnn, T_=-4, active=-1)),
        ("aclnnMoeGatingTopKSoftmaxV2", _gating_args(aclnn, shape=(-6, 16))),
        ("aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=-192)),
        ("aclnnGroupedMatmulV4", _gmm_args(aclnn, M=-64)),
        _combine_args(aclnn, M=-64),
        ("aclnnMoeFinalizeRoutingV2", _fin_args(aclnn, T_=-12)),
    ]
    for api, args in cases:
        code, msg = _status(aclnn, api, args)
        assert code == INVALID and "negative extent" in msg, (api, code, msg)


# ------------------------------------------------------------------------------------------------ strided inputs
def test_strided_inputs_are_staged_in_the_workspace(aclnn):
    """A non-contiguous input costs a contiguous copy in the workspace (rounded up to 256 bytes); outputs must stay
    contiguous; negative strides are refused."""
    T_, K, H = 12, 2, 7
    base = _fin_args(aclnn, T_=T_, K=K, H=H)
    code, ws0 = _status(aclnn, "aclnnMoeFinalizeRoutingV2", base)
    assert code == 0 and ws0 == 0
    args = _fin_args(aclnn, T_=T_, K=K, H=H)
    args[0] = T(aclnn, (T_ * K, H), F32, strides=[2 * H, 1]).h          # expandedX: every row twice as far apart
    code, ws = _status(aclnn, "aclnnMoeFinalizeRoutingV2", args)
    assert code == 0 and ws == (T_ * K * H * 4 + 255) // 256 * 256
    args = _fin_args(aclnn, T_=T_, K=K, H=H)
    args[-1] = T(aclnn, (T_, H), F32, strides=[2 * H, 1]).h             # out
    code, msg = _status(aclnn, "aclnnMoeFinalizeRoutingV2", args)
    assert code == INVALID and "out must be contiguous" in msg
    args = _fin_args(aclnn, T_=T_, K=K, H=H)
    args[0] = T(aclnn, (T_ * K, H), F32, strides=[H, -1]).h
    code, msg = _status(aclnn, "aclnnMoeFinalizeRoutingV2", args)
    assert code == INVALID and "negative strides" in msg

    own = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", _swiglu_args(aclnn, M=16, K=256, N=512, E=4))[1]
    args = _swiglu_args(aclnn, M=16, K=256, N=512, E=4)
    args[0] = T(aclnn, (16, 256), I8, strides=[512, 1]).h                # x
    code, ws = _status(aclnn, "aclnnGroupedMatmulSwigluQuant", args)
    assert code == 0 and ws == (own + 255) // 256 * 256 + 16 * 256
