"""ctypes binding of libcust_opapi.so and Python-level operators mirroring the reference interface.

Each operator follows the reference's two-phase protocol exactly as a C caller would: build ``aclTensor`` descriptors
over caller-owned device memory, call ``aclnn<Op>GetWorkspaceSize``, allocate the workspace, call ``aclnn<Op>`` on the
current HIP stream.  A non-zero status raises :class:`AclnnError` carrying the code and ``aclGetRecentErrMsg()``.

There is no fallback: if the shared library is missing, importing an operator fails with instructions to build it.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.environ.get("OPAPI_LIBRARY_PATH") or os.path.join(_HERE, "lib", "libcust_opapi.so")

ACL_FLOAT, ACL_FLOAT16, ACL_INT8, ACL_INT32, ACL_INT64, ACL_BOOL, ACL_BF16 = 0, 1, 2, 3, 9, 12, 27
ACL_FORMAT_ND = 2
ACL_FORMAT_FRACTAL_NZ = 29

ACLNN_SUCCESS = 0
ACLNN_ERR_PARAM_NULLPTR = 161001
ACLNN_ERR_PARAM_INVALID = 161002
ACLNN_ERR_RUNTIME_ERROR = 361001

_DTYPE_CODE = {
    torch.float32: ACL_FLOAT,
    torch.float16: ACL_FLOAT16,
    torch.int8: ACL_INT8,
    torch.int32: ACL_INT32,
    torch.int64: ACL_INT64,
    torch.bfloat16: ACL_BF16,
    torch.bool: ACL_BOOL,
}


class AclnnError(RuntimeError):
    def __init__(self, api, code, message):
        super().__init__("%s failed with status %d: %s" % (api, code, message))
        self.api = api
        self.code = code
        self.message = message


def library_path():
    return _LIB_PATH


_lib = None

_VP = ctypes.c_void_p
_I64 = ctypes.c_int64
_U64P = ctypes.POINTER(ctypes.c_uint64)
_VPP = ctypes.POINTER(ctypes.c_void_p)

_PHASE1_SIGNATURES = {
    "aclnnMoeInitRoutingV2GetWorkspaceSize":
        [_VP, _VP, _I64, _I64, _I64, _I64, _I64, ctypes.c_bool, _VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnMoeInitRoutingQuantV2GetWorkspaceSize":
        [_VP, _VP, _VP, _VP, _I64, _I64, _I64, _I64, _I64, ctypes.c_bool, _I64, _VP, _VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnMoeGatingTopKSoftmaxV2GetWorkspaceSize":
        [_VP, _VP, _I64, _I64, ctypes.c_bool, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnMoeInitRoutingV3GetWorkspaceSize":
        [_VP, _VP, _VP, _VP, _I64, _I64, _I64, _I64, _I64, ctypes.c_bool, _I64, _VP, _I64, _VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulSwigluQuantGetWorkspaceSize":
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulSwigluQuantWeightNZGetWorkspaceSize":
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulV4GetWorkspaceSize":
        [_VP] * 12 + [_I64, _I64, _I64, _I64] + [_VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulV5GetWorkspaceSize":
        [_VP] * 12 + [_I64, _I64, _I64, _I64] + [_VP, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulWeightNzGetWorkspaceSize":
        [_VP] * 12 + [_I64, _I64, _I64, _I64] + [_VP, _I64, _VP, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulFinalizeRoutingV3GetWorkspaceSize":
        [_VP] * 12 + [_I64, ctypes.c_float, _I64, ctypes.c_bool, ctypes.c_bool, _I64, _VP, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulFinalizeRoutingV2GetWorkspaceSize":
        [_VP] * 12 + [_I64, ctypes.c_float, _I64, ctypes.c_bool, ctypes.c_bool, _I64, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulFinalizeRoutingGetWorkspaceSize":
        [_VP] * 9 + [_I64, ctypes.c_float, _I64, ctypes.c_bool, ctypes.c_bool, _I64, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulFinalizeRoutingWeightNzGetWorkspaceSize":
        [_VP] * 9 + [_I64, ctypes.c_float, _I64, ctypes.c_bool, ctypes.c_bool, _I64, _VP, _U64P, _VPP],
    "aclnnGroupedMatmulFinalizeRoutingWeightNzV2GetWorkspaceSize":
        [_VP] * 12 + [_I64, ctypes.c_float, _I64, ctypes.c_bool, ctypes.c_bool, _I64, _VP, _VP, _U64P, _VPP],
    "aclnnMoeFinalizeRoutingV2GetWorkspaceSize":
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _VP, _U64P, _VPP],
}
_PHASE2 = ["aclnnMoeInitRoutingQuantV2", "aclnnGroupedMatmulSwigluQuantWeightNZ", "aclnnGroupedMatmulWeightNz",
           "aclnnGroupedMatmulFinalizeRoutingWeightNz", "aclnnGroupedMatmulFinalizeRoutingWeightNzV2", "aclnnGroupedMatmulFinalizeRouting", "aclnnGroupedMatmulFinalizeRoutingV2", "aclnnGroupedMatmulFinalizeRoutingV3",
           "aclnnMoeGatingTopKSoftmaxV2", "aclnnMoeInitRoutingV2", "aclnnMoeInitRoutingV3", "aclnnGroupedMatmulSwigluQuant", "aclnnGroupedMatmulV4", "aclnnGroupedMatmulV5",
           "aclnnMoeFinalizeRoutingV2"]


def lib():
    """The loaded C-ABI library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python ops-transformer_amd/build.py` (hipcc, gfx950). "
                "There is no CPU or PyTorch fallback for these operators." % _LIB_PATH)
        l = ctypes.CDLL(_LIB_PATH)
        for name, sig in _PHASE1_SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = sig
            fn.restype = ctypes.c_int32
        for name in _PHASE2:
            fn = getattr(l, name)
            fn.argtypes = [_VP, ctypes.c_uint64, _VP, _VP]
            fn.restype = ctypes.c_int32
        l.aclnnMoeInitRoutingV2StaticWorkspace.argtypes = [_VP, _VP]
        l.aclnnMoeInitRoutingV2StaticWorkspace.restype = ctypes.c_int32
        l.aclCreateTensor.argtypes = [ctypes.POINTER(_I64), ctypes.c_uint64, ctypes.c_int, ctypes.POINTER(_I64), _I64,
                                      ctypes.c_int, ctypes.POINTER(_I64), ctypes.c_uint64, _VP]
        l.aclCreateTensor.restype = _VP
        l.aclDestroyTensor.argtypes = [_VP]
        l.aclCreateTensorList.argtypes = [ctypes.POINTER(_VP), ctypes.c_uint64]
        l.aclCreateTensorList.restype = _VP
        l.aclDestroyTensorList.argtypes = [_VP]
        l.aclDestroyAclOpExecutor.argtypes = [_VP]
        l.aclCreateIntArray.argtypes = [ctypes.POINTER(_I64), ctypes.c_uint64]
        l.aclCreateIntArray.restype = _VP
        l.aclDestroyIntArray.argtypes = [_VP]
        l.aclGetRecentErrMsg.restype = ctypes.c_char_p
        _lib = l
    return _lib


def last_error():
    return lib().aclGetRecentErrMsg().decode("utf-8", "replace")


# ------------------------------------------------------------------------------------------------ descriptors
def create_tensor(shape, dtype_code, data_ptr, strides=None, offset=0, fmt=ACL_FORMAT_ND, storage_shape=None):
    """Raw aclCreateTensor; the caller destroys the handle (or hands it to a tensor list)."""
    n = len(shape)
    dims = (_I64 * max(n, 1))(*shape)
    storage = list(shape) if storage_shape is None else list(storage_shape)
    sdims = (_I64 * max(len(storage), 1))(*storage)
    if strides is None:
        strides = [1] * n
        for i in range(n - 2, -1, -1):
            strides[i] = strides[i + 1] * shape[i + 1]
    st = (_I64 * max(n, 1))(*strides)
    h = lib().aclCreateTensor(dims, n, dtype_code, st, offset, fmt, sdims, len(storage), _VP(data_ptr))
    if not h:
        raise MemoryError("aclCreateTensor failed")
    return h


def tensor_of(t):
    """aclTensor over a torch tensor's memory with its own sizes and strides (no copy)."""
    if t is None:
        return None
    return create_tensor(list(t.shape), _DTYPE_CODE[t.dtype], t.data_ptr(), list(t.stride()))


class _Handles:
    """Owns descriptor handles for the duration of one operator call."""

    def __init__(self):
        self.tensors = []
        self.lists = []
        self.int_arrays = []

    def tensor(self, t):
        if t is None:
            return None
        h = tensor_of(t)
        self.tensors.append(h)
        return h

    def raw(self, handle):
        """Takes ownership of a handle made with create_tensor."""
        self.tensors.append(handle)
        return handle

    def tensor_list(self, ts):
        if ts is None:
            return None
        hs = [tensor_of(t) for t in ts]
        arr = (_VP * max(len(hs), 1))(*hs)
        h = lib().aclCreateTensorList(arr, len(hs))
        self.lists.append(h)  # the list owns its tensors
        return h

    def int_array(self, values):
        if values is None:
            return None
        arr = (_I64 * max(len(values), 1))(*values)
        h = lib().aclCreateIntArray(arr, len(values))
        self.int_arrays.append(h)
        return h

    def close(self):
        l = lib()
        for h in self.int_arrays:
            l.aclDestroyIntArray(h)
        self.int_arrays = []
        for h in self.tensors:
            l.aclDestroyTensor(h)
        for h in self.lists:
            l.aclDestroyTensorList(h)
        self.tensors, self.lists = [], []


class Workspace:
    """A device scratch buffer reused across operator calls; grows to the largest size any call asked for."""

    def __init__(self):
        self.tensor = None
        self.requested = {}  # operator name -> largest workspace size its first phase has asked for

    def reserve(self, nbytes, device, api=None):
        if api is not None:
            self.requested[api] = max(self.requested.get(api, 0), int(nbytes))
        if self.tensor is None or self.tensor.numel() < nbytes:
            self.tensor = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return self.tensor


def _stream_ptr():
    return torch.cuda.current_stream().cuda_stream


def _run_two_phase(api, args, device, workspace=None, static_workspace_api=None):
    """args: phase-1 arguments without the two trailing out-parameters.

    static_workspace_api names a second phase that takes (executor, stream) only and keeps its scratch inside the
    library: no workspace is allocated or passed."""
    l = lib()
    ws_size = ctypes.c_uint64(0)
    executor = ctypes.c_void_p(None)
    st = getattr(l, api + "GetWorkspaceSize")(*args, ctypes.byref(ws_size), ctypes.byref(executor))
    if st != ACLNN_SUCCESS:
        raise AclnnError(api + "GetWorkspaceSize", st, last_error())
    if static_workspace_api is not None:
        st = getattr(l, static_workspace_api)(executor, _VP(_stream_ptr()))
        if st != ACLNN_SUCCESS:
            raise AclnnError(static_workspace_api, st, last_error())
        return None
    ws_ptr = None
    ws_keepalive = None
    if workspace is not None:
        workspace.requested[api] = max(workspace.requested.get(api, 0), int(ws_size.value))
    if ws_size.value > 0:
        if workspace is not None:
            ws_keepalive = workspace.reserve(ws_size.value, device)
        else:
            ws_keepalive = torch.empty(ws_size.value, dtype=torch.uint8, device=device)
        ws_ptr = ws_keepalive.data_ptr()
    st = getattr(l, api)(_VP(ws_ptr), ws_size.value, executor, _VP(_stream_ptr()))
    if st != ACLNN_SUCCESS:
        raise AclnnError(api, st, last_error())
    return ws_keepalive


def workspace_size(api, args):
    """Phase 1 only: returns the workspace byte count and releases the executor."""
    l = lib()
    ws_size = ctypes.c_uint64(0)
    executor = ctypes.c_void_p(None)
    st = getattr(l, api + "GetWorkspaceSize")(*args, ctypes.byref(ws_size), ctypes.byref(executor))
    if st != ACLNN_SUCCESS:
        raise AclnnError(api + "GetWorkspaceSize", st, last_error())
    l.aclDestroyAclOpExecutor(executor)
    return ws_size.value


# ------------------------------------------------------------------------------------------------ operators
def moe_init_routing_v2(x, expert_idx, active_num=0, expert_capacity=0, expert_num=0, drop_pad_mode=0,
                        expert_tokens_count_or_cumsum_flag=0, expert_tokens_before_capacity_flag=False, out=None,
                        workspace=None, static_workspace=False):
    """aclnnMoeInitRoutingV2.  Returns (expanded_x, expanded_row_idx, expert_tokens_count_or_cumsum | None,
    expert_tokens_before_capacity | None).  ``out`` may carry preallocated outputs in that order.
    static_workspace=True runs the second phase through aclnnMoeInitRoutingV2StaticWorkspace (no device allocation;
    with ``out`` given the call allocates nothing on the device at all)."""
    T, H = x.shape
    K = expert_idx.shape[1]
    M = T * K
    dev = x.device
    if out is not None:
        expanded_x, expanded_row_idx, count_out, before_out = out
    else:
        if drop_pad_mode == 0:
            rows = M if active_num == 0 else min(M, active_num)
            expanded_x = torch.empty((rows, H), dtype=x.dtype, device=dev)
        else:
            expanded_x = torch.empty((expert_num, expert_capacity, H), dtype=x.dtype, device=dev)
        expanded_row_idx = torch.empty((M,), dtype=torch.int32, device=dev)
        count_out = (torch.empty((expert_num,), dtype=torch.int32, device=dev)
                     if (drop_pad_mode == 0 and expert_tokens_count_or_cumsum_flag > 0) else None)
        before_out = (torch.empty((expert_num,), dtype=torch.int32, device=dev)
                      if (drop_pad_mode == 1 and expert_tokens_before_capacity_flag) else None)
    h = _Handles()
    try:
        args = [h.tensor(x), h.tensor(expert_idx), active_num, expert_capacity, expert_num, drop_pad_mode,
                expert_tokens_count_or_cumsum_flag, bool(expert_tokens_before_capacity_flag), h.tensor(expanded_x),
                h.tensor(expanded_row_idx), h.tensor(count_out), h.tensor(before_out)]
        _run_two_phase("aclnnMoeInitRoutingV2", args, dev, workspace,
                       static_workspace_api="aclnnMoeInitRoutingV2StaticWorkspace" if static_workspace else None)
    finally:
        h.close()
    return expanded_x, expanded_row_idx, count_out, before_out


def moe_init_routing_quant_v2(x, expert_idx, quant_mode, scale=None, offset=None, active_num=0, expert_capacity=0,
                              expert_num=0, drop_pad_mode=0, expert_tokens_count_or_cumsum_flag=0,
                              expert_tokens_before_capacity_flag=False, workspace=None):
    """aclnnMoeInitRoutingQuantV2.  Returns (expandedX int8, expandedRowIdx, countOrCumsum | None, beforeCapacity | None,
    dynamicQuantScale | None)."""
    T, H = x.shape
    K = expert_idx.shape[1]
    dev = x.device
    if drop_pad_mode == 1:
        expanded_x = torch.zeros((expert_num, expert_capacity, H), dtype=torch.int8, device=dev)
        rows = expert_num * expert_capacity
        count_flag, before_flag = 0, expert_tokens_before_capacity_flag
    else:
        rows = T * K if active_num == 0 else min(T * K, active_num)
        expanded_x = torch.zeros((rows, H), dtype=torch.int8, device=dev)
        count_flag, before_flag = expert_tokens_count_or_cumsum_flag, False
    row_idx = torch.empty((T * K,), dtype=torch.int32, device=dev)
    counts = torch.zeros((expert_num,), dtype=torch.int32, device=dev) if count_flag else None
    before = torch.zeros((expert_num,), dtype=torch.int32, device=dev) if before_flag else None
    dyn = torch.zeros((rows,), dtype=torch.float32, device=dev) if quant_mode == 1 else None
    h = _Handles()
    try:
        args = [h.tensor(x), h.tensor(expert_idx), h.tensor(scale), h.tensor(offset), active_num, expert_capacity,
                expert_num, drop_pad_mode, expert_tokens_count_or_cumsum_flag, expert_tokens_before_capacity_flag,
                quant_mode, h.tensor(expanded_x), h.tensor(row_idx), h.tensor(counts), h.tensor(before), h.tensor(dyn)]
        _run_two_phase("aclnnMoeInitRoutingQuantV2", args, dev, workspace)
    finally:
        h.close()
    return expanded_x, row_idx, counts, before, dyn


def moe_gating_top_k_softmax_v2(x, k, renorm=0, finished=None, output_softmax=False, out=None):
    """aclnnMoeGatingTopKSoftmaxV2.  Returns (y [..., k] in x's dtype, expertIdx int32 [..., k], softmax fp32 or None)."""
    dev = x.device
    lead = tuple(x.shape[:-1])
    if out is not None:
        y, idx, sm = out
    else:
        y = torch.empty(lead + (k,), dtype=x.dtype, device=dev)
        idx = torch.empty(lead + (k,), dtype=torch.int32, device=dev)
        sm = torch.empty(tuple(x.shape), dtype=torch.float32, device=dev) if (output_softmax and renorm == 0) else None
    h = _Handles()
    try:
        args = [h.tensor(x), h.tensor(finished), k, renorm, bool(output_softmax), h.tensor(y), h.tensor(idx), h.tensor(sm)]
        _run_two_phase("aclnnMoeGatingTopKSoftmaxV2", args, dev, None)
    finally:
        h.close()
    return y, idx, sm


def moe_init_routing_v3(x, expert_idx, scale=None, expert_num=0, expert_tokens_num_type=1, quant_mode=-1,
                        active_expert_range=None, row_idx_type=1, active_num=-1, out=None, workspace=None):
    """aclnnMoeInitRoutingV3 (dropless).  Returns (expandedX, expandedRowIdx, tokenCounts int64, expandedScale or None).
    quant_mode -1: scale is the optional per-token scale [T]; quant_mode 1 (dynamic quantisation to int8): scale is the
    optional smooth scale [active experts, H] and expandedScale is always produced."""
    T, H = x.shape
    K = expert_idx.shape[1]
    dev = x.device
    start, end = (0, expert_num) if active_expert_range is None else active_expert_range
    if out is not None:
        expanded_x, row_idx, counts, expanded_scale = out
    else:
        expanded_x = torch.zeros((T * K, H), dtype=torch.int8 if quant_mode == 1 else x.dtype, device=dev)
        row_idx = torch.empty((T * K,), dtype=torch.int32, device=dev)
        counts = torch.zeros((expert_num, 2) if expert_tokens_num_type == 2 else (end - start,), dtype=torch.int64, device=dev)
        expanded_scale = (torch.zeros((T * K,), dtype=torch.float32, device=dev)
                          if (scale is not None or quant_mode == 1) else None)
    h = _Handles()
    try:
        args = [h.tensor(x), h.tensor(expert_idx), h.tensor(scale), None, active_num, 0, expert_num, 0,
                expert_tokens_num_type, True, quant_mode,
                None if active_expert_range is None else h.int_array(list(active_expert_range)), row_idx_type,
                h.tensor(expanded_x), h.tensor(row_idx), h.tensor(counts), h.tensor(expanded_scale)]
        _run_two_phase("aclnnMoeInitRoutingV3", args, dev, workspace)
    finally:
        h.close()
    return expanded_x, row_idx, counts, expanded_scale


def nz_weight_handle(weight_nz, view_3d=False, fmt=ACL_FORMAT_FRACTAL_NZ):
    """Descriptor of a blocked weight held as a contiguous torch tensor [E, N/32, K/16, 16, 32].  view_3d: describe it
    through the 3-D view [E, K, N] over that storage (the form aclnn...WeightNZ entry points accept as well)."""
    E, n1, k1, k0, n0 = weight_nz.shape
    assert (k0, n0) == (16, 32) and weight_nz.is_contiguous()
    shape = [E, k1 * 16, n1 * 32] if view_3d else list(weight_nz.shape)
    return create_tensor(shape, _DTYPE_CODE[weight_nz.dtype], weight_nz.data_ptr(), None, 0, fmt, list(weight_nz.shape))


def grouped_matmul_swiglu_quant(x, weight, group_list, weight_scale, x_scale, bias=None, offset=None, out=None,
                                workspace=None, weight_nz=None):
    """aclnnGroupedMatmulSwigluQuant.  weight is the [E, K, N] view (contiguous, or ``storage.transpose(1, 2)`` over
    [E, N, K] storage); or pass weight=None and weight_nz=(tensor [E, N/32, K/16, 16, 32], how) with how one of
    "nz5d" (FRACTAL_NZ 5-D tensor through the plain entry point), "entry5d" / "entry3d" (through
    aclnnGroupedMatmulSwigluQuantWeightNZ, 5-D shape or 3-D view, ND format field).
    Returns (output int8 [M, N/2], output_scale fp32 [M])."""
    M = x.shape[0]
    N = weight.shape[2] if weight is not None else weight_nz[0].shape[1] * 32
    dev = x.device
    if out is not None:
        output, output_scale = out
    else:
        output = torch.empty((M, N // 2), dtype=torch.int8, device=dev)
        output_scale = torch.empty((M,), dtype=torch.float32, device=dev)
    h = _Handles()
    try:
        api = "aclnnGroupedMatmulSwigluQuant"
        if weight is not None:
            wh = h.tensor(weight)
        else:
            tensor, how = weight_nz
            if how == "nz5d":
                wh = h.raw(nz_weight_handle(tensor))
            else:
                api = "aclnnGroupedMatmulSwigluQuantWeightNZ"
                wh = h.raw(nz_weight_handle(tensor, view_3d=(how == "entry3d"), fmt=ACL_FORMAT_ND))
        args = [h.tensor(x), wh, h.tensor(bias), h.tensor(offset), h.tensor(weight_scale),
                h.tensor(x_scale), h.tensor(group_list), h.tensor(output), h.tensor(output_scale), None]
        _run_two_phase(api, args, dev, workspace)
    finally:
        h.close()
    return output, output_scale


def grouped_matmul_v4(x, weight, bias=None, scale=None, offset=None, antiquant_scale=None, antiquant_offset=None,
                      per_token_scale=None, group_list=None, activation_input=None, activation_quant_scale=None,
                      activation_quant_offset=None, split_item=0, group_type=-1, group_list_type=0, act_type=0,
                      output_dtype=None, out=None, workspace=None, tuning_config=None, weight_nz=None):
    """aclnnGroupedMatmulV4, or aclnnGroupedMatmulV5 when tuning_config (a list of ints whose first value is the expected
    number of rows per expert) is given.  x / weight / scale / per_token_scale / out are lists of tensors as in the
    reference.  weight_nz=(tensor [E, N/32, K/16, 16, 32], how) instead of weight passes a blocked weight: how "nz5d"
    (FRACTAL_NZ 5-D tensor through V4 / V5) or "entry5d" / "entry3d" (aclnnGroupedMatmulWeightNz, 5-D shape or 3-D view).
    Returns the list of outputs."""
    dev = x[0].device
    n_out = weight[0].shape[2] if weight is not None else weight_nz[0].shape[1] * 32
    if out is None:
        if output_dtype is None:
            output_dtype = torch.int32 if scale is None else (
                torch.bfloat16 if scale[0].dtype == torch.bfloat16 else torch.float16)
        out = [torch.empty((x[0].shape[0], n_out), dtype=output_dtype, device=dev)]
    h = _Handles()
    try:
        api = "aclnnGroupedMatmulV5" if tuning_config is not None else "aclnnGroupedMatmulV4"
        if weight is not None:
            wl = h.tensor_list(weight)
        else:
            tensor, how = weight_nz
            if how == "nz5d":
                wh = nz_weight_handle(tensor)
            else:
                api = "aclnnGroupedMatmulWeightNz"
                wh = nz_weight_handle(tensor, view_3d=(how == "entry3d"), fmt=ACL_FORMAT_ND)
            wl = lib().aclCreateTensorList((_VP * 1)(wh), 1)
            h.lists.append(wl)
        args = [h.tensor_list(x), wl, h.tensor_list(bias), h.tensor_list(scale),
                h.tensor_list(offset), h.tensor_list(antiquant_scale), h.tensor_list(antiquant_offset),
                h.tensor_list(per_token_scale), h.tensor(group_list), h.tensor_list(activation_input),
                h.tensor_list(activation_quant_scale), h.tensor_list(activation_quant_offset), split_item, group_type,
                group_list_type, act_type]
        if api == "aclnnGroupedMatmulWeightNz":
            args += [h.int_array(tuning_config), 0]          # tuningConfigOptional (may be null), quantGroupSize
        elif tuning_config is not None:
            args.append(h.int_array(tuning_config))
        args += [h.tensor_list(out), None, None]
        _run_two_phase(api, args, dev, workspace)
    finally:
        h.close()
    return out


def grouped_matmul_v5(x, weight, tuning_config=(), **kwargs):
    """aclnnGroupedMatmulV5: grouped_matmul_v4 plus the tuning hint (an empty list means "no hint")."""
    return grouped_matmul_v4(x, weight, tuning_config=list(tuning_config), **kwargs)


def grouped_matmul_finalize_routing(x, weight, scale, row_index, batch, group_list, group_list_type=1, bias=None,
                                    per_token_scale=None, logit=None, shared_input=None, shared_input_weight=1.0,
                                    shared_input_offset=0, tuning_config=None, out=None, workspace=None, version=3,
                                    weight_nz=None):
    """aclnnGroupedMatmulFinalizeRouting (version 1), V2 or V3: int8 grouped matmul fused with the weighted combine.
    weight is the [E, K, N] view; or weight=None and weight_nz = blocked tensor [E, N/32, K/16, 16, 32], which goes
    through aclnnGroupedMatmulFinalizeRoutingWeightNz (version 1) or WeightNzV2 (any other version) as a 3-D view.
    Returns out fp32 [batch, N]."""
    dev = x.device
    N = weight.shape[2] if weight is not None else weight_nz.shape[1] * 32
    if out is None:
        out = torch.empty((batch, N), dtype=torch.float32, device=dev)
    h = _Handles()
    try:
        wh = h.tensor(weight) if weight is not None else h.raw(nz_weight_handle(weight_nz, view_3d=True, fmt=ACL_FORMAT_ND))
        head = [h.tensor(x), wh, h.tensor(scale), h.tensor(bias)]
        tail = [h.tensor(per_token_scale), h.tensor(group_list), h.tensor(shared_input), h.tensor(logit), h.tensor(row_index),
                0, float(shared_input_weight), int(shared_input_offset), False, False, int(group_list_type)]
        if weight is None and version == 1:
            api, args = "aclnnGroupedMatmulFinalizeRoutingWeightNz", head + tail + [h.tensor(out)]
        elif weight is None:
            api = "aclnnGroupedMatmulFinalizeRoutingWeightNzV2"
            args = head + [None, None, None] + tail + [None if tuning_config is None else h.int_array(list(tuning_config)),
                                                         h.tensor(out)]
        elif version == 1:
            api, args = "aclnnGroupedMatmulFinalizeRouting", head + tail + [h.tensor(out)]
        elif version == 2:
            api, args = "aclnnGroupedMatmulFinalizeRoutingV2", head + [None, None, None] + tail + [h.tensor(out)]
        else:
            api = "aclnnGroupedMatmulFinalizeRoutingV3"
            args = head + [None, None, None] + tail + [None if tuning_config is None else h.int_array(list(tuning_config)),
                                                         h.tensor(out)]
        _run_two_phase(api, args, dev, workspace)
    finally:
        h.close()
    return out


def moe_finalize_routing_v2(expanded_x, expanded_row_idx, x1=None, x2=None, bias=None, scales=None, expert_idx=None,
                            drop_pad_mode=0, out=None):
    """aclnnMoeFinalizeRoutingV2.  Returns out [T, H] in the dtype of expanded_x."""
    K = 1 if scales is None else scales.shape[1]
    T = expanded_row_idx.shape[0] // K
    H = expanded_x.shape[-1]
    dev = expanded_x.device
    if out is None:
        out = torch.empty((T, H), dtype=expanded_x.dtype, device=dev)
    h = _Handles()
    try:
        args = [h.tensor(expanded_x), h.tensor(expanded_row_idx), h.tensor(x1), h.tensor(x2), h.tensor(bias),
                h.tensor(scales), h.tensor(expert_idx), drop_pad_mode, h.tensor(out)]
        _run_two_phase("aclnnMoeFinalizeRoutingV2", args, dev)
    finally:
        h.close()
    return out


# ------------------------------------------------------------------------------------------------ kernel timing
def kernel_timer_enable(enable=True):
    """Turns per-kernel HIP-event timing inside the library on or off (include/opapi_profile.h)."""
    l = lib()
    l.opapiKernelTimerEnable.argtypes = [ctypes.c_int]
    l.opapiKernelTimerEnable.restype = None
    l.opapiKernelTimerEnable(1 if enable else 0)


def kernel_timer_report():
    """Waits for the recorded launches and returns {kernel name: (launches, total milliseconds)}."""
    l = lib()
    l.opapiKernelTimerReport.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    l.opapiKernelTimerReport.restype = ctypes.c_int
    buf = ctypes.create_string_buffer(1 << 14)
    rc = l.opapiKernelTimerReport(buf, len(buf))
    if rc < 0:
        raise RuntimeError("opapiKernelTimerReport failed")
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, total = line.split()
        out[name] = (int(count), float(total))
    return out


def gemm_workgroup_spans_enable(enable=True):
    """Turns the recording of per-workgroup start / end times in the grouped GEMM's persistent kernels on or off."""
    l = lib()
    l.opapiGemmWorkgroupSpansEnable.argtypes = [ctypes.c_int]
    l.opapiGemmWorkgroupSpansEnable.restype = None
    l.opapiGemmWorkgroupSpansEnable(1 if enable else 0)


def gemm_workgroup_spans_report():
    """{kernel kind: {"workgroups", "tile_rows", "span_us", "xcd": [{"end_us", "busy", "tiles_min", "tiles_max"} x 8]}}
    for the last launch of each kind (include/opapi_profile.h)."""
    l = lib()
    l.opapiGemmWorkgroupSpansReport.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    l.opapiGemmWorkgroupSpansReport.restype = ctypes.c_int
    buf = ctypes.create_string_buffer(1 << 14)
    if l.opapiGemmWorkgroupSpansReport(buf, len(buf)) < 0:
        raise RuntimeError("opapiGemmWorkgroupSpansReport failed")
    out = {}
    for line in buf.value.decode().splitlines():
        f = line.split()
        rec = {"workgroups": int(f[2]), "tile_rows": int(f[4]), "span_us": float(f[6]), "xcd": []}
        i = 7
        while i < len(f):
            tmin, tmax = f[i + 6].split("-")
            rec["xcd"].append({"end_us": float(f[i + 2]), "busy": float(f[i + 4]), "tiles_min": int(tmin), "tiles_max": int(tmax)})
            i += 7
        out[f[0]] = rec
    return out


def int8_mfma_rate_probe(uniform_random_operands, iterations=20000):
    """int8 operations per second of back-to-back MFMAs on register operands (include/opapi_profile.h)."""
    l = lib()
    l.opapiInt8MfmaRateProbe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    l.opapiInt8MfmaRateProbe.restype = ctypes.c_int
    out = ctypes.c_double(0.0)
    rc = l.opapiInt8MfmaRateProbe(1 if uniform_random_operands else 0, iterations, ctypes.byref(out))
    if rc != 0:
        raise RuntimeError("opapiInt8MfmaRateProbe failed with status %d" % rc)
    return out.value


def calibration_copy(dst, src):
    """Runs the library's plain copy kernel (include/opapi_profile.h) from src to dst, two same-sized device tensors."""
    assert dst.is_contiguous() and src.is_contiguous() and dst.numel() * dst.element_size() == src.numel() * src.element_size()
    l = lib()
    l.opapiCalibrationCopy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    l.opapiCalibrationCopy.restype = ctypes.c_int
    rc = l.opapiCalibrationCopy(dst.data_ptr(), src.data_ptr(), src.numel() * src.element_size(), _stream_ptr())
    if rc != 0:
        raise AclnnError("opapiCalibrationCopy", rc, last_error())
