"""CPU oracle for the quantized MoE expert-FFN path — TEST INFRASTRUCTURE, never part of the product path.

Thin numpy/ctypes front end over ``liboracle.so`` (built from ``moe_ffn_oracle.c`` by ``make -C oracle``).
Only the test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg import this module; the
shipped library and its Python host layer never do.

Half-precision tensors travel as ``uint16`` numpy arrays holding the raw bits (dtype code 1 = fp16, 27 = bf16,
0 = fp32, the ge::DataType numbering the reference uses).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ORACLE_LIBRARY_PATH: load another build of the oracle (the sanitizer leg of the test-suite)
_LIB_PATH = os.environ.get("ORACLE_LIBRARY_PATH") or os.path.join(_HERE, "liboracle.so")

DT_F32, DT_F16, DT_BF16 = 0, 1, 27


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if os.environ.get("ORACLE_LIBRARY_PATH"):
        return _LIB_PATH  # a build made by whoever set the variable
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(
            os.path.join(_HERE, "moe_ffn_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_moe_init_routing_v2.restype = ctypes.c_int
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return int(lib().oracle_num_threads())


# ----------------------------------------------------------------------------------------------- casts
def f32_to_bf16_bits(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_bf16(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def f32_to_f16_bits(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_f16(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def f16_bits_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().oracle_f16_to_f32(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def bf16_bits_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().oracle_bf16_to_f32(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def to_f32(a, dtype_code):
    if dtype_code == DT_F32:
        return np.asarray(a, np.float32)
    return f16_bits_to_f32(a) if dtype_code == DT_F16 else bf16_bits_to_f32(a)


def from_f32(a, dtype_code):
    if dtype_code == DT_F32:
        return np.asarray(a, np.float32)
    return f32_to_f16_bits(a) if dtype_code == DT_F16 else f32_to_bf16_bits(a)


# ----------------------------------------------------------------------------------------------- gating
def f32_to_f16_bits_away(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_f16_away(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def f32_to_bf16_bits_away(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_bf16_away(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def moe_gating_top_k_softmax_v2(x, k, renorm=0, finished=None, dtype=DT_F32, want_softmax=False):
    """x: fp32 array, or uint16 bit patterns for DT_F16 / DT_BF16, shape [..., cols].
    Returns (y in x's representation [..., k], expertIdx int32 [..., k], softmax fp32 [..., cols] or None)."""
    x = _c(x)
    cols = x.shape[-1]
    rows = x.size // cols
    y = np.empty(x.shape[:-1] + (k,), x.dtype)
    idx = np.empty(x.shape[:-1] + (k,), np.int32)
    sm = np.empty(x.shape, np.float32) if (want_softmax and renorm == 0) else None
    fin = None if finished is None else _c(finished, np.uint8)
    lib().oracle_moe_gating_top_k_softmax_v2(_p(x), ctypes.c_int(dtype), _p(fin), ctypes.c_int64(rows), ctypes.c_int64(cols),
                                             ctypes.c_int64(k), ctypes.c_int64(renorm), _p(y), _p(idx), _p(sm))
    return y, idx, sm


# ----------------------------------------------------------------------------------------------- routing
def moe_init_routing_v2(x, expert_idx, active_num=0, expert_capacity=0, expert_num=0, drop_pad_mode=0,
                        count_flag=0, before_capacity_flag=False):
    """x: [T, H] array of any fixed-size dtype (rows are copied as bytes); expert_idx: int32 [T, K].

    Returns (expandedX, expandedRowIdx, countOrCumsum | None, beforeCapacity | None)."""
    x = _c(x)
    expert_idx = _c(expert_idx, np.int32)
    T, K = expert_idx.shape
    H = x.shape[1]
    M = T * K
    row_bytes = H * x.dtype.itemsize
    if drop_pad_mode == 0:
        rows = M if active_num == 0 else min(M, active_num)
        ex = np.zeros((rows, H), x.dtype)
    else:
        ex = np.zeros((expert_num, expert_capacity, H), x.dtype)
    idx = np.full((M,), -7, np.int32)
    eff_count_flag = 0 if drop_pad_mode == 1 else count_flag
    eff_before = bool(before_capacity_flag) and drop_pad_mode == 1
    cnt = np.zeros((expert_num,), np.int32) if eff_count_flag else None
    bef = np.zeros((expert_num,), np.int32) if eff_before else None
    rc = lib().oracle_moe_init_routing_v2(
        _p(x), ctypes.c_int64(row_bytes), _p(expert_idx), ctypes.c_int64(T), ctypes.c_int64(K),
        ctypes.c_int64(active_num), ctypes.c_int64(expert_capacity), ctypes.c_int64(expert_num),
        ctypes.c_int64(drop_pad_mode), ctypes.c_int64(count_flag), ctypes.c_int(1 if before_capacity_flag else 0),
        _p(ex), _p(idx), _p(cnt), _p(bef))
    if rc != 0:
        raise ValueError("expert id outside [0, expert_num)")
    return ex, idx, cnt, bef


def moe_init_routing_v3(x, expert_idx, scale=None, expert_num=0, expert_range=None, count_mode=1, row_idx_type=1):
    """Dropless, unquantised MoeInitRoutingV3.  Returns (expandedX, idx int32 [M], counts int64, expandedScale or None).
    Output rows that no routed row lands on are zero."""
    x = np.ascontiguousarray(x)
    T = x.shape[0]
    row_bytes = x.strides[0] if x.ndim == 2 and x.shape[1] > 0 else 0
    idx = _c(expert_idx, np.int32)
    K = idx.shape[1]
    M = T * K
    start, end = (0, expert_num) if expert_range is None else expert_range
    ex = np.zeros((M,) + x.shape[1:], x.dtype)
    out_idx = np.zeros((M,), np.int32)
    if count_mode == 2:
        counts = np.zeros((expert_num, 2), np.int64)
    else:
        counts = np.zeros((end - start,), np.int64)
    sc = None if scale is None else _c(scale, np.float32)
    ex_scale = None if scale is None else np.zeros((M,), np.float32)
    lib().oracle_moe_init_routing_v3(
        _p(x), ctypes.c_int64(row_bytes), _p(idx), _p(sc), ctypes.c_int64(T), ctypes.c_int64(K), ctypes.c_int64(expert_num),
        ctypes.c_int64(start), ctypes.c_int64(end), ctypes.c_int64(count_mode), ctypes.c_int64(row_idx_type), _p(ex),
        _p(out_idx), _p(counts), _p(ex_scale))
    return ex, out_idx, counts, ex_scale


def f32_to_f16_trunc_value(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.float32)
    lib().oracle_f32_to_f16_trunc_value(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def moe_init_routing_v3_quant(x, expert_idx, smooth=None, expert_num=0, expert_range=None, count_mode=1, row_idx_type=1,
                              dtype=DT_F32):
    """MoeInitRoutingV3 with quantMode 1.  x: fp32, or uint16 bit patterns for DT_F16 / DT_BF16.
    Returns (expandedX int8 [M, cols], idx int32 [M], counts int64, expandedScale fp32 [M]); unrouted rows are zero."""
    x = _c(x)
    T, cols = x.shape
    idx = _c(expert_idx, np.int32)
    K = idx.shape[1]
    M = T * K
    start, end = (0, expert_num) if expert_range is None else expert_range
    ex = np.zeros((M, cols), np.int8)
    out_idx = np.zeros((M,), np.int32)
    counts = np.zeros((expert_num, 2) if count_mode == 2 else (end - start,), np.int64)
    ex_scale = np.zeros((M,), np.float32)
    sm = None if smooth is None else _c(smooth, np.float32)
    lib().oracle_moe_init_routing_v3_quant(
        _p(x), ctypes.c_int(dtype), ctypes.c_int64(cols), _p(idx), _p(sm), ctypes.c_int64(T), ctypes.c_int64(K),
        ctypes.c_int64(expert_num), ctypes.c_int64(start), ctypes.c_int64(end), ctypes.c_int64(count_mode),
        ctypes.c_int64(row_idx_type), _p(ex), _p(out_idx), _p(counts), _p(ex_scale))
    return ex, out_idx, counts, ex_scale


def moe_init_routing_quant_v2(x, expert_idx, quant_mode, scale=None, offset=None, active_num=0, expert_capacity=0,
                              expert_num=0, drop_pad_mode=0, count_flag=0, before_capacity_flag=False, dtype=DT_F32):
    """MoeInitRoutingQuantV2.  x: fp32, or uint16 bit patterns for DT_F16 / DT_BF16.  quant_mode 0: scale, offset are
    one float each; 1: scale is None or a smooth scale [1 or expert_num, cols].
    Returns (expandedX int8, expandedRowIdx, countOrCumsum | None, beforeCapacity | None, dynamicQuantScale | None)."""
    x = _c(x)
    T, cols = x.shape
    idx = _c(expert_idx, np.int32)
    K = idx.shape[1]
    M = T * K
    if drop_pad_mode == 1:
        ex = np.zeros((expert_num, expert_capacity, cols), np.int8)
        rows = expert_num * expert_capacity
        count_flag = 0
    else:
        rows = M if active_num == 0 else min(M, active_num)
        ex = np.zeros((rows, cols), np.int8)
        before_capacity_flag = False
    ri = np.zeros((M,), np.int32)
    cnt = np.zeros((expert_num,), np.int32) if count_flag else None
    bef = np.zeros((expert_num,), np.int32) if before_capacity_flag else None
    dyn = np.zeros((rows,), np.float32) if quant_mode == 1 else None
    sc = None if scale is None else _c(np.atleast_1d(scale), np.float32)
    of = None if offset is None else _c(np.atleast_1d(offset), np.float32)
    smooth_rows = 1 if (sc is None or quant_mode == 0) else sc.shape[0]
    rc = lib().oracle_moe_init_routing_quant_v2(
        _p(x), ctypes.c_int(dtype), ctypes.c_int64(cols), _p(idx), ctypes.c_int64(T), ctypes.c_int64(K),
        ctypes.c_int64(active_num), ctypes.c_int64(expert_capacity), ctypes.c_int64(expert_num),
        ctypes.c_int64(drop_pad_mode), ctypes.c_int64(count_flag), ctypes.c_int(int(before_capacity_flag)),
        ctypes.c_int64(quant_mode), _p(sc), _p(of), ctypes.c_int64(smooth_rows), _p(ex), _p(ri), _p(cnt), _p(bef), _p(dyn))
    assert rc == 0
    return ex, ri, cnt, bef, dyn


# ----------------------------------------------------------------------------------------------- GEMMs
def _gemm_common(x, w, w_trans, group_list, rows):
    x = _c(x, np.int8)
    w = _c(w, np.int8)
    M, K = x.shape
    if w_trans:
        G, N, K2 = w.shape
    else:
        G, K2, N = w.shape
    assert K2 == K, (w.shape, x.shape)
    gl = _c(group_list, np.int64)
    assert gl.shape[0] <= G
    rows_a = None if rows is None else _c(rows, np.int64)
    cnt = M if rows is None else rows_a.shape[0]
    return x, w, M, K, N, gl, rows_a, cnt


def grouped_matmul_i32(x, w, group_list, list_type=0, w_trans=False, rows=None):
    """Raw int32 accumulators. w: int8 [G, K, N] (w_trans False) or [G, N, K] storage (w_trans True)."""
    x, w, M, K, N, gl, rows_a, cnt = _gemm_common(x, w, w_trans, group_list, rows)
    out = np.zeros((cnt, N), np.int32)
    lib().oracle_grouped_matmul_i32(_p(x), _p(w), ctypes.c_int(int(w_trans)), ctypes.c_int64(M), ctypes.c_int64(K),
                                    ctypes.c_int64(N), ctypes.c_int64(gl.shape[0]), _p(gl), ctypes.c_int64(list_type),
                                    _p(rows_a), ctypes.c_int64(cnt), _p(out))
    return out


def grouped_matmul_swiglu_quant(x, w, w_scale, x_scale, group_list, w_trans=False, w_scale_dtype=DT_F32, rows=None,
                                want_s=False):
    """Returns (y int8 [cnt, N/2], yScale fp32 [cnt]) and, with want_s, also S fp32 [cnt, N/2]."""
    x, w, M, K, N, gl, rows_a, cnt = _gemm_common(x, w, w_trans, group_list, rows)
    ws = _c(w_scale, np.float32 if w_scale_dtype == DT_F32 else np.uint16)
    xs = _c(x_scale, np.float32)
    y = np.zeros((cnt, N // 2), np.int8)
    ys = np.zeros((cnt,), np.float32)
    s = np.zeros((cnt, N // 2), np.float32) if want_s else None
    lib().oracle_grouped_matmul_swiglu_quant(
        _p(x), _p(w), ctypes.c_int(int(w_trans)), _p(ws), ctypes.c_int(w_scale_dtype), _p(xs), ctypes.c_int64(M),
        ctypes.c_int64(K), ctypes.c_int64(N), ctypes.c_int64(gl.shape[0]), _p(gl), _p(rows_a), ctypes.c_int64(cnt),
        _p(y), _p(ys), _p(s))
    return (y, ys, s) if want_s else (y, ys)


def grouped_matmul_dequant(x, w, scale, per_token, group_list, list_type=0, w_trans=False, scale_dtype=DT_F32,
                           out_dtype=DT_BF16, rows=None):
    """Returns the output as fp32 (out_dtype 0) or raw uint16 bits (fp16 / bf16), shape [cnt, N]."""
    x, w, M, K, N, gl, rows_a, cnt = _gemm_common(x, w, w_trans, group_list, rows)
    sc = _c(scale, np.float32 if scale_dtype == DT_F32 else np.uint16)
    pt = _c(per_token, np.float32)
    out = np.zeros((cnt, N), np.float32 if out_dtype == DT_F32 else np.uint16)
    lib().oracle_grouped_matmul_dequant(
        _p(x), _p(w), ctypes.c_int(int(w_trans)), _p(sc), ctypes.c_int(scale_dtype), _p(pt), ctypes.c_int64(M),
        ctypes.c_int64(K), ctypes.c_int64(N), ctypes.c_int64(gl.shape[0]), _p(gl), ctypes.c_int64(list_type), _p(rows_a),
        ctypes.c_int64(cnt), _p(out), ctypes.c_int(out_dtype))
    return out


def grouped_matmul_finalize_routing(x, w, scale, row_index, batch, group_list, list_type=1, w_trans=False, bias=None,
                                    per_token=None, logit=None, shared=None, shared_dtype=DT_BF16, shared_offset=0,
                                    shared_weight=1.0, scale_dtype=DT_F32, bias_dtype=DT_BF16):
    """GroupedMatmulFinalizeRouting with INT8 weights.  scale / bias: fp32 arrays or uint16 bit patterns per their dtype;
    shared: uint16 bit patterns [rows, N].  Returns out fp32 [batch, N]."""
    x, w, M, K, N, gl, _, _ = _gemm_common(x, w, w_trans, group_list, None)
    sc = _c(scale, np.float32 if scale_dtype == DT_F32 else np.uint16)
    bs = None if bias is None else _c(bias, np.float32 if bias_dtype == DT_F32 else np.uint16)
    pt = None if per_token is None else _c(per_token, np.float32)
    lg = None if logit is None else _c(logit, np.float32)
    ri = _c(row_index, np.int64)
    sh = None if shared is None else _c(shared, np.uint16)
    out = np.empty((batch, N), np.float32)
    lib().oracle_grouped_matmul_finalize_routing(
        _p(x), _p(w), ctypes.c_int(int(w_trans)), _p(sc), ctypes.c_int(scale_dtype), _p(bs), ctypes.c_int(bias_dtype), _p(pt),
        _p(lg), _p(ri), ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), ctypes.c_int64(gl.shape[0]), _p(gl),
        ctypes.c_int64(list_type), _p(sh), ctypes.c_int(shared_dtype), ctypes.c_int64(0 if sh is None else sh.shape[0]),
        ctypes.c_int64(shared_offset), ctypes.c_float(shared_weight), ctypes.c_int64(batch), _p(out))
    return out


# ----------------------------------------------------------------------------------------------- finalize
def moe_finalize_routing_v2(expanded_x, expanded_row_idx, x1=None, x2=None, bias=None, scales=None, expert_idx=None,
                            drop_pad_mode=0, dtype=DT_F32, scale_dtype=None):
    """expanded_x/x1/x2/bias: fp32 arrays (dtype 0) or uint16 bit arrays (dtype 1/27); returns the same representation."""
    np_t = np.float32 if dtype == DT_F32 else np.uint16
    if scale_dtype is None:
        scale_dtype = dtype
    np_s = np.float32 if scale_dtype == DT_F32 else np.uint16
    ex = _c(expanded_x, np_t)
    H = ex.shape[-1]
    idx = _c(expanded_row_idx, np.int32)
    sc = _c(scales, np_s)
    K = 1 if sc is None else sc.shape[1]
    T = idx.shape[0] // K
    out = np.zeros((T, H), np_t)
    lib().oracle_moe_finalize_routing_v2(
        _p(ex), _p(idx), _p(_c(x1, np_t)), _p(_c(x2, np_t)), _p(_c(bias, np_t)), _p(sc), _p(_c(expert_idx, np.int32)),
        ctypes.c_int64(drop_pad_mode), ctypes.c_int64(T), ctypes.c_int64(K), ctypes.c_int64(H), ctypes.c_int(dtype),
        ctypes.c_int(scale_dtype), _p(out))
    return out
