"""Pins the routing oracle: numpy stable argsort / bincount (what every golden script of the reference uses,
moe/moe_init_routing_quant_v2/tests/ut/op_kernel/moe_init_routing_quant_v2_data/gen_data.py:38-39), a brute-force
restatement of drop/pad, invariants, and the literal of the reference example
(moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp:71-96)."""
import numpy as np
import pytest


def _numpy_dropless(x, idx, E, active_num=0):
    T, K = idx.shape
    flat = idx.reshape(-1)
    order = np.argsort(flat, kind="stable")
    row_idx = np.empty(T * K, np.int32)
    row_idx[order] = np.arange(T * K, dtype=np.int32)
    hist = np.bincount(flat, minlength=E)[:E].astype(np.int32)
    rows = T * K if active_num == 0 else min(T * K, active_num)
    expanded = x[order[:rows] // K]
    return expanded, row_idx, hist


def _brute_drop_pad(x, idx, E, C):
    T, K = idx.shape
    flat = idx.reshape(-1)
    row_idx = np.full(T * K, -1, np.int32)
    expanded = np.zeros((E, C, x.shape[1]), x.dtype)
    seen = [0] * E
    for i in range(T * K):  # ascending flat index == stable rank within the expert
        e = flat[i]
        if seen[e] < C:
            row_idx[i] = e * C + seen[e]
            expanded[e, seen[e]] = x[i // K]
        seen[e] += 1
    return expanded, row_idx, np.array(seen, np.int32)


@pytest.mark.parametrize("T,K,E,H", [(1, 1, 1, 1), (7, 3, 5, 4), (64, 8, 256, 16), (333, 2, 8, 7), (1000, 4, 33, 3)])
def test_dropless_matches_numpy(oracle, T, K, E, H):
    rng = np.random.default_rng(T * 131 + K)
    x = rng.standard_normal((T, H)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    ex_ref, ri_ref, hist = _numpy_dropless(x, idx, E)
    for flag in (0, 1, 2):
        ex, ri, cnt, bef = oracle.moe_init_routing_v2(x, idx, expert_num=E, count_flag=flag)
        assert np.array_equal(ri, ri_ref)
        assert np.array_equal(ex, ex_ref)
        assert bef is None
        if flag == 0:
            assert cnt is None
        elif flag == 1:
            assert np.array_equal(cnt, np.cumsum(hist).astype(np.int32))
            assert cnt[-1] == T * K
        else:
            assert np.array_equal(cnt, hist)
    # invariants: permutation, sortedness of the gathered expert ids, gather identity
    assert np.array_equal(np.sort(ri_ref), np.arange(T * K))
    sorted_e = np.empty(T * K, np.int32)
    sorted_e[ri_ref] = idx.reshape(-1)
    assert (np.diff(sorted_e) >= 0).all()


def test_active_num_truncates_rows(oracle):
    rng = np.random.default_rng(5)
    T, K, E, H = 50, 4, 9, 6
    x = rng.standard_normal((T, H)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    for active in (1, 37, 199, 200, 5000):
        ex_ref, ri_ref, _ = _numpy_dropless(x, idx, E, active)
        ex, ri, _, _ = oracle.moe_init_routing_v2(x, idx, active_num=active, expert_num=E)
        assert ex.shape == ex_ref.shape
        assert np.array_equal(ex, ex_ref) and np.array_equal(ri, ri_ref)


@pytest.mark.parametrize("T,K,E,C", [(3, 2, 3, 2), (40, 4, 6, 5), (40, 4, 6, 40), (128, 8, 16, 3)])
def test_drop_pad_matches_brute_force(oracle, T, K, E, C):
    rng = np.random.default_rng(T + C)
    x = rng.standard_normal((T, 5)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    ex_ref, ri_ref, hist = _brute_drop_pad(x, idx, E, C)
    ex, ri, cnt, bef = oracle.moe_init_routing_v2(x, idx, expert_capacity=C, expert_num=E, drop_pad_mode=1,
                                                  count_flag=1, before_capacity_flag=True)
    assert cnt is None  # drop/pad never emits count-or-cumsum
    assert np.array_equal(ri, ri_ref) and np.array_equal(ex, ex_ref) and np.array_equal(bef, hist)


def test_reference_example_literal(oracle):
    # x rows 0.1 / 0.2 / 0.3, expertIdx {1,2,0,1,0,2}, E=3, C=2, drop/pad, before-capacity counts requested
    x = np.repeat(np.array([[0.1], [0.2], [0.3]], np.float32), 4, axis=1)
    idx = np.array([[1, 2], [0, 1], [0, 2]], np.int32)
    ex, ri, cnt, bef = oracle.moe_init_routing_v2(x, idx, expert_capacity=2, expert_num=3, drop_pad_mode=1,
                                                  before_capacity_flag=True)
    assert ri.tolist() == [2, 4, 0, 3, 1, 5]
    assert bef.tolist() == [2, 2, 2]
    want = np.array([[0.2, 0.3], [0.1, 0.2], [0.1, 0.3]], np.float32)  # token rows per expert slot
    assert np.array_equal(ex[:, :, 0], want)


def test_unknown_expert_range_sorts_signed(oracle):
    rng = np.random.default_rng(11)
    idx = rng.integers(-50, 5000, (200, 3)).astype(np.int32)
    x = rng.standard_normal((200, 2)).astype(np.float32)
    ex, ri, _, _ = oracle.moe_init_routing_v2(x, idx, expert_num=0)
    order = np.argsort(idx.reshape(-1), kind="stable")
    ref = np.empty(600, np.int32)
    ref[order] = np.arange(600, dtype=np.int32)
    assert np.array_equal(ri, ref)


# ------------------------------------------------------------------------------------------------ MoeInitRoutingV3
def _numpy_v3(x, idx, scale, start, end):
    """Stable argsort of the in-range flat positions: the sort + filter the reference kernels implement
    (moe/moe_init_routing_v3/README.md:12-66)."""
    T, K = idx.shape
    flat = idx.reshape(-1)
    keep = np.nonzero((flat >= start) & (flat < end))[0]
    order = keep[np.argsort(flat[keep], kind="stable")]
    hist = np.bincount(flat[keep] - start, minlength=end - start)
    return order, hist


@pytest.mark.parametrize("T,K,E,H,rng_", [(1, 1, 1, 1, None), (7, 3, 5, 4, (1, 4)), (64, 8, 256, 16, (32, 64)),
                                          (333, 2, 8, 7, None), (500, 4, 33, 3, (0, 1)), (40, 2, 16, 2, (15, 16))])
def test_v3_matches_numpy(oracle, T, K, E, H, rng_):
    rng = np.random.default_rng(T * 17 + K)
    x = rng.integers(-128, 128, (T, H)).astype(np.int8)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    scale = rng.random(T).astype(np.float32)
    start, end = (0, E) if rng_ is None else rng_
    order, hist = _numpy_v3(x, idx, scale, start, end)
    n = len(order)
    for mode in (0, 1, 2):
        for row_idx_type in (0, 1):
            ex, ri, cnt, es = oracle.moe_init_routing_v3(x, idx, scale, E, rng_, mode, row_idx_type)
            assert np.array_equal(ex[:n], x[order // K]) and not ex[n:].any()
            assert np.array_equal(es[:n], scale[order // K])
            if row_idx_type == 0:
                assert np.array_equal(ri[:n], order) and (ri[n:] == -1).all()
            else:
                inverse = np.full(T * K, -1, np.int32)
                inverse[order] = np.arange(n)
                assert np.array_equal(ri, inverse)
            if mode == 0:
                assert np.array_equal(cnt, np.cumsum(hist))
            elif mode == 1:
                assert np.array_equal(cnt, hist)
            else:
                nz = np.nonzero(hist)[0]
                assert cnt.shape == (E, 2)
                assert np.array_equal(cnt[:len(nz), 0], nz + start) and np.array_equal(cnt[:len(nz), 1], hist[nz])
                assert not cnt[len(nz):].any()


def test_v3_full_range_equals_v2(oracle):
    """With the whole expert range active V3 is V2's dropless mode with int64 counts."""
    rng = np.random.default_rng(5)
    T, K, E, H = 200, 4, 24, 6
    x = rng.standard_normal((T, H)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    ex2, ri2, cum2, _ = oracle.moe_init_routing_v2(x, idx, expert_num=E, count_flag=1)
    ex3, ri3, cum3, _ = oracle.moe_init_routing_v3(x, idx, None, E, None, 0, 1)
    assert np.array_equal(ex2, ex3) and np.array_equal(ri2, ri3) and np.array_equal(cum2.astype(np.int64), cum3)


def test_v3_reference_example_literal(oracle):
    """Inputs of moe/moe_init_routing_v3/examples/test_aclnn_moe_init_routing_v3.cpp:123-125 (range [0, 4), count
    mode); the expected values follow from the operator's definition by hand."""
    x = np.array([[0.1, 0.1], [0.2, 0.2], [0.3, 0.3]], np.float32)
    idx = np.array([[1, 2, 0, 3], [0, 2, 1, 3], [0, 1, 3, 2]], np.int32)
    scale = np.array([0.3423, 0.1652, 0.2652], np.float32)
    ex, ri, cnt, es = oracle.moe_init_routing_v3(x, idx, scale, 256, (0, 4), 1, 1)
    assert ri.tolist() == [3, 6, 0, 9, 1, 7, 4, 10, 2, 5, 11, 8]
    assert cnt.tolist() == [3, 3, 3, 3]
    assert np.array_equal(ex[:, 0], np.array([0.1, 0.2, 0.3, 0.1, 0.2, 0.3, 0.1, 0.2, 0.3, 0.1, 0.2, 0.3], np.float32))
    assert np.array_equal(es, scale[[0, 1, 2] * 4])


# ------------------------------------------------------------------------------------------------ V3 dynamic quantisation
def _trunc_to_half_numpy(v):
    """fp32 -> fp16 toward zero through numpy: nearest, then one step toward zero where nearest overshot."""
    h = v.astype(np.float16)
    over = np.abs(h.astype(np.float32)) > np.abs(v)
    h = np.where(over, np.nextafter(h, np.float16(0)), h)
    return h.astype(np.float32)


def test_half_truncation_matches_numpy(oracle):
    rng = np.random.default_rng(2)
    v = np.concatenate([rng.uniform(-130, 130, 300000), rng.standard_normal(100000) * 1e-3,
                        rng.standard_normal(50000) * 1e-6, np.arange(-128, 129) + 0.5, np.arange(-128, 129)]).astype(np.float32)
    assert np.array_equal(oracle.f32_to_f16_trunc_value(v), _trunc_to_half_numpy(v))


@pytest.mark.parametrize("with_smooth", [False, True])
@pytest.mark.parametrize("rng_", [None, (3, 9)])
def test_v3_dynamic_quant_matches_numpy(oracle, with_smooth, rng_):
    """Restatement of moe_v3_gather_dynamic_quant.h:103-141 in numpy: abs-max / 127, true divide, half toward zero,
    halves away from zero."""
    rng = np.random.default_rng(7)
    T, K, E, H = 60, 3, 12, 40
    x = (rng.standard_normal((T, H)) * 4).astype(np.float32)
    x[5] = 0                                                   # an all-zero token
    x[6, 3] = 1000.0                                           # one dominant element
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    start, end = (0, E) if rng_ is None else rng_
    smooth = (rng.random((end - start, H)) + 0.5).astype(np.float32) if with_smooth else None
    ex, ri, cnt, es = oracle.moe_init_routing_v3_quant(x, idx, smooth, E, rng_, 1, 1)
    _, ri_r, cnt_r, _ = oracle.moe_init_routing_v3(x, idx, None, E, rng_, 1, 1)
    assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r)
    flat = idx.reshape(-1)
    for i in range(T * K):
        d = ri[i]
        if d < 0:
            continue
        v = x[i // K] * (smooth[flat[i] - start] if with_smooth else np.float32(1))
        v = v.astype(np.float32)
        mx = np.abs(v).max()
        s = np.float32(mx) / np.float32(127.0)
        assert es[d] == s
        if mx == 0:
            assert not ex[d].any()
            continue
        h = _trunc_to_half_numpy((v / s).astype(np.float32))
        want = (np.sign(h) * np.floor(np.abs(h) + 0.5)).astype(np.int8)
        assert np.array_equal(ex[d], want), i
        assert np.abs(ex[d].astype(np.int32)).max() == 127
        assert np.abs(ex[d].astype(np.float32) * s - v).max() <= s * (0.5 + 1 / 16 + 1e-3)
    routed = (ri >= 0).sum()
    assert not ex[routed:].any() and not es[routed:].any()
    # gather-type index and the other count modes reuse the routing of the unquantised operator
    ex0, ri0, cnt0, es0 = oracle.moe_init_routing_v3_quant(x, idx, smooth, E, rng_, 2, 0)
    _, ri0_r, cnt0_r, _ = oracle.moe_init_routing_v3(x, idx, None, E, rng_, 2, 0)
    assert np.array_equal(ri0, ri0_r) and np.array_equal(cnt0, cnt0_r) and np.array_equal(ex0, ex) and np.array_equal(es0, es)


# ------------------------------------------------------------------------------------------------ MoeInitRoutingQuantV2
@pytest.mark.parametrize("dtype_name", ["f32", "f16", "bf16"])
def test_quant_v2_static_matches_numpy_half_arithmetic(oracle, dtype_name):
    """Static quantisation restated with numpy float16 arithmetic (moe_v2_gather_quant.h:93-133): numpy computes a half
    product or sum in fp32 and rounds it to half, which equals the directly rounded result (24 >= 2 * 11 + 2 bits)."""
    import torch
    rng = np.random.default_rng(8)
    T, K, E, H = 40, 3, 6, 24
    x32 = (rng.standard_normal((T, H)) * 40).astype(np.float32)
    x32[0, 0], x32[1, 1], x32[2, 2] = 1000.0, -2000.0, 366.0          # saturating values and one that lands near +127
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    if dtype_name == "f32":
        bits, code, seen = x32, oracle.DT_F32, x32
    else:
        tdt = torch.float16 if dtype_name == "f16" else torch.bfloat16
        xt = torch.from_numpy(x32).to(tdt)
        bits, seen = xt.view(torch.int16).numpy().view(np.uint16), xt.float().numpy()
        code = oracle.DT_F16 if dtype_name == "f16" else oracle.DT_BF16
    scale, offset = np.float32(0.3452), np.float32(1.8369)
    ex, ri, cnt, _, dyn = oracle.moe_init_routing_quant_v2(bits, idx, 0, scale, offset, expert_num=E, count_flag=1, dtype=code)
    _, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x32, idx, expert_num=E, count_flag=1)
    assert dyn is None and np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r)
    h = seen.astype(np.float16)
    h = (h * np.float16(scale)).astype(np.float16)
    h = (h + np.float16(offset)).astype(np.float16)
    q = np.clip(np.rint(h.astype(np.float32)), -128, 127).astype(np.int8)
    want = np.zeros_like(ex)
    want[ri] = q[np.arange(T * K) // K]
    assert np.array_equal(ex, want)
    assert (np.abs(q.astype(np.int32)) == 127).any() or (q == -128).any()      # the saturation branch is exercised


@pytest.mark.parametrize("smooth_rows", [0, 1, 6])
def test_quant_v2_dynamic_equals_v3_dynamic_and_drop_pad(oracle, smooth_rows):
    rng = np.random.default_rng(12)
    T, K, E, H = 50, 2, 6, 20
    x = (rng.standard_normal((T, H)) * 3).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    smooth = None if smooth_rows == 0 else (rng.random((smooth_rows, H)) + 0.5).astype(np.float32)
    ex, ri, _, _, dyn = oracle.moe_init_routing_quant_v2(x, idx, 1, smooth, expert_num=E)
    full = None if smooth is None else np.broadcast_to(smooth, (E, H)).copy()
    ex3, ri3, _, es3 = oracle.moe_init_routing_v3_quant(x, idx, full, E, None, 1, 1)
    assert np.array_equal(ex, ex3) and np.array_equal(ri, ri3) and np.array_equal(dyn, es3)
    # drop/pad: rows land at expert * capacity + rank, the rest is zero with scale 0
    C = 5
    exd, rid, _, bef, dynd = oracle.moe_init_routing_quant_v2(x, idx, 1, smooth, expert_capacity=C, expert_num=E,
                                                              drop_pad_mode=1, before_capacity_flag=True)
    _, rid_r, _, bef_r = oracle.moe_init_routing_v2(x, idx, expert_capacity=C, expert_num=E, drop_pad_mode=1,
                                                    before_capacity_flag=True)
    assert np.array_equal(rid, rid_r) and np.array_equal(bef, bef_r)
    flat = exd.reshape(E * C, H)
    used = np.zeros(E * C, bool)
    for i in range(T * K):
        if rid[i] >= 0:
            used[rid[i]] = True
            assert np.array_equal(flat[rid[i]], ex[ri[i]]) and dynd[rid[i]] == dyn[ri[i]]
    assert not flat[~used].any() and not dynd[~used].any()
    # activeNum cuts the dropless output
    exa, _, _, _, dyna = oracle.moe_init_routing_quant_v2(x, idx, 1, smooth, active_num=37, expert_num=E)
    assert exa.shape == (37, H) and np.array_equal(exa, ex[:37]) and np.array_equal(dyna, dyn[:37])
