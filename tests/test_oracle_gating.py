"""Pins the gating oracle (MoeGatingTopKSoftmaxV2): float64 softmax + stable descending argsort in numpy, the closed
form of the reference example's input (moe/moe_gating_top_k_softmax_v2/examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp:93),
the tie rule, finished rows, and the ties-away narrowing against an exhaustive walk over all half-precision midpoints.
The reference holds no golden numbers for this operator (its kernel test only runs the kernel)."""
import numpy as np
import pytest


def _softmax64(v):
    e = np.exp(v.astype(np.float64) - v.astype(np.float64).max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def _topk_stable(v, k):
    order = np.argsort(-v, axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(v, order, -1), order.astype(np.int32)


@pytest.mark.parametrize("rows,cols,k", [(1, 1, 1), (3, 4, 2), (17, 8, 8), (64, 256, 8), (5, 1000, 37), (2, 4099, 1024)])
@pytest.mark.parametrize("renorm", [0, 1])
def test_matches_float64_numpy(oracle, rows, cols, k, renorm):
    rng = np.random.default_rng(rows * 31 + cols + renorm)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 3
    y, idx, sm = oracle.moe_gating_top_k_softmax_v2(x, k, renorm, want_softmax=True)
    if renorm == 0:
        p = _softmax64(x)
        np.testing.assert_allclose(sm, p, rtol=2e-6, atol=1e-30)
        assert np.abs(sm.sum(-1) - 1).max() < 1e-5
        # indices: exact against the oracle's own fp32 probabilities (stable order), and a top-k of the exact ones
        vals, order = _topk_stable(sm, k)
        assert np.array_equal(idx, order) and np.array_equal(y, vals)
        assert np.allclose(np.take_along_axis(p, idx.astype(np.int64), -1), -np.sort(-p, axis=-1)[..., :k], rtol=1e-5)
    else:
        assert sm is None
        vals, order = _topk_stable(x, k)
        assert np.array_equal(idx, order)
        np.testing.assert_allclose(y, _softmax64(vals), rtol=2e-6)
        assert np.abs(y.sum(-1) - 1).max() < 1e-5


def test_reference_example_input_closed_form(oracle):
    x = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1], np.float32).reshape(3, 4)
    y, idx, sm = oracle.moe_gating_top_k_softmax_v2(x, 2, 0, want_softmax=True)
    z = 1 + np.exp(-1.0) + np.exp(-2.0) + np.exp(-3.0)      # every row is an arithmetic progression with step 1
    np.testing.assert_allclose(y, np.tile([1 / z, np.exp(-1.0) / z], (3, 1)), rtol=1e-6)
    assert idx.tolist() == [[3, 2]] * 3
    np.testing.assert_allclose(sm, np.tile(np.exp([-3.0, -2.0, -1.0, 0.0]) / z, (3, 1)), rtol=1e-6)
    y1, idx1, _ = oracle.moe_gating_top_k_softmax_v2(x, 2, 1)
    np.testing.assert_allclose(y1, np.tile([1 / (1 + np.exp(-1.0)), np.exp(-1.0) / (1 + np.exp(-1.0))], (3, 1)), rtol=1e-6)
    assert idx1.tolist() == [[3, 2]] * 3


def test_equal_values_keep_index_order_and_finished_rows(oracle):
    x = np.array([[1, 5, 5, 0, 5, 1], [2, 2, 2, 2, 2, 2]], np.float32)
    for renorm in (0, 1):
        y, idx, _ = oracle.moe_gating_top_k_softmax_v2(x, 4, renorm)
        assert idx.tolist() == [[1, 2, 4, 0], [0, 1, 2, 3]]
    y, idx, _ = oracle.moe_gating_top_k_softmax_v2(x, 3, 0, finished=np.array([1, 0], np.uint8))
    assert idx.tolist() == [[6, 6, 6], [0, 1, 2]]
    y2, _, _ = oracle.moe_gating_top_k_softmax_v2(x, 3, 0)
    assert np.array_equal(y, y2)                           # finished only rewrites the indices


def test_ties_away_narrowing(oracle):
    # every midpoint between adjacent non-negative halves is exact in fp32 and must go to the larger magnitude
    h = np.arange(0, 0x7bff, dtype=np.uint16)
    lo, hi = h.view(np.float16).astype(np.float32), (h + 1).view(np.float16).astype(np.float32)
    mid = (lo.astype(np.float64) + hi.astype(np.float64)) / 2
    assert np.array_equal(mid.astype(np.float32).astype(np.float64), mid)
    assert np.array_equal(oracle.f32_to_f16_bits_away(mid.astype(np.float32)), h + 1)
    assert np.array_equal(oracle.f32_to_f16_bits_away(-mid.astype(np.float32)), (h + 1) | 0x8000)
    # away from the midpoints it is ordinary nearest rounding
    rng = np.random.default_rng(0)
    v = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 10 ** rng.uniform(-8, 4, 200000).astype(np.float32),
                        lo, np.nextafter(mid.astype(np.float32), np.float32(0)), np.nextafter(mid.astype(np.float32), np.float32(1e9))])
    v = v[np.abs(v) < 65500]
    exact_tie = np.isin(np.abs(v).astype(np.float64), mid)
    got = oracle.f32_to_f16_bits_away(v)
    assert np.array_equal(got[~exact_tie], v[~exact_tie].astype(np.float16).view(np.uint16))
    # bf16: same rule on 16 dropped bits
    b = rng.integers(0, 0x7f7f, 100000).astype(np.uint32)
    mid_b = ((b << 16) | 0x8000).view(np.float32)
    assert np.array_equal(oracle.f32_to_bf16_bits_away(mid_b), (b + 1).astype(np.uint16))
    w = rng.standard_normal(100000).astype(np.float32)
    nearest = oracle.f32_to_bf16_bits(w)
    away = oracle.f32_to_bf16_bits_away(w)
    tie = (w.view(np.uint32) & 0xffff) == 0x8000
    assert np.array_equal(nearest[~tie], away[~tie])


@pytest.mark.parametrize("dtype_name", ["f16", "bf16"])
def test_sixteen_bit_inputs(oracle, dtype_name):
    rng = np.random.default_rng(11)
    x32 = rng.standard_normal((40, 96)).astype(np.float32) * 2
    code = oracle.DT_F16 if dtype_name == "f16" else oracle.DT_BF16
    bits = oracle.from_f32(x32, code)
    xr = oracle.to_f32(bits, code)                           # the values the operator sees
    for renorm in (0, 1):
        y, idx, sm = oracle.moe_gating_top_k_softmax_v2(bits, 6, renorm, dtype=code, want_softmax=True)
        y32, idx32, sm32 = oracle.moe_gating_top_k_softmax_v2(xr, 6, renorm, want_softmax=True)
        assert np.array_equal(idx, idx32)
        away = oracle.f32_to_f16_bits_away if dtype_name == "f16" else oracle.f32_to_bf16_bits_away
        assert np.array_equal(y, away(y32))
        if renorm == 0:
            assert np.array_equal(sm, sm32)                  # the softmax output stays fp32
