"""Pins the grouped-GEMM oracle.

int32 accumulators: exact float64 matmul per group (|acc| <= K * 127^2 < 2^53).
down-projection epilogue: closed form in numpy fp32 (two separate fp32 multiplies) + torch's bf16 rounding.
SwiGLU + requantisation: float64 evaluation of S (tolerance), exact recomputation of the requant step from the
oracle's own S with numpy float16 (independent of the C casts), and invariants (max |q| == 127, scale == max/127).
The reference's tests hold no expected numbers for either GEMM operator, so the last-ulp behaviour of exp/divide in
SwiGLU is "parity unpinned".
"""
import numpy as np
import pytest
import torch


def _problem(rng, M, K, N, E, ragged=True):
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    w = rng.integers(-127, 128, (E, K, N)).astype(np.int8)
    if ragged:
        cuts = np.sort(rng.integers(0, M + 1, E - 1)) if E > 1 else np.array([], np.int64)
        cumsum = np.concatenate([cuts, [M]]).astype(np.int64)
    else:
        cumsum = (np.arange(1, E + 1) * (M // E)).astype(np.int64)
    return x, w, cumsum


def _f64_grouped(x, w, cumsum):
    out = np.zeros((x.shape[0], w.shape[2]), np.float64)
    start = 0
    for e, end in enumerate(cumsum):
        out[start:end] = x[start:end].astype(np.float64) @ w[e].astype(np.float64)
        start = end
    return out


@pytest.mark.parametrize("M,K,N,E", [(1, 16, 8, 1), (37, 100, 24, 4), (96, 256, 64, 7), (64, 7168, 16, 2)])
def test_int32_accumulators_exact(oracle, M, K, N, E):
    rng = np.random.default_rng(M + K)
    x, w, cumsum = _problem(rng, M, K, N, E)
    ref = _f64_grouped(x, w, cumsum)
    got = oracle.grouped_matmul_i32(x, w, cumsum, list_type=0)
    assert np.array_equal(got.astype(np.float64), ref)
    counts = np.diff(np.concatenate([[0], cumsum])).astype(np.int64)
    assert np.array_equal(oracle.grouped_matmul_i32(x, w, counts, list_type=1), got)
    wt = np.ascontiguousarray(w.transpose(0, 2, 1))  # [E, N, K] storage
    assert np.array_equal(oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True), got)
    rows = np.array([M - 1, 0, M // 2], np.int64)
    assert np.array_equal(oracle.grouped_matmul_i32(x, w, cumsum, rows=rows), got[rows])


def test_int32_extreme_values_do_not_overflow(oracle):
    K = 14336
    x = np.full((2, K), -127, np.int8)
    w = np.full((1, K, 4), -127, np.int8)
    got = oracle.grouped_matmul_i32(x, w, np.array([2], np.int64))
    assert (got == K * 127 * 127).all()


def test_rows_beyond_last_group_untouched(oracle):
    rng = np.random.default_rng(3)
    x, w, _ = _problem(rng, 20, 32, 8, 2)
    got = oracle.grouped_matmul_i32(x, w, np.array([5, 12], np.int64))
    assert (got[12:] == 0).all() and got[:12].any()


@pytest.mark.parametrize("scale_dtype,out_dtype", [("f32", "bf16"), ("bf16", "bf16"), ("f32", "f16")])
def test_dequant_epilogue_closed_form(oracle, scale_dtype, out_dtype):
    rng = np.random.default_rng(9)
    M, K, N, E = 48, 192, 40, 3
    x, w, cumsum = _problem(rng, M, K, N, E)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    per_token = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    if scale_dtype == "bf16":
        scale_t = torch.from_numpy(scale).to(torch.bfloat16)
        scale_f = scale_t.float().numpy()
        scale_arg, sd = scale_t.view(torch.int16).numpy().view(np.uint16), oracle.DT_BF16
    else:
        scale_f, scale_arg, sd = scale, scale, oracle.DT_F32
    acc = _f64_grouped(x, w, cumsum).astype(np.int64).astype(np.float32)  # int32 -> fp32, nearest even
    group = np.searchsorted(cumsum, np.arange(M), side="right")
    y = (acc * scale_f[group]) * per_token[:, None]                       # fp32, this order
    if out_dtype == "bf16":
        ref = torch.from_numpy(y).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        od = oracle.DT_BF16
    else:
        ref = y.astype(np.float16).view(np.uint16)
        od = oracle.DT_F16
    got = oracle.grouped_matmul_dequant(x, w, scale_arg, per_token, cumsum, scale_dtype=sd, out_dtype=od)
    assert np.array_equal(got, ref)
    # static quant (no per-token scale): one multiply
    y1 = acc * scale_f[group]
    got1 = oracle.grouped_matmul_dequant(x, w, scale_arg, None, cumsum, scale_dtype=sd, out_dtype=oracle.DT_F32)
    assert np.array_equal(got1, y1)


def test_int32_to_float_rounds_to_nearest_even(oracle):
    # |acc| beyond 2^24: K=7168 rows of +-127 give 115,612,672-sized sums that fp32 cannot hold exactly
    K = 7168
    x = np.full((1, K), 127, np.int8)
    x[0, :3] = [1, 1, 1]
    w = np.full((1, K, 2), 127, np.int8)
    acc = oracle.grouped_matmul_i32(x, w, np.array([1], np.int64))
    y = oracle.grouped_matmul_dequant(x, w, np.ones((1, 2), np.float32), None, np.array([1], np.int64),
                                      out_dtype=oracle.DT_F32)
    assert np.array_equal(y, acc.astype(np.float32))  # numpy's int->float32 is round-to-nearest-even


def test_swiglu_quant(oracle):
    rng = np.random.default_rng(21)
    M, K, N, E = 80, 256, 96, 4
    x, w, cumsum = _problem(rng, M, K, N, E)
    cumsum[-1] = M - 6  # trailing rows belong to no group
    cumsum = np.minimum(cumsum, M - 6)
    w_scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    x_scale = rng.uniform(5e-3, 5e-2, M).astype(np.float32)
    y, ys, s = oracle.grouped_matmul_swiglu_quant(x, w, w_scale, x_scale, cumsum, want_s=True)
    used = int(cumsum[-1])
    # S against float64 with the split "first half activated, second half linear"
    acc = _f64_grouped(x, w, cumsum)
    group = np.minimum(np.searchsorted(cumsum, np.arange(M), side="right"), E - 1)
    c = acc * x_scale[:, None].astype(np.float64) * w_scale[group].astype(np.float64)
    a, b = c[:, :N // 2], c[:, N // 2:]
    s64 = a / (1.0 + np.exp(-a)) * b
    np.testing.assert_allclose(s[:used], s64[:used], rtol=2e-5, atol=1e-30)
    # requantisation recomputed from the oracle's S with numpy float16 (nearest even twice)
    mx = np.abs(s[:used]).max(axis=1)
    scale_ref = (mx / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(ys[:used], scale_ref)
    inv = (np.float32(1.0) / scale_ref).astype(np.float32)
    q_ref = np.rint((s[:used] * inv[:, None]).astype(np.float16).astype(np.float32)).astype(np.int8)
    assert np.array_equal(y[:used], q_ref)
    assert (np.abs(y[:used].astype(np.int32)).max(axis=1) == 127).all()
    # dequantised output is within half a step of S, plus the fp16 rounding of S*inv (half an fp16 ulp of 1/16 near 127)
    err = np.abs(y[:used].astype(np.float32) * ys[:used, None] - s[:used])
    assert (err <= ys[:used, None] * (0.5 + 1.0 / 32 + 1e-3) + 1e-12).all()
    # rows outside every group are untouched
    assert (y[used:] == 0).all() and (ys[used:] == 0).all()
    # bf16 / fp16 channel scales are widened exactly
    ws_bf16 = torch.from_numpy(w_scale).to(torch.bfloat16)
    y2, ys2 = oracle.grouped_matmul_swiglu_quant(x, w, ws_bf16.view(torch.int16).numpy().view(np.uint16), x_scale, cumsum,
                                                 w_scale_dtype=oracle.DT_BF16)
    y3, ys3 = oracle.grouped_matmul_swiglu_quant(x, w, ws_bf16.float().numpy(), x_scale, cumsum)
    assert np.array_equal(y2, y3) and np.array_equal(ys2, ys3)


def test_swiglu_zero_row_is_defined(oracle):
    x = np.zeros((2, 32), np.int8)
    w = np.ones((1, 32, 8), np.int8)
    y, ys = oracle.grouped_matmul_swiglu_quant(x, w, np.ones((1, 8), np.float32), np.ones(2, np.float32),
                                               np.array([2], np.int64))
    assert (y == 0).all() and (ys == 0).all()


# ------------------------------------------------------------------------------------------------ fused combine
def test_grouped_matmul_finalize_routing_matches_float64(oracle):
    """GroupedMatmulFinalizeRouting: float64 numpy restatement (exact matmul per group, contributions scattered with
    np.add.at).  fp32 against float64: a sum of up to `top_k` products, tolerance 1e-5 of the largest term."""
    rng = np.random.default_rng(4)
    M, K, N, E, batch, topk = 96, 128, 40, 5, 24, 4
    x, w, cumsum = _problem(rng, M, K, N, E)
    counts = np.diff(np.concatenate([[0], cumsum])).astype(np.int64)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    bias32 = rng.standard_normal((E, N)).astype(np.float32)
    bias_bits = oracle.f32_to_bf16_bits(bias32)
    bias = oracle.bf16_bits_to_f32(bias_bits)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    logit = rng.random(M).astype(np.float32)
    row_index = np.repeat(np.arange(batch), topk)
    rng.shuffle(row_index)
    shared_bits = oracle.f32_to_bf16_bits(rng.standard_normal((6, N)).astype(np.float32))
    shared = oracle.bf16_bits_to_f32(shared_bits)
    got = oracle.grouped_matmul_finalize_routing(x, w, scale, row_index, batch, counts, list_type=1, bias=bias_bits,
                                                 per_token=pt, logit=logit, shared=shared_bits, shared_offset=10,
                                                 shared_weight=0.5)
    acc = _f64_grouped(x, w, cumsum)
    group_of = np.searchsorted(cumsum, np.arange(M), side="right")
    contrib = acc * scale[group_of].astype(np.float64) * (pt.astype(np.float64) * logit)[:, None] \
        + logit[:, None].astype(np.float64) * bias[group_of]
    want = np.zeros((batch, N))
    want[10:16] = shared.astype(np.float64) * 0.5
    np.add.at(want, row_index, contrib)
    scale_of_terms = np.abs(contrib).max()
    assert np.abs(got - want).max() <= 1e-5 * scale_of_terms
    # cumsum list, transposed storage, no optional inputs: a plain scatter of the dequantised rows
    wt = np.ascontiguousarray(w.transpose(0, 2, 1))
    got2 = oracle.grouped_matmul_finalize_routing(x, wt, scale, row_index, batch, cumsum, list_type=0, w_trans=True)
    want2 = np.zeros((batch, N))
    np.add.at(want2, row_index, acc * scale[group_of].astype(np.float64))
    assert np.abs(got2 - want2).max() <= 1e-5 * np.abs(acc * scale[group_of]).max()
    # rows beyond the last group and indices outside [0, batch) contribute nothing
    short = cumsum.copy()
    short[-1] = short[-2]
    bad = row_index.copy()
    bad[:3] = [-1, batch, batch + 5]
    got3 = oracle.grouped_matmul_finalize_routing(x, w, scale, bad, batch, short, list_type=0)
    keep = (np.arange(M) < short[-1]) & (bad >= 0) & (bad < batch)
    want3 = np.zeros((batch, N))
    np.add.at(want3, bad[keep], (acc * scale[group_of.clip(max=E - 1)].astype(np.float64))[keep])
    assert np.abs(got3 - want3).max() <= 1e-5 * np.abs(acc).max() * scale.max()
    # equivalence with the unfused pair: down projection to fp32, then a weighted scatter
    y = oracle.grouped_matmul_dequant(x, w, scale, pt, cumsum, out_dtype=oracle.DT_F32)
    want4 = np.zeros((batch, N))
    np.add.at(want4, row_index, y.astype(np.float64) * logit[:, None])
    got4 = oracle.grouped_matmul_finalize_routing(x, w, scale, row_index, batch, cumsum, list_type=0, per_token=pt, logit=logit)
    assert np.abs(got4 - want4).max() <= 1e-5 * np.abs(y).max()
