"""Inputs given as strided views (a column slice of a wider tensor, a transposed index matrix, every second element of
a vector): each operator stages such an input into a contiguous copy in its workspace, as the reference makes its inputs
contiguous first (gmm/grouped_matmul_swiglu_quant/op_host/op_api/aclnn_grouped_matmul_swiglu_quant.cpp:431-445), and
must then give exactly what it gives for contiguous inputs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _cols(t):
    """The same values as a view with a row stride twice the row length."""
    wide = torch.empty((t.shape[0], 2 * t.shape[1]), dtype=t.dtype, device=t.device)
    wide[:, t.shape[1]:] = 0
    wide[:, :t.shape[1]] = t
    v = wide[:, :t.shape[1]]
    assert not v.is_contiguous() and torch.equal(v, t)
    return v


def _every_second(t):
    """1-D: the same values at every second element of a longer vector."""
    wide = torch.zeros((2 * t.shape[0],), dtype=t.dtype, device=t.device)
    wide[::2] = t
    v = wide[::2]
    assert (t.shape[0] < 2 or not v.is_contiguous()) and torch.equal(v, t)
    return v


def _transposed(t):
    """2-D: the same values as the transpose of contiguous [cols, rows] storage."""
    v = t.t().contiguous().t()
    assert not v.is_contiguous() and torch.equal(v, t)
    return v


def _same(a, b):
    for x, y in zip(a, b):
        assert (x is None) == (y is None)
        if x is not None:
            assert torch.equal(x, y)


def test_routing_v2_v3_quant_v2(aclnn, dev):
    rng = np.random.default_rng(0)
    T, K, E, H = 96, 4, 16, 80
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16).to(dev)
    idx = torch.from_numpy(rng.integers(0, E, (T, K)).astype(np.int32)).to(dev)
    scale = torch.from_numpy(rng.random(T).astype(np.float32)).to(dev)
    smooth = torch.from_numpy((rng.random((E, H)) + 0.5).astype(np.float32)).to(dev)
    xv, iv, sv, mv = _cols(x), _transposed(idx), _every_second(scale), _cols(smooth)

    _same(aclnn.moe_init_routing_v2(xv, iv, expert_num=E, expert_tokens_count_or_cumsum_flag=1),
          aclnn.moe_init_routing_v2(x, idx, expert_num=E, expert_tokens_count_or_cumsum_flag=1))
    _same(aclnn.moe_init_routing_v2(xv, iv, expert_num=E, expert_capacity=20, drop_pad_mode=1,
                                    expert_tokens_before_capacity_flag=True),
          aclnn.moe_init_routing_v2(x, idx, expert_num=E, expert_capacity=20, drop_pad_mode=1,
                                    expert_tokens_before_capacity_flag=True))
    _same(aclnn.moe_init_routing_v3(xv, iv, sv, expert_num=E, active_expert_range=(2, 11)),
          aclnn.moe_init_routing_v3(x, idx, scale, expert_num=E, active_expert_range=(2, 11)))
    _same(aclnn.moe_init_routing_v3(xv, iv, mv, expert_num=E, quant_mode=1),
          aclnn.moe_init_routing_v3(x, idx, smooth, expert_num=E, quant_mode=1))
    _same(aclnn.moe_init_routing_quant_v2(xv, iv, 1, mv, None, expert_num=E, expert_tokens_count_or_cumsum_flag=2),
          aclnn.moe_init_routing_quant_v2(x, idx, 1, smooth, None, expert_num=E, expert_tokens_count_or_cumsum_flag=2))
    torch.cuda.synchronize()


def test_gating(aclnn, dev):
    rng = np.random.default_rng(1)
    x = torch.from_numpy(rng.standard_normal((50, 64)).astype(np.float32)).to(dev)
    fin = torch.from_numpy(rng.random(50) < 0.2).to(dev)
    _same(aclnn.moe_gating_top_k_softmax_v2(_cols(x), 6, finished=_every_second(fin), output_softmax=True),
          aclnn.moe_gating_top_k_softmax_v2(x, 6, finished=fin, output_softmax=True))
    torch.cuda.synchronize()


def _gemm_inputs(dev, M=200, K=256, N=512, E=5, seed=2):
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.integers(-127, 128, (M, K)).astype(np.int8)).to(dev)
    w = torch.from_numpy(rng.integers(-127, 128, (E, N, K)).astype(np.int8)).to(dev).transpose(1, 2)
    ws = torch.from_numpy((rng.random((E, N)) * 9e-3 + 1e-3).astype(np.float32)).to(dev)
    xs = torch.from_numpy((rng.random(M) * 0.05 + 0.01).astype(np.float32)).to(dev)
    counts = rng.multinomial(M, np.ones(E) / E)
    gl = torch.from_numpy(np.cumsum(counts).astype(np.int64)).to(dev)
    return x, w, ws, xs, gl


def test_swiglu_quant_and_v4(aclnn, dev):
    x, w, ws, xs, gl = _gemm_inputs(dev)
    _same(aclnn.grouped_matmul_swiglu_quant(_cols(x), w, _every_second(gl), _cols(ws), _every_second(xs)),
          aclnn.grouped_matmul_swiglu_quant(x, w, gl, ws, xs))
    kw = dict(split_item=3, group_type=0, group_list_type=0)
    got = aclnn.grouped_matmul_v4([_cols(x)], [w], scale=[_cols(ws)], per_token_scale=[_every_second(xs)],
                                  group_list=_every_second(gl), output_dtype=torch.bfloat16, **kw)
    want = aclnn.grouped_matmul_v4([x], [w], scale=[ws], per_token_scale=[xs], group_list=gl,
                                   output_dtype=torch.bfloat16, **kw)
    _same(got, want)
    torch.cuda.synchronize()


def test_finalize_and_fused_combine(aclnn, dev):
    rng = np.random.default_rng(3)
    T, K, H, E = 40, 4, 96, 6
    ex = torch.from_numpy(rng.standard_normal((T * K, H)).astype(np.float32)).to(torch.bfloat16).to(dev)
    row_idx = torch.from_numpy(rng.permutation(T * K).astype(np.int32)).to(dev)
    scales = torch.from_numpy(rng.random((T, K)).astype(np.float32)).to(dev)
    x1 = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16).to(dev)
    bias = torch.from_numpy(rng.standard_normal((E, H)).astype(np.float32)).to(torch.bfloat16).to(dev)
    eidx = torch.from_numpy(rng.integers(0, E, (T, K)).astype(np.int32)).to(dev)
    got = aclnn.moe_finalize_routing_v2(_cols(ex), _every_second(row_idx), x1=_cols(x1), bias=_cols(bias),
                                        scales=_transposed(scales), expert_idx=_transposed(eidx), drop_pad_mode=2)
    want = aclnn.moe_finalize_routing_v2(ex, row_idx, x1=x1, bias=bias, scales=scales, expert_idx=eidx, drop_pad_mode=2)
    assert torch.equal(got, want)

    x, w, ws, xs, gl = _gemm_inputs(dev, M=160, K=256, N=128, E=4, seed=4)
    batch = 40
    ri = torch.from_numpy(np.random.default_rng(5).integers(0, batch, 160).astype(np.int64)).to(dev)
    logit = torch.from_numpy(np.random.default_rng(6).random(160).astype(np.float32)).to(dev)
    counts = torch.diff(gl, prepend=torch.zeros(1, dtype=gl.dtype, device=dev))
    # one row index per destination would make the sum order-free; here several rows add into one output row, so the
    # comparison allows the last-bit differences of a different atomic order
    got = aclnn.grouped_matmul_finalize_routing(_cols(x), w, _cols(ws), _every_second(ri), batch, _every_second(counts),
                                                per_token_scale=_every_second(xs), logit=_every_second(logit))
    want = aclnn.grouped_matmul_finalize_routing(x, w, ws, ri, batch, counts, per_token_scale=xs, logit=logit)
    torch.cuda.synchronize()
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5 * float(want.abs().max()))
