"""aclnnMoeGatingTopKSoftmaxV2 on the GPU against the CPU oracle.

Values: fp32 within 1e-5 relative (exp and the order of the sum differ in the last bits; the reference's own arithmetic
for those lives in the CANN library), 16-bit outputs within one unit of the format.  Indices: exact wherever the
oracle's values at the compared positions differ by more than that; two picks whose values the two sides cannot tell
apart may swap."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def _inputs(oracle, rows_shape, cols, dtype_name, seed, scale=3.0):
    rng = np.random.default_rng(seed)
    x32 = (rng.standard_normal(tuple(rows_shape) + (cols,)) * scale).astype(np.float32)
    xt = torch.from_numpy(x32).to(TORCH[dtype_name])
    code = {"f32": oracle.DT_F32, "f16": oracle.DT_F16, "bf16": oracle.DT_BF16}[dtype_name]
    bits = xt.numpy() if dtype_name == "f32" else xt.view(torch.int16).numpy().view(np.uint16)
    return xt, bits, code


def _check(oracle, code, got, ref, x_seen, renorm):
    y, idx, sm = got
    y_r, idx_r, sm_r = ref
    k = idx.shape[-1]
    yf, yf_r = oracle.to_f32(y, code), oracle.to_f32(y_r, code)
    tol = {oracle.DT_F32: 1e-5, oracle.DT_F16: 2e-3, oracle.DT_BF16: 1.6e-2}[code]
    np.testing.assert_allclose(yf, yf_r, rtol=tol, atol=1e-30)
    if sm_r is not None:
        np.testing.assert_allclose(sm, sm_r, rtol=1e-5, atol=1e-37)
    # index parity: where they differ, the selection keys at the two indices must be indistinguishable
    key = sm_r if renorm == 0 else x_seen
    diff = idx != idx_r
    if diff.any():
        a = np.take_along_axis(key, np.where(diff, idx, 0).astype(np.int64), -1)
        b = np.take_along_axis(key, np.where(diff, idx_r, 0).astype(np.int64), -1)
        assert np.all(np.abs(a - b)[diff] <= 4e-6 * np.abs(b)[diff]), "indices differ on distinguishable values"
        assert diff.mean() < 1e-3
    # every row's picks are distinct experts
    srt = np.sort(idx.reshape(-1, k), axis=-1)
    assert (np.diff(srt, axis=-1) > 0).all() or k == 1


CASES = [  # leading shape, cols, k
    ((1,), 1, 1), ((3,), 4, 2), ((7,), 8, 8), ((64,), 128, 8), ((4096,), 256, 8), ((16384,), 8, 2), ((2, 5), 60, 6),
    ((33,), 513, 16), ((9,), 4096, 64), ((3,), 5000, 300), ((2,), 32768, 1024),
]


@pytest.mark.parametrize("lead,cols,k", CASES)
@pytest.mark.parametrize("renorm", [0, 1])
def test_fp32_against_oracle(aclnn, oracle, dev, lead, cols, k, renorm):
    xt, bits, code = _inputs(oracle, lead, cols, "f32", cols * 7 + k)
    y, idx, sm = aclnn.moe_gating_top_k_softmax_v2(xt.to(dev), k, renorm, output_softmax=True)
    torch.cuda.synchronize()
    ref = oracle.moe_gating_top_k_softmax_v2(bits, k, renorm, want_softmax=True)
    _check(oracle, code, (y.cpu().numpy(), idx.cpu().numpy(), None if sm is None else sm.cpu().numpy()), ref, bits, renorm)


@pytest.mark.parametrize("dtype_name", ["f16", "bf16"])
@pytest.mark.parametrize("renorm", [0, 1])
def test_sixteen_bit_against_oracle(aclnn, oracle, dev, dtype_name, renorm):
    for lead, cols, k in [((50,), 256, 8), ((4, 6), 96, 5), ((5,), 1000, 33)]:
        xt, bits, code = _inputs(oracle, lead, cols, dtype_name, cols + renorm)
        y, idx, sm = aclnn.moe_gating_top_k_softmax_v2(xt.to(dev), k, renorm, output_softmax=True)
        torch.cuda.synchronize()
        ref = oracle.moe_gating_top_k_softmax_v2(bits, k, renorm, dtype=code, want_softmax=True)
        y_bits = y.view(torch.int16).cpu().numpy().view(np.uint16)
        _check(oracle, code, (y_bits, idx.cpu().numpy(), None if sm is None else sm.cpu().numpy()), ref,
               oracle.to_f32(bits, code), renorm)


def test_equal_values_finished_rows_and_example(aclnn, oracle, dev):
    x = torch.tensor([[1, 5, 5, 0, 5, 1], [2, 2, 2, 2, 2, 2]], dtype=torch.float32, device=dev)
    for renorm in (0, 1):
        _, idx, _ = aclnn.moe_gating_top_k_softmax_v2(x, 4, renorm)
        assert idx.cpu().tolist() == [[1, 2, 4, 0], [0, 1, 2, 3]]
    fin = torch.tensor([True, False], device=dev)
    y, idx, _ = aclnn.moe_gating_top_k_softmax_v2(x, 3, 0, finished=fin)
    y2, _, _ = aclnn.moe_gating_top_k_softmax_v2(x, 3, 0)
    assert idx.cpu().tolist() == [[6, 6, 6], [0, 1, 2]] and torch.equal(y, y2)
    # -inf logits are ordinary values: they lose to everything else and are still picked once each when k asks for them
    z = torch.tensor([[0.0, float("-inf"), 1.0, float("-inf")]], device=dev)
    yz, iz, _ = aclnn.moe_gating_top_k_softmax_v2(z, 4, 1)
    assert iz.cpu().tolist() == [[2, 0, 1, 3]]
    np.testing.assert_allclose(yz.cpu().numpy(), [[1 / (1 + np.exp(-1.0)), np.exp(-1.0) / (1 + np.exp(-1.0)), 0, 0]], rtol=1e-6)
    # the reference example's input (examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp:93): arithmetic progressions
    ex = torch.arange(12, dtype=torch.float32, device=dev).reshape(3, 4) + 0.1
    y, idx, sm = aclnn.moe_gating_top_k_softmax_v2(ex, 2, 0, output_softmax=True)
    zsum = 1 + np.exp(-1.0) + np.exp(-2.0) + np.exp(-3.0)
    np.testing.assert_allclose(y.cpu().numpy(), np.tile([1 / zsum, np.exp(-1.0) / zsum], (3, 1)), rtol=1e-6)
    assert idx.cpu().tolist() == [[3, 2]] * 3


def test_router_feeds_the_ffn_chain(pkg, aclnn, oracle, dev):
    """Router -> routing -> FFN: the gating operator's outputs are what MoeInitRoutingV3 and MoeFinalizeRoutingV2 take."""
    cfg = pkg.synth.config(0)
    rng = np.random.default_rng(5)
    logits = torch.from_numpy(rng.standard_normal((cfg.tokens, cfg.experts)).astype(np.float32)).to(dev)
    wgt, idx, _ = aclnn.moe_gating_top_k_softmax_v2(logits, cfg.top_k, renorm=1)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
    out = ffn.forward(torch.from_numpy(xq).to(dev), torch.from_numpy(xs).to(dev), idx, wgt)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    counts = np.bincount(idx.cpu().numpy().reshape(-1), minlength=cfg.experts)
    assert np.array_equal(np.cumsum(counts), ffn.cumsum.cpu().numpy())
    np.testing.assert_allclose(wgt.sum(-1).cpu().numpy(), 1.0, rtol=1e-5)
