"""aclnnMoeFinalizeRoutingV2 on the GPU against the CPU oracle (bit-exact: same operation order, no fused multiply-add)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NP2T = {np.float32: torch.float32, np.float16: torch.float16}


def _bits_to_torch(bits, dev):
    return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)


def _case(rng, T, K, H, E, with_x1, with_x2, with_bias, mode, C=0):
    n_rows = E * C if mode in (1, 3) else T * K
    ex = rng.standard_normal((n_rows, H)).astype(np.float32)
    x1 = rng.standard_normal((T, H)).astype(np.float32) if with_x1 else None
    x2 = rng.standard_normal((T, H)).astype(np.float32) if with_x2 else None
    bias = rng.standard_normal((E, H)).astype(np.float32) if with_bias else None
    scales = rng.uniform(0, 1, (T, K)).astype(np.float32)
    expert_idx = rng.integers(0, E, (T, K)).astype(np.int32) if with_bias else None
    if mode in (1, 3):
        idx = rng.integers(-1, n_rows, T * K).astype(np.int32)
        ex = ex.reshape(E, C, H)
    else:
        idx = rng.permutation(T * K).astype(np.int32)
    return ex, idx, x1, x2, bias, scales, expert_idx


REF_SHAPES = [(3, 7, 2, 12), (10, 30, 2, 1024), (10, 30, 3, 10), (300, 7, 257, 12), (471, 30, 4, 933), (16, 20, 4, 12),
              (8, 1024, 2, 256), (256, 7168, 8, 64)]


@pytest.mark.parametrize("E,H,K,T", REF_SHAPES)
@pytest.mark.parametrize("dtype", ["bf16", "bf16_f32scale", "f32", "f16"])
def test_matches_oracle(aclnn, oracle, dev, E, H, K, T, dtype):
    rng = np.random.default_rng(5)
    for mode, x1f, x2f, bf in [(0, True, True, True), (2, False, False, False), (2, True, False, True)]:
        ex, idx, x1, x2, bias, scales, eidx = _case(rng, T, K, H, E, x1f, x2f, bf, mode)
        if dtype.startswith("bf16"):
            enc = oracle.f32_to_bf16_bits
            to_dev = lambda a: None if a is None else _bits_to_torch(enc(a), dev)
            code = oracle.DT_BF16
            if dtype == "bf16":
                s_bits, s_dev, s_code = enc(scales), _bits_to_torch(enc(scales), dev), oracle.DT_BF16
            else:
                s_bits, s_dev, s_code = scales, torch.from_numpy(scales).to(dev), oracle.DT_F32
            ref = oracle.moe_finalize_routing_v2(enc(ex), idx, None if x1 is None else enc(x1),
                                                 None if x2 is None else enc(x2), None if bias is None else enc(bias),
                                                 s_bits, eidx, drop_pad_mode=mode, dtype=code, scale_dtype=s_code)
            got = aclnn.moe_finalize_routing_v2(to_dev(ex), torch.from_numpy(idx).to(dev), to_dev(x1), to_dev(x2),
                                                to_dev(bias), s_dev, None if eidx is None else torch.from_numpy(eidx).to(dev),
                                                drop_pad_mode=mode)
            torch.cuda.synchronize()
            got_bits = got.view(torch.int16).cpu().numpy().view(np.uint16)
            assert np.array_equal(got_bits, ref)
        elif dtype == "f32":
            to_dev = lambda a: None if a is None else torch.from_numpy(a).to(dev)
            ref = oracle.moe_finalize_routing_v2(ex, idx, x1, x2, bias, scales, eidx, drop_pad_mode=mode)
            got = aclnn.moe_finalize_routing_v2(to_dev(ex), to_dev(idx), to_dev(x1), to_dev(x2), to_dev(bias),
                                                to_dev(scales), to_dev(eidx), drop_pad_mode=mode)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), ref)
        else:
            h = lambda a: None if a is None else a.astype(np.float16)
            u = lambda a: None if a is None else a.astype(np.float16).view(np.uint16)
            to_dev = lambda a: None if a is None else torch.from_numpy(h(a)).to(dev)
            ref = oracle.moe_finalize_routing_v2(u(ex), idx, u(x1), u(x2), u(bias), u(scales), eidx, drop_pad_mode=mode,
                                                 dtype=oracle.DT_F16)
            got = aclnn.moe_finalize_routing_v2(to_dev(ex), torch.from_numpy(idx).to(dev), to_dev(x1), to_dev(x2),
                                                to_dev(bias), to_dev(scales),
                                                None if eidx is None else torch.from_numpy(eidx).to(dev), drop_pad_mode=mode)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy().view(np.uint16), ref)


@pytest.mark.parametrize("mode", [1, 3])
def test_drop_pad_arrangements(aclnn, oracle, dev, mode):
    rng = np.random.default_rng(10)
    T, K, H, E, C = 50, 4, 64, 6, 9
    ex, idx, x1, x2, bias, scales, eidx = _case(rng, T, K, H, E, False, False, True, mode, C)
    idx[:K] = -1
    if mode == 1:
        idx.reshape(K, T)[:, 0] = -1
    ref = oracle.moe_finalize_routing_v2(ex, idx, None, None, bias, scales, eidx, drop_pad_mode=mode)
    t = lambda a: torch.from_numpy(a).to(dev)
    got = aclnn.moe_finalize_routing_v2(t(ex), t(idx), None, None, t(bias), t(scales), t(eidx), drop_pad_mode=mode)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), ref)
    assert (got.cpu().numpy()[0] == 0).all()


def test_reference_example(aclnn, oracle, dev):
    """Literal of moe/moe_finalize_routing_v2/examples/test_aclnn_moe_finalize_routing_v2.cpp:102-110."""
    ex = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1] * 2, np.float32).reshape(6, 4)
    x1 = np.array([0.2, 1.2, 2.2, 3.2, 4.2, 5.2, 6.2, 7.2, 8.2, 9.2, 10.2, 11.2], np.float32).reshape(3, 4)
    bias = np.array([0.2, 0.4] * 4, np.float32).reshape(2, 4)
    scales = np.array([1.3, 1.6, 1.2, 1.8, 1.2, 2.3], np.float32).reshape(3, 2)
    eidx = np.array([0, 1, 0, 1, 0, 1], np.int32).reshape(3, 2)
    idx = np.array([2, 1, 4, 3, 0, 5], np.int32)
    t = lambda a: torch.from_numpy(a).to(dev)
    got = aclnn.moe_finalize_routing_v2(t(ex), t(idx), t(x1), t(x1), t(bias), t(scales), t(eidx), drop_pad_mode=0)
    torch.cuda.synchronize()
    ref = oracle.moe_finalize_routing_v2(ex, idx, x1, x1, bias, scales, eidx, drop_pad_mode=0)
    assert np.array_equal(got.cpu().numpy(), ref)
    np.testing.assert_allclose(got.cpu().numpy()[0, 0], 0.4 + 8.3 * 1.3 + 0.3 * 1.6, rtol=1e-6)


def test_no_scales_plain_gather(aclnn, dev):
    rng = np.random.default_rng(9)
    ex = torch.from_numpy(rng.standard_normal((40, 24)).astype(np.float32)).to(dev)
    idx = torch.from_numpy(rng.permutation(40).astype(np.int32)).to(dev)
    got = aclnn.moe_finalize_routing_v2(ex, idx, drop_pad_mode=0)
    torch.cuda.synchronize()
    assert torch.equal(got, ex[idx.long()])


def _to_dtype(oracle, dtype, dev):
    """(encode numpy fp32 -> oracle representation, oracle representation -> device tensor, oracle dtype code)."""
    if dtype == "bf16":
        enc = lambda a: None if a is None else oracle.f32_to_bf16_bits(a)
        return enc, (lambda b: None if b is None else _bits_to_torch(b, dev)), oracle.DT_BF16
    if dtype == "f16":
        enc = lambda a: None if a is None else a.astype(np.float16).view(np.uint16)
        return enc, (lambda b: None if b is None else torch.from_numpy(b.view(np.float16)).to(dev)), oracle.DT_F16
    enc = lambda a: None if a is None else a
    return enc, (lambda b: None if b is None else torch.from_numpy(b).to(dev)), oracle.DT_F32


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("K", [1, 3, 8])
@pytest.mark.parametrize("seeds", ["none", "x1", "x1x2"])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_wide_rows_without_bias(aclnn, oracle, dev, dtype, K, seeds, mode):
    """Rows of 1024 and more elements with no bias and at most eight experts per token take the batched kernel (indices
    and weights loaded up front, row packets in pairs): its branches for dropped rows (index -1 in the drop/pad
    arrangements, with the first term, a middle term or every term of a token dropped), for the x1 / x2 seeds without a
    bias, and for fewer than eight experts per token in both index arrangements."""
    rng = np.random.default_rng(1000 * mode + 10 * K + len(seeds))
    T, H, E, C = 37, 1536, 5, 19
    ex, idx, x1, x2, _, scales, _ = _case(rng, T, K, H, E, seeds != "none", seeds == "x1x2", False, mode, C)
    if mode in (1, 3):
        at = (lambda n, k: k * T + n) if mode == 1 else (lambda n, k: n * K + k)
        idx[at(0, 0)] = -1                       # token 0: first term dropped
        for k in range(K):
            idx[at(1, k)] = -1                   # token 1: every term dropped
        idx[at(2, K - 1)] = -1                   # token 2: last term dropped
        if K >= 3:
            idx[at(3, 0)] = 5                    # token 3: a middle term dropped, neighbours kept
            idx[at(3, 1)] = -1
            idx[at(3, 2)] = 7
    enc, to_dev, code = _to_dtype(oracle, dtype, dev)
    s_code = code
    ref = oracle.moe_finalize_routing_v2(enc(ex), idx, enc(x1), enc(x2), None, enc(scales), None, drop_pad_mode=mode,
                                         dtype=code, scale_dtype=s_code)
    got = aclnn.moe_finalize_routing_v2(to_dev(enc(ex)), torch.from_numpy(idx).to(dev), to_dev(enc(x1)), to_dev(enc(x2)),
                                        None, to_dev(enc(scales)), None, drop_pad_mode=mode)
    torch.cuda.synchronize()
    got_np = got.cpu().numpy() if dtype == "f32" else got.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got_np, ref)
    if mode in (1, 3) and seeds == "none":
        assert (got.float().cpu().numpy()[1] == 0).all()     # every term dropped and no seed: zeros
