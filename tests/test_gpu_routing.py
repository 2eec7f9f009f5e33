"""aclnnMoeInitRoutingV2 on the GPU against the CPU oracle: bit-exact indices, counts and gathered rows."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(aclnn, dev, x, idx, **kw):
    outs = aclnn.moe_init_routing_v2(torch.from_numpy(x).to(dev), torch.from_numpy(idx).to(dev), **kw)
    torch.cuda.synchronize()
    return [None if o is None else o.cpu().numpy() for o in outs]


CASES = [  # T, K, E, H, dtype
    (1, 1, 1, 1, np.float32),
    (3, 2, 3, 4, np.float32),
    (7, 3, 5, 30, np.float16),
    (64, 8, 128, 4096, np.int8),       # decode shape
    (256, 2, 8, 1024, np.int8),        # small config
    (333, 5, 100, 7, np.float32),      # odd row bytes
    (1000, 4, 33, 18, np.int8),        # 18-byte rows: 2-byte vector path
    (4096, 8, 256, 512, np.float16),   # DeepSeek-V3 routing shape (narrow rows keep the host copy small)
    (2048, 6, 2000, 8, np.float32),    # 11-bit digit
]


@pytest.mark.parametrize("T,K,E,H,dtype", CASES)
def test_dropless_bit_exact(aclnn, oracle, dev, T, K, E, H, dtype):
    rng = np.random.default_rng(T * 7 + K)
    x = (rng.standard_normal((T, H)) * 50).astype(dtype)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    for flag in (1, 2, 0):
        ex, ri, cnt, _ = _run(aclnn, dev, x, idx, expert_num=E, expert_tokens_count_or_cumsum_flag=flag)
        ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x, idx, expert_num=E, count_flag=flag)
        assert np.array_equal(ri, ri_r)
        assert np.array_equal(ex.view(np.uint8), ex_r.view(np.uint8))
        if flag:
            assert np.array_equal(cnt, cnt_r)
        else:
            assert cnt is None


def test_skewed_routing_bit_exact(pkg, aclnn, oracle, dev):
    """Zipf-skewed load on the DeepSeek-V3 expert count: many empty experts, one very hot expert."""
    cfg = pkg.synth.config(4)
    idx, _ = pkg.synth.make_routing(cfg, seed=4)
    hist = np.bincount(idx.reshape(-1), minlength=cfg.experts)
    assert (hist == 0).mean() > 0.2 and hist.max() > 10 * hist.mean()
    x = np.arange(cfg.tokens * 16, dtype=np.int32).reshape(cfg.tokens, 16).view(np.float32)
    for flag in (1, 2):
        ex, ri, cnt, _ = _run(aclnn, dev, x, idx, expert_num=cfg.experts, expert_tokens_count_or_cumsum_flag=flag)
        ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x, idx, expert_num=cfg.experts, count_flag=flag)
        assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r)
        assert np.array_equal(ex.view(np.uint32), ex_r.view(np.uint32))


def test_active_num(aclnn, oracle, dev):
    rng = np.random.default_rng(3)
    T, K, E, H = 100, 4, 16, 32
    x = rng.standard_normal((T, H)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    for active in (1, 123, 400, 9999):
        ex, ri, _, _ = _run(aclnn, dev, x, idx, active_num=active, expert_num=E)
        ex_r, ri_r, _, _ = oracle.moe_init_routing_v2(x, idx, active_num=active, expert_num=E)
        assert ex.shape == ex_r.shape and np.array_equal(ex, ex_r) and np.array_equal(ri, ri_r)


@pytest.mark.parametrize("T,K,E,C,H", [(3, 2, 3, 2, 4), (128, 8, 16, 3, 64), (500, 4, 7, 400, 10), (64, 2, 40, 1, 8)])
def test_drop_pad_bit_exact(aclnn, oracle, dev, T, K, E, C, H):
    rng = np.random.default_rng(T + C)
    x = rng.standard_normal((T, H)).astype(np.float32)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    ex, ri, cnt, bef = _run(aclnn, dev, x, idx, expert_capacity=C, expert_num=E, drop_pad_mode=1,
                            expert_tokens_count_or_cumsum_flag=1, expert_tokens_before_capacity_flag=True)
    ex_r, ri_r, _, bef_r = oracle.moe_init_routing_v2(x, idx, expert_capacity=C, expert_num=E, drop_pad_mode=1,
                                                      count_flag=1, before_capacity_flag=True)
    assert cnt is None
    assert np.array_equal(ri, ri_r) and np.array_equal(bef, bef_r) and np.array_equal(ex, ex_r)


def test_reference_example(aclnn, dev):
    """Literal of moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp:71-96."""
    x = np.repeat(np.array([[0.1], [0.2], [0.3]], np.float32), 4, axis=1)
    idx = np.array([[1, 2], [0, 1], [0, 2]], np.int32)
    ex, ri, _, bef = _run(aclnn, dev, x, idx, expert_capacity=2, expert_num=3, drop_pad_mode=1,
                          expert_tokens_before_capacity_flag=True)
    assert ri.tolist() == [2, 4, 0, 3, 1, 5] and bef.tolist() == [2, 2, 2]
    assert np.array_equal(ex[:, :, 0], np.array([[0.2, 0.3], [0.1, 0.2], [0.1, 0.3]], np.float32))


def test_unknown_expert_range(aclnn, oracle, dev):
    """expertNum 0: the id range is unknown, ids sort as signed 32-bit integers (three digit passes)."""
    rng = np.random.default_rng(11)
    idx = rng.integers(-50, 5000, (700, 3)).astype(np.int32)
    x = rng.standard_normal((700, 6)).astype(np.float32)
    ex, ri, _, _ = _run(aclnn, dev, x, idx, expert_num=0)
    ex_r, ri_r, _, _ = oracle.moe_init_routing_v2(x, idx, expert_num=0)
    assert np.array_equal(ri, ri_r) and np.array_equal(ex, ex_r)


def test_many_experts_counts(aclnn, oracle, dev):
    """More than 2048 experts: two digit passes, counts from the sorted keys."""
    rng = np.random.default_rng(12)
    E = 5000
    idx = rng.integers(0, E, (3000, 2)).astype(np.int32)
    x = rng.standard_normal((3000, 4)).astype(np.float32)
    for flag in (1, 2):
        ex, ri, cnt, _ = _run(aclnn, dev, x, idx, expert_num=E, expert_tokens_count_or_cumsum_flag=flag)
        ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x, idx, expert_num=E, count_flag=flag)
        assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r) and np.array_equal(ex, ex_r)


def test_empty_inputs(aclnn, dev):
    x = torch.empty((0, 16), dtype=torch.float32, device=dev)
    idx = torch.empty((0, 4), dtype=torch.int32, device=dev)
    ex, ri, _, _ = aclnn.moe_init_routing_v2(x, idx, expert_num=4)
    torch.cuda.synchronize()
    assert ex.shape == (0, 16) and ri.shape == (0,)


# ------------------------------------------------------------------------------------------------ MoeInitRoutingV3
def _run_v3(aclnn, dev, x, idx, scale, **kw):
    outs = aclnn.moe_init_routing_v3(torch.from_numpy(x).to(dev), torch.from_numpy(idx).to(dev),
                                     None if scale is None else torch.from_numpy(scale).to(dev), **kw)
    torch.cuda.synchronize()
    return [None if o is None else o.cpu().numpy() for o in outs]


V3_CASES = [  # T, K, E, H, dtype, expert range
    (1, 1, 1, 1, np.float32, None),
    (3, 4, 256, 2, np.float32, (0, 4)),          # the reference example's shape
    (7, 3, 5, 30, np.float16, (1, 4)),
    (64, 8, 128, 4096, np.int8, None),           # decode shape
    (64, 8, 256, 512, np.int8, (32, 64)),        # one expert-parallel rank's share of 256 experts
    (333, 5, 100, 7, np.float32, (99, 100)),     # a single active expert, odd row bytes
    (1000, 4, 33, 18, np.int8, (0, 32)),
    (4096, 8, 256, 512, np.int8, None),          # DeepSeek-V3 routing shape
    (2048, 6, 4000, 8, np.float32, (1000, 3047)),  # 2047 active experts + the sentinel: the full 11-bit digit
    (2048, 6, 2048, 8, np.float32, None),
]


@pytest.mark.parametrize("T,K,E,H,dtype,rng_", V3_CASES)
def test_v3_bit_exact(aclnn, oracle, dev, T, K, E, H, dtype, rng_):
    rng = np.random.default_rng(T * 11 + K)
    x = (rng.standard_normal((T, H)) * 50).astype(dtype)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    scale = rng.random(T).astype(np.float32)
    for mode in (0, 1, 2):
        for row_idx_type in (1, 0):
            ex, ri, cnt, es = _run_v3(aclnn, dev, x, idx, scale, expert_num=E, expert_tokens_num_type=mode,
                                      active_expert_range=rng_, row_idx_type=row_idx_type)
            ex_r, ri_r, cnt_r, es_r = oracle.moe_init_routing_v3(x, idx, scale, E, rng_, mode, row_idx_type)
            assert np.array_equal(ri, ri_r), (mode, row_idx_type)
            assert np.array_equal(cnt, cnt_r), (mode, row_idx_type)
            assert np.array_equal(ex.view(np.uint8), ex_r.view(np.uint8))
            assert np.array_equal(es, es_r)


def test_v3_without_scale_and_empty_input(aclnn, oracle, dev):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((50, 12)).astype(np.float32)
    idx = rng.integers(0, 9, (50, 3)).astype(np.int32)
    ex, ri, cnt, es = _run_v3(aclnn, dev, x, idx, None, expert_num=9, active_expert_range=(2, 7))
    ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v3(x, idx, None, 9, (2, 7), 1, 1)
    assert es is None and np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r) and np.array_equal(ex, ex_r)
    # no tokens: the count output is still written
    for mode, shape in ((0, (5,)), (1, (5,)), (2, (9, 2))):
        counts = torch.full(shape, 77, dtype=torch.int64, device=dev)
        out = (torch.empty((0, 12), device=dev), torch.empty((0,), dtype=torch.int32, device=dev), counts, None)
        aclnn.moe_init_routing_v3(torch.empty((0, 12), device=dev), torch.empty((0, 3), dtype=torch.int32, device=dev),
                                  None, expert_num=9, expert_tokens_num_type=mode, active_expert_range=(2, 7), out=out)
        torch.cuda.synchronize()
        got = counts.cpu().numpy()
        if mode == 2:   # min(active + 1, expertNum) = 6 pairs are written, the rest of the buffer is the caller's
            assert not got[:6].any() and (got[6:] == 77).all()
        else:
            assert not got.any()


def test_v3_skewed_routing_matches_v2(pkg, aclnn, dev):
    """Zipf-skewed load, whole range: V3's scatter-type index, cumsum and rows equal V2's (int64 instead of int32)."""
    cfg = pkg.synth.config(4)
    idx, _ = pkg.synth.make_routing(cfg, seed=4)
    x = np.arange(cfg.tokens * 16, dtype=np.int32).reshape(cfg.tokens, 16).view(np.float32)
    ex2, ri2, cum2, _ = _run(aclnn, dev, x, idx, expert_num=cfg.experts, expert_tokens_count_or_cumsum_flag=1)
    ex3, ri3, cum3, _ = _run_v3(aclnn, dev, x, idx, None, expert_num=cfg.experts, expert_tokens_num_type=0)
    assert np.array_equal(ri2, ri3) and np.array_equal(cum2.astype(np.int64), cum3)
    assert np.array_equal(ex2.view(np.uint32), ex3.view(np.uint32))


# ------------------------------------------------------------------------------------------------ V3 dynamic quantisation
QUANT_CASES = [  # T, K, E, H, dtype name, range, smooth
    (3, 2, 4, 8, "f32", None, False),
    (60, 3, 12, 40, "f32", (3, 9), True),
    (64, 8, 128, 4096, "bf16", None, False),       # decode shape
    (64, 8, 256, 512, "bf16", (32, 64), True),
    (200, 4, 16, 7168, "bf16", None, False),       # DeepSeek-V3 row width
    (100, 2, 8, 1000, "f16", None, True),
    (50, 3, 9, 37, "f16", (2, 7), False),          # odd width: byte path
    (33, 5, 10, 130, "bf16", None, True),          # width not a multiple of 4
]


@pytest.mark.parametrize("T,K,E,H,dtype_name,rng_,with_smooth", QUANT_CASES)
def test_v3_dynamic_quant_bit_exact(aclnn, oracle, dev, T, K, E, H, dtype_name, rng_, with_smooth):
    """int8 rows, scales, indices and counts equal the oracle bit for bit: every step is IEEE arithmetic (abs-max, two
    divides, a toward-zero narrowing, a halves-away rounding), none of it a library function."""
    rng = np.random.default_rng(T + H)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype_name]
    code = {"f32": oracle.DT_F32, "f16": oracle.DT_F16, "bf16": oracle.DT_BF16}[dtype_name]
    x32 = (rng.standard_normal((T, H)) * 3).astype(np.float32)
    x32[T // 2] = 0
    xt = torch.from_numpy(x32).to(tdt)
    bits = xt.numpy() if dtype_name == "f32" else xt.view(torch.int16).numpy().view(np.uint16)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    start, end = (0, E) if rng_ is None else rng_
    smooth = (rng.random((end - start, H)) + 0.5).astype(np.float32) if with_smooth else None
    for mode, row_idx_type in ((1, 1), (0, 0), (2, 1)):
        ex, ri, cnt, es = aclnn.moe_init_routing_v3(xt.to(dev), torch.from_numpy(idx).to(dev),
                                                    None if smooth is None else torch.from_numpy(smooth).to(dev),
                                                    expert_num=E, expert_tokens_num_type=mode, quant_mode=1,
                                                    active_expert_range=rng_, row_idx_type=row_idx_type)
        torch.cuda.synchronize()
        ex_r, ri_r, cnt_r, es_r = oracle.moe_init_routing_v3_quant(bits, idx, smooth, E, rng_, mode, row_idx_type, dtype=code)
        assert np.array_equal(ri.cpu().numpy(), ri_r) and np.array_equal(cnt.cpu().numpy(), cnt_r)
        assert np.array_equal(es.cpu().numpy(), es_r)
        assert np.array_equal(ex.cpu().numpy(), ex_r)


def test_v3_dynamic_quant_feeds_the_gemm(pkg, aclnn, oracle, dev):
    """bf16 activations -> V3 with quantMode 1 gives the int8 rows and scales the SwiGLU GEMM operator consumes."""
    cfg = pkg.synth.config(0)
    rng = np.random.default_rng(1)
    x = torch.from_numpy(rng.standard_normal((cfg.tokens, cfg.hidden)).astype(np.float32)).to(torch.bfloat16).to(dev)
    idx, _ = pkg.synth.make_routing(cfg, seed=0)
    w13, w13s, _, _ = pkg.synth.make_weights(cfg, dev, seed=0)
    ex, ri, cum, es = aclnn.moe_init_routing_v3(x, torch.from_numpy(idx).to(dev), None, expert_num=cfg.experts,
                                                expert_tokens_num_type=0, quant_mode=1)
    h, hs = aclnn.grouped_matmul_swiglu_quant(ex, w13.transpose(1, 2), cum, w13s, es)
    torch.cuda.synchronize()
    h_r, hs_r = oracle.grouped_matmul_swiglu_quant(ex.cpu().numpy(), w13.cpu().numpy(), w13s.cpu().numpy(), es.cpu().numpy(),
                                                   cum.cpu().numpy(), w_trans=True)
    assert np.abs(h.cpu().numpy().astype(np.int32) - h_r.astype(np.int32)).max() <= 1
    np.testing.assert_allclose(hs.cpu().numpy(), hs_r, rtol=1e-2)
