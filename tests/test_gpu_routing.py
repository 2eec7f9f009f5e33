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
    (1024, 8, 512, 16, np.int8),       # 8192 keys, 512 experts: the largest input the one-workgroup sort takes
    (8193, 1, 512, 4, np.int8),        # one key more: the three-kernel sort
    (1000, 8, 513, 4, np.int8),        # one expert more: ten digit bits, the three-kernel sort
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
    assert 0.25 <= (hist == 0).mean() <= 0.45 and hist.max() > 10 * hist.mean()   # the benchmark's ~30 % empty experts
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


@pytest.mark.parametrize("E", [200, 256])
def test_expert_ids_outside_the_range_stay_in_bounds(aclnn, dev, E):
    """Ids outside [0, expertNum) are undefined in the reference (its sort keys and count table assume the range).  Here
    they give unspecified rows and counts but never an access outside the tensors: every output is guarded, the index
    output is still a permutation of the expanded rows, and the rows written are rows of x."""
    rng = np.random.default_rng(14)
    T, K, H = 300, 4, 16
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    idx[rng.random((T, K)) < 0.1] = E + 3
    idx[0, 0], idx[1, 1], idx[2, 2] = -1, 2 ** 31 - 1, -2 ** 31
    x = rng.integers(-100, 100, (T, H)).astype(np.int8)
    M = T * K
    guard = 64
    ex = torch.full((M + guard, H), 101, dtype=torch.int8, device=dev)
    ri = torch.full((M + guard,), -7, dtype=torch.int32, device=dev)
    cnt = torch.full((E + guard,), -7, dtype=torch.int32, device=dev)
    aclnn.moe_init_routing_v2(torch.from_numpy(x).to(dev), torch.from_numpy(idx).to(dev), 0, 0, E, 0, 1, False,
                              out=(ex[:M], ri[:M], cnt[:E], None))
    torch.cuda.synchronize()
    assert (ex[M:] == 101).all() and (ri[M:] == -7).all() and (cnt[E:] == -7).all()
    assert np.array_equal(np.sort(ri[:M].cpu().numpy()), np.arange(M))
    got = ex[:M].cpu().numpy()
    assert np.array_equal(got[ri[:M].cpu().numpy()], np.repeat(x, K, axis=0))


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


# ------------------------------------------------------------------------------------------------ QuantV2
def _quant_v2_inputs(rng, T, K, E, H, dtype_name, oracle, spread=3.0):
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype_name]
    code = {"f32": oracle.DT_F32, "f16": oracle.DT_F16, "bf16": oracle.DT_BF16}[dtype_name]
    x32 = (rng.standard_normal((T, H)) * spread).astype(np.float32)
    if T > 1:
        x32[T // 2] = 0
    xt = torch.from_numpy(x32).to(tdt)
    bits = xt.numpy() if dtype_name == "f32" else xt.view(torch.int16).numpy().view(np.uint16)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    return xt, bits, idx, code


def _same(got, want):
    if want is None:
        return got is None
    return np.array_equal(got.cpu().numpy(), want)


QUANT_V2_CASES = [
    # T, K, E, H, dtype
    (3, 2, 3, 4, "f32"),
    (64, 8, 128, 4096, "bf16"),
    (200, 4, 16, 7168, "bf16"),
    (100, 2, 8, 1000, "f16"),
    (50, 3, 9, 37, "f16"),            # odd width: byte path
    (33, 5, 10, 130, "f32"),
]


@pytest.mark.parametrize("T,K,E,H,dtype_name", QUANT_V2_CASES)
def test_quant_v2_static_bit_exact(aclnn, oracle, dev, T, K, E, H, dtype_name):
    """Static quantisation is three half-precision operations and a round-to-nearest-even: bit-exact, saturation
    included (the spread puts a share of the values beyond +-127)."""
    rng = np.random.default_rng(T * 7 + H)
    xt, bits, idx, code = _quant_v2_inputs(rng, T, K, E, H, dtype_name, oracle, spread=60.0)
    scale, offset = np.float32(0.8731), np.float32(-3.37)
    st = torch.tensor([scale], dtype=torch.float32, device=dev)
    ot = torch.tensor([offset], dtype=torch.float32, device=dev)
    C = max(1, min(T, (T * K) // E))
    for kw in (dict(expert_tokens_count_or_cumsum_flag=1), dict(expert_tokens_count_or_cumsum_flag=2, active_num=T),
               dict(drop_pad_mode=1, expert_capacity=C, expert_tokens_before_capacity_flag=True)):
        got = aclnn.moe_init_routing_quant_v2(xt.to(dev), torch.from_numpy(idx).to(dev), 0, st, ot, expert_num=E, **kw)
        torch.cuda.synchronize()
        want = oracle.moe_init_routing_quant_v2(
            bits, idx, 0, scale, offset, active_num=kw.get("active_num", 0), expert_capacity=kw.get("expert_capacity", 0),
            expert_num=E, drop_pad_mode=kw.get("drop_pad_mode", 0), count_flag=kw.get("expert_tokens_count_or_cumsum_flag", 0),
            before_capacity_flag=kw.get("expert_tokens_before_capacity_flag", False), dtype=code)
        for g, w, name in zip(got, want, ("expandedX", "expandedRowIdx", "countOrCumsum", "beforeCapacity", "dynScale")):
            assert _same(g, w), (kw, name)
        q = got[0].cpu().numpy()
        assert T * H < 1000 or ((q == 127).any() and (q == -128).any())


@pytest.mark.parametrize("T,K,E,H,dtype_name", QUANT_V2_CASES)
@pytest.mark.parametrize("smooth_rows", [None, 1, "E"])
def test_quant_v2_dynamic_bit_exact(aclnn, oracle, dev, T, K, E, H, dtype_name, smooth_rows):
    """Dynamic quantisation with no smooth scale, one shared row, or one row per expert, in the dropless form, with
    activeNum, and in the drop/pad form (unused slots keep zero rows and zero scales)."""
    rng = np.random.default_rng(T * 11 + H)
    xt, bits, idx, code = _quant_v2_inputs(rng, T, K, E, H, dtype_name, oracle)
    smooth = None
    if smooth_rows is not None:
        smooth = (rng.random((1 if smooth_rows == 1 else E, H)) + 0.5).astype(np.float32)
    sm_t = None if smooth is None else torch.from_numpy(smooth).to(dev)
    C = max(1, min(T, (T * K) // E))
    for kw in (dict(expert_tokens_count_or_cumsum_flag=2), dict(expert_tokens_count_or_cumsum_flag=1, active_num=T),
               dict(drop_pad_mode=1, expert_capacity=C, expert_tokens_before_capacity_flag=True)):
        got = aclnn.moe_init_routing_quant_v2(xt.to(dev), torch.from_numpy(idx).to(dev), 1, sm_t, None, expert_num=E, **kw)
        torch.cuda.synchronize()
        want = oracle.moe_init_routing_quant_v2(
            bits, idx, 1, smooth, None, active_num=kw.get("active_num", 0), expert_capacity=kw.get("expert_capacity", 0),
            expert_num=E, drop_pad_mode=kw.get("drop_pad_mode", 0), count_flag=kw.get("expert_tokens_count_or_cumsum_flag", 0),
            before_capacity_flag=kw.get("expert_tokens_before_capacity_flag", False), dtype=code)
        for g, w, name in zip(got, want, ("expandedX", "expandedRowIdx", "countOrCumsum", "beforeCapacity", "dynScale")):
            assert _same(g, w), (kw, name)


def test_quant_v2_outputs_are_rewritten_and_empty_input(aclnn, oracle, dev):
    """Outputs that hold stale data get the same result (drop/pad zeroes its unused slots itself), and zero tokens run."""
    rng = np.random.default_rng(5)
    T, K, E, H, C = 40, 2, 6, 48, 20                      # capacity above what any expert receives: unused slots exist
    xt, bits, idx, code = _quant_v2_inputs(rng, T, K, E, H, "bf16", oracle)
    want = oracle.moe_init_routing_quant_v2(bits, idx, 1, None, None, expert_capacity=C, expert_num=E, drop_pad_mode=1,
                                            before_capacity_flag=True, dtype=code)
    # the binding allocates zeroed outputs; poison them through a second call on pre-filled tensors
    h = aclnn._Handles()
    ex = torch.full((E, C, H), 77, dtype=torch.int8, device=dev)
    ri = torch.full((T * K,), -9, dtype=torch.int32, device=dev)
    bef = torch.full((E,), -9, dtype=torch.int32, device=dev)
    dyn = torch.full((E * C,), 5.0, dtype=torch.float32, device=dev)
    x_dev, idx_dev = xt.to(dev), torch.from_numpy(idx).to(dev)         # held until the call has run
    try:
        args = [h.tensor(x_dev), h.tensor(idx_dev), None, None, 0, C, E, 1, 0, True, 1,
                h.tensor(ex), h.tensor(ri), None, h.tensor(bef), h.tensor(dyn)]
        aclnn._run_two_phase("aclnnMoeInitRoutingQuantV2", args, dev, None)
    finally:
        h.close()
    torch.cuda.synchronize()
    for g, w in zip((ex, ri, bef, dyn), (want[0], want[1], want[3], want[4])):
        assert np.array_equal(g.cpu().numpy(), w)
    assert (want[0].reshape(E * C, H) == 0).all(axis=1).any()          # the case does hold unused slots

    empty = aclnn.moe_init_routing_quant_v2(torch.zeros((0, H), dtype=torch.bfloat16, device=dev),
                                            torch.zeros((0, K), dtype=torch.int32, device=dev), 1, None, None,
                                            expert_num=E, expert_tokens_count_or_cumsum_flag=1)
    torch.cuda.synchronize()
    assert empty[0].shape == (0, H) and empty[2].cpu().tolist() == [0] * E


@pytest.mark.parametrize("T,K,E,active", [(64, 8, 128, 0), (64, 8, 128, 100), (4096, 8, 256, 0), (4096, 8, 256, 5000),
                                          (3000, 4, 5000, 0), (3000, 4, 5000, 777)])
@pytest.mark.parametrize("dtype,H", [(np.float32, 1), (np.int8, 4), (np.float16, 2)])
def test_four_byte_rows_are_copied_by_the_sort(aclnn, oracle, dev, T, K, E, active, dtype, H):
    """Rows of exactly four bytes (the column of per-token scales that the chain routes with a second call) are written by
    the sort's last scatter, without a gather launch: one-workgroup sort, three-kernel sort and the two-pass sort of a wide
    expert range, with and without activeNum cutting the rows off."""
    rng = np.random.default_rng(T + K + E + active + H)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    x = rng.integers(-100, 100, (T, H)).astype(dtype)
    ex, ri, cnt, _ = _run(aclnn, dev, x, idx, active_num=active, expert_num=E, expert_tokens_count_or_cumsum_flag=1)
    ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x, idx, active_num=active, expert_num=E, count_flag=1)
    assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r)
    assert ex.shape == ex_r.shape and np.array_equal(ex.view(np.uint8), ex_r.view(np.uint8))


# ------------------------------------------------------------------------------------------------ sort and gather in one launch
@pytest.mark.parametrize("T,K,E,H,dtype", [
    (1, 1, 4, 16, np.int8),            # one token, one 16-byte packet
    (5, 3, 7, 48, np.int8),            # three packets per row, destinations shared out over thread groups
    (64, 8, 128, 7168, np.int8),       # DeepSeek-V3 row width
    (64, 64, 128, 32, np.float16),     # as many ids per token as the kernel caches
    (256, 2, 512, 4096, np.int8),      # the most tokens (one workgroup each) and the most digit values
    (256, 8, 16, 20480, np.float32),   # rows longer than the workgroup has threads for (81920 bytes = 5120 packets)
    (257, 2, 8, 64, np.int8),          # one token more: one-workgroup sort, then the row gather
    (100, 65, 8, 16, np.int8),         # one id per token more than cached: the same
    (64, 8, 128, 24, np.int8),         # rows not a multiple of 16 bytes: the same
])
def test_decode_sized_calls_sort_and_gather_in_one_launch(aclnn, oracle, dev, T, K, E, H, dtype):
    """Up to 256 tokens whose rows are whole 16-byte packets take one kernel for sort and row gather; the cases either side
    of each limit take the separate kernels.  V2 with and without activeNum, V3 with scales and an expert sub-range."""
    rng = np.random.default_rng(T * 131 + K * 7 + H)
    x = (rng.standard_normal((T, H)) * 50).astype(dtype)
    idx = rng.integers(0, E, (T, K)).astype(np.int32)
    for active in (0, max(1, T * K // 3)):
        for flag in (1, 2):
            ex, ri, cnt, _ = _run(aclnn, dev, x, idx, active_num=active, expert_num=E, expert_tokens_count_or_cumsum_flag=flag)
            ex_r, ri_r, cnt_r, _ = oracle.moe_init_routing_v2(x, idx, active_num=active, expert_num=E, count_flag=flag)
            assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r)
            assert ex.shape == ex_r.shape and np.array_equal(ex.view(np.uint8), ex_r.view(np.uint8))
    scale = rng.random(T).astype(np.float32)
    for rng_ in (None, (E // 4, max(E // 4 + 1, 3 * E // 4))):
        for row_idx_type in (1, 0):
            ex, ri, cnt, es = _run_v3(aclnn, dev, x, idx, scale, expert_num=E, expert_tokens_num_type=1,
                                      active_expert_range=rng_, row_idx_type=row_idx_type)
            ex_r, ri_r, cnt_r, es_r = oracle.moe_init_routing_v3(x, idx, scale, E, rng_, 1, row_idx_type)
            assert np.array_equal(ri, ri_r) and np.array_equal(cnt, cnt_r) and np.array_equal(es, es_r)
            assert np.array_equal(ex.view(np.uint8), ex_r.view(np.uint8))
