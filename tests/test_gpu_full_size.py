"""The path at the benchmark's full sizes (DeepSeek-V3 prefill, its Zipf-skewed 8192-token variant, Mixtral prefill).

The oracle cannot run 10^14 MACs in a test, so each configuration is checked three ways:
  * routing (integer / byte work) against the oracle in full, bit-exact;
  * the two GEMM stages against the oracle on a sample of expanded rows that touches every expert (first and last row of
    every non-empty group plus rows either side of the kernel's 32-row sub-tile boundaries), finalize in full;
  * size-independent properties over ALL rows: the routing index is a permutation and the counts sum to M; negating the
    linear half's weight scales and doubling the down-projection scales gives exactly -2 x the output (sign symmetry of
    every rounding, exactness of powers of two); permuting the tokens permutes the output rows bit for bit (no row's
    result may depend on where its tile falls).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _tile_heights_in_use(pkg, forward):
    """Tile heights of the two grouped GEMM launches of one pass, as the kernels themselves record them."""
    aclnn = pkg.aclnn
    aclnn.gemm_workgroup_spans_enable(True)
    try:
        forward()
        spans = aclnn.gemm_workgroup_spans_report()
    finally:
        aclnn.gemm_workgroup_spans_enable(False)
    assert set(spans) >= {"gmm_swiglu", "gmm_dequant"}, spans.keys()
    return sorted({spans["gmm_swiglu"]["tile_rows"], spans["gmm_dequant"]["tile_rows"]})


def _sample_rows(cumsum, per_group_extra, seed, tile_heights=(256,)):
    """First and last row of every non-empty group, the rows either side of every 32-row MFMA sub-tile edge up to the
    tallest tile, and, for each tile height in use, the rows either side of the tile's end, of the boundary between its
    two wave rows (wave row 0 takes the first ceil(active / 2) sub-tiles of a tile with `active` occupied ones) in the
    group's last, partly filled tile, and of every further whole tile; plus random rows."""
    rng = np.random.default_rng(seed)
    start = np.concatenate([[0], cumsum[:-1]]).astype(np.int64)
    rows = []
    for s, e in zip(start, cumsum.astype(np.int64)):
        if e <= s:
            continue
        n = e - s
        offs = {0, n - 1}
        for b in range(32, 257, 32):                   # sub-tile edges: 31/32, 63/64, ..., 255/256
            offs.update((b - 1, b))
        for th in tile_heights:
            for t0 in range(0, int(n), th):            # every m-tile of the group at this height
                offs.update((t0 - 1, t0))
                active = (min(th, n - t0) + 31) // 32
                split = t0 + 32 * ((active + 1) // 2)  # first row of wave row 1
                offs.update((split - 1, split))
        rows += [s + o for o in offs if 0 <= o < n]
        if per_group_extra:
            rows += list(rng.integers(s, e, size=per_group_extra))
    return np.unique(np.array(rows, dtype=np.int64))


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _run_config(pkg, oracle, dev, cfg_index, weights, seed, max_rows, per_group_extra=0, routing="v2"):
    """routing = "v2": the chain as the path is named, aclnnMoeInitRoutingV2 at its head (int8 rows, then the scale
    column, int32 cumsum); "v3": one aclnnMoeInitRoutingV3 call (rows and scales together, int64 cumsum)."""
    cfg = pkg.synth.config(cfg_index)
    idx, wgt = pkg.synth.make_routing(cfg, seed=seed)
    xq, xs = pkg.synth.make_activations(cfg, seed=seed)
    w13, w13s, w2, w2s = weights
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, routing=routing)
    assert ffn.routing == routing
    t = lambda a: torch.from_numpy(a).to(dev)
    d_xq, d_xs, d_idx, d_wgt = t(xq), t(xs), t(idx), t(wgt)
    out = ffn.forward(d_xq, d_xs, d_idx, d_wgt).clone()
    torch.cuda.synchronize()
    M, E = cfg.tokens * cfg.top_k, cfg.experts

    # ---- routing in full
    ex, row_idx, cumsum, _ = oracle.moe_init_routing_v2(xq, idx, expert_num=E, count_flag=1)
    xs_exp, _, _, _ = oracle.moe_init_routing_v2(xs.reshape(-1, 1), idx, expert_num=E)
    got_idx = ffn.expanded_row_idx.cpu().numpy()
    assert np.array_equal(got_idx, row_idx)
    assert np.array_equal(np.sort(got_idx), np.arange(M, dtype=np.int32))
    assert np.array_equal(ffn.cumsum.cpu().numpy(), cumsum) and cumsum[-1] == M
    assert np.array_equal(ffn.expanded_x.cpu().numpy(), ex)
    assert np.array_equal(ffn.expanded_scale.cpu().numpy().reshape(-1), xs_exp.reshape(-1))

    # ---- GEMM stages on sampled rows
    heights = _tile_heights_in_use(pkg, lambda: ffn.forward(d_xq, d_xs, d_idx, d_wgt))
    rows = _sample_rows(cumsum, per_group_extra, seed, tile_heights=heights)
    if rows.shape[0] > max_rows:
        # keep every group's first and last row, draw the rest
        start = np.concatenate([[0], cumsum[:-1]]).astype(np.int64)
        ends = np.unique(np.concatenate([start[cumsum > start], cumsum[cumsum > start].astype(np.int64) - 1]))
        rest = np.setdiff1d(rows, ends)
        keep = np.random.default_rng(seed).choice(rest.shape[0], max(max_rows - ends.shape[0], 0), replace=False)
        rows = np.union1d(ends, rest[keep])
    gl = cumsum.astype(np.int64)
    w13n, w13sn = w13.cpu().numpy(), w13s.cpu().numpy()
    h, hs = oracle.grouped_matmul_swiglu_quant(ex, w13n, w13sn, xs_exp.reshape(-1), gl, w_trans=True, rows=rows)
    del w13n
    h_gpu, hs_gpu = ffn.h.cpu().numpy(), ffn.h_scale.cpu().numpy()
    assert np.abs(h_gpu[rows].astype(np.int32) - h.astype(np.int32)).max() <= 1
    assert (h_gpu[rows] != h).mean() < 0.02          # one-LSB flips are rare, not systematic
    np.testing.assert_allclose(hs_gpu[rows], hs, rtol=1e-2)
    w2n, w2sn = w2.cpu().numpy(), w2s.cpu().numpy()
    y = oracle.grouped_matmul_dequant(h_gpu, w2n, w2sn, hs_gpu, gl, w_trans=True, out_dtype=oracle.DT_BF16, rows=rows)
    del w2n
    y_gpu = _bits(ffn.y)
    assert np.array_equal(y_gpu[rows], y)

    # ---- finalize in full on the GPU's own y
    ref = oracle.moe_finalize_routing_v2(y_gpu, row_idx, scales=wgt, drop_pad_mode=2, dtype=oracle.DT_BF16,
                                         scale_dtype=oracle.DT_F32)
    out_bits = _bits(out)
    assert np.array_equal(out_bits, ref)
    assert np.isfinite(out.float().cpu().numpy()).all()

    # ---- sign symmetry and linearity: negating the scales of the linear (second) half of the gate/up channels negates
    # S, hence h (round-to-nearest-even is odd) and leaves its row scale alone; doubling the down-projection scales
    # doubles y.  Both are exact in every rounding, so out' == -2 out bit for bit, over all rows.
    I = cfg.inter
    w13s_neg = w13s.clone()
    w13s_neg[:, I:] *= -1.0
    ffn2 = pkg.MoeFfnW8A8(w13, w13s_neg, w2, w2s * 2.0, routing=routing)
    out2 = ffn2.forward(d_xq, d_xs, d_idx, d_wgt)
    torch.cuda.synchronize()
    assert np.array_equal(ffn2.h.cpu().numpy(), -h_gpu)
    assert np.array_equal(ffn2.h_scale.cpu().numpy(), hs_gpu)
    assert torch.equal(out2.float(), out.float() * -2.0)
    del ffn2, out2

    # ---- permutation of the tokens permutes the output rows
    perm = torch.from_numpy(np.random.default_rng(seed + 7).permutation(cfg.tokens)).to(dev)
    out3 = ffn.forward(d_xq[perm].contiguous(), d_xs[perm].contiguous(), d_idx[perm].contiguous(),
                       d_wgt[perm].contiguous())
    torch.cuda.synchronize()
    assert np.array_equal(_bits(out3), out_bits[perm.cpu().numpy()])
    return cumsum


@pytest.fixture(scope="module")
def deepseek_weights(pkg, dev):
    w = pkg.synth.make_weights(pkg.synth.config(1), dev, seed=1)
    yield w
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("routing", ["v2", "v3"])
def test_deepseek_v3_prefill_full_size(pkg, oracle, dev, deepseek_weights, routing):
    """c1: T=4096, H=7168, I=2048, E=256, top-8 (M=32768, ~128 rows per expert)."""
    cumsum = _run_config(pkg, oracle, dev, 1, deepseek_weights, seed=1, max_rows=4000, routing=routing)
    counts = np.diff(np.concatenate([[0], cumsum]))
    assert counts.min() > 0            # uniform routing touches every expert


@pytest.mark.parametrize("routing", ["v2", "v3"])
def test_deepseek_v3_skewed_full_size(pkg, oracle, dev, deepseek_weights, routing):
    """c4: T=8192 with Zipf(1.2) expert load: empty experts and groups of thousands of rows in one launch."""
    cumsum = _run_config(pkg, oracle, dev, 4, deepseek_weights, seed=4, max_rows=4000, routing=routing)
    counts = np.diff(np.concatenate([[0], cumsum]))
    assert 0.25 <= (counts == 0).mean() <= 0.45 and counts.max() > 10 * counts.mean()   # the benchmark's ~30 % empty experts


def test_skewed_count_list_equals_cumsum_list(pkg, aclnn, dev, deepseek_weights):
    """groupListType 1 (per-group counts) and 0 (cumsum) give identical down-projection output on the skewed load."""
    cfg = pkg.synth.config(4)
    idx, _ = pkg.synth.make_routing(cfg, seed=4)
    M, E, H, I = cfg.tokens * cfg.top_k, cfg.experts, cfg.hidden, cfg.inter
    counts = np.bincount(idx.reshape(-1), minlength=E).astype(np.int64)
    g = torch.Generator(device=dev)
    g.manual_seed(44)
    h = torch.randint(-127, 128, (M, I), dtype=torch.int8, device=dev, generator=g)
    hs = torch.empty((M,), dtype=torch.float32, device=dev).uniform_(1e-3, 1e-2, generator=g)
    _, _, w2, w2s = deepseek_weights
    outs = []
    for list_type, gl in ((0, np.cumsum(counts)), (1, counts)):
        y = torch.empty((M, H), dtype=torch.bfloat16, device=dev)
        aclnn.grouped_matmul_v4([h], [w2.transpose(1, 2)], scale=[w2s], per_token_scale=[hs],
                                group_list=torch.from_numpy(gl).to(dev), split_item=3, group_type=0,
                                group_list_type=list_type, act_type=0, out=[y])
        outs.append(y)
    torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


def test_mixtral_prefill_full_size(pkg, oracle, dev):
    """c2: T=16384, H=4096, I=14336, E=8, top-2 (M=32768, ~4096 rows per expert; N=28672 exceeds the reference's
    10240 limit, which this build lifts)."""
    cfg = pkg.synth.config(2)
    weights = pkg.synth.make_weights(cfg, dev, seed=2)
    _run_config(pkg, oracle, dev, 2, weights, seed=2, max_rows=1024, per_group_extra=40)
