"""aclnnGroupedMatmulFinalizeRouting (V1 / V2 / V3 entry points) on the GPU against the CPU oracle.

The operator adds the rows of one token with fp32 atomics, so the order of the additions differs from the oracle's
(ascending row): values are compared within 1e-5 of the largest term added into the output (a sum of top-k products
in fp32), the bound the float64 restatement is held to as well."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(rng, M, K, N, E, batch, topk, ragged=True):
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    w = rng.integers(-127, 128, (E, N, K)).astype(np.int8)          # K-contiguous storage
    if ragged:
        cuts = np.sort(rng.integers(0, M + 1, E - 1)) if E > 1 else np.array([], np.int64)
        cumsum = np.concatenate([cuts, [M]]).astype(np.int64)
    else:
        cumsum = (np.arange(1, E + 1) * (M // E)).astype(np.int64)
        cumsum[-1] = M
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    logit = rng.random(M).astype(np.float32)
    row_index = np.resize(np.repeat(np.arange(batch), topk), M).astype(np.int64)
    rng.shuffle(row_index)
    return x, w, cumsum, scale, pt, logit, row_index


def _tolerance(oracle, x, w, cumsum, scale, pt, logit):
    y = oracle.grouped_matmul_dequant(x, w, scale, pt, cumsum, w_trans=True, out_dtype=oracle.DT_F32)
    return 1e-5 * np.abs(y * (1.0 if logit is None else logit[:, None])).max()


SHAPES = [  # M, K, N, E, batch, topk
    (8, 128, 256, 1, 8, 1), (96, 256, 320, 5, 24, 4), (300, 512, 520, 7, 75, 4), (512, 1536, 4096, 128, 64, 8),
    (700, 384, 256, 3, 175, 4), (1024, 2048, 7168, 8, 128, 8),
]


@pytest.mark.parametrize("M,K,N,E,batch,topk", SHAPES)
def test_combine_against_oracle(aclnn, oracle, dev, M, K, N, E, batch, topk):
    rng = np.random.default_rng(M + N)
    x, w, cumsum, scale, pt, logit, row_index = _case(rng, M, K, N, E, batch, topk)
    t = lambda a: torch.from_numpy(a).to(dev)
    wv = t(w).transpose(1, 2)
    out = aclnn.grouped_matmul_finalize_routing(t(x), wv, t(scale), t(row_index), batch, t(cumsum), group_list_type=0,
                                                per_token_scale=t(pt), logit=t(logit))
    torch.cuda.synchronize()
    ref = oracle.grouped_matmul_finalize_routing(x, w, scale, row_index, batch, cumsum, list_type=0, w_trans=True,
                                                 per_token=pt, logit=logit)
    tol = _tolerance(oracle, x, w, cumsum, scale, pt, logit)
    assert np.abs(out.cpu().numpy() - ref).max() <= tol
    # twice in a row gives the same thing up to the same bound: the output is initialised by the operator itself
    out2 = aclnn.grouped_matmul_finalize_routing(t(x), wv, t(scale), t(row_index), batch, t(cumsum), group_list_type=0,
                                                 per_token_scale=t(pt), logit=t(logit), out=out)
    torch.cuda.synchronize()
    assert np.abs(out2.cpu().numpy() - ref).max() <= tol


@pytest.mark.parametrize("version", [1, 2, 3])
def test_all_inputs_and_entry_points(aclnn, oracle, dev, version):
    """bias (bf16), shared rows (bf16, offset), int32 row index, count list, bf16 channel scale, plain [E, K, N] weight."""
    rng = np.random.default_rng(version)
    M, K, N, E, batch, topk = 200, 256, 384, 6, 50, 4
    x, w, cumsum, scale, pt, logit, row_index = _case(rng, M, K, N, E, batch, topk)
    counts = np.diff(np.concatenate([[0], cumsum])).astype(np.int64)
    bias_bits = oracle.f32_to_bf16_bits(rng.standard_normal((E, N)).astype(np.float32))
    scale_bits = oracle.f32_to_bf16_bits(scale)
    shared_bits = oracle.f32_to_bf16_bits(rng.standard_normal((7, N)).astype(np.float32))
    t = lambda a: torch.from_numpy(a).to(dev)
    bf = lambda bits: torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(dev)
    w_plain = np.ascontiguousarray(w.transpose(0, 2, 1))             # [E, K, N] storage: the byte-wise kernel
    for weight, ri in ((t(w).transpose(1, 2), t(row_index)), (t(w_plain), t(row_index.astype(np.int32)))):
        out = aclnn.grouped_matmul_finalize_routing(t(x), weight, bf(scale_bits), ri, batch, t(counts), group_list_type=1,
                                                    bias=bf(bias_bits), per_token_scale=t(pt), logit=t(logit),
                                                    shared_input=bf(shared_bits), shared_input_weight=0.25,
                                                    shared_input_offset=20, version=version)
        torch.cuda.synchronize()
        ref = oracle.grouped_matmul_finalize_routing(x, w, scale_bits, row_index, batch, counts, list_type=1, w_trans=True,
                                                     bias=bias_bits, per_token=pt, logit=logit, shared=shared_bits,
                                                     shared_offset=20, shared_weight=0.25, scale_dtype=oracle.DT_BF16)
        tol = max(_tolerance(oracle, x, w, cumsum, oracle.bf16_bits_to_f32(scale_bits), pt, logit), 1e-5)
        assert np.abs(out.cpu().numpy() - ref).max() <= tol


def test_optional_inputs_absent_and_rows_left_out(aclnn, oracle, dev):
    rng = np.random.default_rng(9)
    M, K, N, E, batch, topk = 160, 128, 256, 4, 40, 4
    x, w, cumsum, scale, pt, logit, row_index = _case(rng, M, K, N, E, batch, topk)
    cumsum[-1] = cumsum[-2]                                          # the last group is empty: trailing rows belong to no group
    row_index[:5] = [-1, batch, batch + 3, 0, 1]                     # indices outside the output are skipped
    t = lambda a: torch.from_numpy(a).to(dev)
    out = aclnn.grouped_matmul_finalize_routing(t(x), t(w).transpose(1, 2), t(scale), t(row_index), batch, t(cumsum),
                                                group_list_type=0, tuning_config=[M // E])
    torch.cuda.synchronize()
    ref = oracle.grouped_matmul_finalize_routing(x, w, scale, row_index, batch, cumsum, list_type=0, w_trans=True)
    assert np.abs(out.cpu().numpy() - ref).max() <= _tolerance(oracle, x, w, cumsum, scale, None, None)


def test_fused_chain_matches_unfused_chain(pkg, dev):
    """The FFN chain ending in the fused operator agrees with the chain ending in GroupedMatmulV4 + MoeFinalizeRoutingV2
    to bf16 resolution (the unfused chain rounds every expanded row to bf16 before the combine, the fused one does not)."""
    cfg = pkg.synth.config(0)
    idx, wgt = pkg.synth.make_routing(cfg, seed=0)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    t = lambda a: torch.from_numpy(a).to(dev)
    plain = pkg.MoeFfnW8A8(w13, w13s, w2, w2s).forward(t(xq), t(xs), t(idx), t(wgt)).float().clone()
    fused = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, routing="v3", fused_combine=True).forward(t(xq), t(xs), t(idx), t(wgt)).clone()
    torch.cuda.synchronize()
    assert fused.dtype == torch.float32
    err = (fused - plain).abs().max().item()
    assert err <= 2e-2 * plain.abs().max().item(), err


@pytest.mark.parametrize("version", [1, 2])
def test_weight_nz_entry_points(aclnn, oracle, dev, version):
    """aclnnGroupedMatmulFinalizeRoutingWeightNz / WeightNzV2: the blocked weight gives what the ND weight gives (to the
    bound of the atomic order) and agrees with the oracle."""
    rng = np.random.default_rng(20 + version)
    M, K, N, E, batch, topk = 300, 512, 544, 7, 75, 4
    x, w, cumsum, scale, pt, logit, row_index = _case(rng, M, K, N, E, batch, topk)
    w_nz = np.ascontiguousarray(w.reshape(E, N // 32, 32, K // 16, 16).transpose(0, 1, 3, 4, 2))   # from [E, N, K] storage
    t = lambda a: torch.from_numpy(a).to(dev)
    counts = np.diff(np.concatenate([[0], cumsum])).astype(np.int64)
    out = aclnn.grouped_matmul_finalize_routing(t(x), None, t(scale), t(row_index), batch, t(counts), group_list_type=1,
                                                per_token_scale=t(pt), logit=t(logit), version=version, weight_nz=t(w_nz))
    torch.cuda.synchronize()
    ref = oracle.grouped_matmul_finalize_routing(x, w, scale, row_index, batch, counts, list_type=1, w_trans=True,
                                                 per_token=pt, logit=logit)
    assert np.abs(out.cpu().numpy() - ref).max() <= _tolerance(oracle, x, w, cumsum, scale, pt, logit)
