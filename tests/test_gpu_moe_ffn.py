"""The chained path (routing -> gate/up GEMM + SwiGLU + requant -> down GEMM -> finalize) on the GPU against the oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _oracle_chain(oracle, cfg, idx, wgt, xq, xs, w13, w13s, w2, w2s, rows=None):
    E = cfg.experts
    ex, row_idx, cumsum, _ = oracle.moe_init_routing_v2(xq, idx, expert_num=E, count_flag=1)
    xs_exp, _, _, _ = oracle.moe_init_routing_v2(xs.reshape(-1, 1), idx, expert_num=E)
    gl = cumsum.astype(np.int64)
    h, hs = oracle.grouped_matmul_swiglu_quant(ex, w13, w13s, xs_exp.reshape(-1), gl, w_trans=True, rows=rows)
    return ex, row_idx, cumsum, xs_exp.reshape(-1), h, hs


def test_small_config_end_to_end(pkg, oracle, dev):
    """c0 (256 tokens, H=1024, I=1024, E=8, top-2): every stage compared in full."""
    cfg = pkg.synth.config(0)
    idx, wgt = pkg.synth.make_routing(cfg, seed=0)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
    t = lambda a: torch.from_numpy(a).to(dev)
    out = ffn.forward(t(xq), t(xs), t(idx), t(wgt))
    torch.cuda.synchronize()
    w13n, w13sn, w2n, w2sn = w13.cpu().numpy(), w13s.cpu().numpy(), w2.cpu().numpy(), w2s.cpu().numpy()
    ex, row_idx, cumsum, xs_exp, h, hs = _oracle_chain(oracle, cfg, idx, wgt, xq, xs, w13n, w13sn, w2n, w2sn)
    assert np.array_equal(ffn.expanded_row_idx.cpu().numpy(), row_idx)
    assert np.array_equal(ffn.cumsum.cpu().numpy(), cumsum)
    assert np.array_equal(ffn.expanded_x.cpu().numpy(), ex)
    assert np.array_equal(ffn.expanded_scale.cpu().numpy().reshape(-1), xs_exp)
    h_gpu, hs_gpu = ffn.h.cpu().numpy(), ffn.h_scale.cpu().numpy()
    assert np.abs(h_gpu.astype(np.int32) - h.astype(np.int32)).max() <= 1
    np.testing.assert_allclose(hs_gpu, hs, rtol=1e-2)
    # downstream of h the GPU's own int8 activations are fed to the oracle, so one-LSB differences upstream do not blur
    # the check of the down projection and finalize: those must then agree bit for bit
    gl = cumsum.astype(np.int64)
    y = oracle.grouped_matmul_dequant(h_gpu, w2n, w2sn, hs_gpu, gl, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(ffn.y.view(torch.int16).cpu().numpy().view(np.uint16), y)
    ref = oracle.moe_finalize_routing_v2(y, row_idx, scales=wgt, drop_pad_mode=2, dtype=oracle.DT_BF16,
                                         scale_dtype=oracle.DT_F32)
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), ref)
    # and the fully independent oracle chain stays within the bf16 tolerance
    y2 = oracle.grouped_matmul_dequant(h, w2n, w2sn, hs, gl, w_trans=True, out_dtype=oracle.DT_BF16)
    ref2 = oracle.bf16_bits_to_f32(oracle.moe_finalize_routing_v2(y2, row_idx, scales=wgt, drop_pad_mode=2,
                                                                  dtype=oracle.DT_BF16, scale_dtype=oracle.DT_F32))
    got = out.float().cpu().numpy()
    rel = np.abs(got - ref2) / np.maximum(np.abs(ref2), 1e-3 * np.abs(ref2).max())
    assert np.quantile(rel, 0.999) < 1e-2


def test_decode_config_sampled(pkg, oracle, dev):
    """c3 (64 tokens, H=4096, I=1536, E=128, top-8): routing in full, GEMM stages on every expanded row."""
    cfg = pkg.synth.config(3)
    idx, wgt = pkg.synth.make_routing(cfg, seed=3)
    xq, xs = pkg.synth.make_activations(cfg, seed=3)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=3)
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
    t = lambda a: torch.from_numpy(a).to(dev)
    out = ffn.forward(t(xq), t(xs), t(idx), t(wgt))
    torch.cuda.synchronize()
    w13n, w13sn, w2n, w2sn = w13.cpu().numpy(), w13s.cpu().numpy(), w2.cpu().numpy(), w2s.cpu().numpy()
    ex, row_idx, cumsum, xs_exp, h, hs = _oracle_chain(oracle, cfg, idx, wgt, xq, xs, w13n, w13sn, w2n, w2sn)
    assert np.array_equal(ffn.expanded_row_idx.cpu().numpy(), row_idx)
    assert np.array_equal(ffn.cumsum.cpu().numpy(), cumsum)
    h_gpu, hs_gpu = ffn.h.cpu().numpy(), ffn.h_scale.cpu().numpy()
    assert np.abs(h_gpu.astype(np.int32) - h.astype(np.int32)).max() <= 1
    np.testing.assert_allclose(hs_gpu, hs, rtol=1e-2)
    gl = cumsum.astype(np.int64)
    y = oracle.grouped_matmul_dequant(h_gpu, w2n, w2sn, hs_gpu, gl, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(ffn.y.view(torch.int16).cpu().numpy().view(np.uint16), y)
    ref = oracle.moe_finalize_routing_v2(y, row_idx, scales=wgt, drop_pad_mode=2, dtype=oracle.DT_BF16,
                                         scale_dtype=oracle.DT_F32)
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), ref)


def test_v2_and_v3_routing_chains_agree(pkg, dev):
    """The chain routed by one MoeInitRoutingV3 call equals the chain routed by two MoeInitRoutingV2 calls, bit for bit."""
    cfg = pkg.synth.config(0)
    idx, wgt = pkg.synth.make_routing(cfg, seed=0)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    t = lambda a: torch.from_numpy(a).to(dev)
    outs = []
    for routing in ("v3", "v2"):
        ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, routing=routing)
        outs.append(ffn.forward(t(xq), t(xs), t(idx), t(wgt)).clone())
        torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


def test_graph_replays_match_eager(pkg, dev):
    """The pass recorded into a HIP graph: every replay, with eager work and synchronisations in between and new
    contents in the input buffers, equals the eager pass on the same contents bit for bit."""
    cfg = pkg.synth.config(0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
    eager = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
    idx, wgt = pkg.synth.make_routing(cfg, seed=0)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    bufs = [torch.from_numpy(a).to(dev) for a in (xq, xs, idx, wgt)]
    graph, out = ffn.capture(*bufs)
    for seed in (0, 1, 2, 1, 3):
        idx, wgt = pkg.synth.make_routing(cfg, seed=seed)
        xq, xs = pkg.synth.make_activations(cfg, seed=seed)
        fresh = [torch.from_numpy(a).to(dev) for a in (xq, xs, idx, wgt)]
        want = eager.forward(*fresh).clone()          # eager work between the replays
        torch.cuda.synchronize()
        for dst, src in zip(bufs, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), seed


@pytest.mark.parametrize("config", [0, 3])
def test_nz_weight_chain_equals_nd_chain(pkg, dev, config):
    """The chain fed FRACTAL_NZ weights, and the chain fed contiguous row-major [E, K, N] weights, equal the chain fed
    the transposed views of K-contiguous storage, bit for bit (c0, and the decode shape c3 with its 32-row tiles)."""
    cfg = pkg.synth.config(config)
    idx, wgt = pkg.synth.make_routing(cfg, seed=0)
    xq, xs = pkg.synth.make_activations(cfg, seed=0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    t = lambda a: torch.from_numpy(a).to(dev)
    a = pkg.MoeFfnW8A8(w13, w13s, w2, w2s).forward(t(xq), t(xs), t(idx), t(wgt)).clone()
    b = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, weight_nz=True).forward(t(xq), t(xs), t(idx), t(wgt)).clone()
    c = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, weight_row_major=True).forward(t(xq), t(xs), t(idx), t(wgt)).clone()
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(a.view(torch.int16), c.view(torch.int16))


def test_two_host_threads_on_their_own_streams(pkg, dev):
    """All state of a call lives in its executor: two host threads that run the chain at the same time, each on its own
    stream with its own buffers, both get the single-threaded result bit for bit (ctypes drops the interpreter lock
    during the calls, so the first and second phases of the two threads do interleave)."""
    import threading
    cfg = pkg.synth.config(0)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=0)
    t = lambda a: torch.from_numpy(a).to(dev)
    inputs, expected = [], []
    for seed in (11, 12):
        idx, wgt = pkg.synth.make_routing(cfg, seed=seed)
        xq, xs = pkg.synth.make_activations(cfg, seed=seed)
        args = (t(xq), t(xs), t(idx), t(wgt))
        inputs.append(args)
        expected.append(pkg.MoeFfnW8A8(w13, w13s, w2, w2s).forward(*args).clone())
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def work(i):
        try:
            stream = torch.cuda.Stream(device=dev)
            ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s)
            with torch.cuda.stream(stream):
                for _ in range(25):
                    out = ffn.forward(*inputs[i])
                results[i] = out.clone()
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    for got, want in zip(results, expected):
        assert got is not None and torch.equal(got, want)
