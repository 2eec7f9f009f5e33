"""Benchmark of the quantized MoE expert-FFN path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu-baseline] [--calibration-copy]
                    [--fused-combine] [--graph] [--weight-nz | --weight-row-major]

A step is one pass of the path (routing -> gate/up GEMM + SwiGLU + requant -> down GEMM -> finalize) over one batch of
synthetic tokens whose inputs and expert weights are already resident in HBM.  Prints ONE JSON line: tokens/s for the
whole pass, the roofline of the dominant kernel (the gate/up grouped GEMM) from HIP-event durations recorded inside the
library during the timed steps, and the CPU oracle timed on a bounded sample of the same workload.

--calibration-copy appends, after the timed region, a few launches of the library's plain 1 GiB copy kernel: under
`rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` its counter readings give the factor that converts the counters to
bytes.  roofline.traffic is read from the text summary of those counter runs under profiles/ (null when there is none
for the workload): a counter run is a separate profiler pass and cannot happen inside this process.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gmm_swiglu_{config}_hbm_traffic.txt")
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0      # dense int8 MFMA (5.0 POP/s)


def _cpu_baseline(pkg, oracle, cfg, idx, wgt, xq, xs, ffn, sample_experts=4):
    """Times the oracle: routing and finalize in full, the two GEMM stages on the rows of a few experts (the heaviest
    included), extrapolated linearly in rows.  Returns (tokens/s, description)."""
    import torch
    E, K, T = cfg.experts, cfg.top_k, cfg.tokens
    M = T * K
    t0 = time.perf_counter()
    ex, row_idx, cumsum, _ = oracle.moe_init_routing_v2(xq, idx, expert_num=E, count_flag=1)
    xs_exp, _, _, _ = oracle.moe_init_routing_v2(xs.reshape(-1, 1), idx, expert_num=E)
    t_route = time.perf_counter() - t0
    counts = np.diff(np.concatenate([[0], cumsum]))
    order = np.argsort(-counts, kind="stable")
    chosen = sorted(set([int(order[0])] + [int(e) for e in order[len(order) // 2: len(order) // 2 + sample_experts - 1]]))
    chosen = [e for e in chosen if counts[e] > 0]
    starts = np.concatenate([[0], cumsum])[:-1]
    rows = np.concatenate([np.arange(starts[e], starts[e] + counts[e]) for e in chosen])
    sub_x = ex[rows]
    sub_xs = xs_exp.reshape(-1)[rows]
    sub_gl = np.cumsum([counts[e] for e in chosen]).astype(np.int64)
    ce = torch.tensor(chosen, device=ffn.device)
    w13 = ffn.w13_view.transpose(1, 2)[ce].cpu().numpy()   # [e, 2I, H] storage
    w13s = ffn.w13_scale[ce].cpu().numpy()
    w2 = ffn.w2_view.transpose(1, 2)[ce].cpu().numpy()
    w2s = ffn.w2_scale[ce].float().cpu().numpy()
    t0 = time.perf_counter()
    h, hs = oracle.grouped_matmul_swiglu_quant(sub_x, w13, w13s, sub_xs, sub_gl, w_trans=True)
    y_sub = oracle.grouped_matmul_dequant(h, w2, w2s, hs, sub_gl, w_trans=True, out_dtype=oracle.DT_BF16)
    t_gemm = time.perf_counter() - t0
    y = np.zeros((M, cfg.hidden), np.uint16)
    y[rows] = y_sub
    t0 = time.perf_counter()
    oracle.moe_finalize_routing_v2(y, row_idx, scales=wgt, drop_pad_mode=2, dtype=oracle.DT_BF16, scale_dtype=oracle.DT_F32)
    t_fin = time.perf_counter() - t0
    total = t_route + t_fin + t_gemm * (M / float(len(rows)))
    desc = ("routing and finalize in full; both GEMM stages on the %d expanded rows of experts %s (of %d rows), "
            "extrapolated linearly in rows" % (len(rows), chosen, M))
    return T / total, desc


def _recorded_traffic(config_name):
    """HBM bytes per launch of the gate/up GEMM from the committed counter summary ("traffic_bytes_per_launch: N")."""
    path = TRAFFIC_FILE.format(config=config_name.split("_")[0])
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            return float(line.split(":", 1)[1])
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c1")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="replay the pass from a HIP graph (second phases only) instead of calling the operators eagerly")
    ap.add_argument("--weight-nz", action="store_true",
                    help="give the GEMM operators FRACTAL_NZ weights ([E, N/32, K/16, 16, 32]) instead of transposed views")
    ap.add_argument("--weight-row-major", action="store_true",
                    help="give the GEMM operators contiguous row-major [E, K, N] weights (the reference's plain ND layout)")
    ap.add_argument("--fused-combine", action="store_true",
                    help="end the chain with aclnnGroupedMatmulFinalizeRoutingV3 instead of GroupedMatmulV4 + MoeFinalizeRoutingV2")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (expert parallelism is a design note only); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__ as graft
    pkg = graft.load_package()
    if not os.path.exists(pkg.library_path()):
        graft.build()
    aclnn = pkg.aclnn
    aclnn.lib()
    dev = torch.device("cuda:0")
    cfg = pkg.synth.config(args.config)
    seed = pkg.synth.CONFIGS.index(cfg)

    idx, wgt = pkg.synth.make_routing(cfg, seed=seed)
    xq, xs = pkg.synth.make_activations(cfg, seed=seed)
    w13, w13s, w2, w2s = pkg.synth.make_weights(cfg, dev, seed=seed)
    ffn = pkg.MoeFfnW8A8(w13, w13s, w2, w2s, fused_combine=args.fused_combine, weight_nz=args.weight_nz,
                         weight_row_major=args.weight_row_major)
    d_xq, d_xs = torch.from_numpy(xq).to(dev), torch.from_numpy(xs).to(dev)
    d_idx, d_wgt = torch.from_numpy(idx).to(dev), torch.from_numpy(wgt).to(dev)

    if args.graph:
        graph, _ = ffn.capture(d_xq, d_xs, d_idx, d_wgt)
        step = graph.replay
    else:
        step = lambda: ffn.forward(d_xq, d_xs, d_idx, d_wgt)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    aclnn.kernel_timer_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    if args.graph:
        # a replay runs no host code of the library, so its event timer sees nothing: the per-kernel durations come
        # from the same number of eager passes run right after the timed region
        for _ in range(args.steps):
            ffn.forward(d_xq, d_xs, d_idx, d_wgt)
        torch.cuda.synchronize()
    kernels = aclnn.kernel_timer_report()
    aclnn.kernel_timer_enable(False)
    if args.calibration_copy:
        src = torch.empty(1 << 30, dtype=torch.int8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            aclnn.calibration_copy(dst, src)
        torch.cuda.synchronize()
        del src, dst

    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = cfg.tokens / (elapsed / args.steps)
    counts = np.bincount(idx.reshape(-1), minlength=cfg.experts)
    touched = int((counts > 0).sum())
    work = pkg.synth.algorithmic_work(cfg, touched)
    M, H, I = cfg.tokens * cfg.top_k, cfg.hidden, cfg.inter

    # dominant kernel: the gate/up grouped GEMM.  Algorithmic bytes of one launch: the touched experts' gate/up weights
    # and channel scales, the expanded int8 rows and their scales in, the int8 activations and their scales out.
    gemm1_bytes = touched * 2 * H * I + touched * 2 * I * 4 + M * H + M * 4 + M * I + M * 4
    gemm1_ops = 4 * M * H * I
    n1, total1 = kernels.get("gmm_swiglu", (0, 0.0))
    gemm1_ms = total1 / max(n1, 1)
    hbm_frac = gemm1_bytes / (gemm1_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if gemm1_ms > 0 else None
    mfma_frac = gemm1_ops / (gemm1_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS if gemm1_ms > 0 else None
    # bound of the kernel at this shape: time at HBM peak vs time at MFMA peak
    t_hbm = gemm1_bytes / (HBM_PEAK_GBS * 1e9)
    t_mfma = gemm1_ops / (INT8_PEAK_TOPS * 1e12)
    if t_hbm >= t_mfma:
        roofline = {"bound": "hbm", "achieved": gemm1_bytes / (gemm1_ms * 1e-3) / 1e9 if gemm1_ms else None,
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_frac, "traffic": _recorded_traffic(cfg.name)}
    else:
        roofline = {"bound": "mfma", "achieved": gemm1_ops / (gemm1_ms * 1e-3) / 1e12 if gemm1_ms else None,
                    "peak": INT8_PEAK_TOPS, "unit": "TFLOP/s", "frac": mfma_frac, "traffic": _recorded_traffic(cfg.name)}
    roofline.update({"kernel": "StreamGemmKernel<..., kSwiglu> (gate/up GEMM + SwiGLU; timer name gmm_swiglu)", "kernel_ms": gemm1_ms,
                     "algorithmic_bytes": gemm1_bytes, "algorithmic_ops": gemm1_ops,
                     "hbm_frac": hbm_frac, "mfma_frac": mfma_frac})

    result = {
        "metric": "MoE FFN tokens/s (W8A8 expert FFN: routing + gate/up GEMM + SwiGLU + requant + down GEMM + finalize), 1 GPU",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "%s: %d tokens, H=%d, I=%d, E=%d, top-%d, %s routing" % (
            cfg.name, cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.top_k,
            "Zipf(%.1f)" % cfg.skew if cfg.skew else "uniform random"),
            "expanded_rows": M, "experts_touched": touched, "weight_layout": "FRACTAL_NZ" if args.weight_nz else "row-major [E, K, N]" if args.weight_row_major
            else "K-contiguous (transposed view)",
            "chain": "V3 routing, SwiGLU GEMM, " + ("fused down GEMM + combine" if args.fused_combine else "down GEMM, finalize"),
            "launch": "HIP graph replay" if args.graph else "eager two-phase calls"},
        "end_to_end": {"tops": work["ops"] / (elapsed / args.steps) / 1e12, "gbps": work["bytes"] / (elapsed / args.steps) / 1e9,
                       "mfma_frac": work["ops"] / (elapsed / args.steps) / 1e12 / INT8_PEAK_TOPS,
                       "hbm_frac": work["bytes"] / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS,
                       "algorithmic_ops": work["ops"], "algorithmic_bytes": work["bytes"]},
        "kernels_ms": {k: v[1] / max(v[0], 1) * (v[0] / float(args.steps)) for k, v in sorted(kernels.items())},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        oracle = graft.load_oracle()
        oracle.build()
        v, desc = _cpu_baseline(pkg, oracle, cfg, idx, wgt, xq, xs, ffn)
        result["cpu_baseline"] = {"value": v, "unit": "tokens/s", "cores": oracle.num_threads(), "kind": "port",
                                  "sample": desc}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
