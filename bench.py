"""Benchmark of the quantized MoE expert-FFN path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu-baseline] [--no-other-configs]
                    [--calibration-copy] [--fused-combine] [--graph] [--routing v2|v3]
                    [--weight-nz | --weight-row-major]

A step is one pass of the path (routing -> gate/up GEMM + SwiGLU + requant -> down GEMM -> finalize) over one batch of
synthetic tokens whose inputs and expert weights are already resident in HBM.  Prints ONE JSON line: tokens/s for the
whole pass -- the K passes run as --repeats consecutive blocks, each between two device synchronisations with nothing
else in the stream, and ms_per_step is the median block (fastest, slowest and the mean over all passes are printed
beside it) --, the rooflines of the two grouped GEMM kernels (`roofline`: the dominant one, gate/up; `roofline_down_gemm`)
from HIP-event durations recorded inside the library, on the launch stream, during up to 20 further passes run right
after (an event pair around every launch costs the stream ~10 us, which is why the two sets of passes are separate;
`ms_per_step_kernel_timer_on` reports the second set), the workspace bytes each operator's first phase asked for, and
the CPU oracle timed on a bounded sample of the same workload.

The headline (`value`, `roofline`) is the configuration named by --config (default c1, the DeepSeek-V3 prefill shape
the target is quoted on) behind the routing operator named by --routing (default v2: aclnnMoeInitRoutingV2 on the int8
rows and on the column of per-token scales), run eagerly.  The same line carries, under `other_configs`, a shorter
measurement of the other halves of the metric: the decode shape c3 (eager and as a HIP-graph replay: HBM-bound), the
Mixtral prefill shape c2 (the MFMA-bound one), the skewed shape c4, and c1 again as a graph replay and behind the other
routing operator -- each with its ms per pass, per-kernel durations and both kernels' rooflines from the same timer
(min(K, 20) passes each; ten times as many for the 0.4 ms decode pass, so that a block between two synchronisations is
long against them -- with --config c3 give --steps 200 or more for the same reason).

--calibration-copy appends, after the timed region, a few launches of the library's plain 1 GiB copy kernel: under
`rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` its counter readings give the factor that converts the counters to
bytes.  roofline.traffic is a RECORDED figure: a counter run is a separate profiler pass and cannot happen inside this
process, so the value is read from the text summary of those counter runs under profiles/, which names the hash of the
kernel sources it was taken on; it is null when there is no summary for the workload or when the kernel sources have
changed since (roofline.traffic_source says which).
"""
import argparse
import gc
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gmm_swiglu_{config}_hbm_traffic.txt")
KERNEL_SOURCES = ["grouped_gemm_i8.hip", "grouped_gemm_i8_kernels.h", "grouped_gemm_i8.h", "opapi_common.h"]
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0      # dense int8 MFMA (5.0 POP/s)


def kernel_source_hash():
    """sha256 (first 16 hex digits) over the source files of the grouped GEMM kernels, in a fixed order."""
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "ops-transformer_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


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
    """(bytes or None, description) of the gate/up GEMM's HBM traffic from the committed counter summary: per launch,
    times the launches of one pass where the operator runs in row bands (like `kernel_ms`).

    The summary carries "traffic_bytes_per_launch: N" and "kernel_source_sha256: H" (hash of the kernel sources the
    counters were read on, see kernel_source_hash); a figure taken on other sources is not reported."""
    path = TRAFFIC_FILE.format(config=config_name.split("_")[0])
    rel = os.path.relpath(path, ROOT)
    now = kernel_source_hash()
    if not os.path.exists(path):
        return None, {"file": None, "kernel_source_sha256": now, "note": "no counter summary for this workload"}
    value, taken_on = None, None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            value = float(line.split(":", 1)[1])
        if line.startswith("kernel_source_sha256:"):
            taken_on = line.split(":", 1)[1].strip()
    src = {"file": rel, "recorded_on_kernel_source_sha256": taken_on, "kernel_source_sha256": now,
           "note": "recorded by separate rocprofv3 --pmc runs, not measured by this run"}
    if taken_on != now:
        src["note"] = "the counter summary was taken on other kernel sources: not reported"
        return None, src
    return value, src


def _kernel_roofline(name, kernel, timer_name, nbytes, ops, kernels, passes, traffic=None, traffic_source=None):
    """Roofline block of one grouped GEMM kernel from the library's event timer: both fractions, and as `bound` the
    roof that is the lower one for the kernel's algorithmic bytes and ops.  The bytes and ops are those of the operator's
    GEMM over all rows; where the operator runs in row bands (the SwiGLU operator above 512 MiB of fp32 result) its
    kernel is launched once per band, `launches_per_pass` says how often, and `kernel_ms` is the sum over the bands of
    one pass, i.e. the average launch duration times `launches_per_pass`."""
    n, total = kernels.get(timer_name, (0, 0.0))
    ms = total / max(passes, 1)
    hbm_frac = nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS if ms > 0 else None
    mfma_frac = ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS if ms > 0 else None
    t_hbm = nbytes / (HBM_PEAK_GBS * 1e9)
    t_mfma = ops / (INT8_PEAK_TOPS * 1e12)
    if t_hbm >= t_mfma:
        roofline = {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9 if ms else None,
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_frac, "traffic": traffic}
    else:
        roofline = {"bound": "mfma", "achieved": ops / (ms * 1e-3) / 1e12 if ms else None,
                    "peak": INT8_PEAK_TOPS, "unit": "TFLOP/s", "frac": mfma_frac, "traffic": traffic}
    if traffic_source is not None:
        roofline["traffic_source"] = traffic_source
    roofline.update({"kernel": kernel, "kernel_ms": ms, "launches_timed": n, "launches_per_pass": n / float(max(passes, 1)),
                     "algorithmic_bytes": nbytes,
                     "algorithmic_ops": ops, "hbm_frac": hbm_frac, "mfma_frac": mfma_frac,
                     "time_at_hbm_peak_ms": t_hbm * 1e3, "time_at_mfma_peak_ms": t_mfma * 1e3})
    return roofline


def _gate_up_roofline(cfg, touched, kernels, passes):
    """Gate/up grouped GEMM.  Algorithmic bytes of one launch: the touched experts' gate/up weights and channel scales,
    the expanded int8 rows and their scales in, the int8 activations and their scales out.  Ops: 4 * M * H * I."""
    M, H, I = cfg.tokens * cfg.top_k, cfg.hidden, cfg.inter
    nbytes = touched * 2 * H * I + touched * 2 * I * 4 + M * H + M * 4 + M * I + M * 4
    traffic, traffic_source = _recorded_traffic(cfg.name)
    return _kernel_roofline("gate_up", "StreamGemmKernel<..., kSwiglu> (gate/up GEMM + SwiGLU; timer name gmm_swiglu)",
                            "gmm_swiglu", nbytes, 4 * M * H * I, kernels, passes, traffic, traffic_source)


def _down_roofline(cfg, touched, kernels, passes):
    """Down-projection grouped GEMM.  Algorithmic bytes of one launch: the touched experts' down weights and channel
    scales, the int8 activations and their scales in, the bf16 rows out.  Ops: 2 * M * H * I."""
    M, H, I = cfg.tokens * cfg.top_k, cfg.hidden, cfg.inter
    nbytes = touched * H * I + touched * H * 4 + M * I + M * 4 + M * H * 2
    return _kernel_roofline("down", "StreamGemmKernel<..., kDequant> (down GEMM + dequant; timer name gmm_dequant)",
                            "gmm_dequant", nbytes, 2 * M * H * I, kernels, passes)


class Workload:
    """One configuration resident on the GPU: routing inputs, quantised activations, expert weights, the chain."""

    def __init__(self, pkg, cfg, dev, routing="v2", **ffn_kwargs):
        import torch
        self.pkg, self.cfg, self.dev = pkg, cfg, dev
        seed = pkg.synth.CONFIGS.index(cfg)
        self.idx, self.wgt = pkg.synth.make_routing(cfg, seed=seed)
        self.xq, self.xs = pkg.synth.make_activations(cfg, seed=seed)
        self.weights = pkg.synth.make_weights(cfg, dev, seed=seed)
        self.ffn_kwargs = ffn_kwargs
        self.ffn = pkg.MoeFfnW8A8(*self.weights, routing=routing, **ffn_kwargs)
        self.d_xq, self.d_xs = torch.from_numpy(self.xq).to(dev), torch.from_numpy(self.xs).to(dev)
        self.d_idx, self.d_wgt = torch.from_numpy(self.idx).to(dev), torch.from_numpy(self.wgt).to(dev)
        self.touched = int((np.bincount(self.idx.reshape(-1), minlength=cfg.experts) > 0).sum())

    def with_routing(self, routing):
        """The same tensors behind a chain that starts with another routing operator."""
        other = object.__new__(Workload)
        other.__dict__.update(self.__dict__)
        other.ffn = self.pkg.MoeFfnW8A8(*self.weights, routing=routing, **self.ffn_kwargs)
        return other

    def measure(self, steps, warmup, graph=False, repeats=5):
        """Times `steps` passes (after `warmup` untimed ones) as `repeats` consecutive blocks, each between two device
        synchronisations with nothing else in the stream; the figure reported per pass is the median block (minimum,
        maximum and the mean over all `steps` passes are kept beside it).  Then runs min(steps, 20) further eager passes
        with the library's HIP-event timer on for the per-kernel durations.

        The timer brackets every kernel launch with a pair of events on the launch stream; on this runtime each pair
        costs the stream about 10 us between kernels (0.08 ms over the eight launches of a decode pass), so the passes
        that give tokens/s run with the timer off and the passes that give the kernel durations follow immediately, in
        the same process, on the same buffers."""
        import torch
        aclnn = self.pkg.aclnn
        args = (self.d_xq, self.d_xs, self.d_idx, self.d_wgt)
        if graph:
            g, _ = self.ffn.capture(*args)
            step = g.replay
        else:
            step = lambda: self.ffn.forward(*args)
        for _ in range(warmup):
            step()
        repeats = max(1, min(repeats, steps))
        blocks = [len(b) for b in np.array_split(np.arange(steps), repeats)]
        per_pass = []
        torch.cuda.synchronize()
        t_all = time.perf_counter()
        for n in blocks:
            t0 = time.perf_counter()
            for _ in range(n):
                step()
            torch.cuda.synchronize()
            per_pass.append((time.perf_counter() - t0) / n)
        elapsed = time.perf_counter() - t_all
        timer_steps = min(steps, 20)
        aclnn.kernel_timer_enable(True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(timer_steps):
            self.ffn.forward(*args)
        torch.cuda.synchronize()
        elapsed_timer = time.perf_counter() - t0
        kernels = aclnn.kernel_timer_report()
        aclnn.kernel_timer_enable(False)
        # how evenly the deal of GEMM tiles ends on the eight XCDs: one more pass with span recording on
        aclnn.gemm_workgroup_spans_enable(True)
        self.ffn.forward(*args)
        self.spans = aclnn.gemm_workgroup_spans_report()
        aclnn.gemm_workgroup_spans_enable(False)
        return {"sec_per_pass": float(np.median(per_pass)), "sec_min": min(per_pass), "sec_max": max(per_pass),
                "sec_mean": elapsed / steps, "blocks": blocks, "kernels": kernels, "timer_steps": timer_steps,
                "sec_with_timer": elapsed_timer / timer_steps}

    def summary(self, measured, steps, launch):
        sec_per_pass, kernels, sec_with_timer = measured["sec_per_pass"], measured["kernels"], measured["sec_with_timer"]
        cfg = self.cfg
        work = self.pkg.synth.algorithmic_work(cfg, self.touched)
        return {
            "workload": "%s: %d tokens, H=%d, I=%d, E=%d, top-%d, %s routing" % (
                cfg.name, cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.top_k,
                "Zipf(%.1f)" % cfg.skew if cfg.skew else "uniform random"),
            "chain": "%s routing, SwiGLU GEMM, down GEMM, finalize" % self.ffn.routing.upper(),
            "launch": launch,
            "experts_touched": self.touched,
            "ms_per_step": sec_per_pass * 1e3,
            "ms_per_step_repeats": {"blocks_of_passes": measured["blocks"], "statistic": "median of the blocks",
                                    "min": measured["sec_min"] * 1e3, "max": measured["sec_max"] * 1e3,
                                    "mean_over_all_passes": measured["sec_mean"] * 1e3},
            "ms_per_step_kernel_timer_on": sec_with_timer * 1e3,
            "tokens_per_s": cfg.tokens / sec_per_pass,
            "end_to_end": {"mfma_frac": work["ops"] / sec_per_pass / 1e12 / INT8_PEAK_TOPS,
                           "hbm_frac": work["bytes"] / sec_per_pass / 1e9 / HBM_PEAK_GBS,
                           "algorithmic_ops": work["ops"], "algorithmic_bytes": work["bytes"]},
            "kernels_ms": {k: v[1] / float(measured["timer_steps"]) for k, v in sorted(kernels.items())},
            "roofline": _gate_up_roofline(cfg, self.touched, kernels, measured["timer_steps"]),
            "roofline_down_gemm": _down_roofline(cfg, self.touched, kernels, measured["timer_steps"]),
            "workspace_bytes": dict(self.ffn.workspace.requested, allocated=int(self.ffn.workspace.tensor.numel())
                                    if self.ffn.workspace.tensor is not None else 0),
            "gemm_tile_balance": self._tile_balance(),
        }

    def _tile_balance(self):
        """Per GEMM kernel: span of the launch and, over the eight XCDs, when the last workgroup of each ended and the
        mean busy fraction of its workgroups (1.0 = every workgroup worked from the first start to the last end)."""
        out = {}
        for name, rec in sorted(getattr(self, "spans", {}).items()):
            ends = [x["end_us"] for x in rec["xcd"]]
            out[name] = {"span_us": rec["span_us"], "tile_rows": rec["tile_rows"],
                         "xcd_end_us_min": min(ends), "xcd_end_us_max": max(ends),
                         "xcd_busy_min": min(x["busy"] for x in rec["xcd"]),
                         "xcd_busy_mean": sum(x["busy"] for x in rec["xcd"]) / len(rec["xcd"]),
                         "tiles_per_workgroup_min": min(x["tiles_min"] for x in rec["xcd"]),
                         "tiles_per_workgroup_max": max(x["tiles_max"] for x in rec["xcd"])}
        return out


def _other_configs(pkg, dev, headline, steps, warmup):
    """The halves of the metric that the headline configuration does not show, measured the same way."""
    import torch
    out = {}

    def release():
        gc.collect()
        torch.cuda.empty_cache()

    if headline.cfg.name.startswith("c1"):
        # the headline's own pass replayed from a HIP graph, for comparison with the ten eager launches (a graph of long
        # kernels need not replay faster than they launch: the decode pass gains from it, this one does not)
        out["c1_graph"] = headline.summary(headline.measure(steps, warmup, graph=True), steps,
                                           "HIP graph replay (kernel durations from eager passes)")
    if headline.cfg.name.startswith("c1"):
        # the same tensors behind the other routing operator (one aclnnMoeInitRoutingV3 call instead of the two
        # aclnnMoeInitRoutingV2 calls, or the other way round)
        name = "v3" if headline.ffn.routing == "v2" else "v2"
        alt = headline.with_routing(name)
        out["c1_%s_routed" % name] = alt.summary(alt.measure(steps, warmup), steps, "eager two-phase calls")
        del alt
    for name in ("c3", "c2", "c4"):
        if headline.cfg.name.startswith(name):
            continue
        release()
        w = Workload(pkg, pkg.synth.config(name), dev, routing=headline.ffn.routing)
        # A decode pass is 0.4 ms: a block of four between two synchronisations would be timing the synchronisations
        # (the first launch of a block has nothing to hide behind, the last wait is a host round trip: together ~0.1 ms).
        # Ten times the passes make a block 16 ms.
        n = steps * 10 if name == "c3" else steps
        out[name] = w.summary(w.measure(n, warmup), n, "eager two-phase calls")
        if name == "c3":
            out["c3_graph"] = w.summary(w.measure(n, warmup, graph=True), n,
                                        "HIP graph replay (kernel durations from eager passes)")
        del w
    release()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--repeats", type=int, default=5,
                    help="the timed passes run as this many blocks, each between two synchronisations; ms_per_step is the median block")
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c1")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="measure the headline configuration only (profiler runs)")
    ap.add_argument("--calibration-copy", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="replay the pass from a HIP graph (second phases only) instead of calling the operators eagerly")
    ap.add_argument("--routing", choices=("v2", "v3"), default="v2",
                    help="routing operator at the head of the chain: aclnnMoeInitRoutingV2 (default, two calls: rows and "
                         "scale column) or aclnnMoeInitRoutingV3 (one call)")
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

    head = Workload(pkg, cfg, dev, routing=args.routing, fused_combine=args.fused_combine, weight_nz=args.weight_nz,
                    weight_row_major=args.weight_row_major)
    measured = head.measure(args.steps, args.warmup, graph=args.graph, repeats=args.repeats)
    sec_per_pass = measured["sec_per_pass"]
    if args.calibration_copy:
        src = torch.empty(1 << 30, dtype=torch.int8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            aclnn.calibration_copy(dst, src)
        torch.cuda.synchronize()
        del src, dst

    s = head.summary(measured, args.steps, "HIP graph replay" if args.graph else "eager two-phase calls")
    work = pkg.synth.algorithmic_work(cfg, head.touched)
    result = {
        "metric": "MoE FFN tokens/s (W8A8 expert FFN: routing + gate/up GEMM + SwiGLU + requant + down GEMM + finalize), 1 GPU",
        "value": s["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": s["ms_per_step"],
        "ms_per_step_repeats": s["ms_per_step_repeats"],
        "ms_per_step_kernel_timer_on": s["ms_per_step_kernel_timer_on"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": s["workload"], "expanded_rows": cfg.tokens * cfg.top_k, "experts_touched": head.touched,
                   "weight_layout": "FRACTAL_NZ" if args.weight_nz else "row-major [E, K, N]" if args.weight_row_major
                   else "K-contiguous (transposed view)",
                   "chain": "%s routing, SwiGLU GEMM, " % args.routing.upper() +
                            ("fused down GEMM + combine" if args.fused_combine else "down GEMM, finalize"),
                   "launch": s["launch"]},
        "end_to_end": dict(s["end_to_end"], tops=work["ops"] / sec_per_pass / 1e12, gbps=work["bytes"] / sec_per_pass / 1e9),
        "kernels_ms": s["kernels_ms"],
        "roofline": s["roofline"],
        "roofline_down_gemm": s["roofline_down_gemm"],
        "workspace_bytes": s["workspace_bytes"],
        "gemm_tile_balance": s["gemm_tile_balance"],
    }
    # what the matrix pipe sustains with nothing else going on: the clock under matrix load follows the switching
    # activity of the operands, so uniform random bytes (the benchmark's weights) run well below all-zero operands
    result["int8_mfma_rate_probe"] = {
        "zero_operands_tops": aclnn.int8_mfma_rate_probe(False) / 1e12,
        "uniform_random_operands_tops": aclnn.int8_mfma_rate_probe(True) / 1e12,
        "note": "back-to-back v_mfma_i32_32x32x32_i8 on register operands, 8 waves per CU, no memory traffic; "
                "roofline.peak stays the published 5000 TOP/s"}
    if not args.no_cpu_baseline:
        oracle = graft.load_oracle()
        oracle.build()
        v, desc = _cpu_baseline(pkg, oracle, cfg, head.idx, head.wgt, head.xq, head.xs, head.ffn)
        result["cpu_baseline"] = {"value": v, "unit": "tokens/s", "cores": oracle.num_threads(), "kind": "port",
                                  "sample": desc}
    if not args.no_other_configs:
        result["other_configs"] = _other_configs(pkg, dev, head, steps=min(args.steps, 20), warmup=min(args.warmup, 2))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
