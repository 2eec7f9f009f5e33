"""Seeded synthetic workloads for the quantized MoE expert FFN (the five benchmark configurations).

Value distributions:
  router logits fp32 N(0,1) [T, E] -> softmax -> top-K (ties to the lower index) -> weights renormalised to sum 1;
  x bf16 N(0,1) [T, H] -> per-token xs = absmax/127 (fp32), xq = clip(rint(x / xs), -127, 127) int8;
  weights int8 uniform[-127, 127]; per-output-channel scales fp32 uniform[1e-3, 1e-2].
The "skewed" configuration adds a per-expert logit bias so that expert load follows Zipf(alpha = 1.2).

Routing inputs and activations are generated with numpy (small, reproducible on any host); the expert weights (up to
11 GB) are generated on the device with a seeded torch generator, expert by expert.
"""
import collections

import numpy as np
import torch

Config = collections.namedtuple("Config", "name tokens hidden inter experts top_k skew")

CONFIGS = [
    Config("c0_small", 256, 1024, 1024, 8, 2, 0.0),
    Config("c1_deepseek_v3_prefill", 4096, 7168, 2048, 256, 8, 0.0),
    Config("c2_mixtral_prefill", 16384, 4096, 14336, 8, 2, 0.0),
    Config("c3_qwen3_moe_decode", 64, 4096, 1536, 128, 8, 0.0),
    Config("c4_deepseek_v3_skewed", 8192, 7168, 2048, 256, 8, 1.2),
]


def config(index_or_name):
    if isinstance(index_or_name, int):
        return CONFIGS[index_or_name]
    for c in CONFIGS:
        if c.name == index_or_name or c.name.split("_")[0] == index_or_name:
            return c
    raise KeyError(index_or_name)


def make_routing(cfg, seed=0):
    """Returns (topk_idx int32 [T, K], topk_weight fp32 [T, K]) as numpy arrays."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((cfg.tokens, cfg.experts), dtype=np.float32)
    if cfg.skew > 0:
        # expert popularity ~ rank^-alpha (Zipf): bias = -alpha * log(rank) on a random ranking of the experts.  With
        # alpha = 1.2, 8192 tokens and top-8 of 256 this leaves 35-40 % of the experts without a row, about thirty
        # experts with more than the mean of 256 rows and the most popular one with nearly every token (31 x the mean).
        perm = rng.permutation(cfg.experts)
        rank = np.empty(cfg.experts, np.float32)
        rank[perm] = np.arange(1, cfg.experts + 1, dtype=np.float32)
        logits = logits + (-cfg.skew * np.log(rank))[None, :].astype(np.float32)
    z = logits - logits.max(axis=1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(axis=1, keepdims=True)
    # top-K, ties to the lower index: stable argsort of -p
    order = np.argsort(-p, axis=1, kind="stable")[:, :cfg.top_k]
    w = np.take_along_axis(p, order, axis=1)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return order.astype(np.int32), w


def quantize_per_token(x_f32):
    """x fp32 [T, H] (bf16-representable values) -> (xq int8, xs fp32): xs = absmax/127, xq = clip(rint(x/xs))."""
    absmax = np.abs(x_f32).max(axis=1)
    xs = (absmax / np.float32(127.0)).astype(np.float32)
    safe = np.where(xs > 0, xs, np.float32(1.0))
    xq = np.clip(np.rint(x_f32 / safe[:, None]), -127, 127).astype(np.int8)
    return xq, xs


def make_activations(cfg, seed=0):
    """Returns (xq int8 [T, H], xs fp32 [T]) as numpy arrays; x is N(0,1) rounded to bf16 before quantisation."""
    rng = np.random.default_rng(seed + 1000)
    x = rng.standard_normal((cfg.tokens, cfg.hidden), dtype=np.float32)
    x = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    return quantize_per_token(x)


def make_weights(cfg, device, seed=0, w2_scale_dtype=torch.float32):
    """Expert weights in the K-contiguous storage the kernels stream:
    w13 int8 [E, 2I, H], w13_scale fp32 [E, 2I], w2 int8 [E, H, I], w2_scale [E, H]."""
    g = torch.Generator(device=device)
    g.manual_seed(seed + 2000)
    E, H, I = cfg.experts, cfg.hidden, cfg.inter
    w13 = torch.empty((E, 2 * I, H), dtype=torch.int8, device=device)
    w2 = torch.empty((E, H, I), dtype=torch.int8, device=device)
    for e in range(E):  # expert by expert keeps the generator's temporaries small
        w13[e] = torch.randint(-127, 128, (2 * I, H), dtype=torch.int8, device=device, generator=g)
        w2[e] = torch.randint(-127, 128, (H, I), dtype=torch.int8, device=device, generator=g)
    w13_scale = torch.empty((E, 2 * I), dtype=torch.float32, device=device).uniform_(1e-3, 1e-2, generator=g)
    w2_scale = torch.empty((E, H), dtype=torch.float32, device=device).uniform_(1e-3, 1e-2, generator=g)
    return w13, w13_scale, w2, w2_scale.to(w2_scale_dtype)


def algorithmic_work(cfg, experts_touched=None):
    """int8 ops (2 per MAC) and HBM bytes of one pass of the path, as the measurement plan defines them."""
    T, H, I, E, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.top_k
    M = T * K
    touched = E if experts_touched is None else experts_touched
    ops = 6 * M * H * I
    weight_bytes = touched * 3 * H * I
    scale_bytes = touched * (2 * I + H) * 4
    act_bytes = (T * H            # xq in
                 + 2 * M * H      # expanded xq write + read
                 + 2 * M * I      # h write + read
                 + 2 * M * H * 2  # y bf16 write + read
                 + T * H * 2      # out bf16
                 + M * 4 * 4 + T * K * 8)  # index / scale vectors
    return {"ops": ops, "weight_bytes": weight_bytes, "scale_bytes": scale_bytes, "act_bytes": act_bytes,
            "bytes": weight_bytes + scale_bytes + act_bytes}
