"""Writes tests/golden/reference_examples.json: the literal inputs of the reference's example programs for the operators
built here, with the outputs that follow from each operator's published definition, computed with plain numpy (no code
of this repository, no code of the reference).

    python tests/golden/make_example_fixtures.py

The reference holds no expected numbers for these operators: its examples print what the device returns and its unit
tests only run the kernels or compare against generators that need absent packages.  What it does hold is inputs:
  moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp:71-96          (drop/pad routing, E=3, C=2)
  moe/moe_init_routing_v3/examples/test_aclnn_moe_init_routing_v3.cpp:123-125        (range [0, 4), counts)
  moe/moe_init_routing_quant_v2/examples/test_aclnn_moe_init_routing_quant_v2.cpp:71-108 (the V2 case, static quantisation)
  moe/moe_finalize_routing_v2/examples/test_aclnn_moe_finalize_routing_v2.cpp:102-110 (fp32, x1 = x2, bias, mode 0)
  moe/moe_gating_top_k_softmax_v2/examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp:93 (softmax then top-2)
Definitions used: moe/moe_init_routing_v2/README.md, moe/moe_init_routing_quant_v2/README.md (half-precision
x * scale + offset, rounded to int8), moe/moe_init_routing_v3/README.md:12-66,
moe/moe_finalize_routing_v2/README.md, moe/moe_gating_top_k_softmax_v2/README.md:12-30.
"""
import json
import os

import numpy as np


def routing_v2_drop_pad():
    x = np.repeat(np.array([[0.1], [0.2], [0.3]], np.float32), 4, axis=1)
    idx = np.array([[1, 2], [0, 1], [0, 2]], np.int32)
    E, C = 3, 2
    flat = idx.reshape(-1)
    K = idx.shape[1]
    order = np.argsort(flat, kind="stable")
    row_idx = np.full(flat.size, -1, np.int32)
    expanded = np.zeros((E, C, x.shape[1]), np.float32)
    seen = np.zeros(E, np.int64)
    for src in order:                                   # ascending expert, ties by ascending position
        e = flat[src]
        if seen[e] < C:
            row_idx[src] = e * C + seen[e]
            expanded[e, seen[e]] = x[src // K]
        seen[e] += 1
    return {"x": x.tolist(), "expert_idx": idx.tolist(), "expert_num": E, "expert_capacity": C, "drop_pad_mode": 1,
            "expanded_row_idx": row_idx.tolist(), "expanded_x": expanded.tolist(),
            "expert_tokens_before_capacity": np.bincount(flat, minlength=E).tolist()}


def routing_quant_v2_static():
    g = routing_v2_drop_pad()
    scale, offset = np.float32(0.3452), np.float32(1.8369)
    rows = np.array(g["expanded_x"], np.float32)
    filled = np.zeros(rows.shape[:2], bool)
    for dst in g["expanded_row_idx"]:
        if dst >= 0:
            filled[dst // g["expert_capacity"], dst % g["expert_capacity"]] = True
    h = rows.astype(np.float16) * np.float16(scale) + np.float16(offset)          # numpy rounds each half operation
    q = np.clip(np.rint(h.astype(np.float32)), -128, 127).astype(np.int8)
    q[~filled] = 0
    g.update({"quant_mode": 0, "scale": float(scale), "offset": float(offset), "expanded_x": q.tolist()})
    return g


def routing_v3_counts():
    x = np.array([[0.1, 0.1], [0.2, 0.2], [0.3, 0.3]], np.float32)
    idx = np.array([[1, 2, 0, 3], [0, 2, 1, 3], [0, 1, 3, 2]], np.int32)
    scale = np.array([0.3423, 0.1652, 0.2652], np.float32)
    start, end, K = 0, 4, 4
    flat = idx.reshape(-1)
    keep = np.nonzero((flat >= start) & (flat < end))[0]
    order = keep[np.argsort(flat[keep], kind="stable")]
    scatter = np.full(flat.size, -1, np.int32)
    scatter[order] = np.arange(order.size, dtype=np.int32)
    return {"x": x.tolist(), "expert_idx": idx.tolist(), "scale": scale.tolist(), "expert_num": 256,
            "active_expert_range": [start, end], "expert_tokens_num_type": 1, "row_idx_type": 1, "quant_mode": -1,
            "expanded_row_idx": scatter.tolist(), "expanded_x": x[order // K].tolist(),
            "expanded_scale": scale[order // K].tolist(),
            "expert_tokens_count": np.bincount(flat[keep] - start, minlength=end - start).tolist()}


def finalize_v2():
    ex = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1] * 2, np.float32).reshape(6, 4)
    x1 = np.array([0.2, 1.2, 2.2, 3.2, 4.2, 5.2, 6.2, 7.2, 8.2, 9.2, 10.2, 11.2], np.float32).reshape(3, 4)
    bias = np.array([0.2, 0.4] * 4, np.float32).reshape(2, 4)
    scales = np.array([1.3, 1.6, 1.2, 1.8, 1.2, 2.3], np.float32).reshape(3, 2)
    expert_idx = np.array([0, 1, 0, 1, 0, 1], np.int32).reshape(3, 2)
    row_idx = np.array([2, 1, 4, 3, 0, 5], np.int32)
    T, K = scales.shape
    out = np.zeros((T, 4), np.float32)
    for n in range(T):                                   # mode 0: expandedRowIdx[k * T + n], fp32, k ascending
        acc = x1[n] + x1[n]
        for k in range(K):
            acc = acc + scales[n, k] * (ex[row_idx[k * T + n]] + bias[expert_idx[n, k]])
        out[n] = acc
    return {"expanded_x": ex.tolist(), "x1": x1.tolist(), "x2": x1.tolist(), "bias": bias.tolist(), "scales": scales.tolist(),
            "expert_idx": expert_idx.tolist(), "expanded_row_idx": row_idx.tolist(), "drop_pad_mode": 0, "out": out.tolist()}


def gating_softmax_topk():
    x = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1], np.float32).reshape(3, 4)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    p = e / e.sum(axis=1, keepdims=True)
    order = np.argsort(-p, axis=1, kind="stable")[:, :2]
    return {"x": x.tolist(), "k": 2, "renorm": 0, "y": np.take_along_axis(p, order, 1).tolist(),
            "expert_idx": order.tolist(), "softmax": p.tolist()}


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    data = {"moe_init_routing_v2_example": routing_v2_drop_pad(), "moe_init_routing_v3_example": routing_v3_counts(),
            "moe_init_routing_quant_v2_example": routing_quant_v2_static(),
            "moe_finalize_routing_v2_example": finalize_v2(), "moe_gating_top_k_softmax_v2_example": gating_softmax_topk()}
    with open(os.path.join(here, "reference_examples.json"), "w") as f:
        json.dump(data, f, indent=1)
    print("wrote", len(data), "fixtures")
