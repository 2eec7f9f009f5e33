"""The committed fixtures (tests/golden/reference_examples.json: the reference examples' literal inputs with the outputs
their operator definitions give, see tests/golden/make_example_fixtures.py) against the oracle on the CPU and against the
library on the GPU."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "reference_examples.json")) as f:
        return json.load(f)


def test_oracle_reproduces_the_fixtures(oracle, golden):
    g = golden["moe_init_routing_v2_example"]
    ex, ri, _, bef = oracle.moe_init_routing_v2(np.array(g["x"], np.float32), np.array(g["expert_idx"], np.int32),
                                                expert_capacity=g["expert_capacity"], expert_num=g["expert_num"],
                                                drop_pad_mode=1, before_capacity_flag=True)
    assert ri.tolist() == g["expanded_row_idx"] and bef.tolist() == g["expert_tokens_before_capacity"]
    assert np.array_equal(ex, np.array(g["expanded_x"], np.float32))

    g = golden["moe_init_routing_v3_example"]
    ex, ri, cnt, es = oracle.moe_init_routing_v3(np.array(g["x"], np.float32), np.array(g["expert_idx"], np.int32),
                                                 np.array(g["scale"], np.float32), g["expert_num"],
                                                 tuple(g["active_expert_range"]), g["expert_tokens_num_type"], g["row_idx_type"])
    assert ri.tolist() == g["expanded_row_idx"] and cnt.tolist() == g["expert_tokens_count"]
    assert np.array_equal(ex, np.array(g["expanded_x"], np.float32)) and np.array_equal(es, np.array(g["expanded_scale"], np.float32))

    g = golden["moe_init_routing_quant_v2_example"]
    ex, ri, _, bef, _ = oracle.moe_init_routing_quant_v2(np.array(g["x"], np.float32), np.array(g["expert_idx"], np.int32), 0,
                                                         g["scale"], g["offset"], expert_capacity=g["expert_capacity"],
                                                         expert_num=g["expert_num"], drop_pad_mode=1, before_capacity_flag=True)
    assert ri.tolist() == g["expanded_row_idx"] and bef.tolist() == g["expert_tokens_before_capacity"]
    assert ex.tolist() == g["expanded_x"]

    g = golden["moe_finalize_routing_v2_example"]
    out = oracle.moe_finalize_routing_v2(np.array(g["expanded_x"], np.float32), np.array(g["expanded_row_idx"], np.int32),
                                         np.array(g["x1"], np.float32), np.array(g["x2"], np.float32),
                                         np.array(g["bias"], np.float32), np.array(g["scales"], np.float32),
                                         np.array(g["expert_idx"], np.int32), drop_pad_mode=g["drop_pad_mode"])
    assert np.array_equal(out, np.array(g["out"], np.float32))

    g = golden["moe_gating_top_k_softmax_v2_example"]
    y, idx, sm = oracle.moe_gating_top_k_softmax_v2(np.array(g["x"], np.float32), g["k"], g["renorm"], want_softmax=True)
    assert idx.tolist() == g["expert_idx"]
    np.testing.assert_allclose(y, np.array(g["y"]), rtol=2e-6)
    np.testing.assert_allclose(sm, np.array(g["softmax"]), rtol=2e-6)


@pytest.mark.gpu
def test_library_reproduces_the_fixtures(aclnn, golden, dev):
    import torch
    t32 = lambda v: torch.tensor(v, dtype=torch.float32, device=dev)
    ti = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)

    g = golden["moe_init_routing_v2_example"]
    ex, ri, _, bef = aclnn.moe_init_routing_v2(t32(g["x"]), ti(g["expert_idx"]), expert_capacity=g["expert_capacity"],
                                               expert_num=g["expert_num"], drop_pad_mode=1,
                                               expert_tokens_before_capacity_flag=True)
    assert ri.cpu().tolist() == g["expanded_row_idx"] and bef.cpu().tolist() == g["expert_tokens_before_capacity"]
    assert torch.equal(ex.cpu(), torch.tensor(g["expanded_x"], dtype=torch.float32))

    g = golden["moe_init_routing_v3_example"]
    ex, ri, cnt, es = aclnn.moe_init_routing_v3(t32(g["x"]), ti(g["expert_idx"]), t32(g["scale"]), expert_num=g["expert_num"],
                                                expert_tokens_num_type=g["expert_tokens_num_type"],
                                                active_expert_range=tuple(g["active_expert_range"]),
                                                row_idx_type=g["row_idx_type"], active_num=12)
    assert ri.cpu().tolist() == g["expanded_row_idx"] and cnt.cpu().tolist() == g["expert_tokens_count"]
    assert torch.equal(ex.cpu(), torch.tensor(g["expanded_x"], dtype=torch.float32))
    assert torch.equal(es.cpu(), torch.tensor(g["expanded_scale"], dtype=torch.float32))

    g = golden["moe_init_routing_quant_v2_example"]
    ex, ri, _, bef, _ = aclnn.moe_init_routing_quant_v2(t32(g["x"]), ti(g["expert_idx"]), 0, t32([g["scale"]]), t32([g["offset"]]),
                                                        expert_capacity=g["expert_capacity"], expert_num=g["expert_num"],
                                                        drop_pad_mode=1, expert_tokens_before_capacity_flag=True)
    assert ri.cpu().tolist() == g["expanded_row_idx"] and bef.cpu().tolist() == g["expert_tokens_before_capacity"]
    assert ex.cpu().tolist() == g["expanded_x"]

    g = golden["moe_finalize_routing_v2_example"]
    out = aclnn.moe_finalize_routing_v2(t32(g["expanded_x"]), ti(g["expanded_row_idx"]), x1=t32(g["x1"]), x2=t32(g["x2"]),
                                        bias=t32(g["bias"]), scales=t32(g["scales"]), expert_idx=ti(g["expert_idx"]),
                                        drop_pad_mode=g["drop_pad_mode"])
    assert torch.equal(out.cpu(), torch.tensor(g["out"], dtype=torch.float32))

    g = golden["moe_gating_top_k_softmax_v2_example"]
    y, idx, sm = aclnn.moe_gating_top_k_softmax_v2(t32(g["x"]), g["k"], g["renorm"], output_softmax=True)
    torch.cuda.synchronize()
    assert idx.cpu().tolist() == g["expert_idx"]
    np.testing.assert_allclose(y.cpu().numpy(), np.array(g["y"]), rtol=2e-6)
    np.testing.assert_allclose(sm.cpu().numpy(), np.array(g["softmax"]), rtol=2e-6)
