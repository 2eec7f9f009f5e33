"""The reference's own example programs, compiled unmodified against this repository's headers and linked to
libcust_opapi.so (recipe: `make -C oracle ref_examples`, binaries in oracle/_ref/examples/), run on the GPU.

  moe/moe_init_routing_v2/examples/test_aclnn_moe_init_routing_v2.cpp        drop/pad routing of 3 tokens, E=3, C=2
  moe/moe_finalize_routing_v2/examples/test_aclnn_moe_finalize_routing_v2.cpp fp32 finalize with x1, x2, bias
  moe/moe_gating_top_k_softmax_v2/examples/test_aclnn_moe_gating_top_k_softmax_v2.cpp   softmax then top-2 of 3x4 logits
  moe/moe_init_routing_quant_v2/examples/test_aclnn_moe_init_routing_quant_v2.cpp       static quantisation (scale 0.3452,
                                                                              offset 1.8369) of the drop/pad routing above
  gmm/grouped_matmul_swiglu_quant/examples/test_aclnn_grouped_matmul_swiglu_quant.cpp   FRACTAL_NZ weight [4, 128, 448, 16, 32],
                                                                              8192 x 7168 rows, all inputs zero
  gmm/grouped_matmul/examples/test_aclnn_grouped_matmul.cpp                   fp16 grouped matmul via V5
  moe/moe_init_routing_v3/examples/test_aclnn_moe_init_routing_v3.cpp         FLOAT rows into an INT8 output, quantMode -1

The first four must print what the oracle computes from the same literals (held below as data); the SwiGLU example
must run through (its group list is all zero, so no row belongs to a group and the outputs keep their zeros).  The
last two use a data type / dtype pairing outside this build's path: they must fail cleanly in the first phase with
ACLNN_ERR_PARAM_INVALID (161002), the reference's code for an unsupported combination, not crash.
"""
import os
import re
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXAMPLES = os.path.join(ROOT, "oracle", "_ref", "examples")


def _run(name):
    path = os.path.join(EXAMPLES, name)
    if not os.path.exists(path):
        pytest.skip("%s is not built (needs the reference sources: make -C oracle ref_examples)" % name)
    res = subprocess.run([path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    return res.returncode, res.stdout


def _values(text, label, cast):
    return [cast(m.group(1)) for m in re.finditer(r"%s\[\d+\] is: (\S+)" % re.escape(label), text)]


def test_routing_example(oracle, dev):
    rc, text = _run("test_aclnn_moe_init_routing_v2")
    assert rc == 0, text
    x = np.repeat(np.array([[0.1], [0.2], [0.3]], np.float32), 4, axis=1)
    idx = np.array([[1, 2], [0, 1], [0, 2]], np.int32)
    ex, ri, _, bef = oracle.moe_init_routing_v2(x, idx, expert_capacity=2, expert_num=3, drop_pad_mode=1,
                                                before_capacity_flag=True)
    assert _values(text, "expandedRowIdxData", int) == ri.tolist() == [2, 4, 0, 3, 1, 5]
    assert _values(text, "expertTokenIdxData", int) == bef.tolist() == [2, 2, 2]
    got = np.array(_values(text, "expandedXData", float), np.float32)
    np.testing.assert_allclose(got, ex.reshape(-1), rtol=0, atol=5e-7)   # printed with six decimals


def test_routing_quant_example(oracle, dev):
    rc, text = _run("test_aclnn_moe_init_routing_quant_v2")
    assert rc == 0, text
    x = np.repeat(np.array([[0.1], [0.2], [0.3]], np.float32), 4, axis=1)
    idx = np.array([[1, 2], [0, 1], [0, 2]], np.int32)
    ex, ri, _, bef, _ = oracle.moe_init_routing_quant_v2(x, idx, 0, 0.3452, 1.8369, expert_capacity=2, expert_num=3,
                                                         drop_pad_mode=1, before_capacity_flag=True)
    assert _values(text, "expandedRowIdxData", int) == ri.tolist() == [2, 4, 0, 3, 1, 5]
    assert _values(text, "expertTokenIdxData", int) == bef.tolist() == [2, 2, 2]
    # 0.1 * 0.3452 + 1.8369 ... 0.3 * 0.3452 + 1.8369 all lie in (1.87, 1.95): every slot holds 2
    assert _values(text, "expandedXData", int) == ex.reshape(-1).tolist() == [2] * 24


def test_finalize_example(oracle, dev):
    rc, text = _run("test_aclnn_moe_finalize_routing_v2")
    assert rc == 0, text
    ex = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1,
                   0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1], np.float32).reshape(6, 4)
    x1 = np.array([0.2, 1.2, 2.2, 3.2, 4.2, 5.2, 6.2, 7.2, 8.2, 9.2, 10.2, 11.2], np.float32).reshape(3, 4)
    bias = np.array([0.2, 0.4, 0.2, 0.4, 0.2, 0.4, 0.2, 0.4], np.float32).reshape(2, 4)
    scales = np.array([1.3, 1.6, 1.2, 1.8, 1.2, 2.3], np.float32).reshape(3, 2)
    expert_idx = np.array([0, 1, 0, 1, 0, 1], np.int32).reshape(3, 2)
    row_idx = np.array([2, 1, 4, 3, 0, 5], np.int32)
    want = oracle.moe_finalize_routing_v2(ex, row_idx, x1, x1, bias, scales, expert_idx, drop_pad_mode=0)
    got = np.array(_values(text, "result", float), np.float32)
    assert got.shape == (12,)
    np.testing.assert_allclose(got, want.reshape(-1), rtol=0, atol=5e-6)  # six printed decimals of values up to ~50


def test_gating_example(oracle, dev):
    rc, text = _run("test_aclnn_moe_gating_top_k_softmax_v2")
    assert rc == 0, text
    x = np.array([0.1, 1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1], np.float32).reshape(3, 4)
    want, _, _ = oracle.moe_gating_top_k_softmax_v2(x, 2, 0)
    got = np.array(_values(text, "result", float), np.float32)
    assert got.shape == (6,)
    np.testing.assert_allclose(got, want.reshape(-1), rtol=0, atol=1e-6)   # six printed decimals


def test_swiglu_example_with_nz_weight(dev, tmp_path):
    """Prints 16.8 million result lines: they go to a file and only its two ends are read."""
    path = os.path.join(EXAMPLES, "test_aclnn_grouped_matmul_swiglu_quant")
    if not os.path.exists(path):
        pytest.skip("the example is not built (needs the reference sources: make -C oracle ref_examples)")
    log = tmp_path / "swiglu_example.txt"
    with open(log, "wb") as f:
        rc = subprocess.run([path], stdout=f, stderr=subprocess.STDOUT, timeout=110).returncode
    size = os.path.getsize(log)
    with open(log, "rb") as f:
        head = f.read(4096).decode(errors="replace")
        f.seek(max(0, size - 4096))
        tail = f.read().decode(errors="replace")
    assert rc == 0, head + " ... " + tail
    assert "ERROR" not in head and "ERROR" not in tail
    assert head.startswith("result[0] is: 0\n") or "result[0] is: 0\n" in head
    assert tail.rstrip().endswith("result[8191] is: 0.000000")      # the last per-row output scale


@pytest.mark.parametrize("name,api", [("test_aclnn_grouped_matmul", "aclnnGroupedMatmulV5GetWorkspaceSize"),
                                      ("test_aclnn_moe_init_routing_v3", "aclnnMoeInitRoutingV3GetWorkspaceSize")])
def test_unsupported_examples_fail_cleanly(name, api, dev):
    rc, text = _run(name)
    assert "%s failed. ERROR: 161002" % api in text, text
    assert rc not in (-11, -6, 139, 134), text
