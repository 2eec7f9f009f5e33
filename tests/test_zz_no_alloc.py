"""aclnnMoeInitRoutingV2StaticWorkspace (the second phase that allocates nothing) against aclnnMoeInitRoutingV2.

Both run the same kernels; the only difference is where the sort tables live (the library's built-in device array
instead of a caller workspace).  Bar: every output bit-identical, on two calls in a row of which the second is smaller
(the array keeps the first call's contents), and no device allocation during the calls.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(rng, T, H, K, E, dev):
    x = torch.from_numpy(rng.integers(-127, 128, (T, H)).astype(np.int8)).to(dev)
    idx = torch.from_numpy(rng.integers(0, E, (T, K)).astype(np.int32)).to(dev)
    return x, idx


def _outputs(T, H, K, E, dev, fill):
    return (torch.full((T * K, H), fill, dtype=torch.int8, device=dev),
            torch.full((T * K,), fill, dtype=torch.int32, device=dev),
            torch.full((E,), fill, dtype=torch.int32, device=dev), None)


def test_static_workspace_matches_workspace_entry_point(aclnn, oracle, dev):
    rng = np.random.default_rng(77)
    # first a prefill-sized call (three sort kernels, 1 MB of tables), then a decode-sized one (one-workgroup sort)
    for T, H, K, E in ((4096, 512, 8, 256), (64, 512, 8, 128)):
        x, idx = _case(rng, T, H, K, E, dev)
        ref = _outputs(T, H, K, E, dev, -3)
        aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=ref)
        got = _outputs(T, H, K, E, dev, -5)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=got, static_workspace=True)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        for g, r in zip(got[:3], ref[:3]):
            assert torch.equal(g, r)
        ex, ri, cs, _ = oracle.moe_init_routing_v2(x.cpu().numpy(), idx.cpu().numpy(), expert_num=E, count_flag=1)
        assert np.array_equal(got[1].cpu().numpy(), ri) and np.array_equal(got[2].cpu().numpy(), cs)
        assert np.array_equal(got[0].cpu().numpy(), ex)


def test_static_workspace_drop_pad_then_smaller(aclnn, dev):
    rng = np.random.default_rng(78)
    for T, H, K, E, C in ((512, 64, 4, 16, 96), (48, 64, 2, 8, 10)):
        x, idx = _case(rng, T, H, K, E, dev)
        outs = []
        for static in (False, True):
            o = (torch.full((E, C, H), -3, dtype=torch.int8, device=dev), torch.full((T * K,), -3, dtype=torch.int32, device=dev),
                 None, torch.full((E,), -3, dtype=torch.int32, device=dev))
            aclnn.moe_init_routing_v2(x, idx, 0, C, E, 1, 0, True, out=o, static_workspace=static)
            outs.append(o)
        torch.cuda.synchronize()
        for a, b in zip(outs[0], outs[1]):
            assert (a is None and b is None) or torch.equal(a, b)


def test_static_workspace_refuses_oversized_calls(aclnn, dev):
    T, K, E = 40000, 4, 64     # 160000 expert ids: the sort tables need more than the built-in 4 MiB
    x = torch.zeros((T, 16), dtype=torch.int8, device=dev)
    idx = torch.zeros((T, K), dtype=torch.int32, device=dev)
    out = _outputs(T, 16, K, E, dev, 0)
    with pytest.raises(aclnn.AclnnError) as err:
        aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=out, static_workspace=True)
    assert err.value.code == aclnn.ACLNN_ERR_PARAM_INVALID and "4194304" in err.value.message
    # the ordinary entry point still takes the same call
    aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=out)
    torch.cuda.synchronize()
    assert int(out[2][-1]) == T * K
