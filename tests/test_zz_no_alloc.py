"""aclnnMoeInitRoutingV2StaticWorkspace (the second phase that allocates nothing) against aclnnMoeInitRoutingV2.

Both run the same kernels; the only difference is where the sort tables live (the library's built-in device array
instead of a caller workspace).  Bar: every output bit-identical, on two calls in a row of which the second is smaller
(the array keeps the first call's contents), and no device allocation during the calls: neither through torch's
allocator nor, seen from the driver's count of free device memory, through a hipMalloc inside the library.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(rng, T, H, K, E, dev):
    x = torch.from_numpy(rng.integers(-127, 128, (T, H)).astype(np.int8)).to(dev)
    idx = torch.from_numpy(rng.integers(0, E, (T, K)).astype(np.int32)).to(dev)
    return x, idx


def _warm_up(aclnn, dev):
    """One small static-workspace call: module load, the library's one-time hipGetSymbolAddress and kernel attributes
    happen here, so that the driver's free-memory figure is steady before the calls that are checked."""
    x = torch.zeros((8, 32), dtype=torch.int8, device=dev)
    idx = torch.zeros((8, 2), dtype=torch.int32, device=dev)
    for static in (False, True):
        aclnn.moe_init_routing_v2(x, idx, 0, 0, 4, 0, 1, False, out=_outputs(8, 32, 2, 4, dev, 0), static_workspace=static)
        aclnn.moe_init_routing_v2(x, idx, 0, 4, 4, 1, 0, True, static_workspace=static,
                                  out=(torch.zeros((4, 4, 32), dtype=torch.int8, device=dev),
                                       torch.zeros((16,), dtype=torch.int32, device=dev), None,
                                       torch.zeros((4,), dtype=torch.int32, device=dev)))
    torch.cuda.synchronize()


class _NoDeviceAllocation:
    """Asserts that neither torch's allocator nor the driver's free-memory count moves inside the block."""

    def __init__(self, dev):
        self.dev = dev

    def __enter__(self):
        torch.cuda.synchronize()
        self.allocated = torch.cuda.memory_stats(self.dev)["allocation.all.allocated"]
        self.free = torch.cuda.mem_get_info(self.dev)[0]

    def __exit__(self, exc_type, exc, tb):
        torch.cuda.synchronize()
        if exc_type is None:
            assert torch.cuda.memory_stats(self.dev)["allocation.all.allocated"] == self.allocated
            # hipMemGetInfo: a hipMalloc made inside the library (not returned before the call ends) lowers this
            assert torch.cuda.mem_get_info(self.dev)[0] == self.free
        return False


def _outputs(T, H, K, E, dev, fill):
    return (torch.full((T * K, H), fill, dtype=torch.int8, device=dev),
            torch.full((T * K,), fill, dtype=torch.int32, device=dev),
            torch.full((E,), fill, dtype=torch.int32, device=dev), None)


def test_static_workspace_matches_workspace_entry_point(aclnn, oracle, dev):
    rng = np.random.default_rng(77)
    _warm_up(aclnn, dev)
    # first a prefill-sized call (three sort kernels, 1 MB of tables), then a decode-sized one (one-workgroup sort)
    for T, H, K, E in ((4096, 512, 8, 256), (64, 512, 8, 128)):
        x, idx = _case(rng, T, H, K, E, dev)
        ref = _outputs(T, H, K, E, dev, -3)
        aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=ref)
        got = _outputs(T, H, K, E, dev, -5)
        with _NoDeviceAllocation(dev):
            aclnn.moe_init_routing_v2(x, idx, 0, 0, E, 0, 1, False, out=got, static_workspace=True)
        for g, r in zip(got[:3], ref[:3]):
            assert torch.equal(g, r)
        ex, ri, cs, _ = oracle.moe_init_routing_v2(x.cpu().numpy(), idx.cpu().numpy(), expert_num=E, count_flag=1)
        assert np.array_equal(got[1].cpu().numpy(), ri) and np.array_equal(got[2].cpu().numpy(), cs)
        assert np.array_equal(got[0].cpu().numpy(), ex)


def test_static_workspace_drop_pad_then_smaller(aclnn, dev):
    rng = np.random.default_rng(78)
    _warm_up(aclnn, dev)
    for T, H, K, E, C in ((512, 64, 4, 16, 96), (48, 64, 2, 8, 10)):
        x, idx = _case(rng, T, H, K, E, dev)
        outs = []
        for static in (False, True):
            o = (torch.full((E, C, H), -3, dtype=torch.int8, device=dev), torch.full((T * K,), -3, dtype=torch.int32, device=dev),
                 None, torch.full((E,), -3, dtype=torch.int32, device=dev))
            if static:
                with _NoDeviceAllocation(dev):
                    aclnn.moe_init_routing_v2(x, idx, 0, C, E, 1, 0, True, out=o, static_workspace=True)
            else:
                aclnn.moe_init_routing_v2(x, idx, 0, C, E, 1, 0, True, out=o, static_workspace=False)
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
