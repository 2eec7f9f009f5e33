"""The synthetic workloads are the ones the benchmark names (CPU only: routing statistics of every configuration)."""
import numpy as np
import pytest


@pytest.mark.parametrize("seed", [0, 4, 11])
def test_skewed_configuration_is_the_benchmarks(pkg, seed):
    """c4: Zipf(1.2) expert load gives about 30 % empty experts and one expert with more than ten times the mean."""
    cfg = pkg.synth.config(4)
    idx, wgt = pkg.synth.make_routing(cfg, seed=seed)
    counts = np.bincount(idx.reshape(-1), minlength=cfg.experts)
    assert counts.sum() == cfg.tokens * cfg.top_k
    assert 0.25 <= (counts == 0).mean() <= 0.45
    assert counts.max() > 10 * counts.mean()
    # Zipf, not a cliff: the load falls off over the whole ranking (a few dozen experts above the mean, most of the
    # touched ones far below it)
    assert 15 <= (counts > counts.mean()).sum() <= 60
    assert (counts > 0).sum() >= 140
    np.testing.assert_allclose(wgt.sum(axis=1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("index", [0, 1, 2, 3])
def test_uniform_configurations(pkg, index):
    cfg = pkg.synth.config(index)
    idx, wgt = pkg.synth.make_routing(cfg, seed=index)
    assert idx.shape == (cfg.tokens, cfg.top_k) and idx.dtype == np.int32
    # top-k picks distinct experts per token
    assert all(len(set(row)) == cfg.top_k for row in idx[:64])
    counts = np.bincount(idx.reshape(-1), minlength=cfg.experts)
    mean = counts.mean()
    assert counts.max() < mean + 6 * np.sqrt(mean) + 4      # uniform random routing
    np.testing.assert_allclose(wgt.sum(axis=1), 1.0, rtol=1e-5)
