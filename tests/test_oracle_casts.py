"""Pins the oracle's fp16 / bf16 conversions against numpy float16 and torch bfloat16 (independent implementations)."""
import numpy as np
import torch


def test_f16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.isnan(got[np.isnan(ref)]).all()


def _interesting_f32(rng, n):
    a = rng.standard_normal(n).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, n).astype(np.float32)
    # exact ties and subnormal-half range
    ties = (np.arange(1, 4097, dtype=np.float32) + np.float32(0.5)) * np.float32(2.0 ** -10)
    tiny = rng.standard_normal(4096).astype(np.float32) * np.float32(2.0 ** -20)
    edge = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 70000.0, -65520.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                     2.0 ** -14, np.inf, -np.inf, 126.5, 127.5, -126.5, 0.5, 1.5, 2.5], dtype=np.float32)
    return np.concatenate([a, ties, -ties, tiny, edge])


def test_f16_encode_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    a = _interesting_f32(rng, 200000)
    with np.errstate(over="ignore"):
        ref = a.astype(np.float16).view(np.uint16)
    got = oracle.f32_to_f16_bits(a)
    assert np.array_equal(got, ref)


def test_bf16_encode_matches_torch(oracle):
    rng = np.random.default_rng(2)
    a = _interesting_f32(rng, 200000)
    ref = torch.from_numpy(a).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.f32_to_bf16_bits(a)
    assert np.array_equal(got, ref)
    back = oracle.bf16_bits_to_f32(got)
    assert np.array_equal(back.view(np.uint32), (got.astype(np.uint32) << 16))
