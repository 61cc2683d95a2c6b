"""Shared helpers for the parity tests."""
import torch

# Tolerances stated by the hot-path contract.
BF16_RTOL = 1e-2
BF16_ATOL = 1e-2
F32_RTOL = 1e-4


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(g, *shape, dtype=torch.bfloat16, std=1.0, mean=0.0):
    """N(mean, std) drawn on the CPU in fp32, then cast: oracle and kernel see the same bits."""
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std + mean).to(dtype)


def close(actual, expected, rtol=BF16_RTOL, atol=BF16_ATOL, what=""):
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    torch.testing.assert_close(a, e, rtol=rtol, atol=atol, msg=lambda m: f"{what}: {m}")
