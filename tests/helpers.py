"""Shared helpers of the test-suite: error measures and the parity gates.

Gates (from the benchmark contract of this path): against the fp32/fp64 CPU oracle on identical
seeded inputs, bf16 inputs must agree within max-abs 2e-2 AND relative-L2 1e-2, fp32 inputs
within 1e-4 on both measures, for the output and the final state alike."""

from __future__ import annotations

import torch


BF16_MAX_ABS = 2e-2
BF16_REL_L2 = 1e-2
FP32_TOL = 1e-4


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    denom = b.norm().item()
    return (a - b).norm().item() / (denom if denom > 0 else 1.0)


def assert_parity(actual: torch.Tensor, expected: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    assert actual.shape == expected.shape, f"{what}: shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    assert torch.isfinite(actual.float()).all(), f"{what}: non-finite values"
    ma, rl = max_abs(actual, expected), rel_l2(actual, expected)
    if dtype == torch.bfloat16:
        assert ma <= BF16_MAX_ABS and rl <= BF16_REL_L2, f"{what}: max-abs {ma:.3e} (<= 2e-2), rel-L2 {rl:.3e} (<= 1e-2)"
    else:
        assert ma <= FP32_TOL and rl <= FP32_TOL, f"{what}: max-abs {ma:.3e}, rel-L2 {rl:.3e} (<= 1e-4)"


def random_inputs(B, T, H, K, V, dtype=torch.float32, seed=0, gated=True, h0=True, g_mean=1.0, beta_max=1.0,
                  normalize=True, N=None):
    """Small seeded inputs in the layout of the operator (see lm_engine_amd.workloads for the
    benchmark distributions)."""
    gen = torch.Generator("cpu").manual_seed(seed)
    q = torch.randn(B, T, H, K, generator=gen)
    k = torch.randn(B, T, H, K, generator=gen)
    if normalize:
        q = torch.nn.functional.normalize(q, dim=-1)
        k = torch.nn.functional.normalize(k, dim=-1)
    v = torch.randn(B, T, H, V, generator=gen)
    beta = torch.randn(B, T, H, generator=gen).sigmoid() * beta_max
    g = torch.nn.functional.logsigmoid(g_mean + torch.randn(B, T, H, generator=gen)) if gated else None
    N = B if N is None else N
    state = 0.02 * torch.randn(N, H, K, V, generator=gen) if h0 else None
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), g=g, beta=beta.to(dtype), initial_state=state)
