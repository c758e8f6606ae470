"""The gradient oracle: autograd through the token loop against central finite differences, and
the closed-form chunked backward against autograd (fp64 throughout)."""

import pytest
import torch

from oracle.gdn_backward_oracle import chunk_gated_delta_rule_bwd_ref, gated_delta_rule_grads_autograd
from oracle.gdn_oracle import recurrent_gated_delta_rule_ref


def _inputs(seed, B, T, H, K, V, with_state, N=None):
    gen = torch.Generator().manual_seed(seed)
    dt = torch.float64
    q = torch.randn(B, T, H, K, generator=gen, dtype=dt)
    k = torch.randn(B, T, H, K, generator=gen, dtype=dt)
    v = torch.randn(B, T, H, V, generator=gen, dtype=dt)
    g = torch.nn.functional.logsigmoid(torch.randn(B, T, H, generator=gen, dtype=dt) + 2.0)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen, dtype=dt))
    N = B if N is None else N
    h0 = torch.randn(N, H, K, V, generator=gen, dtype=dt) * 0.1 if with_state else None
    do = torch.randn(B, T, H, V, generator=gen, dtype=dt)
    dht = torch.randn(N, H, K, V, generator=gen, dtype=dt)
    return q, k, v, g, beta, h0, do, dht


def _loss(q, k, v, g, beta, h0, do, dht, **kw):
    o, ht = recurrent_gated_delta_rule_ref(
        q, k, v, g, beta, initial_state=h0, output_final_state=True, state_dtype=torch.float64, **kw
    )
    return float((o * do).sum() + (ht * dht).sum())


@pytest.mark.parametrize("l2norm", [False, True])
def test_autograd_matches_finite_differences(l2norm):
    B, T, H, K, V = 1, 7, 2, 4, 3
    q, k, v, g, beta, h0, do, dht = _inputs(0, B, T, H, K, V, True)
    if not l2norm:
        k = k * 0.5  # keep beta |k|^2 moderate without the normalisation
    kw = dict(use_qk_l2norm_in_kernel=l2norm)
    grads = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, dht, initial_state=h0, **kw)
    args = [q, k, v, g, beta, h0]
    eps = 1e-6
    gen = torch.Generator().manual_seed(1)
    for which, grad in enumerate(grads):
        x = args[which]
        flat = x.reshape(-1)
        for idx in torch.randint(0, flat.numel(), (6,), generator=gen).tolist():
            keep = float(flat[idx])
            flat[idx] = keep + eps
            up = _loss(*args, do, dht, **kw)
            flat[idx] = keep - eps
            down = _loss(*args, do, dht, **kw)
            flat[idx] = keep
            fd = (up - down) / (2 * eps)
            assert abs(fd - float(grad.reshape(-1)[idx])) <= 1e-6 * max(1.0, abs(fd)), (which, idx)


@pytest.mark.parametrize("l2norm", [False, True])
@pytest.mark.parametrize("with_state", [False, True])
@pytest.mark.parametrize("T,chunk", [(64, 64), (50, 16), (130, 64), (5, 64)])
def test_chunked_backward_matches_autograd(T, chunk, with_state, l2norm):
    B, H, K, V = 2, 2, 8, 6
    q, k, v, g, beta, h0, do, dht = _inputs(T, B, T, H, K, V, with_state)
    if not l2norm:
        k = k * 0.4
    kw = dict(initial_state=h0, use_qk_l2norm_in_kernel=l2norm)
    want = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, dht, **kw)
    got = chunk_gated_delta_rule_bwd_ref(q, k, v, g, beta, do, dht, chunk_size=chunk, **kw)
    for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0"), got, want):
        if b is None:
            assert a is None
            continue
        assert torch.allclose(a, b, rtol=1e-9, atol=1e-9), (name, float((a - b).abs().max()))


def test_chunked_backward_packed_sequences():
    H, K, V = 2, 8, 4
    cu = torch.tensor([0, 3, 40, 41, 90], dtype=torch.int32)
    q, k, v, g, beta, h0, do, dht = _inputs(5, 1, 90, H, K, V, True, N=4)
    kw = dict(initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=True, scale=0.3)
    want = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, dht, **kw)
    got = chunk_gated_delta_rule_bwd_ref(q, k, v, g, beta, do, dht, chunk_size=16, **kw)
    for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0"), got, want):
        assert torch.allclose(a, b, rtol=1e-9, atol=1e-9), (name, float((a - b).abs().max()))


def test_no_final_state_gradient():
    q, k, v, g, beta, h0, do, _ = _inputs(9, 1, 40, 2, 8, 4, False)
    want = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, None, use_qk_l2norm_in_kernel=True)
    got = chunk_gated_delta_rule_bwd_ref(q, k, v, g, beta, do, None, chunk_size=16, use_qk_l2norm_in_kernel=True)
    for a, b in zip(got[:5], want[:5]):
        assert torch.allclose(a, b, rtol=1e-9, atol=1e-9)
