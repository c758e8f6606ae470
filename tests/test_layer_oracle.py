"""Pins oracle/layer_oracle.py: hand-computed values and invariants next to the torch routines."""

import math

import torch

from oracle.layer_oracle import delta_rule_gates_ref, gated_rmsnorm_ref


F64 = torch.float64


def test_gates_hand_values():
    a = torch.tensor([[0.0, 30.0]], dtype=F64)
    b = torch.tensor([[0.0, math.log(3.0)]], dtype=F64)
    A_log = torch.tensor([0.0, math.log(2.0)], dtype=F64)
    dt_bias = torch.tensor([0.0, 1.0], dtype=F64)
    g, beta = delta_rule_gates_ref(a, b, A_log, dt_bias)
    # softplus(0) = ln 2; softplus(31) = 31 up to e^-31
    assert abs(g[0, 0].item() + math.log(2.0)) < 1e-12 and abs(g[0, 1].item() + 2.0 * 31.0) < 1e-10
    assert abs(beta[0, 0].item() - 0.5) < 1e-12 and abs(beta[0, 1].item() - 0.75) < 1e-12
    _, beta2 = delta_rule_gates_ref(a, b, A_log, dt_bias, allow_neg_eigval=True)
    assert torch.equal(beta2, 2 * beta)
    assert (g <= 0).all()


def test_gated_rmsnorm_hand_values_and_invariants():
    o = torch.tensor([[[3.0, 4.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]]], dtype=F64)  # mean square 25 / 8
    y = gated_rmsnorm_ref(o, None, None, 0.0)
    assert torch.allclose(y[0, 0, :2], torch.tensor([3.0, 4.0], dtype=F64) / math.sqrt(25.0 / 8.0), atol=1e-12)
    g = torch.Generator().manual_seed(0)
    o = torch.randn(2, 3, 4, 16, generator=g, dtype=F64)
    gate = torch.randn(2, 3, 4, 16, generator=g, dtype=F64)
    w = torch.randn(16, generator=g, dtype=F64)
    y = gated_rmsnorm_ref(o, gate, w, 1e-6)
    # scale invariance of the normalisation (up to eps), linearity in the weight, rows independent
    assert torch.allclose(gated_rmsnorm_ref(7.0 * o, gate, w, 0.0), gated_rmsnorm_ref(o, gate, w, 0.0), atol=1e-12)
    assert torch.allclose(gated_rmsnorm_ref(o, gate, 2 * w, 1e-6), 2 * y, atol=1e-12)
    y_row = gated_rmsnorm_ref(o[1:2, 2:3, 3:4], gate[1:2, 2:3, 3:4], w, 1e-6)
    assert torch.allclose(y_row, y[1:2, 2:3, 3:4], atol=1e-14)
    # by hand: x = o * gate * sigmoid(gate)
    x = o * gate / (1 + torch.exp(-gate))
    manual = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w
    assert torch.allclose(y, manual, atol=1e-12)
    # a flat gate [.., H * V] means the same
    assert torch.equal(gated_rmsnorm_ref(o, gate.flatten(-2), w, 1e-6), y)
