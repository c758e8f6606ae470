"""Parity of the gates and gated-RMSNorm kernels (through the C ABI) against the CPU oracle.
Gates: fp32 outputs within 1e-5 relative; bf16 outputs within max-abs 2e-2 and relative-L2 1e-2."""

import pytest
import torch

import lm_engine_amd
from oracle.layer_oracle import delta_rule_gates_ref, gated_rmsnorm_ref
from tests.helpers import max_abs, rel_l2


pytestmark = pytest.mark.gpu
BF16, F32, F64 = torch.bfloat16, torch.float32, torch.float64


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("neg", [False, True])
def test_gates_on_slices_of_one_projection(dtype, neg):
    B, T, H, V = 2, 77, 6, 16
    g = torch.Generator().manual_seed(3)
    ab = (3 * torch.randn(B, T, 2 * H + H * V, generator=g)).to(dtype)  # the layer's ab_proj output: a | b | gate
    ab[0, 0, 0] = 40.0  # softplus threshold branch
    a, b = ab[..., :H], ab[..., H : 2 * H]
    A_log = torch.log(torch.rand(H, generator=g) * 16 + 1e-3)
    dt_bias = torch.randn(H, generator=g)
    print(f"case: gates {dtype} neg={neg} a stride {a.stride()}", flush=True)
    g_ref, beta_ref = delta_rule_gates_ref(a.to(F64), b.to(F64), A_log.to(F64), dt_bias.to(F64), neg)
    abd = ab.cuda()
    g_out, beta = lm_engine_amd.delta_rule_gates(abd[..., :H], abd[..., H : 2 * H], A_log.cuda(), dt_bias.cuda(), neg)
    torch.cuda.synchronize()
    assert g_out.dtype == F32 and beta.dtype == dtype and g_out.shape == a.shape and beta.shape == a.shape
    assert (g_out <= 0).all()
    torch.testing.assert_close(g_out.cpu().to(F64), g_ref, rtol=1e-5, atol=1e-6)
    if dtype == F32:
        torch.testing.assert_close(beta.cpu().to(F64), beta_ref, rtol=1e-5, atol=1e-6)
    else:
        assert max_abs(beta, beta_ref) <= 2e-2 and rel_l2(beta, beta_ref) <= 1e-2


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("V", [64, 96, 128, 256, 512])
@pytest.mark.parametrize("gated", [False, True])
def test_gated_rmsnorm(dtype, V, gated):
    B, T, H = 2, 45, 3
    g = torch.Generator().manual_seed(V)
    o = torch.randn(B, T, H, V, generator=g).to(dtype)
    proj = torch.randn(B, T, 8 + H * V, generator=g).to(dtype)  # gate is a slice of a wider projection
    gate = proj[..., 8:] if gated else None
    w = (1 + 0.1 * torch.randn(V, generator=g)).to(dtype)
    print(f"case: gated_rmsnorm {dtype} V={V} gated={gated}", flush=True)
    y_ref = gated_rmsnorm_ref(o.to(F64), None if gate is None else gate.to(F64), w.to(F64), 1e-5)
    pd = proj.cuda()
    y = lm_engine_amd.gated_rmsnorm(o.cuda(), pd[..., 8:] if gated else None, w.cuda(), 1e-5)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == o.shape
    if dtype == F32:
        torch.testing.assert_close(y.cpu().to(F64), y_ref, rtol=1e-5, atol=1e-5)
    else:
        assert max_abs(y, y_ref) <= 2e-2 * max(1.0, float(y_ref.abs().max())) and rel_l2(y, y_ref) <= 1e-2
    # the [.., H, V] view of the gate slice is accepted as well
    if gated:
        y2 = lm_engine_amd.gated_rmsnorm(o.cuda(), pd[..., 8:].view(B, T, H, V), w.cuda(), 1e-5)
        assert torch.equal(y, y2)


def test_gate_slice_off_a_16_byte_boundary():
    # with 2 or 3 heads the gate columns start 2 * H elements into the projection: 8 or 12 bytes in bf16
    B, T, H, V = 2, 33, 3, 512
    g = torch.Generator().manual_seed(9)
    o = torch.randn(B, T, H, V, generator=g).to(BF16)
    proj = torch.randn(B, T, 2 * H + H * V, generator=g).to(BF16)
    y_ref = gated_rmsnorm_ref(o.to(F64), proj[..., 2 * H :].to(F64), None, 1e-6)
    y = lm_engine_amd.gated_rmsnorm(o.cuda(), proj.cuda()[..., 2 * H :], None, 1e-6)
    assert rel_l2(y, y_ref) <= 1e-2


def test_rejected_arguments():
    o = torch.randn(2, 3, 4, 20, device="cuda")
    with pytest.raises(ValueError):
        lm_engine_amd.gated_rmsnorm(o, None, None)  # V not a multiple of 8
    with pytest.raises(ValueError):
        lm_engine_amd.gated_rmsnorm(torch.randn(2, 3, 4, 16), None, None)  # not on the GPU
    a = torch.randn(2, 5, 4, device="cuda")
    with pytest.raises(ValueError):
        lm_engine_amd.delta_rule_gates(a, a, torch.zeros(3), torch.zeros(4))
