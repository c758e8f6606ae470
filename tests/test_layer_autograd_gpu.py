"""Gradients through the layer's single-kernel steps and through the whole chain
(convolution -> gates -> operator -> gated norm), against autograd through the fp64 CPU oracles."""

import pytest
import torch

import lm_engine_amd
from oracle import recurrent_gated_delta_rule_ref
from oracle.conv_oracle import depthwise_causal_convolution_ref
from oracle.layer_oracle import delta_rule_gates_ref, gated_rmsnorm_ref
from tests.helpers import rel_l2


pytestmark = pytest.mark.gpu
BF16, F32, F64 = torch.bfloat16, torch.float32, torch.float64


def _grads(fn, tensors, cotangents):
    leaves = [x.detach().clone().requires_grad_(True) for x in tensors]
    outs = fn(*leaves)
    outs = [o for o in outs if o is not None]
    loss = sum((o.to(c.dtype) * c).sum() for o, c in zip(outs, cotangents))
    return torch.autograd.grad(loss, leaves)


def _grads_allow_unused(fn, tensors, cotangents):
    leaves = [x.detach().clone().requires_grad_(True) for x in tensors]
    outs = [o for o in fn(*leaves) if o is not None]
    loss = sum((o.to(c.dtype) * c).sum() for o, c in zip(outs, cotangents))
    return torch.autograd.grad(loss, leaves, allow_unused=True)


def _compare(got, want, tol, names):
    for name, a, b in zip(names, got, want):
        err = rel_l2(a, b)
        assert err <= tol, f"{name}: rel-L2 {err:.3e} > {tol}"


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 6e-3)])
@pytest.mark.parametrize("shape,H", [((3, 50), 8), ((2, 1031), 12), ((777,), 40)])
def test_gates_gradients(dtype, tol, shape, H):
    """The gates' backward kernel (da, db per token, dA_log and ddt_bias reduced over tokens) against autograd
    through the fp64 oracle, on the values the kernel reads (bf16 inputs are rounded first); a and b are column
    slices of one wider projection, as the layer hands them over."""
    gen = torch.Generator().manual_seed(1)
    proj = torch.randn(*shape, 2 * H + 3, generator=gen).to(dtype)
    A_log, dt_bias = torch.randn(H, generator=gen), torch.randn(H, generator=gen)
    cg, cb = torch.randn(*shape, H, generator=gen), torch.randn(*shape, H, generator=gen).to(dtype)
    cut = lambda p: (p[..., :H], p[..., H + 3 :])  # noqa: E731

    def ref(p, A, d):
        return delta_rule_gates_ref(*cut(p), A, d, True)

    def ours(p, A, d):
        return lm_engine_amd.delta_rule_gates(*cut(p), A, d, True)

    want = _grads(ref, [x.to(F64) for x in (proj, A_log, dt_bias)], [cg.to(F64), cb.to(F64)])
    got = _grads(ours, [x.cuda() for x in (proj, A_log, dt_bias)], [cg.cuda(), cb.cuda()])
    keep = torch.ones(2 * H + 3, dtype=torch.bool)
    keep[H : H + 3] = False
    assert torch.count_nonzero(got[0][..., ~keep]) == 0
    _compare([got[0][..., keep], *got[1:]], [want[0][..., keep], *want[1:]], tol, ("da|db", "dA_log", "ddt_bias"))


def test_gates_gradient_of_one_output_only():
    gen = torch.Generator().manual_seed(4)
    H = 16
    a, b = torch.randn(5, 33, H, generator=gen), torch.randn(5, 33, H, generator=gen)
    A_log, dt_bias = torch.randn(H, generator=gen), torch.randn(H, generator=gen)
    c = torch.randn(5, 33, H, generator=gen)
    for which in (0, 1):
        want = _grads_allow_unused(lambda *t: (delta_rule_gates_ref(*t, False)[which],), [x.to(F64) for x in (a, b, A_log, dt_bias)], [c.to(F64)])
        got = _grads_allow_unused(lambda *t: (lm_engine_amd.delta_rule_gates(*t, False)[which],), [x.cuda() for x in (a, b, A_log, dt_bias)], [c.cuda()])
        for name, x, y in zip(("da", "db", "dA_log", "ddt_bias"), got, want):
            if y is None:
                assert x is None or torch.count_nonzero(x) == 0, name
            else:
                assert rel_l2(x, y) <= 1e-5, name


@pytest.mark.parametrize("gated", [False, True])
def test_gated_rmsnorm_gradients(gated):
    gen = torch.Generator().manual_seed(2)
    o, gate, w = torch.randn(2, 40, 4, 64, generator=gen), torch.randn(2, 40, 4, 64, generator=gen), torch.randn(64, generator=gen)
    c = torch.randn(2, 40, 4, 64, generator=gen)
    if gated:
        want = _grads(lambda o, g, w: (gated_rmsnorm_ref(o, g, w, 1e-5),), [x.to(F64) for x in (o, gate, w)], [c.to(F64)])
        got = _grads(lambda o, g, w: (lm_engine_amd.gated_rmsnorm(o, g, w, 1e-5),), [x.cuda() for x in (o, gate, w)], [c.cuda()])
        _compare(got, want, 1e-5, ("do", "dgate", "dweight"))
    else:
        want = _grads(lambda o, w: (gated_rmsnorm_ref(o, None, w, 1e-5),), [x.to(F64) for x in (o, w)], [c.to(F64)])
        got = _grads(lambda o, w: (lm_engine_amd.gated_rmsnorm(o, None, w, 1e-5),), [x.cuda() for x in (o, w)], [c.cuda()])
        _compare(got, want, 1e-5, ("do", "dweight"))


@pytest.mark.parametrize("V, gated, weighted", [(128, True, True), (256, True, False), (64, False, True), (72, True, True)])
def test_gated_rmsnorm_gradients_bf16(V, gated, weighted):
    """bf16, gate as a strided slice of a wider projection: the backward is ``gdn_gated_rmsnorm_bwd``."""
    gen = torch.Generator().manual_seed(V)
    B, S, H = 2, 33, 3
    o = torch.randn(B, S, H, V, generator=gen).to(BF16)
    proj = torch.randn(B, S, 2 * H + H * V, generator=gen).to(BF16)
    w = (1 + 0.1 * torch.randn(V, generator=gen)).to(BF16)
    c = torch.randn(B, S, H, V, generator=gen).to(BF16)

    def oracle(o, proj, w):
        gate = proj[..., 2 * H :] if gated else None
        return (gated_rmsnorm_ref(o, gate, w if weighted else None, 1e-5),)

    def kernels(o, proj, w):
        gate = proj[..., 2 * H :] if gated else None
        return (lm_engine_amd.gated_rmsnorm(o, gate, w if weighted else None, 1e-5),)

    want = _grads_allow_unused(oracle, [t.to(F64) for t in (o, proj, w)], [c.to(F64)])
    got = _grads_allow_unused(kernels, [t.cuda() for t in (o, proj, w)], [c.cuda()])
    for name, a, b in zip(("do", "dproj", "dweight"), got, want):
        if b is None:
            assert a is None, name
        else:
            assert rel_l2(a, b) <= 1e-2, f"{name}: rel-L2 {rel_l2(a, b):.3e}"


@pytest.mark.parametrize("S, ks", [(1, 4), (2, 3), (64, 4), (130, 2), (200, 4)])
@pytest.mark.parametrize("with_state, masked, silu", [(False, False, True), (True, False, True), (False, True, True), (True, True, False)])
def test_convolution_gradients_bf16_kernel(with_state, masked, silu, S, ks):
    """bf16 x: the backward is ``gdn_causal_conv1d_bwd``; against autograd through the fp64 oracle on the same
    (rounded) inputs.  The gradient is taken of y only (the cache state is not differentiated through)."""
    gen = torch.Generator().manual_seed(100 * S + ks)
    B, C = 3, 72
    rt = lambda t: t.to(BF16)  # noqa: E731
    x, w = rt(torch.randn(B, S, C, generator=gen)), rt(0.5 * torch.randn(C, 1, ks, generator=gen))
    bias, state = rt(torch.randn(C, generator=gen)), rt(torch.randn(B, C, ks - 1, generator=gen))
    cy = rt(torch.randn(B, S, C, generator=gen))
    mask = torch.ones(B, S)
    if masked and S > 1:
        mask[1, : S // 3] = 0
        mask[2, : S - 1] = 0
    m = mask if masked else None
    act = "silu" if silu else None
    tensors = [x, w, bias] + ([state] if with_state else [])
    oracle = lambda x, w, b, s=None: (depthwise_causal_convolution_ref(x, w, b, s, m, False, act)[0],)  # noqa: E731
    kernels = lambda x, w, b, s=None: (lm_engine_amd.depthwise_causal_convolution(  # noqa: E731
        x, w, b, s, None if m is None else m.cuda(), True, act)[0],)  # fmt: skip
    want = _grads(oracle, [t.to(F64) for t in tensors], [cy.to(F64)])
    got = _grads(kernels, [t.cuda() for t in tensors], [cy.cuda()])
    assert [g.dtype for g in got] == [t.dtype for t in tensors]
    names = ("dx", "dweight", "dbias", "dstate")
    for name, a, b in zip(names, got, want):
        if float(b.abs().max()) == 0.0:
            assert not a.any(), name
        else:
            assert rel_l2(a, b) <= 1e-2, f"{name}: rel-L2 {rel_l2(a, b):.3e}"


@pytest.mark.parametrize("S, ks", [(37, 4), (1, 4), (2, 3), (200, 2)])
@pytest.mark.parametrize("with_state, masked", [(False, False), (True, False), (False, True), (True, True)])
def test_convolution_gradients(with_state, masked, S, ks):
    """fp32 x: ``gdn_causal_conv1d_bwd`` again (4 channels per 16-byte access), and the gradient that flows into the
    returned state (rows of dx, or of dstate when the sequence is shorter than the state)."""
    gen = torch.Generator().manual_seed(3)
    B, C = 3, 68
    x, w, bias = torch.randn(B, S, C, generator=gen), 0.5 * torch.randn(C, 1, ks, generator=gen), torch.randn(C, generator=gen)
    state = torch.randn(B, C, ks - 1, generator=gen)
    mask = torch.ones(B, S)
    if masked and S > 1:
        mask[1, : S // 3] = 0
        mask[2, : S - 1] = 0
    cy, cs = torch.randn(B, S, C, generator=gen), torch.randn(B, C, ks - 1, generator=gen)
    m = mask if masked else None
    if with_state:
        want = _grads(lambda x, w, b, s: depthwise_causal_convolution_ref(x, w, b, s, m, True), [t.to(F64) for t in (x, w, bias, state)], [cy.to(F64), cs.to(F64)])
        got = _grads(lambda x, w, b, s: lm_engine_amd.depthwise_causal_convolution(x, w, b, s, None if m is None else m.cuda(), True),
                     [t.cuda() for t in (x, w, bias, state)], [cy.cuda(), cs.cuda()])  # fmt: skip
        _compare(got, want, 1e-5, ("dx", "dweight", "dbias", "dstate"))
    else:
        want = _grads(lambda x, w, b: depthwise_causal_convolution_ref(x, w, b, None, m, True), [t.to(F64) for t in (x, w, bias)], [cy.to(F64), cs.to(F64)])
        got = _grads(lambda x, w, b: lm_engine_amd.depthwise_causal_convolution(x, w, b, None, None if m is None else m.cuda(), True),
                     [t.cuda() for t in (x, w, bias)], [cy.cuda(), cs.cuda()])  # fmt: skip
        _compare(got, want, 1e-5, ("dx", "dweight", "dbias"))


def test_layer_chain_gradients():
    B, S, HK, HV, DK, DV = 2, 130, 2, 4, 128, 128
    key_dim, value_dim = HK * DK, HV * DV
    gen = torch.Generator().manual_seed(4)
    qkv = torch.randn(B, S, 2 * key_dim + value_dim, generator=gen).to(BF16)
    ab = torch.randn(B, S, 2 * HV + value_dim, generator=gen).to(BF16)
    conv_w = (0.4 * torch.randn(2 * key_dim + value_dim, 1, 4, generator=gen)).to(BF16)
    conv_b = (0.1 * torch.randn(2 * key_dim + value_dim, generator=gen)).to(BF16)
    A_log = torch.log(torch.rand(HV, generator=gen) * 4 + 0.1)
    dt_bias = torch.randn(HV, generator=gen) - 2.0
    norm_w = (1 + 0.1 * torch.randn(DV, generator=gen)).to(BF16)
    c = torch.randn(B, S, value_dim, generator=gen)

    def oracle(qkv, ab, conv_w, conv_b, A_log, dt_bias, norm_w):
        y, _ = depthwise_causal_convolution_ref(qkv, conv_w, conv_b, None, None, False)
        q, k, v = y.split((key_dim, key_dim, value_dim), dim=-1)
        q = q.reshape(B, S, HK, DK).repeat_interleave(HV // HK, dim=-2)
        k = k.reshape(B, S, HK, DK).repeat_interleave(HV // HK, dim=-2)
        v = v.reshape(B, S, HV, DV)
        a, b, gate = ab[..., :HV], ab[..., HV : 2 * HV], ab[..., 2 * HV :]
        g, beta = delta_rule_gates_ref(a, b, A_log, dt_bias, False)
        o, _ = recurrent_gated_delta_rule_ref(q, k, v, g=g, beta=beta, use_qk_l2norm_in_kernel=True, state_dtype=F64)
        return (gated_rmsnorm_ref(o, gate, norm_w, 1e-5).flatten(-2),)

    def kernels(qkv, ab, conv_w, conv_b, A_log, dt_bias, norm_w):
        a, b, gate = ab[..., :HV], ab[..., HV : 2 * HV], ab[..., 2 * HV :]
        out, _ = lm_engine_amd.gated_deltanet_mixing(qkv, a, b, gate, conv_w, conv_b, A_log, dt_bias, norm_w, 1e-5,
                                                     HK, HV, DK, DV)  # fmt: skip
        return (out,)

    tensors = (qkv, ab, conv_w, conv_b, A_log, dt_bias, norm_w)
    want = _grads(oracle, [t.to(F64) for t in tensors], [c.to(F64)])
    got = _grads(kernels, [t.cuda() for t in tensors], [c.cuda()])
    assert [g.dtype for g in got] == [t.dtype for t in tensors]
    _compare(got, want, 3e-2, ("dqkv", "dab", "dconv_weight", "dconv_bias", "dA_log", "ddt_bias", "dnorm_weight"))
