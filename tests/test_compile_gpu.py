"""The kernels under ``torch.compile``: with the ``aot_eager`` backend and ``fullgraph=True`` the operator, the
single-kernel layer steps and the whole layer function are captured without a graph break (each kernel is an opaque
``torch.library`` operator with a shape-only implementation and a registered backward), and the captured graph gives
what the eager call gives, forward and backward.  The reference runs its layers under ``torch.compile``
(lm_engine/model_wrapper/base.py:137-144)."""

import pytest
import torch

import lm_engine_amd
from tests.helpers import random_inputs


pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _same_gradient(a, b, name):
    # the backward kernels sum partial results with floating-point atomics: two runs agree to rounding, not bit by bit
    a, b = a.float(), b.float()
    assert (a - b).abs().max().item() <= 1e-4 * max(b.abs().max().item(), 1e-6), name


def _gpu(inp, grad=False):
    out = {}
    for n, x in inp.items():
        if isinstance(x, torch.Tensor):
            x = x.cuda()
            if grad and x.is_floating_point():
                x.requires_grad_(True)
        out[n] = x
    return out


def test_operator_forward_is_one_graph():
    inp = _gpu(random_inputs(B=2, T=257, H=2, K=128, V=128, dtype=BF16, seed=301))

    def fn(q, k, v, g, beta, initial_state):
        o, ht = lm_engine_amd.chunk_gated_delta_rule(q=q, k=k, v=v, g=g, beta=beta, initial_state=initial_state,
                                                     output_final_state=True)  # fmt: skip
        return o * 2, ht

    print("case: aot_eager fullgraph, chunked forward", flush=True)
    compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
    o_c, h_c = compiled(**inp)
    o_e, h_e = fn(**inp)
    assert torch.equal(o_c, o_e) and torch.equal(h_c, h_e)
    # no final state asked for: None comes back, as in eager mode
    no_state = torch.compile(lambda q, k, v, g, beta: lm_engine_amd.chunk_gated_delta_rule(q, k, v, g, beta),
                             backend="aot_eager", fullgraph=True)  # fmt: skip
    o_n, h_n = no_state(inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"])
    assert h_n is None and o_n.shape == o_e.shape


def test_operator_backward_through_the_captured_graph():
    base = random_inputs(B=1, T=192, H=2, K=128, V=128, dtype=BF16, seed=302)

    def loss(q, k, v, g, beta, initial_state):
        o, ht = lm_engine_amd.chunk_gated_delta_rule(q=q, k=k, v=v, g=g, beta=beta, initial_state=initial_state,
                                                     output_final_state=True)  # fmt: skip
        return (o.float() * o.float()).sum() + ht.sum()

    print("case: aot_eager fullgraph, chunked forward + backward", flush=True)
    eager_in, comp_in = _gpu(base, grad=True), _gpu(base, grad=True)
    loss(**eager_in).backward()
    torch.compile(loss, backend="aot_eager", fullgraph=True)(**comp_in).backward()
    for name in ("q", "k", "v", "g", "beta", "initial_state"):
        assert comp_in[name].grad is not None, name
        _same_gradient(comp_in[name].grad, eager_in[name].grad, name)


def test_decode_step_in_place_is_one_graph():
    inp = _gpu(random_inputs(B=4, T=1, H=4, K=128, V=128, dtype=BF16, seed=303))

    def step(q, k, v, g, beta, state):
        o, new_state = lm_engine_amd.fused_recurrent_gated_delta_rule(
            q=q, k=k, v=v, g=g, beta=beta, initial_state=state, output_final_state=True, inplace_state=True)  # fmt: skip
        return o, new_state

    print("case: aot_eager fullgraph, decode step updating the state in place", flush=True)
    s_eager, s_comp = inp["initial_state"].clone(), inp["initial_state"].clone()
    args = [inp[n] for n in ("q", "k", "v", "g", "beta")]
    o_e, h_e = step(*args, s_eager)
    o_c, h_c = torch.compile(step, backend="aot_eager", fullgraph=True)(*args, s_comp)
    assert torch.equal(o_c, o_e) and torch.equal(s_comp, s_eager) and torch.equal(h_c, s_comp)
    assert not torch.equal(s_comp, inp["initial_state"]), "the state was not updated"


def _layer_inputs(B, S, HK, HV, DK, DV, seed, grad):
    gen = torch.Generator("cpu").manual_seed(seed)
    r = lambda *shape, s=1.0: (torch.randn(*shape, generator=gen) * s)  # noqa: E731
    C = 2 * HK * DK + HV * DV
    t = dict(
        qkv=r(B, S, C).to(BF16), a=r(B, S, HV).to(BF16), b=r(B, S, HV).to(BF16), gate=r(B, S, HV * DV).to(BF16),
        conv_weight=r(C, 4, s=0.3).to(BF16), conv_bias=r(C, s=0.1).to(BF16), A_log=r(HV, s=0.3), dt_bias=r(HV, s=0.3),
        norm_weight=(1 + r(DV, s=0.1)).to(BF16),
    )  # fmt: skip
    t = {n: x.cuda().requires_grad_(grad) for n, x in t.items()}
    return t, dict(norm_eps=1e-5, num_k_heads=HK, num_v_heads=HV, k_head_dim=DK, v_head_dim=DV)


@pytest.mark.parametrize("S", [1, 200])
def test_whole_layer_is_one_graph_forward_and_backward(S):
    print(f"case: aot_eager fullgraph, layer function, S={S}", flush=True)
    options = None

    def layer(qkv, a, b, gate, conv_weight, conv_bias, A_log, dt_bias, norm_weight):
        o, cache = lm_engine_amd.gated_deltanet_mixing(qkv, a, b, gate, conv_weight, conv_bias, A_log, dt_bias,
                                                       norm_weight, cache=(None, None), **options)  # fmt: skip
        return o, cache[0], cache[1]

    eager_in, options = _layer_inputs(2, S, 2, 4, 128, 128, 310 + S, grad=True)
    comp_in, _ = _layer_inputs(2, S, 2, 4, 128, 128, 310 + S, grad=True)
    o_e, conv_e, h_e = layer(**eager_in)
    o_c, conv_c, h_c = torch.compile(layer, backend="aot_eager", fullgraph=True)(**comp_in)
    assert torch.equal(o_c, o_e) and torch.equal(conv_c, conv_e) and torch.equal(h_c, h_e)
    o_e.float().square().sum().backward()
    o_c.float().square().sum().backward()
    for name in eager_in:
        assert comp_in[name].grad is not None, name
        _same_gradient(comp_in[name].grad, eager_in[name].grad, name)


def test_compiled_convolution_without_a_backward_kernel_differentiates_its_formula():
    """fp32 inputs and a convolution without activation have no backward kernel: under capture they go in as torch
    operations (decided at trace time), so forward + backward compile and agree with eager mode."""
    gen = torch.Generator().manual_seed(77)
    for dtype, activation in ((torch.float32, "silu"), (BF16, None)):
        x = torch.randn(2, 70, 64, generator=gen).to(dtype).cuda()
        w = (0.3 * torch.randn(64, 1, 4, generator=gen)).to(dtype).cuda()

        def run(fn):
            xs, ws = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
            y, _ = fn(xs, ws)
            (y.float() * torch.arange(y.numel(), device="cuda").view_as(y).float().cos()).sum().backward()
            return y, xs.grad, ws.grad

        f = lambda xs, ws: lm_engine_amd.depthwise_causal_convolution(xs, ws, None, None, None, False, activation)  # noqa: E731
        eager = run(f)
        compiled = run(torch.compile(f, backend="aot_eager", fullgraph=True))
        for name, a, b in zip(("y", "dx", "dw"), compiled, eager):
            assert torch.allclose(a.float(), b.float(), rtol=2e-2, atol=2e-2), f"{dtype} {activation} {name}"
