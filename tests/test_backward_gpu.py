"""Autograd through the operators on the GPU: forward on the HIP kernels, gradients against autograd
through the fp64 token loop of the oracle on the same (rounded) inputs.

Gate for a gradient: relative-L2 <= 1e-2 and max-abs <= 2e-2 x max(1, max |reference|) for bf16 inputs
(the gradients come back rounded to bf16), 1e-4 on both for fp32 inputs."""

import pytest
import torch

import lm_engine_amd
from oracle.gdn_backward_oracle import gated_delta_rule_grads_autograd

from .helpers import max_abs, random_inputs, rel_l2


pytestmark = pytest.mark.gpu

NAMES = ("dq", "dk", "dv", "dg", "dbeta", "dh0")


def _leaves(inp):
    out = {}
    for name, x in inp.items():
        out[name] = None if x is None else x.cuda().requires_grad_(True)
    return out


def _assert_grads(got, want, dtype):
    for name, a, b in zip(NAMES, got, want):
        assert a is not None, name
        assert a.shape == b.shape, name
        ma, rl = max_abs(a, b), rel_l2(a, b)
        top = max(1.0, float(b.abs().max()))
        if dtype == torch.bfloat16:
            assert rl <= 1e-2 and ma <= 2e-2 * top, f"{name}: max-abs {ma:.3e} (top {top:.2f}), rel-L2 {rl:.3e}"
        else:
            assert rl <= 1e-4 and ma <= 1e-4 * top, f"{name}: max-abs {ma:.3e} (top {top:.2f}), rel-L2 {rl:.3e}"


def _run_case(fn, inp, dtype, cu=None, **kw):
    gen = torch.Generator().manual_seed(99)
    leaves = _leaves(inp)
    cu_dev = None if cu is None else cu.cuda()
    o, ht = fn(**leaves, output_final_state=True, cu_seqlens=cu_dev, use_qk_l2norm_in_kernel=True, **kw)
    do = torch.randn(o.shape, generator=gen).to(dtype)
    dht = torch.randn(ht.shape, generator=gen)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    got = [leaves[n].grad for n in ("q", "k", "v", "g", "beta", "initial_state")]
    want = gated_delta_rule_grads_autograd(
        inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"], do, dht, initial_state=inp["initial_state"],
        cu_seqlens=cu, use_qk_l2norm_in_kernel=True,
    )  # fmt: skip
    _assert_grads(got, want, dtype)
    assert [x.dtype for x in got[:3]] == [dtype] * 3


@pytest.mark.parametrize("T", [65, 256])
def test_chunk_bf16(T):
    inp = random_inputs(B=2, T=T, H=2, K=128, V=128, dtype=torch.bfloat16, seed=T, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


def test_chunk_bf16_packed():
    cu = torch.tensor([0, 70, 71, 300], dtype=torch.int32)
    inp = random_inputs(B=1, T=300, H=2, K=128, V=64, dtype=torch.bfloat16, seed=7, normalize=False, N=3)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)


def test_recurrent_fp32():
    inp = random_inputs(B=2, T=40, H=2, K=64, V=64, dtype=torch.float32, seed=8, normalize=False)
    _run_case(lm_engine_amd.fused_recurrent_gated_delta_rule, inp, torch.float32)
