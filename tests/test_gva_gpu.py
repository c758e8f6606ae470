"""Grouped value attention: q and k with fewer heads than v (``gdn_args.qk_heads``).  Value head h reads head
h / (H / HQK) of q and k - what the reference's ``repeat_interleave`` copies would put there
(gated_deltanet/module.py:175-177) - so every result must equal, bit for bit, the run on the expanded tensors (same
kernels, same arithmetic), which in turn is checked against the oracle elsewhere; one case here goes to the oracle
directly.  Gradients of q and k are the sums over a group's copies."""

import pytest
import torch

import lm_engine_amd
from lm_engine_amd.ops import fused_launch_applies
from oracle.gdn_oracle import recurrent_gated_delta_rule_ref
from tests.helpers import assert_parity, rel_l2


pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _inputs(B, T, HQK, H, K, V, dtype, seed, with_state=True, N=None):
    gen = torch.Generator().manual_seed(seed)
    norm = lambda x: x / x.norm(dim=-1, keepdim=True)  # noqa: E731
    q, k = norm(torch.randn(B, T, HQK, K, generator=gen)), norm(torch.randn(B, T, HQK, K, generator=gen))
    v = torch.randn(B, T, H, V, generator=gen)
    g = torch.nn.functional.logsigmoid(3 + torch.randn(B, T, H, generator=gen))
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    h0 = 0.02 * torch.randn(N or B, H, K, V, generator=gen) if with_state else None
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), g=g, beta=beta.to(dtype), initial_state=h0)


def _expanded(inp):
    group = inp["v"].size(2) // inp["q"].size(2)
    out = dict(inp)
    out["q"], out["k"] = inp["q"].repeat_interleave(group, dim=2), inp["k"].repeat_interleave(group, dim=2)
    return out


def _cuda(inp):
    return {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}


@pytest.mark.parametrize(
    "B, T, HQK, H, K, V, l2norm",
    [
        (4, 1024, 4, 16, 128, 128, False),  # runs as one launch
        (2, 300, 2, 6, 128, 128, True),  # two kernels, tail chunk
        (2, 256, 1, 4, 64, 64, False),
        (2, 512, 2, 4, 256, 512, False),  # the shipped head shape with a group of two
        (8, 512, 8, 32, 128, 256, False),  # four slices per workgroup
    ],
)
def test_chunked_forward_equals_the_run_on_expanded_heads(B, T, HQK, H, K, V, l2norm):
    inp = _cuda(_inputs(B, T, HQK, H, K, V, BF16, seed=B * T + H))
    print(f"case: GVA chunked forward q={tuple(inp['q'].shape)} v={tuple(inp['v'].shape)} one launch: "
          f"{fused_launch_applies(inp['q'], inp['v'])}", flush=True)  # fmt: skip
    kw = dict(output_final_state=True, use_qk_l2norm_in_kernel=l2norm)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**inp, **kw)
    o_x, ht_x = lm_engine_amd.chunk_gated_delta_rule(**_expanded(inp), **kw)
    assert o.shape == (B, T, H, V) and ht.shape == (B, H, K, V)
    assert torch.equal(o, o_x) and torch.equal(ht, ht_x)


def test_chunked_forward_against_the_oracle():
    inp = _inputs(2, 200, 2, 8, 128, 128, BF16, seed=5)
    want_o, want_h = recurrent_gated_delta_rule_ref(**{n: (x.double() if isinstance(x, torch.Tensor) else x) for n, x in _expanded(inp).items()},
                                                    output_final_state=True)  # fmt: skip
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**_cuda(inp), output_final_state=True)
    assert_parity(o.cpu(), want_o, BF16, "o")
    assert_parity(ht.cpu(), want_h, BF16, "final state")


def test_packed_batch_equals_the_run_on_expanded_heads():
    lens = [130, 64, 300, 18]
    inp = _inputs(1, sum(lens), 2, 8, 128, 128, BF16, seed=9, N=len(lens))
    inp["cu_seqlens"] = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    inp = _cuda(inp)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    o_x, ht_x = lm_engine_amd.chunk_gated_delta_rule(**_expanded(inp), output_final_state=True)
    assert torch.equal(o, o_x) and torch.equal(ht, ht_x)


@pytest.mark.parametrize("dtype", [BF16, torch.float32])
@pytest.mark.parametrize("T", [1, 7])
def test_recurrent_step_equals_the_run_on_expanded_heads(dtype, T):
    inp = _cuda(_inputs(5, T, 2, 6, 128, 128, dtype, seed=T))
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**inp, output_final_state=True)
    o_x, ht_x = lm_engine_amd.fused_recurrent_gated_delta_rule(**_expanded(inp), output_final_state=True)
    assert torch.equal(o, o_x) and torch.equal(ht, ht_x)


def test_heads_that_do_not_divide_are_refused():
    inp = _cuda(_inputs(1, 64, 3, 8, 128, 128, BF16, seed=1))
    with pytest.raises(ValueError, match="multiple of the heads"):
        lm_engine_amd.chunk_gated_delta_rule(**inp)


@pytest.mark.parametrize("K, V", [(128, 128), (256, 512)])
def test_gradients_are_the_sums_over_a_group(K, V):
    """Autograd through the operator with shared heads against autograd through repeat_interleave in front of it."""
    inp = _cuda(_inputs(2, 192, 2, 4, K, V, BF16, seed=K))
    gen = torch.Generator().manual_seed(77)
    do = torch.randn(2, 192, 4, V, generator=gen).to(BF16).cuda()
    dht = (0.1 * torch.randn(2, 4, K, V, generator=gen)).cuda()
    names = ("q", "k", "v", "g", "beta", "initial_state")

    def grads(expand):
        leaves = {n: inp[n].detach().clone().requires_grad_(True) for n in names}
        args = _expanded(leaves) if expand else leaves
        o, ht = lm_engine_amd.chunk_gated_delta_rule(**args, output_final_state=True)
        return torch.autograd.grad((o.float() * do.float()).sum() + (ht * dht).sum(), [leaves[n] for n in names])

    for name, a, b in zip(names, grads(False), grads(True)):
        assert a.shape == inp[name].shape
        err = rel_l2(a, b)
        print(f"   K={K} V={V} d{name}: rel-L2 {err:.3e}", flush=True)
        assert err <= 4e-3, f"d{name}: rel-L2 {err:.3e}"  # the group's sum is rounded once here, per copy and then summed there
