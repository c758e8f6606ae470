"""End to end over the kernels of the layer (convolution -> gates -> operator -> gated norm), chained as
`GatedDeltaNet.forward` chains them (gated_deltanet/module.py:168-242), against the same chain of CPU
oracles; and prefill + decode through the cache against one long prefill."""

import pytest
import torch

import lm_engine_amd
from oracle import recurrent_gated_delta_rule_ref
from oracle.conv_oracle import depthwise_causal_convolution_ref
from oracle.layer_oracle import delta_rule_gates_ref, gated_rmsnorm_ref
from tests.helpers import max_abs, rel_l2


pytestmark = pytest.mark.gpu
BF16, F64 = torch.bfloat16, torch.float64


def _layer_inputs(B, S, HK, HV, DK, DV, seed):
    g = torch.Generator().manual_seed(seed)
    key_dim, value_dim = HK * DK, HV * DV
    qkv = torch.randn(B, S, 2 * key_dim + value_dim, generator=g).to(BF16)
    ab = torch.randn(B, S, 2 * HV + value_dim, generator=g).to(BF16)
    params = dict(
        conv_weight=(0.4 * torch.randn(2 * key_dim + value_dim, 1, 4, generator=g)).to(BF16),
        conv_bias=(0.1 * torch.randn(2 * key_dim + value_dim, generator=g)).to(BF16),
        A_log=torch.log(torch.rand(HV, generator=g) * 4 + 0.1),
        dt_bias=torch.randn(HV, generator=g) - 2.0,
        norm_weight=(1 + 0.1 * torch.randn(DV, generator=g)).to(BF16),
    )
    return qkv, ab, params


def _oracle_chain(qkv, ab, params, HK, HV, DK, DV, cache, neg):
    """The same steps on the CPU in fp64, rounding to bf16 where the kernels hand bf16 tensors on."""
    B, S, _ = qkv.shape
    key_dim, value_dim = HK * DK, HV * DV
    rt = lambda x: x.to(BF16).to(F64)  # noqa: E731
    conv_state, h = cache
    y, conv_state = depthwise_causal_convolution_ref(qkv.to(F64), params["conv_weight"].to(F64), params["conv_bias"].to(F64),
                                                     None if conv_state is None else conv_state.to(F64), None, True)  # fmt: skip
    y = rt(y)
    q, k, v = y.split((key_dim, key_dim, value_dim), dim=-1)
    q = q.reshape(B, S, HK, DK).repeat_interleave(HV // HK, dim=-2)
    k = k.reshape(B, S, HK, DK).repeat_interleave(HV // HK, dim=-2)
    v = v.reshape(B, S, HV, DV)
    a, b, gate = ab[..., :HV], ab[..., HV : 2 * HV], ab[..., 2 * HV :]
    g, beta = delta_rule_gates_ref(a.to(F64), b.to(F64), params["A_log"].to(F64), params["dt_bias"].to(F64), neg)
    g, beta = g.float().to(F64), rt(beta)
    o, h = recurrent_gated_delta_rule_ref(q, k, v, g=g, beta=beta, initial_state=h, output_final_state=True,
                                          use_qk_l2norm_in_kernel=True)  # fmt: skip
    o = rt(o)
    out = gated_rmsnorm_ref(o, gate.to(F64), params["norm_weight"].to(F64), 1e-5)
    return out.flatten(-2), (conv_state, h)


def _gpu_chain(qkv, ab, params, HK, HV, DK, DV, cache, neg, attention_mask=None):
    dev = {n: x.cuda() for n, x in params.items()}
    abd = ab.cuda()
    a, b, gate = abd[..., :HV], abd[..., HV : 2 * HV], abd[..., 2 * HV :]
    return lm_engine_amd.gated_deltanet_mixing(
        qkv.cuda(), a, b, gate, dev["conv_weight"], dev["conv_bias"], dev["A_log"], dev["dt_bias"], dev["norm_weight"],
        1e-5, HK, HV, DK, DV, cache=cache, allow_neg_eigval=neg,
        attention_mask=None if attention_mask is None else attention_mask.cuda())  # fmt: skip


@pytest.mark.parametrize("HK, HV, DK, DV, S", [(2, 4, 128, 128, 200), (4, 4, 64, 64, 130), (2, 2, 128, 256, 70), (4, 8, 128, 128, 40)])
def test_layer_chain_matches_the_chain_of_oracles(HK, HV, DK, DV, S):
    B = 2
    qkv, ab, params = _layer_inputs(B, S, HK, HV, DK, DV, seed=S)
    print(f"case: layer B={B} S={S} heads {HK}/{HV} dims {DK}/{DV}", flush=True)
    ref, (cs_ref, h_ref) = _oracle_chain(qkv, ab, params, HK, HV, DK, DV, (None, None), neg=True)
    out, (cs, h) = _gpu_chain(qkv, ab, params, HK, HV, DK, DV, (None, None), neg=True)
    torch.cuda.synchronize()
    print(f"   out: max-abs {max_abs(out, ref):.3e} rel-L2 {rel_l2(out, ref):.3e}  h: rel-L2 {rel_l2(h, h_ref):.3e}", flush=True)
    assert out.shape == (B, S, HV * DV) and out.dtype == BF16
    # the normalised output is O(1); intermediate bf16 roundings of the two chains differ by an ulp here and there
    assert rel_l2(out, ref) <= 2e-2 and max_abs(out, ref) <= 1e-1
    assert rel_l2(h, h_ref) <= 1e-2
    assert torch.equal(cs.cpu().to(F64), cs_ref)


def test_prefill_then_decode_steps_through_the_cache_match_one_long_prefill():
    B, HK, HV, DK, DV, S, steps = 2, 2, 4, 128, 128, 150, 3
    qkv, ab, params = _layer_inputs(B, S + steps, HK, HV, DK, DV, seed=5)
    full, (cs_full, h_full) = _gpu_chain(qkv, ab, params, HK, HV, DK, DV, (None, None), neg=False)
    out, cache = _gpu_chain(qkv[:, :S], ab[:, :S], params, HK, HV, DK, DV, (None, None), neg=False)
    pieces = [out]
    for i in range(steps):
        out, cache = _gpu_chain(qkv[:, S + i : S + i + 1], ab[:, S + i : S + i + 1], params, HK, HV, DK, DV, cache, neg=False)
        pieces.append(out)
    torch.cuda.synchronize()
    stitched = torch.cat(pieces, dim=1)
    print(f"   stitched vs full: max-abs {max_abs(stitched, full):.3e} rel-L2 {rel_l2(stitched, full):.3e}", flush=True)
    assert rel_l2(stitched, full) <= 1e-2
    assert torch.equal(cache[0], cs_full)
    assert rel_l2(cache[1], h_full) <= 1e-2


def test_no_cache_returns_none():
    qkv, ab, params = _layer_inputs(1, 66, 2, 2, 64, 64, seed=6)
    out, cache = _gpu_chain(qkv, ab, params, 2, 2, 64, 64, None, neg=False)
    assert cache is None and out.shape == (1, 66, 128)


@pytest.mark.parametrize("S", [150, 40])
def test_left_padded_batch_with_attention_mask_equals_unpadded_runs(S):
    # rows padded on the left as the reference batches prompts of different lengths for generation
    B, HK, HV, DK, DV = 3, 2, 4, 128, 128
    lengths = [S, S - 33, 5]
    qkv, ab, params = _layer_inputs(B, S, HK, HV, DK, DV, seed=7)
    mask = torch.zeros(B, S)
    for b, n in enumerate(lengths):
        mask[b, S - n :] = 1
    out, (cs, h) = _gpu_chain(qkv, ab, params, HK, HV, DK, DV, (None, None), neg=False, attention_mask=mask.to(BF16))
    torch.cuda.synchronize()
    for b, n in enumerate(lengths):
        assert torch.all(out[b, : S - n] == 0), f"row {b}: padding must come out as zeros"
        o_b, (cs_b, h_b) = _gpu_chain(qkv[b : b + 1, S - n :], ab[b : b + 1, S - n :], params, HK, HV, DK, DV,
                                      (None, None), neg=False)  # fmt: skip
        print(f"   row {b} len {n}: rel-L2 {rel_l2(out[b : b + 1, S - n :], o_b):.3e}", flush=True)
        # same kernels on the same values; the chunk / recurrent choice may differ between the two calls
        assert rel_l2(out[b : b + 1, S - n :], o_b) <= 1e-2
        assert rel_l2(h[b : b + 1], h_b) <= 1e-2
        assert torch.equal(cs[b : b + 1], cs_b)
