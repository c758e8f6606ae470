"""Parity of the recurrent / decode HIP kernel (through the C ABI) against the CPU oracle."""

import pytest
import torch

import lm_engine_amd
from lm_engine_amd.workloads import get_workload, make_inputs
from oracle import recurrent_gated_delta_rule_ref
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import assert_parity, random_inputs


pytestmark = pytest.mark.gpu


def _to_gpu(inp):
    return {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}


def _check(inp, dtype, **kwargs):
    print(f"case: recurrent dtype={dtype} shapes q={tuple(inp['q'].shape)} v={tuple(inp['v'].shape)} {kwargs}",
          flush=True)  # fmt: skip
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True, **kwargs)
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**_to_gpu(inp), output_final_state=True, **kwargs)
    torch.cuda.synchronize()
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert_parity(o.float(), o_ref, dtype, "o")
    assert_parity(ht, h_ref, dtype, "final_state")
    return o, ht


def test_cfg0_ungated_fp32_matches_torch_oracle():
    # configuration 0 of the benchmark contract: B=1, T=256, H=2, K=V=64, fp32, g == 0, zero state
    inp = make_inputs(get_workload(0))
    assert inp["g"] is None and inp["initial_state"] is None
    o_ref, h_ref = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=torch.float64)
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**_to_gpu(inp), output_final_state=True)
    assert o.shape == (1, 256, 2, 64) and ht.shape == (1, 2, 64, 64)
    assert_parity(o, o_ref, torch.float32, "o")
    assert_parity(ht, h_ref.float(), torch.float32, "final_state")
    # the chunk entry point serves fp32 inputs with the same exact kernel
    o2, h2 = lm_engine_amd.chunk_gated_delta_rule(**_to_gpu(inp), output_final_state=True)
    assert torch.equal(o2, o) and torch.equal(h2, ht)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K, V", [(64, 32), (64, 64), (128, 128), (128, 256), (256, 64), (256, 512)])
def test_head_dims(dtype, K, V):
    inp = random_inputs(B=2, T=9, H=3, K=K, V=V, dtype=dtype, seed=40 + K + V)
    _check(inp, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_l2norm_in_kernel_and_scale(dtype):
    inp = random_inputs(B=2, T=6, H=2, K=128, V=64, dtype=dtype, seed=41, normalize=False, beta_max=2.0)
    _check(inp, dtype, use_qk_l2norm_in_kernel=True, scale=0.3)


def test_ungated_no_beta_no_state():
    inp = random_inputs(B=1, T=12, H=2, K=64, V=64, dtype=torch.bfloat16, seed=42, gated=False, h0=False)
    inp["beta"] = None
    inp["k"] = inp["k"] * 0.5  # beta == 1 with unit keys would make the rule a projection; keep it contractive
    _check(inp, torch.bfloat16)


def test_varlen_packed_sequences():
    lengths = [1, 17, 64, 3, 40]
    inp = random_inputs(B=1, T=sum(lengths), H=2, K=64, V=64, dtype=torch.bfloat16, seed=43, N=len(lengths))
    inp["cu_seqlens"] = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    _check(inp, torch.bfloat16)


def test_varlen_with_empty_sequences():
    lengths = [0, 9, 0, 30, 0]
    inp = random_inputs(B=1, T=sum(lengths), H=2, K=64, V=64, dtype=torch.bfloat16, seed=44, N=len(lengths))
    inp["cu_seqlens"] = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    _check(inp, torch.bfloat16)


def test_left_padded_batch_equals_separate_runs():
    B, T, H = 3, 20, 2
    lengths = [20, 0, 7]
    inp = random_inputs(B=B, T=T, H=H, K=64, V=64, dtype=torch.bfloat16, seed=45)
    gpu = {n: x.cuda() for n, x in inp.items()}
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32).cuda()
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**gpu, cu_seqlens=cu, output_final_state=True, left_padded=True)
    for b, n in enumerate(lengths):
        assert torch.all(o[b, : T - n] == 0)
        if n == 0:
            assert torch.equal(ht[b], gpu["initial_state"][b])
            continue
        one = {name: x[b : b + 1, T - n :] for name, x in gpu.items() if name != "initial_state"}
        o_b, h_b = lm_engine_amd.fused_recurrent_gated_delta_rule(**one, initial_state=gpu["initial_state"][b : b + 1],
                                                                  output_final_state=True)  # fmt: skip
        assert torch.equal(o[b : b + 1, T - n :], o_b) and torch.equal(ht[b : b + 1], h_b)


def test_strided_views_of_a_fused_projection():
    # q, k, v as the reference layer produces them: slices of one [B, T, 2 H K + H V] projection
    B, T, H, K, V = 2, 5, 2, 64, 128
    gen = torch.Generator().manual_seed(44)
    fused = torch.randn(B, T, 2 * H * K + H * V, generator=gen).to(torch.bfloat16)
    q, k, v = fused.split((H * K, H * K, H * V), dim=-1)
    inp = dict(q=q.view(B, T, H, K), k=k.view(B, T, H, K) * 0.1, v=v.view(B, T, H, V),
               g=-torch.rand(B, T, H, generator=gen), beta=torch.rand(B, T, H, generator=gen).to(torch.bfloat16),
               initial_state=None)  # fmt: skip
    fused_gpu = fused.cuda()
    qg, kg, vg = fused_gpu.split((H * K, H * K, H * V), dim=-1)
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True, use_qk_l2norm_in_kernel=True)
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(
        q=qg.view(B, T, H, K), k=kg.view(B, T, H, K) * 0.1, v=vg.view(B, T, H, V), g=inp["g"].cuda(),
        beta=inp["beta"].cuda(), output_final_state=True, use_qk_l2norm_in_kernel=True)  # fmt: skip
    assert not qg.view(B, T, H, K).is_contiguous()
    assert_parity(o.float(), o_ref, torch.bfloat16, "o")
    assert_parity(ht, h_ref, torch.bfloat16, "final_state")


def test_decode_step_in_place_on_config3_shape():
    # configuration 3: 256 sequences x 32 heads, K = V = 128, fp32 state resident and updated in place
    w = get_workload(3)
    inp = make_inputs(w)
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True)
    gpu = _to_gpu(inp)
    state = gpu["initial_state"]
    ptr = state.data_ptr()
    o, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**gpu, output_final_state=True, inplace_state=True)
    assert ht.data_ptr() == ptr and o.shape == (256, 1, 32, 128)
    assert_parity(o.float(), o_ref, torch.bfloat16, "o")
    assert_parity(ht, h_ref, torch.bfloat16, "final_state")
    # a second step continues from the updated state
    o_ref2, h_ref2 = recurrent_gated_delta_rule_c(**dict(inp, initial_state=h_ref), output_final_state=True)
    o2, ht2 = lm_engine_amd.fused_recurrent_gated_delta_rule(**gpu, output_final_state=True, inplace_state=True)
    assert_parity(o2.float(), o_ref2, torch.bfloat16, "o (2nd step)")
    assert_parity(ht2, h_ref2, torch.bfloat16, "final_state (2nd step)")


def test_decode_equals_prefill_continuation():
    # prefill T tokens then decode one == run T + 1 tokens at once (same kernel, state carried)
    inp = random_inputs(B=3, T=21, H=2, K=128, V=128, dtype=torch.bfloat16, seed=45)
    gpu = _to_gpu(inp)
    o_all, h_all = lm_engine_amd.fused_recurrent_gated_delta_rule(**gpu, output_final_state=True)
    head = {n: (x[:, :20] if n != "initial_state" else x) for n, x in gpu.items()}
    tail = {n: (x[:, 20:] if n != "initial_state" else x) for n, x in gpu.items()}
    _, h_head = lm_engine_amd.fused_recurrent_gated_delta_rule(**head, output_final_state=True)
    tail["initial_state"] = h_head
    o_tail, h_tail = lm_engine_amd.fused_recurrent_gated_delta_rule(**tail, output_final_state=True)
    assert torch.equal(o_tail, o_all[:, 20:]) and torch.equal(h_tail, h_all)


def test_output_final_state_false_returns_none_and_runs_are_bitwise_repeatable():
    inp = _to_gpu(random_inputs(B=2, T=8, H=2, K=64, V=64, dtype=torch.bfloat16, seed=46))
    o1, none = lm_engine_amd.fused_recurrent_gated_delta_rule(**inp)
    o2, ht = lm_engine_amd.fused_recurrent_gated_delta_rule(**inp, output_final_state=True)
    assert none is None and ht is not None
    assert torch.equal(o1, o2)


def test_inplace_state_is_refused_when_gradients_are_needed():
    inp = _to_gpu(random_inputs(B=1, T=4, H=1, K=64, V=64, dtype=torch.float32, seed=47))
    inp["v"].requires_grad_(True)
    with pytest.raises(ValueError, match="inplace_state"):
        lm_engine_amd.fused_recurrent_gated_delta_rule(**inp, output_final_state=True, inplace_state=True)