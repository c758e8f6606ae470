"""Pins the C restatement (oracle/gdn_oracle.c) against the torch oracle and a closed form."""

import pytest
import torch

from oracle import recurrent_gated_delta_rule_ref
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import random_inputs


@pytest.mark.parametrize("l2norm", [False, True])
@pytest.mark.parametrize("gated", [False, True])
def test_c_oracle_matches_torch_oracle(l2norm, gated):
    inp = random_inputs(B=2, T=37, H=3, K=16, V=8, seed=30, gated=gated, normalize=not l2norm)
    o_t, h_t = recurrent_gated_delta_rule_ref(**inp, scale=0.5, output_final_state=True,
                                              use_qk_l2norm_in_kernel=l2norm, state_dtype=torch.float64)  # fmt: skip
    o_c, h_c = recurrent_gated_delta_rule_c(**inp, scale=0.5, output_final_state=True,
                                            use_qk_l2norm_in_kernel=l2norm, f64_state=True)  # fmt: skip
    torch.testing.assert_close(o_c.double(), o_t.double(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(h_c.double(), h_t.double(), rtol=1e-5, atol=1e-6)


def test_c_oracle_varlen_and_defaults():
    lengths = [3, 40, 1, 20]
    inp = random_inputs(B=1, T=sum(lengths), H=2, K=8, V=4, seed=31, N=len(lengths))
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    o_t, h_t = recurrent_gated_delta_rule_ref(**inp, cu_seqlens=cu, output_final_state=True, state_dtype=torch.float64)
    o_c, h_c = recurrent_gated_delta_rule_c(**inp, cu_seqlens=cu, output_final_state=True)
    torch.testing.assert_close(o_c.double(), o_t.double(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(h_c.double(), h_t.double(), rtol=1e-5, atol=1e-6)
    # beta=None, g=None, no initial state, fp32 state
    bare = dict(q=inp["q"], k=inp["k"], v=inp["v"])
    o_t, _ = recurrent_gated_delta_rule_ref(**bare, state_dtype=torch.float64)
    o_c, ht = recurrent_gated_delta_rule_c(**bare, f64_state=False)
    assert ht is None
    torch.testing.assert_close(o_c.double(), o_t.double(), rtol=1e-4, atol=1e-5)


def test_c_oracle_beta_zero_closed_form():
    inp = random_inputs(B=1, T=25, H=2, K=8, V=4, seed=32)
    inp["beta"] = torch.zeros_like(inp["beta"])
    o, ht = recurrent_gated_delta_rule_c(**inp, scale=1.0, output_final_state=True)
    gamma = inp["g"].double().cumsum(dim=1)
    expected = torch.einsum("bhkv,bthk->bthv", inp["initial_state"].double(), inp["q"].double()) * gamma.exp()[..., None]
    torch.testing.assert_close(o.double(), expected, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(ht.double(), inp["initial_state"].double() * gamma[:, -1].exp()[..., None, None],
                               rtol=1e-5, atol=1e-8)  # fmt: skip
