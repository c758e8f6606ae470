"""Pins the CPU oracle (oracle/gdn_oracle.py) against what the mathematics fixes.

The reference holds no golden vector for the gated delta rule (its arithmetic lives in the
un-vendored `fla` package), so each oracle function is checked against something that does not
share its code: a scalar brute force, closed forms of special cases, library routines and
invariants of the recurrence.  A dropped term, a wrong sign, a transposed operand or a state
used before/after its update fails at least one of these.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import (
    chunk_gated_delta_rule_ref,
    decode_step_single_pass_ref,
    l2norm_ref,
    recurrent_gated_delta_rule_ref,
)
from tests.helpers import random_inputs


F64 = torch.float64


def _as64(inp):
    return {k: (x.to(F64) if isinstance(x, torch.Tensor) and x.is_floating_point() else x) for k, x in inp.items()}


def _brute_force(q, k, v, g, beta, h0, scale):
    """Scalar loops over every index, no tensor arithmetic: S[a][c] of one (batch, head)."""
    B, T, H, K = q.shape
    V = v.shape[-1]
    o = torch.zeros(B, T, H, V, dtype=F64)
    ht = torch.zeros(B, H, K, V, dtype=F64)
    for b in range(B):
        for h in range(H):
            S = [[float(h0[b, h, a, c]) for c in range(V)] for a in range(K)]
            for t in range(T):
                decay = math.exp(float(g[b, t, h]))
                kt = [float(k[b, t, h, a]) for a in range(K)]
                qt = [float(q[b, t, h, a]) * scale for a in range(K)]
                for a in range(K):
                    for c in range(V):
                        S[a][c] *= decay
                r = []
                for c in range(V):
                    pred = sum(S[a][c] * kt[a] for a in range(K))
                    r.append(float(beta[b, t, h]) * (float(v[b, t, h, c]) - pred))
                for a in range(K):
                    for c in range(V):
                        S[a][c] += kt[a] * r[c]
                for c in range(V):
                    o[b, t, h, c] = sum(S[a][c] * qt[a] for a in range(K))
            ht[b, h] = torch.tensor(S, dtype=F64)
    return o, ht


def test_recurrent_matches_scalar_brute_force():
    inp = _as64(random_inputs(B=2, T=7, H=2, K=3, V=2, seed=1))
    o, ht = recurrent_gated_delta_rule_ref(**inp, scale=0.7, output_final_state=True, state_dtype=F64)
    o_bf, ht_bf = _brute_force(inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"], inp["initial_state"], 0.7)
    torch.testing.assert_close(o, o_bf, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(ht, ht_bf, rtol=1e-12, atol=1e-12)


def test_beta_zero_is_pure_decay():
    # beta == 0: S_t = e^{gamma_t} S_0 and o_t = e^{gamma_t} S_0^T q_t (one matmul)
    inp = _as64(random_inputs(B=1, T=20, H=2, K=8, V=4, seed=2))
    inp["beta"] = torch.zeros_like(inp["beta"])
    o, ht = recurrent_gated_delta_rule_ref(**inp, scale=1.0, output_final_state=True, state_dtype=F64)
    gamma = inp["g"].cumsum(dim=1)  # [B, T, H]
    expected = torch.einsum("bhkv,bthk->bthv", inp["initial_state"], inp["q"]) * gamma.exp()[..., None]
    torch.testing.assert_close(o, expected, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(ht, inp["initial_state"] * gamma[:, -1].exp()[..., None, None], rtol=1e-12, atol=1e-12)


def test_no_gate_no_beta_keeps_state():
    inp = _as64(random_inputs(B=1, T=9, H=1, K=4, V=4, seed=3, gated=False))
    inp["beta"] = torch.zeros_like(inp["beta"])
    _, ht = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(ht, inp["initial_state"], rtol=0, atol=0)


def test_orthonormal_keys_store_and_retrieve():
    # g == 0, beta == 1, orthonormal keys, zero initial state: S = sum_i k_i v_i^T and querying
    # with k_j returns scale * v_j exactly.
    K, V = 8, 5
    gen = torch.Generator().manual_seed(4)
    Q, _ = torch.linalg.qr(torch.randn(K, K, dtype=F64, generator=gen))
    keys = Q.T[None, :, None, :]  # [1, T=K, 1, K]
    vals = torch.randn(1, K, 1, V, dtype=F64, generator=gen)
    _, ht = recurrent_gated_delta_rule_ref(q=keys, k=keys, v=vals, output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(ht[0, 0], torch.einsum("tk,tv->kv", keys[0, :, 0], vals[0, :, 0]), rtol=1e-12, atol=1e-12)
    # a second pass that only reads (beta = 0) retrieves every stored value
    o, _ = recurrent_gated_delta_rule_ref(q=keys, k=keys, v=vals, beta=torch.zeros(1, K, 1, dtype=F64),
                                          initial_state=ht, scale=0.5, state_dtype=F64)  # fmt: skip
    torch.testing.assert_close(o, 0.5 * vals, rtol=1e-12, atol=1e-12)


def test_repeated_key_overwrites_value():
    # beta == 1 with a unit key: writing (k, v1) then (k, v2) leaves S^T k == v2
    K, V = 6, 3
    gen = torch.Generator().manual_seed(5)
    key = F.normalize(torch.randn(K, dtype=F64, generator=gen), dim=0)
    k = key.expand(1, 2, 1, K)
    v = torch.randn(1, 2, 1, V, dtype=F64, generator=gen)
    h0 = torch.randn(1, 1, K, V, dtype=F64, generator=gen)
    o, ht = recurrent_gated_delta_rule_ref(q=k, k=k, v=v, initial_state=h0, scale=1.0, output_final_state=True,
                                           state_dtype=F64)  # fmt: skip
    torch.testing.assert_close(ht[0, 0].T @ key, v[0, 1, 0], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(o[0, :, 0], v[0, :, 0], rtol=1e-12, atol=1e-12)  # reading right after writing


def test_single_token_closed_form():
    inp = _as64(random_inputs(B=3, T=1, H=2, K=5, V=4, seed=6))
    o, ht = recurrent_gated_delta_rule_ref(**inp, scale=0.3, output_final_state=True, state_dtype=F64)
    q, k, v = inp["q"][:, 0], inp["k"][:, 0], inp["v"][:, 0]
    eg = inp["g"][:, 0].exp()[..., None, None]
    b = inp["beta"][:, 0][..., None]
    S0 = inp["initial_state"]
    S = eg * S0
    r = b * (v - torch.einsum("bhkv,bhk->bhv", S, k))
    S1 = S + torch.einsum("bhk,bhv->bhkv", k, r)
    torch.testing.assert_close(ht, S1, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(o[:, 0], 0.3 * torch.einsum("bhkv,bhk->bhv", S1, q), rtol=1e-12, atol=1e-12)


def test_scalar_recurrence_by_hand():
    # K = V = 1: s <- e^g s (1 - beta k^2) + beta k v ;  o = scale q s
    T = 6
    gen = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(T, dtype=F64, generator=gen) for _ in range(3))
    beta = torch.rand(T, dtype=F64, generator=gen)
    g = -torch.rand(T, dtype=F64, generator=gen)
    s, outs = 0.25, []
    for t in range(T):
        s = math.exp(g[t]) * s * (1 - beta[t] * k[t] ** 2) + beta[t] * k[t] * v[t]
        outs.append(2.0 * q[t] * s)
    shape = (1, T, 1, 1)
    o, ht = recurrent_gated_delta_rule_ref(
        q=q.view(shape), k=k.view(shape), v=v.view(shape), g=g.view(1, T, 1), beta=beta.view(1, T, 1),
        initial_state=torch.full((1, 1, 1, 1), 0.25, dtype=F64), scale=2.0, output_final_state=True, state_dtype=F64,
    )  # fmt: skip
    torch.testing.assert_close(o.flatten(), torch.stack(outs), rtol=1e-12, atol=1e-12)
    assert abs(ht.item() - float(s)) < 1e-12


@pytest.mark.parametrize("chunk_size", [16, 32, 64])
@pytest.mark.parametrize("T", [1, 63, 64, 65, 130])
def test_chunk_equals_recurrent_and_is_chunk_size_invariant(chunk_size, T):
    inp = _as64(random_inputs(B=2, T=T, H=2, K=16, V=8, seed=8, beta_max=2.0))
    o_r, h_r = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    o_c, h_c = chunk_gated_delta_rule_ref(**inp, output_final_state=True, chunk_size=chunk_size, state_dtype=F64)
    torch.testing.assert_close(o_c, o_r, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(h_c, h_r, rtol=1e-9, atol=1e-10)


def test_chunk_equals_recurrent_strong_decay_unnormalised_keys():
    # large |g| (decay factors down to e^-300 inside a chunk) and keys of norm ~ sqrt(K)
    inp = _as64(random_inputs(B=1, T=96, H=2, K=8, V=4, seed=9, g_mean=-5.0, normalize=False))
    inp["k"] = inp["k"] * 0.5
    o_r, h_r = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    o_c, h_c = chunk_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    assert torch.isfinite(o_c).all()
    torch.testing.assert_close(o_c, o_r, rtol=1e-8, atol=1e-9)
    torch.testing.assert_close(h_c, h_r, rtol=1e-8, atol=1e-9)


def test_split_sequence_with_carried_state():
    inp = _as64(random_inputs(B=2, T=50, H=2, K=8, V=4, seed=10))
    o, ht = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    cut = 23
    first = {n: (x[:, :cut] if n != "initial_state" else x) for n, x in inp.items()}
    o1, h1 = recurrent_gated_delta_rule_ref(**first, output_final_state=True, state_dtype=F64)
    second = {n: (x[:, cut:] if n != "initial_state" else h1) for n, x in inp.items()}
    o2, h2 = recurrent_gated_delta_rule_ref(**second, output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(torch.cat([o1, o2], dim=1), o, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(h2, ht, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("fn", [recurrent_gated_delta_rule_ref, chunk_gated_delta_rule_ref])
def test_varlen_equals_separate_sequences(fn):
    lengths = [5, 70, 1, 64]
    total, N = sum(lengths), len(lengths)
    inp = _as64(random_inputs(B=1, T=total, H=2, K=8, V=4, seed=11, N=N))
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    o, ht = fn(**inp, cu_seqlens=cu, output_final_state=True, state_dtype=F64)
    for n in range(N):
        s, e = int(cu[n]), int(cu[n + 1])
        one = {name: x[:, s:e] for name, x in inp.items() if name != "initial_state"}
        o_n, h_n = fn(**one, initial_state=inp["initial_state"][n : n + 1], output_final_state=True, state_dtype=F64)
        torch.testing.assert_close(o[:, s:e], o_n, rtol=1e-10, atol=1e-11)
        torch.testing.assert_close(ht[n : n + 1], h_n, rtol=1e-10, atol=1e-11)


def test_batch_and_head_permutation_equivariance():
    inp = _as64(random_inputs(B=3, T=12, H=4, K=8, V=4, seed=12))
    o, ht = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    pb, ph = torch.tensor([2, 0, 1]), torch.tensor([3, 1, 0, 2])
    perm = {}
    for name, x in inp.items():
        x = x[pb]
        perm[name] = x[:, ph] if name == "initial_state" else x[:, :, ph]
    o_p, h_p = recurrent_gated_delta_rule_ref(**perm, output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(o_p, o[pb][:, :, ph], rtol=0, atol=0)
    torch.testing.assert_close(h_p, ht[pb][:, ph], rtol=0, atol=0)


def test_value_columns_are_independent():
    inp = _as64(random_inputs(B=1, T=17, H=2, K=8, V=6, seed=13))
    o, ht = recurrent_gated_delta_rule_ref(**inp, output_final_state=True, state_dtype=F64)
    cols = [4, 1]
    sub = dict(inp, v=inp["v"][..., cols], initial_state=inp["initial_state"][..., cols])
    o_s, h_s = recurrent_gated_delta_rule_ref(**sub, output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(o_s, o[..., cols], rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(h_s, ht[..., cols], rtol=1e-13, atol=1e-13)


def test_jointly_linear_in_values_and_initial_state():
    a = _as64(random_inputs(B=1, T=15, H=2, K=8, V=4, seed=14))
    b = _as64(random_inputs(B=1, T=15, H=2, K=8, V=4, seed=15))
    shared = {n: a[n] for n in ("q", "k", "g", "beta")}
    run = lambda v, h0: recurrent_gated_delta_rule_ref(**shared, v=v, initial_state=h0, output_final_state=True,
                                                       state_dtype=F64)  # noqa: E731  # fmt: skip
    oa, ha = run(a["v"], a["initial_state"])
    ob, hb = run(b["v"], b["initial_state"])
    oc, hc = run(2.0 * a["v"] - 3.0 * b["v"], 2.0 * a["initial_state"] - 3.0 * b["initial_state"])
    torch.testing.assert_close(oc, 2.0 * oa - 3.0 * ob, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(hc, 2.0 * ha - 3.0 * hb, rtol=1e-11, atol=1e-12)


def test_l2norm_flag_equals_prenormalised_inputs():
    inp = _as64(random_inputs(B=1, T=10, H=2, K=16, V=4, seed=16, normalize=False))
    o1, h1 = recurrent_gated_delta_rule_ref(**inp, use_qk_l2norm_in_kernel=True, output_final_state=True,
                                            state_dtype=F64)  # fmt: skip
    pre = dict(inp, q=l2norm_ref(inp["q"]), k=l2norm_ref(inp["k"]))
    o2, h2 = recurrent_gated_delta_rule_ref(**pre, use_qk_l2norm_in_kernel=False, output_final_state=True,
                                            state_dtype=F64)  # fmt: skip
    torch.testing.assert_close(o1, o2, rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(h1, h2, rtol=1e-13, atol=1e-13)
    o3, _ = chunk_gated_delta_rule_ref(**inp, use_qk_l2norm_in_kernel=True, state_dtype=F64)
    torch.testing.assert_close(o3, o1, rtol=1e-9, atol=1e-10)


def test_l2norm_against_library_normalize():
    x = torch.randn(4, 7, 32, dtype=F64, generator=torch.Generator().manual_seed(17))
    # for rows of ordinary magnitude the eps inside the sqrt is far below rounding
    torch.testing.assert_close(l2norm_ref(x), F.normalize(x, dim=-1), rtol=1e-6, atol=1e-7)
    assert torch.equal(l2norm_ref(torch.zeros(3, 8)), torch.zeros(3, 8))  # eps keeps zero rows finite


def test_default_scale_is_rsqrt_head_dim():
    inp = _as64(random_inputs(B=1, T=5, H=1, K=16, V=4, seed=18))
    o_default, _ = recurrent_gated_delta_rule_ref(**inp, state_dtype=F64)
    o_explicit, _ = recurrent_gated_delta_rule_ref(**inp, scale=16**-0.5, state_dtype=F64)
    o_unit, _ = recurrent_gated_delta_rule_ref(**inp, scale=1.0, state_dtype=F64)
    torch.testing.assert_close(o_default, o_explicit, rtol=0, atol=0)
    torch.testing.assert_close(o_default, 0.25 * o_unit, rtol=1e-13, atol=1e-14)


def test_missing_gate_and_beta_mean_zero_and_one():
    inp = _as64(random_inputs(B=1, T=8, H=2, K=8, V=4, seed=19))
    ones, zeros = torch.ones_like(inp["beta"]), torch.zeros_like(inp["g"])
    o1, h1 = recurrent_gated_delta_rule_ref(**dict(inp, g=None, beta=None), output_final_state=True, state_dtype=F64)
    o2, h2 = recurrent_gated_delta_rule_ref(**dict(inp, g=zeros, beta=ones), output_final_state=True, state_dtype=F64)
    torch.testing.assert_close(o1, o2, rtol=0, atol=0)
    torch.testing.assert_close(h1, h2, rtol=0, atol=0)


def test_decode_single_pass_identity():
    inp = _as64(random_inputs(B=5, T=1, H=3, K=8, V=4, seed=20))
    o, ht = recurrent_gated_delta_rule_ref(**inp, scale=0.4, output_final_state=True, state_dtype=F64)
    o_sp, h_sp = decode_step_single_pass_ref(inp["q"][:, 0], inp["k"][:, 0], inp["v"][:, 0], inp["g"][:, 0],
                                             inp["beta"][:, 0], inp["initial_state"], scale=0.4)  # fmt: skip
    torch.testing.assert_close(o_sp, o[:, 0], rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(h_sp, ht, rtol=1e-12, atol=1e-13)


def test_output_dtype_and_final_state_flag():
    inp = random_inputs(B=1, T=4, H=1, K=8, V=4, seed=21, dtype=torch.bfloat16)
    o, ht = recurrent_gated_delta_rule_ref(**inp)
    assert o.dtype == torch.bfloat16 and ht is None
    o, ht = chunk_gated_delta_rule_ref(**inp, output_final_state=True)
    assert o.dtype == torch.bfloat16 and ht.dtype == torch.float32 and ht.shape == (1, 1, 8, 4)
