"""The batched chunk-by-chunk backward (lm_engine_amd.backward) on CPU tensors against autograd through
the fp64 token loop of the oracle: fixed-length, packed and left-padded batches, optional inputs."""

import pytest
import torch

from lm_engine_amd.backward import gated_delta_rule_backward
from oracle.gdn_backward_oracle import gated_delta_rule_grads_autograd


NAMES = ("dq", "dk", "dv", "dg", "dbeta", "dh0")


def _inputs(seed, B, T, H, K, V, N=None, l2norm=True):
    gen = torch.Generator().manual_seed(seed)
    dt = torch.float64
    q = torch.randn(B, T, H, K, generator=gen, dtype=dt)
    k = torch.randn(B, T, H, K, generator=gen, dtype=dt) * (1.0 if l2norm else 0.3)
    v = torch.randn(B, T, H, V, generator=gen, dtype=dt)
    g = torch.nn.functional.logsigmoid(torch.randn(B, T, H, generator=gen, dtype=dt) + 2.0)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen, dtype=dt))
    N = B if N is None else N
    h0 = torch.randn(N, H, K, V, generator=gen, dtype=dt) * 0.1
    do = torch.randn(B, T, H, V, generator=gen, dtype=dt)
    dht = torch.randn(N, H, K, V, generator=gen, dtype=dt)
    return q, k, v, g, beta, h0, do, dht


def _f32(x):
    return None if x is None else x.float()


def _check(got, want, tol=2e-5):
    for name, a, b in zip(NAMES, got, want):
        if b is None:
            assert a is None, name
            continue
        err = float((a.double() - b).norm() / b.norm().clamp_min(1e-3))
        assert err <= tol, (name, err)


@pytest.mark.parametrize("l2norm", [False, True])
@pytest.mark.parametrize("with_state", [False, True])
@pytest.mark.parametrize("T", [1, 64, 65, 200])
def test_fixed_length(T, with_state, l2norm):
    q, k, v, g, beta, h0, do, dht = _inputs(T, 2, T, 2, 16, 32, l2norm=l2norm)
    h0 = h0 if with_state else None
    kw = dict(initial_state=h0, use_qk_l2norm_in_kernel=l2norm)
    want = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, dht, **kw)
    got = gated_delta_rule_backward(*map(_f32, (q, k, v, g, beta, do, dht)), initial_state=_f32(h0),
                                    use_qk_l2norm_in_kernel=l2norm)  # fmt: skip
    _check(got, want)


def test_packed_sequences_and_scale():
    cu = torch.tensor([0, 3, 70, 71, 200], dtype=torch.int32)
    q, k, v, g, beta, h0, do, dht = _inputs(3, 1, 200, 2, 16, 32, N=4)
    kw = dict(initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=True, scale=0.3)
    want = gated_delta_rule_grads_autograd(q, k, v, g, beta, do, dht, **kw)
    got = gated_delta_rule_backward(*map(_f32, (q, k, v, g, beta, do, dht)), initial_state=_f32(h0), cu_seqlens=cu,
                                    use_qk_l2norm_in_kernel=True, scale=0.3)  # fmt: skip
    _check(got, want)


def test_left_padded_batch_equals_separate_sequences():
    B, T, H, K, V = 3, 100, 2, 16, 32
    lens = [100, 37, 1]
    q, k, v, g, beta, h0, do, dht = map(_f32, _inputs(4, B, T, H, K, V))
    cu = torch.tensor([0, 100, 137, 138], dtype=torch.int32)
    got = gated_delta_rule_backward(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu,
                                    use_qk_l2norm_in_kernel=True, left_padded=True)  # fmt: skip
    for b, n in enumerate(lens):
        sl = lambda x: x[b : b + 1, T - n :]
        one = gated_delta_rule_backward(sl(q), sl(k), sl(v), sl(g), sl(beta), sl(do), dht[b : b + 1],
                                        initial_state=h0[b : b + 1], use_qk_l2norm_in_kernel=True)  # fmt: skip
        for name, a, w in zip(NAMES[:5], got[:5], one[:5]):
            assert torch.allclose(a[b : b + 1, T - n :], w, rtol=1e-5, atol=1e-6), name
            assert not a[b, : T - n].any(), f"{name}: gradient at the padding"
        assert torch.allclose(got[5][b : b + 1], one[5], rtol=1e-5, atol=1e-6)


def test_ungated_without_beta_and_without_final_state_gradient():
    q, k, v, g, beta, h0, do, dht = _inputs(5, 2, 90, 2, 16, 32)
    one = torch.ones_like(beta)
    zero = torch.zeros_like(g)
    want = gated_delta_rule_grads_autograd(q, k, v, zero, one, do, None, use_qk_l2norm_in_kernel=True)
    got = gated_delta_rule_backward(_f32(q), _f32(k), _f32(v), None, None, _f32(do), None,
                                    use_qk_l2norm_in_kernel=True)  # fmt: skip
    assert got[3] is None and got[4] is None and got[5] is None
    _check(got[:3], want[:3])


def test_gradients_come_back_in_the_input_dtypes():
    q, k, v, g, beta, h0, do, dht = _inputs(6, 1, 70, 2, 16, 32)
    bf = lambda x: x.to(torch.bfloat16)
    got = gated_delta_rule_backward(bf(q), bf(k), bf(v), g.float(), bf(beta), bf(do), dht.float(),
                                    initial_state=h0.float(), use_qk_l2norm_in_kernel=True)  # fmt: skip
    assert [x.dtype for x in got] == [torch.bfloat16] * 3 + [torch.float32, torch.bfloat16, torch.float32]


def test_host_copy_of_cu_seqlens_is_made_once_per_tensor_and_version():
    from lm_engine_amd import backward

    cu = torch.tensor([0, 70, 130], dtype=torch.int32)
    first = backward._host_prefix(cu)
    assert first == [0, 70, 130] and backward._host_prefix(cu) is first  # the second call reuses the list
    cu[1] = 64  # an in-place write makes the copy stale
    assert backward._host_prefix(cu) == [0, 64, 130]
    other = torch.tensor([0, 70, 130], dtype=torch.int32)
    assert backward._host_prefix(other) is not first
    key = id(cu)
    del cu
    assert key not in backward._HOST_PREFIX  # the entry goes with its tensor
