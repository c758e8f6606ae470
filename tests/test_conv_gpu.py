"""Parity of the depthwise causal convolution kernel (through the C ABI) against the CPU oracle,
in the three modes of the reference module and with the properties its own tests assert
(tests/depthwise_causal_convolution_test.py of the reference).

Gates: fp32 within 1e-5 (the tolerance the reference's tests use); bf16 within max-abs 2e-2 and
relative-L2 1e-2 of the fp64 oracle on the same rounded inputs."""

import pytest
import torch

import lm_engine_amd
from oracle.conv_oracle import depthwise_causal_convolution_ref as conv_ref
from tests.helpers import max_abs, rel_l2


pytestmark = pytest.mark.gpu
BF16, F32, F64 = torch.bfloat16, torch.float32, torch.float64


def _inputs(B, S, C, ks, dtype, seed, bias=True, state=False, mask=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, C, generator=g).to(dtype)
    w = (torch.randn(C, 1, ks, generator=g) * 0.5).to(dtype)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype) if bias else None
    st = torch.randn(B, C, ks - 1, generator=g).to(dtype) if state else None
    m = None
    if mask:
        m = torch.ones(B, S)
        for i in range(B):
            m[i, : (3 * i + 1) % max(S, 1)] = 0  # left padding of different lengths
        m = m.to(dtype)
    return x, w, b, st, m


def _check(x, w, b, st, m, activation, label):
    print(f"case: conv {label} x={tuple(x.shape)} {x.dtype} ks={w.size(-1)} bias={b is not None} "
          f"state={st is not None} mask={m is not None} act={activation}", flush=True)  # fmt: skip
    up = lambda t: None if t is None else t.to(F64)  # noqa: E731
    y_ref, s_ref = conv_ref(up(x), up(w), up(b), up(st), up(m), output_state=True, activation=activation)
    dev = lambda t: None if t is None else t.cuda()  # noqa: E731
    y, s = lm_engine_amd.depthwise_causal_convolution(dev(x), dev(w), dev(b), dev(st), dev(m), output_state=True,
                                                      activation=activation)  # fmt: skip
    torch.cuda.synchronize()
    assert y.dtype == x.dtype and s.dtype == x.dtype and tuple(s.shape) == (x.size(0), x.size(2), w.size(-1) - 1)
    y, s = y.cpu().to(F64), s.cpu().to(F64)
    print(f"   y: max-abs {max_abs(y, y_ref):.3e} rel-L2 {rel_l2(y, y_ref):.3e}   state: max-abs {max_abs(s, s_ref):.3e}", flush=True)
    if x.dtype == F32:
        torch.testing.assert_close(y, y_ref, rtol=1e-5, atol=1e-5)
    else:
        assert max_abs(y, y_ref) <= 2e-2 * max(1.0, float(y_ref.abs().max())) and rel_l2(y, y_ref) <= 1e-2
    assert torch.equal(s, s_ref)  # the state is a copy of (masked) inputs
    return y, s


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("ks", [2, 3, 4])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("activation", [None, "silu"])
def test_fresh_prefill(dtype, ks, bias, activation):
    x, w, b, st, m = _inputs(2, 70, 64, ks, dtype, seed=ks, bias=bias)
    _check(x, w, b, st, m, activation, "prefill")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("S", [1, 2, 3, 4, 33])
def test_continuation_from_a_state(dtype, S):
    x, w, b, st, m = _inputs(3, S, 32, 4, dtype, seed=10 + S, state=True)
    _check(x, w, b, st, m, "silu", f"continuation S={S}")


@pytest.mark.parametrize("S", [1, 2, 4])
def test_zero_state_matches_fresh_prefill(S):
    x, w, b, _, _ = _inputs(2, S, 8, 4, F32, seed=20 + S)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    y0, s0 = lm_engine_amd.depthwise_causal_convolution(xd, wd, bd, None, None, True)
    y1, s1 = lm_engine_amd.depthwise_causal_convolution(xd, wd, bd, torch.zeros(2, 8, 3, device="cuda"), None, True)
    assert torch.equal(y0, y1) and torch.equal(s0, s1)


@pytest.mark.parametrize("continuation_len", [1, 2, 4])
@pytest.mark.parametrize("n_gen_steps", [1, 2])
@pytest.mark.parametrize("prefill_len", [3, 6, 100])
def test_prefill_continuation_and_steps_match_full_sequence(continuation_len, n_gen_steps, prefill_len):
    total = prefill_len + continuation_len + n_gen_steps
    x, w, b, _, _ = _inputs(2, total, 16, 4, F32, seed=30 + total)
    x, w, b = x.cuda(), w.cuda(), b.cuda()
    conv = lm_engine_amd.depthwise_causal_convolution
    y_full, s_full = conv(x, w, b, None, None, True)
    _, st = conv(x[:, :prefill_len], w, b, None, None, True)
    y_c, st = conv(x[:, prefill_len : prefill_len + continuation_len], w, b, st, None, True)
    torch.testing.assert_close(y_c, y_full[:, prefill_len : prefill_len + continuation_len], rtol=1e-5, atol=1e-5)
    for step in range(n_gen_steps):
        at = prefill_len + continuation_len + step
        last = step == n_gen_steps - 1
        y_s, st_next = conv(x[:, at : at + 1], w, b, st, None, not last)
        torch.testing.assert_close(y_s, y_full[:, at : at + 1], rtol=1e-5, atol=1e-5)
        st = st_next if not last else st
    assert st_next is None
    _, st = conv(x[:, :prefill_len], w, b, None, None, True)
    _, st = conv(x[:, prefill_len:], w, b, st, None, True)
    assert torch.equal(st, s_full)


def test_attention_mask():
    x, w, b, st, m = _inputs(3, 40, 32, 4, BF16, seed=40, mask=True)
    y, _ = _check(x, w, b, st, m, None, "mask")
    assert torch.all(y[1, :4] == 0) and torch.all(y[2, :7] == 0)
    # all ones is a no-op
    y0, _ = lm_engine_amd.depthwise_causal_convolution(x.cuda(), w.cuda(), b.cuda(), None, None, False, None)
    y1, _ = lm_engine_amd.depthwise_causal_convolution(x.cuda(), w.cuda(), b.cuda(), None, torch.ones(3, 40, device="cuda", dtype=BF16), False, None)
    assert torch.equal(y0, y1)


def test_strided_input_rows_and_the_layer_shape():
    # the layer convolves the fused q | k | v projection: C = 2 * key_dim + value_dim; here it is a slice of a wider buffer
    B, S, C = 2, 300, 2 * 256 + 512
    x, w, b, _, _ = _inputs(B, S, C + 64, 4, BF16, seed=50)
    xs = x[:, :, 32 : 32 + C]
    ws, bs = w[32 : 32 + C], b[32 : 32 + C]
    up = lambda t: t.to(F64)  # noqa: E731
    y_ref, _ = conv_ref(up(xs), up(ws), up(bs))
    y, _ = lm_engine_amd.depthwise_causal_convolution(x.cuda()[:, :, 32 : 32 + C], ws.cuda(), bs.cuda())
    assert rel_l2(y.cpu().to(F64), y_ref) <= 1e-2


def test_rejected_arguments():
    x = torch.randn(2, 8, 16, device="cuda")
    w = torch.randn(16, 1, 4, device="cuda")
    with pytest.raises(ValueError):
        lm_engine_amd.depthwise_causal_convolution(x, torch.randn(16, 1, 5, device="cuda"))
    with pytest.raises(ValueError):
        lm_engine_amd.depthwise_causal_convolution(x, w, activation="gelu")
    with pytest.raises(ValueError):
        lm_engine_amd.depthwise_causal_convolution(x, w, input_state=torch.zeros(2, 16, 2, device="cuda"))
    with pytest.raises(ValueError):
        lm_engine_amd.depthwise_causal_convolution(torch.randn(2, 8, 18, device="cuda"), torch.randn(18, 1, 4, device="cuda"))
    with pytest.raises(ValueError):
        lm_engine_amd.depthwise_causal_convolution(x.cpu(), w.cpu())
