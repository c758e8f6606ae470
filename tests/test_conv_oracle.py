"""Pins the CPU restatement of the depthwise causal convolution (oracle/conv_oracle.py).

Checks chosen so that a plausible mistake fails one of them: flipped tap order (library routine,
brute force), state positions off by one (consistency across prefill / continuation / steps),
padding on the wrong side (zero state == fresh), mask applied on one side only."""

import pytest
import torch

from oracle.conv_oracle import conv1d_library_ref, depthwise_causal_convolution_ref as conv_ref


F64 = torch.float64


def _rand(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=F64)


@pytest.mark.parametrize("ks", [2, 3, 4])
@pytest.mark.parametrize("use_bias", [False, True])
@pytest.mark.parametrize("activation", [None, "silu"])
def test_fresh_prefill_equals_library_conv1d(ks, use_bias, activation):
    x, w = _rand(2, 9, 8, seed=1), _rand(8, ks, seed=2)
    b = _rand(8, seed=3) if use_bias else None
    y, _ = conv_ref(x, w, b, activation=activation)
    torch.testing.assert_close(y, conv1d_library_ref(x, w, b, activation), rtol=1e-12, atol=1e-12)


def test_brute_force_triple_loop():
    B, S, C, ks = 2, 5, 3, 4
    x, w, b, st = _rand(B, S, C, seed=4), _rand(C, ks, seed=5), _rand(C, seed=6), _rand(B, C, ks - 1, seed=7)
    y, fs = conv_ref(x, w, b, input_state=st, output_state=True, activation=None)
    for bi in range(B):
        for c in range(C):
            seq = [float(v) for v in st[bi, c]] + [float(v) for v in x[bi, :, c]]
            for s in range(S):
                want = float(b[c]) + sum(float(w[c, j]) * seq[s + j] for j in range(ks))
                assert abs(float(y[bi, s, c]) - want) < 1e-12
            assert [float(v) for v in fs[bi, c]] == seq[-(ks - 1):]


def test_single_tap_kernels_pick_the_right_position():
    # weight = unit vector at tap j delays the input by ks - 1 - j positions
    x = _rand(1, 7, 2, seed=8)
    for j in range(4):
        w = torch.zeros(2, 4, dtype=F64)
        w[:, j] = 1.0
        y, _ = conv_ref(x, w, activation=None)
        d = 3 - j
        assert torch.equal(y[:, d:], x[:, : 7 - d]) and torch.all(y[:, :d] == 0)


@pytest.mark.parametrize("seq_len", [1, 2, 4])
def test_zero_state_matches_fresh_prefill(seq_len):
    x, w, b = _rand(2, seq_len, 8, seed=9), _rand(8, 4, seed=10), _rand(8, seed=11)
    y0, s0 = conv_ref(x, w, b, output_state=True)
    y1, s1 = conv_ref(x, w, b, input_state=torch.zeros(2, 8, 3, dtype=F64), output_state=True)
    assert torch.equal(y0, y1) and torch.equal(s0, s1)


@pytest.mark.parametrize("continuation_len", [1, 2, 4])
@pytest.mark.parametrize("n_gen_steps", [1, 2])
@pytest.mark.parametrize("prefill_len", [3, 6])
def test_prefill_continuation_and_steps_match_full_sequence(continuation_len, n_gen_steps, prefill_len):
    total = prefill_len + continuation_len + n_gen_steps
    x, w, b = _rand(2, total, 8, seed=12), _rand(8, 4, seed=13), _rand(8, seed=14)
    y_full, s_full = conv_ref(x, w, b, output_state=True)
    _, st = conv_ref(x[:, :prefill_len], w, b, output_state=True)
    y_c, st = conv_ref(x[:, prefill_len : prefill_len + continuation_len], w, b, input_state=st, output_state=True)
    torch.testing.assert_close(y_c, y_full[:, prefill_len : prefill_len + continuation_len], rtol=1e-12, atol=1e-12)
    for step in range(n_gen_steps):
        at = prefill_len + continuation_len + step
        y_s, st = conv_ref(x[:, at : at + 1], w, b, input_state=st, output_state=True)
        torch.testing.assert_close(y_s, y_full[:, at : at + 1], rtol=1e-12, atol=1e-12)
    assert torch.equal(st, s_full)


def test_short_prefill_state_is_left_padded():
    x, w = _rand(2, 2, 4, seed=15), _rand(4, 4, seed=16)
    _, st = conv_ref(x, w, output_state=True)
    assert torch.all(st[..., 0] == 0) and torch.equal(st[..., 1:], x.transpose(1, 2))


def test_attention_mask():
    x, w = _rand(2, 6, 8, seed=17), _rand(8, 4, seed=18)
    ones = torch.ones(2, 6, dtype=F64)
    y_plain, _ = conv_ref(x, w, activation=None)
    y_ones, _ = conv_ref(x, w, attention_mask=ones, activation=None)
    assert torch.equal(y_plain, y_ones)
    mask = ones.clone()
    mask[1, :3] = 0
    y_m, _ = conv_ref(x, w, attention_mask=mask, activation=None)
    assert torch.all(y_m[1, :3] == 0)
    # masked inputs do not leak into later positions: same as zeroing them by hand
    xz = x.clone()
    xz[1, :3] = 0
    y_z, _ = conv_ref(xz, w, activation=None)
    assert torch.equal(y_m[1, 3:], y_z[1, 3:]) and torch.equal(y_m[0], y_plain[0])
    # a single sequence or a single token ignores the mask, as the reference does
    y_1, _ = conv_ref(x[:1], w, attention_mask=mask[1:], activation=None)
    assert torch.equal(y_1, y_plain[:1])
