"""CPU restatement of the reference's depthwise causal convolution with carried state.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's CPU
baseline leg; the product path never touches it.

Follows ``DepthwiseCausalConvolution.forward``
(lm_engine/modeling_utils/depthwise_causal_convolution.py:103-241), torch branches:

* mask on the way in and out, only when B > 1 and S > 1                         (:28-37, :127, :248)
* fresh prefill: ``nn.Conv1d(padding=ks-1, groups=C)`` cropped on the right      (:175-184)
* one-token update: window = [state | x], y = sum(window * weight) + bias         (:213-231)
* continuation: conv over [state | x], last S outputs                            (:232-246)
* carried state = last ks - 1 positions of what was convolved (left-padded with zeros) (:53-64)

All three modes are one formula: y[s] = act(bias + sum_j w[j] * xx[s + j]) with
xx = [state or zeros | x * mask]; this file states it that way, in the dtype it is given (tests
pass fp64 or fp32).  Pinned in tests/test_conv_oracle.py against ``torch.nn.functional.conv1d``
(the library routine the reference itself calls), a pure-Python triple loop, and the properties
the reference's own tests assert (tests/depthwise_causal_convolution_test.py:115-199).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def depthwise_causal_convolution_ref(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    input_state: torch.Tensor | None = None,
    attention_mask: torch.Tensor | None = None,
    output_state: bool = False,
    activation: str | None = "silu",
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """x [B, S, C], weight [C, ks] (or [C, 1, ks]), input_state [B, C, ks - 1] -> (y [B, S, C], state)."""
    if weight.dim() == 3:
        weight = weight.squeeze(1)
    B, S, C = x.shape
    ks = weight.size(1)
    dt = x.dtype
    use_mask = attention_mask is not None and attention_mask.shape[1] > 1 and attention_mask.shape[0] > 1
    if use_mask:
        x = x * attention_mask[:, :, None].to(dt)
    xt = x.transpose(1, 2)  # [B, C, S]
    head = torch.zeros(B, C, ks - 1, dtype=dt) if input_state is None else input_state.to(dt)
    xx = torch.cat([head, xt], dim=-1)  # [B, C, ks - 1 + S]
    windows = xx.unfold(-1, ks, 1)  # [B, C, S, ks]: window s holds xx[s .. s + ks - 1]
    y = (windows * weight.to(dt)[None, :, None, :]).sum(-1)
    if bias is not None:
        y = y + bias.to(dt)[None, :, None]
    if activation in ("silu", "swish"):
        y = y * torch.sigmoid(y)
    elif activation is not None:
        raise ValueError(f"activation {activation!r} is not part of this restatement")
    y = y.transpose(1, 2)
    if use_mask:
        y = y * attention_mask[:, :, None].to(dt)
    final_state = xx[..., -(ks - 1):].contiguous() if output_state else None
    return y.contiguous(), final_state


def conv1d_library_ref(x, weight, bias=None, activation="silu"):
    """Fresh prefill exactly as the reference's torch branch spells it (:175-190): nn.Conv1d semantics
    with padding ks - 1 and groups = C, cropped on the right."""
    if weight.dim() == 2:
        weight = weight[:, None, :]
    ks = weight.size(-1)
    y = F.conv1d(x.transpose(1, 2), weight.to(x.dtype), None if bias is None else bias.to(x.dtype),
                 padding=ks - 1, groups=x.size(-1))  # fmt: skip
    y = y[..., : 1 - ks]
    if activation in ("silu", "swish"):
        y = F.silu(y)
    return y.transpose(1, 2)
