"""Depthwise causal convolution with its carried state, the step in front of the gated delta rule.

Functional form of the reference's ``DepthwiseCausalConvolution.forward``
(lm_engine/modeling_utils/depthwise_causal_convolution.py:103-241): same arguments, same three
modes (fresh prefill, one-token update, multi-token continuation), same return ``(y, final_state)``.
It runs one HIP kernel (``gdn_causal_conv1d_fwd`` of libgdn_hip.so); there is no torch fallback.
Under autograd the backward is one more HIP kernel (``gdn_causal_conv1d_bwd``, bf16 and fp32 x); shapes it does not
take (an odd number of channels) differentiate the same formula written in torch
(``_autograd.py``).

    x             [B, S, C]          bf16 or fp32, channels contiguous
    weight        [C, 1, ks] or [C, ks]   nn.Conv1d's depthwise weight, ks in 2..4
    bias          [C] or None
    input_state   [B, C, ks - 1] or None   the last ks - 1 inputs of the previous call
    attention_mask [B, S] or None    0/1 padding mask; applied to x and to y as the reference does
                                     (only when B > 1 and S > 1, depthwise_causal_convolution.py:28-37)
    returns  y [B, S, C], final_state [B, C, ks - 1] (None unless output_state)
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._autograd import kernel_with_formula_backward
from .kernels import Kernel, is_kernel_allowed


_IN_KERNEL_ACTIVATIONS = {None: _lib.GDN_ACT_NONE, "silu": _lib.GDN_ACT_SILU, "swish": _lib.GDN_ACT_SILU}


def _dtype_code(dtype: torch.dtype, what: str) -> int:
    if dtype == torch.bfloat16:
        return _lib.GDN_BF16
    if dtype == torch.float32:
        return _lib.GDN_F32
    raise ValueError(f"{what} must be bfloat16 or float32, got {dtype}")


def convolution_formula(x, weight, bias, input_state, attention_mask, output_state, activation):
    """The convolution in torch operations (fp32 arithmetic): what the backward differentiates when the backward
    kernel does not apply."""
    # y[s] = act(bias + sum_j w[j] xx[s + j]) over xx = [state or zeros | x * mask], y masked again
    w = (weight.squeeze(1) if weight.dim() == 3 else weight).float()
    B, S, C = x.shape
    ks = w.size(1)
    use_mask = attention_mask is not None and attention_mask.shape[1] > 1 and attention_mask.shape[0] > 1
    xm = x.float() * attention_mask[:, :, None].float() if use_mask else x.float()
    head = torch.zeros(B, C, ks - 1, device=x.device) if input_state is None else input_state.float()
    xx = torch.cat([head, xm.transpose(1, 2)], dim=-1)
    y = torch.nn.functional.conv1d(xx, w[:, None, :], None if bias is None else bias.float(), groups=C)
    if activation is not None:
        y = torch.nn.functional.silu(y)
    y = y.transpose(1, 2)
    if use_mask:
        y = y * attention_mask[:, :, None].float()
    return y.to(x.dtype), (xx[..., -(ks - 1):].to(x.dtype) if output_state else None)


def depthwise_causal_convolution(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None = None,
    input_state: torch.Tensor | None = None,
    attention_mask: torch.Tensor | None = None,
    output_state: bool = False,
    activation: str | None = "silu",
) -> tuple[torch.Tensor, torch.Tensor | None]:
    if torch.compiler.is_compiling():  # a graph is being captured: the kernel goes in as an opaque operator
        from . import _opaque

        return _opaque.depthwise_causal_convolution(x, weight, bias, input_state, attention_mask, output_state, activation)

    def formula(x, weight, bias, input_state):
        return convolution_formula(x, weight, bias, input_state, attention_mask, output_state, activation)

    kernel = lambda x, weight, bias, input_state: _depthwise_causal_convolution(  # noqa: E731
        x, weight, bias, input_state, attention_mask, output_state, activation)  # fmt: skip
    needs_grad = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, weight, bias, input_state))
    if needs_grad and _backward_kernel_applies(x, weight, activation):
        return _ConvolutionOnKernels.apply(x, weight, bias, input_state, attention_mask, output_state, activation)
    return kernel_with_formula_backward(kernel, formula, x, weight, bias, input_state)


_BWD_TOKENS_PER_BLOCK = 256  # tokens a thread of the backward kernel walks over (64: 0.196 ms, 128: 0.171, 256: 0.163 at 4 x 4096 x 6144)


def _backward_kernel_applies(x, weight, activation) -> bool:
    if not x.is_cuda or x.dtype not in (torch.bfloat16, torch.float32) or activation not in _IN_KERNEL_ACTIVATIONS or x.dim() != 3:
        return False
    B, S, C = x.shape
    return C % 2 == 0 and weight.dtype in (torch.bfloat16, torch.float32) and B * (-(-S // _BWD_TOKENS_PER_BLOCK)) <= 65535


class _ConvolutionOnKernels(torch.autograd.Function):
    """Forward and backward on the HIP kernels (bf16 or fp32 x).  The gradient that flows into the returned state is
    not propagated: the layer's cache is not differentiated through."""

    @staticmethod
    def forward(ctx, x, weight, bias, input_state, attention_mask, output_state, activation):
        y, final_state = _depthwise_causal_convolution(x, weight, bias, input_state, attention_mask, output_state,
                                                       activation)  # fmt: skip
        ctx.save_for_backward(x, weight, bias, input_state, attention_mask)
        ctx.activation = activation
        ctx.set_materialize_grads(False)
        return y, final_state

    @staticmethod
    def backward(ctx, dy, dstate_out):
        x, weight, bias, input_state, attention_mask = ctx.saved_tensors
        if dy is None:
            dy = torch.zeros_like(x)
        dx, dweight, dbias, dstate = _convolution_backward(x, weight, bias, input_state, attention_mask, dy,
                                                           ctx.activation)  # fmt: skip
        if dstate_out is not None:
            # The returned state is the last ks - 1 rows of [input_state or zeros | x * mask]: its gradient goes to those
            # rows (a few row-sized additions; the layer itself does not differentiate through its cache).
            B, S, C = x.shape
            ks1 = dstate_out.size(-1)
            mask = attention_mask if attention_mask is not None and attention_mask.shape[1] > 1 and attention_mask.shape[0] > 1 else None
            for i in range(ks1):
                t = S + i - ks1
                if t >= 0:
                    row = dstate_out[:, :, i].to(dx.dtype)
                    dx[:, t, :] += row if mask is None else row * mask[:, t, None].to(dx.dtype)
                elif dstate is not None:
                    dstate[:, :, S + i] += dstate_out[:, :, i].to(dstate.dtype)
        return dx, dweight, dbias, dstate, None, None, None


def _convolution_backward(x, weight, bias, input_state, attention_mask, dy, activation):
    """``gdn_causal_conv1d_bwd``: dx, dweight, dbias, dinput_state for bf16 or fp32 x (see include/gdn_hip.h)."""
    lib = _lib.load_library()
    B, S, C = x.shape
    w2 = (weight.squeeze(1) if weight.dim() == 3 else weight).contiguous()
    ks = w2.size(1)
    if x.stride(-1) != 1:
        x = x.contiguous()
    dy = dy.to(x.dtype)
    if dy.stride(-1) != 1:
        dy = dy.contiguous()
    b2 = None if bias is None else bias.to(w2.dtype).contiguous()
    state = None if input_state is None else input_state.to(x.dtype).contiguous()
    mask = None
    if attention_mask is not None and attention_mask.shape[1] > 1 and attention_mask.shape[0] > 1:
        mask = attention_mask.to(x.dtype).contiguous()
    blocks = B * (-(-S // _BWD_TOKENS_PER_BLOCK))
    dx = torch.empty(B, S, C, dtype=x.dtype, device=x.device)
    dstate = None if state is None else torch.empty(B, C, ks - 1, dtype=x.dtype, device=x.device)
    dw_part = torch.empty(blocks, C, ks, dtype=torch.float32, device=x.device)
    db_part = torch.empty(blocks, C, dtype=torch.float32, device=x.device)
    a = _lib.GdnConvBwdArgs()
    a.x, a.dy, a.weight, a.dx = x.data_ptr(), dy.data_ptr(), w2.data_ptr(), dx.data_ptr()
    a.bias = None if b2 is None else b2.data_ptr()
    a.input_state = None if state is None else state.data_ptr()
    a.mask = None if mask is None else mask.data_ptr()
    a.dstate = None if dstate is None else dstate.data_ptr()
    a.dweight_partial, a.dbias_partial = dw_part.data_ptr(), db_part.data_ptr()
    a.x_stride_b, a.x_stride_s, a.dy_stride_b, a.dy_stride_s = x.stride(0), x.stride(1), dy.stride(0), dy.stride(1)
    a.B, a.S, a.C, a.kernel_size, a.tokens_per_block = B, S, C, ks, _BWD_TOKENS_PER_BLOCK
    a.w_dtype = _dtype_code(w2.dtype, "weight")
    a.dtype = _dtype_code(x.dtype, "x")
    a.activation = _IN_KERNEL_ACTIVATIONS[activation]
    with torch.cuda.device(x.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        _lib.check_status(lib.gdn_causal_conv1d_bwd(ctypes.byref(a), stream), "gdn_causal_conv1d_bwd")
    dweight = dw_part.sum(dim=0).to(weight.dtype).reshape(weight.shape)
    dbias = None if bias is None else db_part.sum(dim=0).to(bias.dtype)
    dstate = None if dstate is None else dstate.to(input_state.dtype)
    return dx, dweight, dbias, dstate


def _depthwise_causal_convolution(x, weight, bias, input_state, attention_mask, output_state, activation):
    if not is_kernel_allowed(Kernel.gated_delta_rule):
        raise RuntimeError("Kernel.gated_delta_rule is disabled and this package ships no other implementation")
    if activation not in _IN_KERNEL_ACTIVATIONS:
        # the reference applies any other activation after the kernel (depthwise_causal_convolution.py:172-173)
        raise ValueError(f"activation {activation!r} is not fused; pass activation=None and apply it to the result")
    if x.dim() != 3:
        raise ValueError("x must be [B, S, C]")
    if not x.is_cuda:
        raise ValueError("the convolution runs on the GPU only; x must be a device tensor")
    B, S, C = x.shape
    if weight.dim() == 3:
        if weight.size(1) != 1:
            raise ValueError("weight must be depthwise: [C, 1, kernel_size]")
        weight = weight.squeeze(1)
    if weight.dim() != 2 or weight.size(0) != C:
        raise ValueError(f"weight must be [C, kernel_size] with C = {C}, got {tuple(weight.shape)}")
    ks = weight.size(1)
    if not 2 <= ks <= 4:
        raise ValueError(f"kernel_size {ks} is not supported (2..4)")
    if bias is not None and tuple(bias.shape) != (C,):
        raise ValueError(f"bias must be [C] = {(C,)}, got {tuple(bias.shape)}")
    if bias is not None and bias.dtype != weight.dtype:
        raise ValueError("weight and bias must share a dtype")
    if input_state is not None:
        if tuple(input_state.shape) != (B, C, ks - 1):
            raise ValueError(f"input_state must be [B, C, kernel_size - 1] = {(B, C, ks - 1)}, got {tuple(input_state.shape)}")
        input_state = input_state.to(x.dtype).contiguous()
    for name, t in (("weight", weight), ("bias", bias), ("input_state", input_state), ("attention_mask", attention_mask)):
        if t is not None and t.device != x.device:
            raise ValueError(f"{name} is on {t.device}, x is on {x.device}")

    mask = None
    if attention_mask is not None and attention_mask.shape[1] > 1 and attention_mask.shape[0] > 1:
        if tuple(attention_mask.shape) != (B, S):
            raise ValueError(f"attention_mask must be [B, S] = {(B, S)}, got {tuple(attention_mask.shape)}")
        mask = attention_mask.to(x.dtype).contiguous()

    if x.stride(-1) != 1:
        x = x.contiguous()
    if x.dtype == torch.float32 and weight.dtype != torch.float32:  # the kernel wants weights as wide as the data
        weight = weight.float()
        bias = None if bias is None else bias.float()
    weight = weight.contiguous()
    bias = None if bias is None else bias.contiguous()
    y = torch.empty(B, S, C, dtype=x.dtype, device=x.device)
    final_state = torch.empty(B, C, ks - 1, dtype=x.dtype, device=x.device) if output_state else None

    a = _lib.GdnConvArgs()
    a.x, a.weight, a.y = x.data_ptr(), weight.data_ptr(), y.data_ptr()
    a.bias = None if bias is None else bias.data_ptr()
    a.input_state = None if input_state is None else input_state.data_ptr()
    a.mask = None if mask is None else mask.data_ptr()
    a.final_state = None if final_state is None else final_state.data_ptr()
    a.x_stride_b, a.x_stride_s = x.stride(0), x.stride(1)
    a.y_stride_b, a.y_stride_s = y.stride(0), y.stride(1)
    a.B, a.S, a.C, a.kernel_size = B, S, C, ks
    a.dtype = _dtype_code(x.dtype, "x")
    a.w_dtype = _dtype_code(weight.dtype, "weight")
    a.activation = _IN_KERNEL_ACTIVATIONS[activation]

    lib = _lib.load_library()
    with torch.cuda.device(x.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        _lib.check_status(lib.gdn_causal_conv1d_fwd(ctypes.byref(a), stream), "gdn_causal_conv1d_fwd")
    return y, final_state
