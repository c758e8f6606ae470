"""The kernels as opaque operators of ``torch.library``, for ``torch.compile``.

The eager entry points of this package launch their HIP kernels through ctypes, which a tracing compiler cannot
follow.  While a graph is being captured (``torch.compiler.is_compiling()``) they call the operators below instead:
each is a ``torch.library.custom_op`` with a shape-only ("fake") implementation and a registered backward, so the
operator and the single-kernel layer steps go into a captured graph as single nodes, forward and backward, without a
graph break - what the reference gets for its Triton kernels from ``torch.compile`` itself (the layer runs under
``torch.compile`` in lm_engine/model_wrapper/base.py:137-144).  The operators call the same Python launchers as the
eager path, so results are identical.

An operator of ``torch.library`` returns tensors only: an output that the eager function returns as ``None`` comes
back as an empty tensor here and is turned into ``None`` again by the wrapper functions at the bottom.
"""

from __future__ import annotations

import torch


def _or_empty(x, like):
    return like.new_empty(0) if x is None else x


# ---------------------------------------------------------------------------------------
# the operator: (q, k, v, g, beta, initial_state, cu_seqlens) -> (o, final_state)
# ---------------------------------------------------------------------------------------
@torch.library.custom_op(
    "lm_engine_amd::gated_delta_rule_forward",
    mutates_args=(),
    schema="(Tensor q, Tensor k, Tensor v, Tensor? g, Tensor? beta, Tensor? initial_state, Tensor? cu_seqlens, str mode, "
    "float? scale, bool output_final_state, bool l2norm, bool left_padded) -> (Tensor, Tensor)",
)
def gated_delta_rule_forward(q, k, v, g, beta, initial_state, cu_seqlens, mode, scale, output_final_state, l2norm,
                             left_padded):  # fmt: skip
    from . import ops

    o, ht = ops._run(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm, False,
                     left_padded)  # fmt: skip
    return o, _or_empty(ht, o)


@gated_delta_rule_forward.register_fake
def _(q, k, v, g, beta, initial_state, cu_seqlens, mode, scale, output_final_state, l2norm, left_padded):
    B, T, _, K = q.shape
    H, V = v.size(2), v.size(-1)
    N = B if cu_seqlens is None or left_padded else cu_seqlens.numel() - 1
    o = v.new_empty(B, T, H, V)
    ht = v.new_empty((N, H, K, V), dtype=torch.float32) if output_final_state else v.new_empty(0)
    return o, ht


@torch.library.custom_op(
    "lm_engine_amd::gated_delta_rule_backward",
    mutates_args=(),
    schema="(Tensor q, Tensor k, Tensor v, Tensor? g, Tensor? beta, Tensor? initial_state, Tensor? cu_seqlens, Tensor d_o, "
    "Tensor? d_ht, float? scale, bool l2norm, bool left_padded) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)",
)
def gated_delta_rule_backward(q, k, v, g, beta, initial_state, cu_seqlens, d_o, d_ht, scale, l2norm, left_padded):
    from .backward import gated_delta_rule_backward as run

    dq, dk, dv, dg, dbeta, dh0 = run(q, k, v, g, beta, d_o, d_ht, scale=scale, initial_state=initial_state,
                                     cu_seqlens=cu_seqlens, use_qk_l2norm_in_kernel=l2norm, left_padded=left_padded)  # fmt: skip
    return dq, dk, dv, _or_empty(dg, q), _or_empty(dbeta, q), _or_empty(dh0, q)


@gated_delta_rule_backward.register_fake
def _(q, k, v, g, beta, initial_state, cu_seqlens, d_o, d_ht, scale, l2norm, left_padded):
    empty = q.new_empty(0)
    return (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
            empty if g is None else torch.empty_like(g), empty if beta is None else torch.empty_like(beta),
            empty if initial_state is None else torch.empty_like(initial_state, dtype=torch.float32))  # fmt: skip


def _gdr_setup(ctx, inputs, output):
    q, k, v, g, beta, initial_state, cu_seqlens, mode, scale, output_final_state, l2norm, left_padded = inputs
    ctx.save_for_backward(q, k, v, g, beta, initial_state, cu_seqlens)
    ctx.options = (scale, l2norm, left_padded, output_final_state)


def _gdr_backward(ctx, d_o, d_ht):
    q, k, v, g, beta, initial_state, cu_seqlens = ctx.saved_tensors
    scale, l2norm, left_padded, output_final_state = ctx.options
    d_ht = d_ht if output_final_state else None
    dq, dk, dv, dg, dbeta, dh0 = torch.ops.lm_engine_amd.gated_delta_rule_backward(
        q, k, v, g, beta, initial_state, cu_seqlens, d_o.contiguous(), d_ht, scale, l2norm, left_padded)  # fmt: skip
    return (dq, dk, dv, None if g is None else dg, None if beta is None else dbeta,
            None if initial_state is None else dh0, None, None, None, None, None, None)  # fmt: skip


gated_delta_rule_forward.register_autograd(_gdr_backward, setup_context=_gdr_setup)


@torch.library.custom_op(
    "lm_engine_amd::gated_delta_rule_decode_",
    mutates_args=("state",),
    schema="(Tensor q, Tensor k, Tensor v, Tensor? g, Tensor? beta, Tensor(a!) state, Tensor? cu_seqlens, float? scale, "
    "bool l2norm, bool left_padded) -> Tensor",
)
def gated_delta_rule_decode_(q, k, v, g, beta, state, cu_seqlens, scale, l2norm, left_padded):
    """The recurrent kernel with the state updated in place (inference)."""
    from . import ops

    o, _ = ops._run("recurrent", q, k, v, g, beta, scale, state, True, cu_seqlens, l2norm, True, left_padded)
    return o


@gated_delta_rule_decode_.register_fake
def _(q, k, v, g, beta, state, cu_seqlens, scale, l2norm, left_padded):
    return v.new_empty(v.shape)


# ---------------------------------------------------------------------------------------
# depthwise causal convolution
# ---------------------------------------------------------------------------------------
@torch.library.custom_op(
    "lm_engine_amd::causal_conv1d_forward",
    mutates_args=(),
    schema="(Tensor x, Tensor weight, Tensor? bias, Tensor? input_state, Tensor? attention_mask, bool output_state, "
    "str activation) -> (Tensor, Tensor)",
)
def causal_conv1d_forward(x, weight, bias, input_state, attention_mask, output_state, activation):
    from . import conv

    y, state = conv._depthwise_causal_convolution(x, weight, bias, input_state, attention_mask, output_state,
                                                  activation or None)  # fmt: skip
    return y, _or_empty(state, y)


@causal_conv1d_forward.register_fake
def _(x, weight, bias, input_state, attention_mask, output_state, activation):
    B, S, C = x.shape
    ks = weight.size(-1)
    return x.new_empty(B, S, C), (x.new_empty(B, C, ks - 1) if output_state else x.new_empty(0))


@torch.library.custom_op(
    "lm_engine_amd::causal_conv1d_backward",
    mutates_args=(),
    schema="(Tensor x, Tensor weight, Tensor? bias, Tensor? input_state, Tensor? attention_mask, Tensor dy, "
    "str activation) -> (Tensor, Tensor, Tensor, Tensor)",
)
def causal_conv1d_backward(x, weight, bias, input_state, attention_mask, dy, activation):
    from . import conv

    act = activation or None
    if not conv._backward_kernel_applies(x, weight, act):
        # (eager mode differentiates the formula in torch operations here; an operator cannot run autograd inside itself)
        raise NotImplementedError("in a captured graph the convolution's backward is the HIP kernel only: bf16 x on the "
                                  "GPU, channels a multiple of 8, a fused activation")  # fmt: skip
    dx, dw, db, ds = conv._convolution_backward(x, weight, bias, input_state, attention_mask, dy, act)
    return dx, dw, _or_empty(db, x), _or_empty(ds, x)


@causal_conv1d_backward.register_fake
def _(x, weight, bias, input_state, attention_mask, dy, activation):
    empty = x.new_empty(0)
    return (torch.empty_like(x), torch.empty_like(weight), empty if bias is None else torch.empty_like(bias),
            empty if input_state is None else torch.empty_like(input_state))  # fmt: skip


def _conv_setup(ctx, inputs, output):
    x, weight, bias, input_state, attention_mask, output_state, activation = inputs
    ctx.save_for_backward(x, weight, bias, input_state, attention_mask)
    ctx.activation = activation


def _conv_backward(ctx, dy, _dstate):  # the gradient into the returned state is not propagated (the cache is not differentiated through)
    x, weight, bias, input_state, attention_mask = ctx.saved_tensors
    dx, dw, db, ds = torch.ops.lm_engine_amd.causal_conv1d_backward(x, weight, bias, input_state, attention_mask,
                                                                    dy.contiguous(), ctx.activation)  # fmt: skip
    return dx, dw, None if bias is None else db, None if input_state is None else ds, None, None, None


causal_conv1d_forward.register_autograd(_conv_backward, setup_context=_conv_setup)


# ---------------------------------------------------------------------------------------
# gates
# ---------------------------------------------------------------------------------------
@torch.library.custom_op(
    "lm_engine_amd::delta_rule_gates_forward",
    mutates_args=(),
    schema="(Tensor a, Tensor b, Tensor A_log, Tensor dt_bias, bool allow_neg_eigval) -> (Tensor, Tensor)",
)
def delta_rule_gates_forward(a, b, A_log, dt_bias, allow_neg_eigval):
    from . import layer_ops

    return layer_ops._delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval)


@delta_rule_gates_forward.register_fake
def _(a, b, A_log, dt_bias, allow_neg_eigval):
    return a.new_empty(a.shape, dtype=torch.float32), a.new_empty(a.shape)


@torch.library.custom_op(
    "lm_engine_amd::delta_rule_gates_backward",
    mutates_args=(),
    schema="(Tensor a, Tensor b, Tensor A_log, Tensor dt_bias, Tensor dg, Tensor dbeta, bool allow_neg_eigval) -> "
    "(Tensor, Tensor, Tensor, Tensor)",
)
def delta_rule_gates_backward(a, b, A_log, dt_bias, dg, dbeta, allow_neg_eigval):
    # g = -exp(A_log) softplus(a + dt_bias), beta = s sigmoid(b)
    if a.is_cuda and a.dtype in (torch.bfloat16, torch.float32):
        from . import layer_ops

        return layer_ops._delta_rule_gates_backward(a, b, A_log, dt_bias, dg, dbeta, allow_neg_eigval)
    # elsewhere: the derivatives in closed form, fp32 arithmetic (an operator cannot run autograd inside itself)
    dg = dg.float()
    rate = -torch.exp(A_log.float())
    z = a.float() + dt_bias.float()
    d_z = dg * rate * torch.sigmoid(z)
    tokens = tuple(range(a.dim() - 1))
    d_A_log = (dg * rate * torch.nn.functional.softplus(z)).sum(dim=tokens)
    sig = torch.sigmoid(b.float())
    d_b = dbeta.float() * (2.0 if allow_neg_eigval else 1.0) * sig * (1.0 - sig)
    return d_z.to(a.dtype), d_b.to(b.dtype), d_A_log.to(A_log.dtype), d_z.sum(dim=tokens).to(dt_bias.dtype)


@delta_rule_gates_backward.register_fake
def _(a, b, A_log, dt_bias, dg, dbeta, allow_neg_eigval):
    return torch.empty_like(a), torch.empty_like(b), torch.empty_like(A_log), torch.empty_like(dt_bias)


def _gates_setup(ctx, inputs, output):
    a, b, A_log, dt_bias, allow_neg_eigval = inputs
    ctx.save_for_backward(a, b, A_log, dt_bias)
    ctx.allow_neg_eigval = allow_neg_eigval


def _gates_backward(ctx, dg, dbeta):
    a, b, A_log, dt_bias = ctx.saved_tensors
    grads = torch.ops.lm_engine_amd.delta_rule_gates_backward(a, b, A_log, dt_bias, dg.contiguous(), dbeta.contiguous(),
                                                              ctx.allow_neg_eigval)  # fmt: skip
    return (*grads, None)


delta_rule_gates_forward.register_autograd(_gates_backward, setup_context=_gates_setup)


# ---------------------------------------------------------------------------------------
# gated RMS norm
# ---------------------------------------------------------------------------------------
@torch.library.custom_op(
    "lm_engine_amd::gated_rmsnorm_forward",
    mutates_args=(),
    schema="(Tensor o, Tensor? gate, Tensor? weight, float? eps) -> Tensor",
)
def gated_rmsnorm_forward(o, gate, weight, eps):
    from . import layer_ops

    return layer_ops._gated_rmsnorm(o, gate, weight, eps)


@gated_rmsnorm_forward.register_fake
def _(o, gate, weight, eps):
    return o.new_empty(o.shape)


@torch.library.custom_op(
    "lm_engine_amd::gated_rmsnorm_backward",
    mutates_args=(),
    schema="(Tensor o, Tensor? gate, Tensor? weight, float? eps, Tensor dy) -> (Tensor, Tensor, Tensor)",
)
def gated_rmsnorm_backward(o, gate, weight, eps, dy):
    from . import layer_ops

    d_o, d_gate, d_weight = layer_ops._gated_rmsnorm_backward(o, gate, weight, eps, dy)
    return d_o, _or_empty(d_gate, o), _or_empty(d_weight, o)


@gated_rmsnorm_backward.register_fake
def _(o, gate, weight, eps, dy):
    empty = o.new_empty(0)
    return (torch.empty_like(o), empty if gate is None else torch.empty_like(gate),
            empty if weight is None else torch.empty_like(weight))  # fmt: skip


def _norm_setup(ctx, inputs, output):
    o, gate, weight, eps = inputs
    ctx.save_for_backward(o, gate, weight)
    ctx.eps = eps


def _norm_backward(ctx, dy):
    o, gate, weight = ctx.saved_tensors
    d_o, d_gate, d_weight = torch.ops.lm_engine_amd.gated_rmsnorm_backward(o, gate, weight, ctx.eps, dy.contiguous())
    return d_o, None if gate is None else d_gate, None if weight is None else d_weight, None


gated_rmsnorm_forward.register_autograd(_norm_backward, setup_context=_norm_setup)


# ---------------------------------------------------------------------------------------
# what the eager entry points call while a graph is being captured
# ---------------------------------------------------------------------------------------
def gated_delta_rule(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm, inplace_state,
                     left_padded):  # fmt: skip
    if inplace_state:
        if not output_final_state or initial_state is None:
            raise ValueError("inplace_state needs an initial_state to update and output_final_state=True")
        o = torch.ops.lm_engine_amd.gated_delta_rule_decode_(q, k, v, g, beta, initial_state, cu_seqlens, scale, l2norm,
                                                             left_padded)  # fmt: skip
        return o, initial_state
    o, ht = torch.ops.lm_engine_amd.gated_delta_rule_forward(q, k, v, g, beta, initial_state, cu_seqlens, mode, scale,
                                                             output_final_state, l2norm, left_padded)  # fmt: skip
    return o, (ht if output_final_state else None)


def depthwise_causal_convolution(x, weight, bias, input_state, attention_mask, output_state, activation):
    from . import conv

    # Decided while the graph is traced: where a gradient is needed and the backward kernel does not apply (fp32 x,
    # channels not a multiple of 8, no fused activation, too many token blocks), the convolution goes in as its formula
    # in torch operations, which the compiler can differentiate - what eager mode does for such inputs - instead of an
    # operator whose backward would only fail when it is reached.
    needs_grad = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, weight, bias, input_state))
    if needs_grad and not conv._backward_kernel_applies(x, weight, activation or None):
        return conv.convolution_formula(x, weight, bias, input_state, attention_mask, output_state, activation or None)
    y, state = torch.ops.lm_engine_amd.causal_conv1d_forward(x, weight, bias, input_state, attention_mask, output_state,
                                                             activation or "")  # fmt: skip
    return y, (state if output_state else None)


def delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval):
    return torch.ops.lm_engine_amd.delta_rule_gates_forward(a, b, A_log, dt_bias, allow_neg_eigval)


def gated_rmsnorm(o, gate, weight, eps):
    return torch.ops.lm_engine_amd.gated_rmsnorm_forward(o, gate, weight, eps)
