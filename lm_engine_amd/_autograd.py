"""Autograd for the single-kernel layer steps (convolution, gates, gated norm).

Their forward is one HIP kernel each; their backward differentiates the same function written with
torch operations at the saved inputs (fp32 arithmetic, on the inputs' device).  These steps are
elementwise or row-wise and memory-bound: the backward costs a few passes over the same tensors."""

from __future__ import annotations

import torch


class _KernelWithFormulaBackward(torch.autograd.Function):
    @staticmethod
    def forward(ctx, kernel, formula, *inputs):
        outputs = kernel(*inputs)
        ctx.formula = formula
        ctx.is_tensor = [isinstance(x, torch.Tensor) for x in inputs]
        ctx.others = [None if t else x for t, x in zip(ctx.is_tensor, inputs)]
        ctx.save_for_backward(*[x for x in inputs if isinstance(x, torch.Tensor)])
        return outputs

    @staticmethod
    def backward(ctx, *grad_outputs):
        saved = iter(ctx.saved_tensors)
        inputs, leaves = [], []
        for i, (t, other) in enumerate(zip(ctx.is_tensor, ctx.others)):
            if not t:
                inputs.append(other)
                continue
            x = next(saved).detach()
            if ctx.needs_input_grad[2 + i] and x.is_floating_point():
                x = x.requires_grad_(True)
                leaves.append((i, x))
            inputs.append(x)
        with torch.enable_grad():
            outputs = ctx.formula(*inputs)
        pairs = [(o, g) for o, g in zip(outputs, grad_outputs) if o is not None and g is not None and o.requires_grad]
        grads = [None] * len(inputs)
        if pairs and leaves:
            got = torch.autograd.grad([o for o, _ in pairs], [x for _, x in leaves], [g for _, g in pairs],
                                      allow_unused=True)  # fmt: skip
            for (i, _), gx in zip(leaves, got):
                grads[i] = gx
        return (None, None, *grads)


def kernel_with_formula_backward(kernel, formula, *inputs):
    """``kernel(*inputs)`` (a tuple of tensors / None); when a gradient is needed, recorded so that its
    backward differentiates ``formula(*inputs)``, the same function in torch operations."""
    needs = torch.is_grad_enabled() and any(isinstance(x, torch.Tensor) and x.requires_grad for x in inputs)
    if not needs:
        return kernel(*inputs)
    return _KernelWithFormulaBackward.apply(kernel, formula, *inputs)
