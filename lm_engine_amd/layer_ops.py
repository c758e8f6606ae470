"""The elementwise steps of the GatedDeltaNet layer on either side of the operator, one HIP kernel each.

* ``delta_rule_gates``  - ``beta = sigmoid(b) [* 2]`` and ``g = -exp(A_log) * softplus(a + dt_bias)``:
  lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:179-183 with
  ``SoftplusDecayGate.forward(final_exponential=False)``, softplus_decay_gate/module.py:69-96.
* ``gated_rmsnorm``     - ``o_norm(o * silu(gate))``: module.py:238-242 with the RMSNorm of
  lm_engine/modeling_utils/normalization.py:69-124.

Both take the (strided) slices of the layer's projections as they are; there is no torch fallback.
Under autograd the gated norm's backward is one more HIP kernel (``gdn_gated_rmsnorm_bwd``); the gates'
backward differentiates the same formula written in torch (``_autograd.py``).
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._autograd import kernel_with_formula_backward
from .kernels import Kernel, is_kernel_allowed


def _dtype_code(dtype: torch.dtype, what: str) -> int:
    if dtype == torch.bfloat16:
        return _lib.GDN_BF16
    if dtype == torch.float32:
        return _lib.GDN_F32
    raise ValueError(f"{what} must be bfloat16 or float32, got {dtype}")


def _require(x: torch.Tensor, what: str) -> None:
    if not is_kernel_allowed(Kernel.gated_delta_rule):
        raise RuntimeError("Kernel.gated_delta_rule is disabled and this package ships no other implementation")
    if not x.is_cuda:
        raise ValueError(f"{what} must be a device tensor: these kernels run on the GPU only")


def _token_rows(x: torch.Tensor, width: int, what: str) -> tuple[torch.Tensor, int]:
    """[..., width] view whose leading dims collapse to one token axis with a single stride."""
    if x.size(-1) != width:
        raise ValueError(f"{what}: last dim must be {width}, got {x.size(-1)}")
    if x.stride(-1) != 1:
        x = x.contiguous()
    rows = x.reshape(-1, width) if x.dim() != 2 else x  # a view whenever the leading dims are collapsible
    if rows.stride(-1) != 1:
        rows = rows.contiguous()
    return rows, rows.stride(0) if rows.size(0) > 1 else width


def gates_formula(a, b, A_log, dt_bias, allow_neg_eigval):
    """The gates in torch operations: what their backward differentiates."""
    g = -torch.exp(A_log.float()) * torch.nn.functional.softplus(a.float() + dt_bias.float())
    beta = torch.sigmoid(b.float()) * (2.0 if allow_neg_eigval else 1.0)
    return g, beta.to(b.dtype)


def delta_rule_gates(
    a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, allow_neg_eigval: bool = False
) -> tuple[torch.Tensor, torch.Tensor]:
    """a, b ``[..., H]`` (activation dtype, may be slices of one projection) -> ``(g fp32, beta)`` of the same shape."""

    if torch.compiler.is_compiling():  # a graph is being captured: the kernel goes in as an opaque operator
        from . import _opaque

        return _opaque.delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval)

    def formula(a, b, A_log, dt_bias):
        return gates_formula(a, b, A_log, dt_bias, allow_neg_eigval)

    kernel = lambda a, b, A_log, dt_bias: _delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval)  # noqa: E731
    needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (a, b, A_log, dt_bias))
    if needs_grad and a.is_cuda and a.dtype in (torch.bfloat16, torch.float32):
        return _GatesOnKernels.apply(a, b, A_log, dt_bias, allow_neg_eigval)
    return kernel_with_formula_backward(kernel, formula, a, b, A_log, dt_bias)


class _GatesOnKernels(torch.autograd.Function):
    """Forward and backward on the HIP kernels."""

    @staticmethod
    def forward(ctx, a, b, A_log, dt_bias, allow_neg_eigval):
        ctx.save_for_backward(a, b, A_log, dt_bias)
        ctx.allow_neg_eigval = allow_neg_eigval
        return _delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval)

    @staticmethod
    def backward(ctx, dg, dbeta):
        a, b, A_log, dt_bias = ctx.saved_tensors
        return (*_delta_rule_gates_backward(a, b, A_log, dt_bias, dg, dbeta, ctx.allow_neg_eigval), None)


def _delta_rule_gates_backward(a, b, A_log, dt_bias, dg, dbeta, allow_neg_eigval):
    """``gdn_gates_bwd``: gradients with respect to a, b (contiguous, their dtype), A_log and dt_bias."""
    _require(a, "a")
    H = a.size(-1)
    a2, a_stride = _token_rows(a, H, "a")
    b2, b_stride = _token_rows(b, H, "b")
    tokens = a2.size(0)
    dev = a.device
    dg = (torch.zeros(a.shape, dtype=torch.float32, device=dev) if dg is None else dg.to(torch.float32)).contiguous()
    dbeta = (torch.zeros(a.shape, dtype=a.dtype, device=dev) if dbeta is None else dbeta.to(a.dtype)).contiguous()
    da = torch.empty(a.shape, dtype=a.dtype, device=dev)
    db = torch.empty(a.shape, dtype=a.dtype, device=dev)
    if tokens == 0:
        return da, db, torch.zeros_like(A_log), torch.zeros_like(dt_bias)
    blocks = min(1024, max(1, (tokens * H + 255) // 256))
    parts = torch.empty(2, blocks, H, dtype=torch.float32, device=dev)
    A32 = A_log.to(device=dev, dtype=torch.float32).contiguous()
    dt32 = dt_bias.to(device=dev, dtype=torch.float32).contiguous()
    args = _lib.GdnGateBwdArgs()
    args.a, args.b, args.A_log, args.dt_bias = a2.data_ptr(), b2.data_ptr(), A32.data_ptr(), dt32.data_ptr()
    args.dg, args.dbeta, args.da, args.db = dg.data_ptr(), dbeta.data_ptr(), da.data_ptr(), db.data_ptr()
    args.dA_log_partial, args.ddt_bias_partial = parts[0].data_ptr(), parts[1].data_ptr()
    args.a_stride, args.b_stride, args.tokens, args.H = a_stride, b_stride, tokens, H
    args.dtype = _dtype_code(a.dtype, "a, b")
    args.beta_scale = 2.0 if allow_neg_eigval else 1.0
    args.partial_blocks = blocks
    lib = _lib.load_library()
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        _lib.check_status(lib.gdn_gates_bwd(ctypes.byref(args), stream), "gdn_gates_bwd")
    # two results that share no storage (an operator's outputs must not alias each other)
    return da, db, parts[0].sum(dim=0).to(A_log.dtype), parts[1].sum(dim=0).to(dt_bias.dtype)


def _delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval):
    _require(a, "a")
    H = a.size(-1)
    if b.shape != a.shape or b.dtype != a.dtype:
        raise ValueError("a and b must share shape and dtype")
    if tuple(A_log.shape) != (H,) or tuple(dt_bias.shape) != (H,):
        raise ValueError(f"A_log and dt_bias must be [H] = {(H,)}")
    a2, a_stride = _token_rows(a, H, "a")
    b2, b_stride = _token_rows(b, H, "b")
    A_log = A_log.to(device=a.device, dtype=torch.float32).contiguous()
    dt_bias = dt_bias.to(device=a.device, dtype=torch.float32).contiguous()
    g = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    beta = torch.empty(a.shape, dtype=a.dtype, device=a.device)

    args = _lib.GdnGateArgs()
    args.a, args.b, args.A_log, args.dt_bias = a2.data_ptr(), b2.data_ptr(), A_log.data_ptr(), dt_bias.data_ptr()
    args.g, args.beta = g.data_ptr(), beta.data_ptr()
    args.a_stride, args.b_stride, args.tokens, args.H = a_stride, b_stride, a2.size(0), H
    args.dtype = _dtype_code(a.dtype, "a, b")
    args.beta_scale = 2.0 if allow_neg_eigval else 1.0
    lib = _lib.load_library()
    with torch.cuda.device(a.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
        _lib.check_status(lib.gdn_gates_fwd(ctypes.byref(args), stream), "gdn_gates_fwd")
    return g, beta


def gated_rmsnorm_formula(o, gate, weight, eps_value):
    """The gated norm in torch operations: what its backward differentiates off the GPU."""
    x = o.float()
    if gate is not None:
        x = x * torch.nn.functional.silu(gate.float().reshape(o.shape))
    y = x * torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + eps_value)
    if weight is not None:
        y = y * weight.float()
    return (y.to(o.dtype),)


def gated_rmsnorm(
    o: torch.Tensor, gate: torch.Tensor | None, weight: torch.Tensor | None, eps: float | None = None
) -> torch.Tensor:
    """o ``[..., H, V]``; gate the same shape or ``[..., H * V]`` (a slice of a projection) or None;
    weight ``[V]`` or None.  Returns ``rmsnorm(o * silu(gate)) * weight`` over V, shape and dtype of o.
    ``eps=None`` is torch's default for nn.RMSNorm: the machine epsilon of o's dtype."""
    eps_value = float(torch.finfo(o.dtype).eps if eps is None else eps)

    if torch.compiler.is_compiling():  # a graph is being captured: the kernel goes in as an opaque operator
        from . import _opaque

        return _opaque.gated_rmsnorm(o, gate, weight, eps)

    def formula(o, gate, weight):
        return gated_rmsnorm_formula(o, gate, weight, eps_value)

    kernel = lambda o, gate, weight: (_gated_rmsnorm(o, gate, weight, eps),)  # noqa: E731
    needs_grad = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (o, gate, weight))
    if needs_grad and o.is_cuda and o.dtype in (torch.bfloat16, torch.float32):
        return _GatedRMSNormOnKernels.apply(o, gate, weight, eps)
    return kernel_with_formula_backward(kernel, formula, o, gate, weight)[0]


class _GatedRMSNormOnKernels(torch.autograd.Function):
    """Forward and backward on the HIP kernels."""

    @staticmethod
    def forward(ctx, o, gate, weight, eps):
        ctx.save_for_backward(o, gate, weight)
        ctx.eps = eps
        return _gated_rmsnorm(o, gate, weight, eps)

    @staticmethod
    def backward(ctx, dy):
        o, gate, weight = ctx.saved_tensors
        d_o, d_gate, d_weight = _gated_rmsnorm_backward(o, gate, weight, ctx.eps, dy)
        return d_o, d_gate, d_weight, None


def _gated_rmsnorm_backward(o, gate, weight, eps, dy):
    """``gdn_gated_rmsnorm_bwd``: gradients with respect to o, gate (shaped like gate) and weight."""
    o2, o_stride, g2, g_stride, H, V = _norm_operands(o, gate)
    tokens = o2.size(0)
    dy = dy.to(o.dtype).contiguous()
    d_o = torch.empty(o.shape, dtype=o.dtype, device=o.device)
    d_gate = None if gate is None else torch.empty(o.shape, dtype=o.dtype, device=o.device)
    blocks = min(2048, max(1, (tokens * H * max(V // 8, 8) + 255) // 256))
    dw_part = torch.empty(blocks, V, dtype=torch.float32, device=o.device)
    w = None if weight is None else weight.contiguous()
    args = _lib.GdnNormBwdArgs()
    args.o, args.dy, args.d_o, args.dweight_partial = o2.data_ptr(), dy.data_ptr(), d_o.data_ptr(), dw_part.data_ptr()
    args.gate = None if g2 is None else g2.data_ptr()
    args.d_gate = None if d_gate is None else d_gate.data_ptr()
    args.weight = None if w is None else w.data_ptr()
    args.o_stride_t, args.gate_stride_t, args.tokens, args.H, args.V = o_stride, g_stride, tokens, H, V
    args.dtype = _dtype_code(o.dtype, "o")
    args.w_dtype = _lib.GDN_F32 if w is None else _dtype_code(w.dtype, "weight")
    args.eps = float(torch.finfo(o.dtype).eps if eps is None else eps)
    args.partial_blocks = blocks
    lib = _lib.load_library()
    with torch.cuda.device(o.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(o.device).cuda_stream)
        _lib.check_status(lib.gdn_gated_rmsnorm_bwd(ctypes.byref(args), stream), "gdn_gated_rmsnorm_bwd")
    d_weight = None if weight is None else dw_part.sum(dim=0).to(weight.dtype)
    return d_o, (None if gate is None else d_gate.reshape(gate.shape)), d_weight


def _norm_operands(o, gate):
    """Token-row views of o and gate for the norm kernels: ``(o2, o_stride, g2, g_stride, H, V)``."""
    _require(o, "o")
    if o.dim() < 2:
        raise ValueError("o must be [..., H, V]")
    H, V = o.shape[-2], o.shape[-1]
    if V % 8 != 0 or V > 512:
        raise ValueError(f"V={V} is not supported (multiple of 8, at most 512)")
    o2, o_stride = _token_rows(o.flatten(-2) if o.is_contiguous() else o.contiguous().flatten(-2), H * V, "o")
    g2, g_stride = None, 0
    if gate is not None:
        if gate.dtype != o.dtype or gate.numel() != o.numel():
            raise ValueError("gate must have the dtype and number of elements of o")
        if gate.shape[-2:] == (H, V) and gate.dim() == o.dim():
            gate = gate.flatten(-2) if gate.stride(-2) == V and gate.stride(-1) == 1 else gate.contiguous().flatten(-2)
        g2, g_stride = _token_rows(gate, H * V, "gate")
        if g2.data_ptr() % 16 != 0 or (g_stride * g2.element_size()) % 16 != 0:
            # a slice that starts off a 16-byte boundary (e.g. behind 2 * H gate scalars with H = 2) is compacted
            g2 = g2.contiguous()
            g_stride = H * V
    return o2, o_stride, g2, g_stride, H, V


def _gated_rmsnorm(o, gate, weight, eps):
    o2, o_stride, g2, g_stride, H, V = _norm_operands(o, gate)
    if weight is not None and tuple(weight.shape) != (V,):
        raise ValueError(f"weight must be [V] = {(V,)}")
    weight = None if weight is None else weight.contiguous()
    y = torch.empty(o.shape, dtype=o.dtype, device=o.device)

    args = _lib.GdnNormArgs()
    args.o, args.y = o2.data_ptr(), y.data_ptr()
    args.gate = None if g2 is None else g2.data_ptr()
    args.weight = None if weight is None else weight.data_ptr()
    args.o_stride_t, args.gate_stride_t, args.y_stride_t = o_stride, g_stride, H * V
    args.tokens, args.H, args.V = o2.size(0), H, V
    args.dtype = _dtype_code(o.dtype, "o")
    args.w_dtype = _lib.GDN_F32 if weight is None else _dtype_code(weight.dtype, "weight")
    args.eps = float(torch.finfo(o.dtype).eps if eps is None else eps)
    lib = _lib.load_library()
    with torch.cuda.device(o.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(o.device).cuda_stream)
        _lib.check_status(lib.gdn_gated_rmsnorm_fwd(ctypes.byref(args), stream), "gdn_gated_rmsnorm_fwd")
    return y
