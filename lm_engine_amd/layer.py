"""Everything `GatedDeltaNet.forward` does between its input and output projections, on the HIP kernels.

Follows lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:168-242 step by step:

    qkv, conv_state = conv1d(qkv, conv_state)            :168-170  -> depthwise_causal_convolution
    q, k, v = split / view                                :172-177  (views; GVA heads are shared inside the operator)
    beta, g = sigmoid(b) [* 2], decay_gate(a)             :179-183  -> delta_rule_gates
    o, h = chunk or fused_recurrent (T <= 64)             :193-222  -> gated_delta_rule kernels
    o = o_norm(o * silu(gate))                            :238-241  -> gated_rmsnorm

With an attention mask the reference packs q, k, v, g, beta into one token stream and unpacks the output
(:185-191, :226-227, sequence_packing.py:25-93; as written there the packed tensors lose the batch
dimension the operator wants and the unpack shape is not the output's).  Here nothing is copied: the mask
becomes the prefix sums of the valid lengths (sequence_packing.py:18-22) and the kernels work on the
left-padded batch in place (``left_padded=True``), writing zeros at the padding as the unpack would.
"""

from __future__ import annotations

import torch

from .conv import depthwise_causal_convolution
from .layer_ops import delta_rule_gates, gated_rmsnorm
from .ops import RECURRENT_MAX_TOKENS, chunk_gated_delta_rule, fused_recurrent_gated_delta_rule


def gated_deltanet_mixing(
    qkv: torch.Tensor,
    a: torch.Tensor,
    b: torch.Tensor,
    gate: torch.Tensor | None,
    conv_weight: torch.Tensor,
    conv_bias: torch.Tensor | None,
    A_log: torch.Tensor,
    dt_bias: torch.Tensor,
    norm_weight: torch.Tensor | None,
    norm_eps: float | None,
    num_k_heads: int,
    num_v_heads: int,
    k_head_dim: int,
    v_head_dim: int,
    cache: tuple[torch.Tensor | None, torch.Tensor | None] | None = None,
    allow_neg_eigval: bool = False,
    scale: float | None = None,
    conv_activation: str | None = "silu",
    attention_mask: torch.Tensor | None = None,
) -> tuple[torch.Tensor, tuple[torch.Tensor, torch.Tensor] | None]:
    """qkv ``[B, S, 2 * num_k_heads * k_head_dim + num_v_heads * v_head_dim]`` (output of qkv_proj),
    a, b ``[B, S, num_v_heads]``, gate ``[B, S, num_v_heads * v_head_dim]`` or None (slices of ab_proj's
    output).  ``cache`` is None (no caching), ``(None, None)`` (start caching) or the pair returned by the
    previous call.  ``attention_mask`` ``[B, S]``: 1 for tokens, 0 for the padding on the left of shorter
    sequences.  Returns ``(o [B, S, num_v_heads * v_head_dim], new cache or None)``."""
    B, S, _ = qkv.shape
    key_dim, value_dim = num_k_heads * k_head_dim, num_v_heads * v_head_dim
    if qkv.size(-1) != 2 * key_dim + value_dim:
        raise ValueError(f"qkv must have {2 * key_dim + value_dim} channels, got {qkv.size(-1)}")
    if num_v_heads % num_k_heads != 0:
        raise ValueError("num_v_heads must be a multiple of num_k_heads")
    use_cache = cache is not None
    conv_state, h = cache if use_cache else (None, None)

    qkv, conv_state = depthwise_causal_convolution(qkv, conv_weight, conv_bias, conv_state, attention_mask, use_cache,
                                                   conv_activation)  # fmt: skip
    q, k, v = qkv.split((key_dim, key_dim, value_dim), dim=-1)
    q = q.view(B, S, num_k_heads, k_head_dim)
    k = k.view(B, S, num_k_heads, k_head_dim)
    v = v.view(B, S, num_v_heads, v_head_dim)
    # grouped value attention (num_v_heads > num_k_heads): the operator reads head h / (num_v_heads / num_k_heads) of q
    # and k for value head h, so the reference's repeat_interleave copies (module.py:175-177) are not made

    g, beta = delta_rule_gates(a, b, A_log, dt_bias, allow_neg_eigval)

    cu_seqlens = None
    if attention_mask is not None:  # sequence_packing.py:18-22
        seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
        cu_seqlens = torch.nn.functional.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))

    op = fused_recurrent_gated_delta_rule if S <= RECURRENT_MAX_TOKENS else chunk_gated_delta_rule
    o, h = op(q=q, k=k, v=v, g=g, beta=beta, scale=scale, initial_state=h, output_final_state=use_cache,
              cu_seqlens=cu_seqlens, use_qk_l2norm_in_kernel=True, left_padded=cu_seqlens is not None)  # fmt: skip

    o = gated_rmsnorm(o, gate, norm_weight, norm_eps)
    return o.flatten(-2, -1), ((conv_state, h) if use_cache else None)
