"""CPU restatement of the gated delta rule (torch, fp32 or fp64).

TEST INFRASTRUCTURE ONLY: the shipped package never imports this file.

What is restated, and from where
--------------------------------
The reference layer calls two functions of the third-party package ``fla``
(flash-linear-attention, version unpinned, absent from the reference tree):

* ``chunk_gated_delta_rule``            reference call site
  lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:197-209
* ``fused_recurrent_gated_delta_rule``  reference call site
  lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:210-222

Their published algorithm is the gated delta rule; per (sequence, head) and
token t, with S in R^{K x V}:

    q^ = (l2norm(q_t) if flag else q_t) * scale      k^ = l2norm(k_t) if flag else k_t
    S  <- exp(g_t) * S
    r  =  beta_t * (v_t - S^T k^)
    S  <- S + k^ (outer) r
    o_t = S^T q^                                     (uses the UPDATED state)

``recurrent_gated_delta_rule_ref`` states exactly that as a token loop, in the
house style of the reference's naive ops (fp32 state ``[B, N, K, V]``, python
loop over the sequence):
lm_engine/modeling_utils/sequence_mixer_blocks/linear_attention/op.py:10-44 and
.../m2rnn/op.py:11-66.  ``chunk_gated_delta_rule_ref`` is an independent
restatement through the chunked WY/UT form (house style of
.../mamba2/op.py:225-328) so that one can be checked against the other the way
the reference checks its own chunked ops (tests/mamba2_op_test.py:11-56).

Parity status
-------------
PARITY UNPINNED at the ``fla`` boundary: the reference holds no test, golden
vector or fixture for this path and ``fla`` is not installed.  Every function
here is instead pinned by tests/test_oracle_*.py against what the mathematics
fixes (closed forms, library routines, invariants, brute force in fp64).
"""

from __future__ import annotations

import torch


L2NORM_EPS = 1e-6


def l2norm_ref(x: torch.Tensor, eps: float = L2NORM_EPS) -> torch.Tensor:
    """x / sqrt(sum(x^2) + eps) over the last dim, the in-kernel q/k normalisation the
    reference requests with use_qk_l2norm_in_kernel=True (gated_deltanet/module.py:208,221)."""
    return x * torch.rsqrt(x.square().sum(dim=-1, keepdim=True) + eps)


def _prepare(q, k, v, g, beta, scale, use_qk_l2norm_in_kernel, dtype):
    K = q.size(-1)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    if use_qk_l2norm_in_kernel:
        q, k = l2norm_ref(q), l2norm_ref(k)
    if scale is None:
        scale = K**-0.5
    q = q * scale
    B, T, H = v.shape[:3]
    g = torch.zeros(B, T, H, dtype=dtype) if g is None else g.to(dtype)
    beta = torch.ones(B, T, H, dtype=dtype) if beta is None else beta.to(dtype)
    return q, k, v, g, beta


def _sequence_ranges(B: int, T: int, cu_seqlens) -> list[tuple[int, int, int]]:
    """(batch index, first token, one-past-last token) of every sequence.

    cu_seqlens follows lm_engine/modeling_utils/sequence_packing.py:18-22: int32 with a
    leading 0; with it the batch dim must be 1 and tokens are packed along T."""
    if cu_seqlens is None:
        return [(b, 0, T) for b in range(B)]
    assert B == 1, "packed (cu_seqlens) input needs a batch dim of 1"
    cu = [int(x) for x in cu_seqlens.tolist()]
    assert cu[0] == 0 and cu[-1] == T
    return [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def recurrent_gated_delta_rule_ref(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None = None,
    beta: torch.Tensor | None = None,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    use_qk_l2norm_in_kernel: bool = False,
    state_dtype: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Naive token-by-token gated delta rule.

    q, k: [B, T, H, K]   v: [B, T, H, V]   g, beta: [B, T, H]
    initial_state: [N, H, K, V] (N = B, or the number of packed sequences)
    returns o [B, T, H, V] in v.dtype and the final state [N, H, K, V] in state_dtype.
    """
    out_dtype = v.dtype
    B, T, H, K = q.shape
    V = v.size(-1)
    q, k, v, g, beta = _prepare(q, k, v, g, beta, scale, use_qk_l2norm_in_kernel, state_dtype)
    ranges = _sequence_ranges(B, T, cu_seqlens)
    N = len(ranges)

    o = torch.zeros(B, T, H, V, dtype=state_dtype)
    ht = torch.zeros(N, H, K, V, dtype=state_dtype)

    for n, (b, t0, t1) in enumerate(ranges):
        S = torch.zeros(H, K, V, dtype=state_dtype) if initial_state is None else initial_state[n].to(state_dtype)
        for t in range(t0, t1):
            S = S * g[b, t].exp()[:, None, None]
            # r = beta * (v - S^T k)
            r = beta[b, t][:, None] * (v[b, t] - (k[b, t][:, :, None] * S).sum(dim=1))
            S = S + k[b, t][:, :, None] * r[:, None, :]
            o[b, t] = (q[b, t][:, :, None] * S).sum(dim=1)
        ht[n] = S

    return o.to(out_dtype), (ht if output_final_state else None)


def chunk_gated_delta_rule_ref(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None = None,
    beta: torch.Tensor | None = None,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    use_qk_l2norm_in_kernel: bool = False,
    chunk_size: int = 64,
    state_dtype: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Chunked WY/UT form of the same operator.  Per chunk of C tokens, with
    gamma = cumsum(g) inside the chunk and S0 the state at chunk start:

        A_ij = beta_i exp(gamma_i - gamma_j) (k_i . k_j)   for i > j, else 0
        T    = (I + A)^-1
        W    = T diag(beta exp(gamma)) K          U = T diag(beta) V
        V~   = U - W S0
        O    = diag(exp(gamma)) Q S0 + tril(Q K^T * exp(gamma_i - gamma_j)) V~
        S_C  = exp(gamma_C) S0 + (diag(exp(gamma_C - gamma)) K)^T V~

    Chunks never cross sequence boundaries; the last chunk of a sequence may be short.
    """
    out_dtype = v.dtype
    B, T, H, K = q.shape
    V = v.size(-1)
    dt = state_dtype
    q, k, v, g, beta = _prepare(q, k, v, g, beta, scale, use_qk_l2norm_in_kernel, dt)
    ranges = _sequence_ranges(B, T, cu_seqlens)
    N = len(ranges)

    o = torch.zeros(B, T, H, V, dtype=dt)
    ht = torch.zeros(N, H, K, V, dtype=dt)

    for n, (b, t0, t1) in enumerate(ranges):
        S = torch.zeros(H, K, V, dtype=dt) if initial_state is None else initial_state[n].to(dt).clone()
        for c0 in range(t0, t1, chunk_size):
            c1 = min(c0 + chunk_size, t1)
            C = c1 - c0
            # [H, C, *]
            qc = q[b, c0:c1].transpose(0, 1)
            kc = k[b, c0:c1].transpose(0, 1)
            vc = v[b, c0:c1].transpose(0, 1)
            bc = beta[b, c0:c1].transpose(0, 1)
            gam = g[b, c0:c1].transpose(0, 1).cumsum(dim=-1)

            diff = gam[:, :, None] - gam[:, None, :]  # gamma_i - gamma_j
            strict = torch.ones(C, C, dtype=torch.bool).tril(-1)
            incl = torch.ones(C, C, dtype=torch.bool).tril(0)
            decay_strict = torch.where(strict, diff, torch.zeros_like(diff)).exp() * strict
            decay_incl = torch.where(incl, diff, torch.zeros_like(diff)).exp() * incl

            A = bc[:, :, None] * decay_strict * (kc @ kc.transpose(-1, -2))
            eye = torch.eye(C, dtype=dt).expand(H, C, C)
            Tm = torch.linalg.solve_triangular(eye + A, eye, upper=False)

            W = Tm @ (kc * (bc * gam.exp())[:, :, None])
            U = Tm @ (vc * bc[:, :, None])
            Vn = U - W @ S
            P = decay_incl * (qc @ kc.transpose(-1, -2))
            oc = (qc * gam.exp()[:, :, None]) @ S + P @ Vn
            o[b, c0:c1] = oc.transpose(0, 1)

            gl = gam[:, -1]
            kd = kc * (gl[:, None] - gam).exp()[:, :, None]
            S = gl.exp()[:, None, None] * S + kd.transpose(-1, -2) @ Vn
        ht[n] = S

    return o.to(out_dtype), (ht if output_final_state else None)


def decode_step_single_pass_ref(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    state: torch.Tensor,
    scale: float | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """One token per sequence, written as the single read + single write of the state
    that a streaming decode kernel performs:

        r   = beta (v - e^g S^T k)
        S'  = e^g S + k (outer) r
        o   = e^g (S^T q) + (k . q) r

    q, k: [N, H, K]   v: [N, H, V]   g, beta: [N, H]   state: [N, H, K, V].
    Algebraically identical to one step of recurrent_gated_delta_rule_ref."""
    dt = state.dtype
    K = q.size(-1)
    scale = K**-0.5 if scale is None else scale
    q, k, v = q.to(dt) * scale, k.to(dt), v.to(dt)
    eg = g.to(dt).exp()[..., None]
    Sk = torch.einsum("nhkv,nhk->nhv", state, k)
    Sq = torch.einsum("nhkv,nhk->nhv", state, q)
    r = beta.to(dt)[..., None] * (v - eg * Sk)
    new_state = eg[..., None] * state + k[..., :, None] * r[..., None, :]
    o = eg * Sq + (k * q).sum(-1, keepdim=True) * r
    return o, new_state
