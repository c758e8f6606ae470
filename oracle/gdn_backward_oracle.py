"""CPU restatement of the gradients of the gated delta rule (torch, fp64 by default).

TEST INFRASTRUCTURE ONLY: the shipped package never imports this file.

The reference trains through ``fla``'s ``chunk_gated_delta_rule`` (chunk mode is asserted while
training, lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:194-209), so the
quantities a backward pass of this operator has to return are the gradients of
(o, final_state) with respect to (q, k, v, g, beta, initial_state).  ``fla`` itself is absent
from the reference tree (PARITY UNPINNED at that boundary, as for the forward); the two functions
here are pinned against each other and against what the mathematics fixes:

* ``gated_delta_rule_grads_autograd`` differentiates the token loop of
  ``recurrent_gated_delta_rule_ref`` with torch.autograd in fp64; the tests check it against
  central finite differences of that loop.
* ``chunk_gated_delta_rule_bwd_ref`` states the same gradients in closed form, chunk by chunk, in
  the shape a chunked backward kernel computes them (a reverse scan over the chunks carrying dS,
  then per-chunk products); the tests check it against the autograd result.
"""

from __future__ import annotations

import torch

from .gdn_oracle import L2NORM_EPS, _sequence_ranges, recurrent_gated_delta_rule_ref


def gated_delta_rule_grads_autograd(
    q,
    k,
    v,
    g,
    beta,
    do,
    dht=None,
    scale=None,
    initial_state=None,
    cu_seqlens=None,
    use_qk_l2norm_in_kernel=False,
    dtype=torch.float64,
):
    """Gradients of sum(o * do) + sum(final_state * dht) by autograd through the token loop.

    Returns dq, dk, dv, dg, dbeta, dh0 (dh0 is None without an initial state)."""
    leaves = [x.detach().to(dtype).requires_grad_(True) for x in (q, k, v, g, beta)]
    h0 = None if initial_state is None else initial_state.detach().to(dtype).requires_grad_(True)
    o, ht = recurrent_gated_delta_rule_ref(
        *leaves,
        scale=scale,
        initial_state=h0,
        output_final_state=True,
        cu_seqlens=cu_seqlens,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel,
        state_dtype=dtype,
    )
    loss = (o * do.to(dtype)).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(dtype)).sum()
    inputs = leaves + ([h0] if h0 is not None else [])
    grads = torch.autograd.grad(loss, inputs)
    dh0 = grads[5] if h0 is not None else None
    return (*grads[:5], dh0)


def _l2norm_fwd(x):
    r = torch.rsqrt(x.square().sum(dim=-1, keepdim=True) + L2NORM_EPS)
    return x * r, r


def _l2norm_bwd(y, r, dy):
    """y = x r with r = (|x|^2 + eps)^-1/2:  dx = r (dy - y (y . dy))."""
    return r * (dy - y * (y * dy).sum(dim=-1, keepdim=True))


def chunk_gated_delta_rule_bwd_ref(
    q,
    k,
    v,
    g,
    beta,
    do,
    dht=None,
    scale=None,
    initial_state=None,
    cu_seqlens=None,
    use_qk_l2norm_in_kernel=False,
    chunk_size=64,
    dtype=torch.float64,
):
    """Closed-form chunked backward.  Per chunk, with the forward quantities of
    ``chunk_gated_delta_rule_ref`` (e = exp(gamma), E_ij = exp(gamma_i - gamma_j),
    Kb = diag(beta e) K, Vb = diag(beta) V, Qe = diag(e) Q, Kd = diag(exp(gamma_C - gamma)) K):

        reverse scan over the chunks (dS1 = gradient of the state after the chunk):
            dV~ = P^T dO + Kd dS1
            dS0 = exp(gamma_C) dS1 + Qe^T dO - W^T dV~
        per chunk, given S0, dS1, V~, dV~:
            dP  = tril(dO V~^T)          dQe = dO S0^T         dKd = V~ dS1^T
            dW  = -dV~ S0^T              dU  = dV~
            dKb = T^T dW                 dVb = T^T dU
            dA  = -stril(T^T (dW Kb^T + dU Vb^T) T^T)
            dQ  = (dP . E) K + diag(e) dQe
            dK  = (dP . E)^T Q + diag(exp(gamma_C - gamma)) dKd + diag(beta e) dKb
                  + (H + H^T) K                      with H = dA . diag(beta) E
            dV  = diag(beta) dVb
            dbeta_i  = rowsum(dKb . diag(e) K)_i + rowsum(dVb . V)_i + rowsum(dA . E . K K^T)_i
            dgamma   = rowsum(dP . P) - colsum(dP . P) + rowsum(dQe . Qe) - rowsum(dKd . Kd)
                       + rowsum(dKb . Kb) + rowsum(dA . A) - colsum(dA . A)
            dgamma_C = exp(gamma_C) <dS1, S0> + sum(dKd . Kd)        (added to the chunk's last token)
            dg_t     = sum_{i >= t} dgamma_i                           (reverse cumsum inside the chunk)

    Returns dq, dk, dv, dg, dbeta, dh0."""
    dt = dtype
    B, T, H, K = q.shape
    V = v.size(-1)
    scale = K**-0.5 if scale is None else scale
    q, k, v, g, beta, do = (x.to(dt) for x in (q, k, v, g, beta, do))
    if use_qk_l2norm_in_kernel:
        qn, rq = _l2norm_fwd(q)
        kn, rk = _l2norm_fwd(k)
    else:
        qn, kn = q, k
    qs = qn * scale

    ranges = _sequence_ranges(B, T, cu_seqlens)
    dqs = torch.zeros_like(q)
    dkn = torch.zeros_like(k)
    dv = torch.zeros_like(v)
    dg = torch.zeros_like(g)
    dbeta = torch.zeros_like(beta)
    dh0 = None if initial_state is None else torch.zeros(len(ranges), H, K, V, dtype=dt)

    for n, (b, t0, t1) in enumerate(ranges):
        # forward pass over the chunks, keeping what the backward needs
        S = torch.zeros(H, K, V, dtype=dt) if initial_state is None else initial_state[n].to(dt).clone()
        saved = []
        for c0 in range(t0, t1, chunk_size):
            c1 = min(c0 + chunk_size, t1)
            C = c1 - c0
            qc, kc, vc = (x[b, c0:c1].transpose(0, 1) for x in (qs, kn, v))
            bc = beta[b, c0:c1].transpose(0, 1)
            gam = g[b, c0:c1].transpose(0, 1).cumsum(dim=-1)
            diff = gam[:, :, None] - gam[:, None, :]
            incl = torch.ones(C, C, dtype=torch.bool).tril(0)
            strict = torch.ones(C, C, dtype=torch.bool).tril(-1)
            E = torch.where(incl, diff, torch.zeros_like(diff)).exp() * incl  # zero above the diagonal
            e = gam.exp()
            KK = kc @ kc.transpose(-1, -2)
            A = bc[:, :, None] * E * KK * strict
            eye = torch.eye(C, dtype=dt).expand(H, C, C)
            Tm = torch.linalg.solve_triangular(eye + A, eye, upper=False)
            Kb = kc * (bc * e)[:, :, None]
            Vb = vc * bc[:, :, None]
            W = Tm @ Kb
            U = Tm @ Vb
            Vn = U - W @ S
            P = E * (qc @ kc.transpose(-1, -2))
            Qe = qc * e[:, :, None]
            gl = gam[:, -1]
            Kd = kc * (gl[:, None] - gam).exp()[:, :, None]
            saved.append((c0, c1, S, qc, kc, vc, bc, gam, e, E, incl, strict, KK, A, Tm, Kb, Vb, W, Vn, P, Qe, Kd, gl))
            S = gl.exp()[:, None, None] * S + Kd.transpose(-1, -2) @ Vn

        dS = torch.zeros(H, K, V, dtype=dt) if dht is None else dht[n].to(dt).clone()
        for c0, c1, S0, qc, kc, vc, bc, gam, e, E, incl, strict, KK, A, Tm, Kb, Vb, W, Vn, P, Qe, Kd, gl in reversed(saved):
            doc = do[b, c0:c1].transpose(0, 1)
            dVn = P.transpose(-1, -2) @ doc + Kd @ dS
            dS0 = gl.exp()[:, None, None] * dS + Qe.transpose(-1, -2) @ doc - W.transpose(-1, -2) @ dVn

            dP = (doc @ Vn.transpose(-1, -2)) * incl
            dQe = doc @ S0.transpose(-1, -2)
            dKd = Vn @ dS.transpose(-1, -2)
            dW = -dVn @ S0.transpose(-1, -2)
            dU = dVn
            Tt = Tm.transpose(-1, -2)
            dKb = Tt @ dW
            dVb = Tt @ dU
            dA = -(Tt @ (dW @ Kb.transpose(-1, -2) + dU @ Vb.transpose(-1, -2)) @ Tt) * strict

            G = dP * E
            Hm = dA * bc[:, :, None] * E
            dq_c = G @ kc + dQe * e[:, :, None]
            dk_c = (
                G.transpose(-1, -2) @ qc
                + dKd * (gl[:, None] - gam).exp()[:, :, None]
                + dKb * (bc * e)[:, :, None]
                + (Hm + Hm.transpose(-1, -2)) @ kc
            )
            dv_c = dVb * bc[:, :, None]
            dbeta_c = (dKb * kc * e[:, :, None]).sum(-1) + (dVb * vc).sum(-1) + (dA * E * KK).sum(-1)
            MP = dP * P
            MA = dA * A
            n_kd = (dKd * Kd).sum(-1)
            dgam = MP.sum(-1) - MP.sum(-2) + (dQe * Qe).sum(-1) - n_kd + (dKb * Kb).sum(-1) + MA.sum(-1) - MA.sum(-2)
            dgam[:, -1] += gl.exp() * (dS * S0).sum(dim=(-1, -2)) + n_kd.sum(-1)
            dg_c = dgam.flip(-1).cumsum(-1).flip(-1)

            dqs[b, c0:c1] = dq_c.transpose(0, 1)
            dkn[b, c0:c1] = dk_c.transpose(0, 1)
            dv[b, c0:c1] = dv_c.transpose(0, 1)
            dbeta[b, c0:c1] = dbeta_c.transpose(0, 1)
            dg[b, c0:c1] = dg_c.transpose(0, 1)
            dS = dS0
        if dh0 is not None:
            dh0[n] = dS

    dqn = dqs * scale
    if use_qk_l2norm_in_kernel:
        dq = _l2norm_bwd(qn, rq, dqn)
        dk = _l2norm_bwd(kn, rk, dkn)
    else:
        dq, dk = dqn, dkn
    return dq, dk, dv, dg, dbeta, dh0
