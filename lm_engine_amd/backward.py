"""Backward of the gated delta rule, chunk by chunk, batched over every chain and chunk.

The reference trains through ``chunk_gated_delta_rule`` (chunk mode is asserted while training,
lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:194-209), so autograd needs
the gradients of ``(o, final_state)`` with respect to ``(q, k, v, g, beta, initial_state)``.

This is the first, functional version: the per-chunk products are batched library GEMMs (fp32,
``torch.bmm`` on the tensors' device) and the two sweeps over the chunks of a chain - forward to
rebuild the chunk states, backward to carry the state gradient - are loops of such GEMMs.  It keeps
the shape a fused kernel pipeline has (a state-saving forward scan, a reverse scan, one chunk-local
gradient kernel); those kernels replace the corresponding blocks below one at a time.

Chunk-local quantities (C = 64 tokens, gamma = prefix sum of g inside the chunk, e = exp(gamma),
E_ij = exp(gamma_i - gamma_j) for j <= i):

    A  = stril(diag(beta) (K K^T . E))      T  = (I + A)^-1
    Kb = diag(beta e) K                     Vb = diag(beta) V
    W  = T Kb                               U  = T Vb
    P  = tril(Q K^T . E)                    Qe = diag(e) Q         Kd = diag(exp(gamma_C - gamma)) K

    forward sweep     V~ = U - W S0         S1 = exp(gamma_C) S0 + Kd^T V~        (O = Qe S0 + P V~)
    reverse sweep     dV~ = P^T dO + Kd dS1
                      dS0 = exp(gamma_C) dS1 + Qe^T dO - W^T dV~
"""

from __future__ import annotations

import torch


CHUNK = 64
L2NORM_EPS = 1e-6  # the epsilon of the forward kernels' q/k normalisation


def _chains(B, T, cu_seqlens, left_padded):
    """Start (in the flattened [B * T] token axis) and length of every sequence."""
    if cu_seqlens is None:
        return [b * T for b in range(B)], [T] * B
    cu = cu_seqlens.detach().to("cpu", torch.int64).tolist()
    lens = [cu[n + 1] - cu[n] for n in range(len(cu) - 1)]
    if left_padded:
        return [b * T + T - lens[b] for b in range(B)], lens
    return cu[:-1], lens


class _Packing:
    """Moves between the caller's [B, T, H, D] layout and [chains * H, chunks, C, D], sequences padded
    to whole chunks.  A padding token has k = q = v = 0, beta = 0 and g = 0: it leaves the state and
    every gradient of the real tokens untouched."""

    def __init__(self, B, T, H, cu_seqlens, left_padded, device):
        starts, lens = _chains(B, T, cu_seqlens, left_padded)
        self.N, self.H = len(lens), H
        self.NC = max(1, -(-max(lens + [1]) // CHUNK))
        Tp = self.NC * CHUNK
        t = torch.arange(Tp, device=device)
        lens_t = torch.tensor(lens, device=device)
        self.valid = t[None, :] < lens_t[:, None]  # [N, Tp]
        index = torch.tensor(starts, device=device)[:, None] + t[None, :]
        self.index = torch.where(self.valid, index, torch.zeros_like(index))
        self.shape = (B, T)

    def pack(self, x):
        """[B, T, H, *D] -> fp32 [N * H, NC, C, *D], zero at the padding."""
        tail = x.shape[3:]
        flat = x.reshape(x.shape[0] * x.shape[1], self.H, *tail)
        y = flat[self.index].to(torch.float32)  # [N, Tp, H, *D]
        y = y * self.valid.reshape(self.N, -1, 1, *([1] * len(tail)))
        y = y.reshape(self.N, self.NC, CHUNK, self.H, *tail)
        return y.movedim(3, 1).reshape(self.N * self.H, self.NC, CHUNK, *tail)

    def unpack(self, y, dtype):
        """fp32 [N * H, NC, C, *D] -> [B, T, H, *D] in ``dtype``, zero where no sequence lives."""
        tail = y.shape[3:]
        B, T = self.shape
        y = y.reshape(self.N, self.H, self.NC, CHUNK, *tail).movedim(1, 3).reshape(self.N, -1, self.H, *tail)
        out = torch.zeros(B * T, self.H, *tail, dtype=dtype, device=y.device)
        out[self.index[self.valid]] = y[self.valid].to(dtype)
        return out.reshape(B, T, self.H, *tail)


def _l2norm(x):
    r = torch.rsqrt(x.square().sum(dim=-1, keepdim=True) + L2NORM_EPS)
    return x * r, r


def _l2norm_grad(y, r, dy):
    # y = x r, r = (|x|^2 + eps)^-1/2  =>  dx = r (dy - y <y, dy>)
    return r * (dy - y * (y * dy).sum(dim=-1, keepdim=True))


def gated_delta_rule_backward(
    q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False, left_padded=False,
):  # fmt: skip
    """Gradients of ``sum(o * do) + sum(final_state * dht)``.

    Arguments as for the forward (``g`` or ``beta`` may be None: ungated / beta = 1); ``do`` has the
    shape of ``o``, ``dht`` that of the final state or is None.  Returns
    ``dq, dk, dv, dg, dbeta, dh0`` in the dtypes of the corresponding inputs (fp32 for dh0); entries for
    absent inputs are None."""
    B, T, H, K = q.shape
    V = v.size(-1)
    dev = q.device
    scale = K**-0.5 if scale is None else scale
    pk = _Packing(B, T, H, cu_seqlens, left_padded, dev)
    N, NC, Bt = pk.N, pk.NC, pk.N * H

    qc, kc, vc, doc = pk.pack(q), pk.pack(k), pk.pack(v), pk.pack(do)
    gc = pk.pack(g) if g is not None else torch.zeros(Bt, NC, CHUNK, device=dev)
    if beta is not None:
        bc = pk.pack(beta)
    else:  # beta = 1 on the real tokens, 0 on the padding
        bc = pk.pack(torch.ones(B, T, H, device=dev))
    if use_qk_l2norm_in_kernel:
        qn, rq = _l2norm(qc)
        kn, rk = _l2norm(kc)
    else:
        qn, kn = qc, kc
    qs = qn * scale

    incl = torch.ones(CHUNK, CHUNK, dtype=torch.bool, device=dev).tril(0)
    strict = incl.tril(-1)
    eye = torch.eye(CHUNK, device=dev)

    gam = gc.cumsum(dim=-1)  # [Bt, NC, C]
    e = gam.exp()
    gl = gam[..., -1]  # [Bt, NC]
    egl = gl.exp()
    tail = (gl[..., None] - gam).exp()
    diff = gam[..., :, None] - gam[..., None, :]
    E = torch.where(incl, diff, torch.zeros_like(diff)).exp() * incl
    kT = kn.transpose(-1, -2)
    KK = kn @ kT
    A = bc[..., None] * E * KK * strict
    Tm = torch.linalg.solve_triangular(eye + A, eye.expand_as(A), upper=False)
    Tt = Tm.transpose(-1, -2)
    Kb = kn * (bc * e)[..., None]
    Vb = vc * bc[..., None]
    W = Tm @ Kb
    U = Tm @ Vb
    P = E * (qs @ kT)
    Qe = qs * e[..., None]
    Kd = kn * tail[..., None]

    # forward sweep: the state every chunk starts from, and V~
    S = torch.zeros(Bt, K, V, device=dev)
    if initial_state is not None:
        S = initial_state.to(torch.float32).reshape(Bt, K, V).clone()
    S0 = torch.empty(Bt, NC, K, V, device=dev)
    Vn = torch.empty(Bt, NC, CHUNK, V, device=dev)
    for c in range(NC):
        S0[:, c] = S
        Vn[:, c] = U[:, c] - W[:, c] @ S
        S = egl[:, c, None, None] * S + Kd[:, c].transpose(-1, -2) @ Vn[:, c]

    # reverse sweep: the gradient of the state every chunk ends with, and dV~
    dS = torch.zeros(Bt, K, V, device=dev) if dht is None else dht.to(torch.float32).reshape(Bt, K, V).clone()
    dS1 = torch.empty(Bt, NC, K, V, device=dev)
    dVn = torch.empty(Bt, NC, CHUNK, V, device=dev)
    for c in reversed(range(NC)):
        dS1[:, c] = dS
        dVn[:, c] = P[:, c].transpose(-1, -2) @ doc[:, c] + Kd[:, c] @ dS
        dS = (egl[:, c, None, None] * dS + Qe[:, c].transpose(-1, -2) @ doc[:, c]
              - W[:, c].transpose(-1, -2) @ dVn[:, c])  # fmt: skip
    dh0 = dS.reshape(N, H, K, V) if initial_state is not None else None

    # chunk-local gradients, all chunks at once
    S0t = S0.transpose(-1, -2)
    dP = (doc @ Vn.transpose(-1, -2)) * incl
    dQe = doc @ S0t
    dKd = Vn @ dS1.transpose(-1, -2)
    dW = -(dVn @ S0t)
    dKb = Tt @ dW
    dVb = Tt @ dVn
    dA = -(Tt @ (dW @ Kb.transpose(-1, -2) + dVn @ Vb.transpose(-1, -2)) @ Tt) * strict

    G = dP * E
    Hm = dA * bc[..., None] * E
    dqs = G @ kn + dQe * e[..., None]
    dkn = (G.transpose(-1, -2) @ qs + dKd * tail[..., None] + dKb * (bc * e)[..., None]
           + (Hm + Hm.transpose(-1, -2)) @ kn)  # fmt: skip
    dvc = dVb * bc[..., None]
    dbc = (dKb * kn * e[..., None]).sum(-1) + (dVb * vc).sum(-1) + (dA * E * KK).sum(-1)
    MP = dP * P
    MA = dA * A
    n_kd = (dKd * Kd).sum(-1)
    dgam = MP.sum(-1) - MP.sum(-2) + (dQe * Qe).sum(-1) - n_kd + (dKb * Kb).sum(-1) + MA.sum(-1) - MA.sum(-2)
    dgam[..., -1] += egl * (dS1 * S0).sum(dim=(-1, -2)) + n_kd.sum(-1)
    dgc = dgam.flip(-1).cumsum(-1).flip(-1)

    dqn = dqs * scale
    if use_qk_l2norm_in_kernel:
        dqc, dkc = _l2norm_grad(qn, rq, dqn), _l2norm_grad(kn, rk, dkn)
    else:
        dqc, dkc = dqn, dkn
    return (
        pk.unpack(dqc, q.dtype),
        pk.unpack(dkc, k.dtype),
        pk.unpack(dvc, v.dtype),
        pk.unpack(dgc, g.dtype) if g is not None else None,
        pk.unpack(dbc, beta.dtype) if beta is not None else None,
        dh0,
    )
