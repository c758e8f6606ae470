"""Backward of the gated delta rule, chunk by chunk, batched over every chain and chunk.

The reference trains through ``chunk_gated_delta_rule`` (chunk mode is asserted while training,
lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:194-209), so autograd needs
the gradients of ``(o, final_state)`` with respect to ``(q, k, v, g, beta, initial_state)``.

Three ways through, same formulas:

* bf16, K = 64, 128 or 256, V a multiple of 64 (whole rows, packed or left-padded batches): four kernel launches
  (``_backward_on_kernels``) - ``gdn_chunk_bwd_prepare``, ``gdn_chunk_fwd_saving`` for the forward sweep and
  again over the mirror problem for the reverse sweep, ``gdn_chunk_bwd_local``;
* other bf16 shapes (V a multiple of 32 only): the two sweeps over the chunks of a chain on the scan kernel
  (``gdn_chunk_fwd_saving``: the forward's scan in a variant that also writes the chunk states and V~),
  everything chunk-local as batched library GEMMs (fp32, ``torch.bmm``) and elementwise torch operations on
  sequences padded to whole chunks;
* fp32 inputs, CPU tensors: the sweeps as loops of batched GEMMs as well.

The reverse sweep is the same recurrence as the forward one on other data, which is how it gets onto
that kernel: with the tokens of a chain in reverse order (a transposed lower-triangular matrix is
lower-triangular again), chunk c becomes two chunks of a "mirror" problem,

    A:  v := P^T dO,  k := k,  T' := T^T,  row scales -(Kd's) and -(Kb's)       =>  V~ = Y = T^T dV~,
        state: exp(gamma_C) dS1 - Kb^T Y
    B:  v := dO,      k := q,  T' := I,    row scale Qe's, no decay             =>  state += Qe^T dO

whose rows and records ``gdn_chunk_bwd_prepare`` writes (``_mirror_problem`` on the second way); the states
the scan saves at the A chunks are dS1, its output there is Y.

Chunk-local quantities (C = 64 tokens, gamma = prefix sum of g inside the chunk, e = exp(gamma),
E_ij = exp(gamma_i - gamma_j) for j <= i):

    A  = stril(diag(beta) (K K^T . E))      T  = (I + A)^-1
    Kb = diag(beta e) K                     Vb = diag(beta) V
    W  = T Kb                               U  = T Vb
    P  = tril(Q K^T . E)                    Qe = diag(e) Q         Kd = diag(exp(gamma_C - gamma)) K

    forward sweep     V~ = U - W S0         S1 = exp(gamma_C) S0 + Kd^T V~        (O = Qe S0 + P V~)
    reverse sweep     dV~ = P^T dO + Kd dS1       Y = T^T dV~
                      dS0 = exp(gamma_C) dS1 + Qe^T dO - Kb^T Y
    chunk-local       dP = tril(dO V~^T)    dQe = dO S0^T    dKd = V~ dS1^T    Z = Y S0^T
                      dA = -stril(Y V~^T)   (the gradients with respect to Kb and Vb are -Z and Y)
"""

from __future__ import annotations

import weakref

import torch


CHUNK = 64
L2NORM_EPS = 1e-6  # the epsilon of the forward kernels' q/k normalisation


# Host copies of the prefixes that backward passes have asked for, by tensor object: a model calls the operator once per
# layer with the same cu_seqlens tensor, and only the first backward of a step should wait for the device.  An entry
# is valid for that very object at that version (in-place writes bump it) and goes when the tensor does.
_HOST_PREFIX: dict[int, tuple] = {}


def _host_prefix(cu_seqlens) -> list[int]:
    key = id(cu_seqlens)
    hit = _HOST_PREFIX.get(key)
    if hit is not None and hit[0]() is cu_seqlens and hit[1] == cu_seqlens._version:
        return hit[2]
    values = cu_seqlens.detach().to("cpu", torch.int64).tolist()
    _HOST_PREFIX[key] = (weakref.ref(cu_seqlens, lambda _, key=key: _HOST_PREFIX.pop(key, None)), cu_seqlens._version, values)
    return values


def _chains(B, T, cu_seqlens, left_padded):
    """Start (in the flattened [B * T] token axis) and length of every sequence."""
    if cu_seqlens is None:
        return [b * T for b in range(B)], [T] * B
    # The layout of the packed gradients depends on the longest sequence, so the prefix has to come to the host
    # (one copy of N + 1 integers, once per cu_seqlens tensor).  It is checked here, where it is visible: the forward
    # kernels clamp a malformed prefix, the index arithmetic below would not.
    cu = _host_prefix(cu_seqlens)
    limit = B * T if left_padded else T
    if cu[0] != 0 or any(cu[n + 1] < cu[n] for n in range(len(cu) - 1)) or cu[-1] > limit:
        raise ValueError(f"cu_seqlens must start at 0, be non-decreasing and end at or below {limit}, got {cu}")
    lens = [cu[n + 1] - cu[n] for n in range(len(cu) - 1)]
    if left_padded and max(lens) > T:
        raise ValueError(f"a left-padded row holds at most T = {T} tokens, got lengths {lens}")
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
        self.shape = (B, T)
        # whole chunks, one sequence per row: packing is a change of layout, no gather
        self.aligned = cu_seqlens is None and T % CHUNK == 0
        Tp = self.NC * CHUNK
        t = torch.arange(Tp, device=device)
        lens_t = torch.tensor(lens, device=device)
        self.valid = t[None, :] < lens_t[:, None]  # [N, Tp]
        if not self.aligned:
            index = torch.tensor(starts, device=device)[:, None] + t[None, :]
            self.index = torch.where(self.valid, index, torch.zeros_like(index))

    def pack(self, x):
        """[B, T, H, *D] -> fp32 [N * H, NC, C, *D], zero at the padding."""
        tail = x.shape[3:]
        if self.aligned:
            y = x.reshape(self.N, self.NC, CHUNK, self.H, *tail).movedim(3, 1)
            return y.to(torch.float32, memory_format=torch.contiguous_format).reshape(self.N * self.H, self.NC, CHUNK, *tail)
        flat = x.reshape(x.shape[0] * x.shape[1], self.H, *tail)
        y = flat[self.index].to(torch.float32)  # [N, Tp, H, *D]
        y = y * self.valid.reshape(self.N, -1, 1, *([1] * len(tail)))
        y = y.reshape(self.N, self.NC, CHUNK, self.H, *tail)
        return y.movedim(3, 1).reshape(self.N * self.H, self.NC, CHUNK, *tail)

    def unpack(self, y, dtype):
        """fp32 [N * H, NC, C, *D] -> [B, T, H, *D] in ``dtype``, zero where no sequence lives."""
        tail = y.shape[3:]
        B, T = self.shape
        y = y.reshape(self.N, self.H, self.NC, CHUNK, *tail).movedim(1, 3)
        if self.aligned:
            return y.to(dtype, memory_format=torch.contiguous_format).reshape(B, T, self.H, *tail)
        y = y.reshape(self.N, -1, self.H, *tail)
        out = torch.zeros(B * T, self.H, *tail, dtype=dtype, device=y.device)
        out[self.index[self.valid]] = y[self.valid].to(dtype)
        return out.reshape(B, T, self.H, *tail)


def _l2norm(x):
    r = torch.rsqrt(x.square().sum(dim=-1, keepdim=True) + L2NORM_EPS)
    return x * r, r


def _l2norm_grad(y, r, dy):
    # y = x r, r = (|x|^2 + eps)^-1/2  =>  dx = r (dy - y <y, dy>)
    return r * (dy - y * (y * dy).sum(dim=-1, keepdim=True))


def _sweeps_as_gemm_loops(S_init, dS_init, egl, Kd, Qe, Kb, Tm, Vb, P, doc):
    """Both sweeps as loops of batched GEMMs (any dtype, any K).  Returns S0, V~, dS1, Y, dS0 of chunk 0."""
    Bt, NC = egl.shape
    K, V = S_init.shape[-2:]
    dev = egl.device
    W, U, Tt = Tm @ Kb, Tm @ Vb, Tm.transpose(-1, -2)
    S = S_init.clone()
    S0 = torch.empty(Bt, NC, K, V, device=dev)
    Vn = torch.empty(Bt, NC, CHUNK, V, device=dev)
    for c in range(NC):
        S0[:, c] = S
        Vn[:, c] = U[:, c] - W[:, c] @ S
        S = egl[:, c, None, None] * S + Kd[:, c].transpose(-1, -2) @ Vn[:, c]
    dS = dS_init.clone()
    dS1 = torch.empty(Bt, NC, K, V, device=dev)
    Y = torch.empty(Bt, NC, CHUNK, V, device=dev)
    for c in reversed(range(NC)):
        dS1[:, c] = dS
        Y[:, c] = Tt[:, c] @ (P[:, c].transpose(-1, -2) @ doc[:, c] + Kd[:, c] @ dS)
        dS = (egl[:, c, None, None] * dS + Qe[:, c].transpose(-1, -2) @ doc[:, c]
              - Kb[:, c].transpose(-1, -2) @ Y[:, c])  # fmt: skip
    return S0, Vn, dS1, Y, dS


_FRAGMENT_INDEX = {}


def _fragment_index(device, half_slices=False):
    """Where the entries of a lower-triangular 64 x 64 matrix sit in its six MFMA operand fragments of a chunk
    record (the layouts the prepare kernel writes for T diag(beta) and for P).

    For the 32x32x16 MFMA (K <= 128): fragment f < 2 covers rows 0..31 and columns 16 f .. 16 f + 15, fragment
    f >= 2 rows 32..63 and columns 16 (f - 2) ..; lane l = l32 + 32 h holds, of row 32 (f >= 2) + l32, the columns
    16 s + 4 h + 0..3 and 16 s + 8 + 4 h + 0..3.

    For the 16x16x32 MFMA of the half-slice scan (``half_slices``, K = 256): the fragments are the non-zero blocks
    of 16 rows x 32 columns - row tiles 0, 1 (column slab 0), then row tiles 2 and 3 with slabs 0 and 1 each; lane
    l = l16 + 16 g holds, of row 16 tile + l16, the columns 32 s + 4 g + 0..3 and 32 s + 16 + 4 g + 0..3."""
    key = (device, half_slices)
    if key not in _FRAGMENT_INDEX:
        f = torch.arange(6).view(6, 1, 1)
        lane = torch.arange(64).view(1, 64, 1)
        e = torch.arange(8).view(1, 1, 8)
        if half_slices:
            tile = torch.where(f < 2, f, 2 + (f - 2) // 2)
            slab = torch.where(f < 2, torch.zeros_like(f), f % 2)
            rows = (16 * tile + lane % 16).expand(6, 64, 8)
            cols = 32 * slab + 4 * (lane // 16) + torch.where(e < 4, e, e + 12)
        else:
            tile = (f >= 2).long()
            slab = torch.where(f < 2, f, f - 2)
            rows = (32 * tile + lane % 32).expand(6, 64, 8)
            cols = 16 * slab + 4 * (lane // 32) + torch.where(e < 4, e, e + 4)
        _FRAGMENT_INDEX[key] = (rows.to(device), cols.to(device))
    return _FRAGMENT_INDEX[key]


RECORD_BYTES = 13312  # a chunk record: 12 fragments, 3 x 64 row scales, e^{gamma_C}


def _mirror_problem(N, H, kraw, qraw, doc, Tm, P, egl, cs_a, ks_a, ks_b, aligned_inputs=None, half_slices=False):
    """Tensors and chunk records of the reverse sweep as a forward scan (see the module docstring).

    Inputs are packed [N * H, NC, C, ...] fp32; ``cs_a``, ``ks_a``, ``ks_b`` are the row scales of the A and
    B chunks in forward token order.  ``aligned_inputs`` = the caller's ``(q, k, do)`` when they are whole
    chunks with one sequence per row (the mirrored rows are then taken from them directly).  Returns k, v
    ``[N, 2 NC C, H, D]`` bf16 and the records as a uint8 tensor ``[H, N * 2 NC, RECORD_BYTES]``."""
    Bt, NC = egl.shape
    dev = egl.device
    K, V = kraw.size(-1), doc.size(-1)
    bf = torch.bfloat16

    def mirrored(a_rows, b_rows):  # [Bt, NC, C, D] x 2 -> [N, 2 NC C, H, D]: chunks and tokens reversed, A before B
        x = torch.stack((a_rows.to(bf), b_rows.to(bf)), dim=2).flip(1, 3)  # [Bt, NC, 2, C, D]
        D = x.size(-1)
        return x.reshape(N, H, 2 * NC * CHUNK, D).transpose(1, 2).contiguous()

    U_bar = P.transpose(-1, -2) @ doc
    if aligned_inputs is None:
        k_m = mirrored(kraw, qraw)
        v_m = mirrored(U_bar, doc)
    else:
        # reversing the token axis of [N, T, H, D] reverses the chunks and the tokens inside them at once
        q, k, do = (x.to(bf).flip(1).view(N, NC, CHUNK, H, -1) for x in aligned_inputs)
        k_m = torch.stack((k, q), dim=2).view(N, 2 * NC * CHUNK, H, K)
        v_m = torch.empty(N, NC, 2, CHUNK, H, V, dtype=bf, device=dev)
        v_m[:, :, 0] = U_bar.view(N, H, NC, CHUNK, V).flip(2, 3).permute(0, 2, 3, 1, 4)
        v_m[:, :, 1] = do
        v_m = v_m.view(N, 2 * NC * CHUNK, H, V)

    rows, cols = _fragment_index(dev, half_slices=half_slices)
    eye = torch.eye(CHUNK, device=dev)
    # T^T with rows and columns reversed is lower-triangular again: entry (i', j') is T[63 - j', 63 - i']
    Tmir = Tm.transpose(-1, -2).flip(-1, -2)
    frag_t = Tmir[..., rows, cols].to(bf).reshape(N, H, NC, 6 * 512)
    frag_i = eye[rows, cols].to(bf).reshape(6 * 512)

    def by_head(x):  # [N * H, NC, ...] in forward chunk order -> [H, N, NC, ...] in mirror order
        return x.reshape(N, H, NC, *x.shape[2:]).flip(2).transpose(0, 1)

    rec = torch.zeros(H, N, NC, 2, RECORD_BYTES // 2, dtype=bf, device=dev)
    rec[:, :, :, 0, :3072] = frag_t.flip(2).transpose(0, 1)  # A: T' := mirrored T^T
    rec[:, :, :, 0, 3072:6144] = frag_i                      #    P  := I, so that the output of the chunk is Y
    rec[:, :, :, 1, :3072] = frag_i                          # B: T' := I; P stays 0
    scal = rec.view(torch.float32)  # [H, N, NC, 2, 3328]: row scales of q | of k (update) | of k S0 | e^{gamma_C}
    base = 6144 // 2
    scal[:, :, :, 0, base + 64 : base + 128] = by_head(ks_a).flip(-1)
    scal[:, :, :, 0, base + 128 : base + 192] = by_head(cs_a).flip(-1)
    scal[:, :, :, 0, base + 192] = by_head(egl)
    scal[:, :, :, 1, base + 64 : base + 128] = by_head(ks_b).flip(-1)
    scal[:, :, :, 1, base + 192] = 1.0
    return k_m, v_m, rec.view(torch.uint8).reshape(H, N * NC * 2, RECORD_BYTES)


def _sweeps_on_scan_kernel(q, k, v, do, g, beta, scale, initial_state, cu_seqlens, l2norm, left_padded, pk, dht,
                           kraw, qraw, doc, Tm, P, egl, cs_a, ks_a, ks_b):  # fmt: skip
    """Both sweeps on the HIP scan kernel.  Returns S0, V~, dS1, Y, dS0 of chunk 0 (packed, fp32)."""
    from . import ops  # late: ops imports this module

    N, H, NC = pk.N, pk.H, pk.NC
    Bt = N * H
    K, V = q.size(-1), v.size(-1)
    dev = q.device
    alloc = torch.empty if pk.aligned else torch.zeros  # chains shorter than NC chunks leave entries unwritten
    S0 = alloc(Bt, NC, K, V, device=dev)
    Vn = alloc(Bt, NC, CHUNK, V, device=dev)
    ops.chunk_forward_saving(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, left_padded, S0, Vn, NC)
    live = pk.valid.reshape(N, 1, NC, CHUNK, 1).expand(N, H, NC, CHUNK, 1).reshape(Bt, NC, CHUNK, 1)
    Vn = torch.where(live, Vn, torch.zeros_like(Vn))  # rows past the end of a sequence hold whatever the kernel left

    # K = 256 scans on half-slice waves only; smaller heads do when every slice gets a CU
    half_slices = K > 128 or ops.half_slice_records_pay(Bt, V, dev)
    k_m, v_m, rec = _mirror_problem(N, H, kraw, qraw, doc, Tm, P, egl, cs_a, ks_a, ks_b,
                                    aligned_inputs=(q, k, do) if pk.aligned else None, half_slices=half_slices)  # fmt: skip
    dS1 = torch.empty(Bt, NC, K, V, device=dev)
    dht32 = None if dht is None else dht.to(torch.float32).contiguous()
    # the A chunks are the even ones; mirror chunk 2 r is chunk NC - 1 - r of the forward order
    o_m, dS = ops.chunk_scan_given_records(k_m, v_m, rec, dht32, dS1, NC, save_every=2, save_reverse=True,
                                           half_slice_records=half_slices)  # fmt: skip
    # the A chunks' output, back in forward order: [N, NC, 2, C, H, V] -> [Bt, NC, C, V]
    Y = o_m.view(N, NC, 2, CHUNK, H, V)[:, :, 0].flip(1, 2).permute(0, 3, 1, 2, 4).reshape(Bt, NC, CHUNK, V).float()
    return S0, Vn, dS1, Y, dS.reshape(Bt, K, V)


def _kernels_apply(K, V):
    from . import ops  # late: ops imports this module

    return ops.backward_kernels_apply(K, V)


def _chunk_local_grads(qs, kn, vc, doc, Y, Vn, S0, dS1, gam, bc):
    """The chunk-local gradients with batched GEMMs and elementwise torch operations (any shape, any device):
    what ``gdn_chunk_bwd_local`` computes in one kernel.  Packed fp32 tensors in; returns the gradients with
    respect to qs and kn, dbeta, and the gradient with respect to gamma (before the reverse prefix sum)."""
    dev = qs.device
    incl = torch.ones(CHUNK, CHUNK, dtype=torch.bool, device=dev).tril(0)
    strict = incl.tril(-1)
    e = gam.exp()
    gl = gam[..., -1]
    egl = gl.exp()
    tail = (gl[..., None] - gam).exp()
    diff = gam[..., :, None] - gam[..., None, :]
    E = torch.where(incl, diff, torch.zeros_like(diff)).exp() * incl
    kT = kn.transpose(-1, -2)
    KK = kn @ kT
    A = bc[..., None] * E * KK * strict
    P = E * (qs @ kT)
    Kb = kn * (bc * e)[..., None]
    Qe = qs * e[..., None]
    Kd = kn * tail[..., None]

    S0t = S0.transpose(-1, -2)
    VnT = Vn.transpose(-1, -2)
    dP = (doc @ VnT) * incl
    dQe = doc @ S0t
    dKd = Vn @ dS1.transpose(-1, -2)
    Z = Y @ S0t          # the gradient with respect to Kb is -Z, the one with respect to Vb is Y
    dA = -(Y @ VnT) * strict

    G = dP * E
    Hm = dA * bc[..., None] * E
    dqs = torch.baddbmm((dQe * e[..., None]).flatten(0, 1), G.flatten(0, 1), kn.flatten(0, 1)).view_as(dQe)
    dkn = (dKd * tail[..., None]).addcmul_(Z, (bc * e)[..., None], value=-1.0).flatten(0, 1)
    dkn = dkn.baddbmm_(G.transpose(-1, -2).flatten(0, 1), qs.flatten(0, 1))
    dkn = dkn.baddbmm_((Hm + Hm.transpose(-1, -2)).flatten(0, 1), kn.flatten(0, 1)).view_as(dKd)
    dbc = -(Z * kn * e[..., None]).sum(-1) + (Y * vc).sum(-1) + (dA * E * KK).sum(-1)
    MP = dP * P
    MA = dA * A
    n_kd = (dKd * Kd).sum(-1)
    dgam = MP.sum(-1) - MP.sum(-2) + (dQe * Qe).sum(-1) - n_kd - (Z * Kb).sum(-1) + MA.sum(-1) - MA.sum(-2)
    dgam[..., -1] += egl * (dS1 * S0).sum(dim=(-1, -2)) + n_kd.sum(-1)
    return dqs, dkn, dbc, dgam


def _backward_on_kernels(q, k, v, g, beta, do, dht, scale, initial_state, l2norm, cu_seqlens, left_padded):
    """The whole backward on four kernel launches (bf16; K = 64, 128 or 256; V a multiple of 64): ``gdn_chunk_bwd_prepare``
    (per-chunk scalars, the mirror problem, and for whole-chunk batches the forward sweep's records), the saving
    forward sweep, the saving scan over the mirror problem (reverse sweep), ``gdn_chunk_bwd_local`` writing the
    gradients in the caller's layout.  Chunk states, V~ and Y pass between them as bf16 where the saving scan stages
    its saves through LDS.  Packed and left-padded batches are laid out with the chunk count of their longest
    sequence and run one more launch (their forward sweep prepares its own records)."""
    from . import ops  # late: ops imports this module

    B, T, H, K = q.shape
    V = v.size(-1)
    dev = q.device
    if cu_seqlens is None and T % CHUNK == 0:
        N, NC, sequences = B, T // CHUNK, None
    else:
        starts, lens = _chains(B, T, cu_seqlens, left_padded)
        N, NC = len(lens), max(1, -(-max(lens + [1]) // CHUNK))
        as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
        sequences = (as_i32(starts), as_i32(lens), NC)
    Bt = N * H
    q, k, v, do = (x if x.stride(-1) == 1 else x.contiguous() for x in (q, k, v, do.to(torch.bfloat16)))
    # (ragged batches: a row of the mirror problem is scanned over the two chunks per chunk of ITS sequence, which lie at
    # the row's end, not over those of the longest one; the small tensors that say so are made here, ahead of the launches)
    mirror_lengths = None
    if sequences is not None:
        mirror_lengths = ops.left_padded_rows([2 * CHUNK * max(1, -(-length // CHUNK)) for length in lens], 2 * NC * CHUNK, dev)
    # The sweeps run on the half-slice scan, one 32-column slice per workgroup, whatever the number of chains: it is the
    # variant that stages its saves through LDS (bf16, whole lines) and scans without output, which outweighs the records
    # that four slices per workgroup would share (measured with 2 to 6 workgroups per CU: 1.35 against 2.17 ms at twice
    # configuration 1's batch, 3.17 against 4.29 ms at B = 12, V = 256).
    half_slices = True
    # Where the mirror scan stages its saves through LDS, Y and the gradients of the chunks' final states leave as bf16
    # (the chunk-local products round them to that anyway; their part in dg, <dS1, S0>, moved by less than its third
    # digit in every test), and where it is the scan without output it reads the caller's q, k and dO backwards itself
    # instead of reversed copies of them (whole-chunk batches).
    staged_m = ops.saving_scan_is_staged(N, 2 * NC * CHUNK, H, K, V, None, False, 2 if half_slices else 1, dev,
                                         states_dtype=torch.bfloat16, save_every=2)  # fmt: skip
    mirror_reads = staged_m and K >= 128 and sequences is None
    # a batch of whole chunks gets the forward sweep's records from the same kernel: no prepare launch of its own
    prep = ops.chunk_bwd_prepare(q, k, do, g, beta, scale, l2norm, V, sequences, half_slice_records=half_slices,
                                 forward_records=sequences is None, reversed_copies=not mirror_reads,
                                 skip_empty_chunks=True)  # fmt: skip
    # Where the saving scan stages its saves through LDS, the sweeps write S0, V~ and Y as bf16 (what the chunk-local
    # products round them to anyway) and form no output; elsewhere fp32 saves and Y from the mirror scan's output.
    given = 0 if sequences is not None else 2 if half_slices else 1
    staged = ops.saving_scan_is_staged(N, T, H, K, V, cu_seqlens, left_padded, given, dev)
    # where both sweeps stage their saves, what a scan workgroup saves of a chunk lies in one piece (by 32-column slice)
    sliced = staged and staged_m
    saves = dict(dtype=torch.bfloat16 if staged else torch.float32, device=dev)
    S0 = torch.empty(Bt, NC, K, V, **saves)
    Vn = torch.empty(Bt, NC, CHUNK, V, **saves)
    if sequences is None:
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        ops.chunk_scan_given_records(k, v, prep["records_fwd"], h0, S0, NC, half_slice_records=half_slices, v_new=Vn,
                                     no_output=True, q=q, sliced=sliced)  # fmt: skip
    else:
        ops.chunk_forward_saving(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, left_padded, S0, Vn, NC,
                                 no_output=True, sliced=sliced)  # fmt: skip
    dht32 = None if dht is None else dht.to(torch.float32).contiguous()
    dS1 = torch.empty(Bt, NC, K, V, device=dev, dtype=torch.bfloat16 if staged_m else torch.float32)
    Y = torch.empty(Bt, NC, CHUNK, V, dtype=torch.bfloat16, device=dev) if staged_m else None
    o_m, dS = ops.chunk_scan_given_records(k if mirror_reads else prep["k_mirror"], prep["v_mirror"], prep["records"],
                                           dht32, dS1, NC, save_every=2, save_reverse=True,
                                           half_slice_records=half_slices, v_new=Y, no_output=staged_m,
                                           mirror_odd=(q, do) if mirror_reads else None, sliced=sliced,
                                           valid_lengths=mirror_lengths)  # fmt: skip
    dq, dk, dv, dg, dbeta = ops.chunk_local_grads(q, k, v, do, prep, Y if staged_m else o_m, Vn, S0, dS1, scale, l2norm,
                                                  sequences, sliced=sliced)  # fmt: skip
    return (
        dq,
        dk,
        dv,
        dg.to(g.dtype) if g is not None else None,
        dbeta.to(beta.dtype) if beta is not None else None,
        dS if initial_state is not None else None,
    )


def gated_delta_rule_backward(
    q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False, left_padded=False,
):  # fmt: skip
    """Gradients of ``sum(o * do) + sum(final_state * dht)``.

    Arguments as for the forward (``g`` or ``beta`` may be None: ungated / beta = 1); ``do`` has the
    shape of ``o``, ``dht`` that of the final state or is None.  Returns
    ``dq, dk, dv, dg, dbeta, dh0`` in the dtypes of the corresponding inputs (fp32 for dh0); entries for
    absent inputs are None."""
    if q.size(2) != v.size(2):
        # Grouped value attention: the backward runs on the expanded heads (what the reference's repeat_interleave hands
        # its operator, gated_deltanet/module.py:175-177) and adds the gradients of a group's copies up.
        group = v.size(2) // q.size(2)
        dq, dk, *rest = gated_delta_rule_backward(
            q.repeat_interleave(group, dim=2), k.repeat_interleave(group, dim=2), v, g, beta, do, dht, scale, initial_state,
            cu_seqlens, use_qk_l2norm_in_kernel, left_padded)  # fmt: skip
        fold = lambda d: d.view(*q.shape[:2], q.size(2), group, q.size(3)).sum(dim=3, dtype=torch.float32).to(d.dtype)  # noqa: E731
        return (fold(dq), fold(dk), *rest)
    B, T, H, K = q.shape
    V = v.size(-1)
    dev = q.device
    scale = K**-0.5 if scale is None else scale
    if q.is_cuda and q.dtype == torch.bfloat16 and _kernels_apply(K, V):
        return _backward_on_kernels(q, k, v, g, beta, do, dht, scale, initial_state, use_qk_l2norm_in_kernel,
                                    cu_seqlens, left_padded)  # fmt: skip
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
        rq = rk = torch.ones(Bt, NC, CHUNK, 1, device=dev)
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
    P = E * (qs @ kT)

    on_kernel = q.is_cuda and q.dtype == torch.bfloat16 and K in (64, 128, 256) and V % 32 == 0
    if on_kernel:
        # the scan reads the raw rows of k and q; their norms and e^{gamma} go into the row scales
        S0, Vn, dS1, Y, dS = _sweeps_on_scan_kernel(
            q, k, v, do, g, beta, scale, initial_state, cu_seqlens, use_qk_l2norm_in_kernel, left_padded, pk, dht,
            kc, qc, doc, Tm, P, egl,
            cs_a=-(tail * rk[..., 0]), ks_a=-(bc * e * rk[..., 0]), ks_b=e * rq[..., 0] * scale,
        )  # fmt: skip
    else:
        S_init = torch.zeros(Bt, K, V, device=dev)
        if initial_state is not None:
            S_init = initial_state.to(torch.float32).reshape(Bt, K, V)
        dS_init = torch.zeros(Bt, K, V, device=dev) if dht is None else dht.to(torch.float32).reshape(Bt, K, V)
        S0, Vn, dS1, Y, dS = _sweeps_as_gemm_loops(
            S_init, dS_init, egl, kn * tail[..., None], qs * e[..., None], kn * (bc * e)[..., None], Tm,
            vc * bc[..., None], P, doc,
        )  # fmt: skip
    dh0 = dS.reshape(N, H, K, V) if initial_state is not None else None

    dqs, dkn, dbc, dgam = _chunk_local_grads(qs, kn, vc, doc, Y, Vn, S0, dS1, gam, bc)
    dqn = dqs * scale
    if use_qk_l2norm_in_kernel:
        dqc, dkc = _l2norm_grad(qn, rq, dqn), _l2norm_grad(kn, rk, dkn)
    else:
        dqc, dkc = dqn, dkn
    dvc = Y * bc[..., None]
    dgc = dgam.flip(-1).cumsum(-1).flip(-1)
    return (
        pk.unpack(dqc, q.dtype),
        pk.unpack(dkc, k.dtype),
        pk.unpack(dvc, v.dtype),
        pk.unpack(dgc, g.dtype) if g is not None else None,
        pk.unpack(dbc, beta.dtype) if beta is not None else None,
        dh0,
    )
