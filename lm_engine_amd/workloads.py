"""Seeded synthetic inputs for the five benchmark configurations of the gated delta rule.

Tensors are drawn on the CPU in fp32 from ``torch.Generator().manual_seed(1234 + index)`` in
the fixed order q, k, v, b, g_raw, h0, (sequence lengths), then rounded to the configured
dtype.  A CPU checker that consumes these (rounded) tensors sees bit-identical inputs to the
GPU path.  Shapes follow the operator contract at the reference call site
lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:168-222:
q, k ``[B, T, H, K]``, v ``[B, T, H, V]``, g fp32 ``[B, T, H]`` (log-decay <= 0),
beta ``[B, T, H]``, initial_state fp32 ``[N, H, K, V]``, cu_seqlens int32 ``[N + 1]``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace

import torch
import torch.nn.functional as F


@dataclass(frozen=True)
class Workload:
    name: str
    index: int
    B: int
    T: int
    H: int
    K: int
    V: int
    dtype: torch.dtype
    gated: bool
    g_mean: float = 0.0
    g_std: float = 0.0
    random_h0: bool = False
    varlen: bool = False
    min_len: int = 128
    max_len: int = 8192
    decode: bool = False


WORKLOADS: tuple[Workload, ...] = (
    Workload("cfg0_ungated_recurrent_fp32", 0, B=1, T=256, H=2, K=64, V=64, dtype=torch.float32, gated=False),
    Workload("cfg1_chunk_fwd_bf16", 1, B=4, T=4096, H=16, K=128, V=128, dtype=torch.bfloat16, gated=True,
             g_mean=3.0, g_std=1.0),
    Workload("cfg2_varlen_bf16", 2, B=1, T=32768, H=16, K=128, V=128, dtype=torch.bfloat16, gated=True,
             g_mean=3.0, g_std=1.0, random_h0=True, varlen=True),
    Workload("cfg3_decode_bf16", 3, B=256, T=1, H=32, K=128, V=128, dtype=torch.bfloat16, gated=True,
             g_mean=3.0, g_std=1.0, random_h0=True, decode=True),
    Workload("cfg4_long_context_bf16", 4, B=1, T=65536, H=32, K=128, V=256, dtype=torch.bfloat16, gated=True,
             g_mean=4.0, g_std=0.5, random_h0=True),
)  # fmt: skip


def get_workload(index: int, **overrides) -> Workload:
    """Configuration ``index`` (0-4); keyword overrides (e.g. ``T=512``) give a smaller case of
    the same distribution and seed."""
    w = WORKLOADS[index]
    return replace(w, **overrides) if overrides else w


def draw_sequence_lengths(total: int, min_len: int, max_len: int, generator: torch.Generator) -> list[int]:
    """Lengths uniform in [min_len, max_len] drawn until the running total reaches ``total``;
    the last one is clipped to land exactly on ``total`` and merged into its predecessor if the
    clipped remainder is shorter than min_len."""
    lengths: list[int] = []
    running = 0
    while running < total:
        length = int(torch.randint(min_len, max_len + 1, (1,), generator=generator).item())
        length = min(length, total - running)
        lengths.append(length)
        running += length
    if len(lengths) > 1 and lengths[-1] < min_len:
        last = lengths.pop()
        lengths[-1] += last
    return lengths


def make_inputs(w: Workload, device: str | torch.device = "cpu") -> dict:
    """Returns dict(q, k, v, g, beta, initial_state, cu_seqlens, scale) for workload ``w``."""
    gen = torch.Generator("cpu").manual_seed(1234 + w.index)
    B, T, H, K, V = w.B, w.T, w.H, w.K, w.V

    q = F.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1)
    k = F.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1)
    v = torch.randn(B, T, H, V, generator=gen)
    beta = torch.randn(B, T, H, generator=gen).sigmoid()
    g_raw = torch.randn(B, T, H, generator=gen)
    g = F.logsigmoid(w.g_mean + w.g_std * g_raw) if w.gated else None

    cu_seqlens = None
    N = B
    if w.varlen:
        # h0 is drawn after the lengths are known (its shape depends on N) but from the same stream
        lengths = draw_sequence_lengths(T, min(w.min_len, T), min(w.max_len, T), gen)
        N = len(lengths)
        cu_seqlens = torch.tensor([0] + lengths, dtype=torch.int64).cumsum(0).to(torch.int32)

    h0 = 0.02 * torch.randn(N, H, K, V, generator=gen) if w.random_h0 else None

    out = dict(
        q=q.to(w.dtype),
        k=k.to(w.dtype),
        v=v.to(w.dtype),
        g=g,
        beta=beta.to(w.dtype),
        initial_state=h0,
        cu_seqlens=cu_seqlens,
        scale=K**-0.5,
    )
    return {
        name: (x.to(device) if isinstance(x, torch.Tensor) else x) for name, x in out.items()
    }


# ---------------------------------------------------------------------------------------
# algorithmic work (numerators of the roofline figures)
# ---------------------------------------------------------------------------------------

CHUNK = 64


def chunk_fwd_flops_per_token_head(K: int, V: int, C: int = CHUNK) -> dict:
    """Dense count of the contractions of the chunked forward as the kernels run it, per token and head:
    K K^T, Q K^T                                   -> "prepare" = 2 C (2K)
    K S0, Q S0, K^T V~ (K x V each), T' X, P V~    -> "scan"    = 2 (3 K V + 2 C V)
    with V~ = T diag(beta) (V - diag(cs) K S0): the product T (beta e^gamma K) of the WY form (2 C K) is never
    formed.  "wy" is the count of the WY form's eight contractions, 2 (C (3K + 2V) + 3 K V), for comparison with
    figures quoted on that count.  Triangular solve and all elementwise work are excluded; padding is never
    counted.  "strict" halves the products with a triangular factor."""
    prepare = 2 * C * (2 * K)
    scan = 2 * (3 * K * V + 2 * C * V)
    strict = 2 * ((C // 2) * (2 * K + 2 * V) + 3 * K * V)
    wy = 2 * (C * (3 * K + 2 * V) + 3 * K * V)
    return {"prepare": prepare, "scan": scan, "dense": prepare + scan, "strict": strict, "wy": wy}


def chunk_fwd_bytes_per_token_head(K: int, V: int, in_bytes: int = 2) -> int:
    """q + k + v + o in the activation dtype, g fp32, beta in the activation dtype."""
    return (2 * K + 2 * V) * in_bytes + 4 + in_bytes


def decode_bytes_per_seq_head(K: int, V: int, in_bytes: int = 2) -> int:
    """fp32 state read + write, q, k, v in and o out in the activation dtype, g fp32, beta."""
    return 2 * 4 * K * V + (2 * K + 2 * V) * in_bytes + 4 + in_bytes
