"""ctypes binding of oracle/gdn_oracle.c (TEST INFRASTRUCTURE ONLY, see that file's header).

The C restatement runs the same token loop as ``recurrent_gated_delta_rule_ref`` with
OpenMP over the independent (sequence, head) recurrences, so parity can be checked at the
full benchmark sizes in seconds."""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch


_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgdn_oracle.so")
_lib = None


def build_c_oracle() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "libgdn_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build_c_oracle()
        lib = ctypes.CDLL(_LIB_PATH)
        fp = ctypes.c_void_p
        lib.gdn_oracle_recurrent.argtypes = [fp] * 9 + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_int, ctypes.c_int]
        lib.gdn_oracle_recurrent.restype = ctypes.c_int
        _lib = lib
    return _lib


def recurrent_gated_delta_rule_c(
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
    f64_state: bool = True,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Same contract as oracle.recurrent_gated_delta_rule_ref; inputs of any float dtype are
    upcast to fp32 (exact for bf16), the state is carried in fp64 (default) or fp32."""
    lib = _load()
    B, T, H, K = q.shape
    V = v.size(-1)
    f32 = lambda x: None if x is None else x.detach().to("cpu", torch.float32).contiguous()  # noqa: E731
    qf, kf, vf, gf, bf, h0 = f32(q), f32(k), f32(v), f32(g), f32(beta), f32(initial_state)
    cu = None if cu_seqlens is None else cu_seqlens.detach().to("cpu", torch.int32).contiguous()
    N = B if cu is None else cu.numel() - 1
    o = torch.empty(B, T, H, V, dtype=torch.float32)
    ht = torch.empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
    ptr = lambda x: None if x is None else ctypes.c_void_p(x.data_ptr())  # noqa: E731
    rc = lib.gdn_oracle_recurrent(
        ptr(qf), ptr(kf), ptr(vf), ptr(gf), ptr(bf), ptr(h0), ptr(o), ptr(ht), ptr(cu),
        B, T, H, K, V, N, float(K**-0.5 if scale is None else scale), int(use_qk_l2norm_in_kernel), int(f64_state),
    )  # fmt: skip
    if rc != 0:
        raise RuntimeError(f"gdn_oracle_recurrent failed with code {rc}")
    return o, ht
