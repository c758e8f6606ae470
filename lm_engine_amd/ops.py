"""The gated delta-rule operator behind the signature the reference layer calls.

The reference's ``GatedDeltaNet.forward`` makes exactly two calls on this path
(lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:197-222), both with
the keywords ``q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
use_qk_l2norm_in_kernel`` and both returning ``(o, final_state)``:

* ``chunk_gated_delta_rule``            for sequences longer than 64 tokens (training, prefill)
* ``fused_recurrent_gated_delta_rule``  otherwise, in particular the one-token decode step

Both are provided here with the same names, argument meaning and return convention, on top
of the HIP library (``libgdn_hip.so``, C ABI in include/gdn_hip.h).  PyTorch only owns the
device memory and the stream; there is no eager or CPU fallback: without the library every
call raises.  Both are differentiable (``backward.py``).

    q, k            [B, T, H, K]   bf16 (or fp32), last dim contiguous
    v               [B, T, H, V]
    g               [B, T, H]      fp32 log-decay (<= 0); None = ungated
    beta            [B, T, H]      None = 1
    initial_state   [N, H, K, V]   fp32; N = B, or number of packed sequences
    cu_seqlens      [N + 1]        int32 with leading 0 (then B must be 1)
    returns  o [B, T, H, V] in v.dtype, final_state [N, H, K, V] fp32 or None
"""

from __future__ import annotations

import ctypes
import threading
from collections import OrderedDict

import torch

from . import _lib
from .backward import gated_delta_rule_backward
from .kernels import Kernel, is_kernel_allowed


RECURRENT_MAX_TOKENS = 64  # the reference's mode switch, gated_deltanet/module.py:193

_SUPPORTED_K = (64, 128, 256)


def _dtype_code(dtype: torch.dtype, what: str) -> int:
    if dtype == torch.bfloat16:
        return _lib.GDN_BF16
    if dtype == torch.float32:
        return _lib.GDN_F32
    raise ValueError(f"{what} must be bfloat16 or float32, got {dtype}")


def _require_hip_path() -> None:
    if not is_kernel_allowed(Kernel.gated_delta_rule):
        raise RuntimeError(
            "Kernel.gated_delta_rule is disabled and this package ships no other implementation of the "
            "gated delta rule; enable it (it is on by default) with lm_engine_amd.kernels.enable_kernels"
        )


def _last_dim_contiguous(x: torch.Tensor) -> torch.Tensor:
    return x if x.stride(-1) == 1 else x.contiguous()


def _check_inputs(q, k, v, g, beta, initial_state, cu_seqlens, left_padded=False):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [B, T, H, D] tensors")
    B, T, HQK, K = q.shape
    H, V = v.size(2), v.size(-1)
    if k.shape != q.shape:
        raise ValueError(f"k {tuple(k.shape)} must have the shape of q {tuple(q.shape)}")
    if v.shape[:2] != q.shape[:2]:
        raise ValueError(f"v {tuple(v.shape)} must share [B, T] with q {tuple(q.shape)}")
    if H % HQK != 0:  # grouped value attention: H / HQK consecutive value heads share a head of q and k
        raise ValueError(f"the heads of v ({H}) must be a multiple of the heads of q and k ({HQK})")
    if not q.is_cuda:
        raise ValueError("the gated delta rule runs on the GPU only; inputs must be device tensors")
    for name, x in (("k", k), ("v", v), ("g", g), ("beta", beta), ("initial_state", initial_state),
                    ("cu_seqlens", cu_seqlens)):  # fmt: skip
        if x is not None and x.device != q.device:
            raise ValueError(f"{name} is on {x.device}, q is on {q.device}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError(f"q, k, v must share a dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
    if K not in _SUPPORTED_K:
        raise ValueError(f"head dim K={K} is not supported (supported: {_SUPPORTED_K})")
    if V % 32 != 0:
        raise ValueError(f"value head dim V={V} must be a multiple of 32")
    for name, x in (("g", g), ("beta", beta)):
        if x is not None and tuple(x.shape) != (B, T, H):
            raise ValueError(f"{name} must be [B, T, H] = {(B, T, H)}, got {tuple(x.shape)}")
    if left_padded:
        if cu_seqlens is None or cu_seqlens.dim() != 1 or cu_seqlens.numel() != B + 1:
            raise ValueError(f"left_padded needs cu_seqlens [B + 1] = [{B + 1}]: the prefix sums of the valid lengths")
        N = B
    elif cu_seqlens is not None:
        if B != 1:
            raise ValueError(f"with cu_seqlens the batch dim must be 1 (tokens packed along T), got B={B}")
        if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
            raise ValueError("cu_seqlens must be a 1-D tensor [N + 1]")
        N = cu_seqlens.numel() - 1
    else:
        N = B
    if initial_state is not None:
        if tuple(initial_state.shape) != (N, H, K, V):
            raise ValueError(f"initial_state must be [N, H, K, V] = {(N, H, K, V)}, got {tuple(initial_state.shape)}")
        if initial_state.dtype != torch.float32:
            raise ValueError(f"initial_state must be float32, got {initial_state.dtype}")
    return B, T, H, K, V, N


def _fill_args(q, k, v, g, beta, h0, ht, o, cu_seqlens, scale, l2norm, inplace, dims, left_padded=False) -> _lib.GdnArgs:
    B, T, H, K, V, N = dims
    a = _lib.GdnArgs()
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    a.beta = None if beta is None else beta.data_ptr()
    a.g = None if g is None else g.data_ptr()
    a.h0 = None if h0 is None else h0.data_ptr()
    a.ht = None if ht is None else ht.data_ptr()
    a.cu_seqlens = None if cu_seqlens is None else cu_seqlens.data_ptr()
    a.workspace, a.workspace_bytes = None, 0
    for name, x in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, f"{name}_stride_b", x.stride(0))
        setattr(a, f"{name}_stride_t", x.stride(1))
        setattr(a, f"{name}_stride_h", x.stride(2))
    a.B, a.T, a.H, a.K, a.V, a.N = B, T, H, K, V, N
    a.qk_heads = 0 if q.size(2) == H else q.size(2)
    a.chunk = 64
    a.dtype = _dtype_code(q.dtype, "q, k, v")
    a.beta_dtype = _lib.GDN_F32 if beta is None else _dtype_code(beta.dtype, "beta")
    a.flags = ((_lib.GDN_FLAG_L2NORM if l2norm else 0) | (_lib.GDN_FLAG_STATE_INPLACE if inplace else 0)
               | (_lib.GDN_FLAG_LEFT_PADDED if left_padded else 0)
               | (_lib.GDN_FLAG_FUSED_LAUNCH if is_kernel_allowed(Kernel.gated_delta_rule_fused_launch) else 0))  # fmt: skip
    a.scale = float(K**-0.5 if scale is None else scale)
    return a


# Workspaces of the one-launch chunked forward, kept between calls: one per (device, stream, shape), its header
# (chunk offsets, error latch, ready flags) zero-filled when it is made.  The library then need not clear the ready flags
# before every call (it leaves them clear itself, GDN_FLAG_READY_FLAGS_CLEAR), and a step of that shape no longer asks
# the allocator for tens of megabytes.  Only shapes that run as one launch keep a workspace: every other call (packed
# or left-padded batches, K = 256, shapes outside the window) reads no flag and takes a fresh torch.empty workspace
# from the caching allocator, whatever T it comes with.  Calls on one stream run in order, so they can share a
# workspace; another stream gets its own.  The least recently used entries go when there are more than
# _WORKSPACE_LIMIT of them or they hold more than _WORKSPACE_BYTES_LIMIT together; release_workspaces() drops them
# all.  The dict is guarded by a lock: forward passes on several Python threads (one stream each) may interleave.
_WORKSPACES: "OrderedDict[tuple, torch.Tensor]" = OrderedDict()
_WORKSPACE_LIMIT = 8
_WORKSPACE_BYTES_LIMIT = 1 << 30
_WORKSPACES_LOCK = threading.Lock()

# One pinned int32 per device that the one-launch forward sets when a scan workgroup gave up waiting for a record
# (gdn_args::error_word).  The host reads it without synchronising, before every chunked forward on that device: a
# failure of an earlier call surfaces at the next one, the way asynchronous device errors do.
_ERROR_WORDS: dict[int, torch.Tensor] = {}


def release_workspaces() -> None:
    """Frees the workspaces that ``chunk_gated_delta_rule`` keeps between calls."""
    with _WORKSPACES_LOCK:
        _WORKSPACES.clear()


def _error_word(device) -> torch.Tensor:
    word = _ERROR_WORDS.get(device.index)
    if word is None:
        word = torch.zeros(1, dtype=torch.int32).pin_memory()
        _ERROR_WORDS[device.index] = word
    return word


def _raise_if_forward_failed(device) -> torch.Tensor:
    """The error word of ``device``; raises when an earlier one-launch forward on it reported a time-out (the kept
    workspaces of that device are dropped: their ready flags are in no defined state)."""
    word = _error_word(device)
    if int(word[0]) != 0:
        word.zero_()
        with _WORKSPACES_LOCK:
            for key in [k for k in _WORKSPACES if k[0] == device.index]:
                del _WORKSPACES[key]
        raise RuntimeError(
            "an earlier chunk_gated_delta_rule call on this device gave up waiting for its prepare half "
            "(gdn_chunk_fwd, one-launch mode): the outputs of that call are invalid"
        )
    return word


def _kept_workspace(device, stream_handle, dims, nbytes, header_bytes):
    key = (device.index, stream_handle, dims, nbytes)
    with _WORKSPACES_LOCK:
        workspace = _WORKSPACES.get(key)
        if workspace is not None:
            _WORKSPACES.move_to_end(key)
            return key, workspace
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    workspace[:header_bytes].zero_()
    with _WORKSPACES_LOCK:
        _WORKSPACES[key] = workspace
        while len(_WORKSPACES) > _WORKSPACE_LIMIT or (
            len(_WORKSPACES) > 1 and sum(w.numel() for w in _WORKSPACES.values()) > _WORKSPACE_BYTES_LIMIT
        ):
            _WORKSPACES.popitem(last=False)
    return key, workspace


def _drop_workspace(key) -> None:
    with _WORKSPACES_LOCK:
        _WORKSPACES.pop(key, None)


def _chunk_workspace(lib, args, q, dims, stream_handle):
    """Workspace for one ``gdn_chunk_fwd`` call: fills ``args.workspace`` / ``workspace_bytes`` (and the flag that vouches
    for clear ready flags when the workspace is a kept one).  Returns ``(key, tensor)``; ``key`` is None for a
    workspace that is not kept."""
    nbytes = max(int(lib.gdn_workspace_bytes(ctypes.byref(args))), 256)
    # (memory allocated under graph capture belongs to the graph: nothing of it is kept)
    keep = bool(lib.gdn_chunk_fwd_is_one_launch(ctypes.byref(args))) and not torch.cuda.is_current_stream_capturing()
    if keep:
        header = int(lib.gdn_workspace_header_bytes(ctypes.byref(args)))
        key, workspace = _kept_workspace(q.device, stream_handle, dims, nbytes, header)
        args.flags |= _lib.GDN_FLAG_READY_FLAGS_CLEAR
    else:
        key, workspace = None, torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
    return key, workspace


def _run(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm, inplace_state,
         left_padded=False):
    _require_hip_path()
    lib = _lib.load_library()
    dims = _check_inputs(q, k, v, g, beta, initial_state, cu_seqlens, left_padded)
    B, T, H, K, V, N = dims

    q, k, v = _last_dim_contiguous(q), _last_dim_contiguous(k), _last_dim_contiguous(v)
    if g is not None:
        g = g.to(torch.float32).contiguous()
    if beta is not None:
        beta = beta.contiguous() if beta.dtype in (torch.bfloat16, torch.float32) else beta.float().contiguous()
    if cu_seqlens is not None:
        cu_seqlens = cu_seqlens.to(torch.int32).contiguous()
    h0 = None if initial_state is None else initial_state.contiguous()

    # padding positions of a left-padded batch are not written by the kernels: they read as zeros
    o = (torch.zeros if left_padded else torch.empty)(B, T, H, V, dtype=v.dtype, device=v.device)
    ht = None
    if output_final_state:
        if inplace_state:
            if h0 is None or h0.data_ptr() != initial_state.data_ptr():
                raise ValueError("inplace_state needs a contiguous initial_state to update")
            ht = h0
        else:
            ht = torch.empty(N, H, K, V, dtype=torch.float32, device=v.device)

    args = _fill_args(q, k, v, g, beta, h0, ht, o, cu_seqlens, scale, l2norm, inplace_state and ht is not None, dims,
                      left_padded)  # fmt: skip
    stream = ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)

    with torch.cuda.device(q.device):
        if mode == "chunk":
            args.error_word = _raise_if_forward_failed(q.device).data_ptr()
            key, workspace = _chunk_workspace(lib, args, q, dims, stream.value)
            try:
                _lib.check_status(lib.gdn_chunk_fwd(ctypes.byref(args), stream), "gdn_chunk_fwd")
            except Exception:
                _drop_workspace(key)  # a call that failed may have left flags set
                raise
        else:
            _lib.check_status(lib.gdn_recurrent_fwd(ctypes.byref(args), stream), "gdn_recurrent_fwd")
    return o, ht


def fused_launch_applies(q, v, cu_seqlens=None) -> bool:
    """Whether ``chunk_gated_delta_rule`` runs these inputs as one launch (prepare and scan together): the flag
    ``Kernel.gated_delta_rule_fused_launch`` is on and the library's rule holds - bf16, a fixed-length batch, K 64 or
    128, V a multiple of 64, and the scan's workgroups (one per 64 columns of every sequence-head chain, the chains
    rounded up to a multiple of 8) fill between 3/8 and 1/2 of the compute units."""
    if not is_kernel_allowed(Kernel.gated_delta_rule_fused_launch) or cu_seqlens is not None or q.dtype != torch.bfloat16:
        return False
    B, T, _, K = q.shape
    a = _lib.GdnArgs()  # the library decides (gdn_chunk_fwd_is_one_launch): shape fields and flags are all it reads
    a.B, a.T, a.H, a.K, a.V, a.N = B, T, v.size(2), K, v.size(-1), B
    a.chunk, a.dtype, a.flags = 64, _lib.GDN_BF16, _lib.GDN_FLAG_FUSED_LAUNCH
    with torch.cuda.device(q.device):
        return bool(_lib.load_library().gdn_chunk_fwd_is_one_launch(ctypes.byref(a)))


def chunk_forward_kernel_times(
    q, k, v, g=None, beta=None, scale=None, initial_state=None, output_final_state=False, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False,
) -> dict[str, float]:  # fmt: skip
    """Runs the chunked forward once through ``gdn_chunk_fwd_profile`` and returns the duration of
    each of its kernels in milliseconds, measured with HIP events on the launch stream.  Same
    arguments as ``chunk_gated_delta_rule``; blocks until the kernels have finished."""
    _require_hip_path()
    lib = _lib.load_library()
    dims = _check_inputs(q, k, v, g, beta, initial_state, cu_seqlens)
    B, T, H, K, V, N = dims
    q, k, v = _last_dim_contiguous(q), _last_dim_contiguous(k), _last_dim_contiguous(v)
    g = None if g is None else g.to(torch.float32).contiguous()
    beta = None if beta is None else beta.contiguous()
    cu_seqlens = None if cu_seqlens is None else cu_seqlens.to(torch.int32).contiguous()
    h0 = None if initial_state is None else initial_state.contiguous()
    o = torch.empty(B, T, H, V, dtype=v.dtype, device=v.device)
    ht = torch.empty(N, H, K, V, dtype=torch.float32, device=v.device) if output_final_state else None
    args = _fill_args(q, k, v, g, beta, h0, ht, o, cu_seqlens, scale, use_qk_l2norm_in_kernel, False, dims)
    times = (ctypes.c_float * _lib.GDN_CHUNK_KERNELS)()
    with torch.cuda.device(q.device):
        # the same kept workspace, and the same promise about its flags, as the operator itself
        stream = ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
        args.error_word = _raise_if_forward_failed(q.device).data_ptr()
        key, workspace = _chunk_workspace(lib, args, q, dims, stream.value)
        try:
            _lib.check_status(lib.gdn_chunk_fwd_profile(ctypes.byref(args), stream, times), "gdn_chunk_fwd_profile")
        except Exception:
            _drop_workspace(key)
            raise
    return dict(zip(_lib.CHUNK_KERNEL_NAMES, (float(x) for x in times)))


def _save_dtype_code(x, shape, what):
    if x.dtype not in (torch.float32, torch.bfloat16) or not x.is_contiguous() or tuple(x.shape) != shape:
        raise ValueError(f"{what} must be a contiguous fp32 or bf16 tensor of shape {shape}")
    return _dtype_code(x.dtype, what)


def saving_scan_is_staged(N, T, H, K, V, cu_seqlens=None, left_padded=False, records_given=0, device=None,
                          states_dtype=torch.bfloat16, v_new_dtype=torch.bfloat16, save_every=1, no_output=True) -> bool:
    """Whether ``gdn_chunk_fwd_saving`` runs this batch (``N`` sequences; ``T`` tokens per row, or packed tokens with
    ``cu_seqlens``) and these saves (dtype None: not asked for) on the scan that stages its saves through LDS: only
    that one writes bf16 saves (``gdn_chunk_fwd_saving_is_staged``)."""
    a = _lib.GdnArgs()
    packed = cu_seqlens is not None and not left_padded
    a.B, a.T, a.H, a.K, a.V, a.N = (1 if packed else N), T, H, K, V, N
    a.chunk, a.dtype = 64, _lib.GDN_BF16
    a.flags = _lib.GDN_FLAG_LEFT_PADDED if left_padded else 0
    a.cu_seqlens = None if cu_seqlens is None else cu_seqlens.data_ptr()
    code = lambda dtype: _lib.GDN_BF16 if dtype == torch.bfloat16 else _lib.GDN_F32  # noqa: E731
    saves = _lib.GdnChunkSaves(None if states_dtype is None else 1, None if v_new_dtype is None else 1, 1, records_given,
                               save_every, 0, code(states_dtype), code(v_new_dtype), 1 if no_output else 0, 0)  # fmt: skip
    with torch.cuda.device(device):
        return bool(_lib.load_library().gdn_chunk_fwd_saving_is_staged(ctypes.byref(a), ctypes.byref(saves)))


def chunk_forward_saving(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, left_padded, states, v_new,
                         chunks_per_chain, no_output=False, sliced=False):  # fmt: skip
    """The chunked forward once more, for the backward pass: through ``gdn_chunk_fwd_saving`` it writes the
    state every chunk starts from into ``states`` ``[N * H, chunks_per_chain, K, V]`` and V~ into ``v_new``
    ``[N * H, chunks_per_chain, 64, V]`` (contiguous; fp32, or bf16 where ``saving_scan_is_staged``).  The output
    itself is discarded (``no_output``: the library skips forming it where it has a scan without output)."""
    _require_hip_path()
    lib = _lib.load_library()
    dims = _check_inputs(q, k, v, g, beta, initial_state, cu_seqlens, left_padded)
    B, T, H, K, V, N = dims
    q, k, v = _last_dim_contiguous(q), _last_dim_contiguous(k), _last_dim_contiguous(v)
    g = None if g is None else g.to(torch.float32).contiguous()
    if beta is not None:
        beta = beta.contiguous() if beta.dtype in (torch.bfloat16, torch.float32) else beta.float().contiguous()
    cu_seqlens = None if cu_seqlens is None else cu_seqlens.to(torch.int32).contiguous()
    h0 = None if initial_state is None else initial_state.contiguous()
    states_code = _save_dtype_code(states, (N * H, chunks_per_chain, K, V), "states")
    v_new_code = _save_dtype_code(v_new, (N * H, chunks_per_chain, 64, V), "v_new")
    o = torch.empty(B, T, H, V, dtype=v.dtype, device=v.device)
    args = _fill_args(q, k, v, g, beta, h0, None, o, cu_seqlens, scale, l2norm, False, dims, left_padded)
    saves = _lib.GdnChunkSaves(states.data_ptr(), v_new.data_ptr(), chunks_per_chain, 0, 1, 0, states_code, v_new_code,
                               1 if no_output else 0, 0, 1 if sliced else 0)  # fmt: skip
    with torch.cuda.device(q.device):
        nbytes = lib.gdn_workspace_bytes(ctypes.byref(args))
        workspace = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=q.device)
        args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
        stream = ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
        _lib.check_status(lib.gdn_chunk_fwd_saving(ctypes.byref(args), ctypes.byref(saves), stream),
                          "gdn_chunk_fwd_saving")  # fmt: skip


def half_slice_records_pay(chains: int, V: int, device) -> bool:
    """Whether a scan over given records should get them in the fragment order of the half-slice scan (16x16x32
    MFMA): that scan runs one 32-column slice per workgroup, the faster kernel while the slices of all chains
    (``chains`` = sequences x heads) do not outnumber the compute units."""
    return chains * (V // 32) <= torch.cuda.get_device_properties(device).multi_processor_count


def left_padded_rows(valid_lengths, T: int, device):
    """Device tensors for ``chunk_scan_given_records(..., valid_lengths=...)`` from the rows' valid lengths (host integers,
    positive multiples of 64, at most ``T``): the int32 prefix sums ``[B + 1]`` and the rows longest first ``[B]``.  Making
    them is two small host-to-device copies; a caller that scans several times, or wants the copies out of the way of
    its launches, makes them once and passes the pair."""
    if any(int(n) <= 0 or int(n) % 64 != 0 or int(n) > T for n in valid_lengths):
        raise ValueError(f"valid_lengths must be positive multiples of 64 of at most T = {T}")
    sums = [0]
    for length in valid_lengths:
        sums.append(sums[-1] + int(length))
    longest_first = sorted(range(len(valid_lengths)), key=lambda n: (-int(valid_lengths[n]), n))
    return (torch.tensor(sums, dtype=torch.int32, device=device), torch.tensor(longest_first, dtype=torch.int32, device=device))


def chunk_scan_given_records(k, v, records, initial_state, states, chunks_per_chain, save_every=1, save_reverse=False,
                             half_slice_records=False, v_new=None, no_output=False, q=None, mirror_odd=None, sliced=False,
                             valid_lengths=None):
    """The scan kernel alone over a fixed-length batch whose chunk records the caller has written
    (``records`` uint8 ``[H, B * T / 64, record bytes]``, T a multiple of 64); it reads the rows of ``q``, ``k`` and
    ``v`` (without ``q``, ``k`` stands in its place: the records of a mirror problem carry zero row scales for q).  Returns ``(o, final_state)``
    and writes the state that chunk ``c`` starts from, for every ``c`` divisible by ``save_every``, into entry
    ``c / save_every`` of ``states`` ``[B * H, chunks_per_chain, K, V]`` (counted from the end with
    ``save_reverse``), and V~ of those chunks into ``v_new`` ``[B * H, chunks_per_chain, 64, V]`` when that is given.
    ``half_slice_records``: the fragments of the records are in the lane order of the 16x16x32 MFMA (K = 256 needs
    that) instead of the 32x32x16 one.  bf16 save arrays where ``saving_scan_is_staged``; ``no_output``: the caller
    does not need ``o`` (None is returned; the library skips forming it where it has a scan without output).
    ``mirror_odd = (k_odd, v_odd)`` (with ``no_output``, where the scan without output exists): ``k``, ``v`` and these two
    are ``[B, T / 2, H, .]`` tensors that the scan reads backwards, every chunk twice - the even chunks' rows from ``k``
    and ``v``, the odd chunks' from ``k_odd`` and ``v_odd`` (``gdn_chunk_saves.mirror_reads``): the mirror problem of
    ``chunk_bwd_prepare(..., reversed_copies=False)``.  ``sliced`` (bf16 saves where ``saving_scan_is_staged``): the
    save arrays are laid out by 32-column slice, ``[B H, chunks_per_chain, V / 32, K or 64, 32]`` in the memory of the
    arrays given (``gdn_chunk_saves.sliced``), for ``chunk_local_grads(..., sliced=True)``.
    ``valid_lengths`` (``B`` host integers, positive multiples of 64, or what ``left_padded_rows`` made of them; not with ``mirror_odd``): the rows are left-padded - row ``n`` is
    scanned over its last ``valid_lengths[n]`` tokens only, with the records at the slots of those tokens, and a reverse
    save counts a row's entries from its own last saved chunk (entry 0)."""
    _require_hip_path()
    lib = _lib.load_library()
    q = k if q is None else q
    pad_lens = None
    if valid_lengths is not None:
        if mirror_odd is not None:
            raise ValueError("valid_lengths and mirror_odd exclude each other")
        pad_lens, row_order = valid_lengths if isinstance(valid_lengths, tuple) else left_padded_rows(valid_lengths, k.size(1), k.device)
        if pad_lens.numel() != k.size(0) + 1 or row_order.numel() != k.size(0):
            raise ValueError(f"valid_lengths must describe the {k.size(0)} rows of k")
    dims = _check_inputs(q, k, v, None, None, initial_state, pad_lens, pad_lens is not None)
    B, T, H, K, V, N = dims
    q, k, v = _last_dim_contiguous(q), _last_dim_contiguous(k), _last_dim_contiguous(v)
    if mirror_odd is not None:
        k_odd, v_odd = (_last_dim_contiguous(x) for x in mirror_odd)
        if not no_output or k_odd.shape != k.shape or v_odd.shape != v.shape or k_odd.dtype != k.dtype or v_odd.dtype != v.dtype:
            raise ValueError("mirror_odd needs no_output and tensors of the shapes and dtype of k and v")
        T = 2 * T  # the sequence the scan walks
        dims = (B, T, H, K, V, N)
    if T % 64 != 0 or not records.is_contiguous() or records.dtype != torch.uint8 or tuple(records.shape[:2]) != (H, B * T // 64):
        raise ValueError("records must be contiguous uint8 [H, B * T / 64, record bytes] with T a multiple of 64")
    states_code = _save_dtype_code(states, (B * H, chunks_per_chain, K, V), "states")
    v_new_code = _lib.GDN_F32 if v_new is None else _save_dtype_code(v_new, (B * H, chunks_per_chain, 64, V), "v_new")
    o = torch.empty(B, T, H, V, dtype=v.dtype, device=v.device)
    ht = torch.empty(N, H, K, V, dtype=torch.float32, device=v.device)
    args = _fill_args(q, k, v, None, None, initial_state, ht, o, pad_lens, 1.0, False, False, dims, pad_lens is not None)
    args.workspace, args.workspace_bytes = records.data_ptr(), records.numel()
    saves = _lib.GdnChunkSaves(states.data_ptr(), None if v_new is None else v_new.data_ptr(), chunks_per_chain,
                               2 if half_slice_records else 1, save_every, 1 if save_reverse else 0, states_code,
                               v_new_code, 1 if no_output else 0, 0)  # fmt: skip
    saves.sliced = 1 if sliced else 0
    if pad_lens is not None:
        saves.row_order = row_order.data_ptr()
    if mirror_odd is not None:
        saves.mirror_reads, saves.k_odd, saves.v_odd = 1, k_odd.data_ptr(), v_odd.data_ptr()
        saves.k_odd_stride_b, saves.k_odd_stride_t, saves.k_odd_stride_h = k_odd.stride(0), k_odd.stride(1), k_odd.stride(2)
        saves.v_odd_stride_b, saves.v_odd_stride_t, saves.v_odd_stride_h = v_odd.stride(0), v_odd.stride(1), v_odd.stride(2)
    with torch.cuda.device(k.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream(k.device).cuda_stream)
        _lib.check_status(lib.gdn_chunk_fwd_saving(ctypes.byref(args), ctypes.byref(saves), stream),
                          "gdn_chunk_fwd_saving")  # fmt: skip
    return (None if no_output else o), ht


def backward_kernels_apply(K: int, V: int) -> bool:
    """Head dims ``gdn_chunk_bwd_prepare`` and ``gdn_chunk_bwd_local`` are built for."""
    return K in _SUPPORTED_K and V % 64 == 0


def chunk_local_grads(q, k, v, dout, prep, y_mirror, v_new, states, dstates, scale, l2norm, sequences=None, sliced=False):
    """``gdn_chunk_bwd_local``: q, k, v, dout are the caller's bf16 ``[B, T, H, D]`` tensors (last dim contiguous),
    ``prep`` what ``chunk_bwd_prepare`` returned (same ``sequences``), ``y_mirror`` the output of the scan over its
    mirror problem (bf16 ``[N, 2 NC 64, H, V]``) or, as a 4-D tensor, the V~ that scan saved at its even chunks (bf16
    ``[N H, NC, 64, V]``), ``v_new`` and ``states`` what the saving forward sweep wrote (both fp32 or both bf16),
    ``dstates`` the states the mirror scan saved (fp32 or bf16).  Returns ``dq, dk, dv`` bf16 ``[B, T, H, D]`` and ``dg, dbeta`` fp32
    ``[B, T, H]`` (zero where no sequence lives)."""
    _require_hip_path()
    lib = _lib.load_library()
    B, T, H, K = q.shape
    V = v.size(-1)
    Bt, NC, C = prep["gamma"].shape
    N = Bt // H
    dev = y_mirror.device
    y_chunked = tuple(y_mirror.shape) == (Bt, NC, C, V)
    if (sequences is None and (N != B or NC * C != T)) or (not y_chunked and tuple(y_mirror.shape) != (N, 2 * NC * C, H, V)) \
            or y_mirror.dtype != torch.bfloat16 or not y_mirror.is_contiguous():  # fmt: skip
        raise ValueError("y_mirror must be the contiguous bf16 [N, 2 NC 64, H, V] output of the scan over the mirror "
                         "problem or the [N H, NC, 64, V] V~ it saved")
    if not backward_kernels_apply(K, V):
        raise ValueError(f"chunk-local gradients are built for K in {_SUPPORTED_K} and V a multiple of 64, got {K}, {V}")
    if states.dtype != v_new.dtype or states.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("v_new and states must both be fp32 or both be bf16")
    for name, x, shape, dtype in (("v_new", v_new, (Bt, NC, C, V), states.dtype), ("states", states, (Bt, NC, K, V), states.dtype),
                                  ("dstates", dstates, (Bt, NC, K, V), dstates.dtype)):  # fmt: skip
        if tuple(x.shape) != shape or x.dtype != dtype or not x.is_contiguous():
            raise ValueError(f"{name} must be contiguous {dtype} {shape}")
    alloc = torch.empty if sequences is None else torch.zeros  # tokens outside every sequence are not written
    out = dict(
        dq_out=alloc(B, T, H, K, dtype=torch.bfloat16, device=dev),
        dk_out=alloc(B, T, H, K, dtype=torch.bfloat16, device=dev),
        dv_out=alloc(B, T, H, V, dtype=torch.bfloat16, device=dev),
        dg_out=alloc(B, T, H, dtype=torch.float32, device=dev),
        dbeta_out=alloc(B, T, H, dtype=torch.float32, device=dev),
    )
    a = _lib.GdnChunkLocalArgs()
    a.gamma, a.beta = prep["gamma"].data_ptr(), prep["beta"].data_ptr()
    if l2norm:
        a.rq, a.rk = prep["rq"].data_ptr(), prep["rk"].data_ptr()
    a.v_new, a.states, a.dstates = v_new.data_ptr(), states.data_ptr(), dstates.data_ptr()
    a.saves_dtype = _dtype_code(states.dtype, "states")
    a.dstates_dtype = _dtype_code(dstates.dtype, "dstates")
    a.saves_sliced = 1 if sliced else 0  # (the sweeps wrote v_new, states, dstates and the chunked Y by 32-column slice)
    if y_chunked:
        a.y_chunks = y_mirror.data_ptr()
    else:
        a.y_mirror = y_mirror.data_ptr()
    for name, x in (("q", q), ("k", k), ("v", v), ("dout", dout)):
        if x.dtype != torch.bfloat16 or x.stride(-1) != 1:
            raise ValueError(f"{name} must be bf16 with a contiguous last dim")
        setattr(a, f"{name}_raw", x.data_ptr())
        setattr(a, f"{name}_stride_b", x.stride(0))
        setattr(a, f"{name}_stride_t", x.stride(1))
        setattr(a, f"{name}_stride_h", x.stride(2))
    for name, x in out.items():
        setattr(a, name, x.data_ptr())
    a.chunks, a.K, a.V, a.scale, a.H, a.NC = Bt * NC, K, V, float(scale), H, NC
    if sequences is not None:
        a.seq_start, a.seq_len, a.T_rows = sequences[0].data_ptr(), sequences[1].data_ptr(), T
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        _lib.check_status(lib.gdn_chunk_bwd_local(ctypes.byref(a), stream), "gdn_chunk_bwd_local")
    return out["dq_out"], out["dk_out"], out["dv_out"], out["dg_out"], out["dbeta_out"]


RECORD_BYTES = 13312  # a chunk record: 12 operand fragments, 3 x 64 row scales, e^{gamma_C}


def chunk_bwd_prepare(q, k, dout, g, beta, scale, l2norm, V, sequences=None, half_slice_records=False,
                      forward_records=False, reversed_copies=True, skip_empty_chunks=False):
    """``gdn_chunk_bwd_prepare``.  ``q, k, dout`` are the caller's bf16 ``[B, T, H, D]`` tensors; without
    ``sequences`` every row is one sequence of whole chunks, else ``sequences = (seq_start, seq_len, NC)``: int32
    device tensors ``[N]`` (first token as a flat index over the rows, length) and the chunks per sequence to lay
    the results out with.  Returns a dict: ``gamma, beta, rq, rk`` (fp32 ``[N H, NC, 64]``: prefix sums of g inside
    the chunks, beta, inverse norms of the rows of q and k) and the mirror problem ``k_mirror, v_mirror``
    ``[N, 2 NC 64, H, D]`` bf16, ``records`` uint8 ``[H, N * 2 NC, RECORD_BYTES]`` (their fragments in the lane order
    of the 16x16x32 MFMA with ``half_slice_records``, see ``chunk_scan_given_records``).  ``forward_records``
    (whole-chunk batches only): also ``records_fwd`` ``[H, N * NC, RECORD_BYTES]``, the records of the forward pass
    itself in the same fragment order, for a forward sweep without a prepare launch of its own.  Without
    ``reversed_copies`` (whole-chunk batches only) ``k_mirror`` is None and ``v_mirror`` is ``[N, T, H, V]``: P^T dO in
    the caller's token order, for a scan with ``mirror_odd`` that reads the caller's q, k and dout backwards itself.
    ``skip_empty_chunks`` (with ``sequences``): chunk slots past the end of their sequence get no records and no mirror
    rows (``GDN_FLAG_SKIP_EMPTY_CHUNKS``), for a mirror scan with ``valid_lengths``."""
    _require_hip_path()
    lib = _lib.load_library()
    B, T, H, K = q.shape
    if not reversed_copies and sequences is not None:
        raise ValueError("a batch that is not whole rows of whole chunks needs the reversed copies")
    if not backward_kernels_apply(K, V) or q.dtype != torch.bfloat16:
        raise ValueError(f"built for bf16, K in {_SUPPORTED_K} and V a multiple of 64, got {q.dtype}, {K}, {V}")
    if sequences is None:
        if T % 64 != 0:
            raise ValueError("without `sequences` T must be a multiple of 64")
        N, NC = B, T // 64
    else:
        seq_start, seq_len, NC = sequences
        N = seq_start.numel()
    g = None if g is None else g.to(torch.float32).contiguous()
    if beta is not None:
        beta = beta.contiguous() if beta.dtype in (torch.bfloat16, torch.float32) else beta.float().contiguous()
    dev, Bt = q.device, N * H
    f32 = dict(dtype=torch.float32, device=dev)
    out = dict(
        gamma=torch.empty(Bt, NC, 64, **f32), beta=torch.empty(Bt, NC, 64, **f32),
        rq=torch.empty(Bt, NC, 64, **f32), rk=torch.empty(Bt, NC, 64, **f32),
        k_mirror=torch.empty(N, 2 * NC * 64, H, K, dtype=torch.bfloat16, device=dev) if reversed_copies else None,
        v_mirror=torch.empty(N, (2 if reversed_copies else 1) * NC * 64, H, V, dtype=torch.bfloat16, device=dev),
        records=torch.empty(H, N * 2 * NC, RECORD_BYTES, dtype=torch.uint8, device=dev),
    )  # fmt: skip
    a = _lib.GdnChunkBwdPrepareArgs()
    a.q, a.k, a.dout = q.data_ptr(), k.data_ptr(), dout.data_ptr()
    a.g = None if g is None else g.data_ptr()
    a.beta = None if beta is None else beta.data_ptr()
    for name, x in (("q", q), ("k", k), ("dout", dout)):
        setattr(a, f"{name}_stride_b", x.stride(0))
        setattr(a, f"{name}_stride_t", x.stride(1))
        setattr(a, f"{name}_stride_h", x.stride(2))
    a.N, a.T, a.H, a.K, a.V = N, T, H, K, V
    a.beta_dtype = _lib.GDN_F32 if beta is None else _dtype_code(beta.dtype, "beta")
    a.flags = ((_lib.GDN_FLAG_L2NORM if l2norm else 0) | (_lib.GDN_FLAG_RECORDS_16X16 if half_slice_records else 0)
               | (_lib.GDN_FLAG_SKIP_EMPTY_CHUNKS if skip_empty_chunks and sequences is not None else 0))
    a.scale = float(scale)
    a.gamma, a.beta_packed, a.rq, a.rk = (out[n].data_ptr() for n in ("gamma", "beta", "rq", "rk"))
    a.k_mirror = out["k_mirror"].data_ptr() if reversed_copies else None
    a.v_mirror, a.records = out["v_mirror"].data_ptr(), out["records"].data_ptr()
    a.records_bytes = out["records"].numel()
    if forward_records:
        if sequences is not None:
            raise ValueError("forward records are written for whole-chunk batches only")
        out["records_fwd"] = torch.empty(H, N * NC, RECORD_BYTES, dtype=torch.uint8, device=dev)
        a.records_fwd, a.records_fwd_bytes = out["records_fwd"].data_ptr(), out["records_fwd"].numel()
    if sequences is not None:
        a.seq_start, a.seq_len, a.NC = seq_start.data_ptr(), seq_len.data_ptr(), NC
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        _lib.check_status(lib.gdn_chunk_bwd_prepare(ctypes.byref(a), stream), "gdn_chunk_bwd_prepare")
    return out


class _GatedDeltaRule(torch.autograd.Function):
    """Forward on the HIP kernels; backward by ``backward.gated_delta_rule_backward`` from the saved
    inputs (the forward keeps no intermediate results)."""

    @staticmethod
    def forward(ctx, mode, scale, output_final_state, l2norm, inplace_state, left_padded, q, k, v, g, beta,
                initial_state, cu_seqlens):  # fmt: skip
        if inplace_state:
            raise ValueError("inplace_state overwrites the initial state the backward needs; it is for inference")
        o, ht = _run(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm,
                     inplace_state, left_padded)  # fmt: skip
        ctx.save_for_backward(q, k, v, g, beta, initial_state, cu_seqlens)
        ctx.options = (scale, l2norm, left_padded)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        q, k, v, g, beta, initial_state, cu_seqlens = ctx.saved_tensors
        scale, l2norm, left_padded = ctx.options
        dq, dk, dv, dg, dbeta, dh0 = gated_delta_rule_backward(
            q, k, v, g, beta, do, dht, scale=scale, initial_state=initial_state, cu_seqlens=cu_seqlens,
            use_qk_l2norm_in_kernel=l2norm, left_padded=left_padded,
        )  # fmt: skip
        return None, None, None, None, None, None, dq, dk, dv, dg, dbeta, dh0, None


def _dispatch(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm, inplace_state,
              left_padded=False):
    if torch.compiler.is_compiling():  # a graph is being captured: the kernels go in as opaque operators
        from . import _opaque

        return _opaque.gated_delta_rule(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                                        l2norm, inplace_state, left_padded)  # fmt: skip
    tensors = (q, k, v, g, beta, initial_state)
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in tensors):
        return _GatedDeltaRule.apply(mode, scale, output_final_state, l2norm, inplace_state, left_padded, q, k, v, g,
                                  beta, initial_state, cu_seqlens)  # fmt: skip
    return _run(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm, inplace_state,
                left_padded)  # fmt: skip


def chunk_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None = None,
    beta: torch.Tensor | None = None,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    head_first: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    left_padded: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Chunked (chunk = 64) forward; drop-in for the call at gated_deltanet/module.py:197-209.

    bf16 inputs run the MFMA chunk kernels.  fp32 inputs are computed exactly, token by token,
    by the recurrent kernel (the chunk kernels round their matrix operands to bf16).

    ``left_padded=True`` (not an fla argument) keeps a padded batch ``[B, T, ...]`` as it is: ``cu_seqlens``
    ``[B + 1]`` then holds the prefix sums of the valid lengths and sequence b is the last
    ``cu_seqlens[b+1] - cu_seqlens[b]`` tokens of row b - what the reference derives from its attention mask
    (sequence_packing.py:18-22) before it packs and unpacks around the operator (:25-93).  The kernels skip
    the padding; ``o`` is zero there, as after the reference's unpack."""
    if head_first:
        raise ValueError("head_first layouts are not supported; pass [B, T, H, D] tensors")
    mode = "chunk" if q.dtype == torch.bfloat16 else "recurrent"
    return _dispatch(mode, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                     use_qk_l2norm_in_kernel, False, left_padded)  # fmt: skip


def fused_recurrent_gated_delta_rule(
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
    inplace_state: bool = False,
    left_padded: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Token-by-token forward; drop-in for the call at gated_deltanet/module.py:210-222.

    With ``inplace_state=True`` (and ``output_final_state=True``) the final state overwrites
    ``initial_state`` and that same tensor is returned: one read and one write of the state per
    decode step instead of a fresh allocation.  The reference's cache replaces its tensor with
    whatever is returned (lm_engine/generation_cache/constant.py:17-23), so both modes fit it.
    ``left_padded``: as in ``chunk_gated_delta_rule``."""
    return _dispatch("recurrent", q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                     use_qk_l2norm_in_kernel, inplace_state, left_padded)  # fmt: skip


def gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor | None,
    g: torch.Tensor | None,
    initial_state: torch.Tensor | None = None,
    cu_seqlens: torch.Tensor | None = None,
    scale: float | None = None,
    use_qk_l2norm_in_kernel: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``(q, k, v, beta, g, initial_state, cu_seqlens) -> (o, final_state)``.

    Picks the kernel the way the reference layer does (gated_deltanet/module.py:193): token
    dimension <= 64 runs the recurrent kernel, anything longer the chunked forward."""
    fn = fused_recurrent_gated_delta_rule if q.size(1) <= RECURRENT_MAX_TOKENS else chunk_gated_delta_rule
    return fn(q=q, k=k, v=v, g=g, beta=beta, scale=scale, initial_state=initial_state, output_final_state=True,
              cu_seqlens=cu_seqlens, use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel)  # fmt: skip
