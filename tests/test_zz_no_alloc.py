"""gdn_chunk_fwd_noalloc, the entry point for callers that cannot allocate device memory, against
gdn_chunk_fwd on the same inputs: both run the same kernels, so outputs and final states must be
bit-identical.  Two calls in a row share the library's built-in scratch array; the second is smaller,
so stale records of the first lie behind the ones it writes.  (The arguments carry the library's default flags: the
first shape qualifies for the one-launch forward, whose ready flags then live in the scratch array too.)"""

import ctypes

import pytest
import torch

from lm_engine_amd import _lib, ops
from tests.helpers import random_inputs


pytestmark = pytest.mark.gpu


def _both_entry_points(B, T, H, K, V, seed, cu_seqlens=None):
    lib = _lib.load_library()
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    inp = random_inputs(B, T, H, K, V, dtype=torch.bfloat16, seed=seed, N=N)
    dev = {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}
    cu = None if cu_seqlens is None else torch.tensor(cu_seqlens, dtype=torch.int32, device="cuda")
    q, k, v, g, beta, h0 = dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"], dev["initial_state"]
    dims = ops._check_inputs(q, k, v, g, beta, h0, cu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    results = []
    for entry in ("gdn_chunk_fwd", "gdn_chunk_fwd_noalloc"):
        o = torch.full((B, T, H, V), float("nan"), dtype=torch.bfloat16, device="cuda")
        ht = torch.full((N, H, K, V), float("nan"), dtype=torch.float32, device="cuda")
        args = ops._fill_args(q, k, v, g, beta, h0, ht, o, cu, None, False, False, dims)
        if entry == "gdn_chunk_fwd":
            nbytes = int(lib.gdn_workspace_bytes(ctypes.byref(args)))
            assert 0 < nbytes <= _lib.GDN_NOALLOC_SCRATCH_BYTES
            workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
        print(f"{entry} B={B} T={T} H={H} K={K} V={V} seed={seed} packed={cu_seqlens is not None}", flush=True)
        _lib.check_status(getattr(lib, entry)(ctypes.byref(args), stream), entry)
        torch.cuda.synchronize()
        results.append((o, ht))
    return results


def test_noalloc_entry_point_matches_chunk_fwd_on_two_calls_in_a_row():
    for B, T, H, K, V, seed, cu in [
        (4, 512, 16, 128, 128, 4, None),                 # a shape that runs prepare and scan as one launch (ready flags in the scratch)
        (2, 1024, 8, 128, 128, 5, None),                 # 128 chunk records per head, two kernels
        (1, 200, 4, 128, 128, 6, None),                  # second, smaller call: 4 records, a partial last chunk
        (1, 512, 4, 128, 256, 7, [0, 130, 131, 512]),    # packed: the chunk offsets live in the scratch as well
    ]:  # fmt: skip
        (o_ref, h_ref), (o, h) = _both_entry_points(B, T, H, K, V, seed, cu)
        assert torch.isfinite(o.float()).all() and torch.isfinite(h).all()
        assert torch.equal(o, o_ref), f"output differs at B={B} T={T}"
        assert torch.equal(h, h_ref), f"final state differs at B={B} T={T}"
