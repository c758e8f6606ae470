"""The chunked forward as one launch (Kernel.gated_delta_rule_fused_launch / GDN_FLAG_FUSED_LAUNCH): producer
workgroups run the prepare step while scan workgroups with two compute waves per state slice consume the records.
Same parity gates against the CPU oracle as the two-kernel path (bf16: max-abs 2e-2 and relative-L2 1e-2 on the
output and on the final state); shapes that do not qualify must fall back to the two-kernel path unchanged."""

import pytest
import torch

import lm_engine_amd
from lm_engine_amd.kernels import Kernel, enable_kernels
from lm_engine_amd.ops import chunk_forward_kernel_times, fused_launch_applies
from lm_engine_amd.workloads import get_workload, make_inputs
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import assert_parity, max_abs, random_inputs, rel_l2


pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
FUSED = [Kernel.gated_delta_rule_fused_launch]


def two_kernels():
    """Inside the block the forward runs prepare and scan as two kernels whatever the shape."""
    return enable_kernels([Kernel.gated_delta_rule], reset=True)


def _to_gpu(inp):
    return {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}


def _qualifies(inp):
    """The rule of the library (ops.fused_launch_applies); inputs on the CPU or on the GPU."""
    with enable_kernels(FUSED):
        return fused_launch_applies(inp["q"].cuda(), inp["v"], inp.get("cu_seqlens"))


def _check(inp, label, **kwargs):
    assert _qualifies(inp), "this shape would take the two-kernel path"
    print(f"case: fused launch {label} q={tuple(inp['q'].shape)} v={tuple(inp['v'].shape)} {kwargs}", flush=True)
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True, **kwargs)
    with enable_kernels(FUSED):
        o, ht = lm_engine_amd.chunk_gated_delta_rule(**_to_gpu(inp), output_final_state=True, **kwargs)
    torch.cuda.synchronize()
    print(f"   o: max-abs {max_abs(o.float(), o_ref):.3e} rel-L2 {rel_l2(o.float(), o_ref):.3e}   "
          f"ht: max-abs {max_abs(ht, h_ref):.3e} rel-L2 {rel_l2(ht, h_ref):.3e}", flush=True)  # fmt: skip
    assert_parity(o.float(), o_ref, BF16, "o")
    assert_parity(ht, h_ref, BF16, "final_state")
    return o, ht


def test_the_flag_selects_the_single_launch():
    # what the library itself says it will launch (gdn_chunk_fwd_is_one_launch), with and without the flag
    inp = _to_gpu(random_inputs(B=2, T=4096, H=32, K=128, V=128, dtype=BF16, seed=149))
    assert fused_launch_applies(inp["q"], inp["v"]), "on by default"
    with two_kernels():
        assert not fused_launch_applies(inp["q"], inp["v"])
        split = chunk_forward_kernel_times(**inp, output_final_state=True)
        o_split, _ = lm_engine_amd.chunk_gated_delta_rule(**inp)
    with enable_kernels(FUSED):
        assert fused_launch_applies(inp["q"], inp["v"])
        fused = chunk_forward_kernel_times(**inp, output_final_state=True)
        o_fused, _ = lm_engine_amd.chunk_gated_delta_rule(**inp)
    print(f"kernel times, ms: two kernels {split}, one launch {fused}", flush=True)
    # the two modes run different scan kernels: close, and not the same bits
    assert rel_l2(o_fused.float(), o_split.float()) < 5e-3 and not torch.equal(o_fused, o_split)


@pytest.mark.parametrize("T", [65, 128, 130, 321])
def test_sequence_lengths_with_tail_chunks(T):
    _check(random_inputs(B=4, T=T, H=16, K=128, V=128, dtype=BF16, seed=150 + T), f"T={T}")


@pytest.mark.parametrize("K, V, B, H", [(64, 64, 8, 14), (64, 128, 4, 14), (128, 64, 8, 14), (128, 192, 4, 10)])
def test_head_dims(K, V, B, H):
    _check(random_inputs(B=B, T=200, H=H, K=K, V=V, dtype=BF16, seed=160 + K + V), f"K={K} V={V}")


def test_options_l2norm_scale_no_state_ungated():
    inp = random_inputs(B=4, T=257, H=14, K=128, V=128, dtype=BF16, seed=171, normalize=False)
    _check(inp, "in-kernel l2norm, scale 0.3", use_qk_l2norm_in_kernel=True, scale=0.3)
    inp = random_inputs(B=3, T=192, H=16, K=128, V=128, dtype=BF16, seed=172, gated=False, h0=False)
    _check(dict(inp, beta=None), "ungated, beta = 1, zero state")


def test_strided_projection_slices():
    # q, k, v as slices of one fused projection, the way the layer passes them
    gen = torch.Generator("cpu").manual_seed(173)
    B, T, H, K, V = 4, 300, 16, 128, 128
    proj = torch.randn(B, T, H * (2 * K + V), generator=gen).to(BF16)
    q, k, v = (x.reshape(B, T, H, -1) for x in proj.split([H * K, H * K, H * V], dim=-1))
    q = torch.nn.functional.normalize(q.float(), dim=-1).to(BF16)  # contiguous copy: only k and v stay strided
    inp = dict(random_inputs(B, T, H, K, V, dtype=BF16, seed=174), q=q, k=k, v=v)
    _check(inp, "strided k, v", use_qk_l2norm_in_kernel=True)


def test_config1_full_size():
    _check(make_inputs(get_workload(1)), "cfg1 full size")


def test_long_context_and_the_split_property():
    # configuration 4's distributions (slow decay, random initial state) at T = 8192 (128 chunks per chain) on 64 chains
    # of V = 128: configuration 4 itself (32 chains of V = 256) runs as two kernels, see test_chunk_gpu.py
    inp = make_inputs(get_workload(4, B=2, T=8192, V=128))
    o, ht = _check(inp, "configuration 4's inputs, B=2 V=128 T=8192")
    gpu = _to_gpu(inp)
    cut = 64 * 45
    with enable_kernels(FUSED):
        first = {n: (x[:, :cut] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
        o1, h1 = lm_engine_amd.chunk_gated_delta_rule(**first, output_final_state=True)
        second = {n: (x[:, cut:] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
        second["initial_state"] = h1
        o2, h2 = lm_engine_amd.chunk_gated_delta_rule(**second, output_final_state=True)
        o_again, h_again = lm_engine_amd.chunk_gated_delta_rule(**gpu, output_final_state=True)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([o1, o2], dim=1), o) and torch.equal(h2, ht), "split run differs from the full run"
    assert torch.equal(o_again, o) and torch.equal(h_again, ht), "two runs of the same launch differ"


def test_close_to_the_two_kernel_path_and_fallback_is_unchanged():
    inp = _to_gpu(random_inputs(B=4, T=500, H=16, K=128, V=128, dtype=BF16, seed=180))
    assert _qualifies(inp)
    with two_kernels():
        o_split, h_split = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    with enable_kernels(FUSED):
        o_fused, h_fused = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert rel_l2(o_fused.float(), o_split.float()) < 5e-3 and rel_l2(h_fused, h_split) < 1e-3
    # shapes that do not qualify take the two-kernel path whatever the flag says: packed sequences, V not a multiple of 64,
    # more scan workgroups than half of the CUs, fewer than three eighths, too few chains (configuration 4's 32)
    packed = _to_gpu(random_inputs(B=1, T=300, H=2, K=128, V=128, dtype=BF16, seed=181, N=3))
    cu = torch.tensor([0, 70, 71, 300], dtype=torch.int32, device="cuda")
    odd_v = _to_gpu(random_inputs(B=1, T=130, H=2, K=128, V=96, dtype=BF16, seed=182))
    many = _to_gpu(random_inputs(B=20, T=130, H=16, K=128, V=128, dtype=BF16, seed=183))
    few = _to_gpu(random_inputs(B=1, T=300, H=16, K=128, V=128, dtype=BF16, seed=184))
    wide = _to_gpu(random_inputs(B=1, T=300, H=32, K=128, V=256, dtype=BF16, seed=185))
    assert not any(_qualifies(case) for case in (odd_v, many, few, wide))
    for case, extra in ((packed, dict(cu_seqlens=cu)), (odd_v, {}), (many, {}), (few, {}), (wide, {})):
        with two_kernels():
            a = lm_engine_amd.chunk_gated_delta_rule(**case, output_final_state=True, **extra)
        with enable_kernels(FUSED):
            b = lm_engine_amd.chunk_gated_delta_rule(**case, output_final_state=True, **extra)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_ready_flags_are_left_clear_and_need_no_clearing_when_the_caller_says_so():
    """GDN_FLAG_READY_FLAGS_CLEAR through the C ABI: a workspace that was zero before its first use serves calls in a
    row without the clearing kernel; each gives the bits of a call on a fresh workspace without the flag, and the
    flag region is all zero after every call, with and without the flag."""
    import ctypes

    from lm_engine_amd import _lib, ops

    lib = _lib.load_library()
    B, T, H, K, V = 4, 512, 16, 128, 128  # inside the one-launch window
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    kept = None
    for seed in (31, 32, 33):
        inp = random_inputs(B, T, H, K, V, dtype=BF16, seed=seed)
        q, k, v, g, beta, h0 = (inp[n].cuda() for n in ("q", "k", "v", "g", "beta", "initial_state"))
        assert fused_launch_applies(q, v)
        dims = ops._check_inputs(q, k, v, g, beta, h0, None)
        outs = []
        for promise in (False, True):
            o = torch.full((B, T, H, V), float("nan"), dtype=BF16, device="cuda")
            ht = torch.full((B, H, K, V), float("nan"), dtype=torch.float32, device="cuda")
            args = ops._fill_args(q, k, v, g, beta, h0, ht, o, None, None, False, False, dims)
            assert args.flags & _lib.GDN_FLAG_FUSED_LAUNCH
            nbytes = int(lib.gdn_workspace_bytes(ctypes.byref(args)))
            if promise:
                kept = torch.zeros(nbytes, dtype=torch.uint8, device="cuda") if kept is None else kept
                workspace = kept
                args.flags |= _lib.GDN_FLAG_READY_FLAGS_CLEAR
            else:
                workspace = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device="cuda")  # stale flags all set
            args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
            print(f"gdn_chunk_fwd seed={seed} ready flags promised clear: {promise}", flush=True)
            _lib.check_status(lib.gdn_chunk_fwd(ctypes.byref(args), stream), "gdn_chunk_fwd")
            torch.cuda.synchronize()
            # workspace = [chunk offsets and order, error latch in its last word | flags | records]
            records = H * B * (T // 64) * 13312
            header = int(lib.gdn_workspace_header_bytes(ctypes.byref(args)))
            first = ((2 * B + 2) * 4 + 255) // 256 * 256
            assert header == nbytes - records
            assert not workspace[first - 4 : header].any(), "error latch or ready flags left set"
            assert lib.gdn_chunk_fwd_status(ctypes.byref(args), stream) == 0
            outs.append((o, ht))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_operator_keeps_its_workspaces_between_calls():
    from lm_engine_amd import ops

    ops.release_workspaces()
    inp = {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in random_inputs(4, 512, 16, 128, 128, dtype=BF16, seed=34).items()}
    first = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert len(ops._WORKSPACES) == 1
    again = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert len(ops._WORKSPACES) == 1, "same device, stream and shape: same workspace"
    assert torch.equal(first[0], again[0]) and torch.equal(first[1], again[1])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    side.synchronize()
    assert len(ops._WORKSPACES) == 2, "another stream gets a workspace of its own"
    assert torch.equal(first[0], other[0])
    for t in range(2, 2 + ops._WORKSPACE_LIMIT + 2):
        short = {n: (x[:, : 64 * t] if n in ("q", "k", "v", "g", "beta") else x) for n, x in inp.items()}
        lm_engine_amd.chunk_gated_delta_rule(**short)
    assert len(ops._WORKSPACES) == ops._WORKSPACE_LIMIT
    ops.release_workspaces()
    assert not ops._WORKSPACES


def test_a_scan_whose_wait_runs_out_reports_it_and_the_workspace_recovers():
    """The error path of the one-launch forward, forced from the host: with GDN_FLAG_DEBUG_NO_PRODUCERS the prepare
    workgroups return at once and with a spin limit of a few polls the scan's waits run out.  Every kernel still ends
    normally; the launch latches the error (workspace header, and the caller's pinned word), writes no output, and
    gdn_chunk_fwd_status reports it and clears the header, after which the same workspace serves a good call."""
    import ctypes

    from lm_engine_amd import _lib, ops

    lib = _lib.load_library()
    B, T, H, K, V = 4, 256, 16, 128, 128  # inside the one-launch window
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    inp = random_inputs(B, T, H, K, V, dtype=BF16, seed=41)
    q, k, v, g, beta, h0 = (inp[n].cuda() for n in ("q", "k", "v", "g", "beta", "initial_state"))
    dims = ops._check_inputs(q, k, v, g, beta, h0, None)
    word = torch.zeros(1, dtype=torch.int32).pin_memory()

    def call(debug):
        o = torch.full((B, T, H, V), float("nan"), dtype=BF16, device="cuda")
        ht = torch.full((B, H, K, V), float("nan"), dtype=torch.float32, device="cuda")
        args = ops._fill_args(q, k, v, g, beta, h0, ht, o, None, None, False, False, dims)
        args.flags |= _lib.GDN_FLAG_FUSED_LAUNCH | _lib.GDN_FLAG_READY_FLAGS_CLEAR
        if debug:
            args.flags |= _lib.GDN_FLAG_DEBUG_NO_PRODUCERS
            args.spin_limit = 4
        args.error_word = word.data_ptr()
        args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
        assert lib.gdn_chunk_fwd_is_one_launch(ctypes.byref(args)) == 1
        _lib.check_status(lib.gdn_chunk_fwd(ctypes.byref(args), stream), "gdn_chunk_fwd")
        return args, o, ht

    args = ops._fill_args(q, k, v, g, beta, h0, None, q, None, None, False, False, dims)
    nbytes, header = int(lib.gdn_workspace_bytes(ctypes.byref(args))), int(lib.gdn_workspace_header_bytes(ctypes.byref(args)))
    workspace = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    print("gdn_chunk_fwd without producers, spin limit 4", flush=True)
    args, o, ht = call(debug=True)
    status = lib.gdn_chunk_fwd_status(ctypes.byref(args), stream)
    assert status == _lib.GDN_ERR_TIMEOUT, _lib.strerror(status)
    assert int(word[0]) == 1, "the caller's error word was not set"
    assert torch.isnan(o.float()).all() and torch.isnan(ht).all(), "a workgroup that gave up still wrote output"
    assert not workspace[:header].any(), "gdn_chunk_fwd_status leaves the header clear"
    assert lib.gdn_chunk_fwd_status(ctypes.byref(args), stream) == 0, "the latch is cleared once reported"
    print("gdn_chunk_fwd on the same workspace, producers back", flush=True)
    word.zero_()
    args, o, ht = call(debug=False)
    assert lib.gdn_chunk_fwd_status(ctypes.byref(args), stream) == 0 and int(word[0]) == 0
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True)
    assert_parity(o.float(), o_ref, BF16, "o")
    assert_parity(ht, h_ref, BF16, "final_state")


def test_the_operator_raises_at_the_next_call_after_a_reported_time_out():
    from lm_engine_amd import ops

    ops.release_workspaces()
    inp = _to_gpu(random_inputs(4, 256, 16, 128, 128, dtype=BF16, seed=42))
    good = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert len(ops._WORKSPACES) == 1
    ops._error_word(inp["q"].device)[0] = 1  # what a scan workgroup that gave up stores (previous test)
    with pytest.raises(RuntimeError, match="gave up waiting"):
        lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert not ops._WORKSPACES, "the kept workspaces of the device are dropped: their flags are in no defined state"
    again = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert torch.equal(good[0], again[0]) and torch.equal(good[1], again[1])


def test_only_one_launch_shapes_keep_a_workspace():
    from lm_engine_amd import ops

    ops.release_workspaces()
    packed = _to_gpu(random_inputs(B=1, T=300, H=2, K=128, V=128, dtype=BF16, seed=43, N=3))
    cu = torch.tensor([0, 70, 71, 300], dtype=torch.int32, device="cuda")
    lm_engine_amd.chunk_gated_delta_rule(**packed, cu_seqlens=cu)
    lm_engine_amd.chunk_gated_delta_rule(**_to_gpu(random_inputs(B=1, T=300, H=16, K=128, V=128, dtype=BF16, seed=44)))
    lm_engine_amd.chunk_gated_delta_rule(**_to_gpu(random_inputs(B=2, T=130, H=2, K=256, V=64, dtype=BF16, seed=45)))
    assert not ops._WORKSPACES
