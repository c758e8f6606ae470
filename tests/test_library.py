"""Host-side checks that need no GPU: the C-ABI library loads, exports what include/gdn_hip.h
declares, agrees with the ctypes mirror of the argument struct, and rejects bad arguments
before anything is launched."""

import ctypes
import os
import re
import subprocess
import sys
import tempfile

import pytest
import torch

import lm_engine_amd
from lm_engine_amd import _lib
from lm_engine_amd.kernels import Kernel, enable_kernels, is_kernel_allowed


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gdn_hip.h")


def _declared_functions() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(gdn_[a-z0-9_]+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    lib = _lib.load_library()
    declared = set(_declared_functions())
    assert declared == set(_lib.EXPORTED_SYMBOLS), declared
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.gdn_abi_version() == _lib.GDN_ABI_VERSION


def test_struct_layout_matches_the_header():
    source = r"""
    #include <stdio.h>
    #include <stddef.h>
    #include "gdn_hip.h"
    int main(void) {
        printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(gdn_args), offsetof(gdn_args, workspace_bytes),
               offsetof(gdn_args, q_stride_b), offsetof(gdn_args, o_stride_h), offsetof(gdn_args, B),
               offsetof(gdn_args, flags), offsetof(gdn_args, scale));
        printf("%zu %zu\n", offsetof(gdn_args, spin_limit), offsetof(gdn_args, error_word));
        printf("%zu %zu %zu %zu %zu\n", sizeof(gdn_conv_args), offsetof(gdn_conv_args, final_state),
               offsetof(gdn_conv_args, x_stride_b), offsetof(gdn_conv_args, B), offsetof(gdn_conv_args, activation));
        return 0;
    }
    """
    with tempfile.TemporaryDirectory() as tmp:
        src, exe = os.path.join(tmp, "layout.c"), os.path.join(tmp, "layout")
        open(src, "w").write(source)
        subprocess.run(["gcc", f"-I{os.path.dirname(HEADER)}", src, "-o", exe], check=True)
        values = [int(x) for x in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    A = _lib.GdnArgs
    Cv = _lib.GdnConvArgs
    assert values == [ctypes.sizeof(A), A.workspace_bytes.offset, A.q_stride_b.offset, A.o_stride_h.offset,
                      A.B.offset, A.flags.offset, A.scale.offset, A.spin_limit.offset, A.error_word.offset,
                      ctypes.sizeof(Cv), Cv.final_state.offset, Cv.x_stride_b.offset, Cv.B.offset,
                      Cv.activation.offset]  # fmt: skip


def test_layer_ops_reject_bad_arguments_before_any_launch():
    lib = _lib.load_library()
    g = _lib.GdnGateArgs()
    g.a = g.b = g.A_log = g.dt_bias = g.g = g.beta = 0x1000
    g.tokens, g.H, g.a_stride, g.b_stride, g.dtype, g.beta_scale = 4, 8, 8, 8, _lib.GDN_BF16, 1.0
    for over, status in [(dict(a=None), -1), (dict(tokens=0), -2), (dict(a_stride=4), -2), (dict(dtype=5), -3)]:
        a = _lib.GdnGateArgs.from_buffer_copy(g)
        for name, value in over.items():
            setattr(a, name, value)
        assert lib.gdn_gates_fwd(ctypes.byref(a), None) == status, over
    n = _lib.GdnNormArgs()
    n.o, n.y = 0x1000, 0x2000
    n.tokens, n.H, n.V, n.dtype, n.w_dtype, n.eps = 4, 2, 64, _lib.GDN_BF16, _lib.GDN_F32, 1e-6
    n.o_stride_t = n.y_stride_t = 128
    for over, status in [(dict(o=None), -1), (dict(V=0), -2), (dict(V=20), -3), (dict(V=1024), -3), (dict(o_stride_t=64), -2),
                         (dict(o=0x1002), -4), (dict(gate=0x3008, gate_stride_t=128), -4), (dict(o_stride_t=132), -4)]:  # fmt: skip
        a = _lib.GdnNormArgs.from_buffer_copy(n)
        for name, value in over.items():
            setattr(a, name, value)
        assert lib.gdn_gated_rmsnorm_fwd(ctypes.byref(a), None) == status, over


def test_convolution_rejects_bad_arguments_before_any_launch():
    lib = _lib.load_library()

    def conv_args(**over):
        a = _lib.GdnConvArgs()
        a.x, a.y, a.weight = 0x1000, 0x2000, 0x3000  # never dereferenced
        a.B, a.S, a.C, a.kernel_size = 2, 8, 16, 4
        a.x_stride_s = a.y_stride_s = 16
        a.x_stride_b = a.y_stride_b = 128
        a.dtype, a.w_dtype, a.activation = _lib.GDN_BF16, _lib.GDN_BF16, _lib.GDN_ACT_SILU
        for name, value in over.items():
            setattr(a, name, value)
        return a

    for over, status in [
        (dict(x=None), -1),
        (dict(S=0), -2),
        (dict(kernel_size=5), -3),
        (dict(kernel_size=1), -3),
        (dict(C=12), -3),
        (dict(activation=7), -3),
        (dict(x_stride_s=20), -4),
        (dict(x=0x1008), -4),
        (dict(y=0x1000), -2),
        (dict(x_stride_s=8), -2),
    ]:
        assert lib.gdn_causal_conv1d_fwd(ctypes.byref(conv_args(**over)), None) == status, over


def _args(**over):
    a = _lib.GdnArgs()
    fake = 0x1000  # never dereferenced: validation fails before any launch
    a.q = a.k = a.v = a.o = fake
    a.B, a.T, a.H, a.K, a.V, a.N = 1, 8, 2, 64, 64, 1
    a.q_stride_h = a.k_stride_h = 64
    a.v_stride_h = a.o_stride_h = 64
    a.q_stride_t = a.k_stride_t = a.v_stride_t = a.o_stride_t = 128
    a.q_stride_b = a.k_stride_b = a.v_stride_b = a.o_stride_b = 1024
    a.dtype, a.beta_dtype, a.scale = _lib.GDN_BF16, _lib.GDN_BF16, 0.125
    for name, value in over.items():
        setattr(a, name, value)
    return a


@pytest.mark.parametrize(
    "over, status",
    [
        (dict(q=None), -1),
        (dict(T=0), -2),
        (dict(N=3), -2),
        (dict(K=48), -3),
        (dict(V=40), -3),
        (dict(dtype=7), -3),
        (dict(q_stride_t=129), -4),
        (dict(v=0x1004), -4),
        (dict(cu_seqlens=0x2000, B=2, N=2), -6),
        (dict(flags=_lib.GDN_FLAG_LEFT_PADDED), -1),  # left-padded needs the prefix sums
        (dict(flags=_lib.GDN_FLAG_LEFT_PADDED, cu_seqlens=0x2000, B=2, N=3), -2),  # one sequence per row
        (dict(q_stride_h=32), -2),
    ],
)
def test_bad_arguments_are_rejected_before_launch(over, status):
    lib = _lib.load_library()
    a = _args(**over)
    assert lib.gdn_recurrent_fwd(ctypes.byref(a), None) == status
    assert lib.gdn_chunk_fwd(ctypes.byref(a), None) == status
    assert _lib.strerror(status) != "unknown gdn status"


def test_chunk_fwd_needs_a_workspace():
    lib = _lib.load_library()
    a = _args(T=128, K=128, V=128, q_stride_h=128, k_stride_h=128, v_stride_h=128, o_stride_h=128,
              q_stride_t=256, k_stride_t=256, v_stride_t=256, o_stride_t=256, q_stride_b=256 * 128,
              k_stride_b=256 * 128, v_stride_b=256 * 128, o_stride_b=256 * 128)  # fmt: skip
    need = lib.gdn_workspace_bytes(ctypes.byref(a))
    assert need > 0
    assert lib.gdn_chunk_fwd(ctypes.byref(a), None) == -5
    a.workspace, a.workspace_bytes = 0x10000, need - 1
    assert lib.gdn_chunk_fwd(ctypes.byref(a), None) == -5
    a.dtype = _lib.GDN_F32  # fp32 inputs have no chunk kernel
    assert lib.gdn_workspace_bytes(ctypes.byref(a)) == 0
    assert lib.gdn_chunk_fwd(ctypes.byref(a), None) == -3


def test_python_wrapper_validates_and_never_falls_back():
    q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU only"):
        lm_engine_amd.fused_recurrent_gated_delta_rule(q=q, k=q, v=q)
    with pytest.raises(ValueError, match="shape of q"):
        lm_engine_amd.chunk_gated_delta_rule(q=q, k=q[:, :4], v=q)
    with pytest.raises(ValueError, match="head_first"):
        lm_engine_amd.chunk_gated_delta_rule(q=q, k=q, v=q, head_first=True)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIBRARY_PATH", "/nonexistent/libgdn_hip.so")
    with pytest.raises(_lib.GdnLibraryError, match="no fallback"):
        _lib.load_library()


def test_kernel_flag_registry_follows_the_reference_convention():
    assert is_kernel_allowed(Kernel.gated_delta_rule)
    with enable_kernels([], reset=True):
        assert not is_kernel_allowed(Kernel.gated_delta_rule)
        q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
        with pytest.raises(RuntimeError, match="no other implementation"):
            lm_engine_amd.fused_recurrent_gated_delta_rule(q=q, k=q, v=q)
        with enable_kernels([Kernel.gated_delta_rule]):
            assert is_kernel_allowed(Kernel.gated_delta_rule)
        assert not is_kernel_allowed(Kernel.gated_delta_rule)
    assert is_kernel_allowed(Kernel.gated_delta_rule)


def test_fused_launch_flag_is_on_by_default_and_can_be_switched_off():
    fused = Kernel.gated_delta_rule_fused_launch
    assert is_kernel_allowed(fused)
    with enable_kernels([Kernel.gated_delta_rule], reset=True):
        assert not is_kernel_allowed(fused) and is_kernel_allowed(Kernel.gated_delta_rule)
    assert is_kernel_allowed(fused)
    assert _lib.GDN_FLAG_FUSED_LAUNCH == 8 and _lib.GDN_FLAG_READY_FLAGS_CLEAR == 16


def test_kernel_flag_env_variable():
    code = "from lm_engine_amd.kernels import Kernel, is_kernel_allowed; print(is_kernel_allowed(Kernel.gated_delta_rule))"
    run = lambda env: subprocess.run([sys.executable, "-c", code], env={**os.environ, **env}, cwd=ROOT,
                                     capture_output=True, text=True, check=True).stdout.strip()  # noqa: E731  # fmt: skip
    assert run({"ENABLE_KERNELS": "rmsnorm"}) == "False"
    assert run({"ENABLE_KERNELS": "rmsnorm, gated_delta_rule"}) == "True"
    assert run({"ENABLE_ALL_KERNELS": "1"}) == "True"


def test_fla_shim_resolves_the_reference_imports():
    from lm_engine_amd import install_as_fla, uninstall_fla_shim

    install_as_fla()
    try:
        from fla.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
        import fla  # noqa: F401  (the reference's availability probe, lm_engine/utils/packages.py:56-61)

        assert chunk_gated_delta_rule is lm_engine_amd.chunk_gated_delta_rule
        assert fused_recurrent_gated_delta_rule is lm_engine_amd.fused_recurrent_gated_delta_rule
    finally:
        uninstall_fla_shim()
    assert "fla" not in sys.modules


def test_noalloc_entry_point_rejects_shapes_beyond_its_scratch():
    lib = _lib.load_library()
    args = _lib.GdnArgs()
    args.q = args.k = args.v = args.o = 0x1000
    args.B, args.T, args.H, args.K, args.V, args.N = 8, 8192, 16, 128, 128, 8
    args.chunk, args.dtype, args.beta_dtype, args.scale = 64, _lib.GDN_BF16, _lib.GDN_BF16, 1.0
    for name in ("q", "k", "v", "o"):
        setattr(args, f"{name}_stride_b", 8192 * 16 * 128)
        setattr(args, f"{name}_stride_t", 16 * 128)
        setattr(args, f"{name}_stride_h", 128)
    assert lib.gdn_workspace_bytes(ctypes.byref(args)) > _lib.GDN_NOALLOC_SCRATCH_BYTES
    assert lib.gdn_chunk_fwd_noalloc(ctypes.byref(args), None) == -5  # GDN_ERR_WORKSPACE, before any launch


def test_opaque_operators_are_registered_with_shape_only_implementations():
    # what torch.compile captures in place of the ctypes launches: one torch.library operator per kernel, each with a
    # fake implementation (run here on meta tensors: no kernel is launched)
    import torch

    from lm_engine_amd import _opaque  # noqa: F401

    ops = torch.ops.lm_engine_amd
    for name in ("gated_delta_rule_forward", "gated_delta_rule_backward", "gated_delta_rule_decode_",
                 "causal_conv1d_forward", "causal_conv1d_backward", "delta_rule_gates_forward",
                 "delta_rule_gates_backward", "gated_rmsnorm_forward", "gated_rmsnorm_backward"):  # fmt: skip
        assert hasattr(ops, name), name
    meta = lambda *shape, dtype=torch.bfloat16: torch.empty(*shape, dtype=dtype, device="meta")  # noqa: E731
    B, T, H, K, V = 2, 130, 3, 128, 64
    q, k, v = meta(B, T, H, K), meta(B, T, H, K), meta(B, T, H, V)
    g, beta, h0 = meta(B, T, H, dtype=torch.float32), meta(B, T, H), meta(B, H, K, V, dtype=torch.float32)
    o, ht = ops.gated_delta_rule_forward(q, k, v, g, beta, h0, None, "chunk", None, True, False, False)
    assert tuple(o.shape) == (B, T, H, V) and o.dtype == torch.bfloat16
    assert tuple(ht.shape) == (B, H, K, V) and ht.dtype == torch.float32
    o, ht = ops.gated_delta_rule_forward(q, k, v, None, None, None, None, "chunk", 0.5, False, True, False)
    assert ht.numel() == 0
    cu = torch.empty(4, dtype=torch.int32, device="meta")
    _, ht = ops.gated_delta_rule_forward(q[:1], k[:1], v[:1], None, None, None, cu, "chunk", None, True, False, False)
    assert tuple(ht.shape) == (3, H, K, V)
    grads = ops.gated_delta_rule_backward(q, k, v, g, None, h0, None, o, None, None, False, False)
    assert [tuple(x.shape) for x in grads] == [(B, T, H, K), (B, T, H, K), (B, T, H, V), (B, T, H), (0,), (B, H, K, V)]
    y, state = ops.causal_conv1d_forward(meta(B, T, 96), meta(96, 4), None, None, None, True, "silu")
    assert tuple(y.shape) == (B, T, 96) and tuple(state.shape) == (B, 96, 3)
    gg, bb = ops.delta_rule_gates_forward(meta(B, T, H), meta(B, T, H), meta(H, dtype=torch.float32),
                                          meta(H, dtype=torch.float32), False)  # fmt: skip
    assert gg.dtype == torch.float32 and bb.dtype == torch.bfloat16 and tuple(gg.shape) == (B, T, H)
    assert tuple(ops.gated_rmsnorm_forward(meta(B, T, H, V), meta(B, T, H * V), meta(V), None).shape) == (B, T, H, V)
