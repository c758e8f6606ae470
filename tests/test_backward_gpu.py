"""Autograd through the operators on the GPU: forward on the HIP kernels, gradients against autograd
through the fp64 token loop of the oracle on the same (rounded) inputs.

Gate for a gradient: relative-L2 <= 1e-2 and max-abs <= 2e-2 x max(1, max |reference|) for bf16 inputs
(the gradients come back rounded to bf16), 1e-4 on both for fp32 inputs.  The gradient of g gets relative-L2
<= 2e-2: every dg_t is a sum of signed per-token terms, each an inner product of two products of bf16-rounded
operands (0.3 - 0.4 % apiece), and what is left after they cancel carries their whole error; observed 1e-3 to
1.1e-2 over the sweeps below, the largest values with a random gradient flowing into the final state."""

import os

import pytest
import torch

import lm_engine_amd
from oracle.gdn_backward_oracle import gated_delta_rule_grads_autograd

from .helpers import assert_parity, max_abs, random_inputs, rel_l2


pytestmark = pytest.mark.gpu

NAMES = ("dq", "dk", "dv", "dg", "dbeta", "dh0")


def _leaves(inp):
    out = {}
    for name, x in inp.items():
        out[name] = None if x is None else x.cuda().requires_grad_(True)
    return out


def _assert_grads(got, want, dtype):
    for name, a, b in zip(NAMES, got, want):
        assert a is not None, name
        assert a.shape == b.shape, name
        ma, rl = max_abs(a, b), rel_l2(a, b)
        top = max(1.0, float(b.abs().max()))
        print(f"      {name}: max-abs {ma:.3e} (top {top:.2f}) rel-L2 {rl:.3e}", flush=True)
        if dtype == torch.bfloat16:
            gate = 2e-2 if name == "dg" else 1e-2
            assert rl <= gate and ma <= 2e-2 * top, f"{name}: max-abs {ma:.3e} (top {top:.2f}), rel-L2 {rl:.3e}"
        else:
            assert rl <= 1e-4 and ma <= 1e-4 * top, f"{name}: max-abs {ma:.3e} (top {top:.2f}), rel-L2 {rl:.3e}"


def _run_case(fn, inp, dtype, cu=None, **kw):
    gen = torch.Generator().manual_seed(99)
    leaves = _leaves(inp)
    cu_dev = None if cu is None else cu.cuda()
    o, ht = fn(**leaves, output_final_state=True, cu_seqlens=cu_dev, use_qk_l2norm_in_kernel=True, **kw)
    do = torch.randn(o.shape, generator=gen).to(dtype)
    dht = torch.randn(ht.shape, generator=gen)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    got = [leaves[n].grad for n in ("q", "k", "v", "g", "beta", "initial_state")]
    want = gated_delta_rule_grads_autograd(
        inp["q"], inp["k"], inp["v"], inp["g"], inp["beta"], do, dht, initial_state=inp["initial_state"],
        cu_seqlens=cu, use_qk_l2norm_in_kernel=True,
    )  # fmt: skip
    _assert_grads(got, want, dtype)
    assert [x.dtype for x in got[:3]] == [dtype] * 3


@pytest.mark.parametrize("T", [65, 256])
def test_chunk_bf16(T):
    inp = random_inputs(B=2, T=T, H=2, K=128, V=128, dtype=torch.bfloat16, seed=T, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


def test_chunk_bf16_config1_full_shape():
    # B=4, T=4096, H=16, K=V=128, the shape the backward is timed at.  Autograd through the fp64 token loop
    # keeps every state of every chain, too much for all 64 chains at this length; chains do not interact
    # (a property the oracle tests pin), so the gradients of three chains of the full-shape run are checked
    # against the oracle run on those chains alone.
    from lm_engine_amd.workloads import get_workload, make_inputs

    inp = make_inputs(get_workload(1))
    assert tuple(inp["q"].shape) == (4, 4096, 16, 128)
    names = ("q", "k", "v", "g", "beta")
    leaves = {n: inp[n].cuda().requires_grad_(True) for n in names}
    print("case: backward at configuration 1's full shape", flush=True)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**leaves, scale=inp["scale"], output_final_state=True)
    gen = torch.Generator().manual_seed(123)
    do = torch.randn(o.shape, generator=gen).to(torch.bfloat16)
    dht = torch.randn(ht.shape, generator=gen)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    torch.cuda.synchronize()
    for b, h in [(0, 0), (2, 7), (3, 15)]:
        cut = lambda x: x[b:b + 1, :, h:h + 1]  # noqa: E731
        want = gated_delta_rule_grads_autograd(*(cut(inp[n]) for n in names), cut(do), dht[b:b + 1, h:h + 1],
                                               scale=inp["scale"])  # fmt: skip
        got = [cut(leaves[n].grad) for n in names]
        for name, a, ref in zip(NAMES, got, want):
            ma, rl = max_abs(a, ref), rel_l2(a, ref)
            top = max(1.0, float(ref.abs().max()))
            print(f"   chain ({b}, {h}) {name}: max-abs {ma:.3e} (top {top:.2f}) rel-L2 {rl:.3e}", flush=True)
            assert rl <= 1e-2 and ma <= 2e-2 * top, f"chain ({b}, {h}) {name}: max-abs {ma:.3e}, rel-L2 {rl:.3e}"


def test_chunk_bf16_shipped_head_shape_full_size():
    # B=8, T=4096, H=2, K=256, V=512: the head shape of the reference's shipped configurations
    # (configs/research/m2rnn/400m-normal/gated-deltanet.yml:60-73) at the batch its backward is timed at, with the
    # in-kernel normalisation the reference always asks for (gated_deltanet/module.py:208).  Two chains of the
    # full-shape run against the oracle on those chains alone (chains do not interact).
    from lm_engine_amd.workloads import get_workload, make_inputs

    inp = make_inputs(get_workload(1, B=8, H=2, K=256, V=512))
    assert tuple(inp["q"].shape) == (8, 4096, 2, 256) and tuple(inp["v"].shape) == (8, 4096, 2, 512)
    names = ("q", "k", "v", "g", "beta")
    leaves = {n: inp[n].cuda().requires_grad_(True) for n in names}
    print("case: backward at the shipped head shape, B=8 T=4096 H=2 K=256 V=512", flush=True)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**leaves, scale=inp["scale"], output_final_state=True,
                                                 use_qk_l2norm_in_kernel=True)  # fmt: skip
    gen = torch.Generator().manual_seed(124)
    do = torch.randn(o.shape, generator=gen).to(torch.bfloat16)
    (o.float() * do.cuda().float()).sum().backward()
    torch.cuda.synchronize()
    for b, h in [(0, 1), (5, 0)]:
        cut = lambda x: x[b:b + 1, :, h:h + 1]  # noqa: E731
        want = gated_delta_rule_grads_autograd(*(cut(inp[n]) for n in names), cut(do), None, scale=inp["scale"],
                                               use_qk_l2norm_in_kernel=True)  # fmt: skip
        _assert_grads([cut(leaves[n].grad) for n in names], want[:5], torch.bfloat16)


@pytest.mark.parametrize("V", [32, 64, 128])  # V = 32: chunk-local part as batched GEMMs; else all on kernels
def test_chunk_bf16_packed(V):
    cu = torch.tensor([0, 70, 71, 300], dtype=torch.int32)
    inp = random_inputs(B=1, T=300, H=2, K=128, V=V, dtype=torch.bfloat16, seed=7, normalize=False, N=3)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)


def test_recurrent_fp32():
    inp = random_inputs(B=2, T=40, H=2, K=64, V=64, dtype=torch.float32, seed=8, normalize=False)
    _run_case(lm_engine_amd.fused_recurrent_gated_delta_rule, inp, torch.float32)


def test_chunk_bf16_k64_and_wide_v():
    inp = random_inputs(B=1, T=130, H=3, K=64, V=256, dtype=torch.bfloat16, seed=9, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


@pytest.mark.parametrize("T, V", [(130, 64), (192, 512)])
def test_chunk_bf16_k256(T, V):
    # K = 256 (the head shape of the reference's shipped configurations is K = 256, V = 512): both sweeps on the
    # half-slice scan in its saving variant, the reverse one on records written in that scan's fragment layout
    inp = random_inputs(B=2, T=T, H=2, K=256, V=V, dtype=torch.bfloat16, seed=50 + V, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


def test_chunk_bf16_k256_packed():
    cu = torch.tensor([0, 70, 71, 300], dtype=torch.int32)
    inp = random_inputs(B=1, T=300, H=2, K=256, V=128, dtype=torch.bfloat16, seed=57, normalize=False, N=3)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)


@pytest.mark.parametrize("K, V", [(128, 128), (256, 128)])
def test_chunk_bf16_packed_with_empty_sequences(K, V):
    # sequences of length 0 inside a packed batch: no gradient but that of their initial state (= the gradient of their
    # final state); their rows of the mirror problem are one neutral pair of chunks, which the prepare kernel still writes
    lens = [70, 0, 129, 0, 64]
    cu = torch.tensor([0] + lens, dtype=torch.int32).cumsum(0).to(torch.int32)
    inp = random_inputs(B=1, T=sum(lens), H=2, K=K, V=V, dtype=torch.bfloat16, seed=83, normalize=False, N=len(lens))
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)


@pytest.mark.parametrize("layout", ["rows", "packed", "packed_many"])
def test_chunk_bf16_more_slices_than_compute_units(layout):
    # 6 x 16 chains x 4 slices = 384 scan workgroups for 256 CUs: the sweeps still run on the half-slice scan (bf16 saves
    # through LDS); the packed batch is ragged, so the rows of its mirror problem are scanned over their own lengths
    if layout == "rows":
        inp = random_inputs(B=6, T=192, H=16, K=128, V=128, dtype=torch.bfloat16, seed=71, normalize=False)
        _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)
    elif layout == "packed":
        cu = torch.tensor([0, 200, 230, 520, 584, 800, 1000], dtype=torch.int32)
        inp = random_inputs(B=1, T=1000, H=16, K=128, V=128, dtype=torch.bfloat16, seed=72, normalize=False, N=6)
        _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)
    else:
        # 17 sequences x 16 heads x 4 slices = 1088 workgroups, more than four per CU
        lens = [40 + 7 * n for n in range(17)]
        cu = torch.tensor([0] + lens, dtype=torch.int32).cumsum(0).to(torch.int32)
        inp = random_inputs(B=1, T=sum(lens), H=16, K=128, V=128, dtype=torch.bfloat16, seed=73, normalize=False, N=17)
        _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16, cu=cu)


@pytest.mark.parametrize("V", [128, 256, 512])
def test_chunk_bf16_whole_chunks_all_on_kernels(V):
    # whole chunks, K = 128: prepare, both sweeps and the chunk-local gradients are kernel launches
    inp = random_inputs(B=2, T=192, H=3, K=128, V=V, dtype=torch.bfloat16, seed=30 + V, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


def test_chunk_bf16_many_chains():
    # more than 128 chains at V = 128: the saving scan runs with four column slices per workgroup
    inp = random_inputs(B=9, T=128, H=16, K=128, V=128, dtype=torch.bfloat16, seed=10, normalize=False)
    _run_case(lm_engine_amd.chunk_gated_delta_rule, inp, torch.bfloat16)


def test_chunk_bf16_left_padded_batch():
    B, T, H, K, V = 3, 200, 2, 128, 128
    lens = [200, 70, 1]
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=11, normalize=False)
    cu = torch.tensor([0, 200, 270, 271], dtype=torch.int32)
    leaves = _leaves(inp)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**leaves, output_final_state=True, cu_seqlens=cu.cuda(),
                                                 use_qk_l2norm_in_kernel=True, left_padded=True)  # fmt: skip
    gen = torch.Generator().manual_seed(5)
    do = torch.randn(o.shape, generator=gen).to(torch.bfloat16)
    dht = torch.randn(ht.shape, generator=gen)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    for b, n in enumerate(lens):
        sl = lambda x: x[b : b + 1, T - n :]
        want = gated_delta_rule_grads_autograd(
            sl(inp["q"]), sl(inp["k"]), sl(inp["v"]), sl(inp["g"]), sl(inp["beta"]), sl(do), dht[b : b + 1],
            initial_state=inp["initial_state"][b : b + 1], use_qk_l2norm_in_kernel=True,
        )  # fmt: skip
        got = [sl(leaves[x].grad.cpu()) for x in ("q", "k", "v", "g", "beta")] + [leaves["initial_state"].grad[b : b + 1]]
        _assert_grads(got, want, torch.bfloat16)
        for x in ("q", "k", "v", "g", "beta"):
            assert not leaves[x].grad[b, : T - n].any(), f"gradient of {x} at the padding"


def test_ungated_without_beta():
    inp = random_inputs(B=2, T=100, H=2, K=128, V=64, dtype=torch.bfloat16, seed=12, normalize=False, gated=False)
    inp["beta"] = None
    q, k, v = (inp[x].cuda().requires_grad_(True) for x in ("q", "k", "v"))
    h0 = inp["initial_state"].cuda()
    o, _ = lm_engine_amd.chunk_gated_delta_rule(q, k, v, initial_state=h0, use_qk_l2norm_in_kernel=True)
    do = torch.randn(o.shape, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    (o.float() * do.cuda().float()).sum().backward()
    zero, one = torch.zeros(2, 100, 2), torch.ones(2, 100, 2)
    want = gated_delta_rule_grads_autograd(inp["q"], inp["k"], inp["v"], zero, one, do, None,
                                           initial_state=inp["initial_state"], use_qk_l2norm_in_kernel=True)  # fmt: skip
    _assert_grads([q.grad, k.grad, v.grad], want[:3], torch.bfloat16)


@pytest.mark.parametrize("K, V", [(128, 128), (256, 64)])
def test_saved_chunk_states_are_the_states_of_the_prefixes(K, V):
    """``gdn_chunk_fwd_saving``: the state saved for chunk c is the final state of the first 64 c tokens."""
    from lm_engine_amd import ops
    from oracle.gdn_oracle import recurrent_gated_delta_rule_ref

    B, T, H = 2, 200, 2
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=13)
    dev = {n: (None if x is None else x.cuda()) for n, x in inp.items()}
    NC = 4
    states = torch.zeros(B * H, NC, K, V, device="cuda")
    v_new = torch.zeros(B * H, NC, 64, V, device="cuda")
    ops.chunk_forward_saving(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"], None, dev["initial_state"], None,
                             True, False, states, v_new, NC)  # fmt: skip
    states = states.cpu().reshape(B, H, NC, K, V)
    assert torch.equal(states[:, :, 0], inp["initial_state"])
    for c in range(1, NC):
        cut = {n: inp[n][:, : 64 * c] for n in ("q", "k", "v", "g", "beta")}
        _, want = recurrent_gated_delta_rule_ref(**cut, initial_state=inp["initial_state"], output_final_state=True,
                                                 use_qk_l2norm_in_kernel=True)  # fmt: skip
        assert_parity(states[:, :, c], want, torch.bfloat16, f"state at the start of chunk {c}")


@pytest.mark.parametrize("K, V", [(64, 64), (64, 256), (128, 128), (128, 192), (128, 512), (256, 64), (256, 512)])
@pytest.mark.parametrize("saves", [torch.float32, torch.bfloat16])
def test_chunk_local_kernel_matches_the_batched_gemm_version(K, V, saves):
    """``gdn_chunk_bwd_local`` against the same stage written with torch operations, on random per-chunk inputs (not
    the results of real sweeps): every head dim the kernel is built for, saved states and V~ in fp32 and in bf16, with
    and without the backward of the normalisation."""
    from lm_engine_amd import ops
    from lm_engine_amd.backward import _chunk_local_grads, _l2norm_grad

    gen = torch.Generator().manual_seed(21 + K + V)
    N, H, NC, C = 2, 2, 3, 64
    Bt, T = N * H, NC * C
    bf = torch.bfloat16
    rnd = lambda *shape: torch.randn(*shape, generator=gen)  # noqa: E731
    q, k = rnd(N, T, H, K).to(bf), rnd(N, T, H, K).to(bf)
    v, dout = rnd(N, T, H, V).to(bf), rnd(N, T, H, V).to(bf)
    y = rnd(Bt, NC, C, V).to(bf)  # Y per chunk, forward token order
    v_new = rnd(Bt, NC, C, V).to(saves)
    s0, ds1 = (0.3 * rnd(Bt, NC, K, V)).to(saves), 0.3 * rnd(Bt, NC, K, V)
    gam = torch.nn.functional.logsigmoid(rnd(Bt, NC, C) + 2.0).cumsum(-1)
    beta = torch.sigmoid(rnd(Bt, NC, C))
    scale = K**-0.5
    # the mirror scan's output: [N, NC (reversed), A | B, 64 tokens (reversed), H, V], Y in the A chunks
    y_mirror = torch.zeros(N, NC, 2, C, H, V, dtype=bf)
    y_mirror[:, :, 0] = y.view(N, H, NC, C, V).flip(2, 3).permute(0, 2, 3, 1, 4)
    y_mirror = y_mirror.view(N, 2 * T, H, V)
    pack = lambda x: x.view(N, NC, C, H, -1).permute(0, 3, 1, 2, 4).reshape(Bt, NC, C, -1).double()  # noqa: E731
    for l2norm in (False, True):
        if l2norm:
            rq = torch.rsqrt(q.float().square().sum(-1) + 1e-6)  # [N, T, H]
            rk = torch.rsqrt(k.float().square().sum(-1) + 1e-6)
        else:
            rq, rk = torch.ones(N, T, H), torch.ones(N, T, H)
        chunked = lambda x: x.view(N, NC, C, H).permute(0, 3, 1, 2).reshape(Bt, NC, C).contiguous()  # noqa: E731
        prep = dict(gamma=gam.cuda(), beta=beta.cuda(), rq=chunked(rq).cuda(), rk=chunked(rk).cuda())
        got = ops.chunk_local_grads(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), prep, y_mirror.cuda(), v_new.cuda(),
                                    s0.cuda(), ds1.cuda(), scale, l2norm)  # fmt: skip
        torch.cuda.synchronize()
        if saves == bf:
            # the same call on the sliced layout of the sweeps (all bf16, Y per chunk as the mirror scan saves it: tokens
            # reversed): the kernel's other template variant - at K = 256 the one that keeps the next slab's loads in
            # flight - must give the same numbers up to the rounding of dS1 to bf16
            y_saved = y.flip(2)
            sliced = ops.chunk_local_grads(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), prep, _slice(y_saved).cuda(),
                                           _slice(v_new).cuda(), _slice(s0).cuda(), _slice(ds1.to(bf)).cuda(), scale, l2norm,
                                           sliced=True)  # fmt: skip
            plain = ops.chunk_local_grads(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), prep, y_saved.cuda(), v_new.cuda(),
                                          s0.cuda(), ds1.to(bf).cuda(), scale, l2norm)  # fmt: skip
            torch.cuda.synchronize()
            for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta"), sliced, plain):
                err = rel_l2(a, b)
                assert err <= 1e-5, f"sliced saves, {name}: rel-L2 {err:.3e} against the same call on rows of V columns"
        qn, kn = pack(q) * pack(rq[..., None]), pack(k) * pack(rk[..., None])
        dqs, dkn, dbeta, dgamma = _chunk_local_grads(qn * scale, kn, pack(v), pack(dout), y.double(), v_new.double(),
                                                     s0.double(), ds1.double(), gam.double(), beta.double())  # fmt: skip
        dqn = dqs * scale
        if l2norm:
            dqn, dkn = _l2norm_grad(qn, pack(rq[..., None]), dqn), _l2norm_grad(kn, pack(rk[..., None]), dkn)
        unpack = lambda x: x.view(N, H, NC, C, -1).permute(0, 2, 3, 1, 4).reshape(N, T, H, -1)  # noqa: E731
        want = (unpack(dqn), unpack(dkn), unpack(y.double() * beta.double()[..., None]),
                unpack(dgamma.flip(-1).cumsum(-1).flip(-1))[..., 0], unpack(dbeta)[..., 0])  # fmt: skip
        for name, a, b in zip(("dq", "dk", "dv", "dg", "dbeta"), got, want):
            err = rel_l2(a, b)
            print(f"   K={K} V={V} saves={saves} l2norm={l2norm} {name}: rel-L2 {err:.3e}", flush=True)
            assert err <= 1e-2, f"{name}: rel-L2 {err:.3e}"


def _backward_sweep_case(i):
    """Case ``i`` of a seeded sweep over batch layouts, head dims and options (prepare, sweeps and chunk-local
    gradients all run as kernels)."""
    gen = torch.Generator().manual_seed(9000 + i)
    pick = lambda *xs: xs[int(torch.randint(len(xs), (1,), generator=gen))]  # noqa: E731
    layout = pick("rows", "packed", "left_padded")
    H, V = pick(1, 2, 3), pick(128, 256)
    K = (128, 64, 256)[i % 3]
    l2norm, with_state, with_dht, gated = pick(True, False), pick(True, False), pick(True, False), pick(True, True, False)
    if layout == "rows":
        B, T = pick(1, 2), pick(64, 70, 128, 191)
        lens, cu = [T] * B, None
    elif layout == "packed":
        lens = [int(x) for x in torch.randint(1, 150, (pick(1, 2, 4),), generator=gen)]
        B, T = 1, sum(lens)
        cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    else:
        B, T = pick(2, 3), pick(96, 130)
        lens = [T] + [int(x) for x in torch.randint(1, T + 1, (B - 1,), generator=gen)]
        cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    N = len(lens)
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=9100 + i, normalize=not l2norm, gated=gated, N=N)
    if not with_state:
        inp["initial_state"] = None
    return dict(layout=layout, lens=lens, cu=cu, inp=inp, l2norm=l2norm, with_dht=with_dht, B=B, T=T, H=H, V=V, K=K)


@pytest.mark.parametrize("i", range(int(os.environ.get("GDN_SWEEP_CASES", "15"))))
def test_seeded_sweep_of_layouts_and_options(i):
    c = _backward_sweep_case(i)
    inp, cu, T = c["inp"], c["cu"], c["T"]
    print(f"case {i}: {c['layout']} lens={c['lens']} H={c['H']} K={c['K']} V={c['V']} l2norm={c['l2norm']} "
          f"h0={inp['initial_state'] is not None} dht={c['with_dht']} gated={inp['g'] is not None}", flush=True)  # fmt: skip
    leaves = {n: x.cuda().requires_grad_(True) for n, x in inp.items() if x is not None}
    o, ht = lm_engine_amd.chunk_gated_delta_rule(
        **leaves, output_final_state=True, cu_seqlens=None if cu is None else cu.cuda(),
        use_qk_l2norm_in_kernel=c["l2norm"], left_padded=c["layout"] == "left_padded")  # fmt: skip
    gen = torch.Generator().manual_seed(9200 + i)
    do = torch.randn(o.shape, generator=gen).to(torch.bfloat16)
    dht = torch.randn(ht.shape, generator=gen) if c["with_dht"] else None
    loss = (o.float() * do.cuda().float()).sum()
    if dht is not None:
        loss = loss + (ht * dht.cuda()).sum()
    loss.backward()
    names = [n for n in ("q", "k", "v", "g", "beta", "initial_state") if n in leaves]
    zero_g = torch.zeros(c["B"], T, c["H"])
    for n, length in enumerate(c["lens"]):  # sequence by sequence against the oracle
        if c["layout"] == "rows":
            sl = lambda x: x[n : n + 1]  # noqa: E731
        elif c["layout"] == "packed":
            t0 = int(cu[n])
            sl = lambda x: x[:, t0 : t0 + length]  # noqa: E731
        else:
            sl = lambda x: x[n : n + 1, T - length :]  # noqa: E731
        h0 = None if inp["initial_state"] is None else inp["initial_state"][n : n + 1]
        want = gated_delta_rule_grads_autograd(
            sl(inp["q"]), sl(inp["k"]), sl(inp["v"]), sl(inp["g"] if inp["g"] is not None else zero_g), sl(inp["beta"]),
            sl(do), None if dht is None else dht[n : n + 1], initial_state=h0, use_qk_l2norm_in_kernel=c["l2norm"])  # fmt: skip
        want = dict(zip(("q", "k", "v", "g", "beta", "initial_state"), want))
        got = [sl(leaves[x].grad.cpu()) if x != "initial_state" else leaves[x].grad[n : n + 1] for x in names]
        _assert_grads(got, [want[x] for x in names], torch.bfloat16)
    if c["layout"] == "left_padded":
        for b, length in enumerate(c["lens"]):
            for x in ("q", "k", "v"):
                assert not leaves[x].grad[b, : T - length].any(), f"gradient of {x} at the padding"


def test_recurrent_bf16_short_sequences():
    # T <= 64: the layer calls the recurrent operator; its backward runs the chunk kernels on one ragged chunk
    inp = random_inputs(B=2, T=40, H=2, K=128, V=128, dtype=torch.bfloat16, seed=14, normalize=False)
    _run_case(lm_engine_amd.fused_recurrent_gated_delta_rule, inp, torch.bfloat16)


def test_given_records_in_both_fragment_orders_give_the_same_sweep():
    """``gdn_chunk_fwd_saving`` on given records: the records of one mirror problem written in the lane order of the
    32x32x16 MFMA (``records_given = 1``, whole-slice waves) and of the 16x16x32 MFMA (``records_given = 2``,
    half-slice waves) give the same output, saved states and final state up to the rounding of two different kernels."""
    from lm_engine_amd import ops

    B, T, H, K, V = 2, 256, 2, 128, 128
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=91, normalize=False)
    q, k, g, beta = (inp[n].cuda() for n in ("q", "k", "g", "beta"))
    do = torch.randn(B, T, H, V, generator=torch.Generator().manual_seed(92)).to(torch.bfloat16).cuda()
    NC = T // 64
    results = []
    for half_slices in (False, True):
        prep = ops.chunk_bwd_prepare(q, k, do, g, beta, K**-0.5, True, V, None, half_slice_records=half_slices)
        dS1 = torch.zeros(B * H, NC, K, V, device="cuda")
        o_m, dS = ops.chunk_scan_given_records(prep["k_mirror"], prep["v_mirror"], prep["records"], None, dS1, NC,
                                               save_every=2, save_reverse=True, half_slice_records=half_slices)  # fmt: skip
        torch.cuda.synchronize()
        results.append((o_m.float().cpu(), dS1.cpu(), dS.cpu()))
    for name, a, b in zip(("output", "saved states", "final state"), *results):
        assert rel_l2(a, b) <= 5e-3, f"{name}: rel-L2 {rel_l2(a, b):.3e}"


@pytest.mark.parametrize("K, V, B, T, H", [(128, 128, 2, 256, 2), (256, 512, 1, 192, 2), (128, 256, 3, 128, 4)])
def test_mirror_reads_equal_the_scan_over_reversed_copies(K, V, B, T, H):
    """The reverse sweep with ``gdn_chunk_saves.mirror_reads`` - the scan reads the caller's q, k, dO backwards and
    P^T dO in the caller's order, the odd chunks' operand fragments from chunk 1's record - against the same scan over
    the reversed copies that ``gdn_chunk_bwd_prepare`` otherwise writes: same kernel, same arithmetic, bit for bit."""
    from lm_engine_amd import ops

    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=93, normalize=False)
    q, k, g, beta = (inp[n].cuda() for n in ("q", "k", "g", "beta"))
    gen = torch.Generator().manual_seed(94)
    do = torch.randn(B, T, H, V, generator=gen).to(torch.bfloat16).cuda()
    dht = torch.randn(B, H, K, V, generator=gen).cuda()
    NC = T // 64
    staged = ops.saving_scan_is_staged(B, 2 * T, H, K, V, None, False, 2, q.device, states_dtype=torch.bfloat16, save_every=2)
    assert staged, "this shape should run the scan without output"
    results = []
    for copies in (True, False):
        prep = ops.chunk_bwd_prepare(q, k, do, g, beta, K**-0.5, True, V, None, half_slice_records=True, reversed_copies=copies)
        assert (prep["k_mirror"] is None) == (not copies)
        dS1 = torch.zeros(B * H, NC, K, V, dtype=torch.bfloat16, device="cuda")
        Y = torch.zeros(B * H, NC, 64, V, dtype=torch.bfloat16, device="cuda")
        _, dS = ops.chunk_scan_given_records(prep["k_mirror"] if copies else k, prep["v_mirror"], prep["records"], dht, dS1, NC,
                                             save_every=2, save_reverse=True, half_slice_records=True, v_new=Y, no_output=True,
                                             mirror_odd=None if copies else (q, do))  # fmt: skip
        torch.cuda.synchronize()
        results.append((dS1.cpu(), Y.cpu(), dS.cpu()))
    for name, a, b in zip(("saved states", "saved Y", "final state"), *results):
        assert a.abs().max() > 0, name
        assert torch.equal(a, b), f"{name}: rel-L2 {rel_l2(a.float(), b.float()):.3e}"


@pytest.mark.parametrize("K, V, half", [(128, 128, True), (256, 128, True), (64, 64, True), (128, 128, False), (64, 128, False)])
def test_rows_scanned_over_their_own_lengths_equal_the_fixed_length_scan(K, V, half):
    """The mirror problem of a ragged batch, scanned as a left-padded batch of given records (every row over its own
    chunks, records at the slots of its tokens, reverse saves counted from its own last chunk, ``row_order``) with the
    chunk slots past a sequence's end left unwritten, against the scan of all rows over the chunks of the longest one
    with neutral records there: the same saved states, Y and final states at the real chunks, bit for bit (a neutral
    chunk leaves the state as it is)."""
    from lm_engine_amd import ops

    lens = [70, 300, 129, 64]
    N, H, total = len(lens), 3, sum(lens)
    inp = random_inputs(B=1, T=total, H=H, K=K, V=V, dtype=torch.bfloat16, seed=101, normalize=False, N=N)
    q, k, g, beta = (inp[n].cuda() for n in ("q", "k", "g", "beta"))
    gen = torch.Generator().manual_seed(102)
    do = torch.randn(1, total, H, V, generator=gen).to(torch.bfloat16).cuda()
    dht = torch.randn(N, H, K, V, generator=gen).cuda()
    starts = [sum(lens[:n]) for n in range(N)]
    chunks = [-(-length // 64) for length in lens]
    NC = max(chunks)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    sequences = (i32(starts), i32(lens), NC)
    saves = torch.bfloat16 if half else torch.float32
    results = []
    for own_lengths in (False, True):
        prep = ops.chunk_bwd_prepare(q, k, do, g, beta, K**-0.5, True, V, sequences, half_slice_records=half,
                                     skip_empty_chunks=own_lengths)  # fmt: skip
        if own_lengths:  # what the prepare kernel skipped must not matter
            live = torch.zeros(N, NC, dtype=torch.bool)
            for n in range(N):
                live[n, : chunks[n]] = True
            dead_rows = (~live).flip(1).repeat_interleave(128, dim=1).cuda()  # mirror rows: chunk c at pair NC - 1 - c
            prep["k_mirror"][dead_rows] = float("nan")
            prep["v_mirror"][dead_rows] = float("nan")
        dS1 = torch.zeros(N * H, NC, K, V, dtype=saves, device="cuda")
        Y = torch.zeros(N * H, NC, 64, V, dtype=saves, device="cuda")
        _, dS = ops.chunk_scan_given_records(prep["k_mirror"], prep["v_mirror"], prep["records"], dht, dS1, NC, save_every=2,
                                             save_reverse=True, half_slice_records=half, v_new=Y, no_output=half,
                                             valid_lengths=[128 * c for c in chunks] if own_lengths else None)  # fmt: skip
        torch.cuda.synchronize()
        results.append((dS1.cpu().view(N, H, NC, K, V), Y.cpu().view(N, H, NC, 64, V), dS.cpu()))
    (s_a, y_a, f_a), (s_b, y_b, f_b) = results
    assert torch.equal(f_a, f_b), "final states"
    for n in range(N):
        assert s_a[n, :, : chunks[n]].abs().max() > 0
        assert torch.equal(s_a[n, :, : chunks[n]], s_b[n, :, : chunks[n]]), f"saved states of sequence {n}"
        assert torch.equal(y_a[n, :, : chunks[n]], y_b[n, :, : chunks[n]]), f"saved Y of sequence {n}"


def _slice(x):
    """[chains, entries, rows, V] -> the same values in the memory order of ``gdn_chunk_saves.sliced``, [V / 32][rows][32]
    per entry (shape kept)."""
    ch, nc, rows, V = x.shape
    return x.reshape(ch, nc, rows, V // 32, 32).permute(0, 1, 3, 2, 4).contiguous().view(ch, nc, rows, V)


def _unslice(x, rows):
    """[chains, entries, rows, V] array written with ``gdn_chunk_saves.sliced`` -> its [.., rows, V] meaning: memory is
    [V / 32][rows][32] per entry."""
    ch, nc, r, V = x.shape
    assert r == rows
    return x.reshape(ch, nc, V // 32, rows, 32).permute(0, 1, 3, 2, 4).reshape(ch, nc, rows, V)


@pytest.mark.parametrize("K, V, no_output", [(128, 128, False), (128, 256, True), (256, 512, True), (64, 64, False)])
def test_sliced_saves_hold_the_same_values(K, V, no_output):
    """bf16 saves in the sliced layout (32-column slice by slice: one contiguous block per scan workgroup and chunk) against
    the same saves in rows of V columns: the same values, bit for bit, once the layout is undone."""
    from lm_engine_amd import ops

    B, T, H = 2, 256, 2
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=torch.bfloat16, seed=17)
    dev = {n: (None if x is None else x.cuda()) for n, x in inp.items()}
    NC = T // 64
    assert ops.saving_scan_is_staged(B, T, H, K, V, None, False, 0, "cuda", no_output=no_output)
    out = []
    for sliced in (False, True):
        states = torch.zeros(B * H, NC, K, V, dtype=torch.bfloat16, device="cuda")
        v_new = torch.zeros(B * H, NC, 64, V, dtype=torch.bfloat16, device="cuda")
        ops.chunk_forward_saving(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"], None, dev["initial_state"], None,
                                 True, False, states, v_new, NC, no_output=no_output, sliced=sliced)  # fmt: skip
        torch.cuda.synchronize()
        out.append((states.cpu(), v_new.cpu()))
    assert out[0][0].abs().max() > 0 and out[0][1].abs().max() > 0
    assert torch.equal(out[0][0], _unslice(out[1][0], K)), "states"
    assert torch.equal(out[0][1], _unslice(out[1][1], 64)), "V~"
