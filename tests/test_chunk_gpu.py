"""Parity of the chunked-forward HIP kernels (through the C ABI) against the CPU oracle.

Every case feeds the GPU and the oracle the same bf16-rounded tensors; the gate is the one of
the benchmark contract for bf16 inputs: max-abs <= 2e-2 and relative-L2 <= 1e-2 on both the
output and the final state."""

import os

import pytest
import torch

import lm_engine_amd
from lm_engine_amd.workloads import get_workload, make_inputs
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import assert_parity, max_abs, random_inputs, rel_l2


pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _to_gpu(inp):
    return {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}


def _check(inp, label, **kwargs):
    print(f"case: chunk {label} q={tuple(inp['q'].shape)} v={tuple(inp['v'].shape)} {kwargs}", flush=True)
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True, **kwargs)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**_to_gpu(inp), output_final_state=True, **kwargs)
    torch.cuda.synchronize()
    assert o.dtype == BF16 and ht.dtype == torch.float32
    print(f"   o: max-abs {max_abs(o.float(), o_ref):.3e} rel-L2 {rel_l2(o.float(), o_ref):.3e}   "
          f"ht: max-abs {max_abs(ht, h_ref):.3e} rel-L2 {rel_l2(ht, h_ref):.3e}", flush=True)  # fmt: skip
    assert_parity(o.float(), o_ref, BF16, "o")
    assert_parity(ht, h_ref, BF16, "final_state")
    return o, ht


@pytest.mark.parametrize("T", [65, 128, 130, 321])
def test_sequence_lengths_with_tail_chunks(T):
    _check(random_inputs(B=2, T=T, H=2, K=128, V=128, dtype=BF16, seed=50 + T), f"T={T}")


@pytest.mark.parametrize("K, V", [(64, 32), (64, 64), (128, 64), (128, 256), (256, 128), (256, 512), (128, 160)])
def test_head_dims(K, V):
    _check(random_inputs(B=1, T=200, H=2, K=K, V=V, dtype=BF16, seed=60 + K + V), f"K={K} V={V}")


@pytest.mark.parametrize(
    "B, T, H, K, V, slices_per_workgroup",
    [
        (9, 130, 16, 128, 128, 2),   # 144 chains x 4 slices: more slices than CUs -> two per workgroup
        (20, 130, 16, 128, 128, 4),  # 320 chains x 4 slices -> four per workgroup
        (12, 130, 8, 128, 256, 4),   # 96 chains x 8 slices -> four per workgroup, two groups per chain
        (17, 130, 16, 64, 64, 2),    # 272 chains x 2 slices -> two per workgroup (all of V)
        (30, 130, 16, 128, 96, 1),   # 3 tiles of V: only one slice per workgroup divides them
    ],
)
def test_many_chains_share_records_in_a_workgroup(B, T, H, K, V, slices_per_workgroup):
    # the scan puts 1, 2 or 4 column slices of a chain into one workgroup depending on how many slices
    # there are against the number of CUs (256 on MI355X); ragged length so the last chunk is partial
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=BF16, seed=400 + B + V)
    _check(inp, f"B={B} H={H} K={K} V={V}: {slices_per_workgroup} slice(s) per workgroup")


def _sweep_case(i):
    gen = torch.Generator("cpu").manual_seed(9000 + i)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=gen))]  # noqa: E731
    K = pick([64, 128])
    V = pick([32, 64, 96, 128, 160, 192, 256])
    H = pick([1, 2, 3, 4, 8])
    T = int(torch.randint(1, 400, (1,), generator=gen))
    B = pick([1, 1, 2, 3, 5])
    return dict(
        B=B, T=T, H=H, K=K, V=V,
        l2norm=pick([False, True]), h0=pick([False, True]), gated=pick([True, True, False]),
        g_mean=pick([-1.0, 1.0, 3.0]), packed=B == 1 and T >= 8 and pick([False, True]),
    )  # fmt: skip


@pytest.mark.parametrize("i", range(int(os.environ.get("GDN_SWEEP_CASES", "16"))))
def test_seeded_sweep_of_shapes_and_options(i):
    # shapes and switches drawn from a seeded generator: head dims, column tiles that do not divide evenly over
    # the workgroup sizes, ragged lengths, packed sequences, state in / no state, ungated, in-kernel l2norm
    c = _sweep_case(i)
    kwargs = dict(use_qk_l2norm_in_kernel=True) if c["l2norm"] else {}
    n_seq, cu = None, None
    if c["packed"]:
        gen = torch.Generator("cpu").manual_seed(9100 + i)
        cuts = sorted(set(int(x) for x in torch.randint(1, c["T"], (3,), generator=gen)))
        cu = torch.tensor([0] + cuts + [c["T"]], dtype=torch.int32)
        n_seq = cu.numel() - 1
    inp = random_inputs(B=c["B"], T=c["T"], H=c["H"], K=c["K"], V=c["V"], dtype=BF16, seed=9200 + i, gated=c["gated"],
                        h0=c["h0"], g_mean=c["g_mean"], normalize=not c["l2norm"], N=n_seq)  # fmt: skip
    if cu is not None:
        inp = dict(inp, cu_seqlens=cu)
    _check(inp, f"sweep {i}: {c}", **kwargs)


def test_short_sequence_single_partial_chunk():
    _check(random_inputs(B=3, T=17, H=2, K=128, V=128, dtype=BF16, seed=70), "T=17")


def test_l2norm_in_kernel_scale_and_negative_eigenvalues():
    # un-normalised q/k with the in-kernel normalisation, beta in (0, 2) as with allow_neg_eigval
    inp = random_inputs(B=2, T=192, H=2, K=128, V=128, dtype=BF16, seed=71, normalize=False, beta_max=2.0)
    _check(inp, "l2norm", use_qk_l2norm_in_kernel=True, scale=0.2)


def test_strong_decay():
    # g around -6 per token: decay factors inside one chunk span e^-380 (underflow to 0 must be harmless)
    _check(random_inputs(B=1, T=256, H=2, K=128, V=128, dtype=BF16, seed=72, g_mean=-6.0), "strong decay")


def test_ungated_no_beta_no_initial_state():
    inp = random_inputs(B=1, T=256, H=2, K=128, V=64, dtype=BF16, seed=73, gated=False, h0=False)
    inp["beta"] = None
    inp["k"] = inp["k"] * 0.5
    _check(inp, "ungated")


def test_fp32_beta_is_accepted():
    inp = random_inputs(B=1, T=130, H=2, K=64, V=64, dtype=BF16, seed=74)
    inp["beta"] = inp["beta"].float()
    _check(inp, "fp32 beta")


def test_varlen_packed_sequences_match_and_equal_separate_runs():
    lengths = [130, 64, 1, 200, 63, 65]
    inp = random_inputs(B=1, T=sum(lengths), H=2, K=128, V=128, dtype=BF16, seed=75, N=len(lengths))
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    o, ht = _check(dict(inp, cu_seqlens=cu), "varlen")
    gpu = _to_gpu(inp)
    for n in range(len(lengths)):
        s, e = int(cu[n]), int(cu[n + 1])
        one = {name: x[:, s:e] for name, x in gpu.items() if name != "initial_state"}
        o_n, h_n = lm_engine_amd.chunk_gated_delta_rule(**one, initial_state=gpu["initial_state"][n : n + 1],
                                                        output_final_state=True)  # fmt: skip
        assert torch.equal(o[:, s:e], o_n), f"sequence {n}: packed and separate outputs differ"
        assert torch.equal(ht[n : n + 1], h_n)


@pytest.mark.parametrize("count, H, V", [(40, 8, 128), (1100, 1, 32)])
def test_varlen_many_sequences_start_longest_first(count, H, V):
    # The scan starts the chains of a packed batch by decreasing length (ranked on the device; batches of more than
    # 1024 sequences keep their order): sequences of equal and of very different lengths, empty ones, more chains
    # than CUs in the first case (two workgroups per CU are accepted for packed batches).
    gen = torch.Generator().manual_seed(count)
    lengths = torch.randint(0, 4, (count,), generator=gen).tolist()
    for i in range(0, count, 7):
        lengths[i] = int(torch.randint(60, 200, (1,), generator=gen))
    lengths[count // 2] = 700
    inp = random_inputs(B=1, T=sum(lengths), H=H, K=64, V=V, dtype=BF16, seed=78, N=count)
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    _check(dict(inp, cu_seqlens=cu), f"varlen, {count} sequences")


@pytest.mark.parametrize("K, V", [(128, 128), (64, 64), (256, 128)])
def test_varlen_with_an_empty_sequence(K, V):
    # a sequence of length 0 has no chunk: its final state is its initial state, and its neighbours are untouched
    lengths = [70, 0, 129, 0]
    inp = random_inputs(B=1, T=sum(lengths), H=2, K=K, V=V, dtype=BF16, seed=77, N=len(lengths))
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
    o, ht = _check(dict(inp, cu_seqlens=cu), f"varlen with empty sequences K={K} V={V}")
    assert torch.equal(ht[1].cpu(), inp["initial_state"][1]) and torch.equal(ht[3].cpu(), inp["initial_state"][3])


@pytest.mark.parametrize("K, V", [(128, 128), (256, 128)])
def test_left_padded_batch_equals_separate_runs(K, V):
    # [B, T] batch whose rows are padded on the left; cu_seqlens = prefix sums of the valid lengths
    B, T, H = 4, 200, 2
    lengths = [200, 37, 0, 129]
    inp = random_inputs(B=B, T=T, H=H, K=K, V=V, dtype=BF16, seed=78)
    gpu = _to_gpu(inp)
    cu = torch.tensor([0] + lengths).cumsum(0).to(torch.int32).cuda()
    print(f"case: chunk left-padded lengths {lengths} K={K} V={V}", flush=True)
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**gpu, cu_seqlens=cu, output_final_state=True, left_padded=True)
    for b, n in enumerate(lengths):
        assert torch.all(o[b, : T - n] == 0), f"row {b}: padding must read as zeros"
        if n == 0:
            assert torch.equal(ht[b], gpu["initial_state"][b])
            continue
        one = {name: x[b : b + 1, T - n :] for name, x in gpu.items() if name != "initial_state"}
        o_b, h_b = lm_engine_amd.chunk_gated_delta_rule(**one, initial_state=gpu["initial_state"][b : b + 1], output_final_state=True)
        assert torch.equal(o[b : b + 1, T - n :], o_b), f"row {b}: padded-batch and separate outputs differ"
        assert torch.equal(ht[b : b + 1], h_b)
        # and against the oracle on the valid tokens
        cpu = {name: x[b : b + 1, T - n :] for name, x in inp.items() if name != "initial_state"}
        o_ref, h_ref = recurrent_gated_delta_rule_c(**cpu, initial_state=inp["initial_state"][b : b + 1], output_final_state=True)
        assert_parity(o_b.float(), o_ref, BF16, "o")
        assert_parity(h_b, h_ref, BF16, "final_state")


def test_strided_views_of_a_fused_projection():
    B, T, H, K, V = 2, 150, 2, 128, 128
    gen = torch.Generator().manual_seed(76)
    fused = torch.randn(B, T, 2 * H * K + H * V, generator=gen).to(BF16)
    g = -torch.rand(B, T, H, generator=gen) * 0.1
    beta = torch.rand(B, T, H, generator=gen).to(BF16)

    def views(x):
        q, k, v = x.split((H * K, H * K, H * V), dim=-1)
        return q.view(B, T, H, K), k.view(B, T, H, K), v.view(B, T, H, V)

    q, k, v = views(fused)
    o_ref, h_ref = recurrent_gated_delta_rule_c(q=q, k=k, v=v, g=g, beta=beta, output_final_state=True,
                                                use_qk_l2norm_in_kernel=True)  # fmt: skip
    qg, kg, vg = views(fused.cuda())
    assert not qg.is_contiguous()
    o, ht = lm_engine_amd.chunk_gated_delta_rule(q=qg, k=kg, v=vg, g=g.cuda(), beta=beta.cuda(),
                                                 output_final_state=True, use_qk_l2norm_in_kernel=True)  # fmt: skip
    assert_parity(o.float(), o_ref, BF16, "o")
    assert_parity(ht, h_ref, BF16, "final_state")


def test_split_sequence_with_carried_state():
    # prefill [0, 192) then [192, 400) from the carried state == one run over [0, 400)
    inp = _to_gpu(random_inputs(B=2, T=400, H=2, K=128, V=128, dtype=BF16, seed=77))
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    head = {n: (x[:, :192] if n != "initial_state" else x) for n, x in inp.items()}
    tail = {n: (x[:, 192:] if n != "initial_state" else x) for n, x in inp.items()}
    o1, h1 = lm_engine_amd.chunk_gated_delta_rule(**head, output_final_state=True)
    tail["initial_state"] = h1
    o2, h2 = lm_engine_amd.chunk_gated_delta_rule(**tail, output_final_state=True)
    # 192 is a chunk boundary, so both runs see identical chunks: bitwise equal
    assert torch.equal(torch.cat([o1, o2], dim=1), o) and torch.equal(h2, ht)


def test_chunk_agrees_with_recurrent_kernel_and_is_repeatable():
    inp = _to_gpu(random_inputs(B=2, T=300, H=2, K=128, V=128, dtype=BF16, seed=78))
    o_c, h_c = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    o_r, h_r = lm_engine_amd.fused_recurrent_gated_delta_rule(**inp, output_final_state=True)
    assert_parity(o_c.float(), o_r.float().cpu(), BF16, "o (chunk vs recurrent kernel)")
    assert_parity(h_c, h_r.cpu(), BF16, "final_state (chunk vs recurrent kernel)")
    o_c2, h_c2 = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert torch.equal(o_c, o_c2) and torch.equal(h_c, h_c2)  # no atomics: bitwise repeatable


def test_output_final_state_false():
    inp = _to_gpu(random_inputs(B=1, T=130, H=2, K=128, V=128, dtype=BF16, seed=79))
    o1, none = lm_engine_amd.chunk_gated_delta_rule(**inp)
    o2, _ = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert none is None and torch.equal(o1, o2)


def test_positional_entry_point_picks_the_kernel_by_length():
    inp = _to_gpu(random_inputs(B=1, T=130, H=2, K=128, V=128, dtype=BF16, seed=80))
    o, ht = lm_engine_amd.gated_delta_rule(inp["q"], inp["k"], inp["v"], inp["beta"], inp["g"], inp["initial_state"])
    o_c, h_c = lm_engine_amd.chunk_gated_delta_rule(**inp, output_final_state=True)
    assert torch.equal(o, o_c) and torch.equal(ht, h_c)
    short = {n: (x[:, :64] if n != "initial_state" else x) for n, x in inp.items()}
    o, ht = lm_engine_amd.gated_delta_rule(short["q"], short["k"], short["v"], short["beta"], short["g"],
                                           short["initial_state"])  # fmt: skip
    o_r, h_r = lm_engine_amd.fused_recurrent_gated_delta_rule(**short, output_final_state=True)
    assert torch.equal(o, o_r) and torch.equal(ht, h_r)


def test_config1_full_size():
    # B=4, T=4096, H=16, K=V=128: the configuration the headline metric is quoted on
    _check(make_inputs(get_workload(1)), "cfg1 full size")


def test_config2_varlen_full_size():
    inp = make_inputs(get_workload(2))
    assert inp["cu_seqlens"][-1].item() == 32768
    _check(inp, f"cfg2 varlen, {inp['cu_seqlens'].numel() - 1} sequences")


def test_config4_long_context_reduced_length():
    # the long-context configuration (H=32, K=128, V=256, h0 random) at T=4096: a quick check of its shape
    _check(make_inputs(get_workload(4, T=4096)), "cfg4 at T=4096")


def test_config4_long_context_full_size():
    # B=1, T=65536, H=32, K=128, V=256, g ~ logsigmoid(N(4, 0.5)): 1024 serial chunks per chain with a long
    # memory, the case where bf16 operand rounding has the most room to accumulate in the state.  Same gate
    # as everywhere (max-abs 2e-2, relative-L2 1e-2 on o and on the final state).
    inp = make_inputs(get_workload(4))
    assert tuple(inp["v"].shape) == (1, 65536, 32, 256)
    o, ht = _check(inp, "cfg4 full size")
    # split at a chunk boundary with the state carried over == one run, bitwise (the kernels are deterministic
    # and a chunk's arithmetic does not depend on its position in the sequence)
    gpu = _to_gpu(inp)
    cut = 64 * 389
    first = {n: (x[:, :cut] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
    o1, h1 = lm_engine_amd.chunk_gated_delta_rule(**first, output_final_state=True)
    second = {n: (x[:, cut:] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
    second["initial_state"] = h1
    o2, h2 = lm_engine_amd.chunk_gated_delta_rule(**second, output_final_state=True)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([o1, o2], dim=1), o), "split run differs from the full run"
    assert torch.equal(h2, ht)


def test_shipped_head_shape_full_size():
    # the head shape of the reference's shipped configurations (k_head_dim 256, v_head_dim 512, 2 heads, micro-batch 8,
    # T = 4096; configs/research/m2rnn/400m-normal/gated-deltanet.yml:60-73): the half-slice scan with a single buffer
    # for the rows of q, 16 chains x 16 slices.  Inputs drawn like configuration 1's.
    inp = make_inputs(get_workload(1, B=8, H=2, K=256, V=512))
    assert tuple(inp["q"].shape) == (8, 4096, 2, 256) and tuple(inp["v"].shape) == (8, 4096, 2, 512)
    o, ht = _check(inp, "K=256, V=512, B=8, T=4096, H=2")
    # split at a chunk boundary with the state carried over == one run, bitwise
    gpu = _to_gpu(inp)
    cut = 64 * 23
    first = {n: (x[:, :cut] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
    o1, h1 = lm_engine_amd.chunk_gated_delta_rule(**first, output_final_state=True)
    second = {n: (x[:, cut:] if n in ("q", "k", "v", "g", "beta") else x) for n, x in gpu.items()}
    second["initial_state"] = h1
    o2, h2 = lm_engine_amd.chunk_gated_delta_rule(**second, output_final_state=True)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([o1, o2], dim=1), o), "split run differs from the full run"
    assert torch.equal(h2, ht)
