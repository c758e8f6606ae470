"""Seeded sweep over shapes and options of the chunked forward against the C oracle: every scan variant (half-slice
waves for lone slices, 2 and 4 slices per workgroup, one launch) with tail chunks, packed and left-padded batches,
missing g / beta / initial state, in-kernel l2norm and explicit scales.  bf16 gates as everywhere: max-abs 2e-2 and
relative-L2 1e-2 on the output and on the final state."""

import random

import pytest
import torch

import lm_engine_amd
from lm_engine_amd.ops import fused_launch_applies
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import assert_parity, random_inputs


pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _cases(seed=20240611, first=0, count=36, key_dims=(64, 128, 128), value_dims=(32, 64, 96, 128, 128, 256)):
    rng = random.Random(seed)
    cases = []
    for i in range(first, first + count):
        K = rng.choice(key_dims)
        V = rng.choice(value_dims)
        kind = rng.choice(["batch", "batch", "packed", "padded"])
        H = rng.choice([1, 2, 3, 4, 8, 16])
        if i % 6 == 5:  # many chains: 2 or 4 slices per workgroup
            B, T = rng.choice([(24, 96), (40, 70), (64, 65)]), None
            B, T = B
            kind = "batch"
            H = 16
        elif kind == "batch":
            B, T = rng.choice([1, 2, 3, 4]), rng.choice([1, 63, 64, 65, 127, 130, 257, 500])
        else:
            B, T = rng.choice([2, 3, 5]), rng.choice([70, 200, 333])
        cases.append(dict(i=i, K=K, V=V, kind=kind, B=B, T=T, H=H, gated=rng.random() < 0.8, beta=rng.random() < 0.85,
                          h0=rng.random() < 0.6, l2norm=rng.random() < 0.5, scale=rng.choice([None, None, 0.25])))  # fmt: skip
    return cases


# the second batch: K = 256 (half-slice waves with a single buffer for the rows of q), V up to 512
ALL_CASES = _cases() + _cases(seed=20240612, first=36, count=16, key_dims=(256,), value_dims=(32, 64, 128, 256, 512))


@pytest.mark.parametrize("case", ALL_CASES, ids=lambda c: f"{c['i']}-{c['kind']}-B{c['B']}T{c['T']}H{c['H']}K{c['K']}V{c['V']}")
def test_forward_parity(case):
    c = case
    gen = torch.Generator("cpu").manual_seed(1000 + c["i"])
    B, T, H, K, V = c["B"], c["T"], c["H"], c["K"], c["V"]
    extra = {}
    if c["kind"] == "packed":  # B sequences of random lengths in one row of B * T tokens
        cuts = sorted(torch.randint(1, B * T, (B - 1,), generator=gen).tolist())
        cu = torch.tensor([0] + cuts + [B * T], dtype=torch.int32)
        inp = random_inputs(1, B * T, H, K, V, dtype=BF16, seed=2000 + c["i"], gated=c["gated"], h0=c["h0"],
                            normalize=not c["l2norm"], N=B)  # fmt: skip
        extra["cu_seqlens"] = cu
    else:
        inp = random_inputs(B, T, H, K, V, dtype=BF16, seed=2000 + c["i"], gated=c["gated"], h0=c["h0"],
                            normalize=not c["l2norm"])  # fmt: skip
    if not c["beta"]:
        inp["beta"] = None
    kwargs = dict(use_qk_l2norm_in_kernel=c["l2norm"], scale=c["scale"])
    gpu = {n: (x.cuda() if isinstance(x, torch.Tensor) else x) for n, x in inp.items()}
    print(f"case: {c}  one launch: {fused_launch_applies(gpu['q'], gpu['v'], extra.get('cu_seqlens'))}", flush=True)
    if c["kind"] == "padded":  # left-padded rows: valid lengths per row; the oracle runs the rows one by one
        lens = torch.randint(1, T + 1, (B,), generator=gen)
        cu = torch.nn.functional.pad(lens.cumsum(0), (1, 0)).to(torch.int32)
        o, ht = lm_engine_amd.chunk_gated_delta_rule(**gpu, output_final_state=True, cu_seqlens=cu.cuda(), left_padded=True,
                                                     **kwargs)  # fmt: skip
        for b in range(B):
            n = int(lens[b])
            row = {k: (x[b : b + 1, T - n :] if k in ("q", "k", "v", "g", "beta") and x is not None else x) for k, x in inp.items()}
            if row["initial_state"] is not None:
                row["initial_state"] = inp["initial_state"][b : b + 1]
            o_ref, h_ref = recurrent_gated_delta_rule_c(**row, output_final_state=True, **kwargs)
            assert_parity(o[b : b + 1, T - n :].float(), o_ref, BF16, f"o of row {b}")
            assert_parity(ht[b : b + 1], h_ref, BF16, f"final state of row {b}")
            assert not o[b, : T - n].any(), "the padding of the output is zero"
        return
    o_ref, h_ref = recurrent_gated_delta_rule_c(**inp, output_final_state=True, **extra, **kwargs)
    dev_extra = {k: v.cuda() for k, v in extra.items()}
    o, ht = lm_engine_amd.chunk_gated_delta_rule(**gpu, output_final_state=True, **dev_extra, **kwargs)
    assert_parity(o.float(), o_ref, BF16, "o")
    assert_parity(ht, h_ref, BF16, "final_state")
