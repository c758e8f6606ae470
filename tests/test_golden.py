"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64 token loop).

Without a GPU: the torch oracle (both formulations) and its C restatement must reproduce them.
With a GPU: both HIP kernels must meet the bf16 parity gates against them."""

import glob
import os

import numpy as np
import pytest
import torch

from oracle import chunk_gated_delta_rule_ref, recurrent_gated_delta_rule_ref
from oracle.c_oracle import recurrent_gated_delta_rule_c
from tests.helpers import assert_parity


GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))


def _load(path):
    z = np.load(path, allow_pickle=False)
    t = lambda name: torch.from_numpy(z[name]) if name in z.files else None  # noqa: E731
    inputs = dict(q=t("q"), k=t("k"), v=t("v"), g=t("g"), beta=t("beta"), initial_state=t("initial_state"),
                  cu_seqlens=t("cu_seqlens"))  # fmt: skip
    kwargs = dict(scale=float(z["scale"]), use_qk_l2norm_in_kernel=bool(int(z["use_qk_l2norm_in_kernel"])))
    return inputs, kwargs, t("o"), t("final_state")


def test_fixtures_exist():
    assert len(GOLDEN) == 4, GOLDEN


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracles_reproduce_the_fixtures(path):
    inputs, kwargs, o_gold, h_gold = _load(path)
    f64 = {n: (x.double() if x is not None and x.is_floating_point() else x) for n, x in inputs.items()}
    o, ht = recurrent_gated_delta_rule_ref(**f64, **kwargs, output_final_state=True, state_dtype=torch.float64)
    torch.testing.assert_close(o.float(), o_gold, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(ht.float(), h_gold, rtol=1e-6, atol=1e-7)
    o, ht = chunk_gated_delta_rule_ref(**f64, **kwargs, output_final_state=True, state_dtype=torch.float64)
    torch.testing.assert_close(o.float(), o_gold, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(ht.float(), h_gold, rtol=1e-5, atol=1e-6)
    o, ht = recurrent_gated_delta_rule_c(**inputs, **kwargs, output_final_state=True, f64_state=True)
    torch.testing.assert_close(o, o_gold, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(ht, h_gold, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_hip_kernels_match_the_fixtures(path):
    import lm_engine_amd

    inputs, kwargs, o_gold, h_gold = _load(path)
    print(f"case: golden {os.path.basename(path)}", flush=True)
    gpu = {n: (None if x is None else (x.cuda() if n in ("g", "initial_state", "cu_seqlens") else x.cuda().bfloat16()))
           for n, x in inputs.items()}  # fmt: skip
    for fn in (lm_engine_amd.chunk_gated_delta_rule, lm_engine_amd.fused_recurrent_gated_delta_rule):
        o, ht = fn(**gpu, **kwargs, output_final_state=True)
        assert_parity(o.float(), o_gold, torch.bfloat16, f"{fn.__name__} o")
        assert_parity(ht, h_gold, torch.bfloat16, f"{fn.__name__} final_state")
