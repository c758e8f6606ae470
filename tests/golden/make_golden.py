"""Writes the golden fixtures of the gated delta rule: small seeded inputs and the outputs of the
fp64 CPU oracle (oracle/gdn_oracle.py, the naive token loop) on them.

    python tests/golden/make_golden.py

The reference holds no fixture for this path (its arithmetic is in the un-vendored `fla` package),
so these vectors freeze the oracle itself: tests compare the oracle, its C restatement and the
HIP kernels against them.  Inputs are stored already rounded to bf16 (as float32 values), so that
every consumer sees bit-identical operands; outputs are float32 roundings of the fp64 results.
"""

import os
import sys

import numpy as np
import torch


HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import recurrent_gated_delta_rule_ref  # noqa: E402
from tests.helpers import random_inputs  # noqa: E402


CASES = {
    # name: (random_inputs kwargs, operator kwargs, sequence lengths or None)
    "gated_k64_v64": (dict(B=1, T=130, H=2, K=64, V=64, seed=101), dict(), None),
    "l2norm_neg_eig_k64_v32": (dict(B=2, T=70, H=1, K=64, V=32, seed=102, normalize=False, beta_max=2.0),
                               dict(use_qk_l2norm_in_kernel=True, scale=0.25), None),
    "varlen_k64_v64": (dict(B=1, T=150, H=2, K=64, V=64, seed=103, N=3), dict(), [65, 1, 84]),
    "ungated_zero_state_k64_v64": (dict(B=1, T=96, H=2, K=64, V=64, seed=104, gated=False, h0=False), dict(), None),
}  # fmt: skip


def main():
    for name, (gen, op, lengths) in CASES.items():
        inp = random_inputs(dtype=torch.bfloat16, **gen)
        cu = None if lengths is None else torch.tensor([0] + lengths).cumsum(0).to(torch.int32)
        o, ht = recurrent_gated_delta_rule_ref(
            **{k: (None if v is None else v.double()) for k, v in inp.items()},
            cu_seqlens=cu, output_final_state=True, state_dtype=torch.float64, **op,
        )  # fmt: skip
        arrays = {k: v.float().numpy() for k, v in inp.items() if v is not None}
        arrays["o"] = o.float().numpy()
        arrays["final_state"] = ht.float().numpy()
        if cu is not None:
            arrays["cu_seqlens"] = cu.numpy()
        arrays["use_qk_l2norm_in_kernel"] = np.array(int(op.get("use_qk_l2norm_in_kernel", False)))
        arrays["scale"] = np.array(op.get("scale", gen["K"] ** -0.5), dtype=np.float64)
        path = os.path.join(HERE, f"{name}.npz")
        np.savez_compressed(path, **arrays)
        print(f"{path}: {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
