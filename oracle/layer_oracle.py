"""CPU restatement of the layer's elementwise steps around the operator.

TEST INFRASTRUCTURE ONLY (imported by tests/ and by __graft_entry__.smoke()).

* ``delta_rule_gates_ref``: lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:179-183
  (``beta = b.sigmoid()``, ``* 2`` with allow_neg_eigval) and ``SoftplusDecayGate.forward`` with
  final_exponential=False, softplus_decay_gate/module.py:69-96:
  ``dt = softplus(a.float() + dt_bias)``, ``g = -exp(A_log.float()) * dt`` in fp32.
* ``gated_rmsnorm_ref``: module.py:238-242 (``o = o * silu(gate)``, ``o = o_norm(o)``) with
  nn.RMSNorm (normalization.py:69-124): ``x * rsqrt(mean(x^2, -1) + eps) * weight``.

Both are spelled with the torch library routines the reference itself calls (F.softplus,
torch.sigmoid, F.silu, F.rms_norm), evaluated in the dtype they are given (tests pass fp64), so
the pin is the library; tests/test_layer_oracle.py adds hand-computed values and invariants.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def delta_rule_gates_ref(a, b, A_log, dt_bias, allow_neg_eigval=False):
    beta = torch.sigmoid(b)
    if allow_neg_eigval:
        beta = beta * 2
    dt = F.softplus(a + dt_bias.to(a.dtype))
    g = -torch.exp(A_log.to(a.dtype)) * dt
    return g, beta


def gated_rmsnorm_ref(o, gate, weight, eps):
    x = o if gate is None else o * F.silu(gate.reshape(o.shape))
    return F.rms_norm(x, (o.size(-1),), None if weight is None else weight.to(x.dtype), eps)
