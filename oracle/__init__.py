"""CPU oracle for the gated delta-rule sequence mixer.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may call into it, and only as the
checker, never as the thing measured or shipped.
"""

from .gdn_oracle import (  # noqa: F401
    chunk_gated_delta_rule_ref,
    decode_step_single_pass_ref,
    l2norm_ref,
    recurrent_gated_delta_rule_ref,
)
