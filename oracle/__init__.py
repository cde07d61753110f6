"""CPU oracle for the FlashRNN recurrent hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package ``flashrnn_amd`` imports
this directory; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` do, and only as the checker / the timed CPU baseline.
"""
from .flashrnn_oracle import (  # noqa: F401
    FUNCTIONS,
    flashrnn_oracle,
    flashrnn_oracle_backward,
    flashrnn_oracle_fwbw_manual,
    make_inputs,
    zero_state,
)
