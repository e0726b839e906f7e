"""CPU oracle for the sparse-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``lvar_amd/`` may import this package; it is used by ``tests/``,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``
as the checker / reported CPU baseline, never as the product path.
"""
from .sparse_attn_oracle import *  # noqa: F401,F403
