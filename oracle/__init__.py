"""CPU oracle for the token-log-prob path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The shipped path (``tome_amd``) never
imports it and fails loudly when its HIP library is missing.
"""
from .logprob_oracle import *  # noqa: F401,F403
