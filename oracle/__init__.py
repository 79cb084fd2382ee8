"""CPU restatement of the TeraPipe sliced-layer hot path.

TEST INFRASTRUCTURE ONLY: nothing in the shipped package (``terapipe_amd``)
imports this directory.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.
"""
from .terapipe_oracle import *  # noqa: F401,F403
