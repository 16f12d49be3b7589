"""CPU oracle for the hot path.  TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; ``flex_shard_amd`` never does.

Two independent restatements of the reference arithmetic live here:

* ``flexshard_oracle.c`` (loaded through ctypes by :mod:`oracle.cport`): plain
  C with its own bfloat16 and E4M3FN conversions.
* :mod:`oracle.eager`: the same algorithms spelled in eager torch CPU ops, the
  form the reference itself uses for its CPU-runnable checks.

:mod:`oracle.layout` restates the integer host math (block-row planner, payload
format, compaction order, gradient send rows) in a deliberately naive
"enumerate every unit" style so that it cross-checks the metadata-driven host
code of the package.

Pin status (see tests/test_oracle_*.py): every function here is pinned by a
known answer transcribed from the reference's own tests, a closed form, an
exhaustive comparison with an independent library routine, or brute force on
small inputs.  Nothing is "parity unpinned".
"""

from . import cport, eager, layout  # noqa: F401
