"""CPU oracle of the cortex tensor-math path: test infrastructure only.

Nothing under ``cortex_amd`` imports this package.  It is loaded by the tests,
by ``__graft_entry__.smoke()`` and by the cpu_baseline leg of ``bench.py``.
"""
