"""CPU oracle for the W8A8 LoRA linear forward path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped
product: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it, and there only as the checker.  The product
path (the HIP kernels behind the C ABI) never routes through this package.
"""
