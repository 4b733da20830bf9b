"""CPU oracle for the fused Adam step.

Test infrastructure only: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
CPU-baseline leg of ``bench.py``.  Nothing under ``fairscale_amd/`` may import it.
"""
