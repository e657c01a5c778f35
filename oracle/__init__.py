"""TEST INFRASTRUCTURE ONLY: CPU oracle for the ILGPU.Algorithms hot path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the CPU-baseline leg of
``bench.py`` may import this package.  The shipped library never does.
"""
