"""CPU oracle for the T5 attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
package: it is the checker the HIP kernels are compared against, never a
fallback.  Allowed importers: ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.
"""
