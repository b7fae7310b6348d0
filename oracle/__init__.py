"""CPU oracle for the paged-KV hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the shipped
product: it is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline, never by
``morphserve_amd``.  The product path raises when its HIP library is missing; it
never falls back to this code.
"""
