"""CPU oracle for the streaming paged-KV attention path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline.  Nothing in the
product package imports it, and the product path fails loudly without its HIP library
instead of falling back to this code.
"""
