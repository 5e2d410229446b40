"""CPU oracle for the fused multi-head FFN.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package (``flashmhf_amd``) may import from here; the only
legitimate users are ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py``, and there only as the checker / the reported CPU baseline.
"""
