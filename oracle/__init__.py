"""CPU oracle for the tritonformer_amd kernels: TEST INFRASTRUCTURE ONLY.

Nothing in the product (tritonformer_amd/) imports this package; it is used by
tests/, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker / the timed CPU baseline.
"""
