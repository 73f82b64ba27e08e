"""TEST INFRASTRUCTURE ONLY.

CPU restatement of the reference algorithms of the sparse Clebsch-Gordan tensor-product path.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this package;
the product package ``equitorch_amd`` never does.

Pinning status of each function is listed in the header of its module.
"""
