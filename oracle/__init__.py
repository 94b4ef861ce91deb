"""CPU oracle for the WKV recurrences (test infrastructure only).

Everything under this package is a checker: it restates, in float64 NumPy, the algorithm of the reference's ``inner_loop``
implementations so that the HIP kernels can be compared against it.  Nothing
in the shipped package ``jaxrwkv_amd`` imports it; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.
"""
