"""CPU oracle for the low-precision path — test infrastructure, never the product.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.
"""

from . import cpu_reference, formats, gemm, quantize  # noqa: F401
