"""CPU oracle for the W8A8 linear path. TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker. The product package ``astrai_amd`` never
imports it and raises when its HIP library is missing.
"""
