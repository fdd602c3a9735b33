"""CPU oracle for the FractalTensor hot path.

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the ``fractaltensor_amd``
package, its C-ABI library) may import, call or link anything in this
directory.  The only legitimate users are ``tests/``, the smoke check in
``__graft_entry__.py`` and the ``cpu_baseline`` leg of ``bench.py``, and they
use it as the checker, never as the thing that is measured as the product.
"""
