"""TEST INFRASTRUCTURE — the CPU oracle for the quantized-weight linear path.

Nothing under this package is product code.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  ``torchlette_amd`` never does.
"""
