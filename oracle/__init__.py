"""CPU restatement of the reference's learned-optimizer step.

TEST INFRASTRUCTURE ONLY.  Nothing under ``pylo_amd/`` may import this package:
it exists so that the tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` have something to check the HIP path against (and to time as
the non-fused PyTorch path on host cores).
"""
