"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's quantized-matmul arithmetic.

Nothing under this directory is part of the shipped library.  Only the test-suite,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it,
and there only as the checker: the product path never routes through it.
"""
