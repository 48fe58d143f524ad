"""CPU oracle for the GGUF k-quant matmul path.  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke entry point and the ``cpu_baseline`` leg of the
benchmark may import this package, and only as the checker: the shipped
``hipengine_amd`` package never imports it and has no CPU fallback.
"""
