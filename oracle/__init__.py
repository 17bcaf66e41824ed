"""CPU oracle for the sparse-convolution forward path.  TEST INFRASTRUCTURE ONLY.

Importable from tests/, the smoke check and the benchmark's cpu_baseline leg; never from the
warpconvnet_amd package.
"""
