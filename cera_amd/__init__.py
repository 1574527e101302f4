"""cera_amd: an MI355X-native `hip` compute backend for the dense-transformer
decode/prefill hot path of the cera inference engine.

The compute path is a C-ABI shared library (``include/cera_hip.h``) of
hand-written HIP kernels for gfx950; this package holds its sources
(``csrc/``), the CPU host layer above it (``host/``) and thin ctypes bindings
used by the tests and the benchmark.
"""
__version__ = "0.1.0"
