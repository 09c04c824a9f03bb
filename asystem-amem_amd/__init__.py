"""MI355X-native AMem pause/resume engine: Python access to libamem_nccl.so.1.

The product is the shared library built from csrc/ (C++ and HIP for gfx950); this package
only binds its C ABI (binding.py), generates the synthetic footprints of the benchmark
configurations (footprint.py) and wraps both for tests and benchmarks (harness.py).
"""
from . import binding, footprint  # noqa: F401
