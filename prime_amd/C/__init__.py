"""Counterparts of the reference's ``zeroband.C`` modules (src/zeroband/C/), whose native
code here is libprime_hip.so instead of two JIT-built pybind11 extensions."""
