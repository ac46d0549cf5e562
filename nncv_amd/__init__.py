"""nncv_amd — MI355X (gfx950) implementation of nncv's ResNet-18 conv/GEMM hot path.

The product is the C-ABI shared library built from nncv_amd/csrc (see include/nncv_hip.h);
this package holds its build recipe, a ctypes mirror of the ABI structs, the model.bin tooling
and the seeded synthetic inputs of the benchmark configurations.
"""
