"""MI355X-native kernels and graph runtime for OGLE's convolution hot path.

`ogle_amd.hip` binds the C ABI of the gfx950 kernel library (include/ogle_hip.h);
`ogle_amd.session` binds the C++ graph runtime that mirrors the reference's
Kernel / FBOSession API; `ogle_amd.dlx` reads and writes the .dlx model format.
There is no CPU fallback: loading fails if the HIP library has not been built.
"""
__version__ = "0.1.0"
