"""MI355X-native (gfx950) implementation of N2D2's quantized-inference hot path.

csrc/      hand-written HIP kernels and the C ABI declared in include/n2d2hip.h
capi.py    ctypes binding of that ABI
runtime.py device-buffer plumbing for the tests and the benchmark
"""
