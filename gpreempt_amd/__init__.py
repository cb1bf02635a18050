"""MI355X-native preemptible inference executor (device layer + C++ host classes).

The product is the pair of shared libraries built from csrc/ (C ABI, HIP kernels for gfx950)
and host/ (C++ Executor / BLPExecutor / Model).  The Python modules in this package are thin
ctypes bindings used by the tests and the benchmark driver.
"""
