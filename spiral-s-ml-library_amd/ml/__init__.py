"""Host surface of the MI355X build of Spiral's ML library hot path.

The reference's generated modules are imported as `ml.matmul`, `ml.layers` and `ml.primitives`
(package.spiproj lists the `ml` directory); the same names are kept here.  Every function
enqueues HIP kernels from libspiral_mi355.so through its C ABI (ctypes) on torch's current
stream, with PyTorch-ROCm tensors as device buffers.  There is no CPU or eager fallback: if the
shared library is missing the import of `ml._lib` raises.
"""
