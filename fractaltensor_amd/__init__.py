"""MI355X-native kernels for the FractalTensor hot path, behind a kaleido-compatible API.

``fractaltensor_amd._core``  ctypes binding of the C ABI (include/ftk.h)
``fractaltensor_amd.kaleido`` the reference's Python operator API (Tensor, FractalTensor,
                              operations.map/scan/fold/reduce ...) with GPU fast paths
"""
__version__ = '0.1.0'
