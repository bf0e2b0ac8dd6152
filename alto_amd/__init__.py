"""MI355X-native implementation of ALTO's MXFP4 training hot path.

Python host code here only validates shapes, allocates outputs with torch and calls the hand-written HIP
kernels of ``libalto_mxfp4.so`` through its C ABI (``alto_amd._lib``).  There is no CPU or eager fallback:
every op raises if the tensors are not on a GPU or the library cannot be loaded.
"""
__version__ = "0.1.0"
