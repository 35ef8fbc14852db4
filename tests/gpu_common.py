"""Helpers of the GPU parity tests: device buffers through the C ABI, paired oracle / device contexts."""
import numpy as np

from ckks_llm_amd import Context_23, DeviceBuffer
from oracle import oracle_py as O


def have_gpu():
    try:
        import ctypes
        from ckks_llm_amd import load_library
        n = ctypes.c_int(0)
        return load_library().ckks_device_count(ctypes.byref(n)) == 0 and n.value > 0
    except Exception:
        return False


class Pair:
    """The same context on the device (C ABI) and in the CPU oracle."""

    def __init__(self, logN, p, q, t=(), gamma=0):
        self.dev = Context_23(logN, p, q, t, gamma)
        self.orc = O.OracleContext(logN, p, q, t, gamma)
        self.N = 1 << logN


def to_dev(a):
    return DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.uint64))


def from_dev(buf, shape):
    return buf.download(np.uint64, int(np.prod(shape))).reshape(shape)
