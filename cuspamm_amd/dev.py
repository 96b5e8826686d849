"""ctypes mirror of include/spamm_dev.h: measurement aids that are not part of the engine."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
DEV_LIB_PATH = os.path.join(HERE, "libspamm_dev_gfx950.so")

_lib = None


def load_dev_library():
    global _lib
    if _lib is None:
        if not os.path.exists(DEV_LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m cuspamm_amd.build`" % DEV_LIB_PATH)
        import torch  # noqa: F401  (one copy of the HIP runtime in the process)
        L = ctypes.CDLL(DEV_LIB_PATH)
        L.spamm_dev_mfma_ceiling.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                             ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
        L.spamm_dev_read_reference.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
        _lib = L
    return _lib


def read_reference(device=0, which=0):
    """GB/s of one of the four read-only reference kernels (see include/spamm_dev.h)."""
    g = ctypes.c_double(0)
    rc = load_dev_library().spamm_dev_read_reference(int(device), int(which), ctypes.byref(g))
    if rc != 0:
        raise RuntimeError("spamm_dev_read_reference failed: %d" % rc)
    return float(g.value)


def mfma_ceiling(device=0, random_operands=True, iters=20000):
    """(TFLOP/s, GHz) of a pure fp16 MFMA issue loop on every CU of `device`."""
    tf, ghz = ctypes.c_double(0), ctypes.c_double(0)
    rc = load_dev_library().spamm_dev_mfma_ceiling(int(device), int(bool(random_operands)), int(iters),
                                                   ctypes.byref(tf), ctypes.byref(ghz))
    if rc != 0:
        raise RuntimeError("spamm_dev_mfma_ceiling failed: %d" % rc)
    return float(tf.value), float(ghz.value)
