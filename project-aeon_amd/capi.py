"""ctypes binding of libaeon_mi355.so (include/aeon_mi355.h). The library is the product: if
it is missing, loading fails loudly -- there is no CPU fallback anywhere in this package."""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaeon_mi355.so")

OK, ERR_INVALID_ARGUMENT, ERR_LOGIC, ERR_OUT_OF_RANGE, ERR_HIP, ERR_IO = 0, 1, 2, 3, 4, 5


class AeonLogicError(RuntimeError):
    """std::logic_error on the reference side."""


_EXC = {ERR_INVALID_ARGUMENT: ValueError, ERR_LOGIC: AeonLogicError,
        ERR_OUT_OF_RANGE: IndexError, ERR_HIP: RuntimeError, ERR_IO: OSError}


class W13Table(C.Structure):
    _fields_ = [("w1", C.c_void_p * 8), ("s1", C.c_void_p * 8),
                ("w3", C.c_void_p * 8), ("s3", C.c_void_p * 8)]


class W2Table(C.Structure):
    _fields_ = [("w2", C.c_void_p * 8), ("s2", C.c_void_p * 8)]


class A64Expert(C.Structure):
    _fields_ = [("w1_packed", C.c_void_p), ("w1_scale", C.c_void_p),
                ("w3_packed", C.c_void_p), ("w3_scale", C.c_void_p),
                ("w2_packed", C.c_void_p), ("w2_scale", C.c_void_p)]


class PayloadLayout(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("w1_packed", "w1_scale", "w2_packed", "w2_scale",
                                           "w3_packed", "w3_scale", "total")]


def build(verbose=False):
    """Compile every HIP source for gfx950 into libaeon_mi355.so (hipcc cross-compiles
    without a GPU)."""
    subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-j8", "-B"], check=True,
                   stdout=None if verbose else subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libaeon_mi355.so is not built: run __graft_entry__.build() (or make -C "
                "project-aeon_amd/csrc); there is no fallback path")
        # PyTorch ships its own copy of the HIP runtime under a different file name. If this
        # library is loaded first, the process ends up with two runtimes (the system one bound
        # here, PyTorch's bound to the tensors), and the one bound here finds no device. Loading
        # PyTorch's first makes the loader reuse it for this library too.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = C.CDLL(LIB_PATH)
        _lib.aeon_last_error.restype = C.c_char_p
        _lib.aeon_a64_packed_bytes.restype = C.c_size_t
        _lib.aeon_a64_scale_bytes.restype = C.c_size_t
        _lib.aeon_moe_layer_workspace_bytes.restype = C.c_size_t
        _lib.aeon_router_logits_workspace_bytes.restype = C.c_size_t
        _lib.aeon_a64_slot_bytes.restype = C.c_size_t
        _lib.aeon_expert_catalog_close.restype = None
    return _lib


def check(rc):
    if rc != OK:
        raise _EXC.get(rc, RuntimeError)(lib().aeon_last_error().decode())


def call(name, *args):
    """Call an int-returning entry point and raise the matching exception on failure."""
    check(getattr(lib(), name)(*args))


def vp(x):
    """Device or host pointer argument: a torch tensor, a numpy array, an int or None."""
    if x is None:
        return C.c_void_p(0)
    if isinstance(x, int):
        return C.c_void_p(x)
    if hasattr(x, "data_ptr"):
        return C.c_void_p(x.data_ptr())
    return C.c_void_p(x.ctypes.data)
