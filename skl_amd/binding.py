"""ctypes loader for libskl_gfx950.so."""
import ctypes
import os

import numpy as np

from . import signatures

_HERE = os.path.dirname(os.path.abspath(__file__))
_SUFFIX = "_gfx950"


class LibraryNotBuilt(RuntimeError):
    pass


def library_path():
    return os.path.join(_HERE, "lib", "libskl_gfx950.so")


class _Lib:
    """Holds the CDLL and one Python callable per C entry point."""

    def __init__(self, path):
        if not os.path.exists(path):
            raise LibraryNotBuilt(
                f"{path} is missing: build it with `make -C skl_amd/csrc` (or __graft_entry__.build()); "
                "there is no CPU fallback")
        self.path = path
        self.cdll = ctypes.CDLL(path)
        self.names = []
        for name, (restype, sig) in signatures.RUNTIME.items():
            raw = signatures.bind(self.cdll, name, sig, restype)
            setattr(self, name, _wrap(raw, sig) if "p" in sig else raw)
        for table in (signatures.reference_shared(), signatures.gfx950_only()):
            for stem, sig in table.items():
                cname = stem + _SUFFIX
                raw = signatures.bind(self.cdll, cname, sig)
                setattr(self, cname, _wrap(raw, sig))
                self.names.append(cname)


def _as_pointer(x):
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    if isinstance(x, np.ndarray):
        return x.ctypes.data
    return x  # integer address


class Epilogue:
    """Fused-epilogue operands of the `skl_gemm_fused_*` entry points: `bias` (n values of C's
    type), `max` (one value of C's type), `activation` (ACT_NONE / ACT_RELU; floating-point C also ACT_SILU / ACT_GELU) and the requantised
    copy `q` (int8, element (i, j) at `i * rsq + j * csq`) made with `q_scale` (one float32, or n
    of them with `q_scale_per_column`) and `q_zero`; `q_only` leaves C unwritten. Every operand
    is a DeviceBuffer, a numpy array or None."""

    ACT_NONE, ACT_RELU, ACT_SILU, ACT_GELU = 0, 1, 2, 3

    Q_INT8, Q_F8E4M3, Q_F8E4M3_SAT, Q_F8E5M2, Q_F8E5M2_SAT = range(5)

    def __init__(self, bias=None, max=None, activation=0, q=None, rsq=0, csq=0, q_scale=None,
                 q_scale_per_column=False, q_zero=0, q_only=False, q_format=0):
        self.bias, self.max, self.activation = bias, max, activation
        self.q, self.rsq, self.csq, self.q_scale = q, rsq, csq, q_scale
        self.q_scale_per_column, self.q_zero, self.q_only, self.q_format = q_scale_per_column, q_zero, q_only, q_format

    def as_struct(self):
        return signatures.EpilogueStruct(_as_pointer(self.bias), _as_pointer(self.max), int(self.activation),
                                         int(bool(self.q_scale_per_column)), int(bool(self.q_only)), int(self.q_zero),
                                         _as_pointer(self.q), int(self.rsq), int(self.csq),
                                         _as_pointer(self.q_scale), int(self.q_format))


def _wrap(raw, sig):
    ptr_positions = [i for i, ch in enumerate(sig) if ch == "p"]
    epilogue_positions = [i for i, ch in enumerate(sig) if ch == "E"]

    def call(*args):
        if len(args) != len(sig):
            raise TypeError(f"{raw.__name__}: expected {len(sig)} arguments, got {len(args)}")
        args = list(args)
        for i in ptr_positions:
            args[i] = _as_pointer(args[i])
        keep = []  # descriptors stay alive until the call returns
        for i in epilogue_positions:
            if args[i] is not None:
                keep.append(args[i].as_struct())
                args[i] = ctypes.addressof(keep[-1])
        return raw(*args)

    call.__name__ = raw.__name__
    call.raw = raw
    return call


_lib = None


def load():
    global _lib
    if _lib is None:
        _lib = _Lib(library_path())
    return _lib


def lib():
    return load()


def check_error():
    """Raises if a kernel entry point recorded an error since the last check."""
    code = load().skl_hip_last_error()
    if code != 0:
        raise RuntimeError(f"skl-gfx950 error {code}: {load().skl_hip_last_error_string().decode()}")


class DeviceBuffer:
    """A device allocation made through the library's shim (skl_hip_malloc)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = load().skl_hip_malloc(max(self.nbytes, 1))
        if not self.ptr:
            check_error()
            raise MemoryError(f"skl_hip_malloc({nbytes}) failed")

    @classmethod
    def from_array(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr)
        return buf

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        if arr.nbytes > self.nbytes:
            raise ValueError("array larger than buffer")
        rc = load().skl_hip_memcpy_h2d(self.ptr, arr.ctypes.data, arr.nbytes)
        if rc != 0:
            check_error()

    def download(self, dtype, count=None):
        dtype = np.dtype(dtype)
        if count is None:
            count = self.nbytes // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        rc = load().skl_hip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes)
        if rc != 0:
            check_error()
        return out

    def offset(self, nbytes):
        """Address `nbytes` into the buffer (for misalignment tests)."""
        return self.ptr + int(nbytes)

    def free(self):
        if self.ptr:
            load().skl_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
